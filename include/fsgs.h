/*
 * fsgs.h -- C ABI of libfsgs_hip.so, the MI355X (gfx950) implementation of the Fast-SP-GS `fast_2d_gs/_C` hot path.
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer to contiguous row-major fp32 / int32 / int64 / uint8 data unless it is named
 *    *_host. NULL stands for an absent optional tensor (Python `None` at the reference's pybind boundary).
 *  - `stream` is a hipStream_t (NULL = default stream). Calls enqueue work and return; the only blocking call is
 *    fsgs_gs_prepare_scan, which has to hand the instance count to the host (the reference blocks in the same place).
 *  - The library allocates nothing, neither device nor host memory, on any call: outputs and workspaces come from the
 *    caller (the *_workspace_bytes functions size them). Outputs need not be zero-initialised unless stated. What the
 *    library keeps of its own is in file-scope device arrays that exist once per GPU from the moment the library is
 *    loaded: eight blockIdx -> tile schedule tables of 256 KiB (one per stream that bins or blends, see
 *    fsgs_stream_release) and the 512 KiB of fsgs_image_loss_forward_static.
 *  - Return value 0 = success; otherwise fsgs_last_error() describes the failure (thread local).
 *  - `file:line` citations name the reference interface each entry point replaces (relative to the reference root).
 */
#ifndef FSGS_H
#define FSGS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* fsgs_last_error(void);
int fsgs_version(void);
int fsgs_check_device(void);
/* The binning and blend entry points map blockIdx -> tile through a per-stream schedule table (longest tile lists
 * first). A stream takes one of eight table slots of its GPU on its first such call and keeps it; streams beyond the
 * eighth run without a table (identical results, blocks map to tiles directly). A caller that creates and destroys
 * streams hands a slot back with this call once the stream's work has completed. No counterpart in the reference. */
int fsgs_stream_release(void* stream);
/* ---- 2DGS surfel preprocess ---------------------------------------------------------------------------------- */

/* gs_2d_preprocess_forward -- fast_2d_gs/_C/src/gaussian_splatting/gs_2d_preprocess.cu:331-421 (kernel :158-246).
 * means3D[P,3] scales[P,2] rotations[P,4](x,y,z,w, used un-normalised) opacities[P,1]; sh_degree >= 0: shs[P,n_sh,3]
 * (or shs[P,1,3] + sh_rest[P,n_sh,3]); sh_degree < 0: colours are the caller's own tensor and `colors` is ignored.
 * trans_precomp[P,3,3] replaces the computed transform (then trans_mat is not written). culling[P] != 0 rejects.
 * Every output row is written (zeros for rejected surfels); rows of means2D belonging to rejected surfels are left
 * untouched when means2D_preserve != 0 (the reference's caller-supplied means2D buffer). records (optional, [P,20],
 * 16-byte aligned, no counterpart in the reference) receives the packed per-surfel record of fsgs_gs_2d_pack_records
 * without a second pass over the outputs; keep_masks (optional, [P], no counterpart in the reference) the masks of
 * fsgs_gs_2d_cull_masks, likewise. */
int fsgs_gs_2d_preprocess_forward(int P, int W, int H, int sh_degree, int n_sh, const float* means3D,
    const float* scales, const float* rotations, const float* opacities, const float* shs, const float* sh_rest,
    const float* Tw2v, const float* Tv2c, const float* campos, const float* trans_precomp, const uint8_t* culling,
    int means2D_preserve, float* means2D, float* colors, float* trans_mat, float* normal_opacity, float* depths,
    int32_t* radii, int32_t* tiles_touched, float* records, uint32_t* keep_masks, void* stream);

/* gs_2d_preprocess_backward -- gs_2d_preprocess.cu:423-499 (kernel :268-329). Every row of g_* is ASSIGNED: the
 * gradient for surfels with radii > 0, zeros for the others and for SH coefficients above the active degree (the
 * reference relies on its caller's zero-fill for those), so the outputs need no initialisation. grad_mean2D[P,2] is
 * read and then overwritten in place with the densification proxy (rows with radii <= 0 are left as they are).
 * g_shs / g_sh_rest may be NULL. */
int fsgs_gs_2d_preprocess_backward(int P, int W, int H, int sh_degree, int n_sh, const float* means3D,
    const float* scales, const float* rotations, const float* shs, const float* sh_rest, const float* Tw2v,
    const float* Tv2c, const float* campos, const float* trans_mat, const int32_t* radii, const float* colors,
    float* grad_mean2D, const float* grad_trans, const float* grad_colors, const float* grad_normal_opacity,
    float* g_means3D, float* g_scales, float* g_rot, float* g_opac, float* g_shs, float* g_sh_rest, void* stream);

/* gs_2d_compute_transmat_forward / gs_2d_compute_trans_mat_backward -- gs_2d_preprocess.cu:512-550, :564-599. */
int fsgs_gs_2d_compute_transmat_forward(int P, int W, int H, const float* means3D, const float* scales,
    const float* rotations, const float* Tw2v, const float* Tw2c, float* trans_mat, float* normals, void* stream);
int fsgs_gs_2d_compute_transmat_backward(int P, int W, int H, const float* means3D, const float* scales,
    const float* rotations, const float* Tw2v, const float* Tw2c, const float* g_mat, const float* g_normals,
    float* g_means3D, float* g_scales, float* g_rot, void* stream);

/* ---- tile binning: GS_prepare -- fast_2d_gs/_C/src/gaussian_splatting/gaussian_prepare.cu:222-308 -------------- */

/* Phase 1: inclusive scan of tiles_touched[P] into point_offsets[P] (int64) and the instance count R on the host
 * (gaussian_prepare.cu:231-239). Blocks until R is known. */
size_t fsgs_gs_prepare_scan_workspace_bytes(int P);
int fsgs_gs_prepare_scan(int P, const int32_t* tiles_touched, int64_t* point_offsets, void* workspace,
                         size_t workspace_bytes, int64_t* num_rendered_host, void* stream);

/* Phase 2: key duplication, stable sort on bits [0, 32 + msb(T)), tile ranges (gaussian_prepare.cu:47-83, 254-277,
 * 192-220). ranges[T,2] int64 (empty tile = (0,0)), point_list[R] int32. sorted_keys_out[R] (optional) receives the
 * sorted 64-bit keys (tile << 32 | depth bits). Two caller buffers, neither needs clearing: `workspace` of
 * fsgs_gs_prepare_fill_workspace_bytes(R) bytes for the unsorted entries, and `bins` of
 * fsgs_gs_prepare_bins_bytes(P, W, H) bytes for the per-tile instance counts of the surfel slices (known before R is). */
size_t fsgs_gs_prepare_fill_workspace_bytes(int64_t R);
size_t fsgs_gs_prepare_bins_bytes(int P, int W, int H);
int fsgs_gs_prepare_sort_bits(int W, int H);
int fsgs_gs_prepare_fill(int P, int W, int H, const float* means2D, const float* depths, const int32_t* radii,
                         const int64_t* point_offsets, int64_t R, int64_t* ranges, int32_t* point_list,
                         int64_t* sorted_keys_out, void* bins, size_t bins_bytes, void* workspace,
                         size_t workspace_bytes, void* stream);

/* The same two phases cut where the host has to wait, for callers that want the device to stay busy meanwhile (no
 * counterpart in the reference, which blocks inside GS_prepare). fsgs_gs_prepare_scan_begin queues the scan and the
 * copy of the instance count into *num_rendered_host (page-locked memory, or the copy is not asynchronous) and
 * returns; fsgs_gs_prepare_scan_end blocks the calling host thread until that copy has landed (one scan in flight per
 * host thread). Work queued on the stream in between runs while the host waits and allocates: fsgs_gs_prepare_count is
 * the part of the fill that does not need the count (counts the instances per tile into `bins`, writes the final
 * ranges[T,2]; the caller keeps `bins` until the fill has run); fsgs_gs_prepare_fill_counted is the rest (scatter +
 * per-tile sort). scan_begin + scan_end == fsgs_gs_prepare_scan, count + fill_counted == fsgs_gs_prepare_fill.
 * records (optional): the packed per-surfel records fsgs_gs_2d_preprocess_forward wrote; the scan stores every surfel's
 * exclusive offset into the last word of its record, where the blend backward's ordered-sum path looks for it. */
int fsgs_gs_prepare_scan_begin(int P, const int32_t* tiles_touched, int64_t* point_offsets, void* workspace,
                               size_t workspace_bytes, int64_t* num_rendered_host, float* records, void* stream);
int fsgs_gs_prepare_scan_end(void);
int fsgs_gs_prepare_count(int P, int W, int H, const float* means2D, const int32_t* radii, int64_t* ranges,
                          void* bins, size_t bins_bytes, void* stream);
int fsgs_gs_prepare_fill_counted(int P, int W, int H, const float* means2D, const float* depths, const int32_t* radii,
                                 int64_t R, int64_t* ranges, int32_t* point_list, int64_t* sorted_keys_out,
                                 void* bins, size_t bins_bytes, void* workspace, size_t workspace_bytes, void* stream);

/* The same two phases over the tiles a surfel can actually reach (no counterpart in the reference, whose lists hold
 * every tile of a surfel's rectangle). fsgs_gs_2d_cull_masks evaluates the blend kernels' own bound -- the padded
 * footprint box and diagonal slabs of the alpha >= 1/255 region -- once per surfel from its packed record
 * (records[P,20]: transform, centre, opacity) and leaves masks[P]: a bit per tile of the surfel's rectangle, row-major,
 * set when some pixel of the tile may blend the surfel (rectangles above 32 tiles: all bits set, kept whole). The
 * culled phases leave the other instances out of the tile lists. Images, maps and gradients are the same as with the
 * full lists; the lists are shorter (point_list keeps its length R, the entries behind the last tile's end are unused),
 * n_contrib counts positions of the shorter lists, and the ordered-sum path of the backward must be entered through
 * fsgs_gs_2d_render_backward_culled with the same masks. */
int fsgs_gs_2d_cull_masks(int P, int W, int H, const float* records, const int32_t* radii, uint32_t* masks,
                          void* stream);
/* The masks of 3D Gaussians, from what fsgs_gs_preprocess_forward leaves (means2D[P,2], conic_opacity[P,4], radii[P]):
 * the ellipse on which gaussian_rasterize's alpha reaches 1/255, tested against each tile of the rectangle. The culled
 * binning phases and the culled backwards take them as they take the surfels' masks. */
int fsgs_gs_cull_masks(int P, int W, int H, const float* means2D, const float* conic_opacity, const int32_t* radii,
                       uint32_t* masks, void* stream);
int fsgs_gs_prepare_count_culled(int P, int W, int H, const float* means2D, const int32_t* radii,
                                 const uint32_t* masks, int64_t* ranges, void* bins, size_t bins_bytes, void* stream);
int fsgs_gs_prepare_fill_counted_culled(int P, int W, int H, const float* means2D, const float* depths,
                                        const int32_t* radii, const uint32_t* masks, int64_t R, int64_t* ranges,
                                        int32_t* point_list, int64_t* sorted_keys_out, void* bins, size_t bins_bytes,
                                        void* workspace, size_t workspace_bytes, void* stream);

/* ---- per-tile alpha blend ------------------------------------------------------------------------------------- */

/* Optional accelerator without a counterpart in the reference: packs what the blend kernels gather per surfel
 * (trans_mat, means2D, opacity, normal, colour, and -- when given -- radius and prefix-scan offset) into one 80-byte
 * record, records[P,20] floats, 16-byte aligned. Passing `records` to fsgs_gs_2d_render_forward / _backward makes them
 * read one record per list entry instead of four tensors; results are identical. Pass radii here if the backward is
 * going to use its ordered-sum path (it takes the radius from the record, and the offset too when point_offsets is
 * given here or fsgs_gs_prepare_scan_begin has stored it; a record without an offset holds -1 there and the backward
 * falls back to its point_offsets argument).
 * fsgs_gs_2d_preprocess_forward writes the same record itself when given a records buffer; this entry serves callers
 * whose per-surfel tensors come from elsewhere. */
int fsgs_gs_2d_pack_records(int P, const float* means2D, const float* colors, const float* normal_opacity,
    const float* trans_mat, const int32_t* radii, const int64_t* point_offsets, float* records, void* stream);

/* GS_2D_render_forward -- fast_2d_gs/_C/src/gaussian_splatting/gs_2d_redner.cu:541-629 (kernel :28-236).
 * out_color[3,H,W] out_opacity[H,W] n_contrib[2,H,W]; unless only_image: out_extras[9,H,W]; with trans_mat_t2:
 * out_flow[H,W,2]. accum_* [P] are accumulated into (atomics), all other outputs are fully written. */
int fsgs_gs_2d_render_forward(int P, int W, int H, double near_n, double far_n, int only_image,
    const float* means2D, const float* colors, const float* normal_opacity, const float* trans_mat,
    const int32_t* point_list, const int64_t* ranges, const float* trans_mat_t2, int32_t* accum_max_count,
    float* accum_weights_p, int32_t* accum_weights_count, float* out_color, float* out_opacity, float* out_extras,
    float* out_flow, int32_t* n_contrib, const float* records, void* stream);

/* GS_2D_render_backward -- gs_2d_redner.cu:631-717 (kernel :238-539). Two ways of summing a surfel's gradient over the
 * tiles it touches:
 *  - point_offsets == NULL: device-scope float atomics, as the reference does; g_colors[P,3] g_means2D[P,2]
 *    g_trans[P,3,3] g_normal_opacity[P,4] MUST be zero-filled by the caller.
 *  - point_offsets[P] (the prefix scan fsgs_gs_prepare_scan produced for this point_list) with radii[P], R and a workspace
 *    of fsgs_gs_2d_render_backward_workspace_bytes(R): every (surfel, tile) instance writes one record at its position
 *    in surfel order and a second kernel sums each surfel's records in a fixed order. No atomics to HBM, the four outputs
 *    are fully written and the workspace needs no clearing (every instance's record is written, zeros included).
 *    Requires the point_list of fsgs_gs_prepare_fill for these means2D /
 *    radii (the position of an instance is recomputed from the surfel's tile rectangle). */
size_t fsgs_gs_2d_render_backward_workspace_bytes(int64_t R);
int fsgs_gs_2d_render_backward(int P, int W, int H, double near_n, double far_n, const float* means2D,
    const float* normal_opacity, const float* colors, const float* trans_mat, const float* trans_mat_t2,
    const float* out_opacity, const float* out_extras, const float* out_flow, const float* dL_dpix,
    const float* dL_dopacity, const float* dL_dextras, const float* dL_dflow, const int64_t* ranges,
    const int32_t* point_list, const int32_t* n_contrib, float* g_colors, float* g_means2D, float* g_trans,
    float* g_normal_opacity, int64_t R, const int64_t* point_offsets, const int32_t* radii, void* workspace,
    size_t workspace_bytes, const float* records, void* stream);
/* The same over lists built by fsgs_gs_prepare_*_culled (no counterpart in the reference): the sum of the ordered
 * records reads the binning's keep masks (required with point_offsets) and skips the positions of a surfel's span that
 * were left out of every list, which nobody wrote. R stays the scan's instance count. */
int fsgs_gs_2d_render_backward_culled(int P, int W, int H, double near_n, double far_n, const float* means2D,
    const float* normal_opacity, const float* colors, const float* trans_mat, const float* trans_mat_t2,
    const float* out_opacity, const float* out_extras, const float* out_flow, const float* dL_dpix,
    const float* dL_dopacity, const float* dL_dextras, const float* dL_dflow, const int64_t* ranges,
    const int32_t* point_list, const int32_t* n_contrib, float* g_colors, float* g_means2D, float* g_trans,
    float* g_normal_opacity, int64_t R, const int64_t* point_offsets, const int32_t* radii, void* workspace,
    size_t workspace_bytes, const float* records, const uint32_t* keep_masks, void* stream);

/* ---- "fast" surfel path: transform through camera intrinsics Tv2s[3,3], adjugate-based intersection, fused
 * corner-test binning. Optical flow (trans_mat_t2) is carried by the two blend entry points below. ---- */

/* gs_2d_fast_preprocess_forward (per-surfel part) -- gs_2d_fast_preprocess.cu:160-262, host :611-709.
 * Same outputs as fsgs_gs_2d_preprocess_forward plus inverse_m[P,3,3] (adjugate of trans_mat). Only the z translation
 * of Tw2v enters the transform, as in the reference (:95). keep_masks[P] (optional, no counterpart in the reference)
 * receives the binning's corner test for every tile of a rectangle of at most 32 tiles, bit x * h + y of the surfel's
 * word (x-major over the w x h rectangle, the order of its key span; larger rectangles: all bits set). The binning and
 * the ordered-sum backwards take the masks back and then repeat the test, and its set-up, only for larger rectangles:
 * same lists, keys, ranges and sums. */
int fsgs_gs_2d_fast_preprocess_forward(int P, int W, int H, int sh_degree, int n_sh, const float* means3D,
    const float* scales, const float* rotations, const float* opacities, const float* shs, const float* sh_rest,
    const float* Tw2v, const float* Tv2s, const float* campos, const float* trans_precomp, const uint8_t* culling,
    int means2D_preserve, float* means2D, float* colors, float* trans_mat, float* inverse_m, float* normal_opacity,
    float* depths, int32_t* radii, int32_t* tiles_touched, uint32_t* keep_masks, void* stream);

/* Binning half of gs_2d_fast_preprocess_forward -- gs_2d_fast_preprocess.cu:264-327 (duplicateWithKeys with the
 * per-tile corner test, x-major, unused slots padded with key = T << 32 / value = -1), :711-778 (sort on
 * 32 + msb(T + 1) bits, ranges). The prefix scan is fsgs_gs_prepare_scan. point_list[R] keeps the -1 padding entries
 * at its tail. Workspace: fsgs_gs_2d_fast_prepare_fill_workspace_bytes(P, W, H, R) (no counterpart in the reference);
 * with it the kept instances are counted, scattered and sorted per tile and the padding entries are written behind
 * them -- the same lists, keys and ranges as the reference's device-wide sort of the padded key array, which is what a
 * workspace of only fsgs_gs_prepare_fill_workspace_bytes(R) bytes (and any grid above 16 384 tiles) still gets.
 * keep_masks (optional): what fsgs_gs_2d_fast_preprocess_forward left for these surfels. */
int fsgs_gs_2d_fast_prepare_sort_bits(int W, int H);
size_t fsgs_gs_2d_fast_prepare_fill_workspace_bytes(int P, int W, int H, int64_t R);
int fsgs_gs_2d_fast_prepare_fill(int P, int W, int H, const float* means2D, const float* inverse_m,
    const float* depths, const float* opacities, const int32_t* radii, const int64_t* point_offsets, int64_t R,
    int64_t* ranges, int32_t* point_list, int64_t* sorted_keys_out, void* workspace, size_t workspace_bytes,
    const uint32_t* keep_masks, void* stream);

/* gs_2d_fast_preprocess_backward -- gs_2d_fast_preprocess.cu:536-609, host :784-852. grad_mean2D is read, then
 * overwritten with the densification proxy computed from the ACCUMULATED transform gradient (:606-608). */
int fsgs_gs_2d_fast_preprocess_backward(int P, int W, int H, int sh_degree, int n_sh, const float* means3D,
    const float* scales, const float* rotations, const float* shs, const float* sh_rest, const float* Tw2v,
    const float* Tv2s, const float* campos, const float* trans_mat, const int32_t* radii, const float* colors,
    float* grad_mean2D, const float* grad_trans, const float* grad_inv_m, const float* grad_colors,
    const float* grad_normal_opacity, float* g_means3D, float* g_scales, float* g_rot, float* g_opac, float* g_shs,
    float* g_sh_rest, void* stream);

/* gs_2d_fast_compute_transmat_forward / gs_2d_fast_compute_trans_mat_backward -- gs_2d_fast_preprocess.cu:862-966
 * (device functions :60-140). */
int fsgs_gs_2d_fast_compute_transmat_forward(int P, const float* means3D, const float* scales,
    const float* rotations, const float* Tw2v, const float* Tv2s, float* trans_mat, float* normals, void* stream);
int fsgs_gs_2d_fast_compute_transmat_backward(int P, const float* means3D, const float* scales,
    const float* rotations, const float* Tw2v, const float* Tv2s, const float* g_mat, const float* g_normals,
    float* g_means3D, float* g_scales, float* g_rot, void* stream);

/* GS_2D_fast_render_forward -- gs_2d_fast_redner.cu:839-953 (kernel :22-271). out_extras[8,H,W]. With
 * trans_mat_t2[P,3,3] (optional, not with only_image) out_flow[H,W,2] is the weighted displacement to the second time
 * step divided by the final opacity, 0 where that is 0 (:247-263). With bucket_offset[T] (inclusive cumsum of
 * ceil(len/32) per tile) the kernel also writes max_contrib[T], bucket_to_tile[B], sampled_T[B,256],
 * sampled_acc[B,3,256], sampled_aux[B,C,256] with C = 10 when trans_mat_t2 is given (channels 8, 9: the undivided flow
 * sums) and 8 otherwise (state before every 32nd list entry, for pixels still blending; channel 4 of sampled_aux is
 * never written, as in the reference). */
int fsgs_gs_2d_fast_render_forward(int P, int W, int H, double near_n, double far_n, int only_image,
    const float* means2D, const float* colors, const float* normal_opacity, const float* trans_mat,
    const float* inverse_m, const int32_t* point_list, const int64_t* ranges, const float* trans_mat_t2,
    int32_t* accum_max_count, float* accum_weights_p, int32_t* accum_weights_count, const int64_t* bucket_offset,
    float* out_color, float* out_opacity, float* out_extras, float* out_flow, int32_t* n_contrib,
    int32_t* max_contrib, int32_t* bucket_to_tile, float* sampled_T, float* sampled_acc, float* sampled_aux,
    void* stream);

/* GS_2D_fast_render_backward -- gs_2d_fast_redner.cu:955-1074. per_splat_form = 0: kernel :273-561 (image, opacity,
 * aux 0-5); per_splat_form = 1: the channel set of kernel :563-837 (image, opacity, aux 0-4 and 6-7, no distortion).
 * dL_dflow[H,W,2] (optional, with trans_mat_t2 and out_flow) is taken as the gradient of the UNDIVIDED flow sum, as both
 * reference kernels take it (:366, :704); the per-splat form additionally lowers the opacity map's gradient by
 * (out_flow . dL_dflow), the effect of the reference subtracting the divided flow from its partial sums (:706). No
 * gradient is produced for trans_mat_t2. With point_offsets == NULL all five gradient outputs MUST be zero-filled by the
 * caller (device-scope atomics, as in the reference). With point_offsets[P] (the inclusive prefix scan of tiles_touched
 * that fsgs_gs_prepare_scan returns), radii[P], R = point_offsets[P-1] (the length of point_list, padding included) and
 * a 16-byte aligned workspace of fsgs_gs_2d_fast_render_backward_workspace_bytes(R) bytes (no counterpart in the
 * reference) every row of the outputs is ASSIGNED from per-(surfel, tile) records added in a fixed order. The
 * workspace needs no clearing: every list entry's record is written on every call, and the sum repeats the binning's
 * corner test (or reads its verdicts from keep_masks, optional, as fsgs_gs_2d_fast_preprocess_forward left them) so
 * that it reads no other position of a surfel's key span. */
size_t fsgs_gs_2d_fast_render_backward_workspace_bytes(int64_t R);
int fsgs_gs_2d_fast_render_backward(int P, int W, int H, double near_n, double far_n, int per_splat_form,
    const float* means2D, const float* normal_opacity, const float* colors, const float* trans_mat,
    const float* inverse_m, const float* trans_mat_t2, const float* out_opacity, const float* out_extras,
    const float* out_flow, const float* dL_dpix, const float* dL_dopacity, const float* dL_dextras,
    const float* dL_dflow, const int64_t* ranges, const int32_t* point_list, const int32_t* n_contrib,
    float* g_colors, float* g_means2D, float* g_trans, float* g_inv, float* g_normal_opacity, int64_t R,
    const int64_t* point_offsets, const int32_t* radii, void* workspace, size_t workspace_bytes,
    const uint32_t* keep_masks, void* stream);

/* The per-splat decomposition of gs_2d_fast_redner.cu:563-837 itself (fsgs_gs_2d_fast_render_backward with
 * per_splat_form = 1 returns the same derivative through the back-to-front kernel, which is faster here): a lane owns
 * one list entry and keeps its 21 sums in registers, the tile's pixels pass through the lanes carrying their
 * front-to-back blending state, started from the forward's snapshots (images[3,H,W], max_contrib[T], bucket_offset[T],
 * bucket_to_tile[B], sampled_T[B,256], sampled_acc[B,3,256], sampled_aux[B,8,256], all as the forward wrote them). One
 * wavefront takes two 32-entry buckets; B = number of buckets. No optical flow in this form. Outputs and the optional
 * ordered-sum arguments as fsgs_gs_2d_fast_render_backward. */
int fsgs_gs_2d_fast_render_bucket_backward(int P, int W, int H, double near_n, double far_n, int B,
    const float* means2D, const float* normal_opacity, const float* colors, const float* trans_mat,
    const float* inverse_m, const float* images, const float* out_opacity, const float* out_extras,
    const int32_t* n_contrib, const int32_t* max_contrib, const int64_t* bucket_offset,
    const int32_t* bucket_to_tile, const float* sampled_T, const float* sampled_acc, const float* sampled_aux,
    const float* dL_dpix, const float* dL_dopacity, const float* dL_dextras, const int64_t* ranges,
    const int32_t* point_list, float* g_colors, float* g_means2D, float* g_trans, float* g_inv,
    float* g_normal_opacity, int64_t R, const int64_t* point_offsets, const int32_t* radii, void* workspace,
    size_t workspace_bytes, const uint32_t* keep_masks, void* stream);

/* gs_2d_topk_weights -- fast_2d_gs/_C/src/gaussian_splatting/gaussian_topk.cu:230-250 (kernel :95-210).
 * top_indices[H,W,topk] int32 (-1 = empty), top_weights[H,W,topk] descending blend weights alpha*T; topk <= 16. */
int fsgs_gs_2d_topk_weights(int topk, int P, int W, int H, double near_n, double far_n, const float* means2D,
    const float* normal_opacity, const float* trans_mat, const int64_t* ranges, const int32_t* point_list,
    int32_t* top_indices, float* top_weights, void* stream);

/* ---- spherical harmonics and encoders ------------------------------------------------------------------------- */

/* SH_to_RGB_forward / SH_to_RGB_backward -- fast_2d_gs/_C/src/ops_3d/spherical_harmonics.cu:15-41, :68-102.
 * grad_campos[3] is accumulated into; grad_dir[P,3] and grad_sh[P,F,3] are assigned (first (degree+1)^2 rows). */
int fsgs_sh_to_rgb_forward(int P, int F, int degree, int clamp, const float* pos, const float* campos,
                           const float* sh, float* rgb, void* stream);
int fsgs_sh_to_rgb_backward(int P, int F, int degree, int clamp, const float* pos, const float* campos,
    const float* sh, const float* rgb, const float* grad_rgb, float* grad_dir, float* grad_campos, float* grad_sh,
    void* stream);

/* Element types of the `_typed` entry points below. The reference dispatches these small operators on the tensor's
 * scalar type (AT_DISPATCH_FLOATING_TYPES[_AND_HALF]); a `_typed` entry takes the same buffers as untyped addresses plus
 * this selector. FSGS_DTYPE_F16 is IEEE binary16 storage with single-precision arithmetic. */
#define FSGS_DTYPE_F32 0
#define FSGS_DTYPE_F64 1
#define FSGS_DTYPE_F16 2

/* sh_encode_forward / sh_encode_backward -- fast_2d_gs/_C/src/nerf/shencoder.cu:657-691 (float, double and half, :667,
 * :688). in[B,D>=3], out[B,(C+1)^2]; the backward writes the first three components of every grad_in row. The
 * coefficients are single-precision literals for every element type, as at shencoder.cu:36-176. */
int fsgs_sh_encode_forward(int B, int D, int C, const float* in, float* out, void* stream);
int fsgs_sh_encode_backward(int B, int D, int C, const float* grad, const float* in, float* grad_in, void* stream);
int fsgs_sh_encode_forward_typed(int dtype, int B, int D, int C, const void* in, void* out, void* stream);
int fsgs_sh_encode_backward_typed(int dtype, int B, int D, int C, const void* grad, const void* in, void* grad_in,
                                  void* stream);

/* freq_encode_forward / freq_encode_backward -- fast_2d_gs/_C/src/nerf/freqencoder.cu:63-104 (float and double, :76,
 * :98). out[B, Din * (2 * degree + include_input)] laid out [x | sin 2^0 s x | cos 2^0 s x | sin 2^1 s x | ...]. For
 * double tensors the scaled angle and its sine / cosine are single precision (scalbnf at freqencoder.cu:27-28). */
int fsgs_freq_encode_forward(int B, int Din, int degree, int include_input, double scale, const float* in,
                             float* out, void* stream);
int fsgs_freq_encode_backward(int B, int Din, int degree, int include_input, double scale, const float* grad,
                              const float* outv, float* gin, void* stream);
int fsgs_freq_encode_forward_typed(int dtype, int B, int Din, int degree, int include_input, double scale,
                                   const void* in, void* out, void* stream);
int fsgs_freq_encode_backward_typed(int dtype, int B, int Din, int degree, int include_input, double scale,
                                    const void* grad, const void* outv, void* gin, void* stream);

/* ---- nearest points, K-NN, LBS, optimiser ---------------------------------------------------------------------- */

/* cdist_top / cdist_top_backward -- fast_2d_gs/_C/src/other/cdist_top.cu:34-84, :107-154. x[B,N,D] y[B,M,D] ->
 * dist[B,N] (Euclidean), index[B,N] int64. Ties: smallest keeps the LAST equal minimum, largest the FIRST equal
 * maximum. The backward assigns g1[B,N,D] and accumulates into caller-zeroed g2[B,M,D]. */
int fsgs_cdist_top_forward(int B, int N, int M, int D, int largest, const float* x, const float* y, float* dist,
                           int64_t* index, void* stream);
int fsgs_cdist_top_backward(int B, int N, int M, int D, const float* p1, const float* p2, const float* dist,
                            const int64_t* index, const float* gdist, float* g1, float* g2, void* stream);
/* The same for float or double points (cdist_top.cu:48, :116); dist, gdist, g1, g2 have the points' element type. */
int fsgs_cdist_top_forward_typed(int dtype, int B, int N, int M, int D, int largest, const void* x, const void* y,
                                 void* dist, int64_t* index, void* stream);
int fsgs_cdist_top_backward_typed(int dtype, int B, int N, int M, int D, const void* p1, const void* p2,
                                  const void* dist, const int64_t* index, const void* gdist, void* g1, void* g2,
                                  void* stream);

/* K nearest rows of y[M,D] for every row of x[N,D] (K <= 16): dist2[N,K] squared distances ascending, index[N,K]
 * int64, ties -> lower index first; slots beyond M hold (-1, -1). Replaces the reference's call
 * pytorch3d.ops.knn_points(points[None], sp_points[None], K=K) at fast_2d_gs/network.py:504. */
int fsgs_knn_topk(int N, int M, int D, int K, const float* x, const float* y, float* dist2, int64_t* index,
                  void* stream);

/* The superpoint warp of fast_2d_gs/network.py:498-573 in one call: neighbour weights (calc_LBS_weight, :507-517) and
 * the blend (warp, :545-573) over the K neighbours index[N,K] (int64, from fsgs_knn_topk; slots outside [0, M) get
 * weight 0 and take no part in the normalisation).
 * weight_mode selects what pair_in[N,K] is and how weights are formed:
 *   0  LBS_method 'dist' (:517): pair_in = squared distances, w = softmax(-d2 / temperature);
 *   1  'kernel' / 'weighted_kernel' (:507-513): pair_in = squared distances, u = exp(-d2 / (2 r_j^2)) [* sigmoid(omega_j)]
 *      + 1e-7, w = u / sum u, with r_j = exp(sp_log_radius[j]) (the reference's raw _sp_radius, :255-256) and omega_j =
 *      sp_weight_logit[j] (raw _sp_weight, :259-260; NULL for 'kernel');
 *   2  'W' (:514-515): pair_in = the caller's gather sp_W[n, index[n, k]], w = softmax(pair_in);
 *   3  pair_in = finished weights, used as they are (warp() called on weights the caller computed).
 * warp_mode follows the branches of warp():
 *   0  no local rotation (sp_rot == NULL; the default configuration, :563-564): d_xyz = sum_k w_k sp_t[j_k];
 *   1  'LBS' with sp_rot[M,4] (:545-556): q_j = normalize(sp_rot_j + (0,0,0,1)), d_xyz = sum_k w_k (R(q_j) p + sp_t_j) - p;
 *   2  'LBS_c': as 1 with sp_t_j replaced by sp_t_j + c_j - R(q_j) c_j, c = sp_points (:548-549).
 * Always: d_rot[N,4] = sum_k w_k sp_r[j_k] (apply_rotate 'add', :565-566), d_scale[N,S] = sum_k w_k sp_s[j_k] (S <= 4; S = 0
 * and NULL pointers when the net predicts no scale residual). weights_out[N,K] is optional. K <= 16. */
size_t fsgs_lbs_blend_workspace_bytes(int M);
int fsgs_lbs_blend(int N, int M, int K, int warp_mode, int weight_mode, double temperature, const float* points,
    const float* sp_points, const float* sp_t, const float* sp_rot, const float* sp_r, const float* sp_s, int S,
    const float* pair_in, const int64_t* index, const float* sp_log_radius, const float* sp_weight_logit,
    float* weights_out, float* d_xyz, float* d_rot, float* d_scale, void* workspace, size_t workspace_bytes,
    void* stream);

/* Backward of fsgs_lbs_blend. The reference has no kernel for it: torch autograd differentiates
 * fast_2d_gs/network.py:507-517 and :545-573 op by op. Inputs as in the forward plus g_xyz[N,3], g_rot[N,4],
 * g_scale[N,S]. Every output element is written: g_points[N,3] (optional; zeros in warp mode 0), g_pair[N,K] (the
 * gradient of pair_in: of the squared distances in weight modes 0 and 1, of the logits in mode 2, of the weights in
 * mode 3), g_sp_points[M,3] (optional; the pivot term of warp mode 2, zeros otherwise -- the dependence of the distances
 * on sp_points goes through g_pair and fsgs_knn_topk_backward), g_sp_t[M,3], g_sp_rot[M,4] (warp modes 1, 2), g_sp_r[M,4],
 * g_sp_s[M,S], and in weight mode 1 g_log_radius[M] and (optional, with sp_weight_logit) g_weight_logit[M].
 * Per-control-point sums are taken without float atomics, in a fixed order, when M <= 1024, K <= 4 and M * columns <=
 * 11264 (columns = 7 + S, + 9 with a rotation, + 2 in weight mode 1); larger cases use LDS float atomics inside a block
 * (up to 36864 table cells) or device-scope float atomics, whose last bits can differ between runs. */
size_t fsgs_lbs_blend_backward_workspace_bytes(int N, int M, int S);
int fsgs_lbs_blend_backward(int N, int M, int K, int warp_mode, int weight_mode, double temperature,
    const float* points, const float* sp_points, const float* sp_t, const float* sp_rot, const float* sp_r,
    const float* sp_s, int S, const float* pair_in, const int64_t* index, const float* sp_log_radius,
    const float* sp_weight_logit, const float* g_xyz, const float* g_rot, const float* g_scale, float* g_points,
    float* g_pair, float* g_sp_points, float* g_sp_t, float* g_sp_rot, float* g_sp_r, float* g_sp_s,
    float* g_log_radius, float* g_weight_logit, void* workspace, size_t workspace_bytes, void* stream);

/* Backward of fsgs_knn_topk's squared distances (what autograd through pytorch3d.ops.knn_points gives at
 * fast_2d_gs/network.py:504): g_x[N,D] (optional) = sum_k 2 g_dist2[n,k] (x_n - y_index), g_y[M,D] = minus the same
 * summed over the queries that selected the row. Slots with index -1 are skipped. Both outputs fully written. */
size_t fsgs_knn_topk_backward_workspace_bytes(int N, int M, int D);
int fsgs_knn_topk_backward(int N, int M, int D, int K, const float* x, const float* y, const int64_t* index,
    const float* g_dist2, float* g_x, float* g_y, void* workspace, size_t workspace_bytes, void* stream);

/* ---- 3D-Gaussian (EWA) path ------------------------------------------------------------------------------------ */

/* gs_preprocess_forward -- fast_2d_gs/_C/src/gaussian_splatting/gaussian_preprocess.cu:372-466 (kernel :44-128):
 * scales[P,3], rotations[P,4] (x,y,z,w, used as given), opacities[P,1], shs[P,n_sh,3] (or shs[P,1,3] + sh_rest, or
 * colours[P,3] with sh_degree < 0), Tw2v, Tv2c [4,4], campos[3], tan(FoV/2) per axis -> means2D[P,2] (pixel - 0.5
 * convention unless is_opengl), depths[P], colors[P,3], radii[P], tiles_touched[P], cov3Ds[P,6], conic_opacity[P,4].
 * cov3D_precomp[P,6] (optional) replaces R S^2 R^T (cov3Ds is then not written and may be NULL: the reference's host
 * returns the pre-computed tensor itself, :424); cov2D_precomp[P,3] (optional) is used as the 2D covariance as it is,
 * without the 0.3 low-pass term (:76-78). Every row of every output is written; means2D_preserve keeps the caller's
 * means2D rows of Gaussians that are not rendered. culling: optional P bytes, non-zero = skip. */
int fsgs_gs_preprocess_forward(int P, int W, int H, int sh_degree, int n_sh, int is_opengl, const float* means3D,
    const float* scales, const float* rotations, const float* opacities, const float* shs, const float* sh_rest,
    const float* Tw2v, const float* Tv2c, const float* campos, double tan_fovx, double tan_fovy,
    const uint8_t* culling, const float* cov3D_precomp, const float* cov2D_precomp, int means2D_preserve,
    float* means2D, float* depths, float* colors, int32_t* radii, int32_t* tiles_touched, float* cov3Ds,
    float* conic_opacity, void* stream);

/* gs_preprocess_backward -- gaussian_preprocess.cu:567-636 (kernel :246-372, with gaussian_compute_cov2D.cu:64-186 and
 * gaussian_compute_cov3D.cu:76-118). grad_mean2D[P,2] is rewritten in place as (0.5 W g.x, +-0.5 H g.y) as in the
 * reference; grad_conic[P,4] carries dL/dconic and dL/dopacity. All gradient rows are assigned (zeros for Gaussians
 * that were not rendered). g_scales, g_rot, g_shs, g_sh_rest, g_cov are optional. cov3Ds[P,6] is the forward's output
 * (or the caller's pre-computed tensor) and g_cov is [P,6]; with cov2Ds[P,3] (the caller's pre-computed 2D covariances,
 * :293-301) g_cov is [P,3], nothing reaches the means through the covariance and g_scales / g_rot must be NULL.
 * g_Tw2v[4,4] (rows 0-2) and g_campos[3] (optional, :271, :318-355) are ADDED to, with float atomics. */
int fsgs_gs_preprocess_backward(int P, int W, int H, int sh_degree, int n_sh, int is_opengl, const float* means3D,
    const float* scales, const float* rotations, const float* shs, const float* sh_rest, const float* Tw2v,
    const float* Tv2c, const float* campos, double tan_fovx, double tan_fovy, const int32_t* radii,
    const float* colors, const float* cov3Ds, const float* cov2Ds, float* grad_mean2D, const float* grad_colors,
    const float* grad_conic, float* g_means3D, float* g_scales, float* g_rot, float* g_opac, float* g_shs,
    float* g_sh_rest, float* g_cov, float* g_Tw2v, float* g_campos, void* stream);

/* gaussian_topk_weights -- fast_2d_gs/_C/src/gaussian_splatting/gaussian_topk.cu:212-228 (kernel :12-93): per pixel
 * the topk (<= 16) largest blend weights of the 3D-Gaussian rasteriser and their Gaussian ids, descending;
 * top_indices[H,W,topk] int32 (-1 = empty slot), top_weights[H,W,topk], both fully written. */
int fsgs_gaussian_topk_weights(int topk, int P, int W, int H, const float* means2D, const float* conic_opacity,
    const int64_t* ranges, const int32_t* point_list, int32_t* top_indices, float* top_weights, void* stream);

/* gaussian_rasterize_extra_forward / gaussian_rasterize_extra_backward -- fast_2d_gs/_C/src/gaussian_splatting/
 * gaussian_rasterizer_extra.cu:317-339 and :341-365 (kernels :12-101, :103-209; bound by
 * renderer/gaussian_render.py:925-949): any number E >= 1 of per-Gaussian feature channels extras[P,E] blended with the
 * weights of a finished gaussian_rasterize_forward, whose n_contrib[H,W] bounds each pixel's traversal and whose
 * out_opacity[H,W] seeds the backward. out_pixels[H,W,E] is pixel-major and fully written (16-byte aligned when E is a
 * multiple of 4). The backward takes grad_out[H,W,E] and ADDS into whichever of grad_extras[P,E], grad_means2D[P,2],
 * grad_conic_opacity[P,4] is non-null (the reference's optional tensors); with all three null it does nothing. */
int fsgs_gaussian_rasterize_extra_forward(int P, int W, int H, int E, const float* extras, const float* means2D,
    const float* conic_opacity, const int64_t* ranges, const int32_t* point_list, const int32_t* n_contrib,
    float* out_pixels, void* stream);
int fsgs_gaussian_rasterize_extra_backward(int P, int W, int H, int E, const float* extras, const float* out_opacity,
    const float* grad_out, const float* means2D, const float* conic_opacity, const int64_t* ranges,
    const int32_t* point_list, const int32_t* n_contrib, float* grad_extras, float* grad_means2D,
    float* grad_conic_opacity, void* stream);

/* gs_compute_cov3D_forward / gs_compute_cov3D_backward -- fast_2d_gs/_C/src/gaussian_splatting/
 * gaussian_compute_cov3D.cu:122-161: cov3D[N,6] = upper triangle of R(q) diag(s^2) R(q)^T for q[N,4] (x, y, z, w, used as
 * given, not normalised) and s[N,3]; the backward writes g_q[N,4] and g_s[N,3] in full. */
int fsgs_gs_compute_cov3D_forward(int N, const float* q, const float* s, float* cov3D, void* stream);
int fsgs_gs_compute_cov3D_backward(int N, const float* q, const float* s, const float* g_cov3D, float* g_q, float* g_s,
                                   void* stream);

/* gs_compute_cov2D_forward / gs_compute_cov2D_backward -- gaussian_compute_cov2D.cu:186-248: cov2D[N,3] = (a, b, c) of
 * J W cov3D W^T J^T + 0.3 I with the view-space mean clamped to 1.3 x the field of view (W = rotation block of the
 * row-major Tw2v[4,4]); the backward takes dL/dcov2D[N,3] and writes g_cov3D[N,6] and g_mean[N,3] in full; g_vm[4,4]
 * (optional, :163-183, :223-227) gets the view matrix's gradient ADDED to its rows 0-2 with float atomics. */
int fsgs_gs_compute_cov2D_forward(int N, const float* cov3D, const float* mean, const float* Tw2v, double focal_x,
    double focal_y, double tan_fovx, double tan_fovy, float* cov2D, void* stream);
int fsgs_gs_compute_cov2D_backward(int N, const float* cov3D, const float* mean, const float* Tw2v, double focal_x,
    double focal_y, double tan_fovx, double tan_fovy, const float* g_cov2D, float* g_cov3D, float* g_mean,
    float* g_vm, void* stream);

/* gaussian_rasterize_forward -- gaussian_render.cu:212-293 (kernel :20-173). colors[P,3], extras[P,E] (E <= 4,
 * optional) -> out_color[3,H,W], out_opacity[H,W], out_extras[E,H,W], n_contrib[H,W]; every output element is written.
 * accum_weights_* as in the surfel forward; accum_max_count gets one count per pixel, for the Gaussian with the
 * largest weight (:166). With bucket_offset[T] (inclusive cumsum of ceil(len / 32) per tile) also max_contrib[T],
 * bucket_to_tile[B], sampled_T[B,256], sampled_ar[B,3+E,256]: the state before every 32nd list entry for pixels still
 * blending (the extra channels' running sums in channels 3.., where the reference indexes its colour array past its
 * end, :103). */
int fsgs_gaussian_rasterize_forward(int P, int W, int H, int E, const float* means2D, const float* conic_opacity,
    const float* colors, const float* extras, const int32_t* point_list, const int64_t* ranges,
    int32_t* accum_max_count, float* accum_weights_p, int32_t* accum_weights_count, const int64_t* bucket_offset,
    float* out_color, float* out_opacity, float* out_extras, int32_t* n_contrib, int32_t* max_contrib,
    int32_t* bucket_to_tile, float* sampled_T, float* sampled_ar, void* stream);

/* gaussian_rasterize_backward -- gaussian_render.cu:486-536 (kernel :296-444). g_means2D[P,2], g_conic_opacity[P,4],
 * g_colors[P,3], g_extras[P,E]. With point_offsets == NULL the per-Gaussian sums are accumulated with device-scope
 * atomics into the caller-zeroed outputs, as in the reference. With point_offsets[P] (the inclusive prefix scan of
 * tiles_touched that fsgs_gs_prepare_scan returns), radii[P], the instance count R and a 16-byte aligned workspace of
 * fsgs_gaussian_rasterize_backward_workspace_bytes(R) bytes (no counterpart in the reference) every row of the outputs
 * is ASSIGNED from per-(Gaussian, tile) records added in a fixed order: no zero fill, no atomics, and the sums do not
 * vary from run to run. */
size_t fsgs_gaussian_rasterize_backward_workspace_bytes(int64_t R);
/* For tile lists built by fsgs_gs_prepare_*_culled (masks: fsgs_gs_cull_masks; no counterpart in the reference): the
 * instances left out of the lists are staged by no block, so nobody writes their records. Call this on the workspace
 * before an ordered-sum backward (fsgs_gaussian_rasterize_backward / _fast_backward / _bucket_backward with
 * point_offsets); it zeroes exactly those records. The atomic path needs nothing. */
int fsgs_gaussian_rasterize_clear_culled(int P, int64_t R, const int64_t* point_offsets, const uint32_t* keep_masks,
                                         void* workspace, size_t workspace_bytes, void* stream);
int fsgs_gaussian_rasterize_backward(int P, int W, int H, int E, const float* means2D, const float* conic_opacity,
    const float* colors, const float* extras, const float* out_opacity, const int32_t* n_contrib,
    const float* dL_dpix, const float* dL_dout_extras, const float* dL_dout_opacity, const int32_t* point_list,
    const int64_t* ranges, float* g_means2D, float* g_conic_opacity, float* g_colors, float* g_extras, int64_t R,
    const int64_t* point_offsets, const int32_t* radii, void* workspace, size_t workspace_bytes, void* stream);

/* gaussian_rasterize_fast_backward -- gaussian_render.cu:760-812 (kernel :540-694): the reference's per-Gaussian
 * backward over the forward's bucket snapshots. It is the same derivative as gaussian_rasterize_backward and runs
 * that kernel here; the snapshot arguments must be present but are not read. With E > 0 the reference reads the extra
 * channels' upstream gradient into the wrong registers (:636); the gradient of what the forward computes is returned.
 * Outputs and the optional ordered-sum arguments as above. */
int fsgs_gaussian_rasterize_fast_backward(int P, int W, int H, int E, const float* means2D,
    const float* conic_opacity, const float* colors, const float* extras, const float* images,
    const float* out_extras, const float* out_opacity, const int32_t* n_contrib, const int32_t* max_contrib,
    const int64_t* bucket_offset, const int32_t* bucket_to_tile, const float* sampled_T, const float* sampled_ar,
    const float* dL_dpix, const float* dL_dout_extras, const float* dL_dout_opacity, const int32_t* point_list,
    const int64_t* ranges, float* g_means2D, float* g_conic_opacity, float* g_colors, float* g_extras, int64_t R,
    const int64_t* point_offsets, const int32_t* radii, void* workspace, size_t workspace_bytes, void* stream);

/* The per-Gaussian decomposition of gaussian_render.cu:540-694 itself (fsgs_gaussian_rasterize_fast_backward returns the
 * same derivative through the back-to-front kernel, which is faster here): a lane owns one list entry and keeps its
 * sums in registers, the tile's pixels pass through the lanes carrying their front-to-back blending state, started from
 * the forward's snapshots. One wavefront takes two 32-entry buckets; B = number of buckets (length of bucket_to_tile).
 * With point_offsets == NULL: one device-scope atomic per Gaussian, tile and component into caller-zeroed outputs (the
 * reference's :679-694); with point_offsets / radii / workspace every lane writes its record and the outputs are
 * assigned from the ordered sums, as above. */
int fsgs_gaussian_rasterize_bucket_backward(int P, int W, int H, int E, int B, const float* means2D,
    const float* conic_opacity, const float* colors, const float* extras, const float* images,
    const float* out_extras, const float* out_opacity, const int32_t* n_contrib, const int32_t* max_contrib,
    const int64_t* bucket_offset, const int32_t* bucket_to_tile, const float* sampled_T, const float* sampled_ar,
    const float* dL_dpix, const float* dL_dout_extras, const float* dL_dout_opacity, const int32_t* point_list,
    const int64_t* ranges, float* g_means2D, float* g_conic_opacity, float* g_colors, float* g_extras, int64_t R,
    const int64_t* point_offsets, const int32_t* radii, void* workspace, size_t workspace_bytes, void* stream);

/* ---- render epilogue -------------------------------------------------------------------------------------------- */

/* Everything fast_2d_gs/renderer/gs_2d_render.py:608-617 does per pixel after the blend, in one kernel: normals[3,H,W] =
 * extras[1:4] as row vectors times Tw2v[:3,:3]; depths[H,W] = nan_to_num(extras[4], 0, 0); surf_depth[H,W] =
 * nan_to_num(extras[0], 0, 0) * (1 - depth_ratio) + depth_ratio * depths; surf_normal[3,H,W] = depth_to_normal
 * (gs_2d_render.py:439-470: normalised cross product of the central differences of the back-projected surf_depth, zero
 * on the one-pixel border) times opacity; and, when composited is not NULL, composited[3,H,W] = images + (1 - opacity)
 * * background[3] (fast_2d_gs/network.py:725-726). Tw2v[4,4] must be affine (last row 0 0 0 1), Tv2c[4,4] is the
 * projection; both are read on the device. Every output element is written. */
int fsgs_gs_2d_epilogue_forward(int W, int H, double depth_ratio, const float* Tw2v, const float* Tv2c,
    const float* extras, const float* opacity, const float* images, const float* background, float* normals,
    float* depths, float* surf_depth, float* surf_normal, float* composited, void* stream);

/* Backward of the above (torch autograd in the reference). Any of the six upstream gradients may be NULL (= zero).
 * g_extras[9,H,W] is fully written (channels 6-8 zero); the opacity is treated as detached in surf_normal, as the
 * reference does, so g_opacity[H,W] (optional) only receives the composite's -sum_c g_composited[c] * background[c];
 * the gradient of `images` is g_composited itself. No gradient is produced for the camera matrices. */
int fsgs_gs_2d_epilogue_backward(int W, int H, double depth_ratio, const float* Tw2v, const float* Tv2c,
    const float* extras, const float* opacity, const float* background, const float* g_normals, const float* g_depths,
    const float* g_surf_depth, const float* g_surf_normal, const float* g_distortion, const float* g_composited,
    float* g_extras, float* g_opacity, void* stream);

/* simple_knn -- fast_2d_gs/_C/src/other/knn.cu:180-205 (kernels :57-178). points[P,3] -> mean_dist2[P]: the mean of
 * the three smallest squared distances from each point to the other points (exact search; with fewer than four
 * points the missing distances stay FLT_MAX, so the mean is FLT_MAX / 3 or overflows to inf as it does in the
 * reference). Every output element is written. */
size_t fsgs_simple_knn_workspace_bytes(int P);
int fsgs_simple_knn(int P, const float* points, float* mean_dist2, void* workspace, size_t workspace_bytes,
                    void* stream);

/* ---- fused SSIM ------------------------------------------------------------------------------------------------ */

/* fusedssim -- fast_2d_gs/_C/src/other/structural_similarity.cu:340-363 (kernel :187-277). img1, img2, ssim_map and
 * the three optional partial-derivative maps are [B,CH,H,W]; pass the three maps as NULL for train = false. Every
 * output element is written. */
int fsgs_fusedssim_forward(int B, int CH, int H, int W, double C1, double C2, const float* img1, const float* img2,
    float* ssim_map, float* dm_dmu1, float* dm_dsigma1_sq, float* dm_dsigma12, void* stream);

/* fusedssim_backward -- structural_similarity.cu:365-380 (kernel :279-338) -> dL_dimg1[B,CH,H,W], fully written. */
int fsgs_fusedssim_backward(int B, int CH, int H, int W, const float* img1, const float* img2, const float* dL_dmap,
    const float* dm_dmu1, const float* dm_dsigma1_sq, const float* dm_dsigma12, float* dL_dimg1, void* stream);

/* The photometric loss of a training step in two launches forward and one backward, with no image-sized intermediate:
 * loss = (1 - lambda) * mean|img - target| + lambda * (1 - mean SSIM(img, target)) -- the 'rgb' + 'ssim' terms of
 * fast_2d_gs/gaussian_splatting.py:321 / network.py:1027 with losses/ssim.py:24-47, which the reference evaluates as an
 * L1 in torch, the fusedssim map, two means and their autograd. img, target [B,CH,H,W]. loss_out[3] = (loss, L1 mean,
 * SSIM mean). dm_* are NULL (no gradient wanted) or the three [B,CH,H,W] maps the backward reads. The workspace holds
 * two partial sums per 32x32 block, added in a fixed order. The backward reads the upstream gradient of the scalar loss
 * from device memory (grad_loss[0]) and writes dL_dimg[B,CH,H,W] in full. */
size_t fsgs_image_loss_workspace_bytes(int B, int H, int W);
int fsgs_image_loss_forward(int B, int CH, int H, int W, double C1, double C2, double lambda_dssim, const float* img,
    const float* target, float* loss_out, float* dm_dmu1, float* dm_dsigma1_sq, float* dm_dsigma12, void* workspace,
    size_t workspace_bytes, void* stream);
int fsgs_image_loss_backward(int B, int CH, int H, int W, double lambda_dssim, const float* img, const float* target,
    const float* grad_loss, const float* dm_dmu1, const float* dm_dsigma1_sq, const float* dm_dsigma12, float* dL_dimg,
    void* stream);

/* fsgs_image_loss_forward for callers that cannot allocate device memory or carry a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference. Same inputs,
 * outputs and results as fsgs_image_loss_forward; the per-block partial sums go into a device array built into the
 * library (512 KiB per GPU, held until the process ends) instead of a workspace, so the call allocates nothing. Limit:
 * B * ceil(W / 32) * ceil(H / 32) <= fsgs_image_loss_static_max_blocks() (65536: one 8192 x 8192 image); larger inputs
 * are rejected with an error. All calls on one GPU share that array: calls that overlap on one GPU (two streams, two
 * host threads) race; calls on one stream are ordered. Nothing in the array has to be cleared between calls. */
int fsgs_image_loss_static_max_blocks(void);
int fsgs_image_loss_forward_static(int B, int CH, int H, int W, double C1, double C2, double lambda_dssim,
    const float* img, const float* target, float* loss_out, float* dm_dmu1, float* dm_dsigma1_sq, float* dm_dsigma12,
    void* stream);

/* Deformation MLP forward (bf16 MFMA, fp32 accumulate) -- fast_2d_gs/network.py:1757-1776 (SC_GS_DeformNetwork.forward,
 * fp32 there): n_layers x (Linear(256) + ReLU), input re-concatenated in front after layer `skip`, then n_out <= 32
 * linear outputs (the three heads stacked). in[B,Din] fp32 (already frequency-encoded), Din <= 96, width must be 256.
 * packed: bf16 weights from fsgs_pack_bf16, layer i as a [256][round_up(K_i,16)] matrix (K_0 = Din, K_{skip+1} =
 * Din + 256, else 256), then the heads as [32][256]; fsgs_mlp_packed_elems gives the total element count.
 * fsgs_pack_bf16 converts a row-major fp32 [rows][K] matrix to bf16, zero-padded to [rows_pad][K_pad] (multiples of 32
 * and 16), in the order the matrix cores read it: 32-row x 16-column tiles, tile (r / 32, k / 16) at
 * ((r / 32) * (K_pad / 16) + k / 16) * 512 elements, element (r, k) inside it at (r % 32 + 32 * ((k % 16) / 8)) * 8 +
 * k % 8.
 * bias[n_layers*256 + n_out] fp32. out[B,n_out] fp32. saved: NULL, or [n_layers][B][256] bf16 that receives every
 * layer's post-ReLU hidden state for fsgs_mlp_backward. */
int fsgs_pack_bf16(int rows, int K, int rows_pad, int K_pad, const float* src, uint16_t* dst, void* stream);
size_t fsgs_mlp_packed_elems(int Din, int n_layers, int skip);
/* Every buffer fsgs_mlp_forward / fsgs_mlp_backward read, refreshed from the fp32 torch.nn.Linear parameters in one
 * launch (the reference has no such step: its network runs on the fp32 parameters, network.py:1757-1776). Host arrays
 * of device pointers: weights[n_layers] ([256][K_l] row-major), biases[n_layers] ([256]), head_weights[n_heads]
 * ([head_rows[h]][256]), head_biases[n_heads]; the heads' rows are stacked in the order given (<= 32 rows together).
 * Outputs: packed (fsgs_mlp_packed_elems elements), packed_t (NULL, or (n_layers-1)*65536 elements), bias_out
 * [n_layers*256 + sum(head_rows)], heads_w_out [sum(head_rows)][256] fp32. */
int fsgs_mlp_pack_all(int Din, int n_layers, int skip, const float* const* weights, const float* const* biases,
    int n_heads, const float* const* head_weights, const float* const* head_biases, const int* head_rows,
    uint16_t* packed, uint16_t* packed_t, float* bias_out, float* heads_w_out, void* stream);
int fsgs_mlp_forward(int B, int Din, int width, int n_layers, int skip, int n_out, const float* in,
                     const uint16_t* packed, const float* bias, float* out, uint16_t* saved, void* stream);

/* Backward of fsgs_mlp_forward with respect to the weights and biases (torch autograd in the reference:
 * fast_2d_gs/network.py:1757-1776 is plain nn.Linear / relu). `saved` is the [n_layers][B][256] bf16 post-ReLU state the
 * forward wrote when given a non-NULL `saved`; packed_t holds, for layers 1 .. n_layers-1, the last 256 input columns
 * of the weight transposed to [256 in][256 out] bf16 (fsgs_pack_bf16 of the transposed slice); heads_w[n_out][256] and
 * g_out[B][n_out] are fp32. Outputs, fully written: g_w = the layers' [256][K_l] gradients back to back (unpadded,
 * K_0 = Din, K_{skip+1} = Din + 256, else 256) followed by the heads' [n_out][256]; g_b[n_layers*256 + n_out].
 * Operands are bf16, accumulation fp32. No gradient is produced for `in` directly; the workspace carries what a caller
 * needs to form it: after the call its first n_layers * B * 256 * 2 bytes hold dZ[n_layers][B][256] in bf16, the
 * gradient of every layer's pre-activation (masked by the stored state's zeros), so that
 * dL/d in = dZ[0] W_0 + dZ[skip+1] W_{skip+1}[:, :Din]. The rest of the workspace is scratch. */
size_t fsgs_mlp_backward_workspace_bytes(int B, int n_layers);
int fsgs_mlp_backward(int B, int Din, int width, int n_layers, int skip, int n_out, const float* in,
    const uint16_t* packed_t, const float* heads_w, const uint16_t* saved, const float* g_out, float* g_w, float* g_b,
    void* workspace, size_t workspace_bytes, void* stream);

/* ---- adaptive density control as stream compaction ------------------------------------------------------------- */
/* The reference changes the point set with torch indexing on the host side, one tensor and one Adam moment at a time
 * (fast_2d_gs/gaussian_splatting.py:497-637, fast_2d_gs/network.py:1156-1215, :1276-1282). Here a mask becomes an
 * ascending index list and every structural change is one table source_row[new_row] applied to all tensors at once. */

/* `mask[mask_or_keep]` -> indices: the ascending positions of the non-zero (invert = 0) or zero (invert = 1) bytes of
 * mask[P], i.e. torch.nonzero(mask) / torch.nonzero(~mask) (gaussian_splatting.py:526-527, :558). indices needs room
 * for P entries. Blocks until the count is on the host (torch's boolean indexing blocks in the same place). */
size_t fsgs_select_indices_workspace_bytes(int P);
int fsgs_select_indices(int P, const uint8_t* mask, int invert, int32_t* indices, void* workspace,
                        size_t workspace_bytes, int64_t* count_host, void* stream);

/* dst_t[r] = source_row[r] >= 0 ? src_t[source_row[r]] : zeros, for r < n_rows and every tensor t < n_tensors in one
 * launch (gaussian_splatting.py:524-551: `old[mask]`, `torch.cat`, the zero moments of new points). The three *_host
 * arrays are HOST arrays of n_tensors device pointers / row sizes in bytes; rows are contiguous. A tensor's source and
 * destination must not overlap. At most fsgs_gather_rows_max_tensors() tensors per call. */
int fsgs_gather_rows_max_tensors(void);
int fsgs_gather_rows(int n_tensors, const void* const* src_host, void* const* dst_host, const int64_t* row_bytes_host,
                     int64_t n_rows, const int32_t* source_row, void* stream);

/* densify_and_clone / densify_and_split selection -- gaussian_splatting.py:623-626, :612-615, :585-589. g = grad_accum /
 * denom with NaN -> 0; clone = |g| >= grad_threshold and max(scaling) <= scale_threshold; split = g >= grad_threshold
 * and max(scaling) > scale_threshold. scaling[P,S] holds ACTIVATED scales. Masks are bytes (0 / 1). */
int fsgs_densify_masks(int P, int S, const float* grad_accum, const float* denom, const float* scaling,
                       float grad_threshold, float scale_threshold, uint8_t* clone_mask, uint8_t* split_mask,
                       void* stream);

/* prune selection -- gaussian_splatting.py:630-635: opacity < min_opacity, and with use_size also max_radii2D >
 * max_screen_size or max(scaling) > world_threshold. opacity[P] and scaling[P,S] are ACTIVATED values. */
int fsgs_prune_mask(int P, int S, const float* opacity, const float* max_radii2D, const float* scaling,
                    float min_opacity, int use_size, float max_screen_size, float world_threshold, uint8_t* mask,
                    void* stream);

/* Children of a split -- gaussian_splatting.py:591-597, network.py:1170-1183. Child j < N * n_selected has parent
 * p = selected[j % n_selected]: out_xyz[j] = R(normalize(rotations[p])) * (noise[j] * scaling[p]) + xyz[p] (a surfel,
 * S = 2, has a zero third axis) and out_scaling[j] = log(scaling[p] / (0.8 N)). noise[N * n_selected, 3] are standard
 * normal samples drawn by the caller; scaling holds ACTIVATED scales, out_scaling raw (log) ones. */
int fsgs_split_children(int P, int n_selected, int N, int S, const int32_t* selected, const float* xyz,
                        const float* scaling, const float* rotations, const float* noise, float* out_xyz,
                        float* out_scaling, void* stream);

/* Per-step statistics -- network.py:1276-1282 with gaussian_splatting.py:486-495 / network.py:1152-1154. For points
 * with radii > 0: max_radii2D = max(max_radii2D, radii); grad_accum += |grad[:, :2]| (* factor if given); denom += 1.
 * grad has grad_stride floats per row; visible[P] (optional) receives radii > 0 as bytes. */
int fsgs_densification_stats(int P, int grad_stride, const int32_t* radii, const float* grad, const float* factor,
                             float* max_radii2D, float* grad_accum, float* denom, uint8_t* visible, void* stream);

/* The deformed parameters of a dynamic step -- fast_2d_gs/network.py:630, :643, :645 (torch operators there):
 * out_points = points + d_xyz, out_scales = (log_scales ? exp(scales) : scales) + d_scale with S = 2 or 3 scales per
 * point, out_rot = normalize(rot + d_rot) with a 1e-12 floor on the norm. The backward computes only what differs from
 * the upstream gradient: g_rot[N,4] (shared by rot and d_rot) and, when log_scales, g_scales[N,S] = g_out_scales *
 * exp(scales); points, d_xyz and d_scale take their output's gradient as it is. */
int fsgs_deform_apply_forward(int N, int S, int log_scales, const float* points, const float* d_xyz,
    const float* scales, const float* d_scale, const float* rot, const float* d_rot, float* out_points,
    float* out_scales, float* out_rot, void* stream);
int fsgs_deform_apply_backward(int N, int S, int log_scales, const float* scales, const float* rot, const float* d_rot,
    const float* g_out_scales, const float* g_out_rot, float* g_scales, float* g_rot, void* stream);

/* AdamMasksedUpdated -- fast_2d_gs/_C/src/other/adam_masked_update.cu:30-35 (kernel :9-28). Rows of the [N,M]
 * tensors whose mask byte is 0 are left untouched; eps is added to sqrt(v); lr carries the bias correction. */
int fsgs_adam_masked_update(int64_t N, int64_t M, const uint8_t* mask, double lr, double b1, double b2, double eps,
                            float* param, const float* grad, float* m, float* v, void* stream);
/* The same update for up to fsgs_adam_masked_update_max_tensors() tensors [N, M[q]] of one point set in one launch
 * (the loop over parameter groups of fast_2d_gs/sparse_gaussian_adam.py:20-45, one kernel each there). M, lr, eps,
 * param, grad, m, v are host arrays with one entry per tensor; results equal the single-tensor calls bit for bit. */
int fsgs_adam_masked_update_max_tensors(void);
int fsgs_adam_masked_update_multi(int n_tensors, int64_t N, const int64_t* M, const uint8_t* mask, const double* lr,
    double b1, double b2, const double* eps, float* const* param, const float* const* grad, float* const* m,
    float* const* v, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FSGS_H */
