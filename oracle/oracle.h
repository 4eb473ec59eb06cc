/* TEST INFRASTRUCTURE ONLY. Prototypes of liboracle.so (the CPU parity oracle); host pointers everywhere.
 * The *_f32 functions take float buffers, the *_f64 twins (same argument lists with double) exist for
 * finite-difference checks and are bound by oracle/__init__.py by substituting the scalar type. */
int oracle_gs_2d_preprocess_forward_f32(int P, int W, int H, int sh_degree, int n_sh, const float* means3D,
    const float* scales, const float* rotations, const float* opacities, const float* shs, const float* sh_rest,
    const float* Tw2v, const float* Tv2c, const float* campos, const float* trans_precomp, const uint8_t* culling,
    int means2D_preserve, float* means2D, float* colors, float* trans_mat, float* normal_opacity, float* depths,
    int32_t* radii, int32_t* tiles_touched);
int oracle_gs_2d_preprocess_backward_f32(int P, int W, int H, int sh_degree, int n_sh, const float* means3D,
    const float* scales, const float* rotations, const float* shs, const float* sh_rest, const float* Tw2v,
    const float* Tv2c, const float* campos, const float* trans_mat, const int32_t* radii, const float* colors,
    float* grad_mean2D, const float* grad_trans, const float* grad_colors, const float* grad_normal_opacity,
    float* g_means3D, float* g_scales, float* g_rot, float* g_opac, float* g_shs, float* g_sh_rest);
int oracle_gs_2d_compute_transmat_forward_f32(int P, int W, int H, const float* means3D, const float* scales,
    const float* rotations, const float* Tw2v, const float* Tw2c, float* trans_mat, float* normals);
int oracle_gs_2d_compute_transmat_backward_f32(int P, int W, int H, const float* means3D, const float* scales,
    const float* rotations, const float* Tw2v, const float* Tw2c, const float* g_mat, const float* g_normals,
    float* g_means3D, float* g_scales, float* g_rot);
int oracle_gs_2d_render_forward_f32(int P, int W, int H, double near_n, double far_n, int only_image,
    const float* means2D, const float* colors, const float* normal_opacity, const float* trans_mat,
    const int32_t* point_list, const int64_t* ranges, const float* trans_mat_t2, int32_t* accum_max_count,
    float* accum_weights_p, int32_t* accum_weights_count, float* out_color, float* out_opacity, float* out_extras,
    float* out_flow, int32_t* n_contrib);
int oracle_gs_2d_render_backward_f32(int P, int W, int H, double near_n, double far_n, const float* means2D,
    const float* normal_opacity, const float* colors, const float* trans_mat, const float* trans_mat_t2,
    const float* out_opacity, const float* out_extras, const float* out_flow, const float* dL_dpix,
    const float* dL_dopacity, const float* dL_dextras, const float* dL_dflow, const int64_t* ranges,
    const int32_t* point_list, const int32_t* n_contrib, float* g_colors, float* g_means2D, float* g_trans,
    float* g_normal_opacity);
int oracle_gs_2d_topk_weights_f32(int topk, int W, int H, double near_n, double far_n, const float* means2D,
    const float* normal_opacity, const float* trans_mat, const int64_t* ranges, const int32_t* point_list,
    int32_t* top_idx, float* top_w);
int oracle_sh_to_rgb_forward_f32(int P, int F, int degree, int clamp, const float* pos, const float* campos,
    const float* sh, float* rgb);
int oracle_sh_to_rgb_backward_f32(int P, int F, int degree, int clamp, const float* pos, const float* campos,
    const float* sh, const float* rgb, const float* grad_rgb, float* grad_dir, float* grad_campos, float* grad_sh);
int oracle_sh_encode_forward_f32(int B, int D, int C, const float* in, float* out);
int oracle_sh_encode_backward_f32(int B, int D, int C, const float* grad, const float* in, float* grad_in);
int oracle_freq_encode_forward_f32(int B, int Din, int degree, int include_input, double scale, const float* in,
    float* out);
/* The reference's forward for double tensors: angle, sine and cosine in single precision (freqencoder.cu:27-28). */
int oracle_freq_encode_forward_double_via_single(int B, int Din, int degree, int include_input, double scale,
    const double* in, double* out);
int oracle_freq_encode_backward_f32(int B, int Din, int degree, int include_input, double scale, const float* grad,
    const float* outv, float* gin);
int oracle_fusedssim_forward_f32(int B, int CH, int H, int W, double C1, double C2, const float* img1,
    const float* img2, float* ssim_map, float* dm_dmu1, float* dm_dsigma1_sq, float* dm_dsigma12);
int oracle_fusedssim_backward_f32(int B, int CH, int H, int W, const float* img1, const float* img2,
    const float* dL_dmap, const float* dm_dmu1, const float* dm_dsigma1_sq, const float* dm_dsigma12, float* dL_dimg1);
int oracle_cdist_top_forward_f32(int B, int N, int M, int D, int largest, const float* x, const float* y, float* dist,
    int64_t* index);
int oracle_cdist_top_backward_f32(int B, int N, int M, int D, const float* p1, const float* p2, const float* dist,
    const int64_t* index, const float* gdist, float* g1, float* g2);
int oracle_adam_masked_update_f32(int64_t N, int64_t M, const uint8_t* mask, double lr, double b1, double b2,
    double eps, float* param, const float* grad, float* m, float* v);
int oracle_knn_topk_f32(int N, int M, int D, int K, const float* x, const float* y, float* dist2, int64_t* index);
int oracle_knn_topk_backward_f32(int N, int M, int D, int K, const float* x, const float* y, const int64_t* index,
    const float* g_dist2, float* g_x, float* g_y);
int oracle_gs_2d_epilogue_forward_f32(int W, int H, double ratio, const float* Tw2v, const float* Tv2c,
    const float* extras, const float* opacity, const float* images, const float* background, float* normals,
    float* depths, float* surf_depth, float* surf_normal, float* composited);
int oracle_gs_2d_epilogue_backward_f32(int W, int H, double ratio, const float* Tw2v, const float* Tv2c,
    const float* extras, const float* opacity, const float* background, const float* g_normals, const float* g_depths,
    const float* g_surf_depth, const float* g_surf_normal, const float* g_distortion, const float* g_composited,
    float* g_extras, float* g_opacity);
int oracle_simple_knn_f32(int P, const float* points, float* mean_dist2);
int oracle_gs3d_preprocess_forward_f32(int P, int W, int H, int sh_degree, int n_sh, int is_opengl,
    const float* means3D, const float* scales, const float* rotations, const float* opacities, const float* shs,
    const float* sh_rest, const float* Tw2v, const float* Tv2c, const float* campos, double tanx, double tany,
    const uint8_t* culling, const float* cov3D_precomp, const float* cov2D_precomp, float* means2D, float* depths,
    float* colors, int32_t* radii, int32_t* tiles_touched, float* cov3Ds, float* conic_opacity);
int oracle_gs3d_preprocess_backward_f32(int P, int W, int H, int sh_degree, int n_sh, int is_opengl,
    const float* means3D, const float* scales, const float* rotations, const float* shs, const float* sh_rest,
    const float* Tw2v, const float* Tv2c, const float* campos, double tanx, double tany, const int32_t* radii,
    const float* colors, const float* cov3Ds, const float* cov2Ds, float* grad_mean2D, const float* grad_colors,
    const float* grad_conic, float* g_means3D, float* g_scales, float* g_rot, float* g_opac, float* g_shs,
    float* g_sh_rest, float* g_cov3D, float* g_Tw2v, float* g_campos);
int oracle_gs3d_render_forward_f32(int W, int H, int E, const float* means2D, const float* conic_opacity,
    const float* colors, const float* extras, const int32_t* point_list, const int64_t* ranges, float* out_color,
    float* out_opacity, float* out_extras, int32_t* n_contrib, int32_t* accum_max_count, float* accum_weights_p,
    int32_t* accum_weights_count, const int64_t* bucket_offset, int32_t* max_contrib, int32_t* bucket_to_tile,
    float* sampled_T, float* sampled_ar);
int oracle_gs3d_render_fast_backward_f32(int W, int H, int E, const float* means2D, const float* conic_opacity,
    const float* colors, const float* extras, const float* images, const float* out_extras, const float* out_opacity,
    const int32_t* n_contrib, const int32_t* max_contrib, const int64_t* bucket_offset, const int32_t* bucket_to_tile,
    const float* sampled_T, const float* sampled_ar, const float* dL_dpix, const float* dL_dout_extras,
    const float* dL_dout_opacity, const int32_t* point_list, const int64_t* ranges, int64_t B, float* g_means2D,
    float* g_conic_opacity, float* g_colors, float* g_extras);
int oracle_gs3d_render_backward_f32(int W, int H, int E, const float* means2D, const float* conic_opacity,
    const float* colors, const float* extras, const float* out_opacity, const int32_t* n_contrib,
    const float* dL_dpix, const float* dL_dout_extras, const float* dL_dout_opacity, const int32_t* point_list,
    const int64_t* ranges, float* g_means2D, float* g_conic_opacity, float* g_colors, float* g_extras);
int oracle_gs3d_extra_forward_f32(int W, int H, int E, const float* extras, const float* means2D,
    const float* conic_opacity, const int64_t* ranges, const int32_t* point_list, const int32_t* n_contrib, float* out);
int oracle_gs3d_extra_backward_f32(int W, int H, int E, const float* extras, const float* out_opacity,
    const float* grad_out, const float* means2D, const float* conic_opacity, const int64_t* ranges,
    const int32_t* point_list, const int32_t* n_contrib, float* g_extras, float* g_means2D, float* g_conic_opacity);
int oracle_gs3d_topk_weights_f32(int topk, int W, int H, const float* means2D, const float* conic_opacity,
    const int64_t* ranges, const int32_t* point_list, int32_t* top_idx, float* top_w);
int oracle_gs3d_compute_cov3D_f32(int N, const float* q, const float* s, float* cov3D);
int oracle_gs3d_compute_cov3D_backward_f32(int N, const float* q, const float* s, const float* g, float* gq, float* gs);
int oracle_gs3d_compute_cov2D_f32(int N, const float* cov3D, const float* mean, const float* Tw2v, double fx, double fy,
    double tanx, double tany, float* cov2D);
int oracle_gs3d_compute_cov2D_backward_f32(int N, const float* cov3D, const float* mean, const float* Tw2v, double fx,
    double fy, double tanx, double tany, const float* g, float* g_cov3D, float* g_mean, float* g_vm);
int64_t oracle_gs_prepare_count(int P, const int32_t* tiles_touched, int64_t* offsets);
int oracle_gs_prepare_fill(int P, int W, int H, const float* means2D, const float* depths, const int32_t* radii,
    const int64_t* offsets, int64_t R, int64_t* ranges, int32_t* point_list, int64_t* keys_sorted_out);
uint32_t oracle_higher_msb(uint32_t n);
int oracle_num_threads(void);
int oracle_gs_2d_fast_compute_transmat_forward_f32(int P, const float* means3D, const float* scales,
    const float* rotations, const float* Tw2v, const float* Tv2s, float* trans_mat, float* normals);
int oracle_gs_2d_fast_compute_transmat_backward_f32(int P, const float* means3D, const float* scales,
    const float* rotations, const float* Tw2v, const float* Tv2s, const float* g_mat, const float* g_normals,
    float* g_means3D, float* g_scales, float* g_rot);
int oracle_gs_2d_fast_preprocess_forward_f32(int P, int W, int H, int sh_degree, int n_sh, const float* means3D,
    const float* scales, const float* rotations, const float* opacities, const float* shs, const float* sh_rest,
    const float* Tw2v, const float* Tv2s, const float* campos, const float* trans_precomp, const uint8_t* culling,
    int means2D_preserve, float* means2D, float* colors, float* trans_mat, float* inverse_m, float* normal_opacity,
    float* depths, int32_t* radii, int32_t* tiles_touched);
int oracle_gs_2d_fast_preprocess_backward_f32(int P, int W, int H, int sh_degree, int n_sh, const float* means3D,
    const float* scales, const float* rotations, const float* shs, const float* sh_rest, const float* Tw2v,
    const float* Tv2s, const float* campos, const float* trans_mat, const int32_t* radii, const float* colors,
    float* grad_mean2D, const float* grad_trans, const float* grad_inv_m, const float* grad_colors,
    const float* grad_normal_opacity, float* g_means3D, float* g_scales, float* g_rot, float* g_opac, float* g_shs,
    float* g_sh_rest);
int oracle_gs_2d_fast_render_forward_f32(int W, int H, double near_n, double far_n, int only_image,
    const float* means2D, const float* colors, const float* normal_opacity, const float* trans_mat,
    const float* inverse_m, const int32_t* point_list, const int64_t* ranges, const int64_t* bucket_offset,
    const float* trans_mat_t2, int32_t* accum_max_count, float* accum_weights_p, int32_t* accum_weights_count,
    float* out_color, float* out_opacity, float* out_extras, float* out_flow, int32_t* n_contrib,
    int32_t* max_contrib, int32_t* bucket_to_tile, float* sampled_T, float* sampled_acc, float* sampled_aux);
int oracle_gs_2d_fast_render_backward_f32(int P, int W, int H, double near_n, double far_n, int per_splat_form,
    const float* means2D, const float* normal_opacity, const float* colors, const float* trans_mat,
    const float* inverse_m, const float* trans_mat_t2, const float* out_opacity, const float* out_extras,
    const float* out_flow, const float* dL_dpix, const float* dL_dopacity, const float* dL_dextras,
    const float* dL_dflow, const int64_t* ranges, const int32_t* point_list, const int32_t* n_contrib,
    float* g_colors, float* g_means2D, float* g_trans, float* g_inv, float* g_normal_opacity);
int oracle_gs_fast_prepare_fill(int P, int W, int H, const float* means2D, const float* inverse_m,
    const float* depths, const float* opacities, const int32_t* radii, const int64_t* offsets, int64_t R,
    int64_t* ranges, int32_t* point_list, int64_t* keys_sorted_out);
int oracle_fast_corner_test_f64(const double* inverse_m, double opacity, int x, int y);
