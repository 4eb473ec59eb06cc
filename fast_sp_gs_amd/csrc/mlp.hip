// Fused deformation MLP forward and backward on the CDNA4 matrix cores (bf16 operands, fp32 accumulation) for gfx950.
//
// Reference behaviour reproduced (in fp32 there): fast_2d_gs/network.py:1757-1776 -- h = in; for each of the L layers
// h = relu(W_i h + b_i); after layer index `skip` the input is concatenated in front, h = [in | h]; the heads are plain
// linear maps of the last hidden state (gaussian_warp 3, gaussian_rotation 4, gaussian_scaling 3 stacked into one
// [n_out, 256] matrix by the caller).
//
// One block owns 32 rows (control points) and keeps their activations in LDS for the whole network, so the only HBM/L2
// traffic is the weights (about 1 MB in bf16, shared by all blocks through L2) and 40 bytes of output per row.
// Each of the 8 wavefronts computes a 32 x 32 slab of a layer's output with v_mfma_f32_32x32x16_bf16: A fragments
// (activations) come from LDS as one 16-byte read per lane, B fragments (weights, packed in fragment order, see
// frag_index) as one 16-byte global read per lane; both use the same (lane / 32, element) -> k mapping, so the product
// is independent of how the hardware orders k inside a fragment.
//
// Training: the forward optionally stores every layer's post-ReLU hidden state (bf16, [layer][B][256]). The backward
// (the reference leaves it to torch autograd: one addmm-backward pair and a ReLU mask per layer, ~30 launches) is two
// kernels:
//   * a chain kernel with the forward's structure, one block per 32 rows: dZ_L-1 = (g_out . W_heads) masked by the saved
//     state, then for each layer dH_l-1 = dZ_l . W_l[:, hidden part] on the matrix cores against a transposed bf16 copy
//     of the weights, masked, kept in LDS for the next layer and written to HBM as dZ[l][B][256];
//   * a weight-gradient kernel over all layers at once: every block owns a 32 x 128 tile of one layer's dW = dZ^T X,
//     walks the batch in 32-row chunks transposed through LDS, and the first tile column of a layer also sums dZ over
//     the batch for the bias gradient. No atomics: every output element has one writer.
// Gradients with respect to the (frequency-encoded) input are not produced; the reference detaches it
// (network.py:586).
#include <algorithm>

#include "common.hpp"

namespace fsgs {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kMlpWidth   = 256;
constexpr int kMlpRows    = 32;                       // rows per block
constexpr int kMlpMaxIn   = 96;                       // padded input width limit
constexpr int kMlpStride  = kMlpWidth + kMlpMaxIn + 8;  // LDS row stride in bf16 (+8 keeps 16-byte rows off one bank)
constexpr int kMlpThreads = 256;
// Forward and backward chain: eight wavefronts per block, one 32 x 32 output tile each. The batch is small (16 blocks at
// B = 512) and the nine layers depend on each other, so a layer's time is the latency of its weight fragments: with one
// tile per wavefront a whole layer's 16 fragments fit in registers and are requested together.
constexpr int kChainThreads = 512;

__device__ __forceinline__ uint16_t f32_to_bf16(float f) {  // round to nearest even
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7f800000u) == 0x7f800000u) return (uint16_t) ((u >> 16) | ((u & 0xffffu) ? 0x40u : 0u));
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t) (u >> 16);
}

// Weights are stored in the order the matrix cores consume them: the [rows_pad][K_pad] matrix is cut into tiles of 32
// rows x 16 columns, tile (row tile nt, k-step ks) at ((nt * K_pad / 16) + ks) * 512 elements, and inside a tile the 8
// consecutive k values that lane l of a wavefront feeds to one MFMA (row l % 32, columns 8 * (l / 32) .. + 7) are
// contiguous at l * 8. One fragment load of a wavefront is then a single 1 KB run instead of 64 rows 2 * K_pad bytes apart.
__device__ __forceinline__ size_t frag_index(int r, int k, int K_pad) {
  const int nt = r >> 5, n = r & 31, ks = k >> 4, kk = k & 15;
  return (((size_t) nt * (K_pad >> 4) + ks) * 64 + n + 32 * (kk >> 3)) * 8 + (kk & 7);
}

__global__ void __launch_bounds__(256) pack_bf16_kernel(int rows, int K, int rows_pad, int K_pad,
                                                        const float* __restrict__ src, uint16_t* __restrict__ dst) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows_pad * K_pad) return;
  const int r = i / K_pad, k = i - r * K_pad;
  dst[frag_index(r, k, K_pad)] = (r < rows && k < K) ? f32_to_bf16(src[(size_t) r * K + k]) : (uint16_t) 0;
}

// Every per-step re-pack of the network in one launch: blockIdx.y selects a job of the table passed by value.
struct PackJob {
  const float* src;
  void* dst;
  int rows, K;            // extent of the source that exists: rows x K values
  int rows_cover, K_pad;  // fragment rows this job writes (zeros past `rows`), padded row length of the fragment matrix
  int dst_row0;           // first fragment row
  int src_ld, col0;       // leading dimension and first column of the source
  int kind;               // 0 fragment pack | 1 fragment pack of the transpose | 2 plain float copy of `rows` values
};
constexpr int kMaxPackJobs = 40;
struct PackTable {
  PackJob job[kMaxPackJobs];
};

__global__ void __launch_bounds__(256) pack_jobs_kernel(PackTable table) {
  const PackJob& j = table.job[blockIdx.y];
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (j.kind == 2) {
    if (i < j.rows) ((float*) j.dst)[i] = j.src[i];
    return;
  }
  if (i >= j.rows_cover * j.K_pad) return;
  const int r = i / j.K_pad, k = i - r * j.K_pad;
  float v = 0.0f;
  if (r < j.rows && k < j.K)
    v = j.kind == 0 ? j.src[(size_t) r * j.src_ld + j.col0 + k] : j.src[(size_t) k * j.src_ld + j.col0 + r];
  ((uint16_t*) j.dst)[frag_index(j.dst_row0 + r, k, j.K_pad)] = f32_to_bf16(v);
}

// D layout of the 32x32 accumulator: register r of lane l holds row 8 * (r / 4) + 4 * (l / 32) + (r % 4), column l % 32.
__device__ __forceinline__ int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

template <bool kSave>
__global__ void __launch_bounds__(kChainThreads) mlp_forward_kernel(int B, int Din, int n_layers, int skip, int n_out,
    const float* __restrict__ in, const uint16_t* __restrict__ packed, const float* __restrict__ bias,
    float* __restrict__ out, uint16_t* __restrict__ saved) {
  __shared__ __attribute__((aligned(16))) uint16_t s_act[2][kMlpRows][kMlpStride];
  __shared__ __attribute__((aligned(16))) uint16_t s_in[kMlpRows][kMlpMaxIn + 8];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row0 = blockIdx.x * kMlpRows;
  const int Din_pad = (Din + 15) & ~15;

  // stage the (bf16) input rows, zero padded
  for (int e = threadIdx.x; e < kMlpRows * Din_pad; e += kChainThreads) {
    const int r = e / Din_pad, k = e - r * Din_pad;
    const float v = (row0 + r < B && k < Din) ? in[(size_t) (row0 + r) * Din + k] : 0.0f;
    const uint16_t h = f32_to_bf16(v);
    s_in[r][k] = h;
    s_act[0][r][k] = h;
  }
  __syncthreads();

  int cur = 0;
  int K = Din, K_pad = Din_pad;
  const uint16_t* W = packed;
  const float* bl   = bias;
  // Fragment u (k-step u, clamped to the layer's last step) of row tile `wave` of a layer whose weights start at Wl;
  // consecutive k-steps are 512 elements apart.
  auto fragment = [&](const uint16_t* Wl, int K_pad_l, int u) {
    const int steps = K_pad_l >> 4;
    return *(const bf16x8*) (Wl + ((size_t) wave * steps + min(u, steps - 1)) * 512 + lane * 8);
  };
  // The weights do not depend on the activations: the first sixteen fragments of the NEXT layer are requested at the
  // start of each layer and arrive while this layer's products, epilogue and barrier run.
  bf16x8 ahead[16];
#pragma unroll
  for (int u = 0; u < 16; ++u) ahead[u] = fragment(W, K_pad, u);
  for (int layer = 0; layer < n_layers; ++layer) {
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    const int arow = lane & 31, kofs = 8 * (lane >> 5);
    const uint16_t* wrow = W + (size_t) wave * (K_pad >> 4) * 512 + lane * 8;
    bf16x8 b[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) b[u] = ahead[u];
    if (layer + 1 < n_layers) {
      const int K_after = (((layer == skip) ? Din + kMlpWidth : kMlpWidth) + 15) & ~15;
#pragma unroll
      for (int u = 0; u < 16; ++u) ahead[u] = fragment(W + (size_t) kMlpWidth * K_pad, K_after, u);
    }
    const int first = min(K_pad >> 4, 16);
#pragma unroll
    for (int u = 0; u < 16; ++u)
      if (u < first) {
        const bf16x8 a = *(const bf16x8*) &s_act[cur][arow][16 * u + kofs];
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b[u], acc, 0, 0, 0);
      }
    int k0 = 16 * first;
    for (; k0 + 64 <= K_pad; k0 += 64) {
      bf16x8 b[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) b[u] = *(const bf16x8*) (wrow + (k0 + 16 * u) * 32);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const bf16x8 a = *(const bf16x8*) &s_act[cur][arow][k0 + 16 * u + kofs];
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b[u], acc, 0, 0, 0);
      }
    }
    for (; k0 < K_pad; k0 += 16) {
      const bf16x8 a = *(const bf16x8*) &s_act[cur][arow][k0 + kofs];
      const bf16x8 b = *(const bf16x8*) (wrow + k0 * 32);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
    }
    // bias + ReLU -> bf16 into the other buffer; after the skip layer the input goes in front of the hidden state
    const int nxt = cur ^ 1;
    const int col_shift = (layer == skip) ? Din : 0;
    {
      const int col  = wave * 32 + (lane & 31);
      const float bv = bl[col];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float v    = fmaxf(acc[r] + bv, 0.0f);
        const uint16_t h = f32_to_bf16(v);
        const int row    = acc_row(r, lane);
        s_act[nxt][row][col_shift + col] = h;
        if (kSave && row0 + row < B) saved[((size_t) layer * B + row0 + row) * kMlpWidth + col] = h;
      }
    }
    int K_next = kMlpWidth;
    if (layer == skip) {
      K_next = Din + kMlpWidth;
      for (int e = threadIdx.x; e < kMlpRows * Din; e += kChainThreads) {
        const int r = e / Din, k = e - r * Din;
        s_act[nxt][r][k] = s_in[r][k];
      }
    }
    const int K_next_pad = (K_next + 15) & ~15;
    for (int e = threadIdx.x; e < kMlpRows * (K_next_pad - K_next); e += kChainThreads) {
      const int r = e / (K_next_pad - K_next), k = e - r * (K_next_pad - K_next);
      s_act[nxt][r][K_next + k] = 0;
    }
    lds_barrier();
    W += (size_t) kMlpWidth * K_pad;
    bl += kMlpWidth;
    K = K_next, K_pad = K_next_pad;
    cur = nxt;
  }
  (void) K;

  // heads: one padded 32-column tile, wavefront 0 only
  if (wave == 0) {
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    const int arow = lane & 31, kofs = 8 * (lane >> 5);
    const uint16_t* wrow = W + lane * 8;
    for (int k0 = 0; k0 < K_pad; k0 += 16) {
      const bf16x8 a = *(const bf16x8*) &s_act[cur][arow][k0 + kofs];
      const bf16x8 b = *(const bf16x8*) (wrow + k0 * 32);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
    }
    const int col = lane & 31;
    if (col < n_out) {
      const float bv = bl[col];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = row0 + acc_row(r, lane);
        if (row < B) out[(size_t) row * n_out + col] = acc[r] + bv;
      }
    }
  }
}


__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float((uint32_t) h << 16); }

// dZ[l] for every layer, back to front. packed_t holds, for l = 1 .. n_layers-1, the hidden part of W_l transposed:
// [256 inputs][256 outputs] bf16.
__global__ void __launch_bounds__(kChainThreads) mlp_backward_chain_kernel(int B, int n_layers, int n_out,
    const float* __restrict__ heads_w /*[n_out][256] fp32*/, const uint16_t* __restrict__ packed_t,
    const uint16_t* __restrict__ saved, const float* __restrict__ g_out, uint16_t* __restrict__ dz) {
  __shared__ __attribute__((aligned(16))) uint16_t s_dz[kMlpRows][kMlpWidth + 8];
  __shared__ float s_g[kMlpRows][32];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row0 = blockIdx.x * kMlpRows;
  {
    // dZ of the last layer: (g_out . W_heads) where the stored state is non-zero. Lane t owns column t of all 32 rows.
    for (int e = threadIdx.x; e < kMlpRows * 32; e += kChainThreads) {
      const int r = e >> 5, k = e & 31;
      s_g[r][k] = (row0 + r < B && k < n_out) ? g_out[(size_t) (row0 + r) * n_out + k] : 0.0f;
    }
    __syncthreads();
    if (threadIdx.x < kMlpWidth) {
    const int c = threadIdx.x;
    const size_t top = (size_t) (n_layers - 1) * B;
    uint16_t keep[kMlpRows];  // read at clamped rows, unconditionally, so the loads overlap the products below
#pragma unroll
    for (int r = 0; r < kMlpRows; ++r) keep[r] = saved[(top + min(row0 + r, B - 1)) * kMlpWidth + c];
    float v[kMlpRows];
#pragma unroll
    for (int r = 0; r < kMlpRows; ++r) v[r] = 0.0f;
    for (int k = 0; k < n_out; ++k) {
      const float wv = heads_w[k * kMlpWidth + c];
#pragma unroll
      for (int r = 0; r < kMlpRows; ++r) v[r] += s_g[r][k] * wv;
    }
#pragma unroll
    for (int r = 0; r < kMlpRows; ++r) {
      const bool live  = row0 + r < B;
      const uint16_t h = (live && keep[r] != 0) ? f32_to_bf16(v[r]) : (uint16_t) 0;
      if (live) dz[(top + row0 + r) * kMlpWidth + c] = h;
      s_dz[r][c] = h;
    }
    }
  }
  // all sixteen weight fragments of a wavefront's tile are requested together, one layer ahead (they do not depend on
  // dZ), and the stored states that mask a layer's result are fetched while the matrix cores run
  auto fragment = [&](int layer, int u) {
    return *(const bf16x8*) (packed_t + ((size_t) ((layer - 1) * 8 + wave) * (kMlpWidth / 16) + u) * 512 + lane * 8);
  };
  bf16x8 ahead[16];
  if (n_layers >= 2)
#pragma unroll
    for (int u = 0; u < 16; ++u) ahead[u] = fragment(n_layers - 1, u);
  __syncthreads();
  for (int layer = n_layers - 1; layer >= 1; --layer) {
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    const int arow = lane & 31, kofs = 8 * (lane >> 5);
    bf16x8 b[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) b[u] = ahead[u];
    if (layer >= 2)
#pragma unroll
      for (int u = 0; u < 16; ++u) ahead[u] = fragment(layer - 1, u);
    const size_t base = (size_t) (layer - 1) * B;
    uint16_t keep[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      // rows past the batch reuse the last row's mask: their results stay in LDS and are never stored
      const int row = min(row0 + acc_row(r, lane), B - 1);
      keep[r] = saved[(base + row) * kMlpWidth + wave * 32 + (lane & 31)];
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const bf16x8 a = *(const bf16x8*) &s_dz[arow][16 * u + kofs];
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b[u], acc, 0, 0, 0);
    }
    lds_barrier();  // every wavefront has read dZ[layer] before it is overwritten
    {
      const int col = wave * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row    = acc_row(r, lane);
        const uint16_t h = keep[r] != 0 ? f32_to_bf16(acc[r]) : (uint16_t) 0;
        if (row0 + row < B) dz[(base + row0 + row) * kMlpWidth + col] = h;
        s_dz[row][col] = h;
      }
    }
    lds_barrier();
  }
}

// dW_l = dZ_l^T X_l and db_l = column sums of dZ_l for l = 0 .. n_layers (l == n_layers: the heads, whose "dZ" is g_out).
// X_0 = in, X_{skip+1} = [in | H_skip], X_l = H_{l-1} otherwise. g_w is the layers' [256][K_l] gradients back to back
// followed by the heads' [n_out][256]; g_b has the layout of the forward's bias vector.
__global__ void __launch_bounds__(kMlpThreads) mlp_backward_weights_kernel(int B, int Din, int n_layers, int skip,
    int n_out, const float* __restrict__ in, const uint16_t* __restrict__ saved, const uint16_t* __restrict__ dz,
    const float* __restrict__ g_out, float* __restrict__ g_w, float* __restrict__ g_b) {
  __shared__ __attribute__((aligned(16))) uint16_t s_a[32][kMlpRows + 8];   // [output o][batch row]
  __shared__ __attribute__((aligned(16))) uint16_t s_b[128][kMlpRows + 8];  // [input i][batch row]
  // which (layer, output tile, input group) this block owns
  int layer = 0, K = Din, tile = blockIdx.x;
  size_t w_off = 0;
  for (;; ++layer) {
    const int rows = layer < n_layers ? kMlpWidth : n_out;
    const int tiles = ((rows + 31) / 32) * ((K + 127) / 128);
    if (tile < tiles || layer == n_layers) break;
    tile -= tiles;
    w_off += (size_t) rows * K;
    K = (layer == skip) ? Din + kMlpWidth : kMlpWidth;
  }
  const int rows   = layer < n_layers ? kMlpWidth : n_out;
  const int groups = (K + 127) / 128;
  const int o0 = (tile / groups) * 32, i0 = (tile % groups) * 128;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // X_l's hidden part comes from this saved state, shifted by `shift` columns (the re-concatenated input)
  const int shift = (layer == skip + 1) ? Din : 0;
  const uint16_t* hidden = layer > 0 ? saved + (size_t) (layer - 1) * B * kMlpWidth : nullptr;
  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
  float bias_sum = 0.0f;
  for (int b0 = 0; b0 < B; b0 += kMlpRows) {
    // Loads are unconditional on clamped addresses and out-of-range elements are zeroed afterwards. The empty asm after
    // each group takes all of its values at once: without it the compiler sinks every load into a branch of its own
    // with a full wait behind it; with it a chunk's 20 loads are in flight together.
    uint16_t va[4], vb[16];
    unsigned ra[4], rb[16];
    float fb[16];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int e = threadIdx.x + q * kMlpThreads, b = e >> 5, o = e & 31;
      const int bc = min(b0 + b, B - 1), oc = min(o0 + o, rows - 1);
      ra[q] = layer < n_layers ? dz[((size_t) layer * B + bc) * kMlpWidth + oc]
                               : f32_to_bf16(g_out[(size_t) bc * n_out + oc]);
    }
    const bool from_in = layer == 0 || (shift > 0 && i0 < shift);
    const bool from_hidden = layer > 0;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int e = threadIdx.x + q * kMlpThreads, b = e >> 7, gi = i0 + (e & 127);
      const int bc = min(b0 + b, B - 1);
      fb[q] = from_in ? in[(size_t) bc * Din + min(gi, Din - 1)] : 0.0f;
      rb[q] = from_hidden ? hidden[(size_t) bc * kMlpWidth + min(max(gi - shift, 0), kMlpWidth - 1)] : 0u;
    }
    asm volatile("" : "+v"(ra[0]), "+v"(ra[1]), "+v"(ra[2]), "+v"(ra[3]));
    asm volatile("" : "+v"(rb[0]), "+v"(rb[1]), "+v"(rb[2]), "+v"(rb[3]), "+v"(rb[4]), "+v"(rb[5]), "+v"(rb[6]),
                      "+v"(rb[7]), "+v"(rb[8]), "+v"(rb[9]), "+v"(rb[10]), "+v"(rb[11]), "+v"(rb[12]), "+v"(rb[13]),
                      "+v"(rb[14]), "+v"(rb[15]));
    asm volatile("" : "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]), "+v"(fb[4]), "+v"(fb[5]), "+v"(fb[6]),
                      "+v"(fb[7]), "+v"(fb[8]), "+v"(fb[9]), "+v"(fb[10]), "+v"(fb[11]), "+v"(fb[12]), "+v"(fb[13]),
                      "+v"(fb[14]), "+v"(fb[15]));
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int e = threadIdx.x + q * kMlpThreads, b = e >> 5, o = e & 31;
      va[q] = (b0 + b < B && o0 + o < rows) ? (uint16_t) ra[q] : (uint16_t) 0;
    }
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int e = threadIdx.x + q * kMlpThreads, b = e >> 7, gi = i0 + (e & 127);
      const uint16_t h = (layer == 0 || gi < shift) ? f32_to_bf16(fb[q]) : (uint16_t) rb[q];
      vb[q] = (b0 + b < B && gi < K) ? h : (uint16_t) 0;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int e = threadIdx.x + q * kMlpThreads;
      s_a[e & 31][e >> 5] = va[q];
    }
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int e = threadIdx.x + q * kMlpThreads;
      s_b[e & 127][e >> 7] = vb[q];
    }
    __syncthreads();
    const int kofs = 8 * (lane >> 5);
#pragma unroll
    for (int k0 = 0; k0 < kMlpRows; k0 += 16) {
      const bf16x8 a = *(const bf16x8*) &s_a[lane & 31][k0 + kofs];
      const bf16x8 b = *(const bf16x8*) &s_b[wave * 32 + (lane & 31)][k0 + kofs];
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
    }
    if (i0 == 0 && threadIdx.x < 32) {
#pragma unroll
      for (int b = 0; b < kMlpRows; ++b) bias_sum += bf16_to_f32(s_a[threadIdx.x][b]);
    }
    __syncthreads();
  }
  const int i = i0 + wave * 32 + (lane & 31);
  if (i < K) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int o = o0 + acc_row(r, lane);
      if (o < rows) g_w[w_off + (size_t) o * K + i] = acc[r];
    }
  }
  if (i0 == 0 && threadIdx.x < 32 && o0 + threadIdx.x < rows)
    g_b[(size_t) layer * kMlpWidth + o0 + threadIdx.x] = bias_sum;
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API int fsgs_pack_bf16(int rows, int K, int rows_pad, int K_pad, const float* src, uint16_t* dst, void* stream) {
  FSGS_REQUIRE(rows > 0 && K > 0 && rows_pad >= rows && K_pad >= K && src && dst, "pack_bf16: bad arguments");
  FSGS_REQUIRE(rows_pad % 32 == 0 && K_pad % 16 == 0, "pack_bf16: rows_pad must be a multiple of 32 and K_pad of 16");
  hipLaunchKernelGGL(pack_bf16_kernel, dim3(div_up((int64_t) rows_pad * K_pad, 256)), dim3(256), 0,
                     (hipStream_t) stream, rows, K, rows_pad, K_pad, src, dst);
  return check_launch("pack_bf16");
}

// All buffers the fused network reads, refreshed from the fp32 parameters in one launch: `packed` (what
// fsgs_mlp_forward reads: the layers' fragment matrices, then the heads stacked into one [32][256] matrix), `packed_t`
// (optional; what fsgs_mlp_backward reads: [n_layers - 1][256 in][256 out] fragments of the last 256 input columns of
// layers 1..), `bias_out` (layer biases then head biases) and `heads_w_out` (the heads' fp32 rows stacked).
FSGS_API int fsgs_mlp_pack_all(int Din, int n_layers, int skip, const float* const* weights,
    const float* const* biases, int n_heads, const float* const* head_weights, const float* const* head_biases,
    const int* head_rows, uint16_t* packed, uint16_t* packed_t, float* bias_out, float* heads_w_out, void* stream) {
  FSGS_REQUIRE(Din > 0 && n_layers >= 1 && skip < n_layers - 1 && weights && biases && packed && bias_out,
               "mlp_pack_all: bad arguments");
  FSGS_REQUIRE(n_heads >= 0 && (n_heads == 0 || (head_weights && head_biases && head_rows && heads_w_out)),
               "mlp_pack_all: bad head arguments");
  FSGS_REQUIRE(2 * n_layers + 3 * n_heads + (packed_t ? n_layers - 1 : 0) <= kMaxPackJobs,
               "mlp_pack_all: too many layers / heads for one launch (%d jobs at most)", kMaxPackJobs);
  PackTable table{};
  int n = 0, most = 0;
  auto add = [&](const PackJob& j) {
    most = std::max(most, j.kind == 2 ? j.rows : j.rows_cover * j.K_pad);
    table.job[n++] = j;
  };
  size_t off = 0;
  int K = Din;
  for (int l = 0; l < n_layers; ++l) {
    FSGS_REQUIRE(weights[l] && biases[l], "mlp_pack_all: null layer tensor");
    const int K_pad = (K + 15) & ~15;
    add({weights[l], packed + off, kMlpWidth, K, kMlpWidth, K_pad, 0, K, 0, 0});
    add({biases[l], bias_out + (size_t) l * kMlpWidth, kMlpWidth, 0, 0, 0, 0, 0, 0, 2});
    if (packed_t && l > 0)
      add({weights[l], packed_t + (size_t) (l - 1) * kMlpWidth * kMlpWidth, kMlpWidth, kMlpWidth, kMlpWidth,
           kMlpWidth, 0, K, K - kMlpWidth, 1});
    off += (size_t) kMlpWidth * K_pad;
    K = (l == skip) ? Din + kMlpWidth : kMlpWidth;
  }
  FSGS_REQUIRE(K == kMlpWidth, "mlp_pack_all: the heads must follow a %d-wide layer", kMlpWidth);
  int row0 = 0;
  for (int h = 0; h < n_heads; ++h) {
    FSGS_REQUIRE(head_weights[h] && head_biases[h] && head_rows[h] > 0, "mlp_pack_all: bad head tensor");
    const bool last = h == n_heads - 1;
    FSGS_REQUIRE(row0 + head_rows[h] <= 32, "mlp_pack_all: the heads have more than 32 rows together");
    add({head_weights[h], packed + off, head_rows[h], kMlpWidth, last ? 32 - row0 : head_rows[h], kMlpWidth, row0,
         kMlpWidth, 0, 0});
    add({head_biases[h], bias_out + (size_t) n_layers * kMlpWidth + row0, head_rows[h], 0, 0, 0, 0, 0, 0, 2});
    add({head_weights[h], heads_w_out + (size_t) row0 * kMlpWidth, head_rows[h] * kMlpWidth, 0, 0, 0, 0, 0, 0, 2});
    row0 += head_rows[h];
  }
  if (n_heads == 0) add({weights[0], packed + off, 0, kMlpWidth, 32, kMlpWidth, 0, kMlpWidth, 0, 0});  // zero head block
  hipLaunchKernelGGL(pack_jobs_kernel, dim3(div_up(most, 256), n), dim3(256), 0, (hipStream_t) stream, table);
  return check_launch("mlp_pack_all");
}

// Number of bf16 elements of the packed weight buffer: per layer [256][K_pad_i], then the heads as [32][K_pad_last].
FSGS_API size_t fsgs_mlp_packed_elems(int Din, int n_layers, int skip) {
  size_t n = 0;
  int K = Din;
  for (int l = 0; l < n_layers; ++l) {
    n += (size_t) kMlpWidth * ((K + 15) & ~15);
    K = (l == skip) ? Din + kMlpWidth : kMlpWidth;
  }
  n += (size_t) 32 * ((K + 15) & ~15);
  return n;
}

FSGS_API int fsgs_mlp_forward(int B, int Din, int width, int n_layers, int skip, int n_out, const float* in,
                              const uint16_t* packed, const float* bias, float* out, uint16_t* saved, void* stream) {
  FSGS_REQUIRE(B >= 0 && in && packed && bias && out, "mlp_forward: bad arguments");
  FSGS_REQUIRE(width == kMlpWidth, "mlp_forward: width %d is not supported (only %d)", width, kMlpWidth);
  FSGS_REQUIRE(Din > 0 && ((Din + 15) & ~15) <= kMlpMaxIn, "mlp_forward: input width %d exceeds %d", Din, kMlpMaxIn);
  FSGS_REQUIRE(n_layers >= 1 && skip < n_layers - 1 && n_out >= 1 && n_out <= 32,
               "mlp_forward: bad layer structure (layers %d, skip %d, outputs %d)", n_layers, skip, n_out);
  if (B == 0) return kOk;
  auto kernel = saved ? mlp_forward_kernel<true> : mlp_forward_kernel<false>;
  hipLaunchKernelGGL(kernel, dim3(div_up(B, kMlpRows)), dim3(kChainThreads), 0, (hipStream_t) stream, B, Din, n_layers,
                     skip, n_out, in, packed, bias, out, saved);
  return check_launch("mlp_forward");
}

FSGS_API size_t fsgs_mlp_backward_workspace_bytes(int B, int n_layers) {
  if (B < 0 || n_layers < 1) return 0;
  return align_up((size_t) n_layers * (B > 0 ? B : 1) * kMlpWidth * sizeof(uint16_t), 256);
}

FSGS_API int fsgs_mlp_backward(int B, int Din, int width, int n_layers, int skip, int n_out, const float* in,
    const uint16_t* packed_t, const float* heads_w, const uint16_t* saved, const float* g_out, float* g_w, float* g_b,
    void* workspace, size_t workspace_bytes, void* stream) {
  FSGS_REQUIRE(B >= 0 && in && packed_t && heads_w && saved && g_out && g_w && g_b && workspace,
               "mlp_backward: bad arguments");
  FSGS_REQUIRE(width == kMlpWidth, "mlp_backward: width %d is not supported (only %d)", width, kMlpWidth);
  FSGS_REQUIRE(Din > 0 && ((Din + 15) & ~15) <= kMlpMaxIn, "mlp_backward: input width %d exceeds %d", Din, kMlpMaxIn);
  FSGS_REQUIRE(n_layers >= 1 && n_layers <= 64 && skip < n_layers - 1 && n_out >= 1 && n_out <= 32,
               "mlp_backward: bad layer structure (layers %d, skip %d, outputs %d)", n_layers, skip, n_out);
  if (workspace_bytes < fsgs_mlp_backward_workspace_bytes(B, n_layers))
    return fail(kWorkspaceSmall, "mlp_backward: workspace %zu < %zu bytes", workspace_bytes,
                fsgs_mlp_backward_workspace_bytes(B, n_layers));
  hipStream_t s = (hipStream_t) stream;
  uint16_t* dz  = (uint16_t*) workspace;
  // with an empty batch the weight kernel's chunk loop does not run and it writes zeros
  if (B > 0)
    hipLaunchKernelGGL(mlp_backward_chain_kernel, dim3(div_up(B, kMlpRows)), dim3(kChainThreads), 0, s, B, n_layers,
                       n_out, heads_w, packed_t, saved, g_out, dz);
  int tiles = 0, K = Din;
  for (int l = 0; l <= n_layers; ++l) {
    const int rows = l < n_layers ? kMlpWidth : n_out;
    tiles += ((rows + 31) / 32) * ((K + 127) / 128);
    K = (l == skip) ? Din + kMlpWidth : kMlpWidth;
  }
  hipLaunchKernelGGL(mlp_backward_weights_kernel, dim3(tiles), dim3(kMlpThreads), 0, s, B, Din, n_layers, skip, n_out,
                     in, saved, dz, g_out, g_w, g_b);
  return check_launch("mlp_backward");
}
