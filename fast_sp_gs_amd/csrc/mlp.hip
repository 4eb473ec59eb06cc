// Fused deformation MLP forward on the CDNA4 matrix cores (bf16 inputs, fp32 accumulation) for gfx950.
//
// Reference behaviour reproduced (in fp32 there): fast_2d_gs/network.py:1757-1776 -- h = in; for each of the L layers
// h = relu(W_i h + b_i); after layer index `skip` the input is concatenated in front, h = [in | h]; the heads are plain
// linear maps of the last hidden state (gaussian_warp 3, gaussian_rotation 4, gaussian_scaling 3 stacked into one
// [n_out, 256] matrix by the caller).
//
// One block owns 32 rows (control points) and keeps their activations in LDS for the whole network, so the only HBM/L2
// traffic is the weights (about 1 MB in bf16, shared by all blocks through L2) and 40 bytes of output per row.
// Each of the 4 wavefronts computes a 32 x 64 slab of a layer's output with v_mfma_f32_32x32x16_bf16: A fragments
// (activations) come from LDS as one 16-byte read per lane, B fragments (weights, row-major [out][in]) as one 16-byte
// global read per lane; both use the same (lane / 32, element) -> k mapping, so the product is independent of how the
// hardware orders k inside a fragment.
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

__device__ __forceinline__ uint16_t f32_to_bf16(float f) {  // round to nearest even
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7f800000u) == 0x7f800000u) return (uint16_t) ((u >> 16) | ((u & 0xffffu) ? 0x40u : 0u));
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t) (u >> 16);
}

__global__ void __launch_bounds__(256) pack_bf16_kernel(int rows, int K, int rows_pad, int K_pad,
                                                        const float* __restrict__ src, uint16_t* __restrict__ dst) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows_pad * K_pad) return;
  const int r = i / K_pad, k = i - r * K_pad;
  dst[i] = (r < rows && k < K) ? f32_to_bf16(src[(size_t) r * K + k]) : (uint16_t) 0;
}

// D layout of the 32x32 accumulator: register r of lane l holds row 8 * (r / 4) + 4 * (l / 32) + (r % 4), column l % 32.
__device__ __forceinline__ int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

__global__ void __launch_bounds__(kMlpThreads) mlp_forward_kernel(int B, int Din, int n_layers, int skip, int n_out,
    const float* __restrict__ in, const uint16_t* __restrict__ packed, const float* __restrict__ bias,
    float* __restrict__ out) {
  __shared__ __attribute__((aligned(16))) uint16_t s_act[2][kMlpRows][kMlpStride];
  __shared__ __attribute__((aligned(16))) uint16_t s_in[kMlpRows][kMlpMaxIn + 8];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row0 = blockIdx.x * kMlpRows;
  const int Din_pad = (Din + 15) & ~15;

  // stage the (bf16) input rows, zero padded
  for (int e = threadIdx.x; e < kMlpRows * Din_pad; e += kMlpThreads) {
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
  for (int layer = 0; layer < n_layers; ++layer) {
    floatx16 acc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][r] = 0.0f;
    const int arow = lane & 31, kofs = 8 * (lane >> 5);
    const uint16_t* wrow0 = W + (size_t) (wave * 64 + (lane & 31)) * K_pad + kofs;
    const uint16_t* wrow1 = wrow0 + (size_t) 32 * K_pad;
    for (int k0 = 0; k0 < K_pad; k0 += 16) {
      const bf16x8 a  = *(const bf16x8*) &s_act[cur][arow][k0 + kofs];
      const bf16x8 b0 = *(const bf16x8*) (wrow0 + k0);
      const bf16x8 b1 = *(const bf16x8*) (wrow1 + k0);
      acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b0, acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b1, acc[1], 0, 0, 0);
    }
    // bias + ReLU -> bf16 into the other buffer; after the skip layer the input goes in front of the hidden state
    const int nxt = cur ^ 1;
    const int col_shift = (layer == skip) ? Din : 0;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int col = wave * 64 + t * 32 + (lane & 31);
      const float bv = bl[col];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float v = fmaxf(acc[t][r] + bv, 0.0f);
        s_act[nxt][acc_row(r, lane)][col_shift + col] = f32_to_bf16(v);
      }
    }
    int K_next = kMlpWidth;
    if (layer == skip) {
      K_next = Din + kMlpWidth;
      for (int e = threadIdx.x; e < kMlpRows * Din; e += kMlpThreads) {
        const int r = e / Din, k = e - r * Din;
        s_act[nxt][r][k] = s_in[r][k];
      }
    }
    const int K_next_pad = (K_next + 15) & ~15;
    for (int e = threadIdx.x; e < kMlpRows * (K_next_pad - K_next); e += kMlpThreads) {
      const int r = e / (K_next_pad - K_next), k = e - r * (K_next_pad - K_next);
      s_act[nxt][r][K_next + k] = 0;
    }
    __syncthreads();
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
    const uint16_t* wrow = W + (size_t) (lane & 31) * K_pad + kofs;
    for (int k0 = 0; k0 < K_pad; k0 += 16) {
      const bf16x8 a = *(const bf16x8*) &s_act[cur][arow][k0 + kofs];
      const bf16x8 b = *(const bf16x8*) (wrow + k0);
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

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API int fsgs_pack_bf16(int rows, int K, int rows_pad, int K_pad, const float* src, uint16_t* dst, void* stream) {
  FSGS_REQUIRE(rows > 0 && K > 0 && rows_pad >= rows && K_pad >= K && src && dst, "pack_bf16: bad arguments");
  hipLaunchKernelGGL(pack_bf16_kernel, dim3(div_up((int64_t) rows_pad * K_pad, 256)), dim3(256), 0,
                     (hipStream_t) stream, rows, K, rows_pad, K_pad, src, dst);
  return check_launch("pack_bf16");
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
                              const uint16_t* packed, const float* bias, float* out, void* stream) {
  FSGS_REQUIRE(B >= 0 && in && packed && bias && out, "mlp_forward: bad arguments");
  FSGS_REQUIRE(width == kMlpWidth, "mlp_forward: width %d is not supported (only %d)", width, kMlpWidth);
  FSGS_REQUIRE(Din > 0 && ((Din + 15) & ~15) <= kMlpMaxIn, "mlp_forward: input width %d exceeds %d", Din, kMlpMaxIn);
  FSGS_REQUIRE(n_layers >= 1 && skip < n_layers - 1 && n_out >= 1 && n_out <= 32,
               "mlp_forward: bad layer structure (layers %d, skip %d, outputs %d)", n_layers, skip, n_out);
  if (B == 0) return kOk;
  hipLaunchKernelGGL(mlp_forward_kernel, dim3(div_up(B, kMlpRows)), dim3(kMlpThreads), 0, (hipStream_t) stream, B, Din,
                     n_layers, skip, n_out, in, packed, bias, out);
  return check_launch("mlp_forward");
}
