// Fused SSIM map and its backward for gfx950.
//
// Reference behaviour reproduced: fast_2d_gs/_C/src/other/structural_similarity.cu:187-277 (forward kernel), :279-338
// (backward kernel), :340-380 (host entries): separable 11-tap Gaussian (sigma 1.5, the literal weights of :11-21), zero
// padding, per channel; the forward also returns dm/dmu1, dm/dsigma1^2, dm/dsigma12 for the backward.
//
// Where the reference convolves one quantity at a time through a shared scratchpad (five passes and ~25 barriers per
// channel), each block here loads the 42x42 halo of both images once, forms all five moments (I1, I1^2, I2, I2^2, I1 I2)
// in one horizontal pass into LDS and finishes them in one vertical pass: two barriers per channel. A block is 256 lanes
// (4 wavefronts) for a 32x32 output tile, every lane owning one column of 4 output rows.
#include "common.hpp"

#include <atomic>

namespace fsgs {
namespace {

constexpr int kSsimTile = 32;
constexpr int kSsimHalo = kSsimTile + 10;  // 42
constexpr int kSsimThreads = 256;

__constant__ float kGauss[11] = {0.001028380123898387f, 0.0075987582094967365f, 0.036000773310661316f,
                                 0.10936068743467331f,  0.21300552785396576f,   0.26601171493530273f,
                                 0.21300552785396576f,  0.10936068743467331f,   0.036000773310661316f,
                                 0.0075987582094967365f, 0.001028380123898387f};

__device__ __forceinline__ float pixel_or_zero(const float* __restrict__ plane, int y, int x, int H, int W) {
  return (x >= 0 && y >= 0 && x < W && y < H) ? plane[(size_t) y * W + x] : 0.0f;
}

template <bool kTrain, bool kLoss>
__global__ void __launch_bounds__(kSsimThreads) ssim_forward_kernel(int H, int W, int CH, float C1, float C2,
    const float* __restrict__ img1, const float* __restrict__ img2, float* __restrict__ ssim_map,
    float* __restrict__ dm_dmu1, float* __restrict__ dm_dsigma1_sq, float* __restrict__ dm_dsigma12,
    float* __restrict__ partials) {
  __shared__ float s_a[kSsimHalo][kSsimHalo + 1];
  __shared__ float s_b[kSsimHalo][kSsimHalo + 1];
  __shared__ float s_h[5][kSsimHalo][kSsimTile + 1];  // horizontally filtered moments
  const int x0 = blockIdx.x * kSsimTile, y0 = blockIdx.y * kSsimTile;
  const size_t plane = (size_t) H * W;
  float g[11];
#pragma unroll
  for (int k = 0; k < 11; ++k) g[k] = kGauss[k];
  float sum_ssim = 0.0f, sum_l1 = 0.0f;  // kLoss: this lane's share of the two image sums

  for (int c = 0; c < CH; ++c) {
    const float* p1 = img1 + ((size_t) blockIdx.z * CH + c) * plane;
    const float* p2 = img2 + ((size_t) blockIdx.z * CH + c) * plane;
    for (int e = threadIdx.x; e < kSsimHalo * kSsimHalo; e += kSsimThreads) {
      const int ly = e / kSsimHalo, lx = e - ly * kSsimHalo;
      s_a[ly][lx] = pixel_or_zero(p1, y0 + ly - 5, x0 + lx - 5, H, W);
      s_b[ly][lx] = pixel_or_zero(p2, y0 + ly - 5, x0 + lx - 5, H, W);
    }
    __syncthreads();
    for (int e = threadIdx.x; e < kSsimHalo * kSsimTile; e += kSsimThreads) {
      const int ly = e / kSsimTile, lx = e - ly * kSsimTile;
      float m1 = 0, m11 = 0, m2 = 0, m22 = 0, m12 = 0;
#pragma unroll
      for (int k = 0; k < 11; ++k) {
        const float a = s_a[ly][lx + k], b = s_b[ly][lx + k];
        m1 += g[k] * a, m11 += g[k] * (a * a), m2 += g[k] * b, m22 += g[k] * (b * b), m12 += g[k] * (a * b);
      }
      s_h[0][ly][lx] = m1, s_h[1][ly][lx] = m11, s_h[2][ly][lx] = m2, s_h[3][ly][lx] = m22, s_h[4][ly][lx] = m12;
    }
    __syncthreads();
    const int lx = threadIdx.x & 31;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int ly = (threadIdx.x >> 5) * 4 + r;
      float mu1 = 0, e11 = 0, mu2 = 0, e22 = 0, e12 = 0;
#pragma unroll
      for (int k = 0; k < 11; ++k) {
        mu1 += g[k] * s_h[0][ly + k][lx], e11 += g[k] * s_h[1][ly + k][lx], mu2 += g[k] * s_h[2][ly + k][lx];
        e22 += g[k] * s_h[3][ly + k][lx], e12 += g[k] * s_h[4][ly + k][lx];
      }
      const int px = x0 + lx, py = y0 + ly;
      if (px < W && py < H) {
        const float sigma1_sq = e11 - mu1 * mu1, sigma2_sq = e22 - mu2 * mu2, sigma12 = e12 - mu1 * mu2;
        const float mu1_sq = mu1 * mu1, mu2_sq = mu2 * mu2, mu1_mu2 = mu1 * mu2;
        const float C = 2.0f * mu1_mu2 + C1, D = 2.0f * sigma12 + C2;
        const float A = mu1_sq + mu2_sq + C1, B = sigma1_sq + sigma2_sq + C2;
        const size_t idx = ((size_t) blockIdx.z * CH + c) * plane + (size_t) py * W + px;
        if (kLoss) {
          sum_ssim += (C * D) / (A * B);
          sum_l1 += fabsf(s_a[ly + 5][lx + 5] - s_b[ly + 5][lx + 5]);
        } else {
          ssim_map[idx] = (C * D) / (A * B);
        }
        if (kTrain) {
          dm_dmu1[idx] = (mu2 * 2.0f * D) / (A * B) - (mu2 * 2.0f * C) / (A * B) - (mu1 * 2.0f * C * D) / (A * A * B) +
                         (mu1 * 2.0f * C * D) / (A * B * B);
          dm_dsigma1_sq[idx] = (-C * D) / (A * B * B);
          dm_dsigma12[idx]   = (2.0f * C) / (A * B);
        }
      }
    }
    __syncthreads();  // the next channel overwrites the halo and the filtered moments
  }
  if (kLoss) {
    // block sums in a fixed order: lanes by xor butterfly, then the four wavefronts in turn
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) sum_ssim += __shfl_xor(sum_ssim, d, 64), sum_l1 += __shfl_xor(sum_l1, d, 64);
    float* s_red = &s_h[0][0][0];
    if ((threadIdx.x & 63) == 0) s_red[2 * (threadIdx.x >> 6)] = sum_ssim, s_red[2 * (threadIdx.x >> 6) + 1] = sum_l1;
    __syncthreads();
    if (threadIdx.x == 0) {
      const size_t blk = ((size_t) blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
      float a = 0.0f, b = 0.0f;
      for (int w = 0; w < kSsimThreads / 64; ++w) a += s_red[2 * w], b += s_red[2 * w + 1];
      partials[2 * blk] = a, partials[2 * blk + 1] = b;
    }
  }
}

// loss_out[0] = (1 - lambda) * mean|img - target| + lambda * (1 - mean SSIM); [1] = the L1 mean, [2] = the SSIM mean.
// One block; the per-block partial sums are added in a fixed order.
__global__ void __launch_bounds__(256) image_loss_finish_kernel(int n_blocks, const float* __restrict__ partials,
                                                                float inv_n, float lambda, float* __restrict__ loss_out) {
  __shared__ float s_red[2][256];
  float a = 0.0f, b = 0.0f;
  for (int i = threadIdx.x; i < n_blocks; i += 256) a += partials[2 * i], b += partials[2 * i + 1];
  s_red[0][threadIdx.x] = a, s_red[1][threadIdx.x] = b;
  __syncthreads();
  for (int d = 128; d >= 1; d >>= 1) {
    if ((int) threadIdx.x < d)
      s_red[0][threadIdx.x] += s_red[0][threadIdx.x + d], s_red[1][threadIdx.x] += s_red[1][threadIdx.x + d];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const float ssim_mean = s_red[0][0] * inv_n, l1_mean = s_red[1][0] * inv_n;
    loss_out[0] = (1.0f - lambda) * l1_mean + lambda * (1.0f - ssim_mean);
    loss_out[1] = l1_mean, loss_out[2] = ssim_mean;
  }
}

// kLoss: the gradient of the fused image loss. dL/dmap is the same number at every pixel, -lambda / n times the
// upstream gradient of the scalar loss (read from device memory), and (1 - lambda) / n * sign(img1 - img2) is added.
template <bool kLoss>
__global__ void __launch_bounds__(kSsimThreads) ssim_backward_kernel(int H, int W, int CH,
    const float* __restrict__ img1, const float* __restrict__ img2, const float* __restrict__ dL_dmap,
    const float* __restrict__ dm_dmu1, const float* __restrict__ dm_dsigma1_sq, const float* __restrict__ dm_dsigma12,
    float* __restrict__ dL_dimg1, float map_scale, float l1_scale) {
  __shared__ float s_p[3][kSsimHalo][kSsimHalo + 1];  // dL/dmap times each of the three partials
  __shared__ float s_h[3][kSsimHalo][kSsimTile + 1];
  const int x0 = blockIdx.x * kSsimTile, y0 = blockIdx.y * kSsimTile;
  const size_t plane = (size_t) H * W;
  float g[11];
#pragma unroll
  for (int k = 0; k < 11; ++k) g[k] = kGauss[k];

  for (int c = 0; c < CH; ++c) {
    const size_t off = ((size_t) blockIdx.z * CH + c) * plane;
    for (int e = threadIdx.x; e < kSsimHalo * kSsimHalo; e += kSsimThreads) {
      const int ly = e / kSsimHalo, lx = e - ly * kSsimHalo;
      const int y = y0 + ly - 5, x = x0 + lx - 5;
      const float gmap = kLoss ? ((y >= 0 && y < H && x >= 0 && x < W) ? map_scale * dL_dmap[0] : 0.0f)
                               : pixel_or_zero(dL_dmap + off, y, x, H, W);
      s_p[0][ly][lx] = pixel_or_zero(dm_dmu1 + off, y, x, H, W) * gmap;
      s_p[1][ly][lx] = pixel_or_zero(dm_dsigma1_sq + off, y, x, H, W) * gmap;
      s_p[2][ly][lx] = pixel_or_zero(dm_dsigma12 + off, y, x, H, W) * gmap;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < kSsimHalo * kSsimTile; e += kSsimThreads) {
      const int ly = e / kSsimTile, lx = e - ly * kSsimTile;
      float a0 = 0, a1 = 0, a2 = 0;
#pragma unroll
      for (int k = 0; k < 11; ++k)
        a0 += g[k] * s_p[0][ly][lx + k], a1 += g[k] * s_p[1][ly][lx + k], a2 += g[k] * s_p[2][ly][lx + k];
      s_h[0][ly][lx] = a0, s_h[1][ly][lx] = a1, s_h[2][ly][lx] = a2;
    }
    __syncthreads();
    const int lx = threadIdx.x & 31;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int ly = (threadIdx.x >> 5) * 4 + r;
      float a0 = 0, a1 = 0, a2 = 0;
#pragma unroll
      for (int k = 0; k < 11; ++k)
        a0 += g[k] * s_h[0][ly + k][lx], a1 += g[k] * s_h[1][ly + k][lx], a2 += g[k] * s_h[2][ly + k][lx];
      const int px = x0 + lx, py = y0 + ly;
      if (px < W && py < H) {
        const size_t idx = off + (size_t) py * W + px;
        float grad = a0;
        grad += img1[idx] * 2.0f * a1;
        grad += img2[idx] * a2;
        if (kLoss) {
          const float d = img1[idx] - img2[idx];
          grad += l1_scale * dL_dmap[0] * (d > 0.0f ? 1.0f : (d < 0.0f ? -1.0f : 0.0f));
        }
        dL_dimg1[idx] = grad;
      }
    }
    __syncthreads();
  }
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API int fsgs_fusedssim_forward(int B, int CH, int H, int W, double C1, double C2, const float* img1,
    const float* img2, float* ssim_map, float* dm_dmu1, float* dm_dsigma1_sq, float* dm_dsigma12, void* stream) {
  FSGS_REQUIRE(B >= 0 && CH >= 0 && H >= 0 && W >= 0, "fusedssim: bad sizes");
  if ((size_t) B * CH * H * W == 0) return kOk;
  FSGS_REQUIRE(img1 && img2 && ssim_map, "fusedssim: null pointer");
  const bool train = dm_dmu1 != nullptr;
  FSGS_REQUIRE(!train || (dm_dsigma1_sq && dm_dsigma12), "fusedssim: the three partial-derivative maps go together");
  FSGS_REQUIRE(B <= 65535, "fusedssim: batch %d exceeds the grid limit", B);
  const dim3 grid(div_up(W, kSsimTile), div_up(H, kSsimTile), B), block(kSsimThreads);
  if (train)
    hipLaunchKernelGGL((ssim_forward_kernel<true, false>), grid, block, 0, (hipStream_t) stream, H, W, CH, (float) C1,
                       (float) C2, img1, img2, ssim_map, dm_dmu1, dm_dsigma1_sq, dm_dsigma12, nullptr);
  else
    hipLaunchKernelGGL((ssim_forward_kernel<false, false>), grid, block, 0, (hipStream_t) stream, H, W, CH, (float) C1,
                       (float) C2, img1, img2, ssim_map, dm_dmu1, dm_dsigma1_sq, dm_dsigma12, nullptr);
  return check_launch("fusedssim");
}

FSGS_API int fsgs_fusedssim_backward(int B, int CH, int H, int W, const float* img1, const float* img2,
    const float* dL_dmap, const float* dm_dmu1, const float* dm_dsigma1_sq, const float* dm_dsigma12,
    float* dL_dimg1, void* stream) {
  FSGS_REQUIRE(B >= 0 && CH >= 0 && H >= 0 && W >= 0, "fusedssim_backward: bad sizes");
  if ((size_t) B * CH * H * W == 0) return kOk;
  FSGS_REQUIRE(img1 && img2 && dL_dmap && dm_dmu1 && dm_dsigma1_sq && dm_dsigma12 && dL_dimg1,
               "fusedssim_backward: null pointer");
  FSGS_REQUIRE(B <= 65535, "fusedssim_backward: batch %d exceeds the grid limit", B);
  const dim3 grid(div_up(W, kSsimTile), div_up(H, kSsimTile), B), block(kSsimThreads);
  hipLaunchKernelGGL(ssim_backward_kernel<false>, grid, block, 0, (hipStream_t) stream, H, W, CH, img1, img2, dL_dmap,
                     dm_dmu1, dm_dsigma1_sq, dm_dsigma12, dL_dimg1, 0.0f, 0.0f);
  return check_launch("fusedssim_backward");
}

FSGS_API size_t fsgs_image_loss_workspace_bytes(int B, int H, int W) {
  if (B <= 0 || H <= 0 || W <= 0) return 256;
  return align_up((size_t) B * div_up(W, kSsimTile) * div_up(H, kSsimTile) * 2 * sizeof(float), 256);
}

FSGS_API int fsgs_image_loss_forward(int B, int CH, int H, int W, double C1, double C2, double lambda_dssim,
    const float* img, const float* target, float* loss_out, float* dm_dmu1, float* dm_dsigma1_sq,
    float* dm_dsigma12, void* workspace, size_t workspace_bytes, void* stream) {
  FSGS_REQUIRE(B > 0 && CH > 0 && H > 0 && W > 0 && B <= 65535, "image_loss: bad sizes");
  FSGS_REQUIRE(img && target && loss_out && workspace, "image_loss: null pointer");
  const bool train = dm_dmu1 != nullptr;
  FSGS_REQUIRE(!train || (dm_dsigma1_sq && dm_dsigma12), "image_loss: the three partial-derivative maps go together");
  if (workspace_bytes < fsgs_image_loss_workspace_bytes(B, H, W))
    return fail(kWorkspaceSmall, "image_loss: workspace %zu < %zu bytes", workspace_bytes,
                fsgs_image_loss_workspace_bytes(B, H, W));
  const dim3 grid(div_up(W, kSsimTile), div_up(H, kSsimTile), B), block(kSsimThreads);
  hipStream_t s = (hipStream_t) stream;
  float* partials = (float*) workspace;
  if (train)
    hipLaunchKernelGGL((ssim_forward_kernel<true, true>), grid, block, 0, s, H, W, CH, (float) C1, (float) C2, img,
                       target, nullptr, dm_dmu1, dm_dsigma1_sq, dm_dsigma12, partials);
  else
    hipLaunchKernelGGL((ssim_forward_kernel<false, true>), grid, block, 0, s, H, W, CH, (float) C1, (float) C2, img,
                       target, nullptr, dm_dmu1, dm_dsigma1_sq, dm_dsigma12, partials);
  const double n = (double) B * CH * H * W;
  hipLaunchKernelGGL(image_loss_finish_kernel, dim3(1), dim3(256), 0, s, (int) (grid.x * grid.y * grid.z), partials,
                     (float) (1.0 / n), (float) lambda_dssim, loss_out);
  return check_launch("image_loss");
}

// ---- the same forward for callers that cannot allocate ----------------------------------------------------------------
// The per-block partial sums live in a file-scope device array instead of a caller workspace. Every GPU the library
// runs on holds its own copy of the array at its own address until the process ends; the address is looked up once per
// device and only that pointer is handed to kernels (the array's name is a host-side stand-in, not a device address).
constexpr int kStaticLossMaxBlocks = 65536;  // 32x32-pixel blocks, e.g. one 8192x8192 image or 40 images of 1280x1280
static __device__ __align__(256) float scratch[2 * kStaticLossMaxBlocks];  // 512 KiB
constexpr int kMaxDevices = 64;
static std::atomic<float*> g_scratch_ptr[kMaxDevices];

static int static_scratch(float** out) {
  int dev = -1;
  FSGS_HIP(hipGetDevice(&dev));
  FSGS_REQUIRE(dev >= 0 && dev < kMaxDevices, "image_loss_static: device ordinal %d out of range", dev);
  float* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    FSGS_HIP(hipGetSymbolAddress((void**) &p, HIP_SYMBOL(scratch)));
    FSGS_REQUIRE(p != nullptr, "image_loss_static: no device address for the scratch array");
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return kOk;
}

FSGS_API int fsgs_image_loss_static_max_blocks(void) { return kStaticLossMaxBlocks; }

FSGS_API int fsgs_image_loss_forward_static(int B, int CH, int H, int W, double C1, double C2, double lambda_dssim,
    const float* img, const float* target, float* loss_out, float* dm_dmu1, float* dm_dsigma1_sq,
    float* dm_dsigma12, void* stream) {
  FSGS_REQUIRE(B > 0 && CH > 0 && H > 0 && W > 0 && B <= 65535, "image_loss_static: bad sizes");
  const int64_t blocks = (int64_t) B * div_up(W, kSsimTile) * div_up(H, kSsimTile);
  if (blocks > kStaticLossMaxBlocks)
    return fail(kUnsupported, "image_loss_static: %lld blocks of 32x32 pixels exceed the built-in scratch of %d blocks; "
                "use fsgs_image_loss_forward with a workspace", (long long) blocks, kStaticLossMaxBlocks);
  float* partials = nullptr;
  if (int rc = static_scratch(&partials)) return rc;
  return fsgs_image_loss_forward(B, CH, H, W, C1, C2, lambda_dssim, img, target, loss_out, dm_dmu1, dm_dsigma1_sq,
                                 dm_dsigma12, partials, (size_t) 2 * kStaticLossMaxBlocks * sizeof(float), stream);
}

FSGS_API int fsgs_image_loss_backward(int B, int CH, int H, int W, double lambda_dssim, const float* img,
    const float* target, const float* grad_loss, const float* dm_dmu1, const float* dm_dsigma1_sq,
    const float* dm_dsigma12, float* dL_dimg, void* stream) {
  FSGS_REQUIRE(B > 0 && CH > 0 && H > 0 && W > 0 && B <= 65535, "image_loss_backward: bad sizes");
  FSGS_REQUIRE(img && target && grad_loss && dm_dmu1 && dm_dsigma1_sq && dm_dsigma12 && dL_dimg,
               "image_loss_backward: null pointer");
  const dim3 grid(div_up(W, kSsimTile), div_up(H, kSsimTile), B), block(kSsimThreads);
  const double n = (double) B * CH * H * W;
  hipLaunchKernelGGL(ssim_backward_kernel<true>, grid, block, 0, (hipStream_t) stream, H, W, CH, img, target,
                     grad_loss, dm_dmu1, dm_dsigma1_sq, dm_dsigma12, dL_dimg, (float) (-lambda_dssim / n),
                     (float) ((1.0 - lambda_dssim) / n));
  return check_launch("image_loss_backward");
}
