// Block-cooperative movement of per-surfel SH rows between HBM and LDS for the one-lane-per-surfel preprocess kernels.
// A lane that walks its own 192-byte row touches one 128-byte line per instruction and relies on the caches to keep 96
// lines per wavefront alive between touches; moving the block's rows with consecutive lanes on consecutive addresses
// reads (writes) every line once. Used when the active degree is <= 3 (at most 16 coefficients, 48 floats per row).
#pragma once
#include <hip/hip_runtime.h>

namespace fsgs {

constexpr int kShStageRows   = 256;  // surfels per block
constexpr int kShStageFloats = 48;   // 16 coefficients x rgb
constexpr int kShStageStride = 49;   // odd stride: a lane reading its own row hits a different bank than its neighbours

// e / d for 0 <= e < 2^20 and 1 <= d <= 256 without an integer division: (e + 0.5) / d is at least 0.5 / d away from any
// integer, far more than the rounding error of the float product.
__device__ __forceinline__ int small_div(int e, float inv_d) { return (int) (((float) e + 0.5f) * inv_d); }

// Copies the first n coefficients (n * 3 floats) of every flagged row of the block into LDS. Row r of the block is
// surfel block_base + r. With sh_rest the DC coefficient comes from shs[P,1,3] and the others from sh_rest[P,n_sh,3].
__device__ __forceinline__ void stage_sh_rows(float* __restrict__ s_rows, const unsigned char* __restrict__ s_flag,
                                              int block_base, int P, int n, int n_sh, const float* __restrict__ shs,
                                              const float* __restrict__ sh_rest) {
  const int per_row = n * 3;
  const int rows    = min(kShStageRows, P - block_base);
  if (sh_rest == nullptr) {
    const size_t stride = (size_t) n_sh * 3;
    const float inv     = 1.0f / (float) per_row;
    for (int e = threadIdx.x; e < rows * per_row; e += blockDim.x) {
      const int r = small_div(e, inv), c = e - r * per_row;
      if (s_flag[r]) s_rows[r * kShStageStride + c] = shs[(size_t) (block_base + r) * stride + c];
    }
  } else {
    for (int e = threadIdx.x; e < rows * 3; e += blockDim.x) {
      const int r = e / 3, c = e - r * 3;
      if (s_flag[r]) s_rows[r * kShStageStride + c] = shs[(size_t) (block_base + r) * 3 + c];
    }
    const int rest    = per_row - 3;
    const size_t stride = (size_t) n_sh * 3;
    const float inv     = 1.0f / (float) max(rest, 1);
    for (int e = threadIdx.x; e < rows * rest; e += blockDim.x) {
      const int r = small_div(e, inv), c = e - r * rest;
      if (s_flag[r]) s_rows[r * kShStageStride + 3 + c] = sh_rest[(size_t) (block_base + r) * stride + c];
    }
  }
}

// Writes the block's staged gradient rows (n * 3 floats each, zeros where the owning lane stored zeros) to
// g_shs / g_sh_rest and zero-fills the coefficients above the active degree, so the caller's tensors need no
// initialisation. With the split layout (has_rest) either output may be absent.
__device__ __forceinline__ void unstage_sh_grads(const float* __restrict__ s_rows, int block_base, int P, int n,
                                                 int n_sh, bool has_rest, float* __restrict__ g_shs,
                                                 float* __restrict__ g_sh_rest) {
  const int rows = min(kShStageRows, P - block_base);
  if (!has_rest) {
    if (g_shs == nullptr) return;
    const int per_row = n_sh * 3, live = n * 3;
    const float inv   = 1.0f / (float) per_row;
    for (int e = threadIdx.x; e < rows * per_row; e += blockDim.x) {
      const int r = small_div(e, inv), c = e - r * per_row;
      g_shs[(size_t) (block_base + r) * per_row + c] = c < live ? s_rows[r * kShStageStride + c] : 0.0f;
    }
    return;
  }
  if (g_shs != nullptr) {
    for (int e = threadIdx.x; e < rows * 3; e += blockDim.x) {
      const int r = e / 3, c = e - r * 3;
      g_shs[(size_t) (block_base + r) * 3 + c] = s_rows[r * kShStageStride + c];
    }
  }
  if (g_sh_rest != nullptr) {
    const int per_row = n_sh * 3, live = n * 3 - 3;
    const float inv   = 1.0f / (float) max(per_row, 1);
    for (int e = threadIdx.x; e < rows * per_row; e += blockDim.x) {
      const int r = small_div(e, inv), c = e - r * per_row;
      g_sh_rest[(size_t) (block_base + r) * per_row + c] = c < live ? s_rows[r * kShStageStride + 3 + c] : 0.0f;
    }
  }
}

// ---- wavefront-private variant for complete degree-3 rows -----------------------------------------------------------
// With all 16 coefficients in one [P,16,3] tensor a row is twelve 16-byte pieces. A wavefront then moves its own 64 rows
// by itself: piece e = k * 64 + lane (k < 12) of the wavefront's 768 pieces belongs to row e / 12, so every load or store
// instruction covers 1 KB of consecutive addresses, the loads can be issued before the data is needed (they are held in
// registers while the lane does its geometry) and no block-wide barrier is involved.
constexpr int kShWavePieces = 12;

struct ShWaveRows {
  float4 v[kShWavePieces];
};

__device__ __forceinline__ void wave_piece(int k, int& r, int& c4) {
  const int e = k * 64 + (int) __lane_id();
  r  = (e * 5462) >> 16;  // e / 12 for 0 <= e < 768
  c4 = e - r * 12;
}

// `flags` has bit r set for the rows that are needed (all of them existing rows); the others re-read the first needed
// row's line instead of branching. flags must not be 0.
__device__ __forceinline__ void wave_fetch_sh_rows(ShWaveRows& regs, unsigned long long flags, int wave_base,
                                                   const float4* __restrict__ shs4) {
  const int first = __builtin_ctzll(flags);
#pragma unroll
  for (int k = 0; k < kShWavePieces; ++k) {
    int r, c4;
    wave_piece(k, r, c4);
    const bool on   = (flags >> r) & 1ull;
    const size_t at = (size_t) (wave_base + (on ? r : first)) * kShWavePieces + (on ? c4 : 0);
    regs.v[k]       = shs4[at];
  }
}

__device__ __forceinline__ void wave_rows_to_lds(const ShWaveRows& regs, float* __restrict__ s_wave_rows) {
#pragma unroll
  for (int k = 0; k < kShWavePieces; ++k) {
    int r, c4;
    wave_piece(k, r, c4);
    float* d = s_wave_rows + r * kShStageStride + 4 * c4;
    d[0] = regs.v[k].x, d[1] = regs.v[k].y, d[2] = regs.v[k].z, d[3] = regs.v[k].w;
  }
}

// Orders a wavefront's LDS writes before its later LDS reads of other lanes' data (no instruction is generated: a
// wavefront's LDS operations complete in order; this only stops the compiler from moving them across).
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Writes the wavefront's 64 staged rows (every existing row) to g4[P,12].
__device__ __forceinline__ void wave_rows_to_global(const float* __restrict__ s_wave_rows, int wave_base, int P,
                                                    float4* __restrict__ g4) {
#pragma unroll
  for (int k = 0; k < kShWavePieces; ++k) {
    int r, c4;
    wave_piece(k, r, c4);
    if (wave_base + r < P) {
      const float* s = s_wave_rows + r * kShStageStride + 4 * c4;
      g4[(size_t) (wave_base + r) * kShWavePieces + c4] = make_float4(s[0], s[1], s[2], s[3]);
    }
  }
}

}  // namespace fsgs
