// FP8 MFMA GEMM device code for gfx950 (CDNA4).
//
// Operands: "W" = weight rows [N,K] and "X" = activation rows [M,K], both e4m3fn with K contiguous.
// The MFMA computes the transposed product: W rows are the matrix-core "A" operand, X rows the "B"
// operand, so one lane of a 32x32 result tile holds 16 values of ONE activation row (m = lane%32)
// and four runs of 4 consecutive n.  A block-scaled K step therefore needs a single scale
// as[m,kb]*bs[nb,kb] per lane, and the bf16 output is written as 8-byte runs along n.
#pragma once

#include "fp8k_common.h"

namespace fp8k {

struct GemmArgs {
  const uint8_t* X;   // [M,K]
  const uint8_t* W;   // [N,K]
  const float* sx;    // block mode: as[m*sx_m + kb*sx_k]; row mode: sa[m]
  const float* sw;    // block mode: bs[nb*sw_n + kb*sw_k]; row mode: sb[n]
  const void* bias;   // row mode only, may be null
  void* C;            // [M,N]
  float* partial;     // split-K workspace [splits][M][N] float, or null
  int M, N, K;
  int64_t ldx, ldw, ldc;
  int64_t sx_m, sx_k, sw_n, sw_k;
  int tiles_m, tiles_n;
  int splits;         // K is cut into `splits` runs of kb_per_split K-blocks
  int kb_per_split;
};

enum { kModeBlock = 0, kModeRow = 1 };

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

// 16 bytes per lane straight from global memory into LDS at lds_base + lane*16 (lds_base wave-uniform)
__device__ __forceinline__ void load16_to_lds(const uint8_t* g, uint8_t* lds_base) {
  __builtin_amdgcn_global_load_lds((gbl_ptr_t)g, (lds_ptr_t)lds_base, 16, 0, 0);
}
__device__ __forceinline__ void wait_vm0() { __builtin_amdgcn_s_waitcnt(0x0F70); }  // vmcnt(0)

__device__ __forceinline__ v16f mfma_32x32x64(v8i a, v8i b, v16f c) {
  // cbsz = blgp = 0: both operands e4m3; scale operands 0 select the unscaled instruction form
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

template <int OUT_DT>
__device__ __forceinline__ void store4(void* C, int64_t idx, float a, float b, float c, float d) {
  uint2 o;
  if (OUT_DT == FP8K_BF16) {
    o.x = pack_bf16x2(a, b);
    o.y = pack_bf16x2(c, d);
  } else {
    o.x = f32_to_f16_bits(a) | (f32_to_f16_bits(b) << 16);
    o.y = f32_to_f16_bits(c) | (f32_to_f16_bits(d) << 16);
  }
  *reinterpret_cast<uint2*>((u16*)C + idx) = o;
}

template <int DT>
__device__ __forceinline__ float load_scalar(const void* p, int64_t i) {
  if (DT == FP8K_F32) return ((const float*)p)[i];
  if (DT == FP8K_BF16) return __uint_as_float((uint32_t)((const u16*)p)[i] << 16);
  return f16_bits_to_f32(((const u16*)p)[i]);
}

// ------------------------------------------------------------------------------------------------
// 256(n) x 256(m) x 128(k) workgroup tile, 8 wavefronts (2 along n x 4 along m), wave tile
// 128(n) x 64(m) = 4 x 2 MFMA tiles of 32x32, K step 128 = two v_mfma_f32_32x32x64_f8f6f4.
//
// LDS: two stages of [W 256 rows x 128 B | X 256 rows x 128 B] = 2 x 64 KB, filled by
// global_load_lds_dwordx4 (no register staging).  A 1 KB wave-load covers 8 rows; the 16-byte
// chunk c of row r is stored at chunk position c ^ ((r >> 1) & 7), which makes both the linear
// LDS-DMA writes and the ds_read_b128 operand fetches (32 rows, same logical chunk) bank-conflict
// free.  One barrier per K step: loads for step kb+1 are issued right after the barrier that
// publishes step kb, and run under its 16 MFMAs per wave.
//
// Block mode keeps a second, short-lived accumulator: t = W.X over one K block, then
// acc += t * (as[m,kb] * bs[nb,kb]); row mode accumulates in place and scales in the epilogue.
// ------------------------------------------------------------------------------------------------
constexpr int kTileN = 256, kTileM = 256, kTileK = 128;
constexpr int kStageBytes = (kTileN + kTileM) * kTileK;  // 64 KB
constexpr int kXOff = kTileN * kTileK;                   // X tile offset inside a stage

template <int MODE, int OUT_DT, int BIAS_DT, bool SPLIT>
__global__ __launch_bounds__(512, 1) void gemm_tile256_kernel(const GemmArgs p) {
  __shared__ __attribute__((aligned(1024))) uint8_t smem[2 * kStageBytes];

  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int wn = w & 1, wm = w >> 1;

  // ---- tile coordinates: contiguous chunk of tiles per XCD, groups of 4 m-tiles inside
  const int ntiles = p.tiles_m * p.tiles_n;
  const int per_xcd = (ntiles + 7) >> 3;
  int bid = blockIdx.x;
  int split = 0;
  if (SPLIT) {
    split = bid % p.splits;
    bid /= p.splits;
  }
  const int t = (bid & 7) * per_xcd + (bid >> 3);
  if (t >= ntiles) return;
  constexpr int GM = 4;
  const int group = t / (GM * p.tiles_n);
  const int first_m = group * GM;
  const int gsz = min(p.tiles_m - first_m, GM);
  const int tin = t - group * GM * p.tiles_n;
  const int tile_m = first_m + tin % gsz;
  const int tile_n = tin / gsz;
  const int m0 = tile_m * kTileM, n0 = tile_n * kTileN;

  const int kb_begin = SPLIT ? split * p.kb_per_split : 0;
  const int kb_end = SPLIT ? min(p.K / kTileK, kb_begin + p.kb_per_split) : p.K / kTileK;

  // ---- global -> LDS: this wave fills row groups i = 4w..4w+3 (8 rows each) of W and of X
  const int rl = lane >> 3, cp = lane & 7;
  const uint8_t* gW[4];
  const uint8_t* gX[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = w * 4 + j;
    const int row = i * 8 + rl;
    const int c = cp ^ (((i & 1) << 2) + (rl >> 1));  // data chunk stored at chunk position cp
    const int nrow = min(n0 + row, p.N - 1);        // rows past the edge re-read the last row; never stored
    const int mrow = min(m0 + row, p.M - 1);
    gW[j] = p.W + (int64_t)nrow * p.ldw + c * 16 + (int64_t)kb_begin * kTileK;
    gX[j] = p.X + (int64_t)mrow * p.ldx + c * 16 + (int64_t)kb_begin * kTileK;
  }
  auto issue_loads = [&](int stage, int kstep) {
    uint8_t* base = smem + stage * kStageBytes + w * 4096;
#pragma unroll
    for (int j = 0; j < 4; ++j) load16_to_lds(gW[j] + (int64_t)kstep * kTileK, base + j * 1024);
#pragma unroll
    for (int j = 0; j < 4; ++j) load16_to_lds(gX[j] + (int64_t)kstep * kTileK, base + kXOff + j * 1024);
  };

  // ---- LDS -> MFMA operands
  const int lr = lane & 31, h = lane >> 5;
  const int swz = (lr >> 1) & 7;
  uint32_t co[2][2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int j = 0; j < 2; ++j) co[ks][j] = (uint32_t)(((ks * 4 + h * 2 + j) ^ swz) << 4);
  const uint32_t rdW = (uint32_t)((wn * 128 + lr) * kTileK);
  const uint32_t rdX = (uint32_t)(kXOff + (wm * 64 + lr) * kTileK);
  auto frag = [&](const uint8_t* st, uint32_t rowoff, int ks) -> v8i {
    const v4i lo = *reinterpret_cast<const v4i*>(st + rowoff + co[ks][0]);
    const v4i hi = *reinterpret_cast<const v4i*>(st + rowoff + co[ks][1]);
    v8i r;
    r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
    r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
    return r;
  };

  // ---- scales (block mode)
  const int mrow0 = min(m0 + wm * 64 + lr, p.M - 1);
  const int mrow1 = min(m0 + wm * 64 + 32 + lr, p.M - 1);
  const float* sx0 = p.sx + (int64_t)mrow0 * p.sx_m;
  const float* sx1 = p.sx + (int64_t)mrow1 * p.sx_m;
  const int nb = min(n0 + wn * 128, p.N - 1) >> 7;
  const float* swp = p.sw + (int64_t)nb * p.sw_n;

  v16f acc[4][2];
#pragma unroll
  for (int ns = 0; ns < 4; ++ns)
#pragma unroll
    for (int ms = 0; ms < 2; ++ms)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ns][ms][r] = 0.f;

  float sc_next[2] = {0.f, 0.f};
  if (kb_begin < kb_end) {
    issue_loads(0, 0);
    if (MODE == kModeBlock) {
      const float sb = swp[(int64_t)kb_begin * p.sw_k];
      sc_next[0] = sx0[(int64_t)kb_begin * p.sx_k] * sb;
      sc_next[1] = sx1[(int64_t)kb_begin * p.sx_k] * sb;
    }
  }

  for (int kb = kb_begin; kb < kb_end; ++kb) {
    const int it = kb - kb_begin;
    const int stage = it & 1;
    wait_vm0();
    __syncthreads();
    float sc[2] = {sc_next[0], sc_next[1]};
    if (kb + 1 < kb_end) {
      issue_loads(stage ^ 1, it + 1);
      if (MODE == kModeBlock) {
        const float sb = swp[(int64_t)(kb + 1) * p.sw_k];
        sc_next[0] = sx0[(int64_t)(kb + 1) * p.sx_k] * sb;
        sc_next[1] = sx1[(int64_t)(kb + 1) * p.sx_k] * sb;
      }
    }
    const uint8_t* st = smem + stage * kStageBytes;
    v8i xf[2][2];
#pragma unroll
    for (int ms = 0; ms < 2; ++ms)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) xf[ms][ks] = frag(st, rdX + ms * 32 * kTileK, ks);
#pragma unroll
    for (int ns = 0; ns < 4; ++ns) {
      v8i wf[2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) wf[ks] = frag(st, rdW + ns * 32 * kTileK, ks);
#pragma unroll
      for (int ms = 0; ms < 2; ++ms) {
        if (MODE == kModeBlock) {
          v16f z;
#pragma unroll
          for (int r = 0; r < 16; ++r) z[r] = 0.f;
          v16f tq = mfma_32x32x64(wf[0], xf[ms][0], z);
          tq = mfma_32x32x64(wf[1], xf[ms][1], tq);
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[ns][ms][r] = __builtin_fmaf(tq[r], sc[ms], acc[ns][ms][r]);
        } else {
          acc[ns][ms] = mfma_32x32x64(wf[0], xf[ms][0], acc[ns][ms]);
          acc[ns][ms] = mfma_32x32x64(wf[1], xf[ms][1], acc[ns][ms]);
        }
      }
    }
  }

  // ---- epilogue: lane holds C[m][n..n+3] for 4 n-runs per 32x32 tile
#pragma unroll
  for (int ms = 0; ms < 2; ++ms) {
    const int m = m0 + wm * 64 + ms * 32 + lr;
    if (m >= p.M) continue;
    float sa = 1.f;
    if (MODE == kModeRow && !SPLIT) sa = p.sx[m];
#pragma unroll
    for (int ns = 0; ns < 4; ++ns) {
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const int n = n0 + wn * 128 + ns * 32 + rg * 8 + h * 4;
        if (n >= p.N) continue;
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = acc[ns][ms][rg * 4 + r];
        if (SPLIT) {
          float4 o = make_float4(v[0], v[1], v[2], v[3]);
          *reinterpret_cast<float4*>(p.partial + ((int64_t)split * p.M + m) * p.N + n) = o;
        } else {
          if (MODE == kModeRow) {
            const float4 sb = *reinterpret_cast<const float4*>(p.sw + n);
            v[0] = v[0] * sb.x * sa; v[1] = v[1] * sb.y * sa; v[2] = v[2] * sb.z * sa; v[3] = v[3] * sb.w * sa;
            if (p.bias) {
#pragma unroll
              for (int r = 0; r < 4; ++r) v[r] += load_scalar<BIAS_DT>(p.bias, n + r);
            }
          }
          store4<OUT_DT>(p.C, (int64_t)m * p.ldc + n, v[0], v[1], v[2], v[3]);
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// split-K reduction: C = cast( sum_s partial[s] (* sa*sb + bias in row mode) )
// ------------------------------------------------------------------------------------------------
template <int MODE, int OUT_DT, int BIAS_DT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const GemmArgs p) {
  const int64_t quads = (int64_t)p.M * (p.N / 4);
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= quads) return;
  const int m = (int)(i / (p.N / 4));
  const int n = (int)(i % (p.N / 4)) * 4;
  float4 s = make_float4(0, 0, 0, 0);
  for (int k = 0; k < p.splits; ++k) {
    const float4 v = *reinterpret_cast<const float4*>(p.partial + ((int64_t)k * p.M + m) * p.N + n);
    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
  }
  if (MODE == kModeRow) {
    const float sa = p.sx[m];
    const float4 sb = *reinterpret_cast<const float4*>(p.sw + n);
    s.x = s.x * sb.x * sa; s.y = s.y * sb.y * sa; s.z = s.z * sb.z * sa; s.w = s.w * sb.w * sa;
    if (p.bias) {
      s.x += load_scalar<BIAS_DT>(p.bias, n); s.y += load_scalar<BIAS_DT>(p.bias, n + 1);
      s.z += load_scalar<BIAS_DT>(p.bias, n + 2); s.w += load_scalar<BIAS_DT>(p.bias, n + 3);
    }
  }
  store4<OUT_DT>(p.C, (int64_t)m * p.ldc + n, s.x, s.y, s.z, s.w);
}

// ------------------------------------------------------------------------------------------------
// reference-shaped fallback for K that is not a multiple of 128 (or other shapes the tiled kernels
// do not take): one lane per output, scalar decode.  Correct for every shape the API admits.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float fp8_to_f32(uint32_t word, int byte) {
  switch (byte) {
    case 0: return __builtin_amdgcn_cvt_f32_fp8((int)word, 0);
    case 1: return __builtin_amdgcn_cvt_f32_fp8((int)word, 1);
    case 2: return __builtin_amdgcn_cvt_f32_fp8((int)word, 2);
    default: return __builtin_amdgcn_cvt_f32_fp8((int)word, 3);
  }
}

template <int MODE, int OUT_DT, int BIAS_DT>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const GemmArgs p) {
  const int n = blockIdx.x * 64 + (threadIdx.x & 63);
  const int m = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (n >= p.N || m >= p.M) return;
  const uint8_t* x = p.X + (int64_t)m * p.ldx;
  const uint8_t* wr = p.W + (int64_t)n * p.ldw;
  float acc = 0.f;
  for (int k0 = 0; k0 < p.K; k0 += kTileK) {
    const int kend = min(p.K, k0 + kTileK);
    float part = 0.f;
    for (int k = k0; k < kend; k += 4) {
      const uint32_t xa = *reinterpret_cast<const uint32_t*>(x + k);
      const uint32_t wa = *reinterpret_cast<const uint32_t*>(wr + k);
#pragma unroll
      for (int b = 0; b < 4; ++b) part = __builtin_fmaf(fp8_to_f32(xa, b), fp8_to_f32(wa, b), part);
    }
    if (MODE == kModeBlock) {
      const int kb = k0 / kTileK;
      acc = __builtin_fmaf(part, p.sx[(int64_t)m * p.sx_m + (int64_t)kb * p.sx_k] *
                                     p.sw[(int64_t)(n >> 7) * p.sw_n + (int64_t)kb * p.sw_k], acc);
    } else {
      acc += part;
    }
  }
  if (MODE == kModeRow) {
    acc = acc * p.sw[n] * p.sx[m];
    if (p.bias) acc += load_scalar<BIAS_DT>(p.bias, n);
  }
  if (OUT_DT == FP8K_BF16)
    ((u16*)p.C)[(int64_t)m * p.ldc + n] = (u16)f32_to_bf16_bits(acc);
  else
    ((u16*)p.C)[(int64_t)m * p.ldc + n] = (u16)f32_to_f16_bits(acc);
}

}  // namespace fp8k
