// FP8 (OCP e4m3fn) quantisation kernels for gfx950: per-token-group, per-token, per-tensor.
//
// All three are HBM-bound streaming kernels: 16-byte loads, 8/16-byte stores, one pass over the
// input held in registers, amax by DPP lane exchange inside the wavefront.
#include "fp8k_common.h"
#include "quant_math.h"

namespace fp8k {

// ------------------------------------------------------------------------------------------------
// loading 8 consecutive elements as float
// ------------------------------------------------------------------------------------------------
template <int DT>
struct Raw8;
template <>
struct Raw8<FP8K_BF16> {
  uint4 v;
  __device__ __forceinline__ void load(const void* base, int64_t elem) { v = *reinterpret_cast<const uint4*>((const u16*)base + elem); }
  __device__ __forceinline__ void zero() { v = make_uint4(0, 0, 0, 0); }
  __device__ __forceinline__ void unpack(float (&a)[8]) const {
    a[0] = bf16_lo(v.x); a[1] = bf16_hi(v.x); a[2] = bf16_lo(v.y); a[3] = bf16_hi(v.y);
    a[4] = bf16_lo(v.z); a[5] = bf16_hi(v.z); a[6] = bf16_lo(v.w); a[7] = bf16_hi(v.w);
  }
};
template <>
struct Raw8<FP8K_F16> {
  uint4 v;
  __device__ __forceinline__ void load(const void* base, int64_t elem) { v = *reinterpret_cast<const uint4*>((const u16*)base + elem); }
  __device__ __forceinline__ void zero() { v = make_uint4(0, 0, 0, 0); }
  __device__ __forceinline__ void unpack(float (&a)[8]) const {
    a[0] = f16_bits_to_f32(v.x & 0xffff); a[1] = f16_bits_to_f32(v.x >> 16);
    a[2] = f16_bits_to_f32(v.y & 0xffff); a[3] = f16_bits_to_f32(v.y >> 16);
    a[4] = f16_bits_to_f32(v.z & 0xffff); a[5] = f16_bits_to_f32(v.z >> 16);
    a[6] = f16_bits_to_f32(v.w & 0xffff); a[7] = f16_bits_to_f32(v.w >> 16);
  }
};
template <>
struct Raw8<FP8K_F32> {
  float4 lo, hi;
  __device__ __forceinline__ void load(const void* base, int64_t elem) {
    const float4* p = reinterpret_cast<const float4*>((const float*)base + elem);
    lo = p[0];
    hi = p[1];
  }
  __device__ __forceinline__ void zero() { lo = make_float4(0, 0, 0, 0); hi = lo; }
  __device__ __forceinline__ void unpack(float (&a)[8]) const {
    a[0] = lo.x; a[1] = lo.y; a[2] = lo.z; a[3] = lo.w; a[4] = hi.x; a[5] = hi.y; a[6] = hi.z; a[7] = hi.w;
  }
};

__device__ __forceinline__ float absmax8(const float (&a)[8]) {
  float m = fmaxf(fabsf(a[0]), fabsf(a[1]));
  m = fmaxf(fmaxf(m, fabsf(a[2])), fabsf(a[3]));
  m = fmaxf(fmaxf(m, fabsf(a[4])), fabsf(a[5]));
  m = fmaxf(fmaxf(m, fabsf(a[6])), fabsf(a[7]));
  return m;
}

// ------------------------------------------------------------------------------------------------
// per-token-group quant
//
// The unit of work is a 1 KB "segment" (64 lanes x 8 elements = 512 columns of one row, i.e.
// GPW = 512/GROUP groups; LPG = GROUP/8 adjacent lanes form a group).  A wavefront owns SEG segments:
// SEG consecutive ones of the flat input (contiguous memory whenever K is a multiple of 512) for
// row-major scales, or the same segment of SEG consecutive rows (ROWFAST) for scale layouts whose rows
// are the contiguous direction.  It loads them all with 16-byte nontemporal loads before touching the
// first, and writes each back as one 8-byte store per lane.  Both streams are used once, so they
// bypass cache retention.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ uint4 load16_stream(const void* p) {
  const v4i v = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(p));
  return make_uint4((uint32_t)v[0], (uint32_t)v[1], (uint32_t)v[2], (uint32_t)v[3]);
}
__device__ __forceinline__ void store8_stream(void* p, uint2 o) {
  v2i v;
  v[0] = (int)o.x;
  v[1] = (int)o.y;
  __builtin_nontemporal_store(v, reinterpret_cast<v2i*>(p));
}

template <int DT>
__device__ __forceinline__ void load_stream(Raw8<DT>& r, const void* base, int64_t elem) {
  if constexpr (DT == FP8K_F32) {
    const float* p = (const float*)base + elem;
    const uint4 a = load16_stream(p), b = load16_stream(p + 4);
    r.lo = make_float4(__uint_as_float(a.x), __uint_as_float(a.y), __uint_as_float(a.z), __uint_as_float(a.w));
    r.hi = make_float4(__uint_as_float(b.x), __uint_as_float(b.y), __uint_as_float(b.z), __uint_as_float(b.w));
  } else {
    r.v = load16_stream((const u16*)base + elem);
  }
}

// FUSE: the value that gets quantised is T( T(silu(gate)) * up ) with gate = x[m, c], up = x[m, K + c] of an
// input row of 2K elements - what silu_and_mul would have written to memory, bit for bit (same two roundings).
template <int DT>
__device__ __forceinline__ void silu_mul8(const Raw8<DT>& gate, const Raw8<DT>& up, float (&a)[8]) {
  float g[8], u[8];
  gate.unpack(g);
  up.unpack(u);
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = round_to<DT>(round_to<DT>(silu_f32(g[i])) * u[i]);
}

// MASKED: the M rows are E experts x m_max slots; only the first masked_m[e] slots of expert e are quantised
// (the others are neither read nor written), and the scale of slot i of expert e sits at e*se + i*sm + g*sg.
template <int DT, int GROUP, int KIND, int SEG, bool ROWFAST, bool FUSE, bool MASKED>
__global__ __launch_bounds__(256) void group_quant_kernel(const void* __restrict__ x, uint8_t* __restrict__ q,
                                                          void* __restrict__ s, int M, int G, int64_t K,
                                                          int nseg_row, float eps, int64_t sm, int64_t sg,
                                                          const int32_t* __restrict__ masked_m, int m_max, int64_t se) {
  const int64_t XK = FUSE ? 2 * K : K;  // elements per input row
  auto scale_row = [&](int r) -> int64_t {  // offset of the scales of row r
    if (!MASKED) return (int64_t)r * sm;
    const int e = r / m_max;
    return (int64_t)e * se + (int64_t)(r - e * m_max) * sm;
  };
  constexpr int LPG = GROUP / 8;
  constexpr int GPW = 64 / LPG;
  static_assert(KIND != FP8K_SCALE_UE8M0_PACKED || GROUP == 128, "packed UE8M0 scales need 128-element groups");

  const int lane = threadIdx.x & 63;
  const int lg = lane / LPG, li = lane % LPG;
  // A wave owns SEG tasks (row, segment-in-row).  Row-major scales: SEG consecutive segments, i.e. contiguous
  // memory and SEG*GPW consecutive scales.  ROWFAST (scales whose rows are contiguous: column-major float,
  // packed UE8M0): the same segment of SEG consecutive rows, so that the SEG scales of a group column are
  // adjacent words that leave the wave together.
  const unsigned wave = blockIdx.x * 4u + (unsigned)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const unsigned total = (unsigned)M * (unsigned)nseg_row;
  int row, sr;
  if (ROWFAST) {
    row = (int)(wave / (unsigned)nseg_row) * SEG;
    sr = (int)(wave % (unsigned)nseg_row);
    if (row >= M) return;
  } else {
    if (wave * SEG >= total) return;
    row = (int)(wave * SEG / (unsigned)nseg_row);
    sr = (int)(wave * SEG - (unsigned)row * (unsigned)nseg_row);
  }

  Raw8<DT> raw[SEG], up[FUSE ? SEG : 1];
  int rows[SEG], segs[SEG];
  bool act[SEG];  // wave-uniform: task j exists
  float scv[SEG];
  uint32_t redo_mask = 0;
#pragma unroll
  for (int j = 0; j < SEG; ++j) {
    rows[j] = row;
    segs[j] = sr;
    act[j] = ROWFAST ? row < M : wave * SEG + j < total;
    if (MASKED && act[j]) {
      const int e = row / m_max;
      act[j] = row - e * m_max < masked_m[e];
    }
    if (act[j]) {
      const int g = sr * GPW + lg;
      // lanes past the last group of the row re-read the last group and store nothing
      const int64_t col = (int64_t)(g < G ? g : G - 1) * GROUP + li * 8;
      load_stream<DT>(raw[j], x, (int64_t)row * XK + col);
      if (FUSE) load_stream<DT>(up[j], x, (int64_t)row * XK + K + col);
    }
    if (ROWFAST) {
      ++row;
    } else if (++sr == nseg_row) {
      sr = 0;
      ++row;
    }
  }
#pragma unroll
  for (int j = 0; j < SEG; ++j) {
    if (act[j]) {  // wave-uniform
      const int g = segs[j] * GPW + lg;
      const bool valid = g < G;
      float a[8];
      if (FUSE) silu_mul8<DT>(raw[j], up[FUSE ? j : 0], a);
      else raw[j].unpack(a);
      const float amax = fmaxf(group_max<LPG>(absmax8(a)), eps);
      const float sc = div448<DT != FP8K_F32>(amax);
      uint2 out;
      if (KIND == FP8K_SCALE_UE8M0_PACKED) {
        // round the scale up to a power of two; x / 2^e == x * 2^-e exactly
        const uint32_t b = __float_as_uint(fmaxf(sc, 1e-10f));
        const uint32_t e = (b >> 23) + ((b & 0x7fffffu) != 0u);
        const float rinv = __uint_as_float((254u - e) << 23);
        out.x = cvt4_fp8(a[0] * rinv, a[1] * rinv, a[2] * rinv, a[3] * rinv);
        out.y = cvt4_fp8(a[4] * rinv, a[5] * rinv, a[6] * rinv, a[7] * rinv);
        const uint32_t eb = valid ? e : 0u;  // bytes of groups past the row end stay zero
        const uint32_t w = (uint32_t)__builtin_amdgcn_readlane((int)eb, 0) |
                           ((uint32_t)__builtin_amdgcn_readlane((int)eb, 16) << 8) |
                           ((uint32_t)__builtin_amdgcn_readlane((int)eb, 32) << 16) |
                           ((uint32_t)__builtin_amdgcn_readlane((int)eb, 48) << 24);
        if (lane == 0) reinterpret_cast<uint32_t*>(s)[(int64_t)segs[j] * sg + scale_row(rows[j])] = w;
      } else if (KIND == FP8K_SCALE_UE8M0_F32) {
        // the same power of two, stored as a float at the place of a float scale
        const uint32_t b = __float_as_uint(fmaxf(sc, 1e-10f));
        const uint32_t e = (b >> 23) + ((b & 0x7fffffu) != 0u);
        const float rinv = __uint_as_float((254u - e) << 23);
        out.x = cvt4_fp8(a[0] * rinv, a[1] * rinv, a[2] * rinv, a[3] * rinv);
        out.y = cvt4_fp8(a[4] * rinv, a[5] * rinv, a[6] * rinv, a[7] * rinv);
        if (valid && li == 0) reinterpret_cast<float*>(s)[scale_row(rows[j]) + (int64_t)g * sg] = __uint_as_float(e << 23);
      } else {
        bool redo;
        out = quant8_bracket<DT != FP8K_F32>(a, sc, amax, redo);
        redo_mask |= (redo & valid) ? (1u << j) : 0u;
        scv[j] = sc;
        if (valid && li == 0) reinterpret_cast<float*>(s)[scale_row(rows[j]) + (int64_t)g * sg] = sc;
      }
      if (valid) store8_stream(q + (int64_t)rows[j] * K + (int64_t)g * GROUP + li * 8, out);
    }
  }
  // cold: lanes whose bracket was inconclusive reload their 8 values (still in cache) and divide
  if (KIND == FP8K_SCALE_F32 && __builtin_expect(redo_mask != 0, 0)) {
#pragma unroll 1
    for (int j = 0; j < SEG; ++j) {
      if (redo_mask & (1u << j)) {
        float sc = scv[0];
#pragma unroll
        for (int i = 1; i < SEG; ++i) sc = j == i ? scv[i] : sc;
        int row = rows[0], seg = segs[0];
#pragma unroll
        for (int i = 1; i < SEG; ++i) { row = j == i ? rows[i] : row; seg = j == i ? segs[i] : seg; }
        const int64_t col = (int64_t)(seg * GPW + lg) * GROUP + li * 8;
        Raw8<DT> again;
        again.load(x, (int64_t)row * XK + col);
        float a[8];
        if (FUSE) {
          Raw8<DT> again_up;
          again_up.load(x, (int64_t)row * XK + K + col);
          silu_mul8<DT>(again, again_up, a);
        } else {
          again.unpack(a);
        }
        store8_stream(q + (int64_t)row * K + col, quant8_divide(a, sc));
      }
    }
  }
}

template <int DT, int GROUP, int KIND, bool FUSE = false, bool MASKED = false>
static int launch_group_quant(const void* x, void* q, void* s, int64_t M, int64_t K, float eps, int64_t sm, int64_t sg,
                              hipStream_t st, const int32_t* masked_m = nullptr, int m_max = 1, int64_t se = 0) {
  constexpr int GPW = 64 / (GROUP / 8);
  constexpr int SEG = 4;
  const int G = (int)(K / GROUP);
  const int nseg_row = (G + GPW - 1) / GPW;
  const int64_t total = M * nseg_row;
  if (total > 0x7fffffffLL / SEG) return fail(FP8K_ERR_INVALID, "group_quant: input too large for one launch");
  const bool rowfast = KIND == FP8K_SCALE_UE8M0_PACKED || sm < sg;  // rows of the scale tensor are contiguous
  const int64_t waves = rowfast ? (M + SEG - 1) / SEG * nseg_row : (total + SEG - 1) / SEG;
  const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
  if (rowfast)
    hipLaunchKernelGGL((group_quant_kernel<DT, GROUP, KIND, SEG, true, FUSE, MASKED>), grid, block, 0, st, x, (uint8_t*)q, s,
                       (int)M, G, K, nseg_row, eps, sm, sg, masked_m, m_max, se);
  else
    hipLaunchKernelGGL((group_quant_kernel<DT, GROUP, KIND, SEG, false, FUSE, MASKED>), grid, block, 0, st, x, (uint8_t*)q, s,
                       (int)M, G, K, nseg_row, eps, sm, sg, masked_m, m_max, se);
  return check_launch("group_quant");
}

template <int DT, int KIND>
static int dispatch_group(const void* x, void* q, void* s, int64_t M, int64_t K, int64_t group, float eps, int64_t sm,
                          int64_t sg, hipStream_t st) {
  if (KIND == FP8K_SCALE_UE8M0_PACKED) {
    if (group != 128) return fail(FP8K_ERR_INVALID, "group_quant: packed UE8M0 scales require group_size 128");
    return launch_group_quant<DT, 128, KIND>(x, q, s, M, K, eps, sm, sg, st);
  }
  switch (group) {
    case 16: return launch_group_quant<DT, 16, FP8K_SCALE_F32>(x, q, s, M, K, eps, sm, sg, st);
    case 32: return launch_group_quant<DT, 32, FP8K_SCALE_F32>(x, q, s, M, K, eps, sm, sg, st);
    case 64: return launch_group_quant<DT, 64, FP8K_SCALE_F32>(x, q, s, M, K, eps, sm, sg, st);
    case 128: return launch_group_quant<DT, 128, FP8K_SCALE_F32>(x, q, s, M, K, eps, sm, sg, st);
    case 256: return launch_group_quant<DT, 256, FP8K_SCALE_F32>(x, q, s, M, K, eps, sm, sg, st);
    case 512: return launch_group_quant<DT, 512, FP8K_SCALE_F32>(x, q, s, M, K, eps, sm, sg, st);
  }
  return fail(FP8K_ERR_INVALID, "group_quant: group_size %lld not in {16,32,64,128,256,512}", (long long)group);
}

// ------------------------------------------------------------------------------------------------
// per-token quant: one workgroup per row, row held in registers between the amax and the cast
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float block_max_256(float v, float* red) {
  v = group_max<64>(v);
  const int w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  v = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  return v;
}

template <int DT>
__global__ __launch_bounds__(256) void token_quant_kernel(const void* __restrict__ x, uint8_t* __restrict__ q,
                                                          float* __restrict__ s, int64_t K) {
  constexpr int HOLD = 8;  // 8 chunks x 256 threads x 8 elements = 16384 columns stay in registers
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const int nchunk = (int)(K / 8);
  Raw8<DT> raw[HOLD];
  float m = 0.f;
#pragma unroll
  for (int c = 0; c < HOLD; ++c) {
    const int ch = c * 256 + threadIdx.x;
    if (ch < nchunk) {
      raw[c].load(x, row * K + (int64_t)ch * 8);
      float a[8];
      raw[c].unpack(a);
      m = fmaxf(m, absmax8(a));
    }
  }
  for (int ch = HOLD * 256 + threadIdx.x; ch < nchunk; ch += 256) {
    Raw8<DT> t;
    t.load(x, row * K + (int64_t)ch * 8);
    float a[8];
    t.unpack(a);
    m = fmaxf(m, absmax8(a));
  }
  m = block_max_256(m, red);
  const float sc = m / kFp8Max;
  if (threadIdx.x == 0) s[row] = sc;
  const float inv = (sc == 0.f) ? 0.f : 1.0f / sc;
  auto emit = [&](const float(&a)[8], int ch) {
    float y[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = fmaxf(fminf(a[i] * inv, kFp8Max), -kFp8Max);
    uint2 o;
    o.x = cvt4_fp8(y[0], y[1], y[2], y[3]);
    o.y = cvt4_fp8(y[4], y[5], y[6], y[7]);
    *reinterpret_cast<uint2*>(q + row * K + (int64_t)ch * 8) = o;
  };
#pragma unroll
  for (int c = 0; c < HOLD; ++c) {
    const int ch = c * 256 + threadIdx.x;
    if (ch < nchunk) {
      float a[8];
      raw[c].unpack(a);
      emit(a, ch);
    }
  }
  for (int ch = HOLD * 256 + threadIdx.x; ch < nchunk; ch += 256) {
    Raw8<DT> t;
    t.load(x, row * K + (int64_t)ch * 8);
    float a[8];
    t.unpack(a);
    emit(a, ch);
  }
}

// ------------------------------------------------------------------------------------------------
// per-tensor quant: grid-stride absmax with one atomic max per workgroup, then the cast
// ------------------------------------------------------------------------------------------------
template <int DT>
__device__ __forceinline__ float load1(const void* x, int64_t i) {
  if (DT == FP8K_F32) return ((const float*)x)[i];
  if (DT == FP8K_BF16) return __uint_as_float((uint32_t)((const u16*)x)[i] << 16);
  return f16_bits_to_f32(((const u16*)x)[i]);
}

template <int DT>
__global__ __launch_bounds__(256) void tensor_absmax_kernel(const void* __restrict__ x, float* __restrict__ s,
                                                            int64_t numel) {
  __shared__ float red[4];
  const int64_t nchunk = numel / 8;
  const int64_t stride = (int64_t)gridDim.x * 256;
  float m = 0.f;
  for (int64_t ch = (int64_t)blockIdx.x * 256 + threadIdx.x; ch < nchunk; ch += stride) {
    Raw8<DT> t;
    t.load(x, ch * 8);
    float a[8];
    t.unpack(a);
    m = fmaxf(m, absmax8(a));
  }
  for (int64_t i = nchunk * 8 + (int64_t)blockIdx.x * 256 + threadIdx.x; i < numel; i += stride)
    m = fmaxf(m, fabsf(load1<DT>(x, i)));
  m = block_max_256(m, red);
  // non-negative floats order like their bit patterns
  if (threadIdx.x == 0) atomicMax(reinterpret_cast<unsigned int*>(s), __float_as_uint(m / kFp8Max));
}

template <int DT>
__global__ __launch_bounds__(256) void tensor_quant_kernel(const void* __restrict__ x, uint8_t* __restrict__ q,
                                                           const float* __restrict__ s, int64_t numel) {
  const float inv = 1.0f / s[0];
  const int64_t nchunk = numel / 8;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t ch = (int64_t)blockIdx.x * 256 + threadIdx.x; ch < nchunk; ch += stride) {
    Raw8<DT> t;
    t.load(x, ch * 8);
    float a[8], y[8];
    t.unpack(a);
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = fmaxf(fminf(a[i] * inv, kFp8Max), -kFp8Max);
    uint2 o;
    o.x = cvt4_fp8(y[0], y[1], y[2], y[3]);
    o.y = cvt4_fp8(y[4], y[5], y[6], y[7]);
    *reinterpret_cast<uint2*>(q + ch * 8) = o;
  }
  for (int64_t i = nchunk * 8 + (int64_t)blockIdx.x * 256 + threadIdx.x; i < numel; i += stride) {
    float y = fmaxf(fminf(load1<DT>(x, i) * inv, kFp8Max), -kFp8Max);
    q[i] = (uint8_t)(cvt_pk_fp8_lo(y, 0.f, 0) & 0xff);
  }
}

// ------------------------------------------------------------------------------------------------
// per-tensor quant of a strided [H, S, D] tensor into a contiguous one (the MLA absorbed products): a workgroup takes
// whole rows (h, s) in grid-stride, a lane 8 elements at a time
// ------------------------------------------------------------------------------------------------
template <int DT, bool QUANT>
__global__ __launch_bounds__(256) void rows_tensor_quant_kernel(const void* __restrict__ x, uint8_t* __restrict__ q,
                                                                float* __restrict__ s, int64_t rows, int S, int D,
                                                                int64_t stride_h, int64_t stride_s, float eps) {
  __shared__ float red[4];
  const int chunks = D / 8;                 // per row; the host checks D % 8 == 0 and the alignment of every row
  const int64_t total = rows * chunks;
  const int64_t step = (int64_t)gridDim.x * 256;
  const float inv = QUANT ? 1.0f / s[0] : 0.f;
  float m = 0.f;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += step) {
    const int64_t row = i / chunks;
    const int c = (int)(i - row * chunks);
    const int64_t hh = row / S, ss = row - hh * S;
    Raw8<DT> t;
    t.load(x, hh * stride_h + ss * stride_s + c * 8);
    float a[8];
    t.unpack(a);
    if (QUANT) {
      float y[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = fmaxf(fminf(a[j] * inv, kFp8Max), -kFp8Max);
      uint2 o;
      o.x = cvt4_fp8(y[0], y[1], y[2], y[3]);
      o.y = cvt4_fp8(y[4], y[5], y[6], y[7]);
      *reinterpret_cast<uint2*>(q + row * D + c * 8) = o;
    } else {
      m = fmaxf(m, absmax8(a));
    }
  }
  if (!QUANT) {
    m = block_max_256(fmaxf(m, eps), red);
    // non-negative floats order like their bit patterns
    if (threadIdx.x == 0) atomicMax(reinterpret_cast<unsigned int*>(s), __float_as_uint(m / kFp8Max));
  }
}

}  // namespace fp8k

using namespace fp8k;

extern "C" int fp8k_group_quant(const void* x, void* q, void* s, int64_t M, int64_t K, int64_t group_size, float eps,
                                float fp8_min, float fp8_max, int in_dtype, int64_t s_stride_m, int64_t s_stride_g,
                                int scale_kind, void* stream) {
  clear_error();
  FP8K_REQUIRE(M >= 0 && K >= 0, "group_quant: negative shape");
  FP8K_REQUIRE(group_size > 0 && K % group_size == 0,
               "group_quant: the last dimension of `x` (%lld) cannot be divisible by `group_size` (%lld)", (long long)K,
               (long long)group_size);
  FP8K_REQUIRE(fp8_max == 448.0f && fp8_min == -448.0f, "group_quant: fp8_min/fp8_max must be -448/448 (OCP e4m3fn)");
  FP8K_REQUIRE(in_dtype == FP8K_F32 || in_dtype == FP8K_F16 || in_dtype == FP8K_BF16, "group_quant: bad input dtype %d",
               in_dtype);
  FP8K_REQUIRE(scale_kind == FP8K_SCALE_F32 || scale_kind == FP8K_SCALE_UE8M0_PACKED, "group_quant: bad scale kind %d",
               scale_kind);
  FP8K_REQUIRE(M <= 0x7fffffffLL && K / group_size <= 0x7fffffffLL, "group_quant: shape too large");
  if (M == 0 || K == 0) return FP8K_OK;
  FP8K_REQUIRE(x && q && s, "group_quant: null pointer");
  FP8K_REQUIRE(aligned(x, 16) && aligned(q, 8) && aligned(s, 4), "group_quant: x must be 16-byte, q 8-byte aligned");
  const int64_t G = K / group_size;
  if (scale_kind == FP8K_SCALE_F32) {
    FP8K_REQUIRE(s_stride_m >= 0 && s_stride_g >= 0 && (M == 1 || s_stride_m > 0) && (G == 1 || s_stride_g > 0),
                 "group_quant: scale strides must be positive");
  } else {
    FP8K_REQUIRE(s_stride_m > 0 && ((G + 3) / 4 == 1 || s_stride_g > 0), "group_quant: packed scale strides must be positive");
  }
  // the torch-native formula clamps amax in the input dtype: bf16 sees eps rounded to bf16
  float eps_eff = eps;
  if (in_dtype == FP8K_BF16) {
    uint32_t u;
    memcpy(&u, &eps, 4);
    u = ((u + 0x7fffu + ((u >> 16) & 1u)) >> 16) << 16;
    memcpy(&eps_eff, &u, 4);
  }
  hipStream_t st = (hipStream_t)stream;
#define FP8K_GQ(DT)                                                                                               \
  (scale_kind == FP8K_SCALE_F32                                                                                   \
       ? dispatch_group<DT, FP8K_SCALE_F32>(x, q, s, M, K, group_size, eps_eff, s_stride_m, s_stride_g, st)       \
       : dispatch_group<DT, FP8K_SCALE_UE8M0_PACKED>(x, q, s, M, K, group_size, eps_eff, s_stride_m, s_stride_g, st))
  switch (in_dtype) {
    case FP8K_BF16: return FP8K_GQ(FP8K_BF16);
    case FP8K_F16: return FP8K_GQ(FP8K_F16);
    default: return FP8K_GQ(FP8K_F32);
  }
#undef FP8K_GQ
}

extern "C" int fp8k_silu_mul_group_quant(const void* x, void* q, void* s, int64_t M, int64_t K, int64_t group_size,
                                         float eps, float fp8_min, float fp8_max, int in_dtype, int64_t s_stride_m,
                                         int64_t s_stride_g, int scale_kind, void* stream) {
  clear_error();
  const char* op = "silu_mul_group_quant";
  FP8K_REQUIRE(M >= 0 && K >= 0, "%s: negative shape", op);
  FP8K_REQUIRE(group_size == 128, "%s: the fused form is built for group_size 128 (got %lld)", op, (long long)group_size);
  FP8K_REQUIRE(K % group_size == 0, "%s: the output width (%lld) cannot be divisible by `group_size` (%lld)", op,
               (long long)K, (long long)group_size);
  FP8K_REQUIRE(fp8_max == 448.0f && fp8_min == -448.0f, "%s: fp8_min/fp8_max must be -448/448 (OCP e4m3fn)", op);
  FP8K_REQUIRE(in_dtype == FP8K_F32 || in_dtype == FP8K_F16 || in_dtype == FP8K_BF16, "%s: bad input dtype %d", op, in_dtype);
  FP8K_REQUIRE(scale_kind == FP8K_SCALE_F32 || scale_kind == FP8K_SCALE_UE8M0_PACKED, "%s: bad scale kind %d", op, scale_kind);
  FP8K_REQUIRE(M <= 0x7fffffffLL && K / group_size <= 0x3fffffffLL, "%s: shape too large", op);
  if (M == 0 || K == 0) return FP8K_OK;
  FP8K_REQUIRE(x && q && s, "%s: null pointer", op);
  FP8K_REQUIRE(aligned(x, 16) && aligned(q, 8) && aligned(s, 4), "%s: x must be 16-byte, q 8-byte aligned", op);
  const int64_t G = K / group_size;
  if (scale_kind == FP8K_SCALE_F32) {
    FP8K_REQUIRE(s_stride_m >= 0 && s_stride_g >= 0 && (M == 1 || s_stride_m > 0) && (G == 1 || s_stride_g > 0),
                 "%s: scale strides must be positive", op);
  } else {
    FP8K_REQUIRE(s_stride_m > 0 && ((G + 3) / 4 == 1 || s_stride_g > 0), "%s: packed scale strides must be positive", op);
  }
  float eps_eff = eps;  // clamped in the input dtype, as in fp8k_group_quant
  if (in_dtype == FP8K_BF16) {
    uint32_t u;
    memcpy(&u, &eps, 4);
    u = ((u + 0x7fffu + ((u >> 16) & 1u)) >> 16) << 16;
    memcpy(&eps_eff, &u, 4);
  }
  hipStream_t st = (hipStream_t)stream;
#define FP8K_SGQ(DT)                                                                                                 \
  (scale_kind == FP8K_SCALE_F32                                                                                     \
       ? launch_group_quant<DT, 128, FP8K_SCALE_F32, true>(x, q, s, M, K, eps_eff, s_stride_m, s_stride_g, st)      \
       : launch_group_quant<DT, 128, FP8K_SCALE_UE8M0_PACKED, true>(x, q, s, M, K, eps_eff, s_stride_m, s_stride_g, st))
  switch (in_dtype) {
    case FP8K_BF16: return FP8K_SGQ(FP8K_BF16);
    case FP8K_F16: return FP8K_SGQ(FP8K_F16);
    default: return FP8K_SGQ(FP8K_F32);
  }
#undef FP8K_SGQ
}

extern "C" int fp8k_group_quant_masked(const void* x, void* q, void* s, int64_t E, int64_t m_max, int64_t K,
                                       int64_t group_size, float eps, float fp8_min, float fp8_max, int in_dtype,
                                       int64_t s_stride_e, int64_t s_stride_m, int64_t s_stride_g, int scale_kind,
                                       int fuse_silu_and_mul, const int32_t* masked_m, void* stream) {
  clear_error();
  const char* op = "group_quant_masked";
  FP8K_REQUIRE(E >= 0 && m_max >= 0 && K >= 0, "%s: negative shape", op);
  FP8K_REQUIRE(group_size == 128, "%s: the masked form is built for group_size 128 (got %lld)", op, (long long)group_size);
  FP8K_REQUIRE(K % group_size == 0, "%s: the output width (%lld) cannot be divisible by `group_size` (%lld)", op,
               (long long)K, (long long)group_size);
  FP8K_REQUIRE(fp8_max == 448.0f && fp8_min == -448.0f, "%s: fp8_min/fp8_max must be -448/448 (OCP e4m3fn)", op);
  FP8K_REQUIRE(in_dtype == FP8K_F32 || in_dtype == FP8K_F16 || in_dtype == FP8K_BF16, "%s: bad input dtype %d", op, in_dtype);
  FP8K_REQUIRE(scale_kind == FP8K_SCALE_F32 || scale_kind == FP8K_SCALE_UE8M0_PACKED || scale_kind == FP8K_SCALE_UE8M0_F32,
               "%s: bad scale kind %d", op, scale_kind);
  FP8K_REQUIRE(E * m_max <= 0x7fffffffLL && m_max <= 0x7fffffffLL && K / group_size <= 0x3fffffffLL, "%s: shape too large", op);
  if (E == 0 || m_max == 0 || K == 0) return FP8K_OK;
  FP8K_REQUIRE(x && q && s && masked_m, "%s: null pointer", op);
  FP8K_REQUIRE(aligned(x, 16) && aligned(q, 8) && aligned(s, 4) && aligned(masked_m, 4), "%s: x must be 16-byte, q 8-byte aligned", op);
  FP8K_REQUIRE(s_stride_e >= 0 && s_stride_m >= 0 && s_stride_g >= 0, "%s: negative scale stride", op);
  float eps_eff = eps;  // clamped in the input dtype, as in fp8k_group_quant
  if (in_dtype == FP8K_BF16) {
    uint32_t u;
    memcpy(&u, &eps, 4);
    u = ((u + 0x7fffu + ((u >> 16) & 1u)) >> 16) << 16;
    memcpy(&eps_eff, &u, 4);
  }
  hipStream_t st = (hipStream_t)stream;
  const int64_t M = E * m_max;
#define FP8K_MQ3(DT, KIND, FUSE) \
  launch_group_quant<DT, 128, KIND, FUSE, true>(x, q, s, M, K, eps_eff, s_stride_m, s_stride_g, st, masked_m, (int)m_max, s_stride_e)
#define FP8K_MQ2(DT, KIND) (fuse_silu_and_mul ? FP8K_MQ3(DT, KIND, true) : FP8K_MQ3(DT, KIND, false))
#define FP8K_MQ(DT)                                                  \
  (scale_kind == FP8K_SCALE_F32            ? FP8K_MQ2(DT, FP8K_SCALE_F32) \
   : scale_kind == FP8K_SCALE_UE8M0_PACKED ? FP8K_MQ2(DT, FP8K_SCALE_UE8M0_PACKED) \
                                           : FP8K_MQ2(DT, FP8K_SCALE_UE8M0_F32))
  switch (in_dtype) {
    case FP8K_BF16: return FP8K_MQ(FP8K_BF16);
    case FP8K_F16: return FP8K_MQ(FP8K_F16);
    default: return FP8K_MQ(FP8K_F32);
  }
#undef FP8K_MQ
#undef FP8K_MQ2
#undef FP8K_MQ3
}

extern "C" int fp8k_token_quant(const void* x, void* q, float* s, int64_t M, int64_t K, int in_dtype, void* stream) {
  clear_error();
  FP8K_REQUIRE(M >= 0 && K >= 0, "token_quant: negative shape");
  FP8K_REQUIRE(K % 8 == 0, "token_quant: hidden dimension (%lld) must be divisible by 8", (long long)K);
  FP8K_REQUIRE(in_dtype == FP8K_F32 || in_dtype == FP8K_F16 || in_dtype == FP8K_BF16, "token_quant: bad input dtype %d",
               in_dtype);
  FP8K_REQUIRE(M <= 0x7fffffffLL, "token_quant: too many rows");
  if (M == 0 || K == 0) return FP8K_OK;
  FP8K_REQUIRE(x && q && s, "token_quant: null pointer");
  FP8K_REQUIRE(aligned(x, 16) && aligned(q, 8), "token_quant: x must be 16-byte, q 8-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)M), block(256);
  switch (in_dtype) {
    case FP8K_BF16: hipLaunchKernelGGL(token_quant_kernel<FP8K_BF16>, grid, block, 0, st, x, (uint8_t*)q, s, K); break;
    case FP8K_F16: hipLaunchKernelGGL(token_quant_kernel<FP8K_F16>, grid, block, 0, st, x, (uint8_t*)q, s, K); break;
    default: hipLaunchKernelGGL(token_quant_kernel<FP8K_F32>, grid, block, 0, st, x, (uint8_t*)q, s, K); break;
  }
  return check_launch("token_quant");
}

extern "C" int fp8k_tensor_quant(const void* x, void* q, float* s, int64_t numel, int in_dtype, int is_static,
                                 void* stream) {
  clear_error();
  FP8K_REQUIRE(numel >= 0, "tensor_quant: negative size");
  FP8K_REQUIRE(in_dtype == FP8K_F32 || in_dtype == FP8K_F16 || in_dtype == FP8K_BF16, "tensor_quant: bad input dtype %d",
               in_dtype);
  if (numel == 0) return FP8K_OK;
  FP8K_REQUIRE(x && q && s, "tensor_quant: null pointer");
  FP8K_REQUIRE(aligned(x, 16) && aligned(q, 8), "tensor_quant: x must be 16-byte, q 8-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const int64_t want = (numel / 8 + 255) / 256;
  dim3 grid((unsigned)(want < 1 ? 1 : (want > 2048 ? 2048 : want))), block(256);
#define FP8K_TQ(DT)                                                                                     \
  do {                                                                                                  \
    if (!is_static) hipLaunchKernelGGL(tensor_absmax_kernel<DT>, grid, block, 0, st, x, s, numel);      \
    hipLaunchKernelGGL(tensor_quant_kernel<DT>, grid, block, 0, st, x, (uint8_t*)q, (const float*)s, numel); \
  } while (0)
  switch (in_dtype) {
    case FP8K_BF16: FP8K_TQ(FP8K_BF16); break;
    case FP8K_F16: FP8K_TQ(FP8K_F16); break;
    default: FP8K_TQ(FP8K_F32); break;
  }
#undef FP8K_TQ
  return check_launch("tensor_quant");
}

extern "C" int fp8k_tensor_quant_mla(const void* x, void* q, float* s, int64_t H, int64_t S, int64_t D, int64_t x_stride_h,
                                     int64_t x_stride_s, float eps, int in_dtype, void* stream) {
  clear_error();
  const char* op = "per_tensor_quant_mla_fp8";
  FP8K_REQUIRE(H >= 0 && S >= 0 && D >= 0, "%s: negative shape", op);
  FP8K_REQUIRE(in_dtype == FP8K_F32 || in_dtype == FP8K_F16 || in_dtype == FP8K_BF16, "%s: bad input dtype %d", op, in_dtype);
  FP8K_REQUIRE(S <= 0x7fffffffLL && D <= 0x7fffffffLL, "%s: shape too large", op);
  if (H * S * D == 0) return FP8K_OK;
  const int64_t esz = in_dtype == FP8K_F32 ? 4 : 2;
  FP8K_REQUIRE(x && q && s, "%s: null pointer", op);
  FP8K_REQUIRE(D % 8 == 0, "%s: the last dimension (%lld) must be divisible by 8", op, (long long)D);
  FP8K_REQUIRE(x_stride_h >= 0 && x_stride_s >= 0 && (x_stride_h * esz) % 16 == 0 && (x_stride_s * esz) % 16 == 0 && aligned(x, 16) &&
               aligned(q, 8), "%s: rows of x must be 16-byte aligned, q 8-byte aligned", op);
  hipStream_t st = (hipStream_t)stream;
  const int64_t rows = H * S;
  const int64_t want = (rows * (D / 8) + 255) / 256;
  dim3 grid((unsigned)(want < 1 ? 1 : (want > 2048 ? 2048 : want))), block(256);
#define FP8K_MLAQ(DT)                                                                                                    \
  do {                                                                                                                   \
    hipLaunchKernelGGL((rows_tensor_quant_kernel<DT, false>), grid, block, 0, st, x, (uint8_t*)q, s, rows, (int)S, (int)D, \
                       x_stride_h, x_stride_s, eps);                                                                     \
    hipLaunchKernelGGL((rows_tensor_quant_kernel<DT, true>), grid, block, 0, st, x, (uint8_t*)q, s, rows, (int)S, (int)D,  \
                       x_stride_h, x_stride_s, eps);                                                                     \
  } while (0)
  switch (in_dtype) {
    case FP8K_BF16: FP8K_MLAQ(FP8K_BF16); break;
    case FP8K_F16: FP8K_MLAQ(FP8K_F16); break;
    default: FP8K_MLAQ(FP8K_F32); break;
  }
#undef FP8K_MLAQ
  return check_launch(op);
}
