// Weight-streaming FP8 GEMM for at most 32 activation rows per block (decode and small-batch MoE), gfx950.
//
// With so few activation rows the GEMM is an HBM stream of the weight matrix (2*TM FLOP per weight byte, far under
// the chip's ridge), so everything is arranged around the weight loads.  A wavefront owns 16 weight rows and keeps
// eight K blocks (16 KB) of them in flight in registers: two non-temporal 16-byte loads per lane and K block, each
// instruction covering 8 whole 128-byte lines (lane l: row l/8, 16-byte chunk l%8) - whole-line requests measured
// 25 % more HBM bandwidth here than the half-line requests that loading straight into the matrix-core operand
// layout would make.  The move into that layout (operand "A" of v_mfma_f32_16x16x128_f8f6f4: lane l holds 32 bytes
// of row l%16) is a round trip through a 2 KB LDS slot private to the wave: LDS operations of one wave execute in
// order, so it needs no barrier and no wait beyond the register dependency.  The matrix core only sums over K, so
// the K order inside a 128-byte block is free as long as both operands agree: lane (row, q = l/16) takes chunks
// q and 4+q of the block.
//
// The activation rows (shared by the 8 waves = 128 weight rows of a workgroup) are staged through LDS in chunks
// of 8 K blocks: registers -> ds_write one chunk ahead, one barrier per chunk (an LDS-only barrier: the weight
// loads stay in flight across it), rows padded by 16 bytes so the 16 rows of an operand fetch fall into different
// banks.  In block mode the chunk also carries as[m,kb]*bs[nb,kb] (a workgroup spans exactly one 128-row weight
// scale block), zero past the K range, so the K tail needs no branch.  (Every wave re-reads all activation rows
// of the block from LDS, which is why blocks of 64 and 128 rows measured slower here than through
// gemm_stream_kernel.)
#pragma once

#include "gemm_kernels.h"

namespace fp8k {

constexpr int kDirTileN = 128;                   // 8 waves x 16 weight rows
constexpr int kDirDepth = 8;                     // weight prefetch depth in K blocks = K blocks per activation chunk
constexpr uint32_t kOutOfRange = 0xF0000000u;    // buffer offset past every descriptor range: reads zero

__device__ __forceinline__ v4f mfma_16x16x128(v8i a, v8i b, v4f c) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}
__device__ __forceinline__ v4i buf_load16(rsrc_t r, uint32_t voff) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0);
}
__device__ __forceinline__ v4i buf_load16_stream(rsrc_t r, uint32_t voff) {  // non-temporal: used once
  return __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 2);
}
__device__ __forceinline__ v8i join(v4i lo, v4i hi) {
  v8i r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

template <int TM, int MODE, int OUT_DT, int BIAS_DT, bool SPLIT, bool MOE>
__global__ __launch_bounds__(512, 2) void gemm_direct_kernel(const GemmArgs p) {
  static_assert(TM == 16 || TM == 32, "gemm_direct_kernel: 16 or 32 rows per block (more rows are LDS-read bound here)");
  constexpr int MS = TM / 16;                 // 16-row activation sub-tiles
  constexpr int KC = kDirDepth;               // K blocks per activation chunk
  constexpr int DEPTH = kDirDepth;
  constexpr int U = DEPTH / KC;               // chunks per trip of the unrolled loop
  constexpr int RB = KC * kTileK;             // bytes of one activation row in a chunk
  constexpr int XROW = RB + 16;               // LDS row stride
  constexpr int LPR = RB / 16;                // lanes per staged row
  constexpr int RPI = 64 / LPR;               // rows per staging load
  constexpr int XI = TM / 8 / RPI;            // staging loads per wave per chunk
  static_assert(TM * KC <= 512, "one scale product per lane and chunk");
  __shared__ __attribute__((aligned(16))) uint8_t xs[2][TM * XROW];
  __shared__ float scs[2][KC][TM];
  __shared__ __attribute__((aligned(16))) uint8_t wl[8][16 * kTileK];  // per wave: one K block of its 16 weight rows

  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int r = lane & 15, kq = lane >> 4;

  // ---- work item (same walk as gemm_stream_kernel)
  int bid = blockIdx.x;
  int split = 0;
  int mb, tile_n;
  if (MOE) {
    const int used = p.num_post_pad[0] / p.block_m;
    const int per_xcd = (used + 7) >> 3;
    const int j = bid >> 3;
    const int mbl = j / p.tiles_n;
    if (mbl >= per_xcd) return;
    mb = (bid & 7) * per_xcd + mbl;
    if (mb >= used || mb >= p.m_blocks) return;
    tile_n = j - mbl * p.tiles_n;
  } else {
    if (SPLIT) { split = bid % p.splits; bid /= p.splits; }
    if (bid >= p.tiles_n * p.m_blocks) return;
    mb = bid % p.m_blocks;
    tile_n = bid / p.m_blocks;
  }
  const int block_m = MOE ? p.block_m : TM;
  const int slot0 = mb * block_m;
  const int expert = MOE ? p.expert_ids[mb] : 0;
  const int nrows = MOE ? p.num_valid : p.M;
  const int n0 = tile_n * kDirTileN;
  const int n0w = n0 + w * 16;

  const int kb_begin = SPLIT ? split * p.kb_per_split : 0;
  const int kb_end = SPLIT ? min(p.K / kTileK, kb_begin + p.kb_per_split) : p.K / kTileK;
  // an expert that lives on another rank contributes zeros: run no K block, the epilogue stores them
  const int nkb = (MOE && expert < 0) ? 0 : max(kb_end - kb_begin, 0);
  const int nch = (nkb + KC - 1) / KC;
  const uint32_t kbytes = (uint32_t)nkb * kTileK;   // bytes of this K range per row

  auto slot_of = [&](int i) -> int {   // row slot of block row i, or nrows when the row is padding
    if (i >= block_m) return nrows;
    const int s = MOE ? p.sorted_ids[slot0 + i] : slot0 + i;
    return s < nrows ? s : nrows;
  };

  // ---- weights: 16 rows of this wave, straight into MFMA operand registers
  const uint8_t* Wb = p.W + (MOE && expert >= 0 ? (int64_t)expert * p.w_expert_stride : 0);
  const int rowsW = min(16, p.N - n0w);
  const rsrc_t rW = make_rsrc(Wb + (int64_t)n0w * p.ldw + (int64_t)kb_begin * kTileK,
                              rowsW > 0 ? (uint32_t)((rowsW - 1) * p.ldw) + kbytes : 0u);
  // load j of a K block: row j*8 + lane/8, chunk lane%8; in LDS chunk c of row i sits at position c ^ ((i>>1)&7),
  // which keeps both the line-shaped writes and the operand-shaped reads free of bank conflicts
  const int wrow = lane >> 3, wc = lane & 7;
  const uint32_t voW0 = (uint32_t)(wrow * p.ldw + wc * 16), voW1 = (uint32_t)((wrow + 8) * p.ldw + wc * 16);
  uint8_t* const wslot = wl[w];
  const uint32_t wst0 = (uint32_t)(wrow * kTileK + ((wc ^ ((wrow >> 1) & 7)) << 4));
  const uint32_t wst1 = (uint32_t)((wrow + 8) * kTileK + ((wc ^ (((wrow + 8) >> 1) & 7)) << 4));
  const uint32_t wrd0 = (uint32_t)(r * kTileK + ((kq ^ ((r >> 1) & 7)) << 4));
  const uint32_t wrd1 = (uint32_t)(r * kTileK + (((4 + kq) ^ ((r >> 1) & 7)) << 4));
  v4i wreg[DEPTH][2];
  auto load_w = [&](int slot, int kb) {
    const bool ok = kb < nkb;
    wreg[slot][0] = buf_load16_stream(rW, ok ? voW0 + (uint32_t)kb * kTileK : kOutOfRange);
    wreg[slot][1] = buf_load16_stream(rW, ok ? voW1 + (uint32_t)kb * kTileK : kOutOfRange);
  };
  auto weight_operand = [&](int slot) -> v8i {  // registers (line layout) -> LDS -> registers (operand layout)
    *reinterpret_cast<v4i*>(wslot + wst0) = wreg[slot][0];
    *reinterpret_cast<v4i*>(wslot + wst1) = wreg[slot][1];
    return join(*reinterpret_cast<const v4i*>(wslot + wrd0), *reinterpret_cast<const v4i*>(wslot + wrd1));
  };

  // ---- activations: wave w stages rows w*TM/8 .. of the block, RB bytes per row and chunk;
  // staging load j of a lane covers row w*TM/8 + j*RPI + lane/LPR, bytes (lane%LPR)*16 ..
  const int64_t xrows = MOE ? (int64_t)((p.num_valid + p.top_k - 1) / p.top_k) : (int64_t)p.M;
  const rsrc_t rX = make_rsrc(p.X + (int64_t)kb_begin * kTileK, (uint32_t)((xrows - 1) * p.ldx) + kbytes);
  const int xcol = (lane % LPR) * 16;
  uint32_t voX[XI];
#pragma unroll
  for (int j = 0; j < XI; ++j) {
    const int s = slot_of(w * (TM / 8) + j * RPI + lane / LPR);
    const int64_t xr = MOE ? s / p.top_k : s;
    voX[j] = s < nrows ? (uint32_t)(xr * p.ldx) + xcol : kOutOfRange;
  }
  v4i xreg[XI];
  // ---- block mode: lane t < TM*KC stages as[m,kb]*bs[nb,kb] of (m = t % TM, kb = chunk*KC + t / TM)
  const int sm = threadIdx.x % TM, skb = threadIdx.x / TM;
  const bool stager = MODE == kModeBlock && (int)threadIdx.x < TM * KC;
  const float* sxp = p.sx;
  const float* swp = p.sw;
  bool srow_ok = false;
  if (stager) {
    const int s = slot_of(sm);
    srow_ok = s < nrows;
    const int64_t xr = srow_ok ? (MOE ? s / p.top_k : s) : 0;
    sxp = p.sx + xr * p.sx_m + (int64_t)kb_begin * p.sx_k;
    swp = p.sw + (MOE && expert >= 0 ? (int64_t)expert * p.sw_expert_stride : 0) +
          (int64_t)(min(n0, p.N - 1) >> 7) * p.sw_n + (int64_t)kb_begin * p.sw_k;
  }
  float sreg_x = 0.f, sreg_w = 0.f;  // multiplied at store time: using them here would wait for every load in flight
  auto stage_load = [&](int c) {
    const uint32_t k0 = (uint32_t)c * RB;
#pragma unroll
    for (int j = 0; j < XI; ++j) {
      const bool ok = voX[j] != kOutOfRange && k0 + xcol < kbytes;
      xreg[j] = buf_load16(rX, ok ? voX[j] + k0 : kOutOfRange);
    }
    if (MODE == kModeBlock) {
      const int kb = c * KC + skb;
      sreg_x = 0.f;
      sreg_w = 0.f;
      if (stager && srow_ok && kb < nkb) {
        sreg_x = sxp[(int64_t)kb * p.sx_k];
        sreg_w = swp[(int64_t)kb * p.sw_k];
      }
    }
  };
  auto stage_store = [&](int buf) {
#pragma unroll
    for (int j = 0; j < XI; ++j)
      *reinterpret_cast<v4i*>(&xs[buf][(w * (TM / 8) + j * RPI + lane / LPR) * XROW + xcol]) = xreg[j];
    if (stager) scs[buf][skb][sm] = sreg_x * sreg_w;
  };

  v4f acc[MS];
#pragma unroll
  for (int ms = 0; ms < MS; ++ms) acc[ms] = v4f{0.f, 0.f, 0.f, 0.f};

  // ---- prologue: chunks 0 and 1 requested, then the weights of K blocks 0..7, then chunk 0 into LDS.  The loop
  // keeps the same age order (staging loads older than the weight loads issued after them), so that the wait
  // for a staged chunk never has to drain the weight prefetch.
  stage_load(0);
  v4i xreg0[XI];
#pragma unroll
  for (int j = 0; j < XI; ++j) xreg0[j] = xreg[j];
  const float s0x = sreg_x, s0w = sreg_w;
  stage_load(1);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) load_w(d, d);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int j = 0; j < XI; ++j)
    *reinterpret_cast<v4i*>(&xs[0][(w * (TM / 8) + j * RPI + lane / LPR) * XROW + xcol]) = xreg0[j];
  if (stager) scs[0][skb][sm] = s0x * s0w;

  const uint32_t xrd = (uint32_t)(r * XROW + kq * 16);
  for (int c0 = 0; c0 < nch; c0 += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + u;         // a chunk past the K range holds zeros and zero scales
      const int buf = c & 1;
      lds_barrier();                // chunk c is visible; every wave is done with chunk c-1 (weight loads stay in flight)
      stage_store(buf ^ 1);         // chunk c+1
      stage_load(c + 2);
      // memory operations retire in order: the staging loads must stay OLDER than this trip's weight loads, or
      // the wait for them at the next barrier would drain the weight prefetch
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kbl = 0; kbl < KC; ++kbl) {
        const int slot = u * KC + kbl;
        const v8i wa = weight_operand(slot);
        load_w(slot, c * KC + kbl + DEPTH);
#pragma unroll
        for (int ms = 0; ms < MS; ++ms) {
          const uint8_t* xp = &xs[buf][ms * 16 * XROW + xrd + kbl * kTileK];
          const v8i xa = join(*reinterpret_cast<const v4i*>(xp), *reinterpret_cast<const v4i*>(xp + 64));
          if (MODE == kModeBlock) {
            const v4f t = mfma_16x16x128(wa, xa, v4f{0.f, 0.f, 0.f, 0.f});
            const float sc = scs[buf][kbl][ms * 16 + r];
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[ms][i] = __builtin_fmaf(t[i], sc, acc[ms][i]);
          } else {
            acc[ms] = mfma_16x16x128(wa, xa, acc[ms]);
          }
        }
      }
    }
  }
  // ---- epilogue: lane holds n = n0w + kq*4 .. +3 of activation row ms*16 + r
  const int n = n0w + kq * 4;
  if (n >= p.N) return;
#pragma unroll
  for (int ms = 0; ms < MS; ++ms) {
    const int s = slot_of(ms * 16 + r);
    if (s >= nrows) continue;
    const int64_t orow = s;
    float v[4] = {acc[ms][0], acc[ms][1], acc[ms][2], acc[ms][3]};
    if (SPLIT) {
      *reinterpret_cast<float4*>(p.partial + ((int64_t)split * p.M + orow) * p.N + n) = make_float4(v[0], v[1], v[2], v[3]);
      continue;
    }
    if (MODE == kModeRow) {
      const float sa = p.sx[orow];
      const float4 sb = *reinterpret_cast<const float4*>(p.sw + n);
      v[0] = v[0] * sb.x * sa; v[1] = v[1] * sb.y * sa; v[2] = v[2] * sb.z * sa; v[3] = v[3] * sb.w * sa;
      if (p.bias) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] += load_scalar<BIAS_DT>(p.bias, n + i);
      }
    } else if (MOE && p.topk_w) {
      const float tw = p.topk_w[orow];
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] *= tw;
    }
    store4<OUT_DT>(p.C, orow * p.ldc + n, v[0], v[1], v[2], v[3]);
  }
}

// ------------------------------------------------------------------------------------------------
// The same weight stream for matrices with too few 128-row tiles to fill the chip (N below about 16 K rows): the K
// range is cut across the WAVES of a workgroup instead of across workgroups, so the partial sums meet in LDS and
// neither float partials in memory nor a reduction launch are needed.  A workgroup owns 16 * NW weight rows; its 8
// waves are NW (along n) x KS (along k), NW * KS = 8; wave (nw, ks) streams rows nw*16.. of K blocks
// [ks * kbw, (ks+1) * kbw).  No wave shares an activation K range with another (NW = 1) or only with NW - 1 others,
// so the activations skip LDS: a lane fetches its 32 bytes of a row and K block in matrix-core operand form straight
// from memory (they are L2 hits: every workgroup reads the same few rows).  The K loop has no barrier; each wave keeps
// D K blocks of weights, activations and scales in flight.  At the end the 8 accumulator sets are summed through LDS
// in ascending ks (a fixed order: results do not depend on timing) and the ks = 0 waves write the output.
// ------------------------------------------------------------------------------------------------
template <int TM, int MODE, int OUT_DT, int BIAS_DT>
__global__ __launch_bounds__(512, 2) void gemm_wavek_kernel(const GemmArgs p) {
  static_assert(TM == 16 || TM == 32, "gemm_wavek_kernel: 16 or 32 rows");
  constexpr int MS = TM / 16;
  constexpr int D = 4;  // K blocks in flight per wave
  __shared__ __attribute__((aligned(16))) uint8_t wl[8][16 * kTileK];  // per wave: one K block of its 16 weight rows
  __shared__ __attribute__((aligned(16))) float red[8][MS][64][4];

  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int r = lane & 15, kq = lane >> 4;
  const int NW = p.wk_nw, nw = w % NW, ks = w / NW;
  const int n0w = (blockIdx.x * NW + nw) * 16;
  const int kb_all = p.K / kTileK;
  const int kb0 = ks * p.kb_per_split;
  const int nkb = n0w < p.N ? max(min(kb_all, kb0 + p.kb_per_split) - kb0, 0) : 0;
  const uint32_t kbytes = (uint32_t)nkb * kTileK;

  // ---- weights: line-shaped loads, re-laid out through the wave's LDS slot (as in gemm_direct_kernel)
  const int rowsW = min(16, p.N - n0w);
  const rsrc_t rW = make_rsrc(p.W + (int64_t)n0w * p.ldw + (int64_t)kb0 * kTileK,
                              (rowsW > 0 && nkb > 0) ? (uint32_t)((rowsW - 1) * p.ldw) + kbytes : 0u);
  const int wrow = lane >> 3, wc = lane & 7;
  const uint32_t voW0 = (uint32_t)(wrow * p.ldw + wc * 16), voW1 = (uint32_t)((wrow + 8) * p.ldw + wc * 16);
  uint8_t* const wslot = wl[w];
  const uint32_t wst0 = (uint32_t)(wrow * kTileK + ((wc ^ ((wrow >> 1) & 7)) << 4));
  const uint32_t wst1 = (uint32_t)((wrow + 8) * kTileK + ((wc ^ (((wrow + 8) >> 1) & 7)) << 4));
  const uint32_t wrd0 = (uint32_t)(r * kTileK + ((kq ^ ((r >> 1) & 7)) << 4));
  const uint32_t wrd1 = (uint32_t)(r * kTileK + (((4 + kq) ^ ((r >> 1) & 7)) << 4));
  // ---- activations: lane (r, kq) takes chunks kq and 4 + kq of row ms*16 + r, the K order the weight operand has
  const rsrc_t rX = make_rsrc(p.X + (int64_t)kb0 * kTileK, nkb > 0 ? (uint32_t)((p.M - 1) * p.ldx) + kbytes : 0u);
  uint32_t voX[MS];
#pragma unroll
  for (int ms = 0; ms < MS; ++ms) {
    const int m = ms * 16 + r;
    voX[ms] = m < p.M ? (uint32_t)(m * p.ldx) + kq * 16 : kOutOfRange;
  }
  // ---- block scales: one activation scale per lane row and K block, one weight scale per K block
  const float* sxp[MS];
  const float* swp = p.sw;
  if (MODE == kModeBlock) {
#pragma unroll
    for (int ms = 0; ms < MS; ++ms) sxp[ms] = p.sx + (int64_t)min(ms * 16 + r, p.M - 1) * p.sx_m + (int64_t)kb0 * p.sx_k;
    swp = p.sw + (int64_t)(min(n0w, p.N - 1) >> 7) * p.sw_n + (int64_t)kb0 * p.sw_k;
  }

  v4i wreg[D][2], xreg[D][MS][2];
  float sxr[D][MS], swr[D];
  auto issue = [&](int slot, int kb) {
    const bool ok = kb < nkb;
    const uint32_t ko = (uint32_t)kb * kTileK;
    wreg[slot][0] = buf_load16_stream(rW, ok ? voW0 + ko : kOutOfRange);
    wreg[slot][1] = buf_load16_stream(rW, ok ? voW1 + ko : kOutOfRange);
#pragma unroll
    for (int ms = 0; ms < MS; ++ms) {
      const bool okx = ok && voX[ms] != kOutOfRange;
      xreg[slot][ms][0] = buf_load16(rX, okx ? voX[ms] + ko : kOutOfRange);
      xreg[slot][ms][1] = buf_load16(rX, okx ? voX[ms] + ko + 64 : kOutOfRange);
    }
    if (MODE == kModeBlock) {
      const int kc = min(kb, max(nkb - 1, 0));  // past the range the products are zero: any finite scale will do
#pragma unroll
      for (int ms = 0; ms < MS; ++ms) sxr[slot][ms] = sxp[ms][(int64_t)kc * p.sx_k];
      swr[slot] = swp[(int64_t)kc * p.sw_k];
    }
  };

  v4f acc[MS];
#pragma unroll
  for (int ms = 0; ms < MS; ++ms) acc[ms] = v4f{0.f, 0.f, 0.f, 0.f};

  if (nkb > 0) {
#pragma unroll
    for (int d = 0; d < D; ++d) issue(d, d);
    for (int k0 = 0; k0 < nkb; k0 += D) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        *reinterpret_cast<v4i*>(wslot + wst0) = wreg[d][0];
        *reinterpret_cast<v4i*>(wslot + wst1) = wreg[d][1];
        const v8i wa = join(*reinterpret_cast<const v4i*>(wslot + wrd0), *reinterpret_cast<const v4i*>(wslot + wrd1));
        v8i xa[MS];
        float sc[MS];
#pragma unroll
        for (int ms = 0; ms < MS; ++ms) {
          xa[ms] = join(xreg[d][ms][0], xreg[d][ms][1]);
          if (MODE == kModeBlock) sc[ms] = sxr[d][ms] * swr[d];
        }
        issue(d, k0 + d + D);
#pragma unroll
        for (int ms = 0; ms < MS; ++ms) {
          if (MODE == kModeBlock) {
            const v4f t = mfma_16x16x128(wa, xa[ms], v4f{0.f, 0.f, 0.f, 0.f});
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[ms][i] = __builtin_fmaf(t[i], sc[ms], acc[ms][i]);
          } else {
            acc[ms] = mfma_16x16x128(wa, xa[ms], acc[ms]);
          }
        }
      }
    }
  }
  // ---- the K ranges meet: every wave leaves its sums in LDS, the ks = 0 waves add them up in ascending ks
#pragma unroll
  for (int ms = 0; ms < MS; ++ms) *reinterpret_cast<v4f*>(red[w][ms][lane]) = acc[ms];
  __syncthreads();
  if (ks != 0) return;
  const int KS = 8 / NW;
  const int n = n0w + kq * 4;
  if (n >= p.N) return;
#pragma unroll
  for (int ms = 0; ms < MS; ++ms) {
    const int m = ms * 16 + r;
    if (m >= p.M) continue;
    v4f s = acc[ms];
    for (int k = 1; k < KS; ++k) {
      const v4f o = *reinterpret_cast<const v4f*>(red[k * NW + nw][ms][lane]);
      s[0] += o[0]; s[1] += o[1]; s[2] += o[2]; s[3] += o[3];
    }
    float v[4] = {s[0], s[1], s[2], s[3]};
    if (MODE == kModeRow) {
      const float sa = p.sx[m];
      const float4 sb = *reinterpret_cast<const float4*>(p.sw + n);
      v[0] = v[0] * sb.x * sa; v[1] = v[1] * sb.y * sa; v[2] = v[2] * sb.z * sa; v[3] = v[3] * sb.w * sa;
      if (p.bias) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] += load_scalar<BIAS_DT>(p.bias, n + i);
      }
    }
    store4<OUT_DT>(p.C, (int64_t)m * p.ldc + n, v[0], v[1], v[2], v[3]);
  }
}


}  // namespace fp8k
