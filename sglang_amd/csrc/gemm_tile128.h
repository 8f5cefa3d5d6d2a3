// 128(n) x 128(m) x 128(k) tile kernel for the shapes between the weight-streaming kernels and the 256x256
// tile kernel: a few hundred activation rows, or outputs with fewer 256x256 tiles than the chip has CUs.
//
// 8 wavefronts, 2 along n x 4 along m, wave tile 64(n) x 32(m) = 2 MFMA tiles of 32x32.  LDS: four stages of
// [W 128 rows x 128 B | X 128 rows x 128 B | 2 KB of scales] = 34 KB each, so three K blocks (96 KB) are in
// flight per CU: these shapes read every weight line from HBM exactly once, and it is bytes in flight that
// cover that latency.  The operands take the same road as in gemm_tile256_kernel (buffer_load ... lds with the
// complete offset in the range-checked per-lane operand, 16-byte chunk c of row r at chunk position
// c ^ ((r >> 1) & 7)).
//
// The block scales travel with the operands: one more 4-byte-per-lane load into LDS per wave and K block (waves
// 0 and 1 fetch the 128 activation-row scales of the block, the others the weight scale), so that one partial
// vmcnt wait covers everything a block needs.
//
// One barrier per K block.  After the barrier of block `it` a wave issues the four MFMAs of block it-1 from one
// of two register sets, and between them (a) refills the stage of block it-1 with block it+3 and (b) fetches its
// operands of block `it` from LDS into the other set: all eight waves pass the barrier together, and with the
// LDS reads up front the LDS pipe and the matrix core would take turns instead of overlapping.  The loop body
// is branch-free: loads past the last K block are out of range or unread.
//
// SPLIT: the K range is cut into p.splits runs, every (tile, run) pair is one workgroup, float partials go to
// the workspace [split][M][N] for splitk_reduce_kernel.
#pragma once

#include "gemm_kernels.h"

namespace fp8k {

constexpr int kT128 = 128;
constexpr int kT128Stages = 4;
constexpr int kT128XOff = kT128 * kTileK;            // 16 KB of W rows, then 16 KB of X rows ...
constexpr int kT128SOff = 2 * kT128 * kTileK;        // ... then 8 x 256 B: [128 activation scales | weight scale copies]
constexpr int kT128Stage = kT128SOff + 2048;         // 34 KB

template <int MODE, int OUT_DT, int BIAS_DT, bool SPLIT>
__global__ __launch_bounds__(512, 1) void gemm_tile128_kernel(const GemmArgs p) {
  __shared__ __attribute__((aligned(1024))) uint8_t smem[kT128Stages * kT128Stage];
  constexpr int NST = kT128Stages;
  constexpr int kLoadsPerBlock = MODE == kModeRow ? 4 : 5;   // vector-memory operations a wave issues per K block

  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int wn = w & 1, wm = w >> 1;

  // workgroup -> (tile, K run): each XCD (workgroup id mod 8) walks a contiguous run of the work list
  int t, split;
  {
    const int ntiles = p.tiles_m * p.tiles_n;
    const int total = ntiles * p.splits;
    const int per_xcd = (total + 7) >> 3;
    const int idx = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
    if (idx >= total) return;
    split = idx / ntiles;
    t = idx - split * ntiles;
  }
  int tile_m, tile_n;
  tile_coords(t, p.tiles_m, p.tiles_n, tile_m, tile_n);
  const int m0 = tile_m * kT128, n0 = tile_n * kT128;

  const int kb_begin = SPLIT ? split * p.kb_per_split : 0;
  const int kb_end = SPLIT ? min(p.K / kTileK, kb_begin + p.kb_per_split) : p.K / kTileK;
  const int nkb = kb_end - kb_begin;
  if (nkb <= 0) return;

  // ---- global -> LDS: wave w brings rows [16w, 16w+16) of both tiles, two 1 KB loads (8 rows) each
  const int rowsW = min(kT128, p.N - n0), rowsX = min(kT128, p.M - m0);
  const int kbytes = p.K - kb_begin * kTileK;
  // batched launches (grid y): every batch entry has its own operands and output, the scales are shared
  const uint8_t* const Wb = p.W + (int64_t)blockIdx.y * p.batch_w;
  const uint8_t* const Xb = p.X + (int64_t)blockIdx.y * p.batch_x;
  u16* const Cb = (u16*)p.C + (int64_t)blockIdx.y * p.batch_c;
  const rsrc_t rW = make_rsrc(Wb + (int64_t)n0 * p.ldw + (int64_t)kb_begin * kTileK, (uint32_t)((rowsW - 1) * p.ldw + kbytes));
  const rsrc_t rX = make_rsrc(Xb + (int64_t)m0 * p.ldx + (int64_t)kb_begin * kTileK, (uint32_t)((rowsX - 1) * p.ldx + kbytes));
  const int rl = lane >> 3, cp = lane & 7;
  uint32_t voW[2], voX[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int c = cp ^ ((j << 2) + (rl >> 1));   // row 16w + 8j + rl: swizzle key (row >> 1) & 7
    voW[j] = (uint32_t)((w * 16 + j * 8 + rl) * p.ldw + c * 16);
    voX[j] = (uint32_t)((w * 16 + j * 8 + rl) * p.ldx + c * 16);
  }
  auto L = [&](int stage, int kstep, int idx) {  // idx 0, 1: W slices; 2, 3: X slices
    uint8_t* base = smem + stage * kT128Stage + w * 2048;
    const uint32_t ko = (uint32_t)kstep * kTileK;
    const int j = idx & 1;
    if (idx < 2) buf_load16_to_lds(rW, voW[j] + ko, 0, base + j * 1024);
    else buf_load16_to_lds(rX, voX[j] + ko, 0, base + kT128XOff + j * 1024);
  };
  // scale element this lane fetches for a K block (waves 0, 1: activation row 64w + lane; the others: the weight
  // scale of the tile's 128-row block), as pointer at K block kb_begin plus a stride per block
  const float* sptr;
  int64_t sstep;
  {
    const int mrow = min(m0 + (w & 1) * 64 + lane, p.M - 1);
    const int nb = min(n0, p.N - 1) >> 7;
    if (MODE == kModeScaled) {  // int32 words of four UE8M0 bytes (K blocks 4j..4j+3 of a row), sx_k = word stride
      sptr = w < 2 ? p.sx + (int64_t)mrow * p.sx_m : p.sw + (int64_t)nb * p.sw_n + (int64_t)kb_begin * p.sw_k;
    } else {
      sptr = w < 2 ? p.sx + (int64_t)mrow * p.sx_m + (int64_t)kb_begin * p.sx_k
                   : p.sw + (int64_t)nb * p.sw_n + (int64_t)kb_begin * p.sw_k;
    }
    sstep = w < 2 ? p.sx_k : p.sw_k;
  }
  auto LS = [&](int stage, int kstep) {
    if (MODE == kModeRow) return;
    const int kn = min(kstep, nkb - 1);  // stay inside the scale arrays past the last block
    const float* src = sptr + (MODE == kModeScaled && w < 2 ? (int64_t)((kb_begin + kn) >> 2) * sstep : (int64_t)kn * sstep);
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                     (lds_ptr_t)(smem + stage * kT128Stage + kT128SOff + w * 256), 4, 0, 0);
  };

  // ---- LDS -> MFMA operands
  const int lr = lane & 31, h = lane >> 5;
  const int swz = (lr >> 1) & 7;
  uint32_t co[2][2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int j = 0; j < 2; ++j) co[ks][j] = (uint32_t)(((ks * 4 + h * 2 + j) ^ swz) << 4);
  const uint32_t rdW = (uint32_t)((wn * 64 + lr) * kTileK);
  const uint32_t rdX = (uint32_t)(kT128XOff + (wm * 32 + lr) * kTileK);
  const uint32_t rdS = (uint32_t)(kT128SOff + (wm * 32 + lr) * 4);
  auto frag = [&](const uint8_t* st, uint32_t rowoff, int ks) -> v8i {
    const v4i lo = *reinterpret_cast<const v4i*>(st + rowoff + co[ks][0]);
    const v4i hi = *reinterpret_cast<const v4i*>(st + rowoff + co[ks][1]);
    v8i r;
    r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
    r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
    return r;
  };

  v16f acc[2];
#pragma unroll
  for (int ns = 0; ns < 2; ++ns)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[ns][r] = 0.f;

  // operands and scale of one K block, in registers
  struct Operands { v8i W0[2], W1[2], X[2]; uint32_t sx, sw; };  // sx, sw: raw scale words as they lie in LDS
  Operands oa, ob;
  v16f tb_pend;       // block mode: second tile's product of the block before, not yet added to acc[1]
  float sc_pend = 0.f;
#pragma unroll
  for (int r = 0; r < 16; ++r) tb_pend[r] = 0.f;

  // the four MFMAs of K block `it` from registers; `between(i)` is issued after MFMA i (the LDS reads and global
  // loads of the trip go there, so that they run in the shadow of the matrix core instead of before it)
  auto compute = [&](const Operands& o, int it, auto&& between) {
    if (MODE == kModeBlock) {
      const float sc = __uint_as_float(o.sx) * __uint_as_float(o.sw);
      v16f z, ta, tb;
#pragma unroll
      for (int r = 0; r < 16; ++r) z[r] = 0.f;
      ta = mfma_32x32x64(o.W0[0], o.X[0], z);
      between(0);
#pragma unroll
      for (int r = 0; r < 8; ++r) acc[1][r] = __builtin_fmaf(tb_pend[r], sc_pend, acc[1][r]);
      SB();
      tb = mfma_32x32x64(o.W1[0], o.X[0], z);
      between(1);
#pragma unroll
      for (int r = 8; r < 16; ++r) acc[1][r] = __builtin_fmaf(tb_pend[r], sc_pend, acc[1][r]);
      SB();
      ta = mfma_32x32x64(o.W0[1], o.X[1], ta);
      between(2);
      SB();
      tb = mfma_32x32x64(o.W1[1], o.X[1], tb);
      between(3);
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[0][r] = __builtin_fmaf(ta[r], sc, acc[0][r]);
      tb_pend = tb;
      sc_pend = sc;
    } else {
      int sq = 127, sqw = 127;
      if (MODE == kModeScaled) { sq = (int)(o.sx >> (((kb_begin + it) & 3) * 8)); sqw = (int)(o.sw >> 23); }
      auto MM = [&](const v8i& a, const v8i& b, v16f c) -> v16f {
        if (MODE == kModeScaled) return mfma_32x32x64_scaled(a, b, c, sqw, sq);
        return mfma_32x32x64(a, b, c);
      };
      acc[0] = MM(o.W0[0], o.X[0], acc[0]);
      between(0); SB();
      acc[1] = MM(o.W1[0], o.X[0], acc[1]);
      between(1); SB();
      acc[0] = MM(o.W0[1], o.X[1], acc[0]);
      between(2); SB();
      acc[1] = MM(o.W1[1], o.X[1], acc[1]);
      between(3);
    }
  };
  // trip `it`: barrier of block `it`; refill of the stage that block it-1 has left with block it+3; operands of
  // block `it` from LDS into `rd`; MFMAs of block it-1 from `use`
  auto trip = [&](int it, Operands& rd, const Operands& use) {
    const int kf = it + NST - 1;
    const int fill = kf & (NST - 1);
    const uint8_t* st = smem + (it & (NST - 1)) * kT128Stage;
    SB();  // the MFMAs issued before stay in front of this wait: they are what hides the loads' latency
    lds_barrier<(NST - 2) * kLoadsPerBlock>();
    compute(use, it - 1, [&](int i) {
      // all LDS reads in the first three gaps, so that they have returned when the wave reaches the next barrier
      if (i == 0) {
        rd.W0[0] = frag(st, rdW, 0); rd.X[0] = frag(st, rdX, 0);
        rd.sx = 0; rd.sw = 0;
        if (MODE != kModeRow) {  // combined a trip later: nothing here waits for these reads
          rd.sx = *reinterpret_cast<const uint32_t*>(st + rdS);
          rd.sw = *reinterpret_cast<const uint32_t*>(st + kT128SOff + 512);
        }
        L(fill, kf, 0);
      } else if (i == 1) {
        rd.W1[0] = frag(st, rdW + 32 * kTileK, 0); rd.W0[1] = frag(st, rdW, 1);
        L(fill, kf, 1); L(fill, kf, 2);
      } else if (i == 2) {
        rd.X[1] = frag(st, rdX, 1); rd.W1[1] = frag(st, rdW + 32 * kTileK, 1);
        L(fill, kf, 3);
      } else {
        LS(fill, kf);
      }
    });
  };

  // ---- prologue: blocks 0 .. 2 into stages 0 .. 2, block 0's operands into `oa`
#pragma unroll
  for (int s = 0; s < NST - 1; ++s) {
    L(s, s, 0); L(s, s, 1); L(s, s, 2); L(s, s, 3);
    LS(s, s);
  }
  {
    SB();
    lds_barrier<(NST - 2) * kLoadsPerBlock>();
    L(NST - 1, NST - 1, 0); L(NST - 1, NST - 1, 1); L(NST - 1, NST - 1, 2); L(NST - 1, NST - 1, 3);
    LS(NST - 1, NST - 1);
    oa.W0[0] = frag(smem, rdW, 0); oa.X[0] = frag(smem, rdX, 0);
    oa.W0[1] = frag(smem, rdW, 1); oa.X[1] = frag(smem, rdX, 1);
    oa.W1[0] = frag(smem, rdW + 32 * kTileK, 0); oa.W1[1] = frag(smem, rdW + 32 * kTileK, 1);
    oa.sx = 0; oa.sw = 0;
    if (MODE != kModeRow) {
      oa.sx = *reinterpret_cast<const uint32_t*>(smem + rdS);
      oa.sw = *reinterpret_cast<const uint32_t*>(smem + kT128SOff + 512);
    }
  }
  // ---- block b is fetched in trip b and multiplied in trip b+1; even blocks live in `oa`, odd ones in `ob`
  auto nothing = [](int) {};
  int it = 1;
  for (; it + 1 < nkb; it += 2) {
    trip(it, ob, oa);
    trip(it + 1, oa, ob);
  }
  if (it < nkb) {
    trip(it, ob, oa);
    compute(ob, it, nothing);
  } else {
    compute(oa, it - 1, nothing);
  }
  if (MODE == kModeBlock) {
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[1][r] = __builtin_fmaf(tb_pend[r], sc_pend, acc[1][r]);
  }

  const int nrows = p.M;
  if (SPLIT) {
    wait_vm0();  // the unread loads past the last block must not land in LDS after the workgroup has gone
    float* part = p.partial + (int64_t)split * p.M * p.N;
    const int m = m0 + wm * 32 + lr;
    if (m < nrows) {
#pragma unroll
      for (int ns = 0; ns < 2; ++ns)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          const int n = n0 + wn * 64 + ns * 32 + rg * 8 + h * 4;
          if (n >= p.N) continue;
          *reinterpret_cast<float4*>(part + (int64_t)m * p.N + n) =
              make_float4(acc[ns][rg * 4], acc[ns][rg * 4 + 1], acc[ns][rg * 4 + 2], acc[ns][rg * 4 + 3]);
        }
    }
    return;
  }

  // scaling of row mode + conversion of one run of 4 n
  auto finish4 = [&](int ns, int rg, int n, float sa) -> uint2 {
    float v[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) v[q] = acc[ns][rg * 4 + q];
    if (MODE == kModeRow) {
      float4 sb = make_float4(0.f, 0.f, 0.f, 0.f);
      if (n < p.N) sb = *reinterpret_cast<const float4*>(p.sw + n);
      v[0] = v[0] * sb.x * sa; v[1] = v[1] * sb.y * sa; v[2] = v[2] * sb.z * sa; v[3] = v[3] * sb.w * sa;
      if (p.bias && n < p.N) {
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] += load_scalar<BIAS_DT>(p.bias, n + q);
      }
    }
    uint2 o;
    if (OUT_DT == FP8K_BF16) {
      o.x = pack_bf16x2(v[0], v[1]);
      o.y = pack_bf16x2(v[2], v[3]);
    } else {
      o.x = f32_to_f16_bits(v[0]) | (f32_to_f16_bits(v[1]) << 16);
      o.y = f32_to_f16_bits(v[2]) | (f32_to_f16_bits(v[3]) << 16);
    }
    return o;
  };

  // Finished tiles leave through LDS so that a store instruction writes whole 128-byte row segments: each wave
  // re-lays its 32(m) x 64(n) block out in a private 4 KB slot, 16-byte chunks XOR-swizzled by the row.
  const int m_own = m0 + wm * 32 + lr;
  float sa = 1.f;
  if (MODE == kModeRow && m_own < nrows) sa = p.sx[m_own];
  const bool wide = (p.ldc & 7) == 0 && (reinterpret_cast<uintptr_t>(Cb) & 15) == 0;
  if (wide) {
    wait_vm0_lgkm0();                // own stray loads have landed ...
    __builtin_amdgcn_s_barrier();    // ... and so have everyone's; every wave has taken its last operands
    asm volatile("" ::: "memory");
    uint8_t* ep = smem + w * 4096;
#pragma unroll
    for (int ns = 0; ns < 2; ++ns)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const int n = n0 + wn * 64 + ns * 32 + rg * 8 + h * 4;
        const uint2 o = finish4(ns, rg, n, sa);
        const int chunk = (ns * 4 + rg) ^ (lr & 7);
        *reinterpret_cast<uint2*>(ep + lr * 128 + chunk * 16 + h * 8) = o;
      }
    __builtin_amdgcn_wave_barrier();  // one wave's LDS accesses complete in order
    const int rr = lane >> 3, pc = lane & 7;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = i * 8 + rr;
      const uint4 o = *reinterpret_cast<const uint4*>(ep + r * 128 + ((pc ^ (r & 7)) << 4));
      const int m = m0 + wm * 32 + r;
      const int n = n0 + wn * 64 + (pc << 3);
      if (m < nrows && n < p.N) *reinterpret_cast<uint4*>(Cb + (int64_t)m * p.ldc + n) = o;
    }
    return;
  }

  wait_vm0();
  if (m_own >= nrows) return;
#pragma unroll
  for (int ns = 0; ns < 2; ++ns)
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      const int n = n0 + wn * 64 + ns * 32 + rg * 8 + h * 4;
      if (n >= p.N) continue;
      const uint2 o = finish4(ns, rg, n, sa);
      *reinterpret_cast<uint2*>(Cb + (int64_t)m_own * p.ldc + n) = o;
    }
}

}  // namespace fp8k
