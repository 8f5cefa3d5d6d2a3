// Grouped (MoE) block-FP8 GEMM for experts with about a hundred and more token slots: 256(n) x 256(m) x 128(k) tile,
// 8 wavefronts, weights streamed three K blocks deep.
//
// With a few hundred token slots per expert the grouped GEMM is bound by streaming each expert's weights
// from HBM exactly once.  Two 128-row blocks of one expert in two workgroups fetch the weight tile twice
// (they drift apart by more than an L2's worth of traffic), and the 256x256 MFMA tile kernel keeps only one
// K block of prefetch in flight, which is enough against L2 but not against HBM latency.  This kernel keeps
// the streaming kernel's depth on the weights and pairs both 128-row halves on one weight stage:
//   LDS = 3 weight stages (32 KB each) + 2 activation stages (32 KB each) = 160 KB, the whole CU.
//   Activation tiles are re-read by every n tile of the block and come from L2; one stage ahead is enough.
//   Waves: 4 along n (64 weight rows) x 2 along m; the 32-slot groups of a block alternate between the two wave rows
//   (groups wm, wm + 2, wm + 4, wm + 6), so that a block that is half padding still loads both rows of waves evenly;
//   2 x 4 MFMA tiles of 32x32 each (24 KB of LDS operands per 16 MFMAs); groups without real slots skip their MFMAs.
//   A workgroup can walk several items: the two stage rings run on across items, the last two trips of an item
//   request the first two weight blocks of the next one, and the item is written out through the stages its last
//   block used while the next item's first blocks travel.
// Load order inside a K block is scales, activations, weights, so that at the next barrier only the four
// youngest weight loads of each wave may still be in flight (memory operations retire in order).
#pragma once

#include <type_traits>

#include "gemm_kernels.h"
#include "quant_math.h"

namespace fp8k {

// PAIRS: the activation scales are row-major (stride 1 between K blocks, even stride between rows, base aligned to
// 8 bytes; the host checks), and a lane fetches two K blocks per load.  SORTED: one scale row per position of
// sorted_token_ids (what the layer passes): the rows of a wave's four 32-slot groups are a uniform step apart, so one
// offset register serves them.
// FUSE (GEMM 1 of the layer, sorted scales only): the tile's 256 weight rows are 128 gate rows and the 128 up rows of
// the same activation columns (rows n0 .. n0+127 and I + n0 .. I + n0+127 of the [2 I, K] weight, I = N / 2), and the
// write-out produces what silu_and_mul followed by the group quantisation would have made of the 16-bit GEMM result,
// bit for bit: q_out[slot, n0 .. n0+127] and one scale per slot in the sorted order GEMM 2 reads.  The [slots, 2 I]
// intermediate is never written.
// SCALED (sorted scales only): both scale tensors hold powers of two (UE8M0 checkpoints with UE8M0-rounded activation
// scales) and the matrix core applies them itself (v_mfma_scale_f32_32x32x64_f8f6f4 takes the two exponent bytes):
// the products accumulate in place, the float promote and its second accumulator disappear.
template <int OUT_DT, bool PAIRS, bool SORTED, bool FUSE = false, bool SCALED = false>
__global__ __launch_bounds__(512, 1) void moe_stream256_kernel(const GemmArgs p) {
  static_assert(!FUSE || (SORTED && !PAIRS), "the fused write-out is built for sorted activation scales");
  static_assert(!SCALED || (SORTED && !PAIRS && !FUSE), "hardware scaling is built for sorted activation scales");
  constexpr int TM = 256, WST = 3, XST = 2, MS = 4, NS = 2, LW = 4;  // LW: wave loads per tile per stage
  constexpr int WBYTES = kTileN * kTileK, XBYTES = TM * kTileK;
  constexpr int XBASE = WST * WBYTES;
  __shared__ __attribute__((aligned(1024))) uint8_t smem[WST * WBYTES + XST * XBYTES];

  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int wn = w & 3, wm = w >> 2;
  const int nrows = p.num_valid;
  const int nkb = p.K / kTileK;

  // ---- work items.  One workgroup per CU walks the items of its XCD (workgroup ids are dealt round-robin to the
  // XCDs): item index j of XCD x is what workgroup 8 j + x of a one-item-per-workgroup launch would take
  // (moe_work_item(): contiguous run of blocks per XCD, same-expert blocks of a window grouped), and the CUs of an
  // XCD take consecutive j, so the tiles that run together share an expert's activation rows.  Items past the
  // last block are empty, and so are all after them.
  const int xcd = (int)blockIdx.x & 7, jstep = (int)gridDim.x >> 3;
  int j = (int)blockIdx.x >> 3;
  // an expert of another rank: the reference writes zeros; done here on the spot, and the walk goes on
  auto zero_fill = [&](const MoeItem& it) {
    const int ln = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    const int lr = ln & 31, h = ln >> 5;
    for (int ms = 0; ms < MS; ++ms) {
      const int s = p.sorted_ids[it.mb * TM + wm * 128 + ms * 32 + lr];
      if (FUSE) {  // zero bytes and a zero scale: the slot contributes nothing to GEMM 2
        if (wn == 0 && h == 0) p.qs_out[(int64_t)it.tile_n * p.qs_ld + it.mb * TM + wm * 128 + ms * 32 + lr] = 0.f;
        if (s < nrows && h == 0)
          *reinterpret_cast<uint4*>(p.q_out + (int64_t)s * p.ldq + it.tile_n * 128 + wn * 32) = make_uint4(0, 0, 0, 0),
          *reinterpret_cast<uint4*>(p.q_out + (int64_t)s * p.ldq + it.tile_n * 128 + wn * 32 + 16) = make_uint4(0, 0, 0, 0);
        continue;
      }
      if (s >= nrows) continue;
      for (int q = 0; q < 4; ++q) {
        for (int ns = 0; ns < NS; ++ns) {
          const int n = it.tile_n * kTileN + wn * 64 + ns * 32 + h * 16 + q * 4;
          if (n < p.N) store4<OUT_DT>(p.C, (int64_t)s * p.ldc + n, 0.f, 0.f, 0.f, 0.f);
        }
      }
    }
  };
  auto fetch_item = [&](int& jj) -> MoeItem {  // first item at or after jj that has a GEMM to do (or the end)
    for (;;) {
      const MoeItem it = moe_work_item(p, jj * 8 + xcd);
      if (it.mb < 0 || it.expert >= 0) return it;
      zero_fill(it);
      jj += jstep;
    }
  };
  MoeItem item = fetch_item(j);
  if (item.mb < 0) return;

  const int64_t xrows = (int64_t)((p.num_valid + p.top_k - 1) / p.top_k);
  const rsrc_t rX = make_rsrc(p.X, (uint32_t)((xrows - 1) * p.ldx + p.K));
  const rsrc_t rS = make_rsrc(p.sx, (uint32_t)(((xrows - 1) * p.sx_m + nkb) * 4));  // used by the paired loads only
  // through a buffer descriptor: a 32-bit lane offset and a uniform offset, no 64-bit address per lane and group
  const rsrc_t rSall = make_rsrc(p.sx, 0xFFFFFFFFu);

  // ---- global -> LDS: a wave load covers 8 rows (lane: row lane/8, 16-byte chunk lane%8, stored at chunk
  // position c ^ ((row>>1)&7)); whole offsets travel in the bounds-checked per-lane operand
  rsrc_t rW, rWn;  // weights of the item in work / of the item after it
  uint32_t voW[2], voX[LW], w16;
  int slot0 = 0, n0 = 0, expert = 0;
  // The stages are two rings that run on across the items of a walk: block k of an item sits in weight stage
  // (gw0 + k) % 3 and activation stage (gx0 + k) & 1, the next item's block 0 in the stage after its last block.
  int gw0 = 0, gx0 = 0;
  // Whether any of the wave's four activation loads of the item in work covers a real slot (real slots come first in a
  // block).  A load of padding rows moves nothing and still takes its turn in the CU's address unit, so a wave whose rows
  // are all padding runs a copy of the K loop without activation loads; the rows it leaves as they are belong to padding
  // slots, whose products are never stored and reach no other slot's result.
  bool xreal = true;
  // FUSE: the waves that load tile rows 128..255 (w >= 4) take them from the up rows, I - 128 rows further on
  const int half_n = p.N >> 1;
  const uint32_t wsoff = (FUSE && w >= 4) ? (uint32_t)((int64_t)(half_n - 128) * p.ldw) : 0u;
  auto issue_w = [&](const rsrc_t& r, int kblk, int stage) {
    uint8_t* base = smem + stage * WBYTES + w * (LW * 1024);
    const uint32_t ko = (uint32_t)kblk * kTileK;
#pragma unroll
    for (int q = 0; q < LW; ++q) buf_load16_to_lds(r, voW[q & 1] + (ko + (q >> 1) * w16), wsoff, base + q * 1024);
  };
  auto issue_x = [&](int kblk, int stage) {
    uint8_t* base = smem + XBASE + stage * XBYTES + w * (LW * 1024);
    const uint32_t ko = (uint32_t)kblk * kTileK;
#pragma unroll
    for (int q = 0; q < LW; ++q) buf_load16_to_lds(rX, voX[q] + ko, 0, base + q * 1024);
  };
  // the same, one wave load at a time (q = 0 .. LW-1)
  auto issue_w1 = [&](int q, const rsrc_t& r, int kblk, int stage) {
    buf_load16_to_lds(r, voW[q & 1] + ((uint32_t)kblk * kTileK + (q >> 1) * w16), wsoff, smem + stage * WBYTES + w * (LW * 1024) + q * 1024);
  };
  auto issue_x1 = [&](int q, int kblk, int stage) {
    buf_load16_to_lds(rX, voX[q] + (uint32_t)kblk * kTileK, 0, smem + XBASE + stage * XBYTES + w * (LW * 1024) + q * 1024);
  };
  auto weights_of = [&](const MoeItem& it) -> rsrc_t {
    if (it.mb < 0) return make_rsrc(p.W, 0u);  // no item: every load is out of range and moves nothing
    const uint8_t* Wb = p.W + (int64_t)it.expert * p.w_expert_stride;
    if (FUSE) {  // gate rows from n0 on; the range reaches the last up row of the tile
      const int nn = it.tile_n * 128;
      return make_rsrc(Wb + (int64_t)nn * p.ldw, (uint32_t)((int64_t)(half_n + 127) * p.ldw + p.K));
    }
    const int nn = it.tile_n * kTileN;
    const int rowsW = min(kTileN, p.N - nn);
    return make_rsrc(Wb + (int64_t)nn * p.ldw, (uint32_t)((rowsW - 1) * p.ldw + p.K));
  };
  // Entering an item: its activation block 0 goes into its first activation stage (the weights of its blocks 0 and 1
  // were requested in the last two trips of the item before it, or below for a workgroup's first item).  For every
  // item but the first this runs in front of the previous item's write-out, which keeps to the weight and
  // activation stages that item used last - the ones no request in flight points at.  The lane id is taken anew
  // (from the execution mask): lane-derived values that stayed live across the K loops would be parked in scratch
  // and reloaded inside them, and scratch reloads count against the partial vmcnt waits.
  auto start_item = [&](const MoeItem& it, bool first) {
    int ln = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(ln));
    const int rl = ln >> 3, cp = ln & 7;
    slot0 = it.mb * TM;
    n0 = it.tile_n * (FUSE ? 128 : kTileN);
    expert = it.expert;
    // slot table first, weights behind it: loads retire in order, so the table arrives without waiting for the
    // weights, and the weights do not wait for the table
    int sid[LW];
#pragma unroll
    for (int q = 0; q < LW; ++q) sid[q] = p.sorted_ids[slot0 + (w * LW + q) * 8 + rl];
    if (first) {
      // the wave's 8-row groups g = 4w + q: groups q and q + 2 differ by 16 rows and share the chunk swizzle, so two
      // lane offsets serve the four weight loads (the 16-row step is uniform and joins the K offset)
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const int g = w * LW + q;  // 8-row group, 0..31, of both tiles
        const int c = cp ^ (((g & 1) << 2) + (rl >> 1));
        voW[q] = (uint32_t)((g * 8 + rl) * p.ldw + c * 16);
      }
      w16 = (uint32_t)(16 * p.ldw);
      rW = weights_of(it);
      __builtin_amdgcn_sched_barrier(0);
      issue_w(rW, 0, 0);
      issue_w(rW, 1, 1);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int q = 0; q < LW; ++q) {
      const int g = w * LW + q;
      const int c = cp ^ (((g & 1) << 2) + (rl >> 1));
      const int sd = sid[q];
      voX[q] = sd < nrows ? (uint32_t)((int64_t)(sd / p.top_k) * p.ldx + c * 16) : 0xF0000000u;  // padding reads zeros
    }
    xreal = __builtin_amdgcn_ballot_w64(sid[0] < nrows) != 0;  // the first row of the wave's first group: a prefix
    issue_x(0, gx0);
  };
  start_item(item, true);

  for (;;) {
    int ln = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(ln));
    const int lr = ln & 31, h = ln >> 5;

    // ---- LDS -> MFMA operands
    const int swz = (lr >> 1) & 7;
    // lane part of an operand fetch address (row lr of a 32-row group, swizzled 16-byte chunk); stage, wave position
    // and group are uniform, so weights and activations share these four registers
    uint32_t fa[2][2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int q = 0; q < 2; ++q) fa[ks][q] = (uint32_t)(lr * kTileK + (((ks * 4 + h * 2 + q) ^ swz) << 4));
    auto frag = [&](const uint8_t* grp, int ks) -> v8i {  // grp: first row of the 32-row group inside its stage (uniform)
      const v4i lo = *reinterpret_cast<const v4i*>(grp + fa[ks][0]);
      const v4i hi = *reinterpret_cast<const v4i*>(grp + fa[ks][1]);
      v8i r;
      r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
      r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
      return r;
    };

    // ---- scales: activation scale rows follow the activation rows
    uint32_t sxo[MS];  // element offsets into the activation scales (the host checks they fit 32 bits)
    int nact = 0;      // the wave's 32-slot groups (wm, wm + 2, wm + 4, wm + 6) that hold real slots: a prefix, real slots come first
#pragma unroll
    for (int ms = 0; ms < MS; ++ms) {
      const int s = p.sorted_ids[slot0 + (ms * 2 + wm) * 32 + lr];
      nact += __builtin_amdgcn_readfirstlane(s) < nrows ? 1 : 0;
      sxo[ms] = SORTED ? (uint32_t)((int64_t)(slot0 + wm * 32 + lr) * p.sx_m)  // + ms * 64 rows, added as a uniform
                       : (s < nrows ? (uint32_t)((int64_t)(s / p.top_k) * p.sx_m) : 0u);
    }
    const uint32_t sx32 = SORTED ? (uint32_t)(64 * p.sx_m) : 0u;  // step between the scale rows of two of the wave's groups
    // the wave's 64 weight rows lie inside one 128-row block (FUSE: gate rows for wn 0, 1, up rows for wn 2, 3)
    const int nb = FUSE ? ((wn < 2 ? n0 : half_n + n0) >> 7) : (min(n0 + wn * 64, p.N - 1) >> 7);
    const float* swp = p.sw + (int64_t)expert * p.sw_expert_stride + (int64_t)nb * p.sw_n;

    v16f acc[NS][MS];
#pragma unroll
    for (int ns = 0; ns < NS; ++ns)
#pragma unroll
      for (int ms = 0; ms < MS; ++ms)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[ns][ms][r] = 0.f;

    // Scales.  PAIRS: sxp[ms] holds the activation scales of an even K block and the odd one after it, fetched with
    // one 8-byte load every other trip; with row-major scales the rows of a block are gathered, so every lane's load is
    // a cache line of its own whatever the layout, and what counts is the number of load instructions and that a
    // row's line is met again on the following trips.  Otherwise sxn[ms] / sbn hold the scales of the NEXT K block,
    // requested one trip ahead in front of that trip's stage loads: at the next barrier everything older than the
    // four youngest weight loads has landed, the scales among it.
    constexpr bool pairs = PAIRS;
    v2f sxp[MS];
    float sxn[MS], sbn = 0.f;
    float sba = 0.f, sbb = 0.f;  // PAIRS: weight scales of the even / odd block in flight
    auto load_sb = [&](float& sb, int kb) { sb = swp[(int64_t)min(kb, nkb - 1) * p.sw_k]; };
    auto load_sx = [&](int kb) {
      const uint32_t ko = (uint32_t)(min(kb, nkb - 1) * (int)p.sx_k);
#pragma unroll
      for (int ms = 0; ms < MS; ++ms)
        sxn[ms] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rSall, (int)(sxo[SORTED ? 0 : ms] * 4u),
                                                                                (int)((ko + (uint32_t)ms * sx32) * 4u), 0));
    };
    auto load_sx_pair = [&](int kb) {  // kb even: blocks kb and kb+1 (past the tensor: zero)
#pragma unroll
      for (int ms = 0; ms < MS; ++ms)
        sxp[ms] = __builtin_bit_cast(v2f, __builtin_amdgcn_raw_buffer_load_b64(rS, (int)((sxo[ms] + (uint32_t)kb) * 4u), 0, 0));
    };
    if (pairs) { load_sx_pair(0); load_sb(sba, 0); load_sb(sbb, 1); }
    else { load_sx(0); load_sb(sbn, 0); }
    // the item after this one, looked up while the first blocks arrive
    int jn = j + jstep;
    const MoeItem next = fetch_item(jn);
    rWn = weights_of(next);
    wait_vm0();  // the first trip's partial wait assumes the in-loop order of loads; the previous item's stores are out

    // one K block; its scales sit in sxp[.][parity] and sb on entry; the odd trips reload both blocks' activation
    // scales in the paired form
    auto trip = [&](auto na, int it, int parity, float& sb) {
      constexpr int NA = decltype(na)::value;  // 32-slot groups of the wave's half with real slots
      lds_barrier<LW>();  // everything but the wave's loads of weight block it+1 has landed
      // nothing of this trip may move in front of the barrier: the scale products below would drag a wait for
      // the scale loads of the previous trip with them, and loads return in order - that wait would also be one for
      // the weight block requested before those scales
      __builtin_amdgcn_sched_barrier(0);
      float sc[MS];  // SCALED: the exponent byte of the activation scale, as bits
      int sc_w = 127;  // SCALED: exponent byte of the weight scale
      if (pairs) {
#pragma unroll
        for (int ms = 0; ms < MS; ++ms) sc[ms] = sxp[ms][parity] * sb;
        if (parity) load_sx_pair(it + 1);
        load_sb(sb, it + 2);
      } else {
#pragma unroll
        for (int ms = 0; ms < MS; ++ms) sc[ms] = SCALED ? __uint_as_float(__float_as_uint(sxn[ms]) >> 23) : sxn[ms] * sbn;
        if (SCALED) sc_w = (int)(__float_as_uint(sbn) >> 23);
        load_sx(it + 1);
        load_sb(sbn, it + 1);
      }
      __builtin_amdgcn_sched_barrier(0);  // scales, then activations, then weights
      issue_x(it + 1, (gx0 + it + 1) & 1);  // into the stage of block it-1, which every wave has left (past the item's
                                            // last block the offsets are out of range: nothing moves)
      {
        // block it+2 of this item, or block 0 / 1 of the next one: the weight stream does not stop between items
        const int k2 = it + 2;
        const bool nx = k2 >= nkb;
        issue_w(nx ? rWn : rW, nx ? k2 - nkb : k2, (gw0 + k2) % WST);
      }
      if (NA == 0) return;
      const uint8_t* sw_ = smem + ((gw0 + it) % WST) * WBYTES;
      const uint8_t* sx_ = smem + XBASE + ((gx0 + it) & 1) * XBYTES;
      v8i wf[NS][2];
#pragma unroll
      for (int ns = 0; ns < NS; ++ns) {
        wf[ns][0] = frag(sw_ + (wn * 64 + ns * 32) * kTileK, 0);
        wf[ns][1] = frag(sw_ + (wn * 64 + ns * 32) * kTileK, 1);
      }
      v16f z;
#pragma unroll
      for (int r = 0; r < 16; ++r) z[r] = 0.f;
      if constexpr (SCALED) {
#pragma unroll
        for (int ms = 0; ms < NA; ++ms) {
          const v8i x0 = frag(sx_ + ((ms * 2 + wm) * 32) * kTileK, 0);
          const v8i x1 = frag(sx_ + ((ms * 2 + wm) * 32) * kTileK, 1);
          const int ex = (int)__float_as_uint(sc[ms]);
#pragma unroll
          for (int ns = 0; ns < NS; ++ns) {
            acc[ns][ms] = mfma_32x32x64_scaled(wf[ns][0], x0, acc[ns][ms], sc_w, ex);
            acc[ns][ms] = mfma_32x32x64_scaled(wf[ns][1], x1, acc[ns][ms], sc_w, ex);
          }
        }
      } else if constexpr (NA <= 3 || (SORTED && !FUSE)) {
        // two products in flight: the 16 scale-FMAs of one 32x32 product issue while the matrix core works on the
        // next (with one product at a time the wave sits out the matrix core's latency in front of every group of
        // FMAs, and with two waves per SIMD nobody else fills it).  The four-group copy of the other scale forms has
        // no registers for it; the sorted form's pays four scratch accesses per two trips and still gains (16384
        // tokens: 8.62 -> 8.48 ms).
        v16f tq[2];
        v8i x0 = frag(sx_ + (wm * 32) * kTileK, 0);
        v8i x1 = frag(sx_ + (wm * 32) * kTileK, 1);
        tq[0] = mfma_32x32x64(wf[0][0], x0, z);
        tq[0] = mfma_32x32x64(wf[0][1], x1, tq[0]);
#pragma unroll
        for (int i = 1; i < NA * NS; ++i) {
          const int ms = i >> 1, ns = i & 1;
          if (ns == 0) {
            x0 = frag(sx_ + ((ms * 2 + wm) * 32) * kTileK, 0);
            x1 = frag(sx_ + ((ms * 2 + wm) * 32) * kTileK, 1);
          }
          __builtin_amdgcn_sched_barrier(0);
          tq[i & 1] = mfma_32x32x64(wf[ns][0], x0, z);
          tq[i & 1] = mfma_32x32x64(wf[ns][1], x1, tq[i & 1]);
          __builtin_amdgcn_sched_barrier(0);
          const int pm = (i - 1) >> 1, pn = (i - 1) & 1;
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[pn][pm][r] = __builtin_fmaf(tq[(i - 1) & 1][r], sc[pm], acc[pn][pm][r]);
        }
        __builtin_amdgcn_sched_barrier(0);
        constexpr int L = NA * NS - 1;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[L & 1][L >> 1][r] = __builtin_fmaf(tq[L & 1][r], sc[L >> 1], acc[L & 1][L >> 1][r]);
      } else {
#pragma unroll
        for (int ms = 0; ms < NA; ++ms) {  // groups past the expert's last slot are padding
          const v8i x0 = frag(sx_ + ((ms * 2 + wm) * 32) * kTileK, 0);
          const v8i x1 = frag(sx_ + ((ms * 2 + wm) * 32) * kTileK, 1);
#pragma unroll
          for (int ns = 0; ns < NS; ++ns) {
            v16f tq = mfma_32x32x64(wf[ns][0], x0, z);
            tq = mfma_32x32x64(wf[ns][1], x1, tq);
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ns][ms][r] = __builtin_fmaf(tq[r], sc[ms], acc[ns][ms][r]);
          }
        }
      }
    };
    auto run = [&](auto na) {
      int it = 0;
      for (; it + 1 < nkb; it += 2) {
        trip(na, it, 0, sba);
        trip(na, it + 1, 1, sbb);
      }
      if (it < nkb) trip(na, it, 0, sba);
    };
    // The hardware-scaled form keeps the matrix core fed across the barrier of a trip: the products of a block's LAST
    // slot group are formed behind the NEXT barrier, from registers, and the fragments of the new block are fetched
    // from LDS in their shadow - each weight fragment refilled in place right behind the MFMA that used it last, the
    // first activation fragments of the new block behind the MFMAs that used the old ones.  (Otherwise every wave of
    // the workgroup opens a trip with the same ten LDS fetches and the matrix cores idle until they are back.)  The
    // float-scale forms have no registers for it: their second accumulator set takes the room.
    auto run_scaled = [&](auto na) {
      constexpr int NA = decltype(na)::value;
      using yes = std::integral_constant<bool, true>;
      using no = std::integral_constant<bool, false>;
      v8i wf[NS][2], xa, xb;
      int ex[MS], ew = 127;      // exponent bytes of the block in work
      int exd = 127, ewd = 127;  // ... of the deferred group
      // barrier of trip `it`, the exponents of its block, the next scales and the stage loads
      auto open = [&](int it) {
        lds_barrier<LW>();  // everything but the wave's loads of weight block it+1 has landed
        SB();
#pragma unroll
        for (int ms = 0; ms < MS; ++ms) ex[ms] = (int)(__float_as_uint(sxn[ms]) >> 23);
        ew = (int)(__float_as_uint(sbn) >> 23);
        load_sx(it + 1);
        load_sb(sbn, it + 1);
        SB();  // scales, then activations, then weights
        issue_x(it + 1, (gx0 + it + 1) & 1);
        const int k2 = it + 2;
        const bool nx = k2 >= nkb;
        issue_w(nx ? rWn : rW, nx ? k2 - nkb : k2, (gw0 + k2) % WST);
        SB();
      };
      // the last group of the previous block (fragments xa / xb, exponents exd / ewd); REFILL: the fragments of block
      // `it` take the registers over as they fall free
      auto deferred = [&](auto refill, const uint8_t* sw_, const uint8_t* sx_) {
        constexpr bool RF = decltype(refill)::value;
        constexpr int L = NA > 0 ? NA - 1 : 0;
        const uint8_t* w0 = sw_ + (wn * 64) * kTileK;
        const uint8_t* w1 = sw_ + (wn * 64 + 32) * kTileK;
        const uint8_t* xg = sx_ + (wm * 32) * kTileK;
        acc[0][L] = mfma_32x32x64_scaled(wf[0][0], xa, acc[0][L], ewd, exd); SB();
        if (RF) wf[0][0] = frag(w0, 0);
        SB();
        acc[1][L] = mfma_32x32x64_scaled(wf[1][0], xa, acc[1][L], ewd, exd); SB();
        if (RF) { wf[1][0] = frag(w1, 0); xa = frag(xg, 0); }
        SB();
        acc[0][L] = mfma_32x32x64_scaled(wf[0][1], xb, acc[0][L], ewd, exd); SB();
        if (RF) wf[0][1] = frag(w0, 1);
        SB();
        acc[1][L] = mfma_32x32x64_scaled(wf[1][1], xb, acc[1][L], ewd, exd); SB();
        if (RF) { wf[1][1] = frag(w1, 1); xb = frag(xg, 1); }
        SB();
      };
      // groups 0 .. NA-2 of the block whose fragments sit in wf / xa / xb; leaves the last group's fragments in xa / xb
      auto groups = [&](const uint8_t* sx_) {
#pragma unroll
        for (int ms = 0; ms + 1 < NA; ++ms) {
          acc[0][ms] = mfma_32x32x64_scaled(wf[0][0], xa, acc[0][ms], ew, ex[ms]);
          acc[1][ms] = mfma_32x32x64_scaled(wf[1][0], xa, acc[1][ms], ew, ex[ms]);
          acc[0][ms] = mfma_32x32x64_scaled(wf[0][1], xb, acc[0][ms], ew, ex[ms]);
          acc[1][ms] = mfma_32x32x64_scaled(wf[1][1], xb, acc[1][ms], ew, ex[ms]);
          SB();
          xa = frag(sx_ + (((ms + 1) * 2 + wm) * 32) * kTileK, 0);
          xb = frag(sx_ + (((ms + 1) * 2 + wm) * 32) * kTileK, 1);
          SB();
        }
        exd = ex[NA > 0 ? NA - 1 : 0];
        ewd = ew;
      };
      open(0);
      if constexpr (NA > 0) {
        const uint8_t* sw_ = smem + (gw0 % WST) * WBYTES;
        const uint8_t* sx_ = smem + XBASE + (gx0 & 1) * XBYTES;
#pragma unroll
        for (int ns = 0; ns < NS; ++ns) {
          wf[ns][0] = frag(sw_ + (wn * 64 + ns * 32) * kTileK, 0);
          wf[ns][1] = frag(sw_ + (wn * 64 + ns * 32) * kTileK, 1);
        }
        xa = frag(sx_ + (wm * 32) * kTileK, 0);
        xb = frag(sx_ + (wm * 32) * kTileK, 1);
        SB();
        groups(sx_);
      }
      auto trip = [&](int it) {
        open(it);
        if constexpr (NA > 0) {
          const uint8_t* sw_ = smem + ((gw0 + it) % WST) * WBYTES;
          const uint8_t* sx_ = smem + XBASE + ((gx0 + it) & 1) * XBYTES;
          deferred(yes{}, sw_, sx_);
          groups(sx_);
        }
      };
      int it = 1;
      for (; it + 1 < nkb; it += 2) {  // two trips per round: the scale registers then need no copies between rounds
        trip(it);
        trip(it + 1);
      }
      if (it < nkb) trip(it);
      if constexpr (NA > 0) deferred(no{}, smem, smem);
    };
    // The float-scale loop of the sorted forms, software-pipelined like the dense 256x256 tile kernel's with the roles
    // of weights and activations swapped: the wave keeps the four weight fragments of a K block and walks its slot groups,
    // one step (four MFMAs: n half 0 / 1 on K half 0, then on K half 1) per group.  The products of a step gather in
    // tq[n half] and are folded into the accumulator with the block's scale behind the first MFMAs of the NEXT step, the
    // activation fragments are refilled with the next group's behind their last use, and the step of a block's LAST group
    // runs behind the next barrier, where every weight fragment is refilled from the new block right behind the MFMA that
    // used it last.  The matrix core then has work across the barrier, and the operand fetches of the eight waves no
    // longer come as one burst behind it.  Every wave issues the same loads at the same places whatever its group count.
    auto run_piped = [&](auto na, auto xl) {
      constexpr int NA = decltype(na)::value;
      constexpr bool XL = decltype(xl)::value;  // the wave's activation loads carry real slots
      constexpr int L = NA > 0 ? NA - 1 : 0, L2 = NA > 1 ? NA - 2 : 0;
      using yes = std::integral_constant<bool, true>;
      using no = std::integral_constant<bool, false>;
      v8i wf[NS][2], xa, xb;
      v16f tq[2], z;
#pragma unroll
      for (int r = 0; r < 16; ++r) { z[r] = 0.f; tq[0][r] = 0.f; tq[1][r] = 0.f; }
      float sc[MS] = {0.f, 0.f, 0.f, 0.f};  // activation x weight scale of the block whose products are being formed
      float sd0 = 0.f, sd1 = 0.f;          // ... of groups NA-2 and NA-1 of the block before: their products are folded after the barrier
      // The eight stage loads of a trip (1 KB each) pass through the CU's address unit at 64 bytes a clock, all eight
      // waves' at once: issued in one run behind the barrier they hold every wave for several hundred cycles (the later
      // waves of the queue for more than a thousand) before its first MFMA.  A wave with groups to work on therefore
      // spreads them over the step that follows the barrier, two behind each MFMA.
      int ld_it = 0;
      auto ld = [&](int i) {  // stage load i of trip ld_it: activations of block ld_it+1 (0..3), weights of block ld_it+2 (4..7)
        if (i < 4) {
          if constexpr (XL) issue_x1(i, ld_it + 1, (gx0 + ld_it + 1) & 1);
        } else {
          const int k2 = ld_it + 2;
          const bool nx = k2 >= nkb;
          issue_w1(i - 4, nx ? rWn : rW, nx ? k2 - nkb : k2, (gw0 + k2) % WST);
        }
      };
      auto open = [&](int it, auto all_loads) {
        lds_barrier<LW>();  // everything but the wave's loads of weight block it+1 has landed
        SB();
        sd0 = sc[L2];
        sd1 = sc[L];
#pragma unroll
        for (int ms = 0; ms < MS; ++ms) sc[ms] = sxn[ms] * sbn;
        load_sx(it + 1);
        load_sb(sbn, it + 1);
        SB();  // scales, then activations, then weights
        ld_it = it;
        if constexpr (decltype(all_loads)::value) {
#pragma unroll
          for (int i = 0; i < 8; ++i) ld(i);
        }
        SB();
      };
      auto fold = [&](auto ns_c, auto pg_c, float s) {
        constexpr int NS_ = decltype(ns_c)::value, PG = decltype(pg_c)::value;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[NS_][PG][r] = __builtin_fmaf(tq[NS_][r], s, acc[NS_][PG][r]);
      };
      using n0_t = std::integral_constant<int, 0>;
      using n1_t = std::integral_constant<int, 1>;
      // One step.  PEND: the products of the step before (slot group PG, scale ps) are folded first.  FILL 0: the
      // activation fragments of the group at nx_ follow; 1: those and the weight fragments of the block at nw_; 2: nothing.
      auto step = [&](auto pend_c, auto pg_c, float ps, auto fill_c, const uint8_t* nw_, const uint8_t* nx_) {
        constexpr bool PEND = decltype(pend_c)::value;
        constexpr int FILL = decltype(fill_c)::value;
        constexpr bool LOADS = FILL == 1;  // the step behind a barrier carries the trip's stage loads
        const uint8_t* w0 = nw_ + (wn * 64) * kTileK;
        const uint8_t* w1 = nw_ + (wn * 64 + 32) * kTileK;
        if constexpr (PEND) { fold(n0_t{}, pg_c, ps); SB(); }
        tq[0] = mfma_32x32x64(wf[0][0], xa, z); SB();
        if constexpr (FILL == 1) { wf[0][0] = frag(w0, 0); SB(); }
        if constexpr (LOADS) { ld(0); ld(1); SB(); }
        if constexpr (PEND) { fold(n1_t{}, pg_c, ps); SB(); }
        tq[1] = mfma_32x32x64(wf[1][0], xa, z); SB();
        if constexpr (FILL != 2) xa = frag(nx_, 0);
        if constexpr (FILL == 1) wf[1][0] = frag(w1, 0);
        if constexpr (LOADS) { ld(2); ld(3); }
        SB();
        tq[0] = mfma_32x32x64(wf[0][1], xb, tq[0]); SB();
        if constexpr (FILL == 1) { wf[0][1] = frag(w0, 1); SB(); }
        if constexpr (LOADS) { ld(4); ld(5); SB(); }
        tq[1] = mfma_32x32x64(wf[1][1], xb, tq[1]); SB();
        if constexpr (FILL != 2) xb = frag(nx_, 1);
        if constexpr (FILL == 1) wf[1][1] = frag(w1, 1);
        if constexpr (LOADS) { ld(6); ld(7); }
        SB();
      };
      using fill_x = std::integral_constant<int, 0>;
      using fill_all = std::integral_constant<int, 1>;
      using fill_none = std::integral_constant<int, 2>;
      // groups 0 .. NA-2 of the block whose fragments sit in wf / xa / xb; FIRST: nothing is pending in front of group 0
      auto groups = [&](auto first_c, const uint8_t* sx_) {
        constexpr bool FIRST = decltype(first_c)::value;
        if constexpr (NA >= 2) {
          const uint8_t* g1 = sx_ + ((1 * 2 + wm) * 32) * kTileK;
          if constexpr (FIRST) step(no{}, std::integral_constant<int, 0>{}, 0.f, fill_x{}, smem, g1);
          else step(yes{}, std::integral_constant<int, L>{}, sd1, fill_x{}, smem, g1);
        }
        if constexpr (NA >= 3) step(yes{}, std::integral_constant<int, 0>{}, sc[0], fill_x{}, smem, sx_ + ((2 * 2 + wm) * 32) * kTileK);
        if constexpr (NA >= 4) step(yes{}, std::integral_constant<int, 1>{}, sc[1], fill_x{}, smem, sx_ + ((3 * 2 + wm) * 32) * kTileK);
      };
      open(0, yes{});
      if constexpr (NA > 0) {
        const uint8_t* sw_ = smem + (gw0 % WST) * WBYTES;
        const uint8_t* sx_ = smem + XBASE + (gx0 & 1) * XBYTES;
#pragma unroll
        for (int ns = 0; ns < NS; ++ns) {
          wf[ns][0] = frag(sw_ + (wn * 64 + ns * 32) * kTileK, 0);
          wf[ns][1] = frag(sw_ + (wn * 64 + ns * 32) * kTileK, 1);
        }
        xa = frag(sx_ + (wm * 32) * kTileK, 0);
        xb = frag(sx_ + (wm * 32) * kTileK, 1);
        SB();
        groups(yes{}, sx_);
      }
      for (int it = 1; it < nkb; ++it) {
        open(it, std::integral_constant<bool, NA == 0>{});
        if constexpr (NA > 0) {
          const uint8_t* sw_ = smem + ((gw0 + it) % WST) * WBYTES;
          const uint8_t* sx_ = smem + XBASE + ((gx0 + it) & 1) * XBYTES;
          // the last group of block it-1; the group before it (if the wave has two) is still pending
          if constexpr (NA >= 2) step(yes{}, std::integral_constant<int, L2>{}, sd0, fill_all{}, sw_, sx_ + (wm * 32) * kTileK);
          else step(no{}, std::integral_constant<int, 0>{}, 0.f, fill_all{}, sw_, sx_ + (wm * 32) * kTileK);
          if constexpr (NA == 1) {  // a single group: its products are folded on the spot (the next step comes two barriers later)
            fold(n0_t{}, std::integral_constant<int, 0>{}, sd1); fold(n1_t{}, std::integral_constant<int, 0>{}, sd1);
            SB();
          }
          groups(no{}, sx_);
        }
      }
      if constexpr (NA > 0) {
        if constexpr (NA >= 2) step(yes{}, std::integral_constant<int, L2>{}, sc[L2], fill_none{}, smem, smem);
        else step(no{}, std::integral_constant<int, 0>{}, 0.f, fill_none{}, smem, smem);
        fold(n0_t{}, std::integral_constant<int, L>{}, sc[L]);
        fold(n1_t{}, std::integral_constant<int, L>{}, sc[L]);
      }
    };
    // one copy of the loop per group count keeps every copy straight-line
    if constexpr (SCALED) {
      switch (nact) {  // wave-uniform
        case 4: run_scaled(std::integral_constant<int, 4>{}); break;
        case 3: run_scaled(std::integral_constant<int, 3>{}); break;
        case 2: run_scaled(std::integral_constant<int, 2>{}); break;
        case 1: run_scaled(std::integral_constant<int, 1>{}); break;
        default: run_scaled(std::integral_constant<int, 0>{}); break;
      }
    } else if constexpr (SORTED && !PAIRS) {
      using with_x = std::integral_constant<bool, true>;
      using without_x = std::integral_constant<bool, false>;
      if (xreal) {
        switch (nact) {  // wave-uniform
          case 4: run_piped(std::integral_constant<int, 4>{}, with_x{}); break;
          case 3: run_piped(std::integral_constant<int, 3>{}, with_x{}); break;
          case 2: run_piped(std::integral_constant<int, 2>{}, with_x{}); break;
          case 1: run_piped(std::integral_constant<int, 1>{}, with_x{}); break;
          default: run_piped(std::integral_constant<int, 0>{}, with_x{}); break;
        }
      } else {
        switch (nact) {
          case 4: run_piped(std::integral_constant<int, 4>{}, without_x{}); break;
          case 3: run_piped(std::integral_constant<int, 3>{}, without_x{}); break;
          case 2: run_piped(std::integral_constant<int, 2>{}, without_x{}); break;
          case 1: run_piped(std::integral_constant<int, 1>{}, without_x{}); break;
          default: run_piped(std::integral_constant<int, 0>{}, without_x{}); break;
        }
      }
    } else {
      switch (nact) {  // wave-uniform
        case 4: run(std::integral_constant<int, 4>{}); break;
        case 3: run(std::integral_constant<int, 3>{}); break;
        case 2: run(std::integral_constant<int, 2>{}); break;
        case 1: run(std::integral_constant<int, 1>{}); break;
        default: run(std::integral_constant<int, 0>{}); break;
      }
    }
    // output rows and routed weights, fetched while the stages drain (lane id taken anew, as above)
    const bool wide = (p.ldc & 7) == 0 && (reinterpret_cast<uintptr_t>(p.C) & 15) == 0;
    int lane_e = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(lane_e));
    const int lr_e = lane_e & 31, h_e = lane_e >> 5;
    const int er = lane_e >> 3, ec = lane_e & 7;  // store loop: row inside a group of 8, 16-byte chunk of the wave's 128 bytes
    const int eslot0 = slot0, en0 = n0;
    int oslots[MS], srow[16];
    float rsw[MS];
#pragma unroll
    for (int ms = 0; ms < MS; ++ms) oslots[ms] = p.sorted_ids[eslot0 + (ms * 2 + wm) * 32 + lr_e];
#pragma unroll
    for (int i = 0; i < 16; ++i) srow[i] = (wide && !FUSE) ? p.sorted_ids[eslot0 + ((i >> 2) * 2 + wm) * 32 + (i & 3) * 8 + er] : 0;
#pragma unroll
    for (int ms = 0; ms < MS; ++ms) rsw[ms] = (p.topk_w && oslots[ms] < nrows) ? p.topk_w[oslots[ms]] : 1.f;
    lds_barrier();  // every wave has left the item's last stages; the requests in flight point at the other ones
    const int ews = (gw0 + nkb - 1) % WST, exs = (gx0 + nkb - 1) & 1;  // the stages of the item's last block
    gw0 = (gw0 + nkb) % WST;
    gx0 = (gx0 + nkb) & 1;
    const bool has_next = next.mb >= 0;
    if (has_next) {
      rW = rWn;
      start_item(next, false);  // its first activation block travels while this item is written out
    }

    if constexpr (FUSE) {
      // ---- activation and requantisation of the finished tile, spread over all eight waves.  A gate wave (wn = 0, 1)
      // and the up wave of the same lanes and registers (wn + 2, same wm) hold the two factors of the same 128 slots x
      // 64 activation columns.  They swap halves through LDS as 16-bit values (which is what the reference's
      // intermediate holds): the up wave hands over its slot groups 0, 2, the gate wave its groups 1, 3; then the gate
      // wave forms a = T(T(silu(T(gate))) * T(up)) for groups 0, 2 and the up wave for groups 1, 3 (real slots come
      // first in a block, so a half-empty block leaves every wave one group of real slots; groups that are all
      // padding are skipped, only their zero scales are written).  The two waves
      // that hold the two 64-column halves of the same slots (wn ^ 1) exchange their row maxima, every wave quantises
      // its 64 slots x 64 columns with the quant kernels' arithmetic and stores bytes (re-laid out through LDS for
      // 16-byte stores) and, the lower half's wave, the scale of every slot.  Each pair works inside 16 KB of the
      // stages of the item's last block: [0, 8 KB) belongs to the gate wave, [8 KB, 16 KB) to the up wave.
      const int pr = wn & 1;
      const bool upw = wn >= 2;
      uint8_t* const pair = smem + (wm == 0 ? ews * WBYTES : XBASE + exs * XBYTES) + pr * 16384;
      uint8_t* const own_area = pair + (upw ? 8192 : 0);
      const uint8_t* const partner_area = pair + (upw ? 0 : 8192);
      const float* const mate_max = reinterpret_cast<const float*>(pair + (pr ? -16384 : 16384) + (upw ? 8192 : 0));
      auto pack4 = [&](const float (&v)[4]) -> uint2 {
        uint2 o;
        if (OUT_DT == FP8K_BF16) { o.x = pack_bf16x2(v[0], v[1]); o.y = pack_bf16x2(v[2], v[3]); }
        else { o.x = f32_to_f16_bits(v[0]) | (f32_to_f16_bits(v[1]) << 16); o.y = f32_to_f16_bits(v[2]) | (f32_to_f16_bits(v[3]) << 16); }
        return o;
      };
      // MINE: first of the wave's own two slot groups (MINE, MINE + 2); it hands over the other two; UP: the wave holds
      // up values
      auto finish = [&](auto mine_c, auto up_c) {
        constexpr int MINE = decltype(mine_c)::value, SEND = 1 - MINE;
        constexpr bool UP = decltype(up_c)::value;
        int qrow[4];  // store loop: lane -> row it * 16 + lane / 4 of the wave's 64 slots, 16-byte chunk lane % 4
#pragma unroll
        for (int it4 = 0; it4 < 4; ++it4) {
          const int r = it4 * 16 + (lane_e >> 2);
          qrow[it4] = p.sorted_ids[eslot0 + ((MINE + 2 * (r >> 5)) * 2 + wm) * 32 + (r & 31)];
        }
        // a group holds real slots iff its first slot is real (wave-uniform)
        bool real_mine[2], real_send[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          real_mine[i] = __builtin_amdgcn_readfirstlane(oslots[MINE + 2 * i]) < nrows;
          real_send[i] = __builtin_amdgcn_readfirstlane(oslots[SEND + 2 * i]) < nrows;
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          if (!real_send[i]) continue;
#pragma unroll
          for (int ns = 0; ns < NS; ++ns)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
              const float v[4] = {acc[ns][SEND + 2 * i][rg * 4], acc[ns][SEND + 2 * i][rg * 4 + 1],
                                  acc[ns][SEND + 2 * i][rg * 4 + 2], acc[ns][SEND + 2 * i][rg * 4 + 3]};
              *reinterpret_cast<uint2*>(own_area + ((i * 2 + ns) * 4 + rg) * 512 + lane_e * 8) = pack4(v);
            }
        }
        lds_barrier();
        float amx[2] = {0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          if (!real_mine[i]) continue;
          float m = 0.f;
#pragma unroll
          for (int ns = 0; ns < NS; ++ns)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
              const uint2 u = *reinterpret_cast<const uint2*>(partner_area + ((i * 2 + ns) * 4 + rg) * 512 + lane_e * 8);
              float pv[4];
              if (OUT_DT == FP8K_BF16) { pv[0] = bf16_lo(u.x); pv[1] = bf16_hi(u.x); pv[2] = bf16_lo(u.y); pv[3] = bf16_hi(u.y); }
              else { pv[0] = f16_bits_to_f32(u.x & 0xffff); pv[1] = f16_bits_to_f32(u.x >> 16); pv[2] = f16_bits_to_f32(u.y & 0xffff); pv[3] = f16_bits_to_f32(u.y >> 16); }
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const float own = round_to<OUT_DT>(acc[ns][MINE + 2 * i][rg * 4 + r]);
                const float g = UP ? pv[r] : own, up = UP ? own : pv[r];
                const float a = round_to<OUT_DT>(round_to<OUT_DT>(silu_f32(g)) * up);
                acc[ns][MINE + 2 * i][rg * 4 + r] = a;
                m = fmaxf(m, fabsf(a));
              }
            }
          m = fmaxf(m, __shfl_xor(m, 32));  // the other 16 columns of every tile of the row
          amx[i] = m;
        }
        lds_barrier();  // every wave has read what it was sent: the areas are free for the maxima and the bytes
        if (h_e == 0) {
#pragma unroll
          for (int i = 0; i < 2; ++i) reinterpret_cast<float*>(own_area)[i * 32 + lr_e] = amx[i];
        }
        lds_barrier();
        uint8_t* const st = own_area + 1024;  // 64 rows x 64 B of bytes, behind the maxima
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          if (!real_mine[i]) {  // all padding: nothing to store but the zero scales GEMM 2 reads for these positions
            if (pr == 0 && h_e == 0) p.qs_out[(int64_t)(en0 >> 7) * p.qs_ld + eslot0 + ((MINE + 2 * i) * 2 + wm) * 32 + lr_e] = 0.f;
            continue;
          }
          const float amax = fmaxf(fmaxf(amx[i], mate_max[i * 32 + lr_e]), p.q_eps);
          const float sc = div448<true>(amax);
          const int row = i * 32 + lr_e;
#pragma unroll
          for (int ns = 0; ns < NS; ++ns)
#pragma unroll
            for (int rp = 0; rp < 2; ++rp) {
              float a8[8];
#pragma unroll
              for (int r = 0; r < 4; ++r) { a8[r] = acc[ns][MINE + 2 * i][(rp * 2) * 4 + r]; a8[4 + r] = acc[ns][MINE + 2 * i][(rp * 2 + 1) * 4 + r]; }
              bool redo;
              uint2 o = quant8_bracket<true>(a8, sc, amax, redo);
              if (redo) o = quant8_divide(a8, sc);
              *reinterpret_cast<uint32_t*>(st + row * 64 + ns * 32 + (rp * 2) * 8 + h_e * 4) = o.x;
              *reinterpret_cast<uint32_t*>(st + row * 64 + ns * 32 + (rp * 2 + 1) * 8 + h_e * 4) = o.y;
            }
          if (pr == 0 && h_e == 0) {
            const int pos = eslot0 + ((MINE + 2 * i) * 2 + wm) * 32 + lr_e;
            p.qs_out[(int64_t)(en0 >> 7) * p.qs_ld + pos] = oslots[MINE + 2 * i] < nrows ? sc : 0.f;
          }
        }
        __builtin_amdgcn_wave_barrier();  // one wave's LDS accesses complete in order
#pragma unroll
        for (int it4 = 0; it4 < 4; ++it4) {
          if (!real_mine[it4 >> 1]) continue;
          const int r = it4 * 16 + (lane_e >> 2), c = lane_e & 3;
          const uint4 o = *reinterpret_cast<const uint4*>(st + r * 64 + c * 16);
          const int sdst = qrow[it4];
          if (sdst < nrows) *reinterpret_cast<uint4*>(p.q_out + (int64_t)sdst * p.ldq + en0 + pr * 64 + c * 16) = o;
        }
      };
      if (upw) finish(std::integral_constant<int, 1>{}, std::integral_constant<bool, true>{});
      else finish(std::integral_constant<int, 0>{}, std::integral_constant<bool, false>{});
      if (!has_next) {
        wait_vm0();
        return;
      }
      item = next;
      j = jn;
      continue;
    }

    // ---- write-out through LDS, in two passes of 64 slots.  A wave re-lays 64 slots x 64 n of its block out in a
    // private 8 KB slot inside the weight / activation stage of the item's last block (128 B per row, 16-byte chunk c
    // of row r at position c ^ ((r >> 1) & 7), so that the accumulator-shaped 8-byte writes and the 16-byte reads
    // spread over all banks): no workgroup barrier, and every store instruction writes eight whole 128-byte lines.
    uint8_t* const ep = smem + (w < 4 ? ews * WBYTES + w * 8192 : XBASE + exs * XBYTES + (w - 4) * 8192);
#pragma unroll
    for (int ph = 0; ph < 2; ++ph) {
      if (ph * 2 >= nact) break;  // the wave's remaining slot groups are all padding (real slots come first): nothing to store
#pragma unroll
      for (int mh = 0; mh < 2; ++mh) {
        const int ms = ph * 2 + mh;
        if (ms >= nact) continue;
        const int row = mh * 32 + lr_e;  // inside the pass's 64 slots
        const int oslot = oslots[ms];
        const bool ok = oslot < nrows;
        const float rs = rsw[ms];
#pragma unroll
        for (int nr = 0; nr < NS * 4; ++nr) {
          const int ns = nr >> 2, rg = nr & 3;
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] = acc[ns][ms][rg * 4 + r] * rs;
          if (wide) {
            uint2 o;
            if (OUT_DT == FP8K_BF16) {
              o.x = pack_bf16x2(v[0], v[1]);
              o.y = pack_bf16x2(v[2], v[3]);
            } else {
              o.x = f32_to_f16_bits(v[0]) | (f32_to_f16_bits(v[1]) << 16);
              o.y = f32_to_f16_bits(v[2]) | (f32_to_f16_bits(v[3]) << 16);
            }
            *reinterpret_cast<uint2*>(ep + row * 128 + ((nr ^ ((row >> 1) & 7)) << 4) + h_e * 8) = o;
          } else {
            const int n = en0 + wn * 64 + nr * 8 + h_e * 4;
            if (ok && n < p.N) store4<OUT_DT>(p.C, (int64_t)oslot * p.ldc + n, v[0], v[1], v[2], v[3]);
          }
        }
      }
      if (wide) {
        __builtin_amdgcn_wave_barrier();  // one wave's LDS accesses complete in order: no wait needed
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (ph * 2 + (i >> 2) >= nact) continue;
          const int row = i * 8 + er;
          const int s = srow[ph * 8 + i];
          const int n = en0 + wn * 64 + (ec << 3);
          const uint4 o = *reinterpret_cast<const uint4*>(ep + row * 128 + ((ec ^ ((row >> 1) & 7)) << 4));
          if (s < nrows && n < p.N) *reinterpret_cast<uint4*>((u16*)p.C + (int64_t)s * p.ldc + n) = o;
        }
        __builtin_amdgcn_wave_barrier();
      }
    }
    if (!has_next) {
      wait_vm0();  // the out-of-range requests of the last trips still point at the stages: let them retire before the LDS goes back
      return;
    }
    item = next;
    j = jn;
  }
}

}  // namespace fp8k
