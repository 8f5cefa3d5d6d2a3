// FP8 MFMA GEMM device code for gfx950 (CDNA4).
//
// Operands: "W" = weight rows [N,K] and "X" = activation rows [M,K], both e4m3fn with K contiguous.
// The MFMA computes the transposed product: W rows are the matrix-core "A" operand, X rows the "B"
// operand, so one lane of a 32x32 result tile holds 16 values of ONE activation row (m = lane%32)
// and four runs of 4 consecutive n.  A block-scaled K step therefore needs a single scale
// as[m,kb]*bs[nb,kb] per lane, and the bf16 output is written as 8-byte runs along n.
#pragma once

#include <type_traits>

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
  int tail_first;     // tile256 only: tiles [tail_first, tiles) are the ones cut along K or into halves
  int tail_halves;    // tile256 only: those tiles are computed as two 128-row halves, one workgroup each (no K cut)
  int walkers;        // tile256 only: workgroups [0, walkers) walk the whole tiles (a multiple of 8)
  int tail_shared;    // tile256 only: unit u of the tail belongs to workgroup u (after its walk), else to workgroup walkers + u
  int wk_nw;          // gemm_wavek_kernel only: waves of a workgroup along n (1, 2, 4 or 8; the other 8 / wk_nw cut K)
  // grouped (MoE) form of the streaming kernel; all null / zero for a dense GEMM
  const int32_t* sorted_ids;    // [m_blocks * TM] token slots, padded with values >= num_valid
  const int32_t* expert_ids;    // [m_blocks] expert of each block of TM slots, -1 = not on this rank
  const int32_t* num_post_pad;  // device scalar: slots in use (multiple of TM)
  const float* topk_w;          // routed weight per slot, or null
  int top_k;                    // X row of a slot = slot / top_k
  int num_valid;                // number of real slots (topk_ids.numel())
  int m_blocks;                 // dense: blocks of TM rows; grouped: capacity of sorted_ids in blocks
  int block_m;                  // grouped: slots per block in sorted_ids (<= TM)
  int sx_sorted;                // grouped: sx holds one row per position of sorted_ids (row = position), not per token
  int64_t w_expert_stride;      // bytes between experts in W
  // grouped GEMM 1 with the activation and the requantisation in its write-out (moe_stream256_kernel<..., FUSE>):
  // N = 2 I weight rows (gate rows, then up rows); q_out [slots, I] e4m3fn, qs_out [I/128][capacity of sorted_ids] float
  uint8_t* q_out;
  float* qs_out;
  int64_t ldq;
  int64_t qs_ld;                // floats between the scale rows of two activation column blocks (>= capacity)
  float q_eps;                  // lower clamp of the group maximum (already rounded to the element type)
  int64_t sw_expert_stride;     // floats between experts in sw
  // batched form of the 128x128 tile kernel (grid y = batch entry); zero for a single GEMM
  int64_t batch_x, batch_w;     // bytes between batch entries of X and W
  int64_t batch_c;              // elements between batch entries of C
};

// kModeScaled: block mode with power-of-two scales applied by the matrix core itself (activation scales as packed
// UE8M0 bytes, weight scales as float powers of two): no float promote, one accumulator over the whole K range
enum { kModeBlock = 0, kModeRow = 1, kModeScaled = 2 };

typedef __attribute__((address_space(3))) void* lds_ptr_t;
__device__ __forceinline__ void wait_vm0() { __builtin_amdgcn_s_waitcnt(0x0F70); }  // vmcnt(0)

__device__ __forceinline__ v16f mfma_32x32x64(v8i a, v8i b, v16f c) {
  // cbsz = blgp = 0: both operands e4m3; scale operands 0 select the unscaled instruction form
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}
// the same with block scales: byte 0 of scale_a / scale_b is the E8M0 exponent (value 2^(e-127)) of the 32 K
// elements that this lane holds of its A row / B column
__device__ __forceinline__ v16f mfma_32x32x64_scaled(v8i a, v8i b, v16f c, int scale_a, int scale_b) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, scale_a, 0, scale_b);
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
// LDS: three weight stages and two activation stages of 256 rows x 128 B each = 160 KB, filled by
// buffer_load_dwordx4 ... lds (no register staging; rows past the matrix edge are out of the
// descriptor's range - the complete offset is in the range-checked per-lane operand - and arrive
// as zeros without touching memory).  A 1 KB wave-load covers 8 rows; the 16-byte chunk c of
// row r is stored at chunk position c ^ ((r >> 1) & 7), which makes both the linear LDS-DMA writes
// and the ds_read_b128 operand fetches (32 rows, same logical chunk) bank-conflict free.
//
// Pipeline.  One loop iteration is one barrier interval, and the barrier sits BEFORE the last
// quarter of a K block: by then a wave has every operand of the block in registers, so after the
// barrier (a) the activation stage it just left can be refilled with block it+2 and the weight
// stage with block it+3 at once and (b) the first operands of block it+1 are fetched while the
// last four MFMAs of block it still run.  A wave's loads retire in order and are issued as
// activations, scales, weights: the wait in front of the barrier leaves its four weight loads in
// flight, so the weights - whose lines come from HBM or the memory-side cache, where the
// activations mostly hit the L2 - have two barrier intervals to arrive.  Operand
// fetches are issued two MFMA groups ahead of their use; the eight 1 KB global loads of a wave are
// spread over the first half of the interval, two per group, because the texture-address path
// moves 64 B/clk per CU and a burst would stall the issuing wave.  The loop body is branch-free
// (loads past the last K block are out of range or unread), which keeps the compiler from sinking
// the scale FMAs to the loop latch.
//
// Block mode keeps two short-lived accumulators: t = W.X over one K block, then
// acc += t * (as[m,kb] * bs[nb,kb]), with the 16 FMAs of group g-1 split around the two MFMAs of
// group g; row mode accumulates in place and scales in the epilogue.
// ------------------------------------------------------------------------------------------------
constexpr int kTileN = 256, kTileM = 256, kTileK = 128;

typedef __amdgpu_buffer_rsrc_t rsrc_t;
// raw buffer descriptor: base pointer + byte range; loads past the range return zero
__device__ __forceinline__ rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)p, 0, (int)bytes, 0x00020000);
}
// 16 bytes per lane from buffer + voff (per lane) + soff (uniform) straight into LDS at lds_base + lane*16
__device__ __forceinline__ void buf_load16_to_lds(rsrc_t r, uint32_t voff, uint32_t soff, uint8_t* lds_base) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr_t)lds_base, 16, (int)voff, (int)soff, 0, 0);
}
// 4 bytes per lane into LDS at lds_base + lane*4 (inactive lanes write nothing)
__device__ __forceinline__ void buf_load4_to_lds(rsrc_t r, uint32_t voff, uint32_t soff, uint8_t* lds_base) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr_t)lds_base, 4, (int)voff, (int)soff, 0, 0);
}
__device__ __forceinline__ void wait_vm0_lgkm0() { __builtin_amdgcn_s_waitcnt(0x0070); }  // vmcnt(0) lgkmcnt(0)

// Workgroup barrier that orders LDS traffic only.  __syncthreads() carries a release fence, and on this family
// stores and loads share vmcnt, so it drains every outstanding global load of the wave - which would empty a
// multi-stage prefetch pipeline at each barrier.  Here a wave waits for its own LDS operations (and for all but
// `vm_in_flight` of its vector-memory operations, 63 = no wait), then joins the barrier.
template <int VM_IN_FLIGHT = 63>
__device__ __forceinline__ void lds_barrier() {
  static_assert(VM_IN_FLIGHT >= 0 && VM_IN_FLIGHT < 64, "vmcnt is a 6-bit counter");
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0x0070 | (VM_IN_FLIGHT & 15) | ((VM_IN_FLIGHT >> 4) << 14));  // lgkmcnt(0)
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// tile index -> (tile_m, tile_n): tiles are numbered in groups of 4 m-tiles, m fastest inside a group, so that
// the tiles that run together on one XCD cover 4 activation tiles x a run of weight tiles
__device__ __forceinline__ void tile_coords(int t, int tiles_m, int tiles_n, int& tile_m, int& tile_n) {
  constexpr int GM = 4;
  const int group = t / (GM * tiles_n);
  const int first_m = group * GM;
  const int gsz = min(tiles_m - first_m, GM);
  const int tin = t - group * GM * tiles_n;
  tile_m = first_m + tin % gsz;
  tile_n = tin / gsz;
}

// scheduling barrier: the compiler moves nothing across it (used by the hand-ordered K loops here and in gemm_tile128.h)
#define SB() __builtin_amdgcn_sched_barrier(0)

// Work of a launch.  Tiles [0, tail_first) are computed whole.  The first `walkers` workgroups (a multiple of 8,
// at most one per CU) walk them: workgroup (xcd, c) takes tiles xcd*per_xcd + c, + walkers/8, ... of its XCD's
// contiguous run, and requests the first K block of its next tile before it writes the finished one out, so the
// new tile's first lines travel while the old tile leaves through LDS and neither a workgroup launch nor a cold
// first load sits between two tiles.  Tiles [tail_first, tiles) - the last, partial round over the chip's CUs - are
// either cut into `splits` K ranges that leave float partials in the workspace ([tile - tail_first][split][256 m]
// [256 n]) for tile_reduce_kernel, or (tail_halves) computed as two 128-row halves: the four waves of the lower
// half of the tile do the MFMAs (one per SIMD, so a K block takes half the matrix-core time), the other four only
// take part in the loads, and nothing has to be reduced afterwards.  Unit u of that tail goes to workgroup u after
// its walk (tail_shared: more whole tiles than CUs) or to workgroup walkers + u.
template <int MODE, int OUT_DT, int BIAS_DT>
__global__ __launch_bounds__(512, 1) void gemm_tile256_kernel(const GemmArgs p) {
  // the whole LDS: three weight stages (the weights travel two K blocks ahead: their lines come from HBM or the
  // memory-side cache) and two activation stages (one block ahead: mostly L2 hits)
  constexpr int kWStage = kTileN * kTileK, kXStage = kTileM * kTileK, kXBase = 3 * kWStage;
  __shared__ __attribute__((aligned(1024))) uint8_t smem[3 * kWStage + 2 * kXStage];

  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int wn = w & 1, wm = w >> 1;

  const int bid = blockIdx.x;
  // ---- this workgroup's items: the whole tiles of its walk, then at most one unit of the tail
  int walk_next = 0, walk_step = 1, walk_first = 0, walk_end = 0;
  if (bid < p.walkers) {
    const int per_xcd = (p.tail_first + 7) >> 3;
    walk_next = bid >> 3;
    walk_step = p.walkers >> 3;
    walk_first = (bid & 7) * per_xcd;
    walk_end = min(walk_first + per_xcd, p.tail_first);
  }
  int tail_unit = p.tail_shared ? bid : bid - p.walkers;
  {
    const int units = (p.tiles_m * p.tiles_n - p.tail_first) * (p.tail_halves ? 2 : p.splits);
    if (tail_unit >= units) tail_unit = -1;
  }
  struct Item { int t, split, half; bool is_split, is_half; };
  auto next_item = [&](Item& it) -> bool {
    if (walk_first + walk_next < walk_end) {
      it = Item{walk_first + walk_next, 0, 0, false, false};
      walk_next += walk_step;
      return true;
    }
    if (tail_unit >= 0) {
      if (p.tail_halves) it = Item{p.tail_first + (tail_unit >> 1), 0, tail_unit & 1, false, true};
      else it = Item{p.tail_first + tail_unit / p.splits, tail_unit % p.splits, 0, true, false};
      tail_unit = -1;
      return true;
    }
    return false;
  };
  Item item;
  if (!next_item(item)) return;

  // The LDS stages are two rings that run on across the items of a walk: K block b of an item sits in weight stage
  // (gw0 + b) % 3 and activation stage (gx0 + b) & 1, and the loads that would fall behind an item's last block fetch
  // the first blocks of the next item instead (its activation block 0 and its weight blocks 0 and 1 - the three requests
  // a fresh tile would otherwise wait for with nothing else to do).  `pref`: the item before requested them.
  int gw0 = 0, gx0 = 0;
  bool pref = false;
  for (;;) {
    const int t = item.t, split = item.split, half = item.half;
    const bool is_split = item.is_split, is_half = item.is_half;
    // The lane-dependent constants are derived anew for every tile from a lane id the compiler cannot see through:
    // hoisted out of the tile loop they would all stay live across it and push the K loop's operands into scratch.
    int ln = lane;
    asm volatile("" : "+v"(ln));
    // ---- lane constants of the global -> LDS loads and of the LDS -> MFMA operand fetches
    const int rl = ln >> 3, cp = ln & 7;
    uint32_t voW[2], voX[2];
#pragma unroll
    for (int par = 0; par < 2; ++par) {
      const int c = cp ^ ((par << 2) + (rl >> 1));
      voW[par] = (uint32_t)(rl * p.ldw + c * 16);
      voX[par] = (uint32_t)(rl * p.ldx + c * 16);
    }
    const uint32_t soW = (uint32_t)(w * 32 * p.ldw), soX = (uint32_t)(w * 32 * p.ldx);
    const uint32_t stepW = (uint32_t)(8 * p.ldw), stepX = (uint32_t)(8 * p.ldx);
    const int lr = ln & 31, h = ln >> 5;
    const int swz = (lr >> 1) & 7;
    // lane part of an operand fetch address: row lr of a 32-row group, 16-byte chunk (ks, j) at its swizzled place.
    // Stage, wave position and group are uniform and reach the address through scalar registers, so weights and
    // activations share these four registers.
    uint32_t fa[2][2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int j = 0; j < 2; ++j) fa[ks][j] = (uint32_t)(lr * kTileK + (((ks * 4 + h * 2 + j) ^ swz) << 4));
    auto frag = [&](const uint8_t* grp, int ks) -> v8i {  // grp: first row of the 32-row group inside its stage (uniform)
      const v4i lo = *reinterpret_cast<const v4i*>(grp + fa[ks][0]);
      const v4i hi = *reinterpret_cast<const v4i*>(grp + fa[ks][1]);
      v8i r;
      r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
      r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
      return r;
    };

    // ---- global -> LDS through buffer loads: descriptor at the tile's first row, rows past the matrix edge are out
    // of range and read as zero
    rsrc_t rW = make_rsrc(p.W, 0), rX = make_rsrc(p.X, 0);
    rsrc_t rWn = make_rsrc(p.W, 0), rXn = make_rsrc(p.X, 0);  // the item after this one (empty: every load is a no-op)
    auto tile_rsrcs = [&](rsrc_t& dW, rsrc_t& dX, int tile, int hf, bool halved, int kb0, int kb1) {
      int tm, tn;
      tile_coords(tile, p.tiles_m, p.tiles_n, tm, tn);
      const int mm = tm * kTileM + hf * (kTileM / 2), nn = tn * kTileN;
      const int rowsW = min(kTileN, p.N - nn), rowsX = min(halved ? kTileM / 2 : kTileM, p.M - mm);
      const int kbytes = (kb1 - kb0) * kTileK;  // the item's own K range: a request past it moves nothing
      dW = make_rsrc(p.W + (int64_t)nn * p.ldw + (int64_t)kb0 * kTileK, rowsX > 0 ? (uint32_t)((rowsW - 1) * p.ldw + kbytes) : 0u);
      dX = make_rsrc(p.X + (int64_t)mm * p.ldx + (int64_t)kb0 * kTileK, rowsX > 0 ? (uint32_t)((rowsX - 1) * p.ldx + kbytes) : 0u);
    };

    int tile_m, tile_n;
    tile_coords(t, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * kTileM + half * (kTileM / 2), n0 = tile_n * kTileN;
    if (m0 >= p.M) {                                                    // upper half of a tile past the last row
      wait_vm0();  // requests of the item before may still point at the stages
      return;
    }
    const int nrows = is_half ? min(p.M, m0 + kTileM / 2) : p.M;        // exclusive bound of a valid output row

    const int kb_begin = is_split ? split * p.kb_per_split : 0;
    const int kb_end = is_split ? min(p.K / kTileK, kb_begin + p.kb_per_split) : p.K / kTileK;
    const int nkb = kb_end - kb_begin;

    auto slot_at = [&](int i) -> int { return m0 + i; };
    tile_rsrcs(rW, rX, t, half, is_half, kb_begin, kb_end);
    // the item after this one: with three and more K blocks here its first blocks are requested by this item's last trips
    Item next;
    const bool has_next = next_item(next);
    const bool stream = has_next && nkb >= 3;
    if (has_next) {
      const int nb0 = next.is_split ? next.split * p.kb_per_split : 0;
      const int nb1 = next.is_split ? min(p.K / kTileK, nb0 + p.kb_per_split) : p.K / kTileK;
      tile_rsrcs(rWn, rXn, next.t, next.half, next.is_half, nb0, nb1);
    }
    const rsrc_t rWs = stream ? rWn : make_rsrc(p.W, 0), rXs = stream ? rXn : make_rsrc(p.X, 0);
    // one 1 KB global->LDS load (slice j of the wave's 32 rows) of K block kstep into weight stage ws / activation
    // stage xst; a block behind the item's last one is the next item's block kstep - nkb.  The whole offset travels in
    // the bounds-checked per-lane operand (a uniform offset operand is exempt from the range check, and rows past the
    // matrix edge must read as zero, not touch memory).
    auto LW = [&](int j, int kstep, int ws) {
      const bool nx = kstep >= nkb;
      buf_load16_to_lds(nx ? rWs : rW, voW[j & 1] + (soW + j * stepW + (uint32_t)(nx ? kstep - nkb : kstep) * kTileK), 0,
                        smem + ws * kWStage + w * 4096 + j * 1024);
    };
    auto LX = [&](int j, int kstep, int xst) {
      const bool nx = kstep >= nkb;
      buf_load16_to_lds(nx ? rXs : rX, voX[j & 1] + (soX + j * stepX + (uint32_t)(nx ? kstep - nkb : kstep) * kTileK), 0,
                        smem + kXBase + xst * kXStage + w * 4096 + j * 1024);
    };
    // stages of K block b of this item
    auto wst = [&](int b) -> int { return (gw0 + b) % 3; };
    auto xst = [&](int b) -> int { return (gx0 + b) & 1; };

    // ---- scales (block mode)
    // activation rows whose scales this lane applies (any valid row for padding lanes)
    const int mrow0 = min(m0 + wm * 64 + lr, p.M - 1);
    const int mrow1 = min(m0 + wm * 64 + 32 + lr, p.M - 1);
    // element offsets of this lane's two scale rows (32 bits: the host checks M * K/128 against 2^31)
    const uint32_t sxo0 = (uint32_t)((int64_t)mrow0 * p.sx_m + (int64_t)kb_begin * p.sx_k);
    const uint32_t sxo1 = (uint32_t)((int64_t)mrow1 * p.sx_m + (int64_t)kb_begin * p.sx_k);
    const uint32_t sxk = (uint32_t)p.sx_k;
    const int nb = min(n0 + wn * 128, p.N - 1) >> 7;
    const float* swp = p.sw + (int64_t)nb * p.sw_n + (int64_t)kb_begin * p.sw_k;
    // scaled mode: sx points at int32 words of four UE8M0 bytes (K blocks 4j..4j+3 of a row), sx_k = word stride
    const uint32_t* sqp = reinterpret_cast<const uint32_t*>(p.sx);
    const uint32_t sqo0 = (uint32_t)((int64_t)mrow0 * p.sx_m), sqo1 = (uint32_t)((int64_t)mrow1 * p.sx_m);
    int sq[2] = {127, 127}, sqw = 127;      // exponent bytes of the block the current MFMAs belong to
    uint32_t q0n = 0, q1n = 0;              // words holding the next block's activation exponents

    v16f acc[4][2];
#pragma unroll
    for (int ns = 0; ns < 4; ++ns)
#pragma unroll
      for (int ms = 0; ms < 2; ++ms)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[ns][ms][r] = 0.f;

    // Operand registers: X[ms][ks] the four activation fragments of a K block, W[ks] the two fragments of ONE weight
    // group.  A K block is walked as four steps, one per weight group ns, each step the MFMAs (ms, ks) = (0,0) (1,0)
    // (0,1) (1,1): W[0] is free after the second and W[1] after the fourth, and each is refilled in place with the
    // next group's fragment two MFMAs before its first use.  (A second set of weight registers would push the block
    // mode past 256 registers, and scratch reloads inside the K loop cannot coexist with its partial vmcnt waits.)
    v8i X[2][2], W[2];
    v16f tq[2];
    float sc[2] = {0.f, 0.f}, scn[2] = {0.f, 0.f};
    float s0n = 0.f, s1n = 0.f, sbn = 0.f;

    auto RW = [&](int ks, const uint8_t* st, int ns) { W[ks] = frag(st + (wn * 128 + ns * 32) * kTileK, ks); };
    auto RX = [&](int ms, int ks, const uint8_t* st) { X[ms][ks] = frag(st + (wm * 64 + ms * 32) * kTileK, ks); };
    // one MFMA of step ns.  Block mode: the products of a step gather in tq[ms] (K half 0 starts from zero, K half 1
    // adds), to be folded into acc[ns][ms] with the block's scale during the next step; the other modes accumulate
    // in place.
    auto M = [&](int ms, int ks, int ns) {
      if (MODE == kModeBlock) {
        if (ks == 0) {
          v16f z;
#pragma unroll
          for (int r = 0; r < 16; ++r) z[r] = 0.f;
          tq[ms] = mfma_32x32x64(W[0], X[ms][0], z);
        } else {
          tq[ms] = mfma_32x32x64(W[1], X[ms][1], tq[ms]);
        }
      } else if (MODE == kModeScaled) {
        acc[ns][ms] = mfma_32x32x64_scaled(W[ks], X[ms][ks], acc[ns][ms], sqw, sq[ms]);
      } else {
        acc[ns][ms] = mfma_32x32x64(W[ks], X[ms][ks], acc[ns][ms]);
      }
    };
    // the 16 scale-FMAs that fold a finished product into its accumulator (block mode only)
    auto F = [&](v16f& a, const v16f& tt, float sv) {
      if (MODE == kModeBlock) {
#pragma unroll
        for (int r = 0; r < 16; ++r) a[r] = __builtin_fmaf(tt[r], sv, a[r]);
      }
    };

    if (nkb <= 0) {
      wait_vm0();
      return;
    }
    if (is_half && wm >= 2) {
      // half tile (always a workgroup's last item): the waves of the upper 128 rows issue their share of the weight loads
      // and keep the barriers.  Their activation rows are out of range: those loads would move nothing and still take
      // their turn in the CU's address unit, so they are not issued (nobody reads those rows of the stage)
      if (!pref) {
#pragma unroll
        for (int j = 0; j < 4; ++j) LW(j, 0, wst(0));
#pragma unroll
        for (int j = 0; j < 4; ++j) LW(j, 1, wst(1));
      }
      wait_vm0();
      __syncthreads();
#pragma unroll
      for (int j = 0; j < 4; ++j) LW(j, 2, wst(2));
      int w_ld = wst(0), w_rd = wst(1);
      for (int it = 0; it < nkb - 1; ++it) {
        lds_barrier<4>();
        SB();
#pragma unroll
        for (int j = 0; j < 4; ++j) LW(j, it + 3, w_ld);
        w_ld = w_rd;
        w_rd = w_rd == 2 ? 0 : w_rd + 1;
      }
      wait_vm0();
      lds_barrier();  // the others' barrier in front of the write-out
      return;
    }
    // ---- prologue: blocks 0 and 1 into their stages, steps 0..2 of block 0.  Activation block 0 and weight blocks 0
    // and 1 of every item but a workgroup's first were requested by the item before.
    if (!pref) {
#pragma unroll
      for (int j = 0; j < 4; ++j) LX(j, 0, xst(0));
#pragma unroll
      for (int j = 0; j < 4; ++j) LW(j, 0, wst(0));
#pragma unroll
      for (int j = 0; j < 4; ++j) LW(j, 1, wst(1));
    }
    if (MODE == kModeBlock) { sc[0] = p.sx[sxo0]; sc[1] = p.sx[sxo1]; const float sb = swp[0]; sc[0] *= sb; sc[1] *= sb; }
    auto exponents = [&](uint32_t w0, uint32_t w1, float sb, int kb_abs) {  // -> sq, sqw for K block kb_abs
      const int sh = (kb_abs & 3) * 8;
      sq[0] = (int)(w0 >> sh);
      sq[1] = (int)(w1 >> sh);
      sqw = (int)(__float_as_uint(sb) >> 23);
    };
    if (MODE == kModeScaled) exponents(sqp[sqo0 + (uint32_t)(kb_begin >> 2) * sxk], sqp[sqo1 + (uint32_t)(kb_begin >> 2) * sxk], swp[0], kb_begin);
    wait_vm0();
    __syncthreads();
    // scales of block 1, then activations of block 1, weights of blocks 1 and 2: the order the loop keeps, so that at
    // a barrier only a wave's four youngest loads - weights for the block after next - may still be in flight
    if (MODE == kModeBlock) { const int kn = min(1, nkb - 1); s0n = p.sx[sxo0 + (uint32_t)kn * sxk]; s1n = p.sx[sxo1 + (uint32_t)kn * sxk]; sbn = swp[(int64_t)kn * p.sw_k]; }
    if (MODE == kModeScaled) {
      const int kn = min(1, nkb - 1);
      q0n = sqp[sqo0 + (uint32_t)((kb_begin + kn) >> 2) * sxk]; q1n = sqp[sqo1 + (uint32_t)((kb_begin + kn) >> 2) * sxk]; sbn = swp[(int64_t)kn * p.sw_k];
    }
    SB();
#pragma unroll
    for (int j = 0; j < 4; ++j) LX(j, 1, xst(1));
#pragma unroll
    for (int j = 0; j < 4; ++j) LW(j, 2, wst(2));
    const uint8_t* const stW0 = smem + wst(0) * kWStage;
    const uint8_t* const stX0 = smem + kXBase + xst(0) * kXStage;
    RX(0, 0, stX0); RX(1, 0, stX0); RW(0, stW0, 0);
    RX(0, 1, stX0); RX(1, 1, stX0); RW(1, stW0, 0);
    SB();
    // steps 0..2 of block 0
    M(0, 0, 0); SB();
    M(1, 0, 0); SB();
    RW(0, stW0, 1); SB();
    M(0, 1, 0); SB();
    M(1, 1, 0); SB();
    RW(1, stW0, 1); SB();
    F(acc[0][0], tq[0], sc[0]); SB();
    M(0, 0, 1); SB();
    F(acc[0][1], tq[1], sc[1]); SB();
    M(1, 0, 1); SB();
    RW(0, stW0, 2); SB();
    M(0, 1, 1); SB();
    M(1, 1, 1); SB();
    RW(1, stW0, 2); SB();
    F(acc[1][0], tq[0], sc[0]); SB();
    M(0, 0, 2); SB();
    F(acc[1][1], tq[1], sc[1]); SB();
    M(1, 0, 2); SB();
    RW(0, stW0, 3); SB();
    M(0, 1, 2); SB();
    M(1, 1, 2); SB();
    RW(1, stW0, 3); SB();
    // pending: F(acc[2][0], tq[0], sc[0]), F(acc[2][1], tq[1], sc[1])

    int w_ld = wst(0), w_rd = wst(1);  // weight stages: the one block it left (refilled with block it+3), the one of block it+1
    for (int it = 0; it < nkb - 1; ++it) {
      const uint8_t* stW = smem + w_rd * kWStage;                     // block it+1
      const uint8_t* stX = smem + kXBase + xst(it + 1) * kXStage;
      const int xl = xst(it);                                         // activation stage block it left
      lds_barrier<4>();  // block it+1 has landed; the weights of block it+2 may still be on their way
      SB();
      // Two waves share a SIMD's matrix pipe.  Left to the arbiter, one of them is served first whenever both are ready,
      // runs ahead and then sits at the barrier while the other works through most of its block alone - and one wave
      // alone cannot keep the pipe busy (its products wait for their own scale FMAs).  The issue priority therefore falls
      // with a wave's progress through the trip: whoever is behind goes first, and the two stay interleaved.
      __builtin_amdgcn_s_setprio(3);
      // ---- step 3 of block it; every operand register is refilled from block it+1 after its last use
      F(acc[2][0], tq[0], sc[0]); SB();
      M(0, 0, 3); SB();
      RX(0, 0, stX); LX(0, it + 2, xl); LX(1, it + 2, xl); SB();
      F(acc[2][1], tq[1], sc[1]); SB();
      M(1, 0, 3); SB();
      RX(1, 0, stX); RW(0, stW, 0); LX(2, it + 2, xl); LX(3, it + 2, xl); SB();
      M(0, 1, 3); SB();
      RX(0, 1, stX); SB();
      M(1, 1, 3); SB();
      RX(1, 1, stX); RW(1, stW, 0); SB();
      __builtin_amdgcn_s_setprio(2);
      if (MODE == kModeBlock) { scn[0] = s0n * sbn; scn[1] = s1n * sbn; }
      // ---- step 0 of block it+1; the pending products still belong to block it
      F(acc[3][0], tq[0], sc[0]); SB();
      if (MODE == kModeScaled) exponents(q0n, q1n, sbn, kb_begin + it + 1);  // the MFMAs from here on are block it+1's
      M(0, 0, 0); SB();
      F(acc[3][1], tq[1], sc[1]); SB();
      M(1, 0, 0); SB();
      // the scales of block it+2 are requested after the activation loads and before the weight loads: the wait in
      // front of their use then leaves exactly the weight loads in flight
      if (MODE == kModeBlock) {
        sc[0] = scn[0]; sc[1] = scn[1];
        const int kn = min(it + 2, nkb - 1);
        s0n = p.sx[sxo0 + (uint32_t)kn * sxk]; s1n = p.sx[sxo1 + (uint32_t)kn * sxk]; sbn = swp[(int64_t)kn * p.sw_k];
      }
      if (MODE == kModeScaled) {
        const int kn = min(it + 2, nkb - 1);
        q0n = sqp[sqo0 + (uint32_t)((kb_begin + kn) >> 2) * sxk]; q1n = sqp[sqo1 + (uint32_t)((kb_begin + kn) >> 2) * sxk]; sbn = swp[(int64_t)kn * p.sw_k];
      }
      SB();
      RW(0, stW, 1); LW(0, it + 3, w_ld); LW(1, it + 3, w_ld); SB();
      M(0, 1, 0); SB();
      M(1, 1, 0); SB();
      RW(1, stW, 1); LW(2, it + 3, w_ld); LW(3, it + 3, w_ld); SB();
      __builtin_amdgcn_s_setprio(1);
      // ---- steps 1 and 2 of block it+1
      F(acc[0][0], tq[0], sc[0]); SB();
      M(0, 0, 1); SB();
      F(acc[0][1], tq[1], sc[1]); SB();
      M(1, 0, 1); SB();
      RW(0, stW, 2); SB();
      M(0, 1, 1); SB();
      M(1, 1, 1); SB();
      RW(1, stW, 2); SB();
      __builtin_amdgcn_s_setprio(0);
      F(acc[1][0], tq[0], sc[0]); SB();
      M(0, 0, 2); SB();
      F(acc[1][1], tq[1], sc[1]); SB();
      M(1, 0, 2); SB();
      RW(0, stW, 3); SB();
      M(0, 1, 2); SB();
      M(1, 1, 2); SB();
      RW(1, stW, 3); SB();
      w_ld = w_rd;
      w_rd = w_rd == 2 ? 0 : w_rd + 1;
    }
    // ---- step 3 of the last block
    F(acc[2][0], tq[0], sc[0]); SB();
    M(0, 0, 3); SB();
    F(acc[2][1], tq[1], sc[1]); SB();
    M(1, 0, 3); SB();
    M(0, 1, 3); SB();
    M(1, 1, 3); SB();
    F(acc[3][0], tq[0], sc[0]);
    F(acc[3][1], tq[1], sc[1]);

    // Finished tiles leave through LDS so that every store instruction writes whole 256-byte row segments
    // (the accumulator layout alone gives 8 bytes per row per lane: 32 partial lines per instruction).
    // Each wave re-lays its own 64 x 128 block out, 32 rows at a time, in a private 8 KB slot of the weight or the
    // activation stage of the item's last block, 16-byte chunks XOR-swizzled by the row so that both the 8-byte writes
    // and the 16-byte reads spread over all banks; the other stages meanwhile receive the first blocks of the next item.
    const bool wide = !is_split && (p.ldc & 7) == 0 && (reinterpret_cast<uintptr_t>(p.C) & 15) == 0;
    // every wave has taken its last operands out of the stages.  The requests still in flight (the next item's first
    // blocks, or requests past the last block that move nothing) point at the stages AFTER the last block's, never at
    // the two the write-out uses.
    lds_barrier();
    const int ews = wst(nkb - 1), exs = xst(nkb - 1);  // the stages of the item's last block: free from here on
    if (has_next && !stream) {
      // an item of one or two K blocks has no trips to spare for it: the next item's first blocks are requested here
      SB();
#pragma unroll
      for (int j = 0; j < 4; ++j) buf_load16_to_lds(rXn, voX[j & 1] + (soX + j * stepX), 0, smem + kXBase + xst(nkb) * kXStage + w * 4096 + j * 1024);
#pragma unroll
      for (int j = 0; j < 4; ++j) buf_load16_to_lds(rWn, voW[j & 1] + (soW + j * stepW), 0, smem + wst(nkb) * kWStage + w * 4096 + j * 1024);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        buf_load16_to_lds(rWn, voW[j & 1] + (soW + j * stepW + (uint32_t)kTileK), 0, smem + wst(nkb + 1) * kWStage + w * 4096 + j * 1024);
      SB();
    }

    // value (ns, rg) of row slot ms of this lane, scaled / biased (row mode) and packed to two 16-bit pairs
    auto out_pair = [&](int ns, int ms, int rg, float sa) -> uint2 {
      const int n = n0 + wn * 128 + ns * 32 + rg * 8 + h * 4;
      float v[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) v[q] = acc[ns][ms][rg * 4 + q];
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

    if (wide) {
      uint8_t* ep = smem + (w < 4 ? ews * kWStage + w * 8192 : kXBase + exs * kXStage + (w - 4) * 8192);  // 32 rows x 256 B per pass
#pragma unroll
      for (int ms = 0; ms < 2; ++ms) {
        const int mrow = slot_at(wm * 64 + ms * 32 + lr);
        float sa = 1.f;
        if (MODE == kModeRow && mrow < nrows) sa = p.sx[mrow];
#pragma unroll
        for (int ns = 0; ns < 4; ++ns)
#pragma unroll
          for (int rg = 0; rg < 4; ++rg)
            *reinterpret_cast<uint2*>(ep + lr * 256 + (((ns * 4 + rg) ^ (lr & 15)) << 4) + h * 8) = out_pair(ns, ms, rg, sa);
        __builtin_amdgcn_wave_barrier();  // one wave's LDS accesses complete in order: no wait needed
        const int rr = ln >> 4, pc = ln & 15;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int r = i * 4 + rr;
          const uint4 o = *reinterpret_cast<const uint4*>(ep + r * 256 + ((pc ^ (r & 15)) << 4));
          const int m = slot_at(wm * 64 + ms * 32 + r);
          const int n = n0 + wn * 128 + (pc << 3);  // consecutive lanes store consecutive 16-byte chunks
          if (m < nrows && n < p.N) *reinterpret_cast<uint4*>((u16*)p.C + (int64_t)m * p.ldc + n) = o;
        }
        __builtin_amdgcn_wave_barrier();
      }
    } else {
#pragma unroll
      for (int ms = 0; ms < 2; ++ms) {
        const int ml = wm * 64 + ms * 32 + lr;  // row inside the tile
        const int m = slot_at(ml);               // output row
        if (m >= nrows) continue;
        const float sa = (MODE == kModeRow && !is_split) ? p.sx[m] : 1.f;
#pragma unroll
        for (int ns = 0; ns < 4; ++ns) {
#pragma unroll
          for (int rg = 0; rg < 4; ++rg) {
            const int n = n0 + wn * 128 + ns * 32 + rg * 8 + h * 4;
            if (n >= p.N) continue;
            if (is_split) {
              float* tile_part = p.partial + ((int64_t)(t - p.tail_first) * p.splits + split) * (kTileM * kTileN);
              *reinterpret_cast<float4*>(tile_part + ml * kTileN + (n - n0)) =
                  make_float4(acc[ns][ms][rg * 4], acc[ns][ms][rg * 4 + 1], acc[ns][ms][rg * 4 + 2], acc[ns][ms][rg * 4 + 3]);
            } else {
              *reinterpret_cast<uint2*>((u16*)p.C + (int64_t)m * p.ldc + n) = out_pair(ns, ms, rg, sa);
            }
          }
        }
      }
    }
    if (!has_next) {
      wait_vm0();  // requests that moved nothing still point at the stages: let them retire before the LDS goes back
      return;
    }
    item = next;
    pref = true;
    gw0 = wst(nkb);
    gx0 = xst(nkb);
  }
}


// Work item of a grouped (MoE) launch.  The number of blocks in use is device data; each XCD (workgroup id mod 8)
// takes a contiguous run of those blocks, cut into windows of four.  Inside a window the blocks of one expert form
// a group whose workgroups walk the blocks first and the n tiles second, so the workgroups that stream the same
// weight tile are dispatched together and meet in L2 instead of fetching it once each.  The window's expert ids
// are fetched with four independent loads: a workgroup starts with two dependent memory round trips (block count,
// then the window) before it knows its tile, not one per neighbour it compares with.
struct MoeItem {
  int mb;       // block of token slots, -1: nothing to do
  int tile_n;
  int expert;
};
// blocks in use (a device-side count: the host sizes the grid for the worst case)
__device__ __forceinline__ int moe_blocks_used(const GemmArgs& p) { return min(p.num_post_pad[0] / p.block_m, p.m_blocks); }
__device__ __forceinline__ MoeItem moe_work_item(const GemmArgs& p, int bid, int used) {
  constexpr int kWin = 4;
  MoeItem it{-1, 0, -1};
  const int per_xcd = (used + 7) >> 3;
  const int j = bid >> 3;
  const int pos = j / p.tiles_n;                      // block position inside the XCD's run, before regrouping
  if (pos >= per_xcd) return it;
  const int first_blk = (bid & 7) * per_xcd, end_blk = min(first_blk + per_xcd, used);
  if (first_blk + pos >= end_blk) return it;
  const int w0 = pos & ~(kWin - 1);                   // first position of the window
  int e[kWin];
#pragma unroll
  for (int i = 0; i < kWin; ++i) e[i] = first_blk + w0 + i < end_blk ? p.expert_ids[first_blk + w0 + i] : -2 - i;
  const int pi = pos - w0;
  int a = 0, b = kWin, ex = e[0];                     // group [a, b) of the window that holds position pi
#pragma unroll
  for (int i = 1; i < kWin; ++i) {
    if (e[i] != e[i - 1]) {
      if (i <= pi) { a = i; ex = e[i]; }
      else if (b == kWin) b = i;
    }
  }
  const int g = b - a;
  const int r = j - (w0 + a) * p.tiles_n;             // slot inside the group: 0 .. g*tiles_n-1
  it.tile_n = r / g;
  it.mb = first_blk + w0 + a + (r - it.tile_n * g);
  it.expert = ex;
  return it;
}
__device__ __forceinline__ MoeItem moe_work_item(const GemmArgs& p, int bid) { return moe_work_item(p, bid, moe_blocks_used(p)); }

// ------------------------------------------------------------------------------------------------
// Weight-streaming kernel for 33..128 activation rows: 256(n) x TM(m) x 128(k) tile, TM in {64, 128}.
// Used for small dense batches (with split-K through a float workspace so that every CU streams a share
// of the weights) and for the grouped MoE GEMM, where a block of up to TM token slots belongs to one
// expert and activation / output rows go through sorted_token_ids.  These shapes sit under the chip's
// ridge (2*TM FLOP per weight byte), so the design point is bytes in flight, not MFMA occupancy:
// NSTAGE LDS stages of [W 32 KB | X TM*128 B] are kept full with partial vmcnt waits and an LDS-only
// barrier per K block.  NW = 8 waves: each owns 32 weight rows x all TM rows (the form in use).  NW = 16
// waves: 8 along n x 2 along m, each 32 weight rows x TM/2 rows; it measured 5-8 % slower on the MoE shapes
// (more LDS operand traffic per MFMA) and is kept as a tuning option.
// ------------------------------------------------------------------------------------------------
template <int TM, int NSTAGE, int NW, int MODE, int OUT_DT, int BIAS_DT, bool SPLIT, bool MOE>
__global__ __launch_bounds__(NW * 64, 1) void gemm_stream_kernel(const GemmArgs p) {
  static_assert((TM == 64 || TM == 128) && (NW == 8 || NW == 16), "gemm_stream_kernel: unsupported shape");
  constexpr int MH = NW / 8;                     // waves along m
  constexpr int MS = TM / 32 / MH;               // 32-row activation sub-tiles per wave
  constexpr int WL = 32 / NW;                    // W wave-loads (8 rows each) per wave per stage
  constexpr int XG = TM / 8;                     // 8-row groups of the X tile
  constexpr int XL = (XG + NW - 1) / NW;         // X wave-loads per wave per stage
  constexpr int LPW = WL + XL;                   // LDS-DMA loads per wave per stage
  constexpr int WBYTES = kTileN * kTileK;
  // block mode: the scales of a K block travel with its stage (TM activation scales, then one weight scale per wave)
  constexpr int SOFF = WBYTES + TM * kTileK;
  constexpr int STAGE = SOFF + (MODE == kModeBlock ? 1024 : 0);
  __shared__ __attribute__((aligned(1024))) uint8_t smem[NSTAGE * STAGE + 1024];
  uint8_t* const dummy = smem + NSTAGE * STAGE;  // landing zone of padding loads

  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int wn = w & 7, wm = w >> 3;             // wave position: 32 weight rows, half of the m rows

  // ---- work item.  Workgroup ids are dealt round-robin to the 8 XCDs (one L2 each).
  // Dense: each XCD takes a contiguous run of items, consecutive ids walk the m blocks of one n tile.
  // Grouped: see moe_work_item().
  int bid = blockIdx.x;
  int split = 0;
  int mb, tile_n;
  int expert = 0;
  if (MOE) {
    const MoeItem item = moe_work_item(p, bid);
    if (item.mb < 0) return;
    mb = item.mb; tile_n = item.tile_n; expert = item.expert;
  } else {
    const int nitems = p.tiles_n * p.m_blocks;
    const int per_xcd = (nitems + 7) >> 3;
    if (SPLIT) { split = bid % p.splits; bid /= p.splits; }
    const int t = (bid & 7) * per_xcd + (bid >> 3);
    if (t >= nitems) return;
    mb = t % p.m_blocks;
    tile_n = t / p.m_blocks;
  }
  const int n0 = tile_n * kTileN;
  const int block_m = MOE ? p.block_m : TM;
  const int slot0 = mb * block_m;
  const int nrows = MOE ? p.num_valid : p.M;  // exclusive bound of a valid slot

  const int kb_begin = SPLIT ? split * p.kb_per_split : 0;
  const int kb_end = SPLIT ? min(p.K / kTileK, kb_begin + p.kb_per_split) : p.K / kTileK;
  const int nkb = kb_end - kb_begin;

  // ---- output rows of this lane (block row = wm*TM/2 + ms*32 + lane%32)
  const int lr = lane & 31, h = lane >> 5;
  const int mrow0 = wm * (TM / MH);
  int out_slot[MS];
  bool out_ok[MS];
#pragma unroll
  for (int ms = 0; ms < MS; ++ms) {
    const int r = mrow0 + ms * 32 + lr;
    out_slot[ms] = MOE ? (r < block_m ? p.sorted_ids[slot0 + r] : nrows) : slot0 + r;
    out_ok[ms] = out_slot[ms] < nrows;
  }

  if (MOE && expert < 0) {  // expert lives on another rank: the reference writes zeros
#pragma unroll
    for (int ms = 0; ms < MS; ++ms) {
      if (!out_ok[ms]) continue;
      for (int j = 0; j < 4; ++j) {
        const int n = n0 + wn * 32 + h * 16 + j * 4;
        if (n < p.N) store4<OUT_DT>(p.C, (int64_t)out_slot[ms] * p.ldc + n, 0.f, 0.f, 0.f, 0.f);
      }
    }
    return;
  }

  // ---- global -> LDS: wave load g of W covers rows g*8 .. g*8+7 (lane: row lane/8, chunk lane%8, stored at
  // chunk position c ^ ((row>>1)&7)); the whole offset travels in the bounds-checked per-lane operand
  const uint8_t* Wb = p.W + (MOE ? (int64_t)expert * p.w_expert_stride : 0);
  const int rowsW = min(kTileN, p.N - n0);
  const int kbytes = p.K - kb_begin * kTileK;
  const rsrc_t rW = make_rsrc(Wb + (int64_t)n0 * p.ldw + (int64_t)kb_begin * kTileK, (uint32_t)((rowsW - 1) * p.ldw + kbytes));
  // activations: one descriptor over every row; a padded slot points past the range and reads zeros
  const int64_t xrows = MOE ? (int64_t)((p.num_valid + p.top_k - 1) / p.top_k) : (int64_t)p.M;
  const rsrc_t rX = make_rsrc(p.X + (int64_t)kb_begin * kTileK, (uint32_t)((xrows - 1) * p.ldx + kbytes));
  const int rl = lane >> 3, cp = lane & 7;
  uint32_t voW[WL];
#pragma unroll
  for (int j = 0; j < WL; ++j) {
    const int g = w * WL + j;
    voW[j] = (uint32_t)((g * 8 + rl) * p.ldw + ((cp ^ (((g & 1) << 2) + (rl >> 1))) * 16));
  }
  uint32_t voX[XL];
  bool xload[XL];
  auto issue_w = [&](int kstep) {
    uint8_t* base = smem + (kstep % NSTAGE) * STAGE;
    const uint32_t ko = (uint32_t)kstep * kTileK;
#pragma unroll
    for (int j = 0; j < WL; ++j) buf_load16_to_lds(rW, voW[j] + ko, 0, base + (w * WL + j) * 1024);
  };
  auto issue_x = [&](int kstep) {
    uint8_t* base = smem + (kstep % NSTAGE) * STAGE;
    const uint32_t ko = (uint32_t)kstep * kTileK;
#pragma unroll
    for (int j = 0; j < XL; ++j)
      buf_load16_to_lds(rX, voX[j] + ko, 0, xload[j] ? base + WBYTES + (w * XL + j) * 1024 : dummy);
  };
  // Scales (block mode) go through the stage as well: two 4-byte LDS loads per wave and K block - lanes 0..TM/NW-1
  // fetch the activation scales of the wave's share of the rows, lane 0 the wave's weight scale.  As part of the
  // stage they are covered by the stage's wait; held in registers across trips instead, the compiler's copies
  // between the trips wait for loads of the running trip, and with loads returning in order that drains the
  // stage requested before them.
  constexpr int SR = TM / NW;  // activation scale rows per wave
  rsrc_t rSx, rSw;
  uint32_t voS = 0xF0000000u;
  auto issue_s = [&](int kstep) {
    if (MODE != kModeBlock) return;
    uint8_t* base = smem + (kstep % NSTAGE) * STAGE + SOFF;
    if (lane < SR) buf_load4_to_lds(rSx, voS, (uint32_t)kstep * (uint32_t)(p.sx_k * 4), base + w * (SR * 4));
    if (lane == 0) buf_load4_to_lds(rSw, 0u, (uint32_t)kstep * (uint32_t)(p.sw_k * 4), base + TM * 4 + w * 4);
  };
  auto issue = [&](int kstep) { issue_s(kstep); issue_w(kstep); issue_x(kstep); };
  // Grouped: the slot table is fetched first and the weights of the first stages behind it (loads retire in order:
  // the table arrives without waiting for the weights, and the weights do not wait for the table).
  int sid[XL];
#pragma unroll
  for (int j = 0; j < XL; ++j) {
    const int grp = w * XL + j;             // 8-row group of the X tile
    xload[j] = grp < XG;                    // wave-uniform
    const int row = grp * 8 + rl;
    sid[j] = nrows;
    if (xload[j] && row < block_m) sid[j] = MOE ? p.sorted_ids[slot0 + row] : slot0 + row;
  }
  if (MOE) {
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < NSTAGE - 1; ++s) issue_w(s);
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int j = 0; j < XL; ++j) {
    const int grp = w * XL + j;
    const int c = cp ^ (((grp & 1) << 2) + (rl >> 1));
    const bool ok = sid[j] < nrows;
    const int64_t xr = MOE ? sid[j] / p.top_k : sid[j];
    voX[j] = ok ? (uint32_t)(xr * p.ldx + c * 16) : 0xF0000000u;
  }

  // ---- LDS -> MFMA operands
  const int swz = (lr >> 1) & 7;
  uint32_t co[2][2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int j = 0; j < 2; ++j) co[ks][j] = (uint32_t)(((ks * 4 + h * 2 + j) ^ swz) << 4);
  const uint32_t rdW = (uint32_t)((wn * 32 + lr) * kTileK);
  const uint32_t rdX = (uint32_t)(WBYTES + (mrow0 + lr) * kTileK);
  auto frag = [&](const uint8_t* st, uint32_t rowoff, int ks) -> v8i {
    const v4i lo = *reinterpret_cast<const v4i*>(st + rowoff + co[ks][0]);
    const v4i hi = *reinterpret_cast<const v4i*>(st + rowoff + co[ks][1]);
    v8i r;
    r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
    r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
    return r;
  };

  // ---- scales (block mode): activation scale rows follow the activation rows
  if (MODE == kModeBlock) {
    const int row = w * SR + lane;  // the lane's row of the block (lanes 0..SR-1)
    int64_t xr = -1;
    if (lane < SR && row < block_m) {
      const int s = MOE ? p.sorted_ids[slot0 + row] : slot0 + row;
      if (s < nrows) xr = (MOE && p.sx_sorted) ? slot0 + row : (MOE ? s / p.top_k : s);
    }
    const int64_t srows = (MOE && p.sx_sorted) ? (int64_t)p.m_blocks * block_m : xrows;
    const int kb_all = p.K / kTileK;
    // rows past the range (padding) read zeros; the host keeps the tensor below the marker offset
    rSx = make_rsrc(p.sx + (int64_t)kb_begin * p.sx_k, (uint32_t)(((srows - 1) * p.sx_m + (int64_t)(kb_all - 1 - kb_begin) * p.sx_k + 1) * 4));
    voS = xr >= 0 ? (uint32_t)(xr * p.sx_m * 4) : 0xF0000000u;
    const int nb = min(n0 + wn * 32, p.N - 1) >> 7;
    const float* swp = p.sw + (MOE ? (int64_t)expert * p.sw_expert_stride : 0) + (int64_t)nb * p.sw_n + (int64_t)kb_begin * p.sw_k;
    rSw = make_rsrc(swp, (uint32_t)(((int64_t)(kb_all - 1 - kb_begin) * p.sw_k + 1) * 4));
  }

  v16f acc[MS];
#pragma unroll
  for (int ms = 0; ms < MS; ++ms)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[ms][r] = 0.f;

#pragma unroll
  for (int s = 0; s < NSTAGE - 1; ++s) {
    if (MOE) { issue_s(s); issue_x(s); }  // the weights of these stages are on their way already
    else issue(s);
  }
  constexpr int SL = MODE == kModeBlock ? 2 : 0;  // scale loads per wave and trip
  if (MOE) wait_vm0();  // the grouped prologue issues its loads in another order than the trips' partial waits assume

  // one K block
  auto trip = [&](auto na, int it) {
    constexpr int NA = decltype(na)::value;  // 32-row groups of the wave that hold real rows (grouped form)
    // stage `it` has landed once at most NSTAGE-2 younger trips (stage + scale loads each) are still in flight
    constexpr int kInFlight = (NSTAGE - 2) * (LPW + SL);
    lds_barrier<kInFlight>();
    __builtin_amdgcn_sched_barrier(0);  // nothing of this trip in front of the barrier
    issue(it + NSTAGE - 1);  // refills the stage every wave finished before this barrier
    if (NA == 0) return;
    const uint8_t* st = smem + (it % NSTAGE) * STAGE;
    float sc[MS];
    if (MODE == kModeBlock) {
      const float* ss = reinterpret_cast<const float*>(st + SOFF);
      const float sb = ss[TM + w];
#pragma unroll
      for (int ms = 0; ms < MS; ++ms) sc[ms] = ss[mrow0 + ms * 32 + lr] * sb;
    }
    v8i wf[2];
    wf[0] = frag(st, rdW, 0);
    wf[1] = frag(st, rdW, 1);
#pragma unroll
    for (int ms = 0; ms < NA; ++ms) {
      const v8i x0 = frag(st, rdX + ms * 32 * kTileK, 0);
      const v8i x1 = frag(st, rdX + ms * 32 * kTileK, 1);
      if (MODE == kModeBlock) {
        v16f z;
#pragma unroll
        for (int r = 0; r < 16; ++r) z[r] = 0.f;
        v16f tq = mfma_32x32x64(wf[0], x0, z);
        tq = mfma_32x32x64(wf[1], x1, tq);
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[ms][r] = __builtin_fmaf(tq[r], sc[ms], acc[ms][r]);
      } else {
        acc[ms] = mfma_32x32x64(wf[0], x0, acc[ms]);
        acc[ms] = mfma_32x32x64(wf[1], x1, acc[ms]);
      }
    }
  };
  auto run = [&](auto na) {
    int it = 0;
    for (; it + 1 < nkb; it += 2) {
      trip(na, it);
      trip(na, it + 1);
    }
    if (it < nkb) trip(na, it);
  };
  // Grouped form: the 32-row groups past an expert's last slot are padding (real slots come first in a block) and
  // skip their MFMAs; one straight-line copy of the loop per group count.
  int nact = MS;
  if (MOE) {
    nact = 0;
#pragma unroll
    for (int ms = 0; ms < MS; ++ms) nact += __builtin_amdgcn_readfirstlane(out_slot[ms]) < nrows ? 1 : 0;
  }
  if (!MOE || nact == MS) run(std::integral_constant<int, MS>{});
  else if (MS > 2 && nact == 3) run(std::integral_constant<int, (MS > 2 ? 3 : MS)>{});
  else if (MS > 2 && nact == 2) run(std::integral_constant<int, 2>{});
  else if (nact == 1) run(std::integral_constant<int, 1>{});
  else run(std::integral_constant<int, 0>{});
  // routed weights and the output rows of the store loop, fetched while the stages drain
  const bool wide = !SPLIT && (p.ldc & 7) == 0 && (reinterpret_cast<uintptr_t>(p.C) & 15) == 0;
  float rsw[MS];
  int srow[TM / NW / 2];
  if (MOE) {
#pragma unroll
    for (int ms = 0; ms < MS; ++ms) rsw[ms] = (p.topk_w && out_ok[ms]) ? p.topk_w[out_slot[ms]] : 1.f;
#pragma unroll
    for (int i = 0; i < TM / NW / 2; ++i) {
      const int row = w * (TM / NW) + i * 2 + (lane >> 5);
      srow[i] = (wide && row < block_m) ? p.sorted_ids[slot0 + row] : nrows;
    }
  }
  wait_vm0();  // drain the padding loads before the LDS allocation is released

  // ---- epilogue.  Finished 16-bit tiles leave through LDS ([TM rows][256 n], 512 B per row, 16-byte chunks
  // XOR-swizzled by the row) so that every store instruction writes two whole 512-byte row segments instead
  // of 8 bytes in each of 32 rows.
  if (wide) {
    lds_barrier();  // every wave has left the stages
#pragma unroll
    for (int ms = 0; ms < MS; ++ms) {
      const int row = mrow0 + ms * 32 + lr;
      float rs = 1.f;
      if (MODE == kModeRow && out_ok[ms]) rs = p.sx[out_slot[ms]];
      if (MOE) rs = rsw[ms];
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const int n = n0 + wn * 32 + rg * 8 + h * 4;
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = acc[ms][rg * 4 + r];
        if (MODE == kModeRow) {
          float4 sb = make_float4(0.f, 0.f, 0.f, 0.f);
          if (n < p.N) sb = *reinterpret_cast<const float4*>(p.sw + n);
          v[0] = v[0] * sb.x * rs; v[1] = v[1] * sb.y * rs; v[2] = v[2] * sb.z * rs; v[3] = v[3] * sb.w * rs;
          if (p.bias && n < p.N) {
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] += load_scalar<BIAS_DT>(p.bias, n + r);
          }
        } else if (MOE) {
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] *= rs;
        }
        uint2 o;
        if (OUT_DT == FP8K_BF16) {
          o.x = pack_bf16x2(v[0], v[1]);
          o.y = pack_bf16x2(v[2], v[3]);
        } else {
          o.x = f32_to_f16_bits(v[0]) | (f32_to_f16_bits(v[1]) << 16);
          o.y = f32_to_f16_bits(v[2]) | (f32_to_f16_bits(v[3]) << 16);
        }
        *reinterpret_cast<uint2*>(smem + row * 512 + (((wn * 4 + rg) ^ (row & 31)) << 4) + h * 8) = o;
      }
    }
    lds_barrier();
    const int rr = lane >> 5, pc = lane & 31;
#pragma unroll
    for (int i = 0; i < TM / NW / 2; ++i) {
      const int row = w * (TM / NW) + i * 2 + rr;
      const int slot = MOE ? srow[i] : slot0 + row;
      const int n = n0 + (pc << 3);
      const uint4 o = *reinterpret_cast<const uint4*>(smem + row * 512 + ((pc ^ (row & 31)) << 4));
      if (slot < nrows && n < p.N) *reinterpret_cast<uint4*>((u16*)p.C + (int64_t)slot * p.ldc + n) = o;
    }
    return;
  }
#pragma unroll
  for (int ms = 0; ms < MS; ++ms) {
    if (!out_ok[ms]) continue;
    const int64_t orow = out_slot[ms];
    float rs = 1.f;
    if (MODE == kModeRow && !SPLIT) rs = p.sx[orow];
    if (MOE) rs = rsw[ms];
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      const int n = n0 + wn * 32 + rg * 8 + h * 4;
      if (n >= p.N) continue;
      float v[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] = acc[ms][rg * 4 + r];
      if (SPLIT) {
        *reinterpret_cast<float4*>(p.partial + ((int64_t)split * p.M + orow) * p.N + n) = make_float4(v[0], v[1], v[2], v[3]);
      } else {
        if (MODE == kModeRow) {
          const float4 sb = *reinterpret_cast<const float4*>(p.sw + n);
          v[0] = v[0] * sb.x * rs; v[1] = v[1] * sb.y * rs; v[2] = v[2] * sb.z * rs; v[3] = v[3] * sb.w * rs;
          if (p.bias) {
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] += load_scalar<BIAS_DT>(p.bias, n + r);
          }
        } else if (MOE) {
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] *= rs;
        }
        store4<OUT_DT>(p.C, orow * p.ldc + n, v[0], v[1], v[2], v[3]);
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
// reduction of the K-cut tiles of gemm_tile256_kernel: 64 workgroups per tile, one float4 of 4 n per lane
// ------------------------------------------------------------------------------------------------
template <int MODE, int OUT_DT, int BIAS_DT>
__global__ __launch_bounds__(256) void tile_reduce_kernel(const GemmArgs p) {
  const int tl = blockIdx.x >> 6;
  int tile_m, tile_n;
  tile_coords(p.tail_first + tl, p.tiles_m, p.tiles_n, tile_m, tile_n);
  const int q = ((blockIdx.x & 63) << 8) + threadIdx.x;  // quad index inside the tile
  const int ml = q >> 6, nl = (q & 63) << 2;
  const int m = tile_m * kTileM + ml, n = tile_n * kTileN + nl;
  if (m >= p.M || n >= p.N) return;
  const float* src = p.partial + (int64_t)tl * p.splits * (kTileM * kTileN) + ml * kTileN + nl;
  float4 s = make_float4(0, 0, 0, 0);
  for (int k = 0; k < p.splits; ++k) {
    const float4 v = *reinterpret_cast<const float4*>(src + (int64_t)k * (kTileM * kTileN));
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
