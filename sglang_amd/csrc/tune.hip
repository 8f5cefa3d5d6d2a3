// Measurement aids of the fp8k library (declared in include/fp8k_tune.h): probes of what this machine gives the load
// path and the matrix cores, with none of a GEMM's other work around them.  Timed by the caller.
#include "gemm_kernels.h"

#include "../../include/fp8k_tune.h"

using namespace fp8k;

namespace fp8k {
// every workgroup reads its own contiguous share, a 32 KB stage per trip, two stages in flight
__global__ __launch_bounds__(512, 1) void stream_read_kernel(const uint8_t* __restrict__ src, int64_t share) {
  __shared__ __attribute__((aligned(1024))) uint8_t stage[2 * 32768];
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const uint8_t* base = src + (int64_t)blockIdx.x * share;
  const int trips = (int)(share >> 15);
  auto issue = [&](int t) {
    // the descriptor moves with the trip: a share may exceed the 4 GB a descriptor can span
    const rsrc_t r = make_rsrc(base + (int64_t)t * 32768, 32768u);
#pragma unroll
    for (int q = 0; q < 4; ++q)
      buf_load16_to_lds(r, (uint32_t)((w * 4 + q) * 1024 + lane * 16), 0, stage + (t & 1) * 32768 + (w * 4 + q) * 1024);
  };
  issue(0);
  if (trips > 1) issue(1);
  for (int t = 0; t < trips; ++t) {
    if (t + 1 < trips) lds_barrier<4>();
    else lds_barrier<0>();
    if (t + 2 < trips) issue(t + 2);
  }
  wait_vm0();
}
}  // namespace fp8k

namespace fp8k {
// The same stream in the shape a GEMM fetches an un-shuffled weight: a stage is one K block of a 256-row tile - 256
// pieces of 128 bytes, `pitch` bytes apart - and a workgroup walks the K blocks of its tiles.  Wave w loads rows
// w * 32 .. w * 32 + 31 of the tile, 8 rows (1 KB) per instruction, as the tile kernels do.
__global__ __launch_bounds__(512, 1) void stream_read_tiles_kernel(const uint8_t* __restrict__ src, int64_t pitch, int kblocks,
                                                                   int tiles_per_wg) {
  __shared__ __attribute__((aligned(1024))) uint8_t stage[2 * 32768];
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int trips = tiles_per_wg * kblocks;
  const uint32_t vo = (uint32_t)((lane >> 3) * pitch + (lane & 7) * 16);
  auto issue = [&](int t) {
    const int tile = blockIdx.x * tiles_per_wg + t / kblocks, kb = t % kblocks;
    // one descriptor per tile and K block: a tile of 256 rows may span more than a descriptor's 4 GB
    const rsrc_t r = make_rsrc(src + ((int64_t)tile * 256 + w * 32) * pitch + (int64_t)kb * 128, (uint32_t)(31 * pitch + 128));
#pragma unroll
    for (int q = 0; q < 4; ++q) buf_load16_to_lds(r, vo + (uint32_t)(q * 8 * pitch), 0, stage + (t & 1) * 32768 + (w * 4 + q) * 1024);
  };
  issue(0);
  if (trips > 1) issue(1);
  for (int t = 0; t < trips; ++t) {
    if (t + 1 < trips) lds_barrier<4>();
    else lds_barrier<0>();
    if (t + 2 < trips) issue(t + 2);
  }
  wait_vm0();
}
}  // namespace fp8k

extern "C" int fp8k_tune_stream_read_tiles(const void* src, int64_t rows, int64_t pitch, void* stream) {
  clear_error();
  const char* op = "tune_stream_read_tiles";
  FP8K_REQUIRE(src && aligned(src, 16), "%s: src must be a 16-byte aligned device pointer", op);
  FP8K_REQUIRE(rows >= 0 && pitch >= 128 && pitch % 128 == 0 && pitch < (1LL << 23), "%s: pitch must be a multiple of 128 below 8 MiB", op);
  const int ncu = num_cu();
  const int64_t tiles_per_wg = rows / 256 / ncu;
  if (tiles_per_wg == 0) return FP8K_OK;
  FP8K_REQUIRE(tiles_per_wg * (pitch / 128) < (1LL << 30), "%s: too many stages per workgroup", op);
  hipLaunchKernelGGL(stream_read_tiles_kernel, dim3((unsigned)ncu), dim3(512), 0, (hipStream_t)stream, (const uint8_t*)src, pitch,
                     (int)(pitch / 128), (int)tiles_per_wg);
  return check_launch(op);
}

extern "C" int fp8k_tune_stream_read(const void* src, int64_t bytes, void* stream) {
  clear_error();
  FP8K_REQUIRE(bytes >= 0 && bytes < (1LL << 40), "tune_stream_read: bad size");
  FP8K_REQUIRE(src && aligned(src, 16), "tune_stream_read: src must be a 16-byte aligned device pointer");
  const int ncu = num_cu();
  const int64_t share = bytes / ncu / 65536 * 65536;
  if (share == 0) return FP8K_OK;
  hipLaunchKernelGGL(stream_read_kernel, dim3((unsigned)ncu), dim3(512), 0, (hipStream_t)stream, (const uint8_t*)src, share);
  return check_launch("tune_stream_read");
}

namespace fp8k {
// stream_read_kernel with a write-out after every `spt` stages ("a tile"): each wave stores `spw` times 1 KB (16 bytes a
// lane), the workgroup 8 KB x spw, to a place of its own in dst - the shape of a GEMM that streams weights and writes
// a small output tile per weight tile
__global__ __launch_bounds__(512, 1) void stream_read_write_kernel(const uint8_t* __restrict__ src, int64_t share,
                                                                   uint8_t* __restrict__ dst, int spt, int spw) {
  __shared__ __attribute__((aligned(1024))) uint8_t stage[2 * 32768];
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const uint8_t* base = src + (int64_t)blockIdx.x * share;
  const int trips = (int)(share >> 15);
  const int tiles = trips / spt;
  auto issue = [&](int t) {
    const rsrc_t r = make_rsrc(base + (int64_t)t * 32768, 32768u);
#pragma unroll
    for (int q = 0; q < 4; ++q)
      buf_load16_to_lds(r, (uint32_t)((w * 4 + q) * 1024 + lane * 16), 0, stage + (t & 1) * 32768 + (w * 4 + q) * 1024);
  };
  issue(0);
  if (trips > 1) issue(1);
  int t = 0;
  for (int ti = 0; ti < tiles; ++ti) {
    for (int k = 0; k < spt; ++k, ++t) {
      // stores and loads retire in order: a wait that leaves this wave's four youngest loads in flight has seen every
      // store issued before them complete
      if (t + 1 < trips) lds_barrier<4>();
      else lds_barrier<0>();
      if (t + 2 < trips) issue(t + 2);
    }
    uint4* o = reinterpret_cast<uint4*>(dst + ((((int64_t)blockIdx.x * tiles + ti) * 8 + w) * spw) * 1024) + lane;
    const uint4 v = make_uint4(1u, 2u, 3u, (unsigned)ti);
    for (int i = 0; i < spw; ++i) o[i * 64] = v;
  }
  wait_vm0();
}
}  // namespace fp8k

extern "C" int fp8k_tune_stream_read_write(const void* src, int64_t bytes, void* dst, int64_t dst_bytes, int64_t stages_per_tile,
                                           int64_t stores_per_wave, void* stream) {
  clear_error();
  FP8K_REQUIRE(bytes >= 0 && bytes < (1LL << 40), "tune_stream_read_write: bad size");
  FP8K_REQUIRE(src && aligned(src, 16) && dst && aligned(dst, 16), "tune_stream_read_write: src and dst must be 16-byte aligned device pointers");
  FP8K_REQUIRE(stages_per_tile >= 1 && stages_per_tile <= 4096 && stores_per_wave >= 0 && stores_per_wave <= 64,
               "tune_stream_read_write: stages_per_tile in [1, 4096], stores_per_wave in [0, 64]");
  const int ncu = num_cu();
  const int64_t share = bytes / ncu / (32768 * stages_per_tile) * (32768 * stages_per_tile);  // whole tiles per workgroup
  if (share == 0) return FP8K_OK;
  const int64_t tiles = share / (32768 * stages_per_tile);
  FP8K_REQUIRE(dst_bytes >= (int64_t)ncu * tiles * 8 * stores_per_wave * 1024,
               "tune_stream_read_write: dst holds %lld bytes, %lld are written", (long long)dst_bytes,
               (long long)((int64_t)ncu * tiles * 8 * stores_per_wave * 1024));
  hipLaunchKernelGGL(stream_read_write_kernel, dim3((unsigned)ncu), dim3(512), 0, (hipStream_t)stream, (const uint8_t*)src,
                     share, (uint8_t*)dst, (int)stages_per_tile, (int)stores_per_wave);
  return check_launch("tune_stream_read_write");
}


namespace fp8k {
// Bare matrix-core loop: every wave keeps two weight-side and four activation-side operand fragments of the caller's
// bytes in registers and issues the eight independent products of them, `iters` times over, into eight accumulators -
// no loads, no LDS, no barriers inside the loop.  One workgroup of 8 waves per CU (two waves per SIMD, the occupancy
// of the tile kernels).  The accumulators are folded into `sink` at the end so that the loop stays.
__global__ __launch_bounds__(512, 1) void mfma_peak_kernel(const uint8_t* __restrict__ operands, int64_t bytes, int iters,
                                                           float* __restrict__ sink) {
  const int lane = threadIdx.x & 63;
  const int64_t frag0 = ((int64_t)blockIdx.x * 8 + (threadIdx.x >> 6)) * 6;  // 6 fragments of 64 lanes x 32 bytes per wave
  const int64_t nfrag = bytes / 2048;
  v8i a[2], b[4];
#pragma unroll
  for (int i = 0; i < 6; ++i) {
    const v8i v = *reinterpret_cast<const v8i*>(operands + ((frag0 + i) % nfrag) * 2048 + lane * 32);
    if (i < 2) a[i] = v;
    else b[i - 2] = v;
  }
  v16f acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = mfma_32x32x64(a[i], b[j], acc[i][j]);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) s += acc[i][j][r];
  sink[(int64_t)blockIdx.x * 512 + threadIdx.x] = s;
}
}  // namespace fp8k

namespace fp8k {
// The K loop of the 256x256 block-scaled tile kernel built up from the bare MFMA loop, one ingredient at a time, on
// operands that never change (LDS filled once, the stage loads fetch a small cache-resident range), so that what each
// ingredient costs the matrix cores can be read off:
//   FORM 1  the block-scaled product form: two MFMAs into a short-lived accumulator, folded into the long-lived one by 16
//           scale FMAs placed behind the first MFMAs of the next product (8 products = 16 MFMAs per K block, as a wave of
//           the tile kernel has them)
//   FORM 2  + the operand fragments refilled from LDS behind their last use (24 ds_read_b128 per wave and K block)
//   FORM 3  + one LDS-only workgroup barrier per K block
//   FORM 4  + the eight 1 KB stage loads per wave and K block (global -> LDS) and the partial vmcnt wait at the barrier
//   FORM 5  form 4 without the scale FMAs: the products accumulate in place, as in the row-scaled and the
//           hardware-scaled modes of the tile kernel
//   FORM 6  form 5 with 16 multiplies per 32x32 tile and K block in the place of the FMAs: what a loop would issue that
//           accumulates in place and multiplies the accumulators by the ratio of two consecutive blocks' scales
// The instruction order is the tile kernel's (steps 3, 0, 1, 2 of its loop).
template <int FORM>
__global__ __launch_bounds__(512, 1) void mfma_loop_kernel(const uint8_t* __restrict__ operands, int64_t bytes, int iters,
                                                           float* __restrict__ sink) {
  __shared__ __attribute__((aligned(1024))) uint8_t smem[5 * 32768];
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int wn = w & 1, wm = w >> 1;
  const uint32_t span = (uint32_t)std::min<int64_t>(bytes, 1 << 24) & ~65535u;  // the range the stage loads walk
  const rsrc_t r = make_rsrc(operands, span);
  for (int st = 0; st < 5; ++st)
#pragma unroll
    for (int q = 0; q < 4; ++q)
      buf_load16_to_lds(r, (uint32_t)(((blockIdx.x * 5 + st) * 32768 + (w * 4 + q) * 1024 + lane * 16) % span), 0,
                        smem + st * 32768 + (w * 4 + q) * 1024);
  wait_vm0();
  __syncthreads();
  // a fragment = 64 lanes x 32 bytes, kept as two conflict-free 1 KB halves; a weight stage holds 16 of them, an
  // activation stage 16
  auto frag = [&](const uint8_t* base) -> v8i {
    const v4i lo = *reinterpret_cast<const v4i*>(base + lane * 16);
    const v4i hi = *reinterpret_cast<const v4i*>(base + 1024 + lane * 16);
    v8i f;
    f[0] = lo[0]; f[1] = lo[1]; f[2] = lo[2]; f[3] = lo[3];
    f[4] = hi[0]; f[5] = hi[1]; f[6] = hi[2]; f[7] = hi[3];
    return f;
  };
  v8i X[2][2], W[2];
  v16f acc[4][2], tq[2], z;
#pragma unroll
  for (int q = 0; q < 16; ++q) { z[q] = 0.f; tq[0][q] = 0.f; tq[1][q] = 0.f; }
#pragma unroll
  for (int ns = 0; ns < 4; ++ns)
#pragma unroll
    for (int ms = 0; ms < 2; ++ms)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[ns][ms][q] = 0.f;
  float sc[2] = {1.0f + lane * 1e-9f, 1.0f - lane * 1e-9f};
  W[0] = frag(smem + (wn * 8) * 2048); W[1] = frag(smem + (wn * 8 + 1) * 2048);
#pragma unroll
  for (int ms = 0; ms < 2; ++ms)
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) X[ms][ks] = frag(smem + 3 * 32768 + (wm * 4 + ms * 2 + ks) * 2048);
  // without the refills the operands would be loop constants, and the products with them: the register is passed through
  // an empty asm statement instead, which the compiler cannot see through
  auto RW = [&](int ks, const uint8_t* st, int ns) {
    if (FORM >= 2) {
      W[ks] = frag(st + (wn * 8 + ns * 2 + ks) * 2048);
    } else {
      int t = W[ks][0];
      asm volatile("" : "+v"(t));
      W[ks][0] = t;
    }
  };
  auto RX = [&](int ms, int ks, const uint8_t* st) { if (FORM >= 2) X[ms][ks] = frag(st + (wm * 4 + ms * 2 + ks) * 2048); };
  constexpr bool kFold = FORM != 5 && FORM != 6;
  int step_ns = 0;  // the accumulator row the in-place form is working on (a constant after unrolling)
  auto M = [&](int ms, int ks) {
    if (!kFold) acc[step_ns][ms] = mfma_32x32x64(W[ks], X[ms][ks], acc[step_ns][ms]);
    else if (ks == 0) tq[ms] = mfma_32x32x64(W[0], X[ms][0], z);
    else tq[ms] = mfma_32x32x64(W[1], X[ms][1], tq[ms]);
  };
  auto F = [&](v16f& a, const v16f& t, float sv) {
    if (FORM == 6) {
#pragma unroll
      for (int q = 0; q < 16; ++q) a[q] = a[q] * sv;
      return;
    }
    if (!kFold) return;
#pragma unroll
    for (int q = 0; q < 16; ++q) a[q] = __builtin_fmaf(t[q], sv, a[q]);
  };
  int w_ld = 0, w_rd = 1;
  for (int it = 0; it < iters; ++it) {
    const uint8_t* stW = smem + w_rd * 32768;
    const uint8_t* stX = smem + 3 * 32768 + ((it + 1) & 1) * 32768;
    uint8_t* const ldX = smem + 3 * 32768 + (it & 1) * 32768 + w * 4096;
    uint8_t* const ldW = smem + w_ld * 32768 + w * 4096;
    const uint32_t go = (uint32_t)(((blockIdx.x * 3 + it) * 65536) % span) + w * 4096 + lane * 16;
    auto LX = [&](int j) { if (FORM >= 4) buf_load16_to_lds(r, go + j * 1024, 0, ldX + j * 1024); };
    auto LW = [&](int j) { if (FORM >= 4) buf_load16_to_lds(r, go + 32768 + j * 1024, 0, ldW + j * 1024); };
    if (FORM >= 4) lds_barrier<4>();
    else if (FORM == 3) lds_barrier();
    SB();
    step_ns = 3;
    F(acc[2][0], tq[0], sc[0]); SB();
    M(0, 0); SB();
    RX(0, 0, stX); LX(0); LX(1); SB();
    F(acc[2][1], tq[1], sc[1]); SB();
    M(1, 0); SB();
    RX(1, 0, stX); RW(0, stW, 0); LX(2); LX(3); SB();
    M(0, 1); SB();
    RX(0, 1, stX); SB();
    M(1, 1); SB();
    RX(1, 1, stX); RW(1, stW, 0); SB();
    step_ns = 0;
    F(acc[3][0], tq[0], sc[0]); SB();
    M(0, 0); SB();
    F(acc[3][1], tq[1], sc[1]); SB();
    M(1, 0); SB();
    RW(0, stW, 1); LW(0); LW(1); SB();
    M(0, 1); SB();
    M(1, 1); SB();
    RW(1, stW, 1); LW(2); LW(3); SB();
    step_ns = 1;
    F(acc[0][0], tq[0], sc[0]); SB();
    M(0, 0); SB();
    F(acc[0][1], tq[1], sc[1]); SB();
    M(1, 0); SB();
    RW(0, stW, 2); SB();
    M(0, 1); SB();
    M(1, 1); SB();
    RW(1, stW, 2); SB();
    step_ns = 2;
    F(acc[1][0], tq[0], sc[0]); SB();
    M(0, 0); SB();
    F(acc[1][1], tq[1], sc[1]); SB();
    M(1, 0); SB();
    RW(0, stW, 3); SB();
    M(0, 1); SB();
    M(1, 1); SB();
    RW(1, stW, 3); SB();
    w_ld = w_rd;
    w_rd = w_rd == 2 ? 0 : w_rd + 1;
  }
  wait_vm0();
  float sum = tq[0][0] + tq[1][0];
#pragma unroll
  for (int ns = 0; ns < 4; ++ns)
#pragma unroll
    for (int ms = 0; ms < 2; ++ms)
#pragma unroll
      for (int q = 0; q < 16; ++q) sum += acc[ns][ms][q];
  sink[(int64_t)blockIdx.x * 512 + threadIdx.x] = sum;
}
}  // namespace fp8k

extern "C" int fp8k_tune_mfma_loop(const void* operands, int64_t bytes, int64_t iters, int form, float* sink,
                                   int64_t sink_floats, int64_t* flops, void* stream) {
  clear_error();
  const char* op = "tune_mfma_loop";
  FP8K_REQUIRE(operands && aligned(operands, 32), "%s: operands must be a 32-byte aligned device pointer", op);
  FP8K_REQUIRE(bytes >= (1 << 20) && bytes < (1LL << 40), "%s: at least 1 MiB of operand bytes is needed", op);
  FP8K_REQUIRE(iters >= 1 && iters <= (1 << 24), "%s: iters must be in [1, 2^24]", op);
  FP8K_REQUIRE(form >= 1 && form <= 6, "%s: form must be 1..6", op);
  const int ncu = num_cu();
  FP8K_REQUIRE(sink && sink_floats >= (int64_t)ncu * 512, "%s: sink must hold %lld floats", op, (long long)ncu * 512);
  if (flops) *flops = (int64_t)ncu * 8 * iters * 16 * (2LL * 32 * 32 * 64);
  const dim3 grid((unsigned)ncu), block(512);
  hipStream_t st = (hipStream_t)stream;
  const uint8_t* o = (const uint8_t*)operands;
  switch (form) {
    case 1: hipLaunchKernelGGL(mfma_loop_kernel<1>, grid, block, 0, st, o, bytes, (int)iters, sink); break;
    case 2: hipLaunchKernelGGL(mfma_loop_kernel<2>, grid, block, 0, st, o, bytes, (int)iters, sink); break;
    case 3: hipLaunchKernelGGL(mfma_loop_kernel<3>, grid, block, 0, st, o, bytes, (int)iters, sink); break;
    case 4: hipLaunchKernelGGL(mfma_loop_kernel<4>, grid, block, 0, st, o, bytes, (int)iters, sink); break;
    case 5: hipLaunchKernelGGL(mfma_loop_kernel<5>, grid, block, 0, st, o, bytes, (int)iters, sink); break;
    default: hipLaunchKernelGGL(mfma_loop_kernel<6>, grid, block, 0, st, o, bytes, (int)iters, sink); break;
  }
  return check_launch(op);
}

extern "C" int fp8k_tune_mfma_peak(const void* operands, int64_t bytes, int64_t iters, float* sink, int64_t sink_floats,
                                   int64_t* flops, void* stream) {
  clear_error();
  const char* op = "tune_mfma_peak";
  FP8K_REQUIRE(operands && aligned(operands, 32), "%s: operands must be a 32-byte aligned device pointer", op);
  FP8K_REQUIRE(bytes >= 2048 && bytes < (1LL << 40), "%s: at least 2048 operand bytes are needed", op);
  FP8K_REQUIRE(iters >= 1 && iters <= (1 << 24), "%s: iters must be in [1, 2^24]", op);
  const int ncu = num_cu();
  FP8K_REQUIRE(sink && sink_floats >= (int64_t)ncu * 512, "%s: sink must hold %lld floats", op, (long long)ncu * 512);
  if (flops) *flops = (int64_t)ncu * 8 * iters * 8 * (2LL * 32 * 32 * 64);
  hipLaunchKernelGGL(mfma_peak_kernel, dim3((unsigned)ncu), dim3(512), 0, (hipStream_t)stream, (const uint8_t*)operands, bytes,
                     (int)iters, sink);
  return check_launch(op);
}
