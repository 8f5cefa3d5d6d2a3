// Host side of the FP8 GEMM entry points: argument checks mirrored from the reference ops, kernel
// choice, launch.  No allocation, no synchronisation.
#include <algorithm>
#include <atomic>
#include <mutex>

#include "gemm_direct.h"
#include "gemm_tile128.h"

#include "../../include/fp8k_tune.h"

namespace fp8k {

struct Plan {
  int kind;    // 0 = generic, 1 = tile256, 2 = weight-streaming through LDS (33..128 rows), 3 = direct (<= 32 rows),
               // 4 = tile128, 5 = direct with K cut across the waves of a workgroup (<= 32 rows, N below 16 K)
  int splits;  // >1: split-K through the float workspace
  int kb_per_split;
  int tm;      // rows per block of the streaming kernels
  int tail_first;   // tile256: first tile that is cut along K or into halves (== number of tiles when none is)
  int halves;       // tile256: the tiles from tail_first on are computed as two 128-row halves
  int64_t ws_bytes; // float workspace the plan needs
};

// tuning aid: force the kernel family (and the K split of the uniform-split families) of later calls made by the
// calling thread; other threads keep the automatic choice
static thread_local int g_force_kind = -1, g_force_splits = 0;
static thread_local int g_tail_halves = 1;  // tuning aid: 0 keeps the last round of 256x256 tiles whole

static Plan plan_tile128(int64_t M, int64_t N, int kb, int splits) {
  Plan pl{4, 1, 0, 0, 0, 0};
  if (splits > kb) splits = kb;
  if (splits < 1) splits = 1;
  pl.kb_per_split = (kb + splits - 1) / splits;
  pl.splits = (kb + pl.kb_per_split - 1) / pl.kb_per_split;
  pl.ws_bytes = pl.splits > 1 ? (int64_t)pl.splits * M * N * 4 : 0;
  return pl;
}

// decode-sized, up to 32 rows: weights go HBM -> registers -> matrix core.  K is cut so that about 512 workgroups
// (two per CU, one round) stream at once, at least 8 K blocks each, while the float partials stay a small fraction
// of the weight bytes
static Plan plan_direct(int64_t M, int64_t N, int64_t K) {
  Plan pl{3, 1, 0, 0, 0, 0};
  const int kb = (int)(K / kTileK);
  pl.tm = M <= 16 ? 16 : 32;
  const int64_t tiles_n = (N + kDirTileN - 1) / kDirTileN;
  int64_t splits = std::max<int64_t>(1, 512 / tiles_n);
  splits = std::min<int64_t>(splits, std::max<int64_t>(1, kb / kDirDepth));
  splits = std::min<int64_t>(splits, std::max<int64_t>(1, K / (64 * M)));
  // 128 and more n tiles keep half the CUs streaming on their own: no K cut and no reduction launch (18432 x 7168:
  // 26.6 us against 28.6 us with three cuts; two cuts, 288 workgroups, leave the CUs unevenly loaded: 33 us)
  if (tiles_n >= 128) splits = 1;
  // a share of 9 or 10 K blocks is one full prefetch round of 8 and a round for the one or two left over: one more cut
  // gives every workgroup a single shorter round (7168 x 2304, 18 K blocks: 10.2 -> 8.5 us at M = 1 with three cuts)
  while (splits > 1 && splits < kb) {
    const int64_t per = (kb + splits - 1) / splits;
    if (per > kDirDepth && per % kDirDepth >= 1 && per % kDirDepth <= 2 && (kb + splits) / (splits + 1) >= 4) ++splits;
    else break;
  }
  if (g_force_kind == 3 && g_force_splits > 0) splits = std::min<int64_t>(g_force_splits, kb);  // tuning aid
  const int kbps = (int)((kb + splits - 1) / splits);
  pl.kb_per_split = kbps;
  pl.splits = (kb + kbps - 1) / kbps;
  pl.ws_bytes = pl.splits > 1 ? (int64_t)pl.splits * M * N * 4 : 0;
  return pl;
}

// decode-sized with fewer than 128 tiles of 128 weight rows: a workgroup owns 16 (or 32) weight rows and its waves cut
// K between them, so that every CU streams without float partials in memory or a reduction launch.  `splits` stays 1
// (nothing goes through the workspace); kb_per_split is the K range of one wave, tm reuses the row-count slot, and
// the number of waves along n travels in `halves`.
constexpr int64_t kWaveKMaxN = 16384;
static Plan plan_wavek(int64_t M, int64_t N, int64_t K) {
  Plan pl{5, 1, 0, 0, 0, 0};
  const int kb = (int)(K / kTileK);
  pl.tm = M <= 16 ? 16 : 32;
  // waves along n: the choice that leaves the busiest CU the fewest weight rows (workgroups go two to a CU at most);
  // among equals the widest workgroup whose waves still get at most 16 K blocks each (measured: wider workgroups
  // re-read less of the activations, longer per-wave K ranges start to serialise)
  int nw = 1;
  int64_t best_rows = -1;
  for (int cand = 1; cand <= 4; cand *= 2) {
    const int64_t wgs = (N + 16 * cand - 1) / (16 * cand);
    if (wgs > 2 * (int64_t)num_cu() && cand < 4) continue;
    const int64_t rows = (wgs + num_cu() - 1) / num_cu() * 16 * cand;
    const int per_wave = (kb + 8 / cand - 1) / (8 / cand);
    if (best_rows < 0 || rows < best_rows || (rows == best_rows && per_wave <= 16)) { best_rows = rows; nw = cand; }
  }
  if (g_force_kind == 5 && (g_force_splits == 1 || g_force_splits == 2 || g_force_splits == 4 || g_force_splits == 8))
    nw = g_force_splits;  // tuning aid
  pl.halves = nw;
  pl.kb_per_split = (kb + 8 / nw - 1) / (8 / nw);
  return pl;
}
// Which of the two decode kernels: every workgroup of the wave-cut kernel reads all of the activations' K range for its
// 16 * nw weight rows, so its traffic through the CUs' load path grows with the rows of the batch; the workgroup-cut
// kernel shares the activations among 128 weight rows but pays float partials and a reduction launch.  Measured
// (M = 1 .. 32 on the DeepSeek-V3 and Llama projection shapes): the wave cut wins for up to 8 rows, and for up to 32
// rows while the weights are at most about 24 MB.
static bool prefers_wavek(int64_t M, int64_t N, int64_t K) {
  if (N >= kWaveKMaxN) return false;  // 128 and more tiles of 128 rows: the workgroup-cut kernel runs uncut
  return M <= 8 || N * K <= (24LL << 20);
}

// up to 128 rows: stream the weights once, every CU takes a K slice of one 256-row weight tile
static Plan plan_stream(int64_t M, int64_t N, int64_t K) {
  Plan pl{2, 1, 0, 0, 0, 0};
  const int kb = (int)(K / kTileK);
  pl.tm = M <= 64 ? 64 : 128;
  const int64_t tiles_n = (N + kTileN - 1) / kTileN;
  int splits = (int)(256 / tiles_n);
  if (splits > kb / 4) splits = kb / 4;
  if (splits < 1) splits = 1;
  pl.kb_per_split = (kb + splits - 1) / splits;
  pl.splits = (kb + pl.kb_per_split - 1) / pl.kb_per_split;
  pl.ws_bytes = pl.splits > 1 ? (int64_t)pl.splits * M * N * 4 : 0;
  return pl;
}

// One workgroup (one CU) per 256x256 tile.  The tiles of the last, partial round over the CUs are cut along K
// so that the round keeps every CU busy for 1/splits of a tile time (>= 4 K blocks per piece).
static Plan plan_tile256(int64_t M, int64_t N, int64_t K) {
  Plan pl{1, 1, 0, 0, 0, 0};
  const int kb = (int)(K / kTileK);
  const int64_t tiles = ((M + kTileM - 1) / kTileM) * ((N + kTileN - 1) / kTileN);
  const int64_t rest = tiles % num_cu();
  int splits = rest ? (int)(num_cu() / rest) : 1;
  if (splits > kb / 4) splits = kb / 4;
  if (splits < 1) splits = 1;
  // With at least one full round before it, the cut only pays when the tile time it saves (about 2 us per K block)
  // outweighs writing and re-reading the float partials (256 KB per piece): measured break-even.
  if (tiles > num_cu() && kb * (splits - 1) * 8 <= rest * splits * splits) splits = 1;
  pl.kb_per_split = (kb + splits - 1) / splits;
  pl.splits = (kb + pl.kb_per_split - 1) / pl.kb_per_split;
  pl.tail_first = (int)(pl.splits > 1 ? tiles - rest : tiles);
  pl.ws_bytes = pl.splits > 1 ? rest * pl.splits * (int64_t)(kTileM * kTileN) * 4 : 0;
  // A last round that fills at most half the CUs and is not worth a K cut: its tiles run as two 128-row halves, one
  // workgroup each (half the matrix-core time per K block, nothing to reduce).
  if (pl.splits == 1 && tiles > num_cu() && rest > 0 && rest <= num_cu() / 2 && M > kTileM / 2 && g_tail_halves) {
    pl.halves = 1;
    pl.tail_first = (int)(tiles - rest);
  }
  return pl;
}

// the plan without the 128x128 tile kernel: direct / streaming / 256x256 tiles by the number of rows
static Plan plan_base(int64_t M, int64_t N, int64_t K) {
  const bool fits32 = M * K < (1LL << 31);
  if (g_force_kind == 3 && M <= 32 && fits32) return plan_direct(M, N, K);
  if (g_force_kind == 5 && M <= 32 && fits32) return plan_wavek(M, N, K);
  if (g_force_kind == 2 && M <= 128 && fits32) return plan_stream(M, N, K);
  if (g_force_kind == 1) return plan_tile256(M, N, K);
  if (M <= 32 && fits32 && prefers_wavek(M, N, K)) return plan_wavek(M, N, K);
  if (M <= 32 && fits32) return plan_direct(M, N, K);
  if (M <= 128 && fits32) return plan_stream(M, N, K);
  return plan_tile256(M, N, K);
}


// Rough device-time models in microseconds, fitted to sweeps over M = 48..2048 on the DeepSeek-V3 and Llama
// projection shapes; they only have to rank the two candidates where the gap is large.
//  * 128x128 tiles: a workgroup spends 0.42 us per K block when its operands come out of the L2, up to 0.72 us
//    when every CU streams lines that are new to the chip (the share of such lines falls with the number of
//    tiles that share a weight or activation tile); first loads + tile write-out 2.5 us per round of tiles,
//    launch 1 us; more than two rounds are left to the 256x256 kernel, two rounds measure about 15 % over the
//    model; a K cut adds the reduction launch (4 us) and the float partials (written and read back at about
//    5 TB/s).
//  * streaming kernel: 10-11 us fixed, the weights once at 5.5 TB/s, its partials at about 8 TB/s.
//  * 256x256 tiles: 1.6 us per K block and tile, 8 us fixed, 6 us + partials (8 TB/s) for a cut last round.
static double est_tile128(int64_t M, int64_t N, int kb, int* best_splits) {
  const int64_t tm = (M + kT128 - 1) / kT128, tn = (N + kT128 - 1) / kT128;
  const int64_t tiles = tm * tn;
  const double cold = std::min(1.0, 1.0 / (double)tm + 1.0 / (double)tn);
  double best = 1e30;
  for (int s = 1; s <= 8; ++s) {
    if (s > 1 && (s > kb / 4 || tiles * s > 256)) break;  // a K cut stays within one round of workgroups
    const int64_t wgs = tiles * s;
    const int64_t rounds = (wgs + num_cu() - 1) / num_cu();
    if (rounds > 2) break;
    const int kbps = (kb + s - 1) / s;
    const double tb = 0.42 + 0.30 * cold * std::min(1.0, (double)wgs / num_cu());
    double t = 1.0 + (double)rounds * (kbps * tb + 2.5);
    if (rounds == 2) t *= 1.15;
    if (s > 1) t += 4.0 + (double)s * M * N * 8.0 / 5e6;
    if (t < best) { best = t; *best_splits = s; }
  }
  return best;
}

static double est_base(const Plan& pl, int64_t M, int64_t N, int64_t K) {
  const int kb = (int)(K / kTileK);
  if (pl.kind == 2)
    return (M <= 64 ? 10.0 : 11.0) + (double)N * K / 5.5e6 + (pl.splits > 1 ? (double)pl.splits * M * N * 8.0 / 8e6 : 0.0);
  const int64_t tiles = ((M + kTileM - 1) / kTileM) * ((N + kTileN - 1) / kTileN);
  if (pl.splits == 1) return 8.0 + (double)((tiles + num_cu() - 1) / num_cu()) * kb * 1.6;
  const int64_t rest = tiles % num_cu();
  return 8.0 + (double)(tiles / num_cu()) * kb * 1.6 + pl.kb_per_split * 1.6 + 6.0 +
         (double)rest * pl.splits * (kTileM * kTileN * 4) * 2.0 / 8e6;
}

static Plan make_plan(int64_t M, int64_t N, int64_t K) {
  Plan pl{0, 1, 0, 0, 0, 0};
  if (K % kTileK != 0 || N % 4 != 0) return pl;
  const int kb = (int)(K / kTileK);
  if (g_force_kind == 4 && N % 8 == 0) return plan_tile128(M, N, kb, g_force_splits);
  pl = plan_base(M, N, K);
  if (g_force_kind >= 0 || M <= 32 || N % 8 != 0 || (pl.kind != 1 && pl.kind != 2)) return pl;
  // a few hundred rows, or fewer 256x256 tiles than CUs: the 128x128 tile kernel when the model puts it ahead
  int s128 = 1;
  const double t128 = est_tile128(M, N, kb, &s128);
  if (t128 < 0.92 * est_base(pl, M, N, K)) return plan_tile128(M, N, kb, s128);
  return pl;
}

static int64_t workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  return make_plan(M, N, K).ws_bytes;
}

// Row-major activation scales ([M, K/128], the layout of the reference's Triton path) make every lane of a tile
// kernel's scale load touch a cache line of its own: 32 lines per load instead of one, which costs the 256x256
// kernel 17 % and the streaming kernel 20 %.  When the caller's workspace has room, the block GEMM first copies
// them into column-major order behind the float partials (a few microseconds for at most M*K/128 floats) and
// runs on the copy; fp8k_block_gemm_workspace_bytes counts that area for every call that could need it.
static int64_t align256(int64_t v) { return (v + 255) & ~(int64_t)255; }
static bool wants_scale_copy(const Plan& pl, int64_t M) { return M > 32 && (pl.kind == 1 || pl.kind == 2 || pl.kind == 4); }
static int64_t block_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const Plan pl = make_plan(M, N, K);
  return wants_scale_copy(pl, M) ? align256(pl.ws_bytes) + M * ((K + kTileK - 1) / kTileK) * 4 : pl.ws_bytes;
}
__global__ __launch_bounds__(256) void scale_to_column_major_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                                    int M, int kb, int64_t stride_m) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // m fastest: the writes are contiguous
  if (i >= (int64_t)M * kb) return;
  const int k = (int)(i / M), m = (int)(i - (int64_t)k * M);
  dst[i] = src[(int64_t)m * stride_m + k];
}

// the two tile kernels (plan kinds 1 and 4); `a` carries the operands, the plan the tiling
template <int MODE, int OUT_DT, int BIAS_DT>
static int launch_tiles(const GemmArgs& a0, const Plan& pl, hipStream_t st) {
  GemmArgs a = a0;
  a.tiles_m = (a.M + kTileM - 1) / kTileM;
  a.tiles_n = (a.N + kTileN - 1) / kTileN;
  a.splits = pl.splits;
  a.kb_per_split = pl.kb_per_split;
  if (pl.kind == 4) {
    a.tiles_m = (a.M + kT128 - 1) / kT128;
    a.tiles_n = (a.N + kT128 - 1) / kT128;
    const unsigned nwg = (unsigned)(((int64_t)a.tiles_m * a.tiles_n * pl.splits + 7) / 8 * 8);
    if (pl.splits == 1) {
      hipLaunchKernelGGL((gemm_tile128_kernel<MODE, OUT_DT, BIAS_DT, false>), dim3(nwg), dim3(512), 0, st, a);
      return check_launch("gemm_tile128");
    }
    hipLaunchKernelGGL((gemm_tile128_kernel<MODE, OUT_DT, BIAS_DT, true>), dim3(nwg), dim3(512), 0, st, a);
    int rc = check_launch("gemm_tile128");
    if (rc) return rc;
    const int64_t quads = (int64_t)a.M * (a.N / 4);
    hipLaunchKernelGGL((splitk_reduce_kernel<MODE, OUT_DT, BIAS_DT>), dim3((unsigned)((quads + 255) / 256)), dim3(256),
                       0, st, a);
    return check_launch("splitk_reduce");
  }
  const int ntiles = a.tiles_m * a.tiles_n;
  a.tail_first = pl.tail_first;
  a.tail_halves = pl.halves;
  const int ncu8 = std::max(8, num_cu() / 8 * 8);
  const int tail_units = (ntiles - pl.tail_first) * (pl.halves ? 2 : pl.splits);
  unsigned nwg;
  if (pl.tail_first > ncu8) {
    // more whole tiles than CUs: one walking workgroup per CU, which also takes a unit of the tail at the end
    a.walkers = ncu8;
    a.tail_shared = 1;
    nwg = (unsigned)std::max(ncu8, tail_units);
  } else {
    a.walkers = (pl.tail_first + 7) / 8 * 8;
    a.tail_shared = 0;
    nwg = (unsigned)(a.walkers + tail_units);
  }
  hipLaunchKernelGGL((gemm_tile256_kernel<MODE, OUT_DT, BIAS_DT>), dim3(nwg), dim3(512), 0, st, a);
  int rc = check_launch("gemm_tile256");
  if (rc || pl.tail_first == ntiles || pl.halves) return rc;
  hipLaunchKernelGGL((tile_reduce_kernel<MODE, OUT_DT, BIAS_DT>), dim3((unsigned)((ntiles - pl.tail_first) * 64)), dim3(256),
                     0, st, a);
  return check_launch("tile_reduce");
}

template <int MODE, int OUT_DT, int BIAS_DT>
static int launch(const GemmArgs& a0, const Plan& pl, hipStream_t st) {
  GemmArgs a = a0;
  if (pl.kind == 0) {
    dim3 grid((unsigned)((a.N + 63) / 64), (unsigned)((a.M + 3) / 4));
    hipLaunchKernelGGL((gemm_generic_kernel<MODE, OUT_DT, BIAS_DT>), grid, dim3(256), 0, st, a);
    return check_launch("gemm_generic");
  }
  a.tiles_m = (a.M + kTileM - 1) / kTileM;
  a.tiles_n = (a.N + kTileN - 1) / kTileN;
  a.splits = pl.splits;
  a.kb_per_split = pl.kb_per_split;
  if (pl.kind == 3) {
    a.m_blocks = 1;
    a.tiles_n = (a.N + kDirTileN - 1) / kDirTileN;
    const unsigned nwg = (unsigned)(a.tiles_n * pl.splits);
#define FP8K_DIRECT(TM)                                                                                             \
  do {                                                                                                              \
    if (pl.splits == 1)                                                                                             \
      hipLaunchKernelGGL((gemm_direct_kernel<TM, MODE, OUT_DT, BIAS_DT, false, false>), dim3(nwg), dim3(512), 0, st, a); \
    else                                                                                                            \
      hipLaunchKernelGGL((gemm_direct_kernel<TM, MODE, OUT_DT, BIAS_DT, true, false>), dim3(nwg), dim3(512), 0, st, a);  \
  } while (0)
    if (pl.tm == 16) FP8K_DIRECT(16);
    else FP8K_DIRECT(32);
#undef FP8K_DIRECT
    int rc = check_launch("gemm_direct");
    if (rc || pl.splits == 1) return rc;
    const int64_t quads = (int64_t)a.M * (a.N / 4);
    hipLaunchKernelGGL((splitk_reduce_kernel<MODE, OUT_DT, BIAS_DT>), dim3((unsigned)((quads + 255) / 256)), dim3(256),
                       0, st, a);
    return check_launch("splitk_reduce");
  }
  if (pl.kind == 5) {
    a.wk_nw = pl.halves;
    const unsigned nwg = (unsigned)((a.N + 16 * a.wk_nw - 1) / (16 * a.wk_nw));
    if (pl.tm == 16) hipLaunchKernelGGL((gemm_wavek_kernel<16, MODE, OUT_DT, BIAS_DT>), dim3(nwg), dim3(512), 0, st, a);
    else hipLaunchKernelGGL((gemm_wavek_kernel<32, MODE, OUT_DT, BIAS_DT>), dim3(nwg), dim3(512), 0, st, a);
    return check_launch("gemm_wavek");
  }
  if (pl.kind == 2) {
    a.m_blocks = 1;
    const unsigned nwg = (unsigned)(((a.tiles_n + 7) / 8) * 8 * pl.splits);
#define FP8K_STREAM(TM, NST, NW)                                                                                      \
  do {                                                                                                                \
    if (pl.splits == 1)                                                                                               \
      hipLaunchKernelGGL((gemm_stream_kernel<TM, NST, NW, MODE, OUT_DT, BIAS_DT, false, false>), dim3(nwg),           \
                         dim3(NW * 64), 0, st, a);                                                                    \
    else                                                                                                              \
      hipLaunchKernelGGL((gemm_stream_kernel<TM, NST, NW, MODE, OUT_DT, BIAS_DT, true, false>), dim3(nwg),            \
                         dim3(NW * 64), 0, st, a);                                                                    \
  } while (0)
    if (pl.tm == 64) FP8K_STREAM(64, 3, 8);
    else FP8K_STREAM(128, 3, 8);
#undef FP8K_STREAM
    int rc = check_launch("gemm_stream");
    if (rc || pl.splits == 1) return rc;
    const int64_t quads = (int64_t)a.M * (a.N / 4);
    hipLaunchKernelGGL((splitk_reduce_kernel<MODE, OUT_DT, BIAS_DT>), dim3((unsigned)((quads + 255) / 256)), dim3(256),
                       0, st, a);
    return check_launch("splitk_reduce");
  }
  return launch_tiles<MODE, OUT_DT, BIAS_DT>(a, pl, st);
}

static int common_checks(const char* op, const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                         int64_t lda, int64_t ldb, int64_t ldc, int out_dtype) {
  FP8K_REQUIRE(M >= 0 && N >= 0 && K >= 0, "%s: negative shape", op);
  FP8K_REQUIRE(M <= 0x7fffffffLL && N <= 0x7fffffffLL && K <= 0x7fffffffLL, "%s: shape too large", op);
  FP8K_REQUIRE(out_dtype == FP8K_F16 || out_dtype == FP8K_BF16, "%s: out_dtype must be Half or BFloat16", op);
  FP8K_REQUIRE(K % 16 == 0, "%s: mat_a must be multiple of 16 bytes for memory alignment", op);
  FP8K_REQUIRE((N * 2) % 16 == 0, "%s: out must be multiple of 16 bytes for memory alignment", op);
  FP8K_REQUIRE(lda >= K && ldb >= K && ldc >= N, "%s: leading dimension smaller than the row length", op);
  FP8K_REQUIRE(lda % 16 == 0 && ldb % 16 == 0 && (ldc * 2) % 8 == 0, "%s: rows must be 16-byte aligned", op);
  FP8K_REQUIRE(lda < (1LL << 23) && ldb < (1LL << 23) && K < (1LL << 23), "%s: rows longer than 8 MiB are not supported", op);
  if (M == 0 || N == 0) return FP8K_OK;
  FP8K_REQUIRE(A && B && C, "%s: null pointer", op);
  FP8K_REQUIRE(aligned(A, 16) && aligned(B, 16) && aligned(C, 8), "%s: operands must be 16-byte aligned", op);
  return FP8K_OK;
}

}  // namespace fp8k

using namespace fp8k;

extern "C" void fp8k_tune_force_gemm_plan(int kind, int splits) {
  g_tail_halves = kind != -2;  // -2: automatic choice with the last round of 256x256 tiles kept whole
  g_force_kind = kind == -2 ? -1 : kind;
  g_force_splits = splits;
}

extern "C" int64_t fp8k_block_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) { return block_gemm_workspace_bytes(M, N, K); }
extern "C" int64_t fp8k_scaled_mm_workspace_bytes(int64_t M, int64_t N, int64_t K) { return workspace_bytes(M, N, K); }

static int block_gemm_impl(const void* A, const void* B, const float* As, const float* Bs, void* C, int64_t M, int64_t N,
                           int64_t K, int64_t lda, int64_t ldb, int64_t as_stride_m, int64_t as_stride_k,
                           int64_t bs_stride_n, int64_t bs_stride_k, int64_t ldc, int out_dtype, void* workspace,
                           int64_t workspace_bytes_given, void* stream) {
  int rc = common_checks("fp8_blockwise_scaled_mm", A, B, C, M, N, K, lda, ldb, ldc, out_dtype);
  if (rc) return rc;
  if (M == 0 || N == 0) return FP8K_OK;
  FP8K_REQUIRE(K > 0, "fp8_blockwise_scaled_mm: K must be positive");
  FP8K_REQUIRE(As && Bs, "fp8_blockwise_scaled_mm: null scale pointer");
  FP8K_REQUIRE(as_stride_m >= 0 && as_stride_k >= 0 && bs_stride_n >= 0 && bs_stride_k >= 0,
               "fp8_blockwise_scaled_mm: negative scale stride");
  FP8K_REQUIRE((M - 1) * as_stride_m + ((K + kTileK - 1) / kTileK - 1) * as_stride_k < 0x38000000LL,
               "fp8_blockwise_scaled_mm: scales_a spans more than 3.5 GiB");
  const Plan pl = make_plan(M, N, K);
  const int64_t kb = (K + kTileK - 1) / kTileK;
  const int64_t need = wants_scale_copy(pl, M) ? align256(pl.ws_bytes) + M * kb * 4 : pl.ws_bytes;
  if (need > 0 && (!workspace || workspace_bytes_given < need))
    return fail(FP8K_ERR_WORKSPACE, "fp8_blockwise_scaled_mm: workspace of %lld bytes required, %lld given",
                (long long)need, (long long)(workspace ? workspace_bytes_given : 0));
  GemmArgs a{};
  a.X = (const uint8_t*)A; a.W = (const uint8_t*)B; a.sx = As; a.sw = Bs; a.bias = nullptr; a.C = C;
  a.partial = (float*)workspace;
  a.M = (int)M; a.N = (int)N; a.K = (int)K; a.ldx = lda; a.ldw = ldb; a.ldc = ldc;
  a.sx_m = as_stride_m; a.sx_k = as_stride_k; a.sw_n = bs_stride_n; a.sw_k = bs_stride_k;
  hipStream_t st = (hipStream_t)stream;
  if (wants_scale_copy(pl, M) && as_stride_k == 1 && as_stride_m > 1 && kb > 1) {
    float* cm = reinterpret_cast<float*>(static_cast<char*>(workspace) + align256(pl.ws_bytes));
    hipLaunchKernelGGL(scale_to_column_major_kernel, dim3((unsigned)((M * kb + 255) / 256)), dim3(256), 0, st, As, cm, (int)M,
                       (int)kb, as_stride_m);
    rc = check_launch("scale_to_column_major");
    if (rc) return rc;
    a.sx = cm; a.sx_m = 1; a.sx_k = M;
  }
  return out_dtype == FP8K_BF16 ? launch<kModeBlock, FP8K_BF16, FP8K_F32>(a, pl, st)
                                : launch<kModeBlock, FP8K_F16, FP8K_F32>(a, pl, st);
}

extern "C" int fp8k_block_gemm(const void* A, const void* B, const float* As, const float* Bs, void* C, int64_t M,
                               int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t as_stride_m, int64_t as_stride_k,
                               int64_t bs_stride_n, int64_t bs_stride_k, int64_t ldc, int out_dtype, void* workspace,
                               int64_t workspace_bytes_given, void* stream) {
  clear_error();
  return block_gemm_impl(A, B, As, Bs, C, M, N, K, lda, ldb, as_stride_m, as_stride_k, bs_stride_n, bs_stride_k, ldc,
                         out_dtype, workspace, workspace_bytes_given, stream);
}

// ---- the same GEMM for callers that cannot allocate: its scratch is a fixed array in device memory, one copy per GPU
// that loads this library, held until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; kernels and every other use take the device address that call returns, kept per device.
constexpr int64_t kStaticScratchBytes = 80ll << 20;  // 64 MiB of float partials (one 256x256 tile per CU) + 16 MiB of copied scales
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

static int static_scratch(void** out, hipStream_t stream) {
  constexpr int kMaxDev = 64;
  static std::mutex mu;
  static void* ptrs[kMaxDev];  // device address of `scratch` on each device, resolved on the first call there
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(FP8K_ERR_LAUNCH, "fp8k_block_gemm_noalloc: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDev) return fail(FP8K_ERR_UNSUPPORTED, "fp8k_block_gemm_noalloc: device index %d not supported", dev);
  // every GPU holds its own copy of the array: the copy used must be the one of the GPU the launches go to
  if (stream) {
    int sdev = -1;
    e = hipStreamGetDevice(stream, &sdev);
    if (e != hipSuccess) return fail(FP8K_ERR_LAUNCH, "fp8k_block_gemm_noalloc: hipStreamGetDevice: %s", hipGetErrorString(e));
    if (sdev != dev)
      return fail(FP8K_ERR_INVALID, "fp8k_block_gemm_noalloc: the stream belongs to device %d but device %d is current; make the "
                  "stream's device current before the call", sdev, dev);
  }
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    // the look-up is not a stream operation; under a capture it would break the capture, so it is refused there
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (stream && hipStreamIsCapturing(stream, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone)
      return fail(FP8K_ERR_UNSUPPORTED, "fp8k_block_gemm_noalloc: the first call on a device resolves the scratch address and "
                  "cannot run while the stream is capturing; make one call outside the capture first");
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return fail(FP8K_ERR_LAUNCH, "fp8k_block_gemm_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e));
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  return FP8K_OK;
}

extern "C" int fp8k_block_gemm_noalloc(const void* A, const void* B, const float* As, const float* Bs, void* C, int64_t M,
                                       int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t as_stride_m,
                                       int64_t as_stride_k, int64_t bs_stride_n, int64_t bs_stride_k, int64_t ldc,
                                       int out_dtype, void* stream) {
  clear_error();
  const int64_t need = block_gemm_workspace_bytes(M, N, K);
  if (need > kStaticScratchBytes)
    return fail(FP8K_ERR_WORKSPACE, "fp8k_block_gemm_noalloc: M=%lld N=%lld K=%lld needs %lld bytes of scratch, the built-in "
                "buffer holds %lld; use fp8k_block_gemm with a caller-owned workspace", (long long)M, (long long)N,
                (long long)K, (long long)need, (long long)kStaticScratchBytes);
  void* ws = nullptr;
  if (need > 0) {
    const int rc = static_scratch(&ws, (hipStream_t)stream);
    if (rc) return rc;
  }
  // nothing in the buffer has to start at zero: every float partial and every copied scale that a launch reads was
  // written by the same call
  return block_gemm_impl(A, B, As, Bs, C, M, N, K, lda, ldb, as_stride_m, as_stride_k, bs_stride_n, bs_stride_k, ldc,
                         out_dtype, ws, need > 0 ? kStaticScratchBytes : 0, stream);
}

extern "C" int fp8k_block_gemm_ue8m0(const void* A, const void* B, const int32_t* As_packed, const float* Bs, void* C,
                                     int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t as_stride_m,
                                     int64_t as_stride_w, int64_t bs_stride_n, int64_t bs_stride_k, int64_t ldc,
                                     int out_dtype, void* workspace, int64_t workspace_bytes_given, void* stream) {
  clear_error();
  const char* op = "block_gemm_ue8m0";
  int rc = common_checks(op, A, B, C, M, N, K, lda, ldb, ldc, out_dtype);
  if (rc) return rc;
  if (M == 0 || N == 0) return FP8K_OK;
  FP8K_REQUIRE(K > 0, "%s: K must be positive", op);
  FP8K_REQUIRE(As_packed && Bs, "%s: null scale pointer", op);
  FP8K_REQUIRE(as_stride_m >= 0 && as_stride_w >= 0 && bs_stride_n >= 0 && bs_stride_k >= 0, "%s: negative scale stride", op);
  FP8K_REQUIRE((M - 1) * as_stride_m + ((K + kTileK - 1) / kTileK / 4) * as_stride_w < (1LL << 31), "%s: scales span more than 2^31 elements", op);
  const Plan pl = make_plan(M, N, K);
  // the matrix core applies the scales only in the tile kernels; smaller problems take the float-scale
  // entry point with the exponents expanded to floats
  FP8K_REQUIRE(pl.kind == 1 || pl.kind == 4, "%s: built for M > 128 with K a multiple of 128 (got M=%lld, K=%lld); expand the scales "
               "and call fp8k_block_gemm", op, (long long)M, (long long)K);
  const int64_t need = pl.ws_bytes;
  if (need > 0 && (!workspace || workspace_bytes_given < need))
    return fail(FP8K_ERR_WORKSPACE, "%s: workspace of %lld bytes required, %lld given", op, (long long)need,
                (long long)(workspace ? workspace_bytes_given : 0));
  GemmArgs a{};
  a.X = (const uint8_t*)A; a.W = (const uint8_t*)B; a.sx = reinterpret_cast<const float*>(As_packed); a.sw = Bs;
  a.bias = nullptr; a.C = C; a.partial = (float*)workspace;
  a.M = (int)M; a.N = (int)N; a.K = (int)K; a.ldx = lda; a.ldw = ldb; a.ldc = ldc;
  a.sx_m = as_stride_m; a.sx_k = as_stride_w; a.sw_n = bs_stride_n; a.sw_k = bs_stride_k;
  hipStream_t st = (hipStream_t)stream;
  return out_dtype == FP8K_BF16 ? launch_tiles<kModeScaled, FP8K_BF16, FP8K_F32>(a, pl, st)
                                : launch_tiles<kModeScaled, FP8K_F16, FP8K_F32>(a, pl, st);
}

extern "C" int fp8k_scaled_mm(const void* A, const void* B, const float* sa, const float* sb, const void* bias, void* C,
                              int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int out_dtype,
                              int bias_dtype, void* workspace, int64_t workspace_bytes_given, void* stream) {
  clear_error();
  int rc = common_checks("fp8_scaled_mm", A, B, C, M, N, K, lda, ldb, ldc, out_dtype);
  if (rc) return rc;
  if (M == 0 || N == 0) return FP8K_OK;
  FP8K_REQUIRE(K > 0, "fp8_scaled_mm: K must be positive");
  FP8K_REQUIRE(sa && sb, "fp8_scaled_mm: null scale pointer");
  FP8K_REQUIRE(aligned(sb, 16), "fp8_scaled_mm: scales_b must be 16-byte aligned");
  if (bias)
    FP8K_REQUIRE(bias_dtype == FP8K_F32 || bias_dtype == FP8K_F16 || bias_dtype == FP8K_BF16,
                 "fp8_scaled_mm: bias dtype must be float32, float16 or bfloat16");
  const Plan pl = make_plan(M, N, K);
  const int64_t need = pl.ws_bytes;
  if (need > 0 && (!workspace || workspace_bytes_given < need))
    return fail(FP8K_ERR_WORKSPACE, "fp8_scaled_mm: workspace of %lld bytes required, %lld given", (long long)need,
                (long long)(workspace ? workspace_bytes_given : 0));
  GemmArgs a{};
  a.X = (const uint8_t*)A; a.W = (const uint8_t*)B; a.sx = sa; a.sw = sb; a.bias = bias; a.C = C;
  a.partial = (float*)workspace;
  a.M = (int)M; a.N = (int)N; a.K = (int)K; a.ldx = lda; a.ldw = ldb; a.ldc = ldc;
  hipStream_t st = (hipStream_t)stream;
  const int bd = bias ? bias_dtype : FP8K_F32;
#define FP8K_SMM(O, B) launch<kModeRow, O, B>(a, pl, st)
  if (out_dtype == FP8K_BF16) {
    if (bd == FP8K_F32) return FP8K_SMM(FP8K_BF16, FP8K_F32);
    if (bd == FP8K_BF16) return FP8K_SMM(FP8K_BF16, FP8K_BF16);
    return FP8K_SMM(FP8K_BF16, FP8K_F16);
  }
  if (bd == FP8K_F32) return FP8K_SMM(FP8K_F16, FP8K_F32);
  if (bd == FP8K_BF16) return FP8K_SMM(FP8K_F16, FP8K_BF16);
  return FP8K_SMM(FP8K_F16, FP8K_F16);
#undef FP8K_SMM
}

// ---- batched per-tensor-scaled FP8 GEMM (the MLA absorbed products): every batch entry is a row-mode GEMM on the
// 128x128 tile kernel (grid y = entry), whose per-row / per-column scale vectors are shared by all entries.
extern "C" int fp8k_bmm_fp8(const void* A, const void* B, const float* sa, const float* sb, void* C, int64_t batch, int64_t M,
                            int64_t N, int64_t K, int64_t a_stride_b, int64_t lda, int64_t b_stride_b, int64_t ldb,
                            int64_t c_stride_b, int64_t ldc, int out_dtype, void* stream) {
  clear_error();
  const char* op = "bmm_fp8";
  int rc = common_checks(op, A, B, C, M, N, K, lda, ldb, ldc, out_dtype);
  if (rc) return rc;
  FP8K_REQUIRE(batch >= 0 && batch <= 65535, "%s: batch must be in [0, 65535] (got %lld)", op, (long long)batch);
  if (batch == 0 || M == 0 || N == 0) return FP8K_OK;
  FP8K_REQUIRE(K > 0 && K % kTileK == 0, "%s: K must be a positive multiple of 128 (got %lld)", op, (long long)K);
  FP8K_REQUIRE(N % 8 == 0, "%s: N must be a multiple of 8 (got %lld)", op, (long long)N);
  FP8K_REQUIRE(sa && sb, "%s: null scale pointer", op);
  FP8K_REQUIRE(aligned(sb, 16), "%s: the column scale vector must be 16-byte aligned", op);
  FP8K_REQUIRE(a_stride_b % 16 == 0 && b_stride_b % 16 == 0 && (c_stride_b * 2) % 16 == 0 && a_stride_b >= 0 && b_stride_b >= 0 &&
               c_stride_b >= 0, "%s: batch strides must be non-negative multiples of 16 bytes", op);
  GemmArgs a{};
  a.X = (const uint8_t*)A; a.W = (const uint8_t*)B; a.sx = sa; a.sw = sb; a.bias = nullptr; a.C = C; a.partial = nullptr;
  a.M = (int)M; a.N = (int)N; a.K = (int)K; a.ldx = lda; a.ldw = ldb; a.ldc = ldc;
  a.batch_x = a_stride_b; a.batch_w = b_stride_b; a.batch_c = c_stride_b;
  a.tiles_m = (int)((M + kT128 - 1) / kT128);
  a.tiles_n = (int)((N + kT128 - 1) / kT128);
  a.splits = 1;
  a.kb_per_split = (int)(K / kTileK);
  const unsigned nwg = (unsigned)(((int64_t)a.tiles_m * a.tiles_n + 7) / 8 * 8);
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == FP8K_BF16)
    hipLaunchKernelGGL((gemm_tile128_kernel<kModeRow, FP8K_BF16, FP8K_F32, false>), dim3(nwg, (unsigned)batch), dim3(512), 0, st, a);
  else
    hipLaunchKernelGGL((gemm_tile128_kernel<kModeRow, FP8K_F16, FP8K_F32, false>), dim3(nwg, (unsigned)batch), dim3(512), 0, st, a);
  return check_launch(op);
}
