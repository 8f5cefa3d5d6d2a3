// Block-FP8 fused-MoE building blocks for gfx950: token alignment (integer), the grouped block-scaled
// GEMM (host side; the device code is the grouped form of gemm_direct_kernel for 16/32-slot blocks, of
// gemm_stream_kernel for 64/128 and moe_stream256_kernel for 256), silu_and_mul and the top-k sum.  No allocation, no synchronisation, no host reads of device data.
#include "gemm_direct.h"
#include "gemm_moe256.h"

namespace fp8k {

// ------------------------------------------------------------------------------------------------
// moe_align_block_size
//
// One workgroup of 1024 lanes: histogram of the bucket of every id (bucket = id + 1, bucket 0 holds
// id -1) with LDS atomics, an exclusive scan of the counts rounded up to the block size by the first
// wavefront, then per-block expert ids by binary search, the scatter of token slots through LDS
// cursors and the padding tail of every bucket.  Ids outside [-1, buckets-1) are ignored.
// With SCATTER = false the kernel stops after writing the start offsets to `cumsum` (the many-id path below).
// ------------------------------------------------------------------------------------------------
constexpr int kAlignThreads = 1024;
constexpr int kAlignMaxBuckets = 4096;
constexpr int64_t kAlignFusedMax = 8192;  // ids up to which one workgroup does the whole job

template <typename IdT>
__device__ __forceinline__ int bucket_of(const IdT* ids, int64_t i, int nb) {
  const int64_t b = (int64_t)ids[i] + 1;
  return (b >= 0 && b < nb) ? (int)b : -1;
}

// histogram of ids[first, last) into an LDS table (zeroed by the caller, barriers around the call are the caller's):
// eight ids per lane and trip, eight loads in flight instead of one load latency per id
template <typename IdT>
__device__ __forceinline__ void count_ids(const IdT* __restrict__ ids, int64_t first, int64_t last, int nb, int32_t* counts) {
  for (int64_t i0 = first + threadIdx.x; i0 < last; i0 += 8 * kAlignThreads) {
    int b8[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t i = i0 + (int64_t)u * kAlignThreads;
      b8[u] = i < last ? bucket_of(ids, i, nb) : -1;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (b8[u] >= 0) atomicAdd(&counts[b8[u]], 1);
  }
}
// ids[first, last) to their places: cursor[b] (LDS) is the next free position of bucket b
template <typename IdT>
__device__ __forceinline__ void place_ids(const IdT* __restrict__ ids, int64_t first, int64_t last, int nb, int32_t* cursor,
                                          int32_t* __restrict__ sorted) {
  for (int64_t i0 = first + threadIdx.x; i0 < last; i0 += 8 * kAlignThreads) {
    int b8[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t i = i0 + (int64_t)u * kAlignThreads;
      b8[u] = i < last ? bucket_of(ids, i, nb) : -1;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (b8[u] >= 0) sorted[atomicAdd(&cursor[b8[u]], 1)] = (int32_t)(i0 + (int64_t)u * kAlignThreads);
  }
}

// Many ids: the histogram and the placement are spread over workgroups that each take a contiguous run of
// kAlignChunk ids.  moe_count_kernel adds every workgroup's LDS histogram to the (zeroed) global table, the single
// workgroup of moe_align_kernel<PRECOUNTED> turns the table into start offsets, and moe_place_kernel reserves a
// workgroup's share of every bucket with one global atomic per bucket in use and places its ids through LDS cursors.
constexpr int kAlignChunk = 4096;
__global__ __launch_bounds__(256) void zero_ints_kernel(int32_t* __restrict__ p, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0;
}
template <typename IdT>
__global__ __launch_bounds__(kAlignThreads) void moe_count_kernel(const IdT* __restrict__ ids, int64_t numel, int nb,
                                                                  int32_t* __restrict__ table) {
  __shared__ int32_t counts[kAlignMaxBuckets];
  for (int b = threadIdx.x; b < nb; b += kAlignThreads) counts[b] = 0;
  __syncthreads();
  const int64_t first = (int64_t)blockIdx.x * kAlignChunk;
  count_ids(ids, first, min(numel, first + kAlignChunk), nb, counts);
  __syncthreads();
  for (int b = threadIdx.x; b < nb; b += kAlignThreads)
    if (counts[b]) atomicAdd(&table[b], counts[b]);
}
template <typename IdT>
__global__ __launch_bounds__(kAlignThreads) void moe_place_kernel(const IdT* __restrict__ ids, int64_t numel, int nb,
                                                                  int32_t* __restrict__ sorted, int32_t* __restrict__ cumsum) {
  __shared__ int32_t counts[kAlignMaxBuckets];
  for (int b = threadIdx.x; b < nb; b += kAlignThreads) counts[b] = 0;
  __syncthreads();
  const int64_t first = (int64_t)blockIdx.x * kAlignChunk, last = min(numel, first + kAlignChunk);
  count_ids(ids, first, last, nb, counts);
  __syncthreads();
  for (int b = threadIdx.x; b < nb; b += kAlignThreads) {
    const int c = counts[b];
    counts[b] = c ? atomicAdd(&cumsum[b], c) : 0;  // from here on the workgroup's cursor inside bucket b
  }
  __syncthreads();
  place_ids(ids, first, last, nb, counts, sorted);
}

template <typename IdT, bool SCATTER, bool PRECOUNTED = false>
__global__ __launch_bounds__(kAlignThreads) void moe_align_kernel(const IdT* __restrict__ ids, int64_t numel, int nb,
                                                                  int block, int32_t* __restrict__ sorted,
                                                                  int32_t* __restrict__ expert_ids,
                                                                  int32_t* __restrict__ post_pad,
                                                                  int32_t* __restrict__ cumsum, int pad_ids) {
  __shared__ int32_t counts[kAlignMaxBuckets];
  __shared__ int32_t prefix[kAlignMaxBuckets + 1];
  __shared__ int32_t cursor[kAlignMaxBuckets];
  const int tid = threadIdx.x;
  if (PRECOUNTED) {  // cumsum holds the histogram (moe_count_kernel)
    for (int b = tid; b < nb; b += kAlignThreads) counts[b] = cumsum[b];
  } else {
    for (int b = tid; b < nb; b += kAlignThreads) counts[b] = 0;
    __syncthreads();
    count_ids(ids, 0, numel, nb, counts);
  }
  __syncthreads();
  if (tid < 64) {
    // lane l scans buckets [l*per, (l+1)*per)
    const int per = (nb + 63) / 64;
    const int b0 = tid * per;
    int sum = 0;
    for (int b = b0; b < min(nb, b0 + per); ++b) sum += (counts[b] + block - 1) / block * block;
    int incl = sum;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int v = __shfl_up(incl, off);
      if (tid >= off) incl += v;
    }
    int run = incl - sum;
    for (int b = b0; b < min(nb, b0 + per); ++b) {
      prefix[b] = run;
      run += (counts[b] + block - 1) / block * block;
    }
    if (tid == 63) prefix[nb] = incl;
  }
  __syncthreads();
  const int total = prefix[nb];
  if (tid == 0) post_pad[0] = total;
  for (int b = tid; b <= nb; b += kAlignThreads) {
    if (cumsum) cumsum[b] = prefix[b];
    if (b < nb) cursor[b] = prefix[b];
  }
  // expert of every block in use: the bucket whose [prefix[b], prefix[b+1]) range holds the block start
  const int nblocks = total / block;
  for (int i = tid; i < nblocks; i += kAlignThreads) {
    const int start = i * block;
    int lo = 0, hi = nb;  // first bucket with prefix[b+1] > start
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (prefix[mid + 1] <= start) lo = mid + 1;
      else hi = mid;
    }
    expert_ids[i] = lo - 1;
  }
  if (pad_ids) {
    // a wavefront per bucket, a lane per slot: up to block-1 slots per bucket, far too many for one lane each
    for (int b = tid >> 6; b < nb; b += kAlignThreads / 64)
      for (int j = prefix[b] + counts[b] + (tid & 63); j < prefix[b + 1]; j += 64) sorted[j] = (int32_t)numel;
  }
  if (SCATTER) {
    __syncthreads();
    place_ids(ids, 0, numel, nb, cursor, sorted);
  }
}

// ------------------------------------------------------------------------------------------------
// silu_and_mul / gelu_and_mul: out[r, c] = T( T(act(x[r, c])) * x[r, d + c] ), T = bf16 / f16 (two roundings, as
// the reference kernel computes Activation(x) * y on 16-bit values); float32 input has one rounding.
// One lane handles 8 columns: two 16-byte loads, one 16-byte store.
// ------------------------------------------------------------------------------------------------
template <int DT>
__device__ __forceinline__ void load8(const void* base, int64_t elem, float (&a)[8]) {
  if (DT == FP8K_F32) {
    const float4* p = reinterpret_cast<const float4*>((const float*)base + elem);
    const float4 lo = p[0], hi = p[1];
    a[0] = lo.x; a[1] = lo.y; a[2] = lo.z; a[3] = lo.w; a[4] = hi.x; a[5] = hi.y; a[6] = hi.z; a[7] = hi.w;
  } else {
    const uint4 v = *reinterpret_cast<const uint4*>((const u16*)base + elem);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (DT == FP8K_BF16) { a[2 * i] = bf16_lo(w[i]); a[2 * i + 1] = bf16_hi(w[i]); }
      else { a[2 * i] = f16_bits_to_f32(w[i] & 0xffff); a[2 * i + 1] = f16_bits_to_f32(w[i] >> 16); }
    }
  }
}

template <int DT>
__device__ __forceinline__ void store8(void* base, int64_t elem, const float (&a)[8]) {
  if (DT == FP8K_F32) {
    float4* p = reinterpret_cast<float4*>((float*)base + elem);
    p[0] = make_float4(a[0], a[1], a[2], a[3]);
    p[1] = make_float4(a[4], a[5], a[6], a[7]);
  } else {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (DT == FP8K_BF16) w[i] = pack_bf16x2(a[2 * i], a[2 * i + 1]);
      else w[i] = f32_to_f16_bits(a[2 * i]) | (f32_to_f16_bits(a[2 * i + 1]) << 16);
    }
    *reinterpret_cast<uint4*>((u16*)base + elem) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

template <int DT, bool GELU>
__global__ __launch_bounds__(256) void act_and_mul_kernel(const void* __restrict__ x, void* __restrict__ out,
                                                          int64_t rows, int d, int64_t ldx, int64_t ldo) {
  const int chunks = d / 8;
  const int64_t total = rows * chunks;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / chunks;
    const int c = (int)(i - r * chunks) * 8;
    float g[8], u[8], o[8];
    load8<DT>(x, r * ldx + c, g);
    load8<DT>(x, r * ldx + d + c, u);
#pragma unroll
    for (int k = 0; k < 8; ++k) o[k] = round_to<DT>(GELU ? gelu_f32(g[k]) : silu_f32(g[k])) * u[k];
    store8<DT>(out, r * ldo + c, o);
  }
}

// activation without the second factor (the ungated experts of fused_experts_impl): out[r, c] = T(act(x[r, c])) with
// act = silu, gelu (erf form) or relu(x)^2 in float32 and one rounding, as the tensor library's 16-bit ops round
template <int DT, int KIND>
__global__ __launch_bounds__(256) void act_only_kernel(const void* __restrict__ x, void* __restrict__ out, int64_t rows,
                                                       int d, int64_t ldx, int64_t ldo) {
  const int chunks = d / 8;
  const int64_t total = rows * chunks;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / chunks;
    const int c = (int)(i - r * chunks) * 8;
    float g[8], o[8];
    load8<DT>(x, r * ldx + c, g);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      if (KIND == FP8K_ACT_SILU) o[k] = silu_f32(g[k]);
      else if (KIND == FP8K_ACT_GELU) o[k] = gelu_f32(g[k]);
      else { const float t = g[k] > 0.f ? g[k] : (g[k] == g[k] ? 0.f : g[k]); o[k] = t * t; }  // NaN stays NaN, as relu keeps it
    }
    store8<DT>(out, r * ldo + c, o);
  }
}

// ------------------------------------------------------------------------------------------------
// moe_sum_reduce: out[t, :] = T( scale * sum_k float(x[t, k, :]) ), k ascending, float32 accumulate
// ------------------------------------------------------------------------------------------------
// ELEM (moe_sum with 2..4 experts per token): the running sum is rounded to the element type after every addition
template <int DT, bool ELEM = false>
__global__ __launch_bounds__(256) void moe_sum_reduce_kernel(const void* __restrict__ x, void* __restrict__ out,
                                                             int64_t tokens, int topk, int hidden, int64_t stride_t,
                                                             int64_t stride_k, int64_t out_stride_t, float scale) {
  const int chunks = hidden / 8;
  const int64_t total = tokens * chunks;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    const int64_t t = i / chunks;
    const int c = (int)(i - t * chunks) * 8;
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.f;
    for (int k = 0; k < topk; ++k) {
      float v[8];
      load8<DT>(x, t * stride_t + (int64_t)k * stride_k + c, v);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = (ELEM && k > 0) ? round_to<DT>(acc[j] + v[j]) : acc[j] + v[j];
    }
    if (!ELEM) {
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] *= scale;
    }
    store8<DT>(out, t * out_stride_t + c, acc);
  }
}

static unsigned stream_grid(int64_t work_items) {
  const int64_t want = (work_items + 255) / 256;
  return (unsigned)(want < 1 ? 1 : (want > 256 * 16 ? 256 * 16 : want));
}

}  // namespace fp8k

using namespace fp8k;

extern "C" int fp8k_moe_align_block_size(const void* topk_ids, int ids_are_int64, int64_t numel, int64_t num_buckets,
                                         int64_t block_size, int32_t* sorted_token_ids, int64_t sorted_capacity,
                                         int32_t* expert_ids, int64_t expert_capacity, int32_t* num_tokens_post_pad,
                                         int32_t* cumsum_buffer, int pad_sorted_token_ids, void* stream) {
  clear_error();
  FP8K_REQUIRE(numel >= 0 && numel < 0x7fffffffLL, "moe_align_block_size: bad number of ids (%lld)", (long long)numel);
  FP8K_REQUIRE(num_buckets >= 1 && num_buckets <= kAlignMaxBuckets,
               "moe_align_block_size: num_experts must be in [1, %d] (got %lld)", kAlignMaxBuckets, (long long)num_buckets);
  FP8K_REQUIRE(block_size >= 1 && block_size <= 1024, "moe_align_block_size: block_size must be in [1, 1024]");
  // worst case: every bucket in use carries block_size-1 padding slots
  const int64_t used_buckets = numel < num_buckets ? numel : num_buckets;
  const int64_t worst = numel + used_buckets * (block_size - 1);
  FP8K_REQUIRE(sorted_capacity >= worst, "moe_align_block_size: sorted_token_ids holds %lld slots, %lld may be needed",
               (long long)sorted_capacity, (long long)worst);
  FP8K_REQUIRE(expert_capacity >= worst / block_size,
               "moe_align_block_size: experts_ids holds %lld blocks, %lld may be needed", (long long)expert_capacity,
               (long long)(worst / block_size));
  FP8K_REQUIRE(sorted_token_ids && expert_ids && num_tokens_post_pad, "moe_align_block_size: null output pointer");
  FP8K_REQUIRE(numel == 0 || topk_ids, "moe_align_block_size: null topk_ids");
  hipStream_t st = (hipStream_t)stream;
  // one workgroup does everything up to kAlignFusedMax ids (and whenever the caller gives no scratch table); more ids
  // are counted and placed by one workgroup per kAlignChunk ids
  const bool fused = numel <= kAlignFusedMax || !cumsum_buffer;
  const unsigned chunks = (unsigned)((numel + kAlignChunk - 1) / kAlignChunk);
#define FP8K_ALIGN(T)                                                                                                \
  do {                                                                                                               \
    if (fused) {                                                                                                     \
      hipLaunchKernelGGL((moe_align_kernel<T, true>), dim3(1), dim3(kAlignThreads), 0, st, (const T*)topk_ids, numel, \
                         (int)num_buckets, (int)block_size, sorted_token_ids, expert_ids, num_tokens_post_pad,        \
                         cumsum_buffer, pad_sorted_token_ids);                                                        \
    } else {                                                                                                         \
      hipLaunchKernelGGL(zero_ints_kernel, dim3((unsigned)((num_buckets + 1 + 255) / 256)), dim3(256), 0, st,         \
                         cumsum_buffer, (int)num_buckets + 1);                                                        \
      hipLaunchKernelGGL((moe_count_kernel<T>), dim3(chunks), dim3(kAlignThreads), 0, st, (const T*)topk_ids, numel,  \
                         (int)num_buckets, cumsum_buffer);                                                            \
      hipLaunchKernelGGL((moe_align_kernel<T, false, true>), dim3(1), dim3(kAlignThreads), 0, st, (const T*)topk_ids, \
                         numel, (int)num_buckets, (int)block_size, sorted_token_ids, expert_ids, num_tokens_post_pad, \
                         cumsum_buffer, pad_sorted_token_ids);                                                        \
      hipLaunchKernelGGL((moe_place_kernel<T>), dim3(chunks), dim3(kAlignThreads), 0, st, (const T*)topk_ids, numel,  \
                         (int)num_buckets, sorted_token_ids, cumsum_buffer);                                          \
    }                                                                                                                \
  } while (0)
  if (ids_are_int64) FP8K_ALIGN(int64_t);
  else FP8K_ALIGN(int32_t);
#undef FP8K_ALIGN
  return check_launch("moe_align_block_size");
}

namespace fp8k {
// Activation scales in the order of sorted_token_ids: out[kb * capacity + i] = As[sorted_token_ids[i] / top_k, kb]
// (0 for padding), for i < num_tokens_post_padded.  One lane per position walks its row's K blocks, so every
// store instruction writes 256 contiguous bytes.
__global__ __launch_bounds__(256) void moe_sort_scales_kernel(const float* __restrict__ As, float* __restrict__ out,
                                                              const int32_t* __restrict__ sorted_ids,
                                                              const int32_t* __restrict__ npad, int capacity, int kb,
                                                              int top_k, int num_valid, int64_t sm, int64_t sk) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= min(npad[0], capacity)) return;
  const int s = sorted_ids[i];
  const bool ok = s < num_valid;
  const float* row = As + (int64_t)(ok ? s / top_k : 0) * sm;
  for (int k = 0; k < kb; ++k) out[(int64_t)k * capacity + i] = ok ? row[(int64_t)k * sk] : 0.f;
}
}  // namespace fp8k

namespace fp8k {
// moe_align_block_size fills every block of an expert but its last one, so an expert with 600 slots gets blocks of 256,
// 256 and 88.  The workgroups of the grouped GEMM that take those blocks against the same weight tile are dispatched
// together and share the tile in their XCD's L2 only while they keep pace - and a block of 88 slots runs away from one of
// 256.  This kernel deals an expert's slots out evenly over the blocks it already has (200 / 200 / 200): slot number r of
// the expert goes to block r mod nb, position r / nb.  Real slots still come first in every block, the block table
// (expert_ids, the padded length) is unchanged, and which slot meets which row of a block is as unspecified as before.
// Every workgroup finds the experts' first blocks, block counts and slot counts for itself; then one wavefront per block.
__global__ __launch_bounds__(kAlignThreads) void moe_balance_blocks_kernel(const int32_t* __restrict__ sorted_in,
                                                                           const int32_t* __restrict__ expert_ids,
                                                                           const int32_t* __restrict__ post_pad, int capacity,
                                                                           int block, int pad_value, int buckets,
                                                                           int32_t* __restrict__ sorted_out) {
  __shared__ int32_t first[kAlignMaxBuckets + 1], nblk[kAlignMaxBuckets + 1], creal[kAlignMaxBuckets + 1];
  const int tid = threadIdx.x, wave = tid >> 6, ln = tid & 63, waves = kAlignThreads / 64;
  const int nblocks = min(post_pad[0], capacity) / block;
  for (int e = tid; e < buckets; e += kAlignThreads) { first[e] = 0x7fffffff; nblk[e] = 0; creal[e] = 0; }
  __syncthreads();
  for (int b = tid; b < nblocks; b += kAlignThreads) {
    const int e = expert_ids[b] + 1;  // bucket 0: blocks of ids that belong to no expert of this rank
    if (e >= 0 && e < buckets) { atomicMin(&first[e], b); atomicAdd(&nblk[e], 1); }
  }
  __syncthreads();
  for (int e = tid; e < buckets; e += kAlignThreads) {  // slots of the expert = full blocks + the real entries of its last block
    if (nblk[e] == 0) continue;
    const int32_t* last = sorted_in + (int64_t)(first[e] + nblk[e] - 1) * block;
    int lo = 0, hi = block;  // first padding entry of the last block (real slots come first)
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (last[mid] < pad_value) lo = mid + 1;
      else hi = mid;
    }
    creal[e] = (nblk[e] - 1) * block + lo;
  }
  __syncthreads();
  for (int b = blockIdx.x * waves + wave; b < nblocks; b += gridDim.x * waves) {
    const int e = expert_ids[b] + 1;
    if (e < 0 || e >= buckets) {  // not a bucket of this table: the block is copied as it is
      for (int p = ln; p < block; p += 64) sorted_out[b * block + p] = sorted_in[b * block + p];
      continue;
    }
    const int f = first[e], nb = nblk[e], c = creal[e], j = b - f;
    for (int p = ln; p < block; p += 64) {
      const int r = p * nb + j;
      sorted_out[b * block + p] = r < c ? sorted_in[(f + r / block) * block + r % block] : pad_value;
    }
  }
  // behind the blocks in use the table keeps the padding value
  for (int i = nblocks * block + blockIdx.x * kAlignThreads + tid; i < capacity; i += gridDim.x * kAlignThreads) sorted_out[i] = pad_value;
}
}  // namespace fp8k

extern "C" int fp8k_moe_balance_blocks(const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                       const int32_t* num_tokens_post_padded, int64_t sorted_capacity, int64_t block_m,
                                       int64_t num_valid_tokens, int64_t num_experts, int32_t* sorted_out, void* stream) {
  clear_error();
  const char* op = "moe_balance_blocks";
  FP8K_REQUIRE(sorted_capacity >= 0 && sorted_capacity < 0x7fffffffLL && block_m >= 1 && block_m <= 1024, "%s: bad shape", op);
  FP8K_REQUIRE(num_valid_tokens >= 0 && num_valid_tokens < 0x7fffffffLL, "%s: bad slot count", op);
  FP8K_REQUIRE(num_experts >= 1 && num_experts < kAlignMaxBuckets, "%s: num_experts must be in [1, %d) (got %lld)", op,
               kAlignMaxBuckets, (long long)num_experts);
  if (sorted_capacity == 0) return FP8K_OK;
  FP8K_REQUIRE(sorted_token_ids && expert_ids && num_tokens_post_padded && sorted_out, "%s: null pointer", op);
  FP8K_REQUIRE(sorted_out != sorted_token_ids, "%s: the balanced table needs a buffer of its own", op);
  const int64_t blocks = sorted_capacity / block_m;
  const unsigned grid = (unsigned)std::max<int64_t>(1, std::min<int64_t>(32, (blocks + 15) / 16));
  hipLaunchKernelGGL(moe_balance_blocks_kernel, dim3(grid), dim3(kAlignThreads), 0, (hipStream_t)stream, sorted_token_ids,
                     expert_ids, num_tokens_post_padded, (int)sorted_capacity, (int)block_m, (int)num_valid_tokens,
                     (int)num_experts + 1, sorted_out);
  return check_launch(op);
}

extern "C" int fp8k_moe_sort_scales(const float* As, float* out, const int32_t* sorted_token_ids,
                                    const int32_t* num_tokens_post_padded, int64_t sorted_capacity, int64_t k_blocks,
                                    int64_t top_k, int64_t num_valid_tokens, int64_t as_stride_m, int64_t as_stride_k,
                                    void* stream) {
  clear_error();
  const char* op = "moe_sort_scales";
  FP8K_REQUIRE(sorted_capacity >= 0 && sorted_capacity < 0x7fffffffLL && k_blocks >= 0 && k_blocks < 0x7fffffffLL,
               "%s: bad shape", op);
  FP8K_REQUIRE(top_k > 0 && num_valid_tokens >= 0 && num_valid_tokens < 0x7fffffffLL, "%s: bad shape", op);
  FP8K_REQUIRE(as_stride_m >= 0 && as_stride_k >= 0, "%s: negative scale stride", op);
  if (sorted_capacity == 0 || k_blocks == 0) return FP8K_OK;
  FP8K_REQUIRE(As && out && sorted_token_ids && num_tokens_post_padded, "%s: null pointer", op);
  hipLaunchKernelGGL(moe_sort_scales_kernel, dim3((unsigned)((sorted_capacity + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, As, out, sorted_token_ids, num_tokens_post_padded, (int)sorted_capacity,
                     (int)k_blocks, (int)top_k, (int)num_valid_tokens, as_stride_m, as_stride_k);
  return check_launch(op);
}

// whether the 256-slot grouped kernel runs as one walking workgroup per CU (the walk hands the weight stream on two K
// blocks ahead, so K must have them)
static bool moe256_walks(int64_t num_valid_tokens, int64_t num_experts, int64_t K, bool balanced) {
  return (balanced || num_valid_tokens <= num_experts * 192) && K >= 2 * kTileK;
}

static int moe_block_gemm_impl(const void* A, const void* B, const float* As, const float* Bs, void* C,
                               const int32_t* sorted_token_ids, const int32_t* expert_ids,
                               const int32_t* num_tokens_post_padded, const float* topk_weights,
                               int64_t sorted_capacity, int64_t block_m, int64_t num_valid_tokens, int64_t top_k,
                               int64_t num_experts, int64_t N, int64_t K, int64_t lda, int64_t as_stride_m,
                               int64_t as_stride_k, int64_t b_stride_e, int64_t ldb, int64_t bs_stride_e,
                               int64_t bs_stride_n, int64_t bs_stride_k, int64_t ldc, int out_dtype, int as_sorted,
                               bool pow2_scales, void* stream) {
  clear_error();
  const char* op = pow2_scales ? "moe_block_gemm_ue8m0" : "moe_block_gemm";
  FP8K_REQUIRE(N > 0 && K > 0 && num_experts > 0 && top_k > 0, "%s: bad shape", op);
  FP8K_REQUIRE(N <= 0x7fffffffLL && K <= 0x7fffffffLL && num_valid_tokens >= 0 && num_valid_tokens < 0x7fffffffLL,
               "%s: shape too large", op);
  FP8K_REQUIRE(out_dtype == FP8K_F16 || out_dtype == FP8K_BF16, "%s: out_dtype must be Half or BFloat16", op);
  FP8K_REQUIRE(K % kTileK == 0, "%s: K (%lld) must be a multiple of 128", op, (long long)K);
  FP8K_REQUIRE(N % 8 == 0, "%s: N (%lld) must be a multiple of 8", op, (long long)N);
  FP8K_REQUIRE(block_m == 16 || block_m == 32 || block_m == 64 || block_m == 128 || block_m == 256,
               "%s: block_m must be 16, 32, 64, 128 or 256 (got %lld)", op, (long long)block_m);
  FP8K_REQUIRE(sorted_capacity >= 0 && sorted_capacity < 0x7fffffffLL, "%s: bad sorted_token_ids length", op);
  FP8K_REQUIRE(lda >= K && ldb >= K && ldc >= N, "%s: leading dimension smaller than the row length", op);
  FP8K_REQUIRE(lda % 16 == 0 && ldb % 16 == 0 && (ldc * 2) % 8 == 0, "%s: rows must be 16-byte aligned", op);
  if (num_valid_tokens == 0 || sorted_capacity < block_m) return FP8K_OK;
  FP8K_REQUIRE(A && B && As && Bs && C && sorted_token_ids && expert_ids && num_tokens_post_padded, "%s: null pointer", op);
  FP8K_REQUIRE(aligned(A, 16) && aligned(B, 16) && aligned(C, 8) && b_stride_e % 16 == 0,
               "%s: operands must be 16-byte aligned", op);
  const int64_t xrows = (num_valid_tokens + top_k - 1) / top_k;
  FP8K_REQUIRE(xrows * lda < 0xE0000000LL, "%s: activation matrix exceeds 3.5 GiB, split the token batch", op);
  FP8K_REQUIRE(ldb < (1LL << 23) && lda < (1LL << 23), "%s: rows longer than 8 MiB are not supported", op);
  FP8K_REQUIRE(as_stride_m >= 0 && as_stride_k >= 0 && bs_stride_n >= 0 && bs_stride_k >= 0 && bs_stride_e >= 0,
               "%s: negative scale stride", op);

  GemmArgs a{};
  a.X = (const uint8_t*)A; a.W = (const uint8_t*)B; a.sx = As; a.sw = Bs; a.C = C;
  a.M = (int)num_valid_tokens; a.N = (int)N; a.K = (int)K; a.ldx = lda; a.ldw = ldb; a.ldc = ldc;
  a.sx_m = as_stride_m; a.sx_k = as_stride_k; a.sw_n = bs_stride_n; a.sw_k = bs_stride_k;
  a.tiles_m = 0; a.tiles_n = (int)((N + kTileN - 1) / kTileN);
  a.splits = 1; a.kb_per_split = (int)(K / kTileK);
  a.sorted_ids = sorted_token_ids; a.expert_ids = expert_ids; a.num_post_pad = num_tokens_post_padded;
  a.topk_w = topk_weights; a.top_k = (int)top_k; a.num_valid = (int)num_valid_tokens;
  a.m_blocks = (int)(sorted_capacity / block_m);
  a.block_m = (int)block_m;
  a.w_expert_stride = b_stride_e; a.sw_expert_stride = bs_stride_e;
  const bool balanced = (as_sorted & 2) != 0;  // the table went through fp8k_moe_balance_blocks
  as_sorted &= 1;
  a.sx_sorted = as_sorted ? 1 : 0;
  FP8K_REQUIRE(!as_sorted || block_m >= 64, "%s: scales in sorted order are taken with block_m >= 64", op);
  const bool direct = block_m <= 32;  // few rows per expert: weights go straight to registers, 128-row tiles
  if (direct) a.tiles_n = (int)((N + kDirTileN - 1) / kDirTileN);
  const int64_t per_xcd = (a.m_blocks + 7) / 8;
  const int64_t nwg = per_xcd * 8 * a.tiles_n;
  FP8K_REQUIRE(nwg < 0x7fffffffLL, "%s: grid too large", op);
  hipStream_t st = (hipStream_t)stream;
#define FP8K_MOE_DIRECT(TM, O) \
  hipLaunchKernelGGL((gemm_direct_kernel<TM, kModeBlock, O, FP8K_F32, false, true>), dim3((unsigned)nwg), dim3(512), 0, st, a)
  if (direct) {
    if (out_dtype == FP8K_BF16) {
      if (block_m == 16) FP8K_MOE_DIRECT(16, FP8K_BF16);
      else FP8K_MOE_DIRECT(32, FP8K_BF16);
    } else {
      if (block_m == 16) FP8K_MOE_DIRECT(16, FP8K_F16);
      else FP8K_MOE_DIRECT(32, FP8K_F16);
    }
    return check_launch(op);
  }
#undef FP8K_MOE_DIRECT
  FP8K_REQUIRE((as_sorted ? sorted_capacity : xrows) * as_stride_m + (K / kTileK) * as_stride_k < 0x38000000LL,
               "%s: activation scale tensor too large", op);
  if (block_m == 256) {
    // Up to about 200 slots per expert nearly every expert is one block and the items cost about the same: one walking
    // workgroup per CU (a multiple of 8: one share per XCD), which requests an item's first blocks in front of the
    // previous item's write-out (M = 4096 tokens, top-8 of 256 experts: both GEMMs 4 % faster).  With several blocks per
    // expert, some of them nearly empty, the item times differ and a fixed share per CU loses more than the overlap
    // gains (M = 16384: 6 % slower): one workgroup per item, handed out by the dispatcher as CUs fall free - unless the
    // caller says that the blocks of an expert are equally full (moe_balance_blocks): then the walk is ahead at every
    // size (16384 tokens: 2 %).
    const bool walk = moe256_walks(num_valid_tokens, num_experts, K, balanced);
    const int64_t nwg = walk ? std::min<int64_t>(per_xcd * 8 * a.tiles_n, std::max(8, num_cu() / 8 * 8)) : per_xcd * 8 * a.tiles_n;
    // row-major activation scales (what fused_experts_impl produces for 256-slot blocks) take the form that fetches
    // two K blocks per load
    const bool pairs = !as_sorted && as_stride_k == 1 && (as_stride_m & 1) == 0 && aligned(As, 8);  // 129..256 and more slots per expert: both 128-row halves on one weight stage
#define FP8K_MOE256(O) \
  do { \
    if (pairs) hipLaunchKernelGGL((moe_stream256_kernel<O, true, false>), dim3((unsigned)nwg), dim3(512), 0, st, a); \
    else if (as_sorted && pow2_scales) hipLaunchKernelGGL((moe_stream256_kernel<O, false, true, false, true>), dim3((unsigned)nwg), dim3(512), 0, st, a); \
    else if (as_sorted) hipLaunchKernelGGL((moe_stream256_kernel<O, false, true>), dim3((unsigned)nwg), dim3(512), 0, st, a); \
    else hipLaunchKernelGGL((moe_stream256_kernel<O, false, false>), dim3((unsigned)nwg), dim3(512), 0, st, a); \
  } while (0)
    if (out_dtype == FP8K_BF16) FP8K_MOE256(FP8K_BF16);
    else FP8K_MOE256(FP8K_F16);
#undef FP8K_MOE256
    return check_launch(op);
  }
#define FP8K_MOE(TM, NST, NW, O) \
  hipLaunchKernelGGL((gemm_stream_kernel<TM, NST, NW, kModeBlock, O, FP8K_F32, false, true>), dim3((unsigned)nwg), dim3(NW * 64), 0, st, a)
  if (out_dtype == FP8K_BF16) {
    if (block_m == 64) FP8K_MOE(64, 3, 8, FP8K_BF16);
    else FP8K_MOE(128, 3, 8, FP8K_BF16);
  } else {
    if (block_m == 64) FP8K_MOE(64, 3, 8, FP8K_F16);
    else FP8K_MOE(128, 3, 8, FP8K_F16);
  }
#undef FP8K_MOE
  return check_launch(op);
}

extern "C" int fp8k_moe_block_gemm(const void* A, const void* B, const float* As, const float* Bs, void* C,
                                   const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                   const int32_t* num_tokens_post_padded, const float* topk_weights,
                                   int64_t sorted_capacity, int64_t block_m, int64_t num_valid_tokens, int64_t top_k,
                                   int64_t num_experts, int64_t N, int64_t K, int64_t lda, int64_t as_stride_m,
                                   int64_t as_stride_k, int64_t b_stride_e, int64_t ldb, int64_t bs_stride_e,
                                   int64_t bs_stride_n, int64_t bs_stride_k, int64_t ldc, int out_dtype, int as_sorted,
                                   void* stream) {
  return moe_block_gemm_impl(A, B, As, Bs, C, sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights,
                             sorted_capacity, block_m, num_valid_tokens, top_k, num_experts, N, K, lda, as_stride_m,
                             as_stride_k, b_stride_e, ldb, bs_stride_e, bs_stride_n, bs_stride_k, ldc, out_dtype, as_sorted,
                             false, stream);
}

extern "C" int fp8k_moe_block_gemm_ue8m0(const void* A, const void* B, const float* As, const float* Bs, void* C,
                                         const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                         const int32_t* num_tokens_post_padded, const float* topk_weights,
                                         int64_t sorted_capacity, int64_t block_m, int64_t num_valid_tokens, int64_t top_k,
                                         int64_t num_experts, int64_t N, int64_t K, int64_t lda, int64_t as_stride_m,
                                         int64_t as_stride_k, int64_t b_stride_e, int64_t ldb, int64_t bs_stride_e,
                                         int64_t bs_stride_n, int64_t bs_stride_k, int64_t ldc, int out_dtype,
                                         int as_sorted, void* stream) {
  return moe_block_gemm_impl(A, B, As, Bs, C, sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights,
                             sorted_capacity, block_m, num_valid_tokens, top_k, num_experts, N, K, lda, as_stride_m,
                             as_stride_k, b_stride_e, ldb, bs_stride_e, bs_stride_n, bs_stride_k, ldc, out_dtype, as_sorted,
                             true, stream);
}

extern "C" int fp8k_moe_block_gemm_silu_quant(const void* A, const void* B, const float* As_sorted, const float* Bs, void* q_out,
                                              float* qs_out, const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                              const int32_t* num_tokens_post_padded, int64_t sorted_capacity,
                                              int64_t num_valid_tokens, int64_t top_k, int64_t num_experts, int64_t N,
                                              int64_t K, int64_t lda, int64_t as_stride_k, int64_t b_stride_e, int64_t ldb,
                                              int64_t bs_stride_e, int64_t bs_stride_n, int64_t bs_stride_k, int64_t ldq,
                                              int64_t qs_stride_g, float eps, int act_dtype, int balanced, void* stream) {
  clear_error();
  const char* op = "moe_block_gemm_silu_quant";
  constexpr int64_t block_m = 256;
  FP8K_REQUIRE(N > 0 && K > 0 && num_experts > 0 && top_k > 0, "%s: bad shape", op);
  FP8K_REQUIRE(N <= 0x7fffffffLL && K <= 0x7fffffffLL && num_valid_tokens >= 0 && num_valid_tokens < 0x7fffffffLL,
               "%s: shape too large", op);
  FP8K_REQUIRE(act_dtype == FP8K_F16 || act_dtype == FP8K_BF16, "%s: the activation type must be Half or BFloat16", op);
  FP8K_REQUIRE(K % kTileK == 0, "%s: K (%lld) must be a multiple of 128", op, (long long)K);
  FP8K_REQUIRE(N % 256 == 0, "%s: N = 2 I with I a multiple of 128 (got N = %lld)", op, (long long)N);
  const int64_t I = N / 2;
  FP8K_REQUIRE(sorted_capacity >= 0 && sorted_capacity < 0x7fffffffLL, "%s: bad sorted_token_ids length", op);
  FP8K_REQUIRE(lda >= K && ldb >= K && ldq >= I, "%s: leading dimension smaller than the row length", op);
  FP8K_REQUIRE(lda % 16 == 0 && ldb % 16 == 0 && ldq % 16 == 0, "%s: rows must be 16-byte aligned", op);
  FP8K_REQUIRE(qs_stride_g >= sorted_capacity, "%s: the scale rows must hold one float per position of sorted_token_ids", op);
  if (num_valid_tokens == 0 || sorted_capacity < block_m) return FP8K_OK;
  FP8K_REQUIRE(A && B && As_sorted && Bs && q_out && qs_out && sorted_token_ids && expert_ids && num_tokens_post_padded,
               "%s: null pointer", op);
  FP8K_REQUIRE(aligned(A, 16) && aligned(B, 16) && aligned(q_out, 16) && b_stride_e % 16 == 0, "%s: operands must be 16-byte aligned", op);
  const int64_t xrows = (num_valid_tokens + top_k - 1) / top_k;
  FP8K_REQUIRE(xrows * lda < 0xE0000000LL, "%s: activation matrix exceeds 3.5 GiB, split the token batch", op);
  FP8K_REQUIRE(ldb < (1LL << 23) && lda < (1LL << 23), "%s: rows longer than 8 MiB are not supported", op);
  FP8K_REQUIRE((I + 128) * ldb + K < 0xF0000000LL, "%s: an expert's weight exceeds 3.75 GiB", op);
  FP8K_REQUIRE(as_stride_k >= sorted_capacity && bs_stride_n >= 0 && bs_stride_k >= 0 && bs_stride_e >= 0, "%s: bad scale stride", op);
  FP8K_REQUIRE(sorted_capacity + (K / kTileK) * as_stride_k < 0x38000000LL, "%s: activation scale tensor too large", op);

  GemmArgs a{};
  a.X = (const uint8_t*)A; a.W = (const uint8_t*)B; a.sx = As_sorted; a.sw = Bs; a.C = nullptr;
  a.M = (int)num_valid_tokens; a.N = (int)N; a.K = (int)K; a.ldx = lda; a.ldw = ldb; a.ldc = 0;
  a.sx_m = 1; a.sx_k = as_stride_k; a.sw_n = bs_stride_n; a.sw_k = bs_stride_k;
  a.tiles_m = 0; a.tiles_n = (int)(I / 128);
  a.splits = 1; a.kb_per_split = (int)(K / kTileK);
  a.sorted_ids = sorted_token_ids; a.expert_ids = expert_ids; a.num_post_pad = num_tokens_post_padded;
  a.topk_w = nullptr; a.top_k = (int)top_k; a.num_valid = (int)num_valid_tokens;
  a.m_blocks = (int)(sorted_capacity / block_m);
  a.block_m = (int)block_m;
  a.w_expert_stride = b_stride_e; a.sw_expert_stride = bs_stride_e;
  a.sx_sorted = 1;
  a.q_out = (uint8_t*)q_out; a.qs_out = qs_out; a.ldq = ldq; a.qs_ld = qs_stride_g;
  // the group maximum is clamped in the activation type, as the quantisation kernels do
  a.q_eps = eps;
  if (act_dtype == FP8K_BF16) {
    uint32_t u;
    memcpy(&u, &eps, 4);
    u = ((u + 0x7fffu + ((u >> 16) & 1u)) >> 16) << 16;
    memcpy(&a.q_eps, &u, 4);
  }
  const int64_t per_xcd = (a.m_blocks + 7) / 8;
  const bool walk = moe256_walks(num_valid_tokens, num_experts, K, balanced != 0);
  const int64_t nwg = walk ? std::min<int64_t>(per_xcd * 8 * a.tiles_n, std::max(8, num_cu() / 8 * 8)) : per_xcd * 8 * a.tiles_n;
  FP8K_REQUIRE(nwg < 0x7fffffffLL, "%s: grid too large", op);
  hipStream_t st = (hipStream_t)stream;
  if (act_dtype == FP8K_BF16) hipLaunchKernelGGL((moe_stream256_kernel<FP8K_BF16, false, true, true>), dim3((unsigned)nwg), dim3(512), 0, st, a);
  else hipLaunchKernelGGL((moe_stream256_kernel<FP8K_F16, false, true, true>), dim3((unsigned)nwg), dim3(512), 0, st, a);
  return check_launch(op);
}

template <bool GELU>
static int act_and_mul_impl(const char* op, const void* x, void* out, int64_t rows, int64_t d, int64_t ldx, int64_t ldo, int dtype,
                            void* stream) {
  clear_error();
  FP8K_REQUIRE(rows >= 0 && d >= 0, "%s: negative shape", op);
  FP8K_REQUIRE(dtype == FP8K_F32 || dtype == FP8K_F16 || dtype == FP8K_BF16, "%s: bad dtype %d", op, dtype);
  FP8K_REQUIRE(d % 8 == 0 && d <= 0x7fffffffLL, "%s: the output width (%lld) must be a multiple of 8", op, (long long)d);
  FP8K_REQUIRE(ldx >= 2 * d && ldo >= d && ldx % 8 == 0 && ldo % 8 == 0, "%s: bad row strides", op);
  if (rows == 0 || d == 0) return FP8K_OK;
  FP8K_REQUIRE(x && out, "%s: null pointer", op);
  FP8K_REQUIRE(aligned(x, 16) && aligned(out, 16), "%s: The pointers must be multiple of 16 bytes.", op);
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(stream_grid(rows * (d / 8))), block(256);
  switch (dtype) {
    case FP8K_BF16: hipLaunchKernelGGL((act_and_mul_kernel<FP8K_BF16, GELU>), grid, block, 0, st, x, out, rows, (int)d, ldx, ldo); break;
    case FP8K_F16: hipLaunchKernelGGL((act_and_mul_kernel<FP8K_F16, GELU>), grid, block, 0, st, x, out, rows, (int)d, ldx, ldo); break;
    default: hipLaunchKernelGGL((act_and_mul_kernel<FP8K_F32, GELU>), grid, block, 0, st, x, out, rows, (int)d, ldx, ldo); break;
  }
  return check_launch(op);
}

extern "C" int fp8k_silu_and_mul(const void* x, void* out, int64_t rows, int64_t d, int64_t ldx, int64_t ldo, int dtype,
                                 void* stream) {
  return act_and_mul_impl<false>("silu_and_mul", x, out, rows, d, ldx, ldo, dtype, stream);
}

extern "C" int fp8k_gelu_and_mul(const void* x, void* out, int64_t rows, int64_t d, int64_t ldx, int64_t ldo, int dtype,
                                 void* stream) {
  return act_and_mul_impl<true>("gelu_and_mul", x, out, rows, d, ldx, ldo, dtype, stream);
}

template <int KIND>
static void launch_act_only(dim3 grid, hipStream_t st, const void* x, void* out, int64_t rows, int d, int64_t ldx, int64_t ldo,
                            int dtype) {
  const dim3 block(256);
  switch (dtype) {
    case FP8K_BF16: hipLaunchKernelGGL((act_only_kernel<FP8K_BF16, KIND>), grid, block, 0, st, x, out, rows, d, ldx, ldo); break;
    case FP8K_F16: hipLaunchKernelGGL((act_only_kernel<FP8K_F16, KIND>), grid, block, 0, st, x, out, rows, d, ldx, ldo); break;
    default: hipLaunchKernelGGL((act_only_kernel<FP8K_F32, KIND>), grid, block, 0, st, x, out, rows, d, ldx, ldo); break;
  }
}

extern "C" int fp8k_activation(const void* x, void* out, int64_t rows, int64_t d, int64_t ldx, int64_t ldo, int kind, int dtype,
                               void* stream) {
  clear_error();
  const char* op = "activation";
  FP8K_REQUIRE(rows >= 0 && d >= 0, "%s: negative shape", op);
  FP8K_REQUIRE(kind == FP8K_ACT_SILU || kind == FP8K_ACT_GELU || kind == FP8K_ACT_RELU2, "%s: bad kind %d", op, kind);
  FP8K_REQUIRE(dtype == FP8K_F32 || dtype == FP8K_F16 || dtype == FP8K_BF16, "%s: bad dtype %d", op, dtype);
  FP8K_REQUIRE(d % 8 == 0 && d <= 0x7fffffffLL, "%s: the width (%lld) must be a multiple of 8", op, (long long)d);
  FP8K_REQUIRE(ldx >= d && ldo >= d && ldx % 8 == 0 && ldo % 8 == 0, "%s: bad row strides", op);
  if (rows == 0 || d == 0) return FP8K_OK;
  FP8K_REQUIRE(x && out, "%s: null pointer", op);
  FP8K_REQUIRE(aligned(x, 16) && aligned(out, 16), "%s: the pointers must be 16-byte aligned", op);
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(stream_grid(rows * (d / 8)));
  if (kind == FP8K_ACT_SILU) launch_act_only<FP8K_ACT_SILU>(grid, st, x, out, rows, (int)d, ldx, ldo, dtype);
  else if (kind == FP8K_ACT_GELU) launch_act_only<FP8K_ACT_GELU>(grid, st, x, out, rows, (int)d, ldx, ldo, dtype);
  else launch_act_only<FP8K_ACT_RELU2>(grid, st, x, out, rows, (int)d, ldx, ldo, dtype);
  return check_launch(op);
}

static int moe_sum_impl(const void* x, void* out, int64_t tokens, int64_t topk, int64_t hidden, int64_t stride_token,
                        int64_t stride_topk, int64_t out_stride_token, float scale, int dtype, bool elem, void* stream) {
  FP8K_REQUIRE(tokens >= 0 && topk >= 0 && hidden >= 0, "moe_sum_reduce: negative shape");
  FP8K_REQUIRE(dtype == FP8K_F32 || dtype == FP8K_F16 || dtype == FP8K_BF16, "moe_sum_reduce: bad dtype %d", dtype);
  FP8K_REQUIRE(hidden % 8 == 0 && hidden <= 0x7fffffffLL && topk <= 0x7fffffffLL,
               "moe_sum_reduce: hidden size (%lld) must be a multiple of 8", (long long)hidden);
  FP8K_REQUIRE(stride_token % 8 == 0 && stride_topk % 8 == 0 && out_stride_token % 8 == 0 && stride_topk >= hidden &&
                   out_stride_token >= hidden,
               "moe_sum_reduce: strides must be multiples of 8 elements and cover a row");
  if (tokens == 0 || hidden == 0) return FP8K_OK;
  FP8K_REQUIRE(x && out, "moe_sum_reduce: null pointer");
  FP8K_REQUIRE(aligned(x, 16) && aligned(out, 16), "moe_sum_reduce: pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(stream_grid(tokens * (hidden / 8))), block(256);
#define FP8K_SR(DT)                                                                                                         \
  do {                                                                                                                      \
    if (elem)                                                                                                               \
      hipLaunchKernelGGL((moe_sum_reduce_kernel<DT, true>), grid, block, 0, st, x, out, tokens, (int)topk, (int)hidden,     \
                         stride_token, stride_topk, out_stride_token, scale);                                               \
    else                                                                                                                    \
      hipLaunchKernelGGL((moe_sum_reduce_kernel<DT, false>), grid, block, 0, st, x, out, tokens, (int)topk, (int)hidden,    \
                         stride_token, stride_topk, out_stride_token, scale);                                               \
  } while (0)
  switch (dtype) {
    case FP8K_BF16: FP8K_SR(FP8K_BF16); break;
    case FP8K_F16: FP8K_SR(FP8K_F16); break;
    default: FP8K_SR(FP8K_F32); break;
  }
#undef FP8K_SR
  return check_launch("moe_sum_reduce");
}

extern "C" int fp8k_moe_sum_reduce(const void* x, void* out, int64_t tokens, int64_t topk, int64_t hidden,
                                   int64_t stride_token, int64_t stride_topk, int64_t out_stride_token, float scale,
                                   int dtype, void* stream) {
  clear_error();
  return moe_sum_impl(x, out, tokens, topk, hidden, stride_token, stride_topk, out_stride_token, scale, dtype, false, stream);
}

extern "C" int fp8k_moe_sum(const void* x, void* out, int64_t tokens, int64_t topk, int64_t hidden, int64_t stride_token,
                            int64_t stride_topk, int64_t out_stride_token, int dtype, void* stream) {
  clear_error();
  // 2, 3 and 4 experts per token: one rounding to the element type per addition; otherwise the float-accumulated sum
  return moe_sum_impl(x, out, tokens, topk, hidden, stride_token, stride_topk, out_stride_token, 1.0f, dtype,
                      topk >= 2 && topk <= 4, stream);
}

// ------------------------------------------------------------------------------------------------
// moe_fused_gate: grouped top-k routing with a selection bias (DeepSeek-V3 style), one token per sub-group of
// TPR = num_expert_group lanes, VPT = experts / groups values per lane (a lane holds one whole expert group).
//   score  = T(sigmoid(x));  choice = T(score + bias)                       (arithmetic in the input type T)
//   group weight = T(top1 + top2 of choice inside the group); the groups with the smallest weight are dropped
//   one at a time until topk_group remain (ties: the higher group goes), then the topk best choices among the
//   remaining groups are taken one at a time (ties: the lower expert wins).  Weights are the un-biased scores,
//   renormalised to sum 1 (shared experts, if any, are appended with weight sum / routed_scaling_factor before
//   the renormalisation), optionally times routed_scaling_factor.
// ------------------------------------------------------------------------------------------------
template <int DT>
__device__ __forceinline__ float gate_load(const void* p, int64_t i) {
  if (DT == FP8K_F32) return ((const float*)p)[i];
  if (DT == FP8K_BF16) return __uint_as_float((uint32_t)((const u16*)p)[i] << 16);
  return f16_bits_to_f32(((const u16*)p)[i]);
}

template <int DT, int VPT>
__global__ __launch_bounds__(256) void moe_fused_gate_kernel(const void* __restrict__ input, const void* __restrict__ bias,
                                                             float* __restrict__ out_w, int32_t* __restrict__ out_i,
                                                             int64_t num_rows, int tpr, int topk_group, int topk,
                                                             int num_shared, double rsf, int scale_output) {
  const int lane_in_row = threadIdx.x % tpr;
  const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) / tpr;
  const bool live = row < num_rows;            // dead sub-groups run along (shuffles stay inside a sub-group)
  const int first = lane_in_row * VPT;
  const int experts = tpr * VPT;
  const float kCleared = __builtin_inff();

  float score[VPT], choice[VPT];
  {
    float xin[VPT], bin[VPT];
    constexpr int kPer16 = DT == FP8K_F32 ? 4 : 8;  // elements per 16-byte load
    if constexpr (VPT % kPer16 == 0) {
      // a lane's VPT values are contiguous: 16-byte loads (rows and the lane's offset are multiples of VPT elements)
#pragma unroll
      for (int c = 0; c < VPT / kPer16; ++c) {
        const int64_t at = (live ? row * experts : 0) + first + c * kPer16;
        if constexpr (DT == FP8K_F32) {
          const float4 a = *reinterpret_cast<const float4*>((const float*)input + at);
          const float4 b = *reinterpret_cast<const float4*>((const float*)bias + first + c * 4);
          xin[c * 4] = a.x; xin[c * 4 + 1] = a.y; xin[c * 4 + 2] = a.z; xin[c * 4 + 3] = a.w;
          bin[c * 4] = b.x; bin[c * 4 + 1] = b.y; bin[c * 4 + 2] = b.z; bin[c * 4 + 3] = b.w;
        } else {
          load8<DT>(input, at, *reinterpret_cast<float(*)[8]>(&xin[c * 8]));
          load8<DT>(bias, first + c * 8, *reinterpret_cast<float(*)[8]>(&bin[c * 8]));
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        xin[i] = live ? gate_load<DT>(input, row * experts + first + i) : 0.f;
        bin[i] = gate_load<DT>(bias, first + i);
      }
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      score[i] = round_to<DT>(1.0f / (1.0f + expf(-xin[i])));
      choice[i] = round_to<DT>(score[i] + bin[i]);
    }
  }

  // drop the weakest groups: a group's weight does not change while other groups are dropped
  {
    float m1 = -__builtin_inff(), m2 = -__builtin_inff();
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const float v = choice[i];
      if (v > m1) { m2 = m1; m1 = v; }
      else if (v > m2) m2 = v;
    }
    const float gsum = VPT > 1 ? round_to<DT>(m1 + m2) : m1;
    bool dropped = false;
    for (int k = 0; k < tpr - topk_group; ++k) {
      float sum = dropped ? kCleared : gsum;
      int grp = lane_in_row;
      for (int mask = tpr >> 1; mask > 0; mask >>= 1) {
        const float osum = __shfl_xor(sum, mask, tpr);
        const int ogrp = __shfl_xor(grp, mask, tpr);
        if (sum > osum || (osum == sum && ogrp > grp)) { sum = osum; grp = ogrp; }
      }
      dropped = dropped || lane_in_row == grp;
    }
    if (dropped) {
#pragma unroll
      for (int i = 0; i < VPT; ++i) choice[i] = kCleared;
    }
  }

  // pick k is kept by lane k % tpr of the row in slot k / tpr, so that the row's lanes write their entries
  // side by side once the normaliser is known
  constexpr int kSlots = 4;
  float keep_w[kSlots];
  int keep_i[kSlots];
#pragma unroll
  for (int j = 0; j < kSlots; ++j) { keep_w[j] = 0.f; keep_i[j] = 0; }
  const int take = topk - num_shared;
  float wsum = 0.f;
  for (int k = 0; k < take; ++k) {
    // local argmax as a tree (the lower index wins ties, as a left-to-right scan would have it)
    float tv[VPT];
    int ti[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) { tv[i] = choice[i]; ti[i] = first + i; }
#pragma unroll
    for (int stride = 1; stride < VPT; stride *= 2) {
#pragma unroll
      for (int i = 0; i + stride < VPT; i += 2 * stride) {
        if (tv[i + stride] > tv[i]) { tv[i] = tv[i + stride]; ti[i] = ti[i + stride]; }
      }
    }
    float best = tv[0];
    int idx = ti[0];
    if (choice[0] == kCleared) { best = -__builtin_inff(); idx = first; }
    for (int mask = tpr >> 1; mask > 0; mask >>= 1) {
      const float obest = __shfl_xor(best, mask, tpr);
      const int oidx = __shfl_xor(idx, mask, tpr);
      if (obest > best || (obest == best && oidx < idx)) { best = obest; idx = oidx; }
    }
    const int owner = idx / VPT, slot = idx - owner * VPT;
    float w = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      if (i == slot) {
        w = score[i];
        if (lane_in_row == owner) choice[i] = -__builtin_inff();
      }
    }
    w = __shfl(w, owner, tpr);
    wsum += w;
    const bool mine = lane_in_row == k % tpr;
    const int slot_k = k / tpr;
#pragma unroll
    for (int j = 0; j < kSlots; ++j) {
      if (mine && j == slot_k) { keep_w[j] = w; keep_i[j] = idx; }
    }
  }
  if (!live) return;
#pragma unroll
  for (int j = 0; j < kSlots; ++j) {
    const int k = j * tpr + lane_in_row;
    float w = keep_w[j];
    int id = keep_i[j];
    if (k >= take) {  // shared experts follow the routed ones
      w = (float)((double)wsum / rsf);
      id = experts + (k - take);
    }
    if (k < topk) {
      w = w / wsum;
      if (scale_output) w = (float)((double)w * rsf);
      out_w[row * topk + k] = w;
      out_i[row * topk + k] = id;
    }
  }
}

extern "C" int fp8k_moe_fused_gate(const void* input, const void* bias, float* topk_weights, int32_t* topk_ids,
                                   int64_t num_rows, int64_t num_experts, int64_t num_expert_group, int64_t topk_group,
                                   int64_t topk, int64_t num_fused_shared_experts, double routed_scaling_factor,
                                   int apply_routed_scaling_factor_on_output, int dtype, void* stream) {
  clear_error();
  const char* op = "moe_fused_gate";
  FP8K_REQUIRE(num_rows >= 0 && num_experts > 0 && num_expert_group > 0, "%s: bad shape", op);
  FP8K_REQUIRE(dtype == FP8K_F32 || dtype == FP8K_F16 || dtype == FP8K_BF16, "%s: bad dtype %d", op, dtype);
  FP8K_REQUIRE((num_experts & (num_experts - 1)) == 0, "%s: num_experts must be a power of 2, but got %lld", op,
               (long long)num_experts);
  FP8K_REQUIRE(num_experts % num_expert_group == 0, "%s: num_experts must be divisible by num_expert_group, but got %lld / %lld",
               op, (long long)num_experts, (long long)num_expert_group);
  const int64_t vpt = num_experts / num_expert_group;
  FP8K_REQUIRE(vpt <= 32, "%s: Per group experts: num_experts / num_expert_group = (%lld) exceeds the maximum supported (32)",
               op, (long long)vpt);
  FP8K_REQUIRE(num_expert_group <= 64, "%s: at most 64 expert groups (got %lld)", op, (long long)num_expert_group);
  FP8K_REQUIRE(topk_group >= 1 && topk_group <= num_expert_group, "%s: topk_group out of range", op);
  FP8K_REQUIRE(num_fused_shared_experts >= 0 && topk > num_fused_shared_experts &&
                   topk - num_fused_shared_experts <= topk_group * vpt,
               "%s: topk (%lld) does not fit the experts of the selected groups", op, (long long)topk);
  FP8K_REQUIRE(topk <= 4 * num_expert_group, "%s: topk (%lld) larger than 4 x num_expert_group is not built", op, (long long)topk);
  FP8K_REQUIRE(num_fused_shared_experts == 0 || routed_scaling_factor != 0.0,
               "%s: shared experts need a non-zero routed_scaling_factor", op);
  if (num_rows == 0) return FP8K_OK;
  FP8K_REQUIRE(input && bias && topk_weights && topk_ids, "%s: null pointer", op);
  FP8K_REQUIRE(num_rows * num_experts < (1LL << 40), "%s: input too large", op);
  FP8K_REQUIRE(aligned(input, 16) && aligned(bias, 16), "%s: input and bias must be 16-byte aligned", op);
  hipStream_t st = (hipStream_t)stream;
  const int64_t lanes = num_rows * num_expert_group;
  const dim3 grid((unsigned)((lanes + 255) / 256)), block(256);
#define FP8K_GATE2(DT, V)                                                                                              \
  hipLaunchKernelGGL((moe_fused_gate_kernel<DT, V>), grid, block, 0, st, input, bias, topk_weights, topk_ids, num_rows, \
                     (int)num_expert_group, (int)topk_group, (int)topk, (int)num_fused_shared_experts,                  \
                     routed_scaling_factor, apply_routed_scaling_factor_on_output)
#define FP8K_GATE(DT)                \
  switch (vpt) {                     \
    case 1: FP8K_GATE2(DT, 1); break;   \
    case 2: FP8K_GATE2(DT, 2); break;   \
    case 4: FP8K_GATE2(DT, 4); break;   \
    case 8: FP8K_GATE2(DT, 8); break;   \
    case 16: FP8K_GATE2(DT, 16); break; \
    default: FP8K_GATE2(DT, 32); break; \
  }
  switch (dtype) {
    case FP8K_BF16: FP8K_GATE(FP8K_BF16); break;
    case FP8K_F16: FP8K_GATE(FP8K_F16); break;
    default: FP8K_GATE(FP8K_F32); break;
  }
#undef FP8K_GATE
#undef FP8K_GATE2
  return check_launch(op);
}

namespace fp8k {

// ------------------------------------------------------------------------------------------------
// Expert-major MoE layout: the rows of every expert contiguous and un-padded, described by start offsets.
//
// moe_prepare_kernel: one workgroup.  Histogram of the expert of every (token, k) slot with LDS atomics, exclusive
// scan by the first wavefront, then every slot takes the next free row of its expert (LDS cursor): the order of
// the rows inside an expert is not defined, the rows themselves do not depend on it.
//   expert_offsets [E + 1], optional blockscale_offsets [E + 1] (counts rounded up to 128),
//   problem_sizes1 [E, 3] = (rows, 2n, k), problem_sizes2 [E, 3] = (rows, k, n),
//   input_permutation[row] = token of the slot in that row, output_permutation[slot] = row.
// Ids outside [0, E) take no row and leave their output_permutation entry untouched.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kAlignThreads) void moe_prepare_kernel(const int32_t* __restrict__ ids, int numel, int topk,
                                                                    int E, int n, int k, int32_t* __restrict__ offsets,
                                                                    int32_t* __restrict__ bs_offsets,
                                                                    int32_t* __restrict__ ps1, int32_t* __restrict__ ps2,
                                                                    int32_t* __restrict__ in_perm,
                                                                    int32_t* __restrict__ out_perm) {
  __shared__ int32_t counts[kAlignMaxBuckets];
  __shared__ int32_t cursor[kAlignMaxBuckets];
  __shared__ int32_t rounded[kAlignMaxBuckets];
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += kAlignThreads) counts[e] = 0;
  __syncthreads();
  // eight ids per lane and trip: eight loads in flight instead of one load latency per id
  for (int i0 = tid; i0 < numel; i0 += 8 * kAlignThreads) {
    int e8[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kAlignThreads;
      e8[u] = i < numel ? ids[i] : -1;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (e8[u] >= 0 && e8[u] < E) atomicAdd(&counts[e8[u]], 1);
  }
  __syncthreads();
  if (tid < 64) {
    const int per = (E + 63) / 64;
    const int e0 = tid * per, e1 = min(E, e0 + per);
    int sum = 0, rsum = 0;
    for (int e = e0; e < e1; ++e) { sum += counts[e]; rsum += (counts[e] + 127) / 128 * 128; }
    int incl = sum, rincl = rsum;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int v = __shfl_up(incl, off), rv = __shfl_up(rincl, off);
      if (tid >= off) { incl += v; rincl += rv; }
    }
    int run = incl - sum, rrun = rincl - rsum;
    for (int e = e0; e < e1; ++e) {
      cursor[e] = run; rounded[e] = rrun;
      run += counts[e]; rrun += (counts[e] + 127) / 128 * 128;
    }
    if (tid == 63) { offsets[E] = incl; if (bs_offsets) bs_offsets[E] = rincl; }
  }
  __syncthreads();
  for (int e = tid; e < E; e += kAlignThreads) {
    offsets[e] = cursor[e];
    if (bs_offsets) bs_offsets[e] = rounded[e];
    ps1[e * 3] = counts[e]; ps1[e * 3 + 1] = 2 * n; ps1[e * 3 + 2] = k;
    ps2[e * 3] = counts[e]; ps2[e * 3 + 1] = k; ps2[e * 3 + 2] = n;
  }
  __syncthreads();
  for (int i0 = tid; i0 < numel; i0 += 8 * kAlignThreads) {
    int e8[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kAlignThreads;
      e8[u] = i < numel ? ids[i] : -1;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int e = e8[u], i = i0 + u * kAlignThreads;
      if (e >= 0 && e < E) {
        const int row = atomicAdd(&cursor[e], 1);
        in_perm[row] = i / topk;
        out_perm[i] = row;
      }
    }
  }
}

// Many ids (more than kAlignFusedMax): the same in four launches over workgroups that take kAlignChunk ids each, with the
// caller's outputs as the only memory.  The row counts are summed up in problem_sizes1[e, 0] (zeroed first), one
// workgroup turns them into offsets and sizes, and the placing workgroups reserve their share of an expert's rows with one
// global atomic on the cell AFTER the expert's own in expert_offsets: that cell starts at the expert's first row and,
// once every row of the expert is handed out, holds the first row of the next expert - its final value.
__global__ __launch_bounds__(kAlignThreads) void moe_prepare_count_kernel(const int32_t* __restrict__ ids, int numel, int E,
                                                                          int32_t* __restrict__ ps1) {
  __shared__ int32_t counts[kAlignMaxBuckets];
  for (int e = threadIdx.x; e < E; e += kAlignThreads) counts[e] = 0;
  __syncthreads();
  const int first = blockIdx.x * kAlignChunk, last = min(numel, first + kAlignChunk);
  for (int i0 = first + threadIdx.x; i0 < last; i0 += 8 * kAlignThreads) {
    int e8[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kAlignThreads;
      e8[u] = i < last ? ids[i] : -1;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (e8[u] >= 0 && e8[u] < E) atomicAdd(&counts[e8[u]], 1);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += kAlignThreads)
    if (counts[e]) atomicAdd(&ps1[e * 3], counts[e]);
}
__global__ __launch_bounds__(kAlignThreads) void moe_prepare_scan_kernel(int E, int n, int k, int32_t* __restrict__ offsets,
                                                                         int32_t* __restrict__ bs_offsets,
                                                                         int32_t* __restrict__ ps1, int32_t* __restrict__ ps2) {
  __shared__ int32_t counts[kAlignMaxBuckets];
  __shared__ int32_t start[kAlignMaxBuckets];
  __shared__ int32_t rounded[kAlignMaxBuckets];
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += kAlignThreads) counts[e] = ps1[e * 3];
  __syncthreads();
  if (tid < 64) {
    const int per = (E + 63) / 64;
    const int e0 = tid * per, e1 = min(E, e0 + per);
    int sum = 0, rsum = 0;
    for (int e = e0; e < e1; ++e) { sum += counts[e]; rsum += (counts[e] + 127) / 128 * 128; }
    int incl = sum, rincl = rsum;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int v = __shfl_up(incl, off), rv = __shfl_up(rincl, off);
      if (tid >= off) { incl += v; rincl += rv; }
    }
    int run = incl - sum, rrun = rincl - rsum;
    for (int e = e0; e < e1; ++e) {
      start[e] = run; rounded[e] = rrun;
      run += counts[e]; rrun += (counts[e] + 127) / 128 * 128;
    }
    if (tid == 63 && bs_offsets) bs_offsets[E] = rincl;
  }
  __syncthreads();
  if (tid == 0) offsets[0] = 0;
  for (int e = tid; e < E; e += kAlignThreads) {
    offsets[e + 1] = start[e];  // the cursor of expert e; its final value is the start of expert e + 1
    if (bs_offsets) bs_offsets[e] = rounded[e];
    ps1[e * 3 + 1] = 2 * n; ps1[e * 3 + 2] = k;
    ps2[e * 3] = counts[e]; ps2[e * 3 + 1] = k; ps2[e * 3 + 2] = n;
  }
}
__global__ __launch_bounds__(kAlignThreads) void moe_prepare_place_kernel(const int32_t* __restrict__ ids, int numel, int topk,
                                                                          int E, int32_t* __restrict__ offsets,
                                                                          int32_t* __restrict__ in_perm,
                                                                          int32_t* __restrict__ out_perm) {
  __shared__ int32_t cursor[kAlignMaxBuckets];
  for (int e = threadIdx.x; e < E; e += kAlignThreads) cursor[e] = 0;
  __syncthreads();
  const int first = blockIdx.x * kAlignChunk, last = min(numel, first + kAlignChunk);
  for (int i0 = first + threadIdx.x; i0 < last; i0 += 8 * kAlignThreads) {
    int e8[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kAlignThreads;
      e8[u] = i < last ? ids[i] : -1;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (e8[u] >= 0 && e8[u] < E) atomicAdd(&cursor[e8[u]], 1);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += kAlignThreads) {
    const int c = cursor[e];
    cursor[e] = c ? atomicAdd(&offsets[e + 1], c) : 0;  // from here on the workgroup's next free row of expert e
  }
  __syncthreads();
  for (int i0 = first + threadIdx.x; i0 < last; i0 += 8 * kAlignThreads) {
    int e8[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kAlignThreads;
      e8[u] = i < last ? ids[i] : -1;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int e = e8[u], i = i0 + u * kAlignThreads;
      if (e >= 0 && e < E) {
        const int row = atomicAdd(&cursor[e], 1);
        in_perm[row] = i / topk;
        out_perm[i] = row;
      }
    }
  }
}

// out[d, :] = in[map[d], :], rows moved in units of T (16 bytes a lane when the rows allow it); a map entry outside
// [0, src_rows) leaves its destination row untouched.
template <typename T>
__global__ __launch_bounds__(256) void shuffle_rows_kernel(const T* __restrict__ in, const int32_t* __restrict__ map,
                                                           T* __restrict__ out, int64_t src_rows, int64_t dst_rows,
                                                           int chunks) {
  const int64_t total = dst_rows * chunks;
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += step) {
    const int64_t d = i / chunks;
    const int c = (int)(i - d * chunks);
    const int64_t s = map[d];
    if (s >= 0 && s < src_rows) out[d * chunks + c] = in[s * chunks + c];
  }
}

// out[t, :] = T( sum_j float(factor[t * topk + j]) * float(in[perm[t * topk + j], :]) ), ascending j, float32 sum
template <int DT>
__global__ __launch_bounds__(256) void shuffle_mul_sum_kernel(const void* __restrict__ in, void* __restrict__ out,
                                                              const int32_t* __restrict__ perm, const void* __restrict__ factors,
                                                              int64_t m, int topk, int cols, int64_t in_rows) {
  const int chunks = cols / 8;
  const int64_t total = m * chunks;
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += step) {
    const int64_t t = i / chunks;
    const int c = (int)(i - t * chunks) * 8;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < topk; ++j) {
      const int64_t slot = t * topk + j;
      const int64_t r = perm ? perm[slot] : slot;
      if (r < 0 || r >= in_rows) continue;
      float f = 1.0f;
      if (factors) {
        if (DT == FP8K_F32) f = ((const float*)factors)[slot];
        else if (DT == FP8K_BF16) f = __uint_as_float((uint32_t)((const u16*)factors)[slot] << 16);
        else f = f16_bits_to_f32(((const u16*)factors)[slot]);
      }
      float v[8];
      load8<DT>(in, r * cols + c, v);
#pragma unroll
      for (int q = 0; q < 8; ++q) acc[q] = fmaf(f, v[q], acc[q]);
    }
    store8<DT>(out, t * cols + c, acc);
  }
}

// Block table of the grouped GEMM for the expert-major layout: expert e owns rows [starts[e], starts[e] + sizes[3e]).
// Every expert's rows are cut into blocks of `block` slots (the last one padded with the id `rows`), experts in
// ascending order.  One workgroup: scan of the block counts by the first wavefront, then one pass over the slots.
// With slot_expert / slot_row given (the routed expert of every (token, k) slot and the expert-major row that
// moe_prepare_kernel gave it) the table holds the SLOT at the position of its row, padded with num_slots: the grouped
// GEMM then gathers token slot / top_k straight from the un-shuffled activations and writes its rows in slot order.
template <bool SCATTER>
__global__ __launch_bounds__(kAlignThreads) void moe_offset_blocks_kernel(const int32_t* __restrict__ starts,
                                                                          const int32_t* __restrict__ sizes, int E, int rows,
                                                                          int block, int32_t* __restrict__ sorted,
                                                                          int32_t* __restrict__ expert_ids,
                                                                          int32_t* __restrict__ post_pad, int max_blocks,
                                                                          const int32_t* __restrict__ slot_expert,
                                                                          const int32_t* __restrict__ slot_row,
                                                                          int num_slots) {
  // Every workgroup scans the experts' block counts for itself (a few hundred values) and then takes its share of the
  // work.  SCATTER = false: the blocks - the expert of each and its entries (rows, or with slot_row given the padding
  // value num_slots in every entry); SCATTER = true, a second launch behind the first: the slots, each to the position of
  // its row, so that a position no slot claims keeps the padding value.
  __shared__ int32_t first_block[kAlignMaxBuckets + 1];
  __shared__ int32_t lstart[kAlignMaxBuckets], lsize[kAlignMaxBuckets];  // the experts' first rows and row counts
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += kAlignThreads) { lstart[e] = starts[e]; lsize[e] = max(sizes[e * 3], 0); }
  __syncthreads();
  if (tid < 64) {
    const int per = (E + 63) / 64;
    const int e0 = tid * per, e1 = min(E, e0 + per);
    int sum = 0;
    for (int e = e0; e < e1; ++e) sum += (lsize[e] + block - 1) / block;
    int incl = sum;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int v = __shfl_up(incl, off);
      if (tid >= off) incl += v;
    }
    int run = incl - sum;
    for (int e = e0; e < e1; ++e) {
      first_block[e] = run;
      run += (lsize[e] + block - 1) / block;
    }
    if (tid == 63) first_block[E] = incl;
  }
  __syncthreads();
  const int nblocks = min(first_block[E], max_blocks);
  const int total = nblocks * block;
  if (!SCATTER) {
    if (blockIdx.x == 0 && tid == 0) post_pad[0] = nblocks * block;
    // one wavefront per block: its expert by a search that is uniform across the wave, then the block's entries with
    // consecutive lanes on consecutive entries (a search per entry cost 60 us at 190 000 entries)
    const int waves = kAlignThreads / 64, wave = blockIdx.x * waves + (tid >> 6), ln = tid & 63;
    for (int b = wave; b < nblocks; b += gridDim.x * waves) {
      int lo = 0, hi = E;  // first expert with first_block[e + 1] > b
      while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (first_block[mid + 1] <= b) lo = mid + 1;
        else hi = mid;
      }
      if (ln == 0) expert_ids[b] = lo;
      const int base = (b - first_block[lo]) * block, st = lstart[lo], sz = lsize[lo];
      for (int j = ln; j < block; j += 64) {
        const int within = base + j, row = st + within;
        sorted[b * block + j] = slot_row ? num_slots : ((within < sz && row >= 0 && row < rows) ? row : rows);
      }
    }
    return;
  }
  for (int i0 = blockIdx.x * 8 * kAlignThreads + tid; i0 < num_slots; i0 += gridDim.x * 8 * kAlignThreads) {
    int e8[8], r8[8];  // eight loads of each table in flight
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kAlignThreads;
      e8[u] = i < num_slots ? slot_expert[i] : -1;
      r8[u] = i < num_slots ? slot_row[i] : 0;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int e = e8[u];
      if (e < 0 || e >= E) continue;
      const int within = r8[u] - lstart[e];
      if (within < 0 || within >= lsize[e]) continue;
      const int64_t pos = (int64_t)first_block[e] * block + within;
      if (pos < total) sorted[pos] = i0 + u * kAlignThreads;
    }
  }
}

}  // namespace fp8k

extern "C" int fp8k_moe_prepare_input(const int32_t* topk_ids, int64_t numel, int64_t topk, int64_t num_experts, int64_t n,
                                      int64_t k, int32_t* expert_offsets, int32_t* blockscale_offsets,
                                      int32_t* problem_sizes1, int32_t* problem_sizes2, int32_t* input_permutation,
                                      int32_t* output_permutation, void* stream) {
  clear_error();
  const char* op = "prepare_moe_input";
  FP8K_REQUIRE(numel >= 0 && numel < 0x7fffffffLL && topk >= 1 && numel % topk == 0,
               "%s: topk_ids must hold a whole number of rows of topk ids (numel %lld, topk %lld)", op, (long long)numel,
               (long long)topk);
  FP8K_REQUIRE(num_experts >= 1 && num_experts <= kAlignMaxBuckets, "%s: num_experts must be in [1, %d] (got %lld)", op,
               kAlignMaxBuckets, (long long)num_experts);
  FP8K_REQUIRE(n >= 0 && k >= 0 && 2 * n <= 0x7fffffffLL && k <= 0x7fffffffLL, "%s: bad n / k", op);
  FP8K_REQUIRE(expert_offsets && problem_sizes1 && problem_sizes2, "%s: null output pointer", op);
  FP8K_REQUIRE(numel == 0 || (topk_ids && input_permutation && output_permutation), "%s: null pointer", op);
  hipStream_t st = (hipStream_t)stream;
  if (numel <= kAlignFusedMax) {
    hipLaunchKernelGGL(moe_prepare_kernel, dim3(1), dim3(kAlignThreads), 0, st, topk_ids, (int)numel, (int)topk,
                       (int)num_experts, (int)n, (int)k, expert_offsets, blockscale_offsets, problem_sizes1, problem_sizes2,
                       input_permutation, output_permutation);
    return check_launch(op);
  }
  const int E = (int)num_experts;
  const unsigned chunks = (unsigned)((numel + kAlignChunk - 1) / kAlignChunk);
  hipLaunchKernelGGL(zero_ints_kernel, dim3((3 * E + 255) / 256), dim3(256), 0, st, problem_sizes1, 3 * E);
  hipLaunchKernelGGL(moe_prepare_count_kernel, dim3(chunks), dim3(kAlignThreads), 0, st, topk_ids, (int)numel, E, problem_sizes1);
  hipLaunchKernelGGL(moe_prepare_scan_kernel, dim3(1), dim3(kAlignThreads), 0, st, E, (int)n, (int)k, expert_offsets,
                     blockscale_offsets, problem_sizes1, problem_sizes2);
  hipLaunchKernelGGL(moe_prepare_place_kernel, dim3(chunks), dim3(kAlignThreads), 0, st, topk_ids, (int)numel, (int)topk, E,
                     expert_offsets, input_permutation, output_permutation);
  return check_launch(op);
}

extern "C" int fp8k_shuffle_rows(const void* input, const int32_t* dst2src_map, void* output, int64_t src_rows,
                                 int64_t dst_rows, int64_t row_bytes, void* stream) {
  clear_error();
  const char* op = "shuffle_rows";
  FP8K_REQUIRE(src_rows >= 0 && dst_rows >= 0 && row_bytes >= 0, "%s: negative shape", op);
  FP8K_REQUIRE(row_bytes <= 0x7fffffffLL, "%s: rows longer than 2 GiB are not supported", op);
  if (dst_rows == 0 || row_bytes == 0) return FP8K_OK;
  FP8K_REQUIRE(input && dst2src_map && output, "%s: null pointer", op);
  hipStream_t st = (hipStream_t)stream;
#define FP8K_SHUF(T)                                                                                                       \
  hipLaunchKernelGGL(shuffle_rows_kernel<T>, dim3(stream_grid(dst_rows * (row_bytes / (int64_t)sizeof(T)))), dim3(256), 0, \
                     st, (const T*)input, dst2src_map, (T*)output, src_rows, dst_rows, (int)(row_bytes / (int64_t)sizeof(T)))
  if (row_bytes % 16 == 0 && aligned(input, 16) && aligned(output, 16)) FP8K_SHUF(uint4);
  else if (row_bytes % 4 == 0 && aligned(input, 4) && aligned(output, 4)) FP8K_SHUF(uint32_t);
  else FP8K_SHUF(uint8_t);
#undef FP8K_SHUF
  return check_launch(op);
}

extern "C" int fp8k_apply_shuffle_mul_sum(const void* input, void* output, const int32_t* permutation, const void* factors,
                                          int64_t m, int64_t topk, int64_t cols, int64_t input_rows, int dtype, void* stream) {
  clear_error();
  const char* op = "apply_shuffle_mul_sum";
  FP8K_REQUIRE(m >= 0 && topk >= 0 && cols >= 0 && input_rows >= 0 && topk <= 0x7fffffffLL, "%s: negative shape", op);
  FP8K_REQUIRE(dtype == FP8K_F32 || dtype == FP8K_F16 || dtype == FP8K_BF16, "%s: bad dtype %d", op, dtype);
  FP8K_REQUIRE(cols % 8 == 0 && cols <= 0x7fffffffLL, "%s: the row length (%lld) must be a multiple of 8", op, (long long)cols);
  if (m == 0 || cols == 0) return FP8K_OK;
  FP8K_REQUIRE(output && (topk == 0 || input), "%s: null pointer", op);
  FP8K_REQUIRE(aligned(input, 16) && aligned(output, 16), "%s: pointers must be 16-byte aligned", op);
  const dim3 grid(stream_grid(m * (cols / 8))), block(256);
  hipStream_t st = (hipStream_t)stream;
#define FP8K_SMS(DT) \
  hipLaunchKernelGGL(shuffle_mul_sum_kernel<DT>, grid, block, 0, st, input, output, permutation, factors, m, (int)topk, (int)cols, input_rows)
  switch (dtype) {
    case FP8K_BF16: FP8K_SMS(FP8K_BF16); break;
    case FP8K_F16: FP8K_SMS(FP8K_F16); break;
    default: FP8K_SMS(FP8K_F32); break;
  }
#undef FP8K_SMS
  return check_launch(op);
}

extern "C" int fp8k_moe_blocks_from_offsets(const int32_t* expert_starts, const int32_t* problem_sizes, int64_t num_experts,
                                            int64_t rows, int64_t block_m, int32_t* sorted_token_ids, int64_t sorted_capacity,
                                            int32_t* expert_ids, int64_t expert_capacity, int32_t* num_tokens_post_pad,
                                            void* stream) {
  clear_error();
  const char* op = "moe_blocks_from_offsets";
  FP8K_REQUIRE(num_experts >= 1 && num_experts <= kAlignMaxBuckets, "%s: num_experts must be in [1, %d] (got %lld)", op,
               kAlignMaxBuckets, (long long)num_experts);
  FP8K_REQUIRE(rows >= 0 && rows < 0x7fffffffLL && block_m >= 1 && block_m <= 1024, "%s: bad rows / block size", op);
  FP8K_REQUIRE(expert_starts && problem_sizes && sorted_token_ids && expert_ids && num_tokens_post_pad, "%s: null pointer", op);
  // the kernel never writes past the capacities (blocks beyond them are dropped); sizes that sum to `rows` need at most this
  const int64_t used = rows < num_experts ? rows : num_experts;
  const int64_t worst = rows + used * (block_m - 1);
  FP8K_REQUIRE(sorted_capacity >= worst / block_m * block_m && expert_capacity >= worst / block_m,
               "%s: block table too small (%lld slots, %lld blocks; %lld slots may be needed)", op, (long long)sorted_capacity,
               (long long)expert_capacity, (long long)(worst / block_m * block_m));
  const int64_t max_blocks = sorted_capacity / block_m < expert_capacity ? sorted_capacity / block_m : expert_capacity;
  const int64_t worst_blocks = std::min<int64_t>(worst / block_m, max_blocks);
  const unsigned grid = (unsigned)std::max<int64_t>(1, std::min<int64_t>(64, (worst_blocks + 63) / 64));
  hipLaunchKernelGGL(moe_offset_blocks_kernel<false>, dim3(grid), dim3(kAlignThreads), 0, (hipStream_t)stream, expert_starts,
                     problem_sizes, (int)num_experts, (int)rows, (int)block_m, sorted_token_ids, expert_ids,
                     num_tokens_post_pad, (int)(max_blocks > 0x7fffffffLL ? 0x7fffffffLL : max_blocks),
                     (const int32_t*)nullptr, (const int32_t*)nullptr, 0);
  return check_launch(op);
}

extern "C" int fp8k_moe_slot_blocks_from_offsets(const int32_t* expert_starts, const int32_t* problem_sizes,
                                                 int64_t num_experts, const int32_t* topk_ids, const int32_t* slot_rows,
                                                 int64_t num_slots, int64_t block_m, int32_t* sorted_token_ids,
                                                 int64_t sorted_capacity, int32_t* expert_ids, int64_t expert_capacity,
                                                 int32_t* num_tokens_post_pad, void* stream) {
  clear_error();
  const char* op = "moe_slot_blocks_from_offsets";
  FP8K_REQUIRE(num_experts >= 1 && num_experts <= kAlignMaxBuckets, "%s: num_experts must be in [1, %d] (got %lld)", op,
               kAlignMaxBuckets, (long long)num_experts);
  FP8K_REQUIRE(num_slots >= 0 && num_slots < 0x7fffffffLL && block_m >= 1 && block_m <= 1024, "%s: bad slot count / block size", op);
  FP8K_REQUIRE(expert_starts && problem_sizes && sorted_token_ids && expert_ids && num_tokens_post_pad, "%s: null pointer", op);
  FP8K_REQUIRE(num_slots == 0 || (topk_ids && slot_rows), "%s: null pointer", op);
  const int64_t used = num_slots < num_experts ? num_slots : num_experts;
  const int64_t worst = num_slots + used * (block_m - 1);
  FP8K_REQUIRE(sorted_capacity >= worst / block_m * block_m && expert_capacity >= worst / block_m,
               "%s: block table too small (%lld slots, %lld blocks; %lld slots may be needed)", op, (long long)sorted_capacity,
               (long long)expert_capacity, (long long)(worst / block_m * block_m));
  const int64_t max_blocks = sorted_capacity / block_m < expert_capacity ? sorted_capacity / block_m : expert_capacity;
  // slot_rows of an empty problem is never read: any non-null pointer keeps the kernel on its slot path
  const int64_t worst_blocks = std::min<int64_t>(worst / block_m, max_blocks);
  const unsigned grid = (unsigned)std::max<int64_t>(1, std::min<int64_t>(64, (worst_blocks + 63) / 64));
  const int mb = (int)(max_blocks > 0x7fffffffLL ? 0x7fffffffLL : max_blocks);
  const int32_t* rows_map = slot_rows ? slot_rows : expert_starts;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(moe_offset_blocks_kernel<false>, dim3(grid), dim3(kAlignThreads), 0, st, expert_starts, problem_sizes,
                     (int)num_experts, (int)num_slots, (int)block_m, sorted_token_ids, expert_ids, num_tokens_post_pad, mb,
                     topk_ids, rows_map, (int)num_slots);
  if (num_slots > 0) {  // behind the first launch: a slot lands on the padding value of its position
    const unsigned sgrid = (unsigned)std::max<int64_t>(1, std::min<int64_t>(64, (num_slots + 8 * kAlignThreads - 1) / (8 * kAlignThreads)));
    hipLaunchKernelGGL(moe_offset_blocks_kernel<true>, dim3(sgrid), dim3(kAlignThreads), 0, st, expert_starts, problem_sizes,
                       (int)num_experts, (int)num_slots, (int)block_m, sorted_token_ids, expert_ids, num_tokens_post_pad, mb,
                       topk_ids, rows_map, (int)num_slots);
  }
  return check_launch(op);
}
