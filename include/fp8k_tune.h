/*
 * fp8k_tune - tuning and measurement aids of the fp8k library.  None of them has a counterpart in the reference and no
 * product path calls them: bench.py and the tests use them to pin a kernel family, and to measure what the machine at
 * hand gives the load path and the matrix cores, the practical ceilings under the data-sheet peaks.
 * Conventions as in fp8k.h (status codes, fp8k_last_error, stream as void*).
 */
#ifndef FP8K_TUNE_H
#define FP8K_TUNE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Tuning and test aid (no counterpart in the reference): pins the kernel family that the dense GEMM entry points
 * pick for later calls made by the calling thread (the setting is thread-local; other threads keep the automatic
 * choice).  kind -1: automatic (the default).  kind 4: the 128x128 tile kernel with K
 * cut into `splits` runs (0 or 1: none).  kind 0: the choice by the number of rows alone, without the 128x128
 * kernel.  kind 1: 256x256 tiles; kind 2: the streaming kernel (up to 128 rows); kind 3: the direct kernel (up to 32
 * rows, `splits` > 0 pins its K cut too); kind 5: the direct kernel that cuts K across the waves of a workgroup (up to
 * 32 rows); where a pinned family cannot take the shape, the choice by rows stands.
 * `splits` is ignored for kinds 0..2.
 * kind -2: automatic, but the last round of 256x256 tiles is kept whole instead of being computed in 128-row halves.
 * fp8k_*_workspace_bytes, called from the same thread, follows the pinned choice.
 */
void fp8k_tune_force_gemm_plan(int kind, int splits);

/*
 * Measurement aid (no counterpart in the reference): streams `bytes` of device memory at `src` once through the load
 * path of the weight-streaming kernels - one workgroup of 8 wavefronts per CU, 32 KB stages of 16-byte-per-lane loads
 * straight into LDS, two stages in flight, a workgroup barrier per stage - and drops the data.  Timed by the caller, it
 * gives the read rate this load path reaches on the machine at hand, the practical ceiling under the 8 TB/s of the
 * data sheet.  `bytes` is rounded down to a multiple of 64 KB per CU; src 16-byte aligned; bytes < 2^40.
 */
int fp8k_tune_stream_read(const void* src, int64_t bytes, void* stream);

/*
 * Measurement aid (no counterpart in the reference): the same read stream in the shape a GEMM fetches a weight that was
 * NOT re-ordered after loading: the byte matrix [rows, pitch] at `src` is read as tiles of 256 rows, one K block (256
 * pieces of 128 bytes, `pitch` bytes apart) per 32 KB stage, each workgroup walking the K blocks of its
 * rows / 256 / CUs tiles.  Timed against fp8k_tune_stream_read on the same buffer it shows what a pre-shuffled
 * (tile-contiguous) copy of the weights could gain on this machine.  pitch a multiple of 128; rows are rounded down to
 * whole tiles per CU.
 */
int fp8k_tune_stream_read_tiles(const void* src, int64_t rows, int64_t pitch, void* stream);

/*
 * Measurement aid (no counterpart in the reference): fp8k_tune_stream_read with a write-out inside the stream.  After
 * every stages_per_tile stages of 32 KB ("a weight tile") each of the workgroup's 8 wavefronts stores stores_per_wave
 * times 1 KB (16 bytes a lane) to a place of its own in dst: 8 KB x stores_per_wave per tile and workgroup, the shape of
 * a weight-streaming GEMM that writes a small output tile per weight tile.  Timed by the caller against
 * stores_per_wave = 0 it shows what the stores cost the read stream.  `bytes` is rounded down to whole tiles per CU;
 * dst must hold CUs x tiles x 8 KB x stores_per_wave; both pointers 16-byte aligned.
 */
int fp8k_tune_stream_read_write(const void* src, int64_t bytes, void* dst, int64_t dst_bytes, int64_t stages_per_tile,
                                int64_t stores_per_wave, void* stream);

/*
 * Measurement aid: the bare matrix-core rate.  One workgroup of 8 wavefronts per CU; every wavefront loads six operand
 * fragments (2 KB each) of the caller's bytes once and then issues iters x 8 independent
 * v_mfma_f32_32x32x64 (e4m3 x e4m3) products of them with nothing else in the loop.  *flops receives the number of
 * floating-point operations the launch performs (2 x 32 x 32 x 64 per instruction); timed by the caller it gives the
 * rate the matrix cores sustain on this machine for THESE operand bytes - the power management clocks the chip by what
 * the data toggles, so random FP8 bytes and all-zero bytes give different ceilings.  sink receives one float per lane
 * (CUs x 512) so that the loop cannot be optimised away.
 */
int fp8k_tune_mfma_peak(const void* operands, int64_t bytes, int64_t iters, float* sink, int64_t sink_floats, int64_t* flops,
                        void* stream);

/*
 * Measurement aid (no counterpart in the reference): the K loop of the 256x256 block-scaled tile kernel built up from the
 * bare MFMA loop of fp8k_tune_mfma_peak one ingredient at a time, on operands that never change, in the tile kernel's
 * instruction order (16 MFMAs per wave and K block, 8 waves per CU).  form 1: the block-scaled product form (two MFMAs
 * into a short-lived accumulator, 16 scale FMAs fold it into the long-lived one); form 2: + the operand fragments
 * refilled from LDS behind their last use; form 3: + one LDS-only workgroup barrier per K block; form 4: + the eight
 * 1 KB global -> LDS stage loads per wave and K block (from the first 16 MiB of `operands`, cache-resident) and the
 * partial wait for them at the barrier; form 5: form 4 without the scale FMAs (the products accumulate in place, as in the
 * row-scaled and hardware-scaled modes); form 6: form 5 with 16 multiplies per 32x32 tile and K block in the place of
 * the FMAs (a loop that accumulates in place and rescales the accumulators between K blocks).  `iters` K blocks; *flops receives the matrix FLOPs of the launch.  Timed by the
 * caller, the steps down from form to form are what each ingredient costs the matrix cores.
 * operands 32-byte aligned, bytes >= 1 MiB; sink: CUs x 512 floats.
 */
int fp8k_tune_mfma_loop(const void* operands, int64_t bytes, int64_t iters, int form, float* sink, int64_t sink_floats,
                        int64_t* flops, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* FP8K_TUNE_H */
