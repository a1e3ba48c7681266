/* Measurement library of the gfx950 expert path (libnestor_hip_probes.so).
 *
 * Nothing here belongs to the drop-in interface (include/nestor_hip.h) and nothing
 * here has a counterpart in the reference: these entry points exist so that a
 * benchmark can put numbers of known size beside the product kernels' -- how the
 * hardware counters price the kernels' requests, what the matrix cores sustain with
 * no memory traffic, what the kernels' main loop reaches by itself, and which shader
 * clock the part holds under each GEMM.  The library also holds an instrumented
 * build of the bf16 grouped-GEMM translation unit (the same source compiled with
 * NESTOR_GEMM_CLOCK_HOOK=1): it exports the five nestor_hip_grouped_gemm_* entry
 * points of include/nestor_hip.h under their own names plus
 * nestor_hip_gemm_clock_sink, so a benchmark can run a GEMM through either library
 * on the same buffers.  The product library carries none of this.
 */
#ifndef NESTOR_HIP_PROBES_H_
#define NESTOR_HIP_PROBES_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------
 * Measurement aid (no counterpart in the reference): a stream of LDS-DMA
 * transfers over `rows` x `row_bytes` bytes at `src`, every byte fetched exactly
 * once, with the request shapes of the grouped GEMMs' operand fetches -- 1 KiB
 * per instruction as 1024 / piece_bytes consecutive rows x piece_bytes (64 ... 1024)
 * contiguous bytes, each wavefront walking along its rows (along_rows = 0) or down
 * its columns (along_rows = 1).  Run under `rocprofv3 --pmc FETCH_SIZE` it tells
 * how that counter prices such requests, which a plain copy kernel does not.
 * row_bytes % piece_bytes == 0 and rows % (1024 / piece_bytes) == 0; src_bytes is the
 * size of the buffer at src, and a walk that would leave it is refused (EINVAL)
 * before anything is launched.
 * ---------------------------------------------------------------------- */
int nestor_hip_dma_stream_probe(
    const void* src, int64_t src_bytes, int64_t rows, int64_t row_bytes, int32_t piece_bytes,
    int32_t along_rows, void* stream);

/* ------------------------------------------------------------------------
 * Measurement aids for the shader clock (no counterpart in the reference).  The
 * published matrix-core peak assumes the nominal clock; under a GEMM's load the
 * power management holds a lower one, and no profiler counter shows it.  A kernel
 * can: the ratio of its shader cycle counter to the constant-rate wall clock
 * (nestor_hip_wall_clock_khz ticks per millisecond) is the clock it ran at.
 *
 * nestor_hip_mfma_clock_probe: one workgroup per CU, four wavefronts each, issue
 * v_mfma_f32_32x32x16_bf16 back to back on 16 independent accumulator tiles with
 * no memory traffic, `iters` rounds; operands constant (random_operands = 0) or
 * random.  counters (device, 4 x uint64, the last one scratch) receives workgroup
 * 0's {shader cycles, wall-clock ticks} and the number of matrix instructions the
 * launch issued (each 2 * 32 * 32 * 16 flops); the caller times the launch.
 *
 * nestor_hip_gemm_clock_sink: from this call on the direct-to-LDS grouped-GEMM
 * kernels of THIS library's instrumented build (row-tiled and weight-gradient) add, per workgroup, {shader cycles, wall
 * ticks, 1, K steps} to slot (workgroup index % 64) of sink (device, 64 x 4 uint64,
 * zeroed by the caller); NULL switches the hook off again.  Process-wide, not
 * synchronised with launches in flight: set it between synchronisations.
 * ---------------------------------------------------------------------- */
int nestor_hip_mfma_clock_probe(int32_t random_operands, int32_t iters, uint64_t* counters,
                                void* stream);
/* The main loop of the GEMM kernels and nothing around it: a wavefront multiplies a
 * 128 x 128 accumulator tile in blocks of 16 MFMAs on fragments it read from LDS during
 * the block before (random bf16 values, two register sets), with reads_per_step 1 KiB
 * fragment reads and transfers_per_step 1 KiB LDS-DMA transfers per K step of 32 MFMAs
 * between the matrix instructions at the kernels' spacing -- no barriers, no waiting for
 * the transfers' data, no epilogue, no tile switches, every transfer an L2 hit (the
 * workgroups of an XCD share region_bytes of src, which holds 8 regions; region_bytes a
 * multiple of 32 KiB, at least 64 KiB).  Supported (reads, transfers): (0,0) (16,0) (0,8)
 * (16,8) (16,10) (16,12) -- 16/8 is the mix of the 256 x 256 x 32 kernels, 16/10 that of
 * the 128 x 512 x 32 ones with both operands read as whole fragments.  One round is 32
 * MFMAs; counters as above.  src_bytes is the size of the buffer at src: less than
 * 8 * region_bytes is refused (EINVAL). */
int nestor_hip_mfma_mix_probe(int32_t reads_per_step, int32_t transfers_per_step, int32_t iters,
                              const void* src, int64_t src_bytes, int64_t region_bytes,
                              uint64_t* counters, void* stream);
int nestor_hip_wall_clock_khz(void); /* ticks of wall_clock64() per millisecond; < 0 on error */
int nestor_hip_gemm_clock_sink(uint64_t* sink);

#ifdef __cplusplus
}
#endif

#endif  /* NESTOR_HIP_PROBES_H_ */
