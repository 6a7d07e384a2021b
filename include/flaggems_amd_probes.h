/*
 * flaggems_amd -- measurement aids of the benchmark, exported by the same library but no part of the product
 * interface (include/flaggems_amd.h): two kernels that state the floors the GEMM kernels are measured against.
 * Same conventions: raw device pointers, a HIP stream, 0 or a negative fg_status.
 */
#ifndef FLAGGEMS_AMD_PROBES_H_
#define FLAGGEMS_AMD_PROBES_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Measurement aid, no reference counterpart: enqueues a kernel that reads `bytes` bytes at `src` once (16-byte
 * non-temporal loads from every compute unit) and does nothing else.  Its duration is the floor for any kernel that
 * must stream a buffer of that size from memory, launch cost included; the benchmark reports the decode GEMMs next
 * to it.  `sink` (4 bytes of device memory, may be NULL) is written only for data no real buffer holds.
 */
int fg_stream_read_probe(const void* src, size_t bytes, void* sink, void* stream);

/*
 * Measurement aid without counterpart in the reference: the multiply phase of the persistent GEMM kernel alone --
 * eight wavefronts on every compute unit issue `iterations` x 32 e4m3 MFMAs (16x16x128) each on operands held in
 * registers, with the four scale FMAs per MFMA of the block-scaled form (with_scale_fmas != 0) or accumulating in
 * the matrix pipe (0); no LDS, no memory traffic, no barriers.  `operands`: at least 64 KB of device memory, 32-byte
 * aligned, whose bytes are the fp8 operands (the clock the part holds under matrix load depends on them).  The
 * launch performs iterations * 32 * 65536 * 8 * (compute units) flops; benchmarks time it to state what fraction
 * of the matrix pipes' rate under their own instruction mix a GEMM reaches.  `sink` may be NULL.
 */
int fg_mfma_issue_probe(const void* operands, int iterations, int with_scale_fmas, void* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLAGGEMS_AMD_PROBES_H_ */
