/*
 * Measurement aids of the benchmark (libaeon_calibrate.so). None of them has a counterpart in the
 * reference and none is part of the product library or its ABI: they measure what this GPU
 * sustains (matrix pipe, a read-only HBM stream, LDS read orders), the figures the routed-expert
 * kernels' rates are read against. Conventions as in aeon_mi355.h: device pointers are named
 * d_..., work is enqueued on `stream` (a hipStream_t as void*, NULL = the default stream) and
 * timed by the caller; the return value is a status and aeon_calibrate_last_error() the
 * calling thread's message.
 */
#ifndef AEON_CALIBRATE_H
#define AEON_CALIBRATE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AEON_CALIBRATE_OK 0
#define AEON_CALIBRATE_ERR_INVALID_ARGUMENT 1
#define AEON_CALIBRATE_ERR_HIP 4

const char* aeon_calibrate_last_error(void);

/* Launches `workgroups` workgroups of four waves that each run `iterations` rounds of 16
 * independent v_mfma_f32_16x16x32_f16 out of registers, with constant (random_operands = 0) or
 * pseudo-random fp16 operands, and writes one float per thread to d_sink (>= workgroups*256
 * floats). *flop (host, optional) receives the FLOPs of the launch. Gives the matrix-pipe rate
 * this GPU sustains at the clock its power limit allows for such data: the practical ceiling
 * next to the published fp16 peak. */
int aeon_calibrate_mfma_f16(int random_operands, int iterations, int workgroups, float* d_sink,
                            size_t sink_floats, double* flop, void* stream);

/* The same loop with random operands in rounds of 32 matrix slots (16 cycles each): one
 * v_mfma_f32_16x16x32_f16 per slot (mfma_shape 16) or one v_mfma_f32_32x32x16_f16 per two slots
 * (mfma_shape 32), `valu_per_slot` independent VALU instructions of the int4 unpack
 * (v_and_or_b32, v_pk_add_f16) after every slot's MFMA, `lds_reads_per_16` 16-byte LDS reads
 * per 16 slots (waited for at the end of each round), at `waves_per_simd` 1 or 2. Served:
 * both shapes at two waves with (valu, lds) in (0..4, 0), (1..3, 4), (1, 8), (3, 8) and at one
 * wave with (0, 0), (1, 4), (2, 4), (2, 2); anything else is an invalid argument. Gives the rate
 * an instruction mix reaches with no memory wait at all, which is what the grouped GEMM's window
 * bodies are read against. */
int aeon_calibrate_mfma_mix(int mfma_shape, int valu_per_slot, int lds_reads_per_16,
                            int waves_per_simd, int iterations, int workgroups, float* d_sink,
                            size_t sink_floats, double* flop, void* stream);

/* Launches `workgroups` workgroups that each read their own contiguous bytes/workgroups share
 * of d_buffer once (16-byte loads, eight in flight per lane; the share must be a multiple of
 * 32 KiB) and write one folded word per thread to d_sink (>= workgroups*256 words). Gives the
 * rate a read-only stream sustains from HBM on this GPU: the practical ceiling of the
 * weight-streaming kernels next to the published bandwidth. */
int aeon_calibrate_read_stream(const void* d_buffer, size_t bytes, int workgroups,
                               uint32_t* d_sink, size_t sink_words, void* stream);

/* Launches `workgroups` workgroups of four waves that each issue `iterations` rounds of eight
 * 16-byte-per-lane LDS reads of a 1 KiB fragment, every read waited for, the lanes addressing the
 * fragment by `pattern`: 0 = their own order (linear), 1 = the matrix instruction's lanes reading
 * a fragment stored position-major (16-byte unit 4 n + chunk for n = lane % 16, chunk = lane / 16),
 * 2 = the same with each position's four pieces rotated by n / 2 (unit 4 n + (chunk + n / 2) % 4:
 * what the grouped kernel reads), 3 = rotated by n / 4. Writes one word per thread to d_sink
 * (>= workgroups*256 words); *wave_reads (host, optional) receives the number of wave-wide reads
 * of the launch. Shows which orders are free of bank conflicts. */
int aeon_calibrate_lds_read(int pattern, int iterations, int workgroups, uint32_t* d_sink,
                            size_t sink_words, double* wave_reads, void* stream);

#ifdef __cplusplus
}
#endif
#endif
