/*
 * miles_quant_probes.h -- C ABI of libmq_probes.so: self-tests and streaming probes for the MI355X (gfx950) weight-
 * quantization library.  None of this is part of the product: libmiles_quant.so does not contain it and nothing in the
 * miles_amd package calls it.  The GPU test suite loads it to prove, on the device, the properties of gfx950
 * instructions that the product kernels rely on; bench.py loads it to calibrate what an access shape reaches on a
 * GPU and what rocprof's traffic counters read for a copy of known size.  No entry point has a counterpart in the
 * reference.
 *
 * Conventions as in miles_quant.h: device pointers, `stream` a hipStream_t passed as void*, calls only enqueue work;
 * return 0, or -1 (bad argument) / -2 (HIP error) with a thread-local message in mqp_last_error().
 */
#ifndef MILES_QUANT_PROBES_H_
#define MILES_QUANT_PROBES_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* mqp_last_error(void);

/* Conversion self-test: compares the gfx950 convert instructions used by the kernels with the
 * software round-to-nearest-even forms over every fp32 bit pattern.  counts: 8 uint64 on the device
 * (cleared by the call): [0] e4m3 mismatches for |x| <= 448, [1] NaN inputs whose e4m3 code is not
 * 0x7F/0xFF, [2] e2m1 mismatches over all non-NaN inputs, [3] bf16 mismatches over all non-NaN
 * inputs, [4] e4m3 decode mismatches (256 codes), [5] NaN inputs whose e2m1 code is not +-6,
 * [6] inputs in (448, 464] whose e4m3 code is not +-448, [7] 1 if the packed e2m1 convert does not put
 * its first operand in the low nibble.  The kernels rely on [0], [2], [3], [4], [7] being zero. */
int mqp_selftest_convert(uint64_t* counts, void* stream);

/* Reciprocal self-test.  The INT4 packers divide a group's elements by its scale through y = 1/scale, taken from the
 * hardware reciprocal and one Newton step instead of an IEEE division; the codes are only right if y is the correctly
 * rounded reciprocal.  count: one uint64 on the device (cleared by the call) = divisors of both signs in [2^-91, 2^90],
 * the range in which the kernels use y, for which it differs from 1.0f / scale.  The kernels rely on it being zero. */
int mqp_selftest_reciprocal(uint64_t* count, void* stream);

/* Plain copy, one 16-byte unit per lane: the yardstick for achievable HBM bandwidth and for what rocprof's FETCH_SIZE /
 * WRITE_SIZE read per byte moved.  Pointers and size are multiples of 16. */
int mqp_copy_bytes(const void* src, void* dst, int64_t nbytes, void* stream);

/* Streaming probes: kernels that only move bytes in the access shapes of the quantizers.  nbytes counts the larger
 * side; dst must hold nbytes as well (the probes write at most that).
 *   MQP_FLAT_2_1   16 bytes read, 8 written per unit, one-shot workgroups; param = units per lane (1, 2, 4, 8)
 *   MQP_FLAT_1_2   8 bytes read, 16 written per unit; param = units per lane
 *   MQP_LOOP_2_1   the 2:1 mix as a grid of param workgroups striding over the buffer (param % 512 == 0)
 *   MQP_TILE_2_1 / _READ / _WRITE   128 x 128 tiles of a row-major matrix of 2-byte elements, param = its row
 *                  length K; both sides, the reads alone, the writes alone */
enum { MQP_FLAT_2_1 = 0, MQP_FLAT_1_2 = 1, MQP_LOOP_2_1 = 2, MQP_TILE_2_1 = 3, MQP_TILE_READ = 4, MQP_TILE_WRITE = 5 };
int mqp_stream_probe(int shape, const void* src, void* dst, int64_t nbytes, int64_t param, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MILES_QUANT_PROBES_H_ */
