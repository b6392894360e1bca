/*
 * miles_quant.h -- C ABI of the MI355X (gfx950) weight-quantization library.
 *
 * Drop-in boundary for the per-tensor quantize / dequantize kernels of Miles' weight path.  The
 * reference has no FFI for this path: its quantizers are Python callables backed by Triton, a
 * pybind11 CUDA extension and Transformer Engine.  Each entry point below names the reference
 * callable it stands in for (paths relative to the reference repository root); the Python
 * wrappers in miles_amd/ keep those callables' signatures and bind these symbols with ctypes.
 *
 * Conventions
 *   - every pointer is a device pointer unless stated otherwise; plain pointers and sizes only;
 *   - outputs are allocated by the caller; inputs are never written;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); calls only enqueue
 *     work, they never synchronise and never allocate, so they are safe from several host threads;
 *   - return value: MQ_OK (0) or a negative MQ_ERR_* code; mq_last_error() returns a
 *     thread-local message for the last failure on the calling thread;
 *   - dtype codes: MQ_BF16, MQ_F16, MQ_F32.
 */
#ifndef MILES_QUANT_H_
#define MILES_QUANT_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MQ_VERSION 1
#define MQ_NVFP4_SECTION_WORDS 256
#define MQ_NVFP4_SECTIONS 4
#define MQ_NVFP4_RECORD_WORDS (MQ_NVFP4_SECTION_WORDS * (MQ_NVFP4_SECTIONS + 1))
/* words of an amax record behind its sections: the folded amax (float bits), three scale factors derived from it,
 * then the state words of the carried-over amax (see MQ_NVFP4_CARRY_AMAX): REDO is 1 when the last carried submission
 * quantized the tensor in its second pass, VOLATILE is 1 when the amax moved on the last two carried submissions (the
 * word behind it counts them) */
#define MQ_NVFP4_RECORD_AMAX_WORD (MQ_NVFP4_SECTION_WORDS * MQ_NVFP4_SECTIONS)
#define MQ_NVFP4_RECORD_REDO_WORD (MQ_NVFP4_RECORD_AMAX_WORD + 4)
#define MQ_NVFP4_RECORD_VOLATILE_WORD (MQ_NVFP4_RECORD_AMAX_WORD + 5)

enum { MQ_BF16 = 0, MQ_F16 = 1, MQ_F32 = 2 };
enum { MQ_OK = 0, MQ_ERR_ARG = -1, MQ_ERR_HIP = -2, MQ_ERR_UNSUPPORTED = -3 };

int mq_version(void);
const char* mq_last_error(void);

/* block_fp8(weight, block_size)                      tools/convert_hf_to_fp8.py:39-70
 *   w      [M,K] dtype, row stride ldw elements, unit column stride
 *   q      [M,K] e4m3fn bytes, contiguous
 *   scale  [ceil(M/block_m), ceil(K/block_k)] fp32 = amax/448; an all-zero tile: scale 0, bytes 0xFF */
int mq_fp8_block_quant(const void* w, int dtype, int64_t ldw, void* q, float* scale, int64_t M, int64_t K,
                       int block_m, int block_k, void* stream);

/* fp8_blockwise_cast(x, block_size)                  miles/kernels/quant/fp8_blockwise.py:61-79
 *   x any strides (elements); y [M,N] e4m3fn contiguous; s [ceil(M/bm), ceil(N/bn)] fp32
 *   absmax floored at 1e-10, multiply by the rounded reciprocal of the scale */
int mq_fp8_blockwise_cast(const void* x, int dtype, int64_t stride_m, int64_t stride_n, void* y, float* s,
                          int64_t M, int64_t N, int block_m, int block_n, void* stream);

/* tensor_fp8 / channel_fp8                           tools/convert_hf_to_fp8.py:73-86
 * and the per-tensor branch of the sync path         .../processors/quantizer_fp8.py:153-158
 *   per_channel != 0: scale [M] (one per row); else scale [1]
 *   floor_in_dtype: 1e-12 rounded to the weight dtype; amax_ws: >= max(M,1) uint32 of scratch */
int mq_fp8_scaled_quant(const void* w, int dtype, int64_t ldw, void* q, float* scale, void* amax_ws, int64_t M,
                        int64_t K, int per_channel, float floor_in_dtype, void* stream);

/* mq_fp8_scaled_quant without the workspace argument.  No counterpart in the reference: it is for callers that
 * cannot allocate device memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  The amax workspace is a static device array of MQ_FP8_STATIC_MAX_ROWS words (1 MiB, held by every
 * GPU the library runs on until the process ends); the call allocates nothing.  Results are those of
 * mq_fp8_scaled_quant.  per_channel != 0 with M > MQ_FP8_STATIC_MAX_ROWS is refused with MQ_ERR_ARG.
 * The device that is current at the call must be the one holding the tensors.  Every call on a GPU takes its words
 * from that GPU's one array, consecutive calls taking consecutive pieces of it (one 256-byte line for a per-tensor call,
 * M words for a per-channel one) and starting over at its beginning when a piece no longer fits.  Calls that overlap in
 * time on one GPU (two streams, two host threads) therefore race only when the pieces handed out while the earlier one
 * is still running add up to more than the array: 4 096 per-tensor calls, or per-channel calls of 262 144 rows in all.
 * A caller that keeps more than that in flight on one GPU must order its calls itself.  The first call on a device looks
 * the array's address up (hipGetSymbolAddress); make that call (M = 0 is enough) before starting a graph capture. */
#define MQ_FP8_STATIC_MAX_ROWS 262144
int mq_fp8_scaled_quant_static(const void* w, int dtype, int64_t ldw, void* q, float* scale, int64_t M, int64_t K,
                               int per_channel, float floor_in_dtype, void* stream);

/* transform_scale_ue8m0(sf, mn)                     .../processors/quantizer_fp8.py:141-142 (SGLang; DeepGEMM layout)
 *   sf  [batch, tile_rows, kb] fp32 power-of-two tile scales of a [mn, 128*kb] weight, tile_rows >= ceil(mn/128)
 *   out [batch, ceil(kb/4), align(mn,4)] int32: out[b,j,r] = sum_e exponent_byte(sf[b, r/128, 4j+e]) << 8e,
 *   zero where r >= mn or 4j+e >= kb; the caller views it transposed as [batch, mn, ceil(kb/4)]
 *   row_major != 0: out is that view made contiguous instead, [batch, mn, ceil(kb/4)] with no padding rows */
int mq_ue8m0_pack_scales(const float* sf, int32_t* out, int64_t batch, int64_t mn, int64_t kb, int64_t tile_rows,
                         int row_major, void* stream);

/* weight_dequant(x, s, block_size)                   tools/fp8_cast_bf16.py:30-40
 *   x [M,N] e4m3fn contiguous; s [ceil(M/block), ceil(N/block)] fp32; y [M,N] bf16 */
int mq_fp8_block_dequant(const void* x, const float* s, void* y, int64_t M, int64_t N, int block, void* stream);

/* per_block_cast_to_fp8(x)                           SGLang (third party; called at .../processors/quantizer_fp8.py:139-147)
 *   128x128 tiles, power-of-two fp32 scale 2^ceil(log2(max(amax, 1e-4) / 448)), q = e4m3(x / scale); shapes as
 *   mq_fp8_block_quant.  Restated from the published source: parity with SGLang itself is not pinned. */
int mq_fp8_block_quant_pow2(const void* w, int dtype, int64_t ldw, void* q, float* scale, int64_t M, int64_t K,
                            void* stream);

/* mxfp8_quantize(weight)                             miles/utils/mxfp8.py:51-78
 *   w [rows,K] contiguous, K % 32 == 0; q [rows,K] e4m3fn; scale [rows,K/32] E8M0 bytes */
int mq_mxfp8_quant(const void* w, int dtype, void* q, uint8_t* scale, int64_t rows, int64_t K, void* stream);

/* FP8 128x128 block-scaled source -> MXFP8           tools/convert_hf_to_mxfp8.py:56-102,180-195
 * A source tensor is e4m3fn codes x [M,K] with one scale per 128x128 tile: a grid of at least ceil(M/128) rows and
 * ceil(K/128) columns whose rows are lds elements apart (the reference crops a larger grid, :79,:91).
 * mq_fp8_scales_pow2_flag: _load_source_scale_u8's test of an fp32 grid (:81-86): *flag (one uint32 on the device) <- 1
 *   when every one of its rows x cols scales has a zero mantissa and a clear sign bit, else 0.  The caller reads the
 *   flag and picks the branch, as the reference does with .item().
 * mq_e8m0_expand_tile_scales: _source_fp8_to_mxfp8_scale_u8 (:98-102): out [M, groups] bytes (groups = K/32),
 *   out[r,g] = exponent byte of tile (r/128, g/4); the grid holds the bytes themselves, or (scales_are_f32 != 0) fp32
 *   powers of two whose byte is bits 23..30 (:85).  The codes of such a source are kept as they are.
 * mq_fp8_block_to_mxfp8: every other source (:187-190): block_quant_dequant(x, s, [128,128], float32) -- SGLang's
 *   function, third party: the scales repeated over their tiles and one fp32 multiply f32(code) * s -- followed by
 *   mxfp8_quantize; q [M,K] e4m3fn, scale [M,K/32] E8M0 bytes; K % 32 == 0.  The fp32 tensor exists in registers only.
 *   (A source tensor that stays unquantized becomes bf16 through mq_fp8_block_dequant, :203-215.)
 * mq_e8m0_bytes_to_f32: the fp32 scales of a grid stored as exponent bytes (:93): out[i] = the float whose bits are
 *   s[i] << 23, n contiguous values. */
int mq_e8m0_bytes_to_f32(const uint8_t* s, float* out, int64_t n, void* stream);
int mq_fp8_scales_pow2_flag(const float* s, int64_t rows, int64_t cols, int64_t lds, uint32_t* flag, void* stream);
int mq_e8m0_expand_tile_scales(const void* s, int scales_are_f32, int64_t lds, uint8_t* out, int64_t M, int64_t groups,
                               void* stream);
int mq_fp8_block_to_mxfp8(const void* x, const float* s, int64_t lds, void* q, uint8_t* scale, int64_t M, int64_t K,
                          void* stream);

/* quantize_mxfp4(weight, group_size)                  miles/utils/mxfp4.py:11-31
 *   w: numel elements, contiguous, groups of `group` consecutive elements (numel % group == 0, numel % 2 == 0)
 *   packed [numel/2] bytes (element 2j in the low nibble: magnitude code | sign << 3); scale [numel/group] E8M0 */
int mq_mxfp4_quant(const void* w, int dtype, uint8_t* packed, uint8_t* scale, int64_t numel, int group,
                   void* stream);

/* dequantize_mxfp4(weight_packed, weight_scale, group_size)   miles/utils/mxfp4.py:34-59
 *   packed [bytes]; scale [2*bytes/group]; y [2*bytes] bf16 */
int mq_mxfp4_dequant(const uint8_t* packed, const uint8_t* scale, void* y, int64_t bytes, int group, void* stream);

/* fake_int4_quant_cuda(x, (block_m, block_n), sym)   miles/kernels/quant/int4_fake/fake_int4_quant_cuda.cu:319-364
 *   x [M,N] contiguous; a group is a block_m x block_n tile (block_m * block_n % 32 == 0), entries past the edge
 *   count as 0; out [M,N], scale [ceil(M/block_m), ceil(N/block_n)], zero (asym only) in the dtype of x */
int mq_int4_fake_quant(const void* x, int dtype, void* out, void* scale, void* zero, int64_t M, int64_t N,
                       int block_m, int block_n, int sym, void* stream);

/* pack_layer(weight, group_size, sym=True)           .../processors/quantizer_compressed_tensors.py:235-265
 *                                                    (== tools/convert_hf_to_int4_direct.py:121-151)
 *   w [M,K] contiguous, K % group == 0, K % 8 == 0
 *   packed [M,K/8] int32 (nibble i of word j = code of element 8j+i, code = q+8)
 *   scale  [M,K/group] in the dtype of w */
int mq_int4_group_quant_pack(const void* w, int dtype, int32_t* packed, void* scale, int64_t M, int64_t K,
                             int group, void* stream);

/* pack_layer(weight, group_size, sym=False)          .../processors/quantizer_compressed_tensors.py:235-265
 *   w [M,K] contiguous and 16-byte aligned, K % group == 0, group % 8 == 0, M % 8 == 0
 *   packed    [M,K/8] int32: sum_i code(8j+i) << 4i with int32 wraparound; codes are uint8 in [0,255] after the
 *             reference's dequantize/requantize round trip in the dtype of w (nothing clamps them to 15)
 *   scale     [M,K/group] in the dtype of w
 *   zero      [M,K/group] uint8 zero points in [0,15] (also the staging area for packed_zp)
 *   packed_zp [K/group, M/8] int32: zero point of row 8j+i in nibble {0,4,1,5,2,6,3,7}[i] */
int mq_int4_group_quant_pack_asym(const void* w, int dtype, int32_t* packed, void* scale, uint8_t* zero,
                                  int32_t* packed_zp, int64_t M, int64_t K, int group, void* stream);

/* _dequantize_tensor(weight_packed, weight_scale, weight_shape, group_size)   tools/convert_kimi_int4_to_bf16.py:57-86
 *   packed [M, ceil(K/8)] int32 (nibble i of word j = element 8j+i, code = value + 8)
 *   scale  [M, K/group] bf16 / fp16 / fp32;  y [M,K] bf16 = bf16(f32(code - 8) * f32(scale)) */
int mq_int4_unpack_dequant(const int32_t* packed, const void* scale, int scale_dtype, void* y, int64_t M, int64_t K,
                           int group, void* stream);

/* cast_e2m1fn_to_e4m3fn(x, scale)                     tools/convert_mxfp4_to_fp8.py:30-49
 *   packed [out,in/2] e2m1 pairs; scale [out,in/32] E8M0 bytes; out % 128 == 0, in % 128 == 0
 *   y [out,in] e4m3fn; tile_scale [out/128,in/128] fp32 = max scale of the tile / 64 */
int mq_mxfp4_to_fp8_block(const uint8_t* packed, const uint8_t* scale, void* y, float* tile_scale, int64_t out_dim,
                          int64_t in_dim, void* stream);

/* fake_quant_{fp8,fp4,compressed_kv}_forward(x)       miles/kernels/quant/fake_quant.py:66-99 (kernel :25-63)
 *   quantize + dequantize in one pass, y in the dtype of x; blocks of consecutive elements (numel % block == 0)
 *   mode 0: e4m3, 1x32, power-of-two scale   mode 1: e2m1, 1x32, power-of-two scale   mode 2: e2m1, 1x16, e4m3 scale */
int mq_fake_quant(const void* x, int dtype, void* y, int64_t numel, int mode, void* stream);

/* act_quant(x, block_size, scale_fmt, scale_dtype, inplace)   miles/kernels/quant/fp8_act_quant.py:110-137 (kernel :49-107)
 *   FP8 e4m3 quantization of 1 x block groups of consecutive elements (numel % block == 0):
 *   s = max(amax, 1e-4) * f32(1/448), code = e4m3(clamp(x / s, +-448)) with a true fp32 division.
 *   flags: MQ_ACT_ROUND_SCALE  s rounded up to a power of two (scale_fmt given)
 *          MQ_ACT_SCALE_E8M0   scale [numel/block] stored as E8M0 exponent bytes instead of fp32 (needs ROUND_SCALE)
 *          MQ_ACT_INPLACE      y gets dtype(f32(code) * s) in the dtype of x instead of the codes; y may be x itself
 *   ROUND_SCALE | INPLACE is fp8_simulate (miles_plugins/models/deepseek_v4/ops/qat.py:8-23).
 *   Tuned for block 16 / 32 / 64 / 128 on 16-byte aligned tensors; any other block size runs a plain kernel. */
enum { MQ_ACT_ROUND_SCALE = 1, MQ_ACT_SCALE_E8M0 = 2, MQ_ACT_INPLACE = 4 };
int mq_fp8_act_quant(const void* x, int dtype, void* y, void* scale, int64_t numel, int block, int flags, void* stream);

/* NVFP4                                              miles/utils/nvfp4.py:54-114
 * The global amax travels on the device in an "amax record": MQ_NVFP4_RECORD_WORDS uint32 words made of
 * MQ_NVFP4_SECTIONS sections of MQ_NVFP4_SECTION_WORDS partial maxima (float bit patterns).  Each tensor that
 * shares the amax writes ONE whole section (no atomics, nothing to clear beforehand); the amax is the maximum
 * over the first n_sections sections.  A single tensor uses section 0 with n_sections = 1; a gate/up pair
 * uses sections 0 and 1 with n_sections = 2 (nvfp4.py:100-103).  The words after the last section hold the
 * folded amax and the two scale factors derived from it (written by mq_nvfp4_quant).
 * mq_nvfp4_amax: record section <- partial maxima of |w| (every word of the section is written).
 * mq_nvfp4_quant: folds the record, then quantizes: w [M,K] contiguous, K % 16 == 0; q [M,K/2] (element 2i in
 *   the low nibble);
 *   block_scale [M,K/16] e4m3fn bytes; global_scale (may be NULL) receives weight_scale_2 =
 *   1 / min(e4m3_max*6/amax, FLT_MAX) as one fp32 (nvfp4.py:19-39).
 * flags: MQ_NVFP4_4OVER6 selects Transformer Engine's Four Over Six block scaling (NVTE_NVFP4_4OVER6; restated in
 *   miles/kernels/quant/nvfp4_qdq.py:893-990): every block is quantized for a maximum of 6 and of 4 and keeps the
 *   candidate with the smaller error; MQ_NVFP4_ERR_MSE squares the error terms (NVTE_NVFP4_4OVER6_ERR_MODE=MSE),
 *   MQ_NVFP4_ERR_FP16 uses the fp16 candidate-error form (NVTE_NVFP4_4OVER6_ERR_USE_FAST_MATH=1). */
enum { MQ_NVFP4_4OVER6 = 1, MQ_NVFP4_ERR_MSE = 2, MQ_NVFP4_ERR_FP16 = 4,
       /* jobs of mq_run_jobs only: see the NVFP4 note there */
       MQ_NVFP4_CARRY_AMAX = 8 };
int mq_fill_u32(void* p, uint32_t value, int64_t n, void* stream);
int mq_nvfp4_amax(const void* w, int dtype, int64_t numel, void* record, int section, void* stream);
int mq_nvfp4_quant(const void* w, int dtype, const void* record, int n_sections, void* q, void* block_scale,
                   float* global_scale, int64_t M, int64_t K, int e4m3_max, int flags, void* stream);

/* Training-forward NVFP4 fake quantization          miles/kernels/quant/nvfp4_qdq.py:1213-1229 (kernel :1067-1105)
 * mq_nvfp4_fold: reduces the first n_sections sections of a record (written by mq_nvfp4_amax) into the amax,
 *   stored as float bits in word MQ_NVFP4_SECTIONS * MQ_NVFP4_SECTION_WORDS of the record (compute_nvfp4_amax).
 * mq_nvfp4_qdq: fused_nvfp4_qdq(x, amax) (flags as for mq_nvfp4_quant): x bf16 / fp16, numel % 16 == 0, amax a device
 *   fp32 scalar; y = dtype(e2m1 code * (f32(block scale) * amax / (6 * e4m3_max))) in the dtype of x. */
int mq_nvfp4_fold(void* record, int n_sections, int e4m3_max, void* stream);
int mq_nvfp4_qdq(const void* x, int dtype, const float* amax, void* y, int64_t numel, int e4m3_max, int flags,
                 void* stream);

/* Batched driver: runs a list of quantization jobs on one stream, in order, with the same results as calling
 * the single-tensor entry points one by one.  Consecutive jobs of the same kind are fused into grouped
 * launches (up to 64 tensors per kernel launch, descriptors passed as kernel arguments), which is what
 * keeps a weight sync of thousands of small tensors bandwidth-bound instead of launch-bound.
 * Stands in for the per-parameter Python loop of the reference's sync path
 * (miles/backends/megatron_utils/update_weight/hf_weight_iterator_direct.py:140-146 calling
 *  .../megatron_to_hf/processors/__init__.py:17-30 once per parameter).
 *
 *   kind                        in            out           scale          aux / aux2                  p0, p1
 *   MQ_JOB_FP8_BLOCK            w[rows,cols]  e4m3          fp32 tiles     -                           block_m, block_k
 *   MQ_JOB_FP8_BLOCKWISE_CAST   x[rows,cols]  e4m3          fp32 tiles     -                           block_m, block_n
 *   MQ_JOB_FP8_DEQUANT          e4m3          bf16          -              aux = fp32 tile scales (in) block, -
 *   MQ_JOB_MXFP8                w             e4m3          E8M0 bytes     -                           -
 *   MQ_JOB_INT4_PACK            w             int32 words   scales (dtype) -                           group, -
 *   MQ_JOB_NVFP4                w             packed e2m1   e4m3 bytes     aux = amax record,          e4m3_max, flags
 *                                                                          aux2 = fp32 weight_scale_2
 *   MQ_JOB_MXFP4                w             packed e2m1   E8M0 bytes     -                           group, -
 *   MQ_JOB_COPY                 bytes         bytes         -              -                           -
 *     (rows * cols bytes copied verbatim: how a pass-through tensor reaches its place in a packed transport bucket,
 *      the flattened payload of miles/backends/training_utils/weight_update/protocols/broadcast.py:191-208.  With
 *      rows > 1 the job is a 2-D copy of rows runs of cols bytes each: source runs ld bytes apart, destination runs
 *      block_stride bytes apart (0: back to back) -- one job regroups the q rows of a fused QKV weight or swaps the
 *      column halves of a matrix; both pitches must be at least cols)
 *   MQ_JOB_FP8_BLOCK_POW2       w[rows,cols]  e4m3          fp32 tiles     -                           128, 128
 *   MQ_JOB_UE8M0_PACK           fp32 tiles    int32 words   -              -                           batch, tile_rows
 *   MQ_JOB_FP8_TENSOR           w[rows,cols]  e4m3          fp32 [1]       aux = amax record           floor bits, flags
 *     (tensor_fp8 / the per-tensor branch of the sync path, see mq_fp8_scaled_quant: bf16 or fp16, contiguous, cols % 8 == 0,
 *      16-byte aligned input; p0 = bit pattern of 1e-12 rounded to the weight dtype; p1 = 0 or MQ_NVFP4_CARRY_AMAX)
 *   MQ_JOB_INT4_PACK_ASYM       w             int32 words   scales (dtype) aux = uint8 zero points,    group, -
 *                                                                          aux2 = int32 packed_zp
 *     (mq_int4_group_quant_pack_asym; bf16 or fp16 tensors on a 16-byte boundary with groups of 32 / 64 / 128 share their two
 *      launches, codes and then packed zero points, with up to MQ_MAX_GROUP tensors)
 *     (mq_ue8m0_pack_scales with mn = rows, kb = cols, row_major = ld; its input is usually the scale output of an
 *      earlier job)
 *   MQ_JOB_MXFP4_TO_FP8         e2m1 pairs    e4m3          fp32 tiles     aux = E8M0 bytes (in)       -
 *     (mq_mxfp4_to_fp8_block with out_dim = rows, in_dim = cols, both multiples of 128: the experts of a checkpoint
 *      shard re-coded in launches of up to MQ_MAX_GROUP tensors)
 *   MQ_JOB_FP8_TO_MXFP8         e4m3          e4m3          E8M0 bytes     aux = fp32 tile scales (in) -
 *     (mq_fp8_block_to_mxfp8 with M = rows, K = cols, lds = ld; 16-byte aligned tensors share launches of up to
 *      MQ_MAX_GROUP)
 *   MQ_JOB_E8M0_EXPAND          tile scales   E8M0 bytes    -              -                           -
 *     (mq_e8m0_expand_tile_scales with M = rows, groups = cols, lds = ld; dtype MQ_F32: the grid holds fp32 powers of
 *      two, any other dtype code: exponent bytes)
 *   MQ_JOB_INT4_UNPACK          int32 words   bf16          -              aux = scales (dtype, in)    group, -
 *     (mq_int4_unpack_dequant with M = rows, K = cols; dtype is the scales' dtype.  Jobs with one group size and one
 *      scale dtype share launches of up to MQ_MAX_GROUP tensors: a checkpoint shard's experts unpacked together)
 *   MQ_JOB_MXFP4_DEQUANT        e2m1 pairs    bf16          -              aux = E8M0 bytes (in)       group, -
 *     (mq_mxfp4_dequant with bytes = rows * cols / 2; jobs of one group size share launches the same way)
 * ld is the input row stride in elements for the two FP8 quantizers (column stride 1) and ignored elsewhere;
 * rows_per_block / block_stride describe a row-blocked input (see the struct).
 * The three FP8 tile kinds (FP8_BLOCK, FP8_BLOCKWISE_CAST, FP8_BLOCK_POW2), MXFP8, MXFP4, INT4_PACK, INT4_PACK_ASYM, FP8_TENSOR and NVFP4 run their tuned
 * kernels on bf16 and on fp16 inputs; consecutive jobs share a launch when they also share the input dtype (NVFP4 jobs
 * that share an amax record must have one dtype to take them).
 * NVFP4: the driver reduces every job's tensor into a section of its record and then quantizes; jobs that
 * share one record (a gate/up pair; at most MQ_NVFP4_SECTIONS) must be adjacent in the list.
 * MQ_NVFP4_CARRY_AMAX in p1 of NVFP4 and FP8_TENSOR jobs (no counterpart in the reference): a caller that submits the
 * same job list again, amax records included and untouched in between, after at least one submission without the
 * flag, may set it on bf16 or fp16 jobs.  The driver then quantizes in ONE pass with the amax and scales the record still holds from the last
 * submission, collects the new amax on the way, and quantizes a tensor a second time only if its amax changed
 * (results are identical either way; a weight tensor's amax rarely moves between two syncs).  A tensor whose amax
 * changed on two submissions in a row is marked volatile in its record: on the next submission the single pass only
 * collects its amax and the second pass quantizes it (what the plain two-pass form costs), and it returns to the
 * single pass once its amax has stayed the same for one submission. */
enum {
    MQ_JOB_FP8_BLOCK = 0,
    MQ_JOB_FP8_BLOCKWISE_CAST = 1,
    MQ_JOB_FP8_DEQUANT = 2,
    MQ_JOB_MXFP8 = 3,
    MQ_JOB_INT4_PACK = 4,
    MQ_JOB_NVFP4 = 5,
    MQ_JOB_MXFP4 = 6,
    MQ_JOB_COPY = 7,
    MQ_JOB_FP8_BLOCK_POW2 = 8,
    MQ_JOB_UE8M0_PACK = 9,
    MQ_JOB_FP8_TENSOR = 10,
    MQ_JOB_INT4_PACK_ASYM = 11,
    MQ_JOB_MXFP4_TO_FP8 = 12,
    MQ_JOB_FP8_TO_MXFP8 = 13,
    MQ_JOB_E8M0_EXPAND = 14,
    MQ_JOB_INT4_UNPACK = 15,
    MQ_JOB_MXFP4_DEQUANT = 16
};
typedef struct mq_job {
    int32_t kind;
    int32_t dtype;
    const void* in;
    void* out;
    void* scale;
    void* aux;
    void* aux2;
    int64_t rows, cols, ld;
    int32_t p0, p1;
    /* FP8 quantizers only: the input rows come in blocks of rows_per_block consecutive rows (stride ld) whose
     * first rows are block_stride elements apart -- e.g. the q / k / v rows of a fused per-group QKV weight,
     * read in place.  0 / 0 = one block (plain matrix).  rows_per_block must be a multiple of the tile height,
     * the input bf16 or fp16. */
    int64_t rows_per_block, block_stride;
} mq_job;
/* Consecutive jobs of one kind (and, for the flat kernels, of similar size) are fused into launches of up to
 * MQ_MAX_GROUP tensors, counted from the first job of the call; a run of FP8 tile jobs of more than 36 864 tiles is
 * cut into launches of equal size (the tile kernel streams faster in launches of moderate length).
 * mq_tune_tile_launch_tiles (no counterpart in the reference) sets that length for the process, 0 for no cutting, and
 * stores the length it replaces in *previous (a host pointer, may be NULL); the environment variable
 * MQ_TILE_LAUNCH_TILES, read once when the library first needs the length and ignored unless it holds a whole number,
 * sets the starting value. */
#define MQ_MAX_GROUP 64
int mq_run_jobs(const mq_job* jobs, int64_t n, void* stream);
int mq_tune_tile_launch_tiles(int64_t tiles, int64_t* previous);

/* mq_run_jobs with the per-tensor descriptors of its launches kept in device memory (no counterpart in the reference; for
 * callers that submit one job list again and again, as a replayed weight sync does).  The kernel arguments of a launch
 * hold MQ_MAX_GROUP descriptors at most; a model of thousands of small tensors (the 18 432 expert matrices of a
 * Qwen3-30B-A3B sync, 3 MB each) then drains and refills the chip every 64 tensors.  With a table a launch of the
 * MXFP8, MXFP4, INT4 (symmetric and asymmetric), NVFP4 (standard block scaling), per-tensor FP8 and 128x128 FP8 jobs
 * covers up to MQ_TABLE_GROUP tensors of similar size; every other job kind, Four Over Six NVFP4 jobs and FP8 jobs of
 * mixed shapes run as in mq_run_jobs.
 * mq_job_table_fill writes n entries of MQ_JOB_TABLE_ENTRY_BYTES bytes into host memory, entry i for jobs[i]; the
 * caller copies them to device memory (any 8-byte aligned address) and passes that address, together with the same
 * jobs, to mq_run_jobs_tabled.  A call may cover a sub-range of the list: pass jobs + k, n' and the address of entry k.
 * The table must not change while a submitted call may still run; a NULL table makes the call mq_run_jobs. */
#define MQ_JOB_TABLE_ENTRY_BYTES 56
#define MQ_TABLE_GROUP 8192
int mq_job_table_fill(const mq_job* jobs, int64_t n, void* host_table);
int mq_run_jobs_tabled(const mq_job* jobs, int64_t n, const void* device_table, void* stream);

/* mq_run_jobs_tabled that also reports how many amax records moved (no counterpart in the reference).  device_moved
 * points to two uint32 in device memory, counters that the call never clears: every fold of NVFP4 or per-tensor FP8 amax
 * records made by the call adds the number of tensors it folded to word 1, and to word 0 the number of those whose
 * record held another amax before.  host_mirror (may be NULL) points to two uint32 of pinned host memory (hipHostMalloc;
 * anything else is refused): every fold launch first refreshes them with the counters as the launches before it left
 * them, so that the host can read them at any time without a copy, an event or a wait.  The mirror must stay allocated
 * until every submitted call that named it has finished on the GPU: the kernels store through its address.
 * When most tensors keep moving from one submission to the next -- where MQ_NVFP4_CARRY_AMAX costs a second pass over
 * every such tensor -- the caller submits the list without the flag until they hold still again; the records stay valid
 * for either form.  device_table and device_moved may be NULL (then host_mirror must be NULL too). */
int mq_run_jobs_feedback(const mq_job* jobs, int64_t n, const void* device_table, uint32_t* device_moved,
                         uint32_t* host_mirror, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MILES_QUANT_H_ */
