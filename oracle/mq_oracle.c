/*
 * mq_oracle.c -- CPU restatement of the Miles weight-quantization hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the parity checker for the HIP
 * kernels in miles_amd/csrc and the "port" CPU baseline timed by bench.py.
 * Nothing in the product package may import, link or call it.
 *
 * Every function cites the reference file:line (relative to the reference
 * repository root) whose arithmetic it follows.  All arithmetic is IEEE
 * binary32 round-to-nearest-even; build with -ffp-contract=off so that the
 * compiler never fuses a multiply and an add (see oracle/Makefile).
 *
 * Pin status of each function (what independent evidence fixes its output)
 * is listed in oracle/README.md; functions that restate third-party
 * arithmetic whose source is not in the reference repository (Transformer
 * Engine's MXFP8 / NVFP4 quantizers) are marked "parity unpinned" there.
 *
 * Input dtype codes: 0 = bfloat16, 1 = float16, 2 = float32.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define MQ_BF16 0
#define MQ_F16 1
#define MQ_F32 2
/* NVFP4 option flags, as in include/miles_quant.h */
#define MQ_NVFP4_4OVER6 1
#define MQ_NVFP4_ERR_MSE 2
#define MQ_NVFP4_ERR_FP16 4

/* ------------------------------------------------------------------ */
/* bit-level helpers                                                    */
/* ------------------------------------------------------------------ */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

static inline float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* float32 -> bfloat16, round to nearest even; NaN -> 0x7FC0 (PyTorch's
 * c10::BFloat16 rounding). */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t m = h & 0x3FFu;
    if (e == 0) {
        if (m == 0) return u2f(sign);
        /* subnormal: value = m * 2^-24 */
        float v = (float)m * 5.9604644775390625e-8f;
        return u2f(f2u(v) | sign);
    }
    if (e == 31) return u2f(sign | 0x7F800000u | (m << 13));
    return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

/* float32 -> float16 round to nearest even (IEEE), used only for the
 * dtype-generic INT4 python-half chain. */
static inline uint16_t f32_to_f16(float f) {
    uint32_t u = f2u(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return sign | 0x7E00;
    if (a >= 0x477FF000u) return sign | 0x7C00; /* >= 65520 -> inf */
    if (a < 0x38800000u) {                      /* < 2^-14: subnormal half */
        float v = u2f(a) * 16777216.0f;         /* * 2^24, exact */
        float r = nearbyintf(v);
        return sign | (uint16_t)r;
    }
    uint32_t lsb = (a >> 13) & 1u;
    a += 0xFFFu + lsb;
    return sign | (uint16_t)((a - 0x38000000u) >> 13);
}

static inline float load_as_f32(const void* p, int64_t i, int dtype) {
    switch (dtype) {
        case MQ_BF16: return bf16_to_f32(((const uint16_t*)p)[i]);
        case MQ_F16: return f16_to_f32(((const uint16_t*)p)[i]);
        default: return ((const float*)p)[i];
    }
}

/* round a float to the storage dtype and widen back (torch elementwise ops
 * on a low-precision tensor compute in fp32 and round the result once). */
static inline float round_to_dtype(float f, int dtype) {
    switch (dtype) {
        case MQ_BF16: return bf16_to_f32(f32_to_bf16(f));
        case MQ_F16: return f16_to_f32(f32_to_f16(f));
        default: return f;
    }
}

/* ------------------------------------------------------------------ */
/* float32 -> float8_e4m3fn                                            */
/* ------------------------------------------------------------------ */
/* Shared core: |x| finite, below 480.  Returns the 7-bit magnitude code
 * (may be 0x7F when the value rounds past 448). */
static inline uint8_t e4m3_mag_rne(uint32_t a) {
    if (a < 0x3C800000u) { /* |x| < 2^-6: e4m3 subnormal, step 2^-9 */
        float k = nearbyintf(u2f(a) * 512.0f); /* exact scaling, RNE */
        return (uint8_t)k;                     /* 0..8 ; 8 == 0x08 == 2^-6 */
    }
    int e = (int)(a >> 23) - 127; /* -6 .. 8 */
    uint32_t m = a & 0x7FFFFFu;
    uint32_t m3 = m >> 20;
    uint32_t rem = m & 0xFFFFFu;
    if (rem > 0x80000u || (rem == 0x80000u && (m3 & 1u))) m3++;
    if (m3 == 8) { m3 = 0; e++; }
    uint32_t code = ((uint32_t)(e + 7) << 3) | m3;
    return code > 0x7Fu ? 0x7F : (uint8_t)code;
}

/* PyTorch `tensor.to(torch.float8_e4m3fn)` (c10::Float8_e4m3fn): RNE, NO
 * saturation: |x| > 464 (incl. inf) and NaN -> 0x7F | sign; 464 ties to 448.
 * Follows tools/convert_hf_to_fp8.py:65 (the .to(float8_e4m3fn) cast). */
uint8_t mqo_f32_to_e4m3fn(float x) {
    uint32_t u = f2u(x);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a >= 0x43F00000u) return sign | 0x7F; /* >= 480, inf, NaN */
    return sign | e4m3_mag_rne(a);
}

/* Saturating variant (PTX cvt.rn.satfinite.e4m3x2.f32 as used at
 * miles/kernels/quant/nvfp4_qdq.py:489-511 and by Transformer Engine's
 * casts): |x| >= 448 and inf -> 448 with sign; NaN -> 0x7F. */
uint8_t mqo_f32_to_e4m3fn_sat(float x) {
    uint32_t u = f2u(x);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return 0x7F;
    if (a >= 0x43E00000u) return sign | 0x7E; /* >= 448 */
    return sign | e4m3_mag_rne(a);
}

float mqo_e4m3fn_to_f32(uint8_t c) {
    uint32_t sign = (uint32_t)(c & 0x80u) << 24;
    uint32_t e = (c >> 3) & 0xFu, m = c & 7u;
    if (e == 15 && m == 7) return u2f(sign | 0x7FC00000u);
    if (e == 0) return u2f(f2u((float)m * 0.001953125f) | sign); /* m * 2^-9 */
    return u2f(sign | ((e + 120u) << 23) | (m << 20));
}

/* ------------------------------------------------------------------ */
/* float32 -> e2m1 (4-bit)                                             */
/* ------------------------------------------------------------------ */
/* PTX cvt.rn.satfinite.e2m1x2.f32 (miles/kernels/quant/nvfp4_qdq.py:541-585):
 * grid {0,.5,1,1.5,2,3,4,6}, round to nearest, ties to the even code,
 * |x| > 6 and inf saturate to 6, NaN -> 0x7, bit 3 is the sign (-0 -> 0x8). */
uint8_t mqo_f32_to_e2m1(float x) {
    uint32_t u = f2u(x);
    uint8_t sign = (uint8_t)((u >> 28) & 0x8u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return 0x7;
    float v = u2f(a);
    uint8_t c;
    if (v <= 0.25f) c = 0;
    else if (v < 0.75f) c = 1;
    else if (v <= 1.25f) c = 2;
    else if (v < 1.75f) c = 3;
    else if (v <= 2.5f) c = 4;
    else if (v < 3.5f) c = 5;
    else if (v <= 5.0f) c = 6;
    else c = 7;
    return sign | c;
}

/* ------------------------------------------------------------------ */
/* A-1a  block_fp8   (tools/convert_hf_to_fp8.py:39-70)                */
/* ------------------------------------------------------------------ */
/* w: [M,K] with row stride ldw (elements).  q: [M,K] contiguous e4m3fn.
 * scale: [ceil(M/bm), ceil(K/bk)] fp32.
 *   amax  = max |w| over the zero-padded tile           (:49-58)
 *   scale = f32(amax) / 448                             (:60)  true division
 *   q     = e4m3fn( clamp(f32(w)/scale, -448, 448) )    (:61-66) true division
 * A tile whose amax is 0 gives scale 0 and 0/0 = NaN for every element; the
 * x86 default NaN has its sign bit set, so the byte is 0xFF (clamp keeps NaN). */
void mqo_block_fp8(const void* w, int dtype, int64_t M, int64_t K, int64_t ldw,
                   int bm, int bk, uint8_t* q, float* scale) {
    int64_t nt = (M + bm - 1) / bm, kt = (K + bk - 1) / bk;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t ti = 0; ti < nt; ti++) {
        for (int64_t tj = 0; tj < kt; tj++) {
            int64_t r0 = ti * bm, r1 = r0 + bm < M ? r0 + bm : M;
            int64_t c0 = tj * bk, c1 = c0 + bk < K ? c0 + bk : K;
            float amax = 0.0f;
            for (int64_t r = r0; r < r1; r++)
                for (int64_t c = c0; c < c1; c++) {
                    float a = fabsf(load_as_f32(w, r * ldw + c, dtype));
                    /* torch.max propagates NaN */
                    if (a > amax || a != a) amax = a;
                }
            float s = amax / 448.0f;
            scale[ti * kt + tj] = s;
            for (int64_t r = r0; r < r1; r++)
                for (int64_t c = c0; c < c1; c++) {
                    float x = load_as_f32(w, r * ldw + c, dtype);
                    float v = x / s;
                    uint8_t code;
                    if (v != v) {
                        /* x86 SSE: 0/0 produces the default NaN (sign set);
                         * a NaN operand propagates with its own sign. */
                        uint32_t sign = (x != x) ? (f2u(x) >> 31)
                                       : (s != s) ? (f2u(s) >> 31) : 1u;
                        code = (uint8_t)(0x7F | (sign << 7));
                    } else {
                        if (v < -448.0f) v = -448.0f;
                        if (v > 448.0f) v = 448.0f;
                        code = mqo_f32_to_e4m3fn(v);
                    }
                    q[r * K + c] = code;
                }
        }
    }
}

/* a2: tensor_fp8 / channel_fp8 (tools/convert_hf_to_fp8.py:73-86) and the
 * per-tensor branch of the sync path (quantizer_fp8.py:153-158):
 *   scale = f32( max(amax_in_dtype, dtype(1e-12)) ) / 448 ; q = e4m3fn(clamp(w/scale))
 * per_channel != 0: one scale per row ([M,1]), quotient in fp32; else one 0-dim scale,
 * quotient rounded to the weight dtype before the clamp (torch type promotion).
 * floor_in_dtype is 1e-12 already rounded to the tensor dtype by the caller. */
void mqo_fp8_per_tensor_or_channel(const void* w, int dtype, int64_t M, int64_t K,
                                   int64_t ldw, int per_channel, float floor_in_dtype,
                                   uint8_t* q, float* scale) {
    float tmax = 0.0f;
    if (!per_channel) {
        for (int64_t r = 0; r < M; r++)
            for (int64_t c = 0; c < K; c++) {
                float a = fabsf(load_as_f32(w, r * ldw + c, dtype));
                if (a > tmax || a != a) tmax = a;
            }
    }
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < M; r++) {
        float amax = tmax;
        if (per_channel) {
            amax = 0.0f;
            for (int64_t c = 0; c < K; c++) {
                float a = fabsf(load_as_f32(w, r * ldw + c, dtype));
                if (a > amax || a != a) amax = a;
            }
        }
        if (amax < floor_in_dtype) amax = floor_in_dtype;
        float s = amax / 448.0f;
        if (per_channel) scale[r] = s; else if (r == 0) scale[0] = s;
        for (int64_t c = 0; c < K; c++) {
            float v = load_as_f32(w, r * ldw + c, dtype) / s;
            /* a 0-dim scale does not promote the result: `weight / scale` stays in the
             * weight's dtype (one extra rounding) for the per-tensor strategy only */
            if (!per_channel) v = round_to_dtype(v, dtype);
            if (v < -448.0f) v = -448.0f;
            if (v > 448.0f) v = 448.0f;
            q[r * K + c] = mqo_f32_to_e4m3fn(v);
        }
    }
}

/* ------------------------------------------------------------------ */
/* A-1b  fp8_blockwise_cast (miles/kernels/quant/fp8_blockwise.py:43-58)*/
/* ------------------------------------------------------------------ */
/*   absmax = max( max|f32(x)| over tile , 1e-10f )      (:51)
 *   x_s    = absmax / 448   ; s_inv = 1 / x_s           (:52-53) IEEE division
 *   y      = e4m3( clamp(f32(x) * s_inv, -448, 448) )   (:54)
 * strides in elements for x; y contiguous; S contiguous.
 * NaN: tl.max, tl.maximum and tl.clamp are called without propagate_nan, i.e. they lower to the maxnum / minnum
 * operations that return the operand which is not NaN: the tile maximum skips NaN elements and a NaN product leaves
 * the clamp as max(NaN, -448) = -448. */
void mqo_fp8_blockwise_cast(const void* x, int dtype, int64_t M, int64_t N,
                            int64_t sxm, int64_t sxn, int bm, int bn,
                            uint8_t* y, float* S) {
    int64_t nt = (M + bm - 1) / bm, kt = (N + bn - 1) / bn;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t ti = 0; ti < nt; ti++) {
        for (int64_t tj = 0; tj < kt; tj++) {
            int64_t r0 = ti * bm, r1 = r0 + bm < M ? r0 + bm : M;
            int64_t c0 = tj * bn, c1 = c0 + bn < N ? c0 + bn : N;
            float amax = 0.0f;
            for (int64_t r = r0; r < r1; r++)
                for (int64_t c = c0; c < c1; c++) {
                    float a = fabsf(load_as_f32(x, r * sxm + c * sxn, dtype));
                    if (a > amax) amax = a;
                }
            float absmax = amax > 1e-10f ? amax : 1e-10f;
            float x_s = absmax / 448.0f;
            float s_inv = 1.0f / x_s;
            S[ti * kt + tj] = x_s;
            for (int64_t r = r0; r < r1; r++)
                for (int64_t c = c0; c < c1; c++) {
                    float v = load_as_f32(x, r * sxm + c * sxn, dtype) * s_inv;
                    v = fminf(fmaxf(v, -448.0f), 448.0f);
                    y[r * N + c] = mqo_f32_to_e4m3fn(v);
                }
        }
    }
}

/* per_block_cast_to_fp8 (SGLang, sglang.srt.layers.quantization.fp8_utils; third party, pinned by the reference
 * at sglang v0.5.x and absent from its tree -- PARITY UNPINNED; called at
 * miles/backends/megatron_utils/megatron_to_hf/processors/quantizer_fp8.py:139-147).  Published algorithm:
 *   x_amax = max|f32(x)| over the zero-padded 128x128 tile, clamped below at 1e-4
 *   sf     = 2 ^ ceil(log2(x_amax / 448))
 *   y      = e4m3(f32(x) * (1 / sf))
 * x row-major with row stride ld. */
void mqo_fp8_block_pow2(const void* x, int dtype, int64_t M, int64_t N, int64_t ld, uint8_t* y, float* S) {
    int64_t nt = (M + 127) / 128, kt = (N + 127) / 128;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t ti = 0; ti < nt; ti++)
        for (int64_t tj = 0; tj < kt; tj++) {
            int64_t r0 = ti * 128, r1 = r0 + 128 < M ? r0 + 128 : M;
            int64_t c0 = tj * 128, c1 = c0 + 128 < N ? c0 + 128 : N;
            float amax = 0.0f;
            for (int64_t r = r0; r < r1; r++)
                for (int64_t c = c0; c < c1; c++) {
                    float a = fabsf(load_as_f32(x, r * ld + c, dtype));
                    if (a > amax || a != a) amax = a;                  /* torch's amax hands a NaN on */
                }
            if (amax < 1e-4f) amax = 1e-4f;
            float sf = powf(2.0f, ceilf(log2f(amax / 448.0f)));
            float inv = 1.0f / sf;
            S[ti * kt + tj] = sf;
            for (int64_t r = r0; r < r1; r++)
                for (int64_t c = c0; c < c1; c++) y[r * N + c] = mqo_f32_to_e4m3fn(load_as_f32(x, r * ld + c, dtype) * inv);
        }
}

/* ------------------------------------------------------------------ */
/* A-5  FP8 block dequant (tools/fp8_cast_bf16.py:15-40;               */
/*      tools/convert_mimo_v2_to_bf16.py:44-47)                        */
/* ------------------------------------------------------------------ */
/* SGLang's transform_scale_ue8m0 (called at quantizer_fp8.py:142; third party, not in the reference tree; restated
 * from DeepGEMM's published get_mn_major_tma_aligned_packed_ue8m0_tensor): weight row r takes the scales of tile
 * row r/128; byte = (bits(sf) >> 23) & 255; four neighbours along k share one int32, lowest byte first, missing
 * ones zero; storage is [batch][ceil(kb/4)][align(mn,4)] (rows contiguous), rows >= mn zero.  Parity unpinned. */
void mqo_ue8m0_pack_scales(const float* sf, int64_t batch, int64_t mn, int64_t kb, int32_t* out) {
    int64_t amn = (mn + 3) / 4 * 4, kw = (kb + 3) / 4, tile_rows = (mn + 127) / 128;
    for (int64_t b = 0; b < batch; b++)
        for (int64_t j = 0; j < kw; j++)
            for (int64_t r = 0; r < amn; r++) {
                uint32_t word = 0;
                for (int e = 0; e < 4 && r < mn; e++) {
                    if (4 * j + e >= kb) break;
                    uint32_t bits;
                    memcpy(&bits, sf + (b * tile_rows + r / 128) * kb + 4 * j + e, 4);
                    word |= ((bits >> 23) & 0xFFu) << (8 * e);
                }
                out[(b * kw + j) * amn + r] = (int32_t)word;
            }
}

/* y[i,j] = bf16_rne( f32(e4m3(x[i,j])) * s[i/B, j/B] ) */
void mqo_fp8_block_dequant(const uint8_t* x, const float* s, int64_t M, int64_t N,
                           int block, uint16_t* y) {
    int64_t kt = (N + block - 1) / block;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < M; r++)
        for (int64_t c = 0; c < N; c++) {
            float v = mqo_e4m3fn_to_f32(x[r * N + c]) * s[(r / block) * kt + c / block];
            y[r * N + c] = f32_to_bf16(v);
        }
}

/* ------------------------------------------------------------------ */
/* A-2  MXFP8 1x32 E8M0 (miles/utils/mxfp8.py:51-78; arithmetic is     */
/*      Transformer Engine 2.17 MXFP8Quantizer -- third party)          */
/* ------------------------------------------------------------------ */
/* E8M0 = ceil-to-power-of-two of amax * f32(1/448), saturating at 0xFE;
 * corroborated in-repo by miles/kernels/quant/fake_quant.py:15-21. */
uint8_t mqo_f32_to_e8m0_ceil(float v) {
    uint32_t u = f2u(v);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0xFF;
    if ((u & 0x7FFFFFFFu) == 0x7F800000u) return 0xFE;
    if (v == 0.0f) return 0;
    uint32_t e = (u >> 23) & 0xFFu, m = u & 0x7FFFFFu;
    if ((m > 0 && e != 0xFE) && !(e == 0 && m <= 0x400000u)) e++;
    return (uint8_t)e;
}

void mqo_mxfp8(const void* w, int dtype, int64_t rows, int64_t K, uint8_t* q, uint8_t* scale) {
    const float inv448 = u2f(0x3B124925u); /* f32(1/448) */
    int64_t g = K / 32;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++)
        for (int64_t j = 0; j < g; j++) {
            int64_t base = r * K + j * 32;
            float amax = 0.0f;
            for (int i = 0; i < 32; i++) {
                float a = fabsf(load_as_f32(w, base + i, dtype));
                if (a > amax) amax = a;
            }
            uint8_t e = mqo_f32_to_e8m0_ceil(amax * inv448);
            float inv;                                   /* 2^(127-e), exact */
            if (e == 0) inv = 1.0f;
            else if (e == 254) inv = u2f(0x00400000u);   /* 2^-127, subnormal */
            else if (e == 255) inv = u2f(0x00200000u);   /* NaN amax: 2^-128 */
            else inv = u2f((uint32_t)(254 - e) << 23);
            scale[r * g + j] = e;
            for (int i = 0; i < 32; i++)
                q[base + i] = mqo_f32_to_e4m3fn_sat(load_as_f32(w, base + i, dtype) * inv);
        }
}

/* ------------------------------------------------------------------ */
/* FP8 128x128 block-scaled source -> MXFP8                             */
/* (tools/convert_hf_to_mxfp8.py:56-102,180-195)                        */
/* ------------------------------------------------------------------ */
/* The general-scale branch (:187-190):
 *   w32 = block_quant_dequant(x, s, [128,128], torch.float32)   SGLang (third party, not in the tree): the tile scales
 *         repeated 128 x 128, cropped, and ONE fp32 multiply  f32(e4m3(x)) * s[i/128, j/128]
 *   q, scale = mxfp8_quantize(w32)                              mqo_mxfp8 on the fp32 tensor
 * lds: row stride of the tile-scale grid in elements (the reference crops a larger grid, :79). */
void mqo_fp8_block_to_mxfp8(const uint8_t* x, const float* s, int64_t lds, int64_t M, int64_t K,
                            uint8_t* q, uint8_t* scale) {
    float* w32 = (float*)malloc((size_t)(M * K > 0 ? M * K : 1) * sizeof(float));
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < M; r++)
        for (int64_t c = 0; c < K; c++)
            w32[r * K + c] = mqo_e4m3fn_to_f32(x[r * K + c]) * s[(r / 128) * lds + c / 128];
    mqo_mxfp8(w32, MQ_F32, M, K, q, scale);
    free(w32);
}

/* _load_source_scale_u8's test of an fp32 scale grid (:81-86): 1 when every mantissa is zero and no
 * value has its sign bit set (the scales are then relabelled, not re-quantized), else 0. */
int mqo_fp8_scales_pow2(const float* s, int64_t rows, int64_t cols, int64_t lds) {
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < cols; c++) {
            uint32_t u = f2u(s[r * lds + c]);
            if ((u & 0x007FFFFFu) != 0 || (u >> 31) != 0) return 0;
        }
    return 1;
}

/* _source_fp8_to_mxfp8_scale_u8 (:98-102): one exponent byte per 128x128 tile -> one per 1x32 group
 * (repeated 128 down and 4 across, cropped to [M, groups]).  is_f32: the grid holds fp32 powers of
 * two and the byte is (bits >> 23) & 0xFF (:85); otherwise it holds the bytes themselves (:89-93). */
void mqo_e8m0_expand_tile_scales(const void* s, int is_f32, int64_t lds, int64_t M, int64_t groups, uint8_t* out) {
    for (int64_t r = 0; r < M; r++)
        for (int64_t g = 0; g < groups; g++) {
            int64_t i = (r / 128) * lds + g / 4;
            out[r * groups + g] = is_f32 ? (uint8_t)((f2u(((const float*)s)[i]) >> 23) & 0xFFu) : ((const uint8_t*)s)[i];
        }
}

/* ------------------------------------------------------------------ */
/* MXFP4 (miles/utils/mxfp4.py:11-59): torch ops restated one by one    */
/* ------------------------------------------------------------------ */
/* quantize_mxfp4 (:11-31).  Groups of G consecutive elements of the flattened tensor.
 *   amax = max|x| (.float())                      (:16)
 *   e = clamp(ceil(log2(amax / 6.0)), -127, 127)  (:17)  log2f(0) = -inf clamps to -127
 *   n = f32(x) * exp2(-e)                         (:18)  exp2 of an integer is an exact power of two
 *   magnitude = number of bounds below |n|        (:20-22) strict '>': a tie takes the smaller magnitude
 *   code = magnitude | signbit(n) << 3            (:23)
 *   byte j = code[2j] | code[2j+1] << 4           (:25)
 *   scale = uint8(e + 127)                        (:27) */
void mqo_mxfp4_quant(const void* w, int dtype, int64_t numel, int G, uint8_t* packed, uint8_t* scale) {
    static const float bound[7] = {0.25f, 0.75f, 1.25f, 1.75f, 2.5f, 3.5f, 5.0f};
    int64_t groups = numel / G;
    uint8_t* code = (uint8_t*)malloc((size_t)numel + 1);
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < groups; g++) {
        float amax = 0.0f;
        for (int j = 0; j < G; j++) amax = fmaxf(amax, fabsf(load_as_f32(w, g * G + j, dtype)));
        float e = ceilf(log2f(amax / 6.0f));
        if (e < -127.0f) e = -127.0f;
        if (e > 127.0f) e = 127.0f;
        float mult = ldexpf(1.0f, -(int)e);
        for (int j = 0; j < G; j++) {
            float n = load_as_f32(w, g * G + j, dtype) * mult;
            uint8_t mag = 0;
            for (int b = 0; b < 7; b++) mag += fabsf(n) > bound[b];
            code[g * G + j] = (uint8_t)(mag | ((signbit(n) ? 1 : 0) << 3));
        }
        scale[g] = (uint8_t)(e + 127.0f);
    }
    for (int64_t j = 0; j < numel / 2; j++) packed[j] = (uint8_t)(code[2 * j] | (code[2 * j + 1] << 4));
    free(code);
}

/* dequantize_mxfp4 (:34-59): value = sign * {0,.5,1,1.5,2,3,4,6}[code & 7], sign = 1 - 2*bit3 (so a set sign
 * bit on magnitude 0 gives -0); y = bf16(value * exp2(scale - 127)); exp2(128) overflows to inf. */
void mqo_mxfp4_dequant(const uint8_t* packed, const uint8_t* scale, int64_t bytes, int G, uint16_t* y) {
    static const float value[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < 2 * bytes; i++) {
        uint8_t c = (i & 1) ? (packed[i / 2] >> 4) : (packed[i / 2] & 0xF);
        float sign = 1.0f - 2.0f * (float)((c >> 3) & 1);
        float s = ldexpf(1.0f, (int)scale[i / G] - 127);
        y[i] = f32_to_bf16(sign * value[c & 7] * s);
    }
}

/* ------------------------------------------------------------------ */
/* Block fake quantization (miles/kernels/quant/fake_quant.py:16-63)     */
/* ------------------------------------------------------------------ */
/* _ceil_pow2 (:16-22): exponent + (mantissa != 0), rebuilt as a power of two (inputs are normal). */
static inline float fq_ceil_pow2(float v) {
    uint32_t bits = f2u(v);
    int32_t e = (int32_t)((bits >> 23) & 0xFF) - 127 + ((bits & 0x7FFFFF) != 0);
    return u2f((uint32_t)(e + 127) << 23);
}
/* mode 0 fp8 1x32, mode 1 fp4 1x32 (power-of-two scales), mode 2 fp4 1x16 with an e4m3 scale (:41-62):
 *   E4M3_SCALE: scale = f32(e4m3(min(max(amax * INV_FMAX, FLOOR), 448))); scaled = div_rn(x, scale)
 *   else      : scale = ceil_pow2(max(amax, FLOOR) * INV_FMAX);            scaled = x / scale (exact)
 *   scaled = clamp(scaled, -FMAX, FMAX)
 *   FP4: q = rint(|s| / step) * step * sign(s), step 0.5 / 1 / 2 below 2 / 4 / above; sign(0) = 0
 *   FP8: q = f32(e4m3(s))
 *   out = dtype(q * scale)
 * INV_FMAX is the fp32 constant nearest 1/448 or 1/6. */
void mqo_fake_quant(const void* x, int dtype, int64_t numel, int mode, void* y) {
    const int block = mode == 2 ? 16 : 32;
    const float fmax_ = mode == 0 ? 448.0f : 6.0f;
    const float inv = mode == 0 ? u2f(0x3B124925u) : u2f(0x3E2AAAABu);
    const float floor_ = mode == 0 ? 1e-4f : mode == 1 ? u2f(0x01C00000u) : 0.001953125f;
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < numel / block; g++) {
        float amax = 0.0f;
        for (int j = 0; j < block; j++) amax = fmaxf(amax, fabsf(load_as_f32(x, g * block + j, dtype)));
        float scale;
        if (mode == 2) scale = mqo_e4m3fn_to_f32(mqo_f32_to_e4m3fn(fminf(fmaxf(amax * inv, floor_), 448.0f)));
        else scale = fq_ceil_pow2(fmaxf(amax, floor_) * inv);
        for (int j = 0; j < block; j++) {
            float s = load_as_f32(x, g * block + j, dtype) / scale;
            s = fminf(fmaxf(s, -fmax_), fmax_);
            float q;
            if (mode == 0) q = mqo_e4m3fn_to_f32(mqo_f32_to_e4m3fn(s));
            else {
                float mag = fabsf(s);
                float step = mag < 2.0f ? 0.5f : mag < 4.0f ? 1.0f : 2.0f;
                float sign = s > 0.0f ? 1.0f : s < 0.0f ? -1.0f : 0.0f;
                q = rintf(mag / step) * step * sign;
            }
            float o = q * scale;
            int64_t i = g * block + j;
            if (dtype == MQ_F32) ((float*)y)[i] = o;
            else ((uint16_t*)y)[i] = dtype == MQ_BF16 ? f32_to_bf16(o) : f32_to_f16(o);
        }
    }
}

/* act_quant (miles/kernels/quant/fp8_act_quant.py:49-137): FP8 quantization of 1 x block groups of the last
 * dimension, the form DeepSeek-V4's activation / KV simulation uses.
 *   amax  = max(max|x|, 1e-4)                                                        (:84)
 *   s     = amax * f32(1/448);  round_scale: s = 2^ceil(log2(s)) read off the bits   (:85-88, :29-46)
 *   code  = e4m3(min(max(x / s, -448), 448))      <- fp32 division                   (:100-101)
 *   inplace: y = dtype(f32(code) * s)                                                (:90-98)
 *   scale stored as fp32, or (power-of-two scales only) as its E8M0 exponent byte    (:102-103)
 * flags: 1 = round_scale, 2 = E8M0 scale bytes, 4 = inplace (y has the input dtype).
 * fp8_simulate (miles_plugins/models/deepseek_v4/ops/qat.py:8-23) = flags 1|4: the TileKernels cast-back it calls
 * multiplies the decoded code by the scale and rounds to the output dtype, as the inplace branch does. */
void mqo_fp8_act_quant(const void* x, int dtype, int64_t numel, int block, int flags, void* y, void* scale) {
    const float inv = u2f(0x3B124925u);
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < numel / block; g++) {
        float amax = 0.0f;
        for (int j = 0; j < block; j++) amax = fmaxf(amax, fabsf(load_as_f32(x, g * block + j, dtype)));
        float s = fmaxf(amax, 1e-4f) * inv;
        if (flags & 1) s = fq_ceil_pow2(s);
        if (flags & 2) ((uint8_t*)scale)[g] = (uint8_t)(f2u(s) >> 23);
        else ((float*)scale)[g] = s;
        for (int j = 0; j < block; j++) {
            int64_t i = g * block + j;
            float r = load_as_f32(x, i, dtype) / s;
            uint8_t code = mqo_f32_to_e4m3fn(fminf(fmaxf(r, -448.0f), 448.0f));
            if (!(flags & 4)) { ((uint8_t*)y)[i] = code; continue; }
            float o = mqo_e4m3fn_to_f32(code) * s;
            if (dtype == MQ_F32) ((float*)y)[i] = o;
            else ((uint16_t*)y)[i] = dtype == MQ_BF16 ? f32_to_bf16(o) : f32_to_f16(o);
        }
    }
}

/* cast_e2m1fn_to_e4m3fn (tools/convert_mxfp4_to_fp8.py:30-49): per 128x128 tile
 *   tile_scale = max(f32(scale)) / 64;  offset = f32(scale) / tile_scale;  y = e4m3(table[code] * offset)
 * scale bytes are float8_e8m0fnu: f32 = 2^(s-127) (s = 0 is the fp32 denormal 2^-127, s = 255 NaN). */
void mqo_mxfp4_to_fp8_block(const uint8_t* packed, const uint8_t* scale, int64_t out_dim, int64_t in_dim,
                            uint8_t* y, float* tile_scale) {
    static const float table[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                    -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};
    int64_t b_out = out_dim / 128, b_in = in_dim / 128, gpr = in_dim / 32;
#pragma omp parallel for schedule(static) collapse(2)
    for (int64_t ti = 0; ti < b_out; ti++)
        for (int64_t tj = 0; tj < b_in; tj++) {
            float top = 0.0f;
            for (int r = 0; r < 128; r++)
                for (int g = 0; g < 4; g++) {
                    uint8_t sb = scale[(ti * 128 + r) * gpr + tj * 4 + g];
                    float f = sb == 255 ? NAN : ldexpf(1.0f, (int)sb - 127);
                    top = (f > top || f != f) ? f : top;      /* amax propagates NaN */
                }
            float ts = top / 64.0f;
            tile_scale[ti * b_in + tj] = ts;
            for (int r = 0; r < 128; r++)
                for (int c = 0; c < 128; c++) {
                    int64_t row = ti * 128 + r, col = tj * 128 + c;
                    uint8_t byte = packed[row * (in_dim / 2) + col / 2];
                    uint8_t code = (col & 1) ? (byte >> 4) : (byte & 0xF);
                    uint8_t sb = scale[row * gpr + col / 32];
                    float offset = (sb == 255 ? NAN : ldexpf(1.0f, (int)sb - 127)) / ts;
                    y[row * in_dim + col] = mqo_f32_to_e4m3fn(table[code] * offset);
                }
        }
}

/* ------------------------------------------------------------------ */
/* A-3  INT4 fake quant (miles/kernels/quant/int4_fake/                 */
/*      fake_int4_quant_cuda.cu:159-259 for (1,G); :29-91 for (1,32))   */
/* ------------------------------------------------------------------ */
/* symmetric:  scale = fmaxf(amax * (1.0f/7.0f), 1e-5f); out = rintf(x/scale)
 * asymmetric: scale = fmaxf((max-min) * (1.0f/15.0f), 1e-5f);
 *             zero  = clamp(-rintf(min/scale), 0, 15); out = rintf(x/scale)+zero
 * out/scale/zero are stored in the input dtype (.cu:251-254).  Columns past N
 * in a ragged last group read as 0 (.cu:209-213). */
/* General block (BM, BN): a group is a BM x BN tile of the matrix, rows and columns past the edge read as 0
 * (.cu:95-150 for (32,1), :159-259 for the rest); one scale / zero per tile, shape [ceil(M/BM), ceil(N/BN)]. */
void mqo_int4_fake_quant_block(const void* x, int dtype, int64_t M, int64_t N, int BM, int BN, int sym,
                               void* out, void* scale_out, void* zero_out) {
    const float SYM = 1.0f / 7.0f, ASYM = 1.0f / 15.0f;
    int64_t gm = (M + BM - 1) / BM, gn = (N + BN - 1) / BN;
#pragma omp parallel for schedule(static) collapse(2)
    for (int64_t bi = 0; bi < gm; bi++)
        for (int64_t bj = 0; bj < gn; bj++) {
            float mx = -INFINITY, mn = INFINITY;
            for (int64_t r = bi * BM; r < (bi + 1) * BM; r++)
                for (int64_t c = bj * BN; c < (bj + 1) * BN; c++) {
                    float v = (r < M && c < N) ? load_as_f32(x, r * N + c, dtype) : 0.0f;
                    if (sym) mx = fmaxf(mx, fabsf(v));
                    else { mx = fmaxf(mx, v); mn = fminf(mn, v); }
                }
            float scale, zero = 0.0f;
            if (sym) scale = fmaxf(mx * SYM, 1e-5f);
            else {
                scale = fmaxf((mx - mn) * ASYM, 1e-5f);
                zero = fminf(fmaxf(-rintf(mn / scale), 0.0f), 15.0f);
                /* the device max orders -0 below +0, so a group whose minimum is 0 gets +0 (C's fmaxf
                 * may return either zero) */
                if (zero == 0.0f) zero = 0.0f;
            }
            for (int64_t r = bi * BM; r < (bi + 1) * BM && r < M; r++)
                for (int64_t c = bj * BN; c < (bj + 1) * BN && c < N; c++) {
                    float v = rintf(load_as_f32(x, r * N + c, dtype) / scale); /* keeps -0 */
                    if (!sym) v = v + zero;
                    if (dtype == MQ_F32) ((float*)out)[r * N + c] = v;
                    else ((uint16_t*)out)[r * N + c] = dtype == MQ_BF16 ? f32_to_bf16(v) : f32_to_f16(v);
                }
            int64_t g = bi * gn + bj;
            if (dtype == MQ_F32) {
                ((float*)scale_out)[g] = scale;
                if (!sym) ((float*)zero_out)[g] = zero;
            } else {
                ((uint16_t*)scale_out)[g] = dtype == MQ_BF16 ? f32_to_bf16(scale) : f32_to_f16(scale);
                if (!sym) ((uint16_t*)zero_out)[g] = dtype == MQ_BF16 ? f32_to_bf16(zero) : f32_to_f16(zero);
            }
        }
}
void mqo_int4_fake_quant(const void* x, int dtype, int64_t M, int64_t N, int G, int sym,
                         void* out, void* scale_out, void* zero_out) {
    mqo_int4_fake_quant_block(x, dtype, M, N, 1, G, sym, out, scale_out, zero_out);
}

/* pack_layer(weight, G, sym=True)
 * (miles/backends/megatron_utils/megatron_to_hf/processors/
 *  quantizer_compressed_tensors.py:235-265; quantize :196-225;
 *  round_to_quantized_type_dtype :183-193; pack_to_int32 :137-180):
 *   (out, scale_b) = fake_int4_quant(x)         -- in the input dtype
 *   w = dtype(out * scale_b)                    (:241)
 *   r = dtype(w / scale_b)                      (:213)
 *   q = int8(round_half_even(clamp(r,-128,127)))(:190)
 *   code = uint8(q + 8)                         (:153-155)
 *   packed[m,j] = sum_i code[m,8j+i] << 4i      (:173-175) int32 wraparound
 * K must be a multiple of G and of 8. */
void mqo_int4_pack_layer(const void* w, int dtype, int64_t M, int64_t K, int G,
                         int32_t* packed, void* scale_out) {
    size_t esz = dtype == MQ_F32 ? 4 : 2;
    void* out = malloc((size_t)M * K * esz);
    mqo_int4_fake_quant(w, dtype, M, K, G, 1, out, scale_out, NULL);
    int64_t ng = K / G, np = K / 8;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < M; r++)
        for (int64_t j = 0; j < np; j++) {
            uint32_t word = 0;
            for (int i = 0; i < 8; i++) {
                int64_t c = j * 8 + i;
                float q0 = load_as_f32(out, r * K + c, dtype);
                float sb = load_as_f32(scale_out, r * ng + c / G, dtype);
                float wv = round_to_dtype(q0 * sb, dtype);
                float rv = round_to_dtype(wv / sb, dtype);
                if (rv < -128.0f) rv = -128.0f;
                if (rv > 127.0f) rv = 127.0f;
                int8_t qi = (int8_t)nearbyintf(rv);
                uint8_t code = (uint8_t)(qi + 8);
                word += (uint32_t)code << (4 * i);
            }
            packed[r * np + j] = (int32_t)word;
        }
    free(out);
}

/* pack_layer(weight, G, sym=False)  (same file, :235-264):
 *   (out, scale_b, zero_b) = fake_int4_quant(x, sym=False)   -- in the input dtype
 *   w  = dtype(dtype(out - zero_b) * scale_b)                (:243)
 *   r  = dtype(dtype(w / scale_b) + zero_b)                  (:213-217)
 *   q  = uint8(round_half_even(clamp(r, 0, 255)))            (:190)
 *   packed[m,j] = sum_i q[m,8j+i] << 4i                      (:173-175; no offset when sym=False, :153)
 *   packed_zp[g,j] = sum_i int32(zero[8j+i,g]) << 4*{0,4,1,5,2,6,3,7}[i]   (:247-254)
 * K % G == 0, G % 8 == 0, M % 8 == 0. */
void mqo_int4_pack_layer_asym(const void* w, int dtype, int64_t M, int64_t K, int G,
                              int32_t* packed, void* scale_out, int32_t* packed_zp) {
    static const int order[8] = {0, 4, 1, 5, 2, 6, 3, 7};
    size_t esz = dtype == MQ_F32 ? 4 : 2;
    int64_t ng = K / G, np = K / 8;
    void* out = malloc((size_t)M * K * esz);
    void* zero = malloc((size_t)M * ng * esz);
    mqo_int4_fake_quant(w, dtype, M, K, G, 0, out, scale_out, zero);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < M; r++)
        for (int64_t j = 0; j < np; j++) {
            uint32_t word = 0;
            for (int i = 0; i < 8; i++) {
                int64_t c = j * 8 + i;
                float q0 = load_as_f32(out, r * K + c, dtype);
                float sb = load_as_f32(scale_out, r * ng + c / G, dtype);
                float zb = load_as_f32(zero, r * ng + c / G, dtype);
                float wv = round_to_dtype(round_to_dtype(q0 - zb, dtype) * sb, dtype);
                float rv = round_to_dtype(round_to_dtype(wv / sb, dtype) + zb, dtype);
                if (rv < 0.0f) rv = 0.0f;
                if (rv > 255.0f) rv = 255.0f;
                uint8_t code = (uint8_t)nearbyintf(rv);
                word += (uint32_t)code << (4 * i);
            }
            packed[r * np + j] = (int32_t)word;
        }
    for (int64_t g = 0; g < ng; g++)
        for (int64_t j = 0; j < M / 8; j++) {
            uint32_t word = 0;
            for (int i = 0; i < 8; i++)
                word += (uint32_t)(int32_t)load_as_f32(zero, (j * 8 + i) * ng + g, dtype) << (4 * order[i]);
            packed_zp[g * (M / 8) + j] = (int32_t)word;
        }
    free(out);
    free(zero);
}

/* _dequantize_tensor (tools/convert_kimi_int4_to_bf16.py:57-86): compressed-tensors' unpack_from_int32 (third
 * party, not in the reference tree; its published algorithm: element 8j+i = ((word_j >> 4i) & 15) - 8, rows
 * cropped to K) followed by bf16(f32(value) * f32(scale)) with one scale per G columns. */
void mqo_int4_unpack_dequant(const int32_t* packed, const void* scale, int scale_dtype, int64_t M, int64_t K, int G,
                             uint16_t* y) {
    int64_t wpr = (K + 7) / 8, gpr = K / G;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < M; r++)
        for (int64_t c = 0; c < K; c++) {
            uint32_t word = (uint32_t)packed[r * wpr + c / 8];
            float v = (float)((int)((word >> (4 * (c & 7))) & 0xFu) - 8);
            y[r * K + c] = f32_to_bf16(v * load_as_f32(scale, r * gpr + c / G, scale_dtype));
        }
}

/* ------------------------------------------------------------------ */
/* A-4  NVFP4 (miles/utils/nvfp4.py:19-134; block arithmetic restated   */
/*      from miles/kernels/quant/nvfp4_qdq.py:716-743,859-889,1079-1081)*/
/* ------------------------------------------------------------------ */
#define MQO_FLT_MAX 3.402823466e+38f

/* global amax = max |f32(x)| over the tensor (nvfp4_qdq.py:1213-1217). */
float mqo_nvfp4_amax(const void* w, int dtype, int64_t numel) {
    float amax = 0.0f;
#pragma omp parallel for reduction(max : amax) schedule(static)
    for (int64_t i = 0; i < numel; i++) {
        float a = fabsf(load_as_f32(w, i, dtype));
        if (a > amax) amax = a;
    }
    return amax;
}

/* Published global scale (miles/utils/nvfp4.py:19-39):
 *   enc = min(e4m3_max*6 / amax, FLT_MAX); enc == 0 -> 1; weight_scale_2 = 1/enc
 * torch.clamp_max / torch.min propagate NaN. */
float mqo_nvfp4_global_encode_scale(float amax, int e4m3_max) {
    float enc = ((float)e4m3_max * 6.0f) / amax;
    if (enc == enc && enc > MQO_FLT_MAX) enc = MQO_FLT_MAX;
    if (enc == 0.0f) enc = 1.0f;
    return enc;
}
float mqo_nvfp4_global_decode_scale(float amax, int e4m3_max) {
    return 1.0f / mqo_nvfp4_global_encode_scale(amax, e4m3_max);
}

/* In-kernel encode scale (nvfp4_qdq.py:859-867): additionally amax == 0 -> 1;
 * PTX min.f32 returns the non-NaN operand. */
static inline float nvfp4_kernel_encode_scale(float amax, int e4m3_max) {
    float enc = ((float)e4m3_max * 6.0f) / amax;
    enc = fminf(enc, MQO_FLT_MAX);
    if (amax == 0.0f) enc = 1.0f;
    if (enc == 0.0f) enc = 1.0f;
    return enc;
}

float mqo_e2m1_to_f32(uint8_t c);

/* Candidate error of Four Over Six (nvfp4_qdq.py:893-953): the sum, in element order and in fp32, of
 *   default : | RN(RN(RN(value * f32(scale)) * amax) / (6 * e4m3_max)) - x |        (or its square, MSE)
 *   fp16    : | f32(RN_f16(f16(value) * f16(scale))) - RN(x * S_enc) |              (or its square)
 * over the 16 elements of the block. */
static float nvfp4_candidate_error(const float* x, const uint8_t* codes, uint8_t scale, float amax, float S_enc,
                                   int e4m3_max, int flags) {
    const int mse = flags & MQ_NVFP4_ERR_MSE, fp16 = flags & MQ_NVFP4_ERR_FP16;
    const float denom = (float)(6 * e4m3_max), scale_f = mqo_e4m3fn_to_f32(scale);
    float error = 0.0f;
    for (int i = 0; i < 16; i++) {
        float cand = mqo_e2m1_to_f32(codes[i]), diff;
        if (fp16) {
            /* both factors are exact in fp16 and their product is exact in fp32: one rounding to fp16 */
            float prod = f16_to_f32(f32_to_f16(cand * scale_f));
            diff = prod - x[i] * S_enc;
        } else {
            float dq = cand * scale_f;
            dq = dq * amax;
            dq = dq / denom;
            diff = dq - x[i];
        }
        error = error + (mse ? diff * diff : fabsf(diff));
    }
    return error;
}

/* w: [M,K] contiguous, K % 16 == 0.  q: [M,K/2] (element 2i in the low
 * nibble).  s8: [M,K/16] e4m3fn bytes.  amax: global amax (for a gate/up
 * pair: over both tensors).
 * flags & MQ_NVFP4_4OVER6 (nvfp4_qdq.py:956-990): two candidates per block,
 *   scale6 = e4m3(min(RN(RN(bmax / 6) * S_enc), 448)), scale4 = e4m3(min(RN(that product * 1.5), 448)),
 * each quantized with its own inverse; the map-to-4 candidate wins only on a strictly smaller error. */
void mqo_nvfp4_quant_ex(const void* w, int dtype, int64_t M, int64_t K, float amax,
                        int e4m3_max, int flags, uint8_t* q, uint8_t* s8) {
    const float sixth = u2f(0x3E2AAAABu);
    float S_enc = nvfp4_kernel_encode_scale(amax, e4m3_max);
    float S_dec = 1.0f / S_enc;                      /* nvfp4_qdq.py:1081 */
    float enc_sixth = S_enc * sixth;                 /* :728 association */
    int64_t nb = K / 16;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < M; r++)
        for (int64_t b = 0; b < nb; b++) {
            int64_t base = r * K + b * 16;
            float x[16], bmax = 0.0f;
            for (int i = 0; i < 16; i++) {
                x[i] = load_as_f32(w, base + i, dtype);
                float a = fabsf(x[i]);
                if (a > bmax) bmax = a;
            }
            uint8_t sc, codes[16];
            if (flags & MQ_NVFP4_4OVER6) {
                float s6_hp = (bmax / 6.0f) * S_enc;
                float s4_hp = s6_hp * 1.5f;
                uint8_t sc4 = mqo_f32_to_e4m3fn_sat(fminf(s4_hp, 448.0f)), sc6 = mqo_f32_to_e4m3fn_sat(fminf(s6_hp, 448.0f));
                float inv4 = fminf(1.0f / (mqo_e4m3fn_to_f32(sc4) * S_dec), MQO_FLT_MAX);
                float inv6 = fminf(1.0f / (mqo_e4m3fn_to_f32(sc6) * S_dec), MQO_FLT_MAX);
                uint8_t c4[16], c6[16];
                for (int i = 0; i < 16; i++) {
                    c4[i] = mqo_f32_to_e2m1(x[i] * inv4);
                    c6[i] = mqo_f32_to_e2m1(x[i] * inv6);
                }
                float e4 = nvfp4_candidate_error(x, c4, sc4, amax, S_enc, e4m3_max, flags);
                float e6 = nvfp4_candidate_error(x, c6, sc6, amax, S_enc, e4m3_max, flags);
                int pick4 = e4 < e6;
                sc = pick4 ? sc4 : sc6;
                memcpy(codes, pick4 ? c4 : c6, 16);
            } else {
                float s_hp = (bmax == 0.0f) ? 0.0f : bmax * enc_sixth; /* :716-743 */
                sc = mqo_f32_to_e4m3fn_sat(s_hp);                     /* :489-511 */
                float inv = fminf(1.0f / (mqo_e4m3fn_to_f32(sc) * S_dec), MQO_FLT_MAX); /* :870-873 */
                for (int i = 0; i < 16; i++) codes[i] = mqo_f32_to_e2m1(x[i] * inv);
            }
            s8[r * nb + b] = sc;
            for (int i = 0; i < 16; i += 2) q[(base + i) / 2] = (uint8_t)(codes[i] | (codes[i + 1] << 4)); /* :571-575 */
        }
}
void mqo_nvfp4_quant(const void* w, int dtype, int64_t M, int64_t K, float amax,
                     int e4m3_max, uint8_t* q, uint8_t* s8) {
    mqo_nvfp4_quant_ex(w, dtype, M, K, amax, e4m3_max, 0, q, s8);
}

/* fused_nvfp4_qdq (miles/kernels/quant/nvfp4_qdq.py:877-890, 956-1029, 1067-1105):
 * quantize exactly as mqo_nvfp4_quant_ex, then
 *   final = RN(RN(f32(s8) * amax) * f32(1 / (6 * e4m3_max)));  y = dtype(RN(e2m1 value * final))
 * x bf16 or fp16, numel % 16 == 0. */
void mqo_nvfp4_qdq(const void* x, int dtype, int64_t numel, float amax, int e4m3_max, int flags, uint16_t* y) {
    const float inv_numer = (float)(1.0 / (double)(6 * e4m3_max));
    int64_t nb = numel / 16;
    uint8_t* q = (uint8_t*)malloc((size_t)numel / 2 + 1);
    uint8_t* s8 = (uint8_t*)malloc((size_t)nb + 1);
    mqo_nvfp4_quant_ex(x, dtype, nb, 16, amax, e4m3_max, flags, q, s8);
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < nb; b++) {
        float final = (mqo_e4m3fn_to_f32(s8[b]) * amax) * inv_numer;
        for (int i = 0; i < 16; i++) {
            uint8_t byte = q[(b * 16 + i) / 2];
            float v = mqo_e2m1_to_f32((i & 1) ? (byte >> 4) : (byte & 0xF)) * final;
            y[b * 16 + i] = dtype == MQ_BF16 ? f32_to_bf16(v) : f32_to_f16(v);
        }
    }
    free(q);
    free(s8);
}

/* ------------------------------------------------------------------ */
/* decode helpers used by round-trip property tests                     */
/* ------------------------------------------------------------------ */
float mqo_e2m1_to_f32(uint8_t c) {
    static const float tab[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
    float v = tab[c & 7];
    return (c & 8) ? -v : v;
}

/* vector forms so that tests can sweep many values quickly */
void mqo_f32_to_e4m3fn_vec(const float* x, int64_t n, uint8_t* out, int sat) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) out[i] = sat ? mqo_f32_to_e4m3fn_sat(x[i]) : mqo_f32_to_e4m3fn(x[i]);
}
void mqo_f32_to_e2m1_vec(const float* x, int64_t n, uint8_t* out) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) out[i] = mqo_f32_to_e2m1(x[i]);
}
void mqo_f32_to_bf16_vec(const float* x, int64_t n, uint16_t* out) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) out[i] = f32_to_bf16(x[i]);
}
void mqo_f32_to_e8m0_vec(const float* x, int64_t n, uint8_t* out) {
    for (int64_t i = 0; i < n; i++) out[i] = mqo_f32_to_e8m0_ceil(x[i]);
}

/* 64-bit FNV-1a over a byte range: cheap whole-tensor fingerprint for the
 * full-size parity checks (the same routine hashes oracle and GPU output). */
uint64_t mqo_fnv1a64(const uint8_t* p, int64_t n) {
    uint64_t h = 1469598103934665603ull;
    for (int64_t i = 0; i < n; i++) { h ^= p[i]; h *= 1099511628211ull; }
    return h;
}
