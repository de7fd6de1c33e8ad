/*
 * TEST INFRASTRUCTURE — CPU oracle for single-query ("decoding") attention.
 *
 * This file is the checker, never the product: only tests/, the smoke check and
 * the benchmark's cpu_baseline leg may load it.  The shipped library does not
 * link it and has no CPU fallback.
 *
 * It restates, from scratch, the algorithm of the reference's scalar CPU path
 * Tester<T>::attn_cpu (reference csrc/common/tester.h:133-259):
 *   pass 1  S[j] = sum_t f32(Q[b,h,t]) * f32(K[start+j, hk, t])      (tester.h:158-180)
 *   pass 2  s = S*scale (+ slope*(j-(len-1))), max, exp, sum, divide   (tester.h:186-229)
 *   pass 3  O[t] = cast( sum_j P[j] * f32(V[start+j, hk, t]) )         (tester.h:231-258)
 * with hk = h / (head_q/head_k) (tester.h:166,238), scale = 1/sqrt(dim)
 * (tester.h:186), slope_h = 1/exp2(8(h+1)/head_q) (tester.h:193), V == K's
 * buffer with K's row pitch when v is null (tester.h:149,244 and
 * csrc/ops/decoding_attn.cpp:30-37), fp32 accumulation in loop order, and a
 * round-to-nearest-even cast of the result (tester.h:250-254).
 *
 * Deliberate differences from the reference text, none of which changes a
 * result the reference can produce:
 *   - the score row is a per-(b,h) scratch vector; the reference indexes a
 *     [total_q, head_q, max_seq_k] buffer with the per-sequence length as the
 *     row pitch (tester.h:176,201), which is only right for equal lengths;
 *   - softmax scale and ALiBi slopes may be passed in; the defaults are the
 *     reference's closed forms;
 *   - a distinct V with dim_v != dim is read with its own pitch
 *     (head_k*dim_v); the reference has no caller for that case;
 *   - len <= 0 writes zeros to the output row (the reference leaves it
 *     untouched);
 *   - an optional OpenMP loop over (b,h); nthreads = 1 is the reference's
 *     behaviour (it contains no parallel pragma).
 *
 * Pinned by tests/test_oracle.py against float64 textbook attention, torch's
 * CPU scaled_dot_product_attention, head-expansion / slicing / closed-form
 * ALiBi identities and RNE tie cases; the reference holds no golden vectors.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                man <<= 1;
                ++e;
            } while ((man & 0x400u) == 0);
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static inline float bf16_to_f32(uint16_t h) {
    uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* fp32 -> bf16, round to nearest even (what __float2bfloat16 does). */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u); /* quiet NaN */
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7fffu + lsb;
    return (uint16_t)(x >> 16);
}

/* fp32 -> fp16, round to nearest even (what __float2half does). */
static inline uint16_t f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);  /* NaN */
    if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to inf */
    if (ax < 0x33000001u) return (uint16_t)sign;              /* <= 2^-25 rounds to zero */
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t man = (ax & 0x7fffffu) | 0x800000u;
    if (e < -14) { /* subnormal half: shift so that the unit is 2^-24 */
        int shift = (-14 - e) + 13;
        uint32_t q = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) ++q;
        return (uint16_t)(sign | q);
    }
    uint32_t q = ((uint32_t)(e + 15) << 10) | ((man >> 13) & 0x3ffu);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) ++q; /* carry into exponent is correct */
    return (uint16_t)(sign | q);
}

static inline float load_elem(const uint16_t *p, int is_bf16) {
    return is_bf16 ? bf16_to_f32(*p) : f16_to_f32(*p);
}

/* Exposed for the rounding known-answer tests. */
uint16_t oracle_f32_to_f16(float f) { return f32_to_f16(f); }
uint16_t oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }
float oracle_f16_to_f32(uint16_t h) { return f16_to_f32(h); }
float oracle_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }

int oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_num_procs();
#else
    return 1;
#endif
}

/*
 * q [batch, head_q, dim], k [total_k, head_k, dim], v [total_k, head_k, dim_v] or NULL,
 * o [batch, head_q, dim_v] (16-bit, same type as the inputs), cu_seq_k [batch+1].
 * softmax_scale <= 0 selects 1/sqrt(dim); alibi_slopes NULL selects 2^(-8(h+1)/head_q).
 * o_f32 (nullable) receives the un-rounded fp32 result, for tolerance studies.
 * Returns 0, or a negative code for an argument the reference would reject
 * (csrc/ops/decoding_attn.cpp:16-22).
 */
int oracle_attn_cpu(const uint16_t *q, const uint16_t *k, const uint16_t *v, uint16_t *o, const int32_t *cu_seq_k,
                    size_t max_seq_k, size_t batch, size_t head_q, size_t head_k, size_t dim, size_t dim_v,
                    int is_alibi, int is_bf16, float softmax_scale, const float *alibi_slopes, int nthreads,
                    float *o_f32) {
    if (!q || !k || !o || !cu_seq_k) return -1;
    if (head_k == 0 || head_q % head_k != 0) return -2;
    if (dim > 576 || dim_v > 512) return -3;
    if (!v && dim_v > dim) return -4;
    const size_t ratio = head_q / head_k;
    const size_t k_row = head_k * dim;
    const size_t v_row = v ? head_k * dim_v : head_k * dim;
    const size_t v_head = v ? dim_v : dim; /* tester.h:244 uses h_k*dim; equal whenever the reference runs */
    const uint16_t *vbuf = v ? v : k;
    const float scale = softmax_scale > 0.0f ? softmax_scale : (float)(1.0 / sqrt((double)dim));
    (void)max_seq_k;
    (void)nthreads;

    const long long work = (long long)batch * (long long)head_q;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 1) num_threads(nthreads > 0 ? nthreads : 1)
#endif
    for (long long w = 0; w < work; ++w) {
        const size_t b = (size_t)(w / (long long)head_q);
        const size_t h = (size_t)(w % (long long)head_q);
        const size_t hk = h / ratio;
        const long long start = cu_seq_k[b];
        const long long len = (long long)cu_seq_k[b + 1] - start;
        uint16_t *orow = o + (b * head_q + h) * dim_v;
        float *frow = o_f32 ? o_f32 + (b * head_q + h) * dim_v : NULL;
        if (len <= 0) {
            for (size_t t = 0; t < dim_v; ++t) {
                orow[t] = 0;
                if (frow) frow[t] = 0.0f;
            }
            continue;
        }
        float *s = (float *)malloc((size_t)len * sizeof(float));
        const uint16_t *qrow = q + (b * head_q + h) * dim;

        /* pass 1: raw dot products, fp32, ascending t (tester.h:167-176) */
        for (long long j = 0; j < len; ++j) {
            const uint16_t *krow = k + (size_t)(start + j) * k_row + hk * dim;
            float acc = 0.0f;
            for (size_t t = 0; t < dim; ++t) acc += load_elem(qrow + t, is_bf16) * load_elem(krow + t, is_bf16);
            s[j] = acc;
        }

        /* pass 2: scale, bias, softmax (tester.h:193-219) */
        float slope = 0.0f;
        if (is_alibi) slope = alibi_slopes ? alibi_slopes[h] : (float)(1.0 / exp2(8.0 * (double)(h + 1) / (double)head_q));
        const long long row_shift = len - 1;
        float mx = -3.402823466e+38f;
        for (long long j = 0; j < len; ++j) {
            float x = s[j] * scale;
            if (is_alibi && j < row_shift) x += slope * (float)((int)j - (int)row_shift);
            s[j] = x;
            if (x > mx) mx = x;
        }
        float sum = 0.0f;
        for (long long j = 0; j < len; ++j) {
            s[j] = expf(s[j] - mx);
            sum += s[j];
        }
        for (long long j = 0; j < len; ++j) s[j] = s[j] / sum;

        /* pass 3: O = P V, normalised P, fp32, ascending j (tester.h:239-254) */
        for (size_t t = 0; t < dim_v; ++t) {
            float acc = 0.0f;
            const uint16_t *vcol = vbuf + (size_t)start * v_row + hk * v_head + t;
            for (long long j = 0; j < len; ++j) acc += s[j] * load_elem(vcol + (size_t)j * v_row, is_bf16);
            orow[t] = is_bf16 ? f32_to_bf16(acc) : f32_to_f16(acc);
            if (frow) frow[t] = acc;
        }
        free(s);
    }
    return 0;
}
