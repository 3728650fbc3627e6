/*
 * C restatement of the MoE dispatch / combine path.  TEST INFRASTRUCTURE ONLY:
 * it is the checker of the parity tests and the timed CPU baseline of the
 * benchmark, never part of the shipped library.
 *
 * Scalar code, one thread unless oracle_set_threads asks for more (tokens are
 * then split over OpenMP threads), written from the algorithm of the reference (cited
 * per function, paths relative to the reference checkout).  Choices where the
 * reference leaves something open are the same as in a2a_oracle.py: stable
 * (token, k) order inside an expert, and the bf16 -> fp8 e4m3 quantiser defined
 * below.  The number formats here use bit manipulation where the numpy oracle
 * uses arithmetic, so that the two pin each other.
 */
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* Threads used by oracle_dispatch_rank and oracle_combine_rank (tokens are split
 * over them; results do not depend on the number).  1 = the scalar port. */
static int g_threads = 1;
void oracle_set_threads(int n) { g_threads = n > 1 ? n : 1; }

static inline float bf16_to_f32(uint16_t v) {
    uint32_t b = (uint32_t)v << 16;
    float f;
    memcpy(&f, &b, 4);
    return f;
}

/* round to nearest even, the rounding of cvt.rn.bf16x2.f32 (combine_utils.cuh:14-23) */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    if ((b & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((b >> 16) | 0x40);
    b += 0x7FFFu + ((b >> 16) & 1u);
    return (uint16_t)(b >> 16);
}

/* float -> OCP fp8 e4m3 ("fn"), round to nearest even, no saturation: what
 * rounds beyond 448 becomes the NaN code. */
uint8_t oracle_e4m3fn_encode(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    const uint8_t sign = (uint8_t)((b >> 24) & 0x80);
    b &= 0x7FFFFFFFu;
    if (b > 0x43E80000u) return sign | 0x7F; /* NaN, inf, or above 464 (ties at 464 go to 448) */
    const int exp = (int)(b >> 23) - 127;
    const uint32_t man = b & 0x7FFFFFu;
    if (exp < -10) return sign;
    if (exp >= -6) {
        uint32_t code = ((uint32_t)(exp + 7) << 3) | (man >> 20);
        const uint32_t rem = man & 0xFFFFFu;
        if (rem > 0x80000u || (rem == 0x80000u && (code & 1u))) code++;
        return sign | (uint8_t)code;
    }
    /* subnormal result: multiples of 2^-9 */
    const uint32_t full = man | 0x800000u;
    const int shift = 23 - (exp + 9);
    uint32_t q = full >> shift;
    const uint32_t rem = full & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return sign | (uint8_t)q;
}

float oracle_e4m3fn_decode(uint8_t c) {
    const int e = (c >> 3) & 0xF, m = c & 7;
    float v;
    if ((c & 0x7F) == 0x7F) return NAN;
    v = e == 0 ? ldexpf((float)m, -9) : ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return (c & 0x80) ? -v : v;
}

void oracle_e4m3fn_encode_array(const float *in, uint8_t *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = oracle_e4m3fn_encode(in[i]);
}

/*
 * Histogram, stable rank of every entry inside its expert, inclusive scan
 * (a2a_dispatch_send.cu:176-243).  Tokens at or beyond `num_tokens` are not
 * routed.  Returns nonzero if an expert id is out of range.
 */
int oracle_route(const int32_t *indices, size_t indices_stride, uint32_t num_tokens, uint32_t K,
                 uint32_t E, uint32_t *count, uint32_t *token_offset, uint32_t *expert_offsets) {
    memset(count, 0, (size_t)E * sizeof *count);
    for (uint32_t t = 0; t < num_tokens; ++t) {
        for (uint32_t k = 0; k < K; ++k) {
            const uint32_t e = (uint32_t)indices[(size_t)t * indices_stride + k];
            if (e >= E) return 1;
            token_offset[(size_t)t * K + k] = count[e]++;
        }
    }
    uint32_t run = 0;
    for (uint32_t e = 0; e < E; ++e) {
        run += count[e];
        expert_offsets[e] = run;
    }
    return 0;
}

/* i-th source receiver `rank` lays out (a2a_worker.rs:681-694, dp_size 1). */
static uint32_t source_order(uint32_t rank, uint32_t i, uint32_t N, uint32_t node_size) {
    const uint32_t num_nodes = N / node_size, rank_node = rank / node_size;
    const uint32_t remote = (num_nodes - 1) * node_size;
    if (i < remote) return ((rank_node + 1 + i / node_size) % num_nodes) * node_size + i % node_size;
    const uint32_t local = i - remote + 1;
    if (local < node_size) return rank_node * node_size + (rank + local) % node_size;
    return rank;
}

/*
 * Receiver layout for every rank: tokens_per_expert[e], padded_offset[e] and
 * base[g*E+e], the first row of source g's run in expert e
 * (a2a_worker.rs:577-581,598-606,621-634,669-671).
 */
void oracle_layout(const uint32_t *num_routed, uint32_t N, uint32_t E, uint32_t node_size,
                   uint32_t expert_padding, uint32_t *tokens_per_expert, uint32_t *padded_offset,
                   uint32_t *base) {
    const uint32_t Le = (E + N - 1) / N;
    for (uint32_t r = 0; r < N; ++r) {
        uint32_t off = 0;
        for (uint32_t e = r * Le; e < (r + 1) * Le && e < E; ++e) {
            uint32_t tpe = 0;
            for (uint32_t g = 0; g < N; ++g) tpe += num_routed[(size_t)g * E + e];
            tokens_per_expert[e] = tpe;
            padded_offset[e] = off;
            uint32_t running = off;
            for (uint32_t i = 0; i < N; ++i) {
                const uint32_t g = source_order(r, i, N, node_size);
                base[(size_t)g * E + e] = running;
                running += num_routed[(size_t)g * E + e];
            }
            off += (tpe + expert_padding - 1) / expert_padding * expert_padding;
        }
    }
}

/*
 * bf16 row -> fp8 e4m3 codes + one float scale per 128 elements.  Not in the
 * reference; the rule (all float32, separately rounded operations):
 *   amax = max(max|x|, 1e-4); scale = amax / 448;
 *   q = e4m3fn(clamp(x * (448 / amax), -448, 448))
 * with maxima that propagate NaN and one spelling of NaN on output: a NaN in
 * the group gives scale 0x7FC00000 and 128 codes 0x7F; an infinity (no NaN)
 * gives scale +inf, code 0x7F for an infinite value (inf * 0) and a zero with
 * its sign for a finite one (x * 0).
 */
void oracle_quantize_row(const uint16_t *x, uint32_t H, uint8_t *q, float *scale) {
    for (uint32_t g = 0; g < H / 128; ++g) {
        float amax = 0.0f;
        int has_nan = 0;
        for (uint32_t i = 0; i < 128; ++i) {
            const float a = fabsf(bf16_to_f32(x[g * 128 + i]));
            if (a != a) has_nan = 1;
            if (a > amax) amax = a;
        }
        if (has_nan) {
            const uint32_t quiet = 0x7FC00000u;
            memcpy(&scale[g], &quiet, 4);
            memset(q + g * 128, 0x7F, 128);
            continue;
        }
        if (!(amax > 1e-4f)) amax = 1e-4f;
        volatile float inv = 448.0f / amax;
        scale[g] = amax / 448.0f;
        for (uint32_t i = 0; i < 128; ++i) {
            volatile float v = bf16_to_f32(x[g * 128 + i]) * inv;
            float c = v;
            if (c > 448.0f) c = 448.0f;
            if (c < -448.0f) c = -448.0f;
            const uint8_t code = oracle_e4m3fn_encode(c);
            q[g * 128 + i] = (code & 0x7F) == 0x7F ? 0x7F : code;
        }
    }
}

/*
 * dispatch of one source rank into the receivers' buffers: for every token and
 * route, the quantised row and its scales go to row base[e] + token_offset of
 * receiver e / Le (a2a_dispatch_send.cu:341-367, a2a_dispatch_recv.cu:139-155).
 * out_x[r] / out_scale[r] are the receivers' buffers (row strides H and Hs).
 * `qrow` / `srow` are scratch of H bytes / Hs floats.
 */
static void dispatch_tokens(const uint16_t *x, size_t x_stride_elems, const int32_t *indices,
                            size_t indices_stride, uint32_t t0, uint32_t t1, uint32_t H, uint32_t K,
                            uint32_t Le, const uint32_t *token_offset, const uint32_t *base_g,
                            uint8_t *const *out_x, float *const *out_scale, uint8_t *qrow, float *srow) {
    const uint32_t Hs = H / 128;
    for (uint32_t t = t0; t < t1; ++t) {
        oracle_quantize_row(x + (size_t)t * x_stride_elems, H, qrow, srow);
        for (uint32_t k = 0; k < K; ++k) {
            const uint32_t e = (uint32_t)indices[(size_t)t * indices_stride + k];
            const uint32_t r = e / Le;
            const size_t row = (size_t)base_g[e] + token_offset[(size_t)t * K + k];
            memcpy(out_x[r] + row * H, qrow, H);
            memcpy(out_scale[r] + row * Hs, srow, (size_t)Hs * sizeof(float));
        }
    }
}

void oracle_dispatch_rank(const uint16_t *x, size_t x_stride_elems, const int32_t *indices,
                          size_t indices_stride, uint32_t num_tokens, uint32_t H, uint32_t K,
                          uint32_t Le, const uint32_t *token_offset, const uint32_t *base_g,
                          uint8_t *const *out_x, float *const *out_scale, uint8_t *qrow,
                          float *srow) {
    if (g_threads <= 1) {
        dispatch_tokens(x, x_stride_elems, indices, indices_stride, 0, num_tokens, H, K, Le, token_offset, base_g,
                        out_x, out_scale, qrow, srow);
        return;
    }
    /* tokens are independent: split them over the threads, each with scratch of its own */
#pragma omp parallel num_threads(g_threads)
    {
        uint8_t *q = (uint8_t *)malloc(H);
        float *sc = (float *)malloc((size_t)(H / 128 + 1) * sizeof(float));
        const uint32_t n = (uint32_t)omp_get_num_threads(), i = (uint32_t)omp_get_thread_num();
        const uint32_t per = (num_tokens + n - 1) / n;
        const uint32_t t0 = i * per < num_tokens ? i * per : num_tokens;
        const uint32_t t1 = t0 + per < num_tokens ? t0 + per : num_tokens;
        if (q != NULL && sc != NULL)
            dispatch_tokens(x, x_stride_elems, indices, indices_stride, t0, t1, H, K, Le, token_offset, base_g,
                            out_x, out_scale, q, sc);
        free(q);
        free(sc);
    }
}

/*
 * combine for one source rank: out[t] = (accumulate ? out[t] : 0) + sum_k
 * w[t,k] * y(t,k), one fused multiply-add per k in float, k ascending, one
 * rounding to bf16 (a2a_combine_recv.cu:131-146, combine_utils.cuh:108-114).
 * expert_y[r] are the receivers' bf16 rows (row stride H).
 */
static void combine_tokens(uint16_t *out, size_t out_stride_elems, const int32_t *indices,
                           size_t indices_stride, const float *weights, size_t weights_stride,
                           uint32_t t0, uint32_t t1, uint32_t H, uint32_t K, uint32_t Le,
                           const uint32_t *token_offset, const uint32_t *base_g,
                           const uint16_t *const *expert_y, int accumulate, float *acc) {
    for (uint32_t t = t0; t < t1; ++t) {
        uint16_t *o = out + (size_t)t * out_stride_elems;
        for (uint32_t h = 0; h < H; ++h) acc[h] = accumulate ? bf16_to_f32(o[h]) : 0.0f;
        for (uint32_t k = 0; k < K; ++k) {
            const uint32_t e = (uint32_t)indices[(size_t)t * indices_stride + k];
            const float w = weights[(size_t)t * weights_stride + k];
            const size_t row = (size_t)base_g[e] + token_offset[(size_t)t * K + k];
            const uint16_t *y = expert_y[e / Le] + row * H;
            for (uint32_t h = 0; h < H; ++h) acc[h] = fmaf(w, bf16_to_f32(y[h]), acc[h]);
        }
        for (uint32_t h = 0; h < H; ++h) o[h] = f32_to_bf16(acc[h]);
    }
}

void oracle_combine_rank(uint16_t *out, size_t out_stride_elems, const int32_t *indices,
                         size_t indices_stride, const float *weights, size_t weights_stride,
                         uint32_t num_tokens, uint32_t H, uint32_t K, uint32_t Le,
                         const uint32_t *token_offset, const uint32_t *base_g,
                         const uint16_t *const *expert_y, int accumulate, float *acc) {
    if (g_threads <= 1) {
        combine_tokens(out, out_stride_elems, indices, indices_stride, weights, weights_stride, 0, num_tokens, H, K,
                       Le, token_offset, base_g, expert_y, accumulate, acc);
        return;
    }
#pragma omp parallel num_threads(g_threads)
    {
        float *a = (float *)malloc((size_t)H * sizeof(float));
        const uint32_t n = (uint32_t)omp_get_num_threads(), i = (uint32_t)omp_get_thread_num();
        const uint32_t per = (num_tokens + n - 1) / n;
        const uint32_t t0 = i * per < num_tokens ? i * per : num_tokens;
        const uint32_t t1 = t0 + per < num_tokens ? t0 + per : num_tokens;
        if (a != NULL)
            combine_tokens(out, out_stride_elems, indices, indices_stride, weights, weights_stride, t0, t1, H, K, Le,
                           token_offset, base_g, expert_y, accumulate, a);
        free(a);
    }
}

/* 2 * dequantised row as bf16: the stand-in for the experts used by the
 * reference's test and benchmark (test_p2p_all_to_all.py:44-50,
 * bench_all_to_all.py:40-50). */
void oracle_act_rows(const uint8_t *q, const float *scale, size_t rows, uint32_t H, uint16_t *y) {
    const uint32_t Hs = H / 128;
    for (size_t r = 0; r < rows; ++r) {
        for (uint32_t h = 0; h < H; ++h) {
            float v = oracle_e4m3fn_decode(q[r * H + h]);
            if (v != v) v = 0.0f;
            volatile float d = v * scale[r * Hs + h / 128];
            y[r * H + h] = f32_to_bf16(d * 2.0f);
        }
    }
}
