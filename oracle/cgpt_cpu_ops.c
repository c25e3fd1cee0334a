/*
 * TEST INFRASTRUCTURE — NOT PART OF THE PRODUCT.
 *
 * Float32 CPU restatement of the operators of B4rtekk1/CGPT that sit on the
 * training hot path. It is the checker the GPU kernels are compared with and
 * the "port" CPU baseline that bench.py times; nothing under cgpt_amd/ may
 * call it. Each function follows the arithmetic (operation order, fused
 * multiply-adds, rounding to the storage dtype after every store, OpenMP loop
 * structure) of the reference file cited above it; paths are relative to the
 * reference checkout. Written from the reference's behaviour, not copied.
 *
 * The reference's own CPU sources include <cuda_runtime.h> and <cublasLt.h>
 * through include/core/tensor.h:9 and include/core/dtype.h:3, neither of which
 * exists in this image, so they cannot be compiled here; this restatement is
 * pinned instead by the known-answer vectors of the reference's tests and by
 * the float64 formulas in oracle64.py (see tests/test_oracle_*.py).
 *
 * Pinned functions: all of them except where a header below says
 * "parity unpinned".
 *
 * Build: see oracle/build.py (gcc -O2 -fopenmp -mavx2 -mfma -mf16c, the
 * reference's CPU flags, CMakeLists.txt:19-22, 63-66).
 */
#include <immintrin.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { CG_F16 = 0, CG_BF16 = 1, CG_F32 = 2 };

/* Element load/store with the conversions of every reference CPU op, e.g.
 * src/ops/cpu/backward/rmsnorm_backward_cpu.cpp:27-58: F16 through F16C,
 * BF16 by bit shift on load and round-to-nearest-even on store. */
static inline float load1(const void* p, int t, size_t i) {
    if (t == CG_F32) return ((const float*)p)[i];
    const uint16_t h = ((const uint16_t*)p)[i];
    if (t == CG_F16) return _cvtsh_ss(h);
    const uint32_t b = (uint32_t)h << 16;
    float x;
    memcpy(&x, &b, 4);
    return x;
}

static inline void store1(void* p, int t, size_t i, float x) {
    if (t == CG_F32) {
        ((float*)p)[i] = x;
        return;
    }
    if (t == CG_F16) {
        ((uint16_t*)p)[i] = _cvtss_sh(x, 0);
        return;
    }
    uint32_t b;
    memcpy(&b, &x, 4);
    ((uint16_t*)p)[i] = (uint16_t)((b + 0x7fff + ((b >> 16) & 1)) >> 16);
}

/* Eight-lane FMA dot product, lanes summed 0..7, then a scalar FMA tail:
 * src/ops/cpu/backward/attention_backward_cpu.cpp:76-93. */
static inline float dot8(const void* a, const void* b, int t, size_t ia, size_t ib, size_t d) {
    float s[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    size_t i = 0;
    for (; i + 7 < d; i += 8)
        for (int z = 0; z < 8; ++z) s[z] = fmaf(load1(a, t, ia + i + z), load1(b, t, ib + i + z), s[z]);
    float r = 0;
    for (int z = 0; z < 8; ++z) r += s[z];
    for (; i < d; ++i) r = fmaf(load1(a, t, ia + i), load1(b, t, ib + i), r);
    return r;
}

/* ------------------------------------------------------------------ RMSNorm */

/* src/ops/cpu/backward/rmsnorm_backward_cpu.cpp:86-133. */
void cg_rmsnorm_backward_cpu(void* gi, void* gw, const void* go, const void* x, const void* w, size_t rows,
                             size_t hidden, float eps, int t) {
    float* inv = (float*)malloc(rows * sizeof(float));
    float* dot = (float*)malloc(rows * sizeof(float));
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < (int64_t)rows; ++r) {
        const size_t base = (size_t)r * hidden;
        float ss = 0, dd = 0;
        for (size_t i = 0; i < hidden; ++i) {
            const float xv = load1(x, t, base + i), dy = load1(go, t, base + i), wv = load1(w, t, i);
            ss = fmaf(xv, xv, ss);
            dd = fmaf(dy * wv, xv, dd);
        }
        inv[r] = 1.0f / sqrtf(ss / (float)hidden + eps);
        dot[r] = dd;
    }
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < (int64_t)rows; ++r) {
        const size_t base = (size_t)r * hidden;
        const float iv = inv[r];
        const float corr = dot[r] * iv * iv * iv / (float)hidden;
        for (size_t i = 0; i < hidden; ++i) {
            const float xv = load1(x, t, base + i), dy = load1(go, t, base + i), wv = load1(w, t, i);
            store1(gi, t, base + i, dy * wv * iv - xv * corr);
        }
    }
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < (int64_t)hidden; ++j) {
        float s = 0;
        for (size_t r = 0; r < rows; ++r) {
            const size_t base = r * hidden;
            s = fmaf(load1(go, t, base + j), load1(x, t, base + j) * inv[r], s);
        }
        store1(gw, t, (size_t)j, s);
    }
    free(inv);
    free(dot);
}

/* src/ops/cpu/rmsnorm_cpu.cpp:150-165 (scalar branch): ss by FMA, y = x*inv*w. */
void cg_rmsnorm_forward_cpu(void* y, const void* x, const void* w, size_t rows, size_t hidden, float eps, int t) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < (int64_t)rows; ++r) {
        const size_t base = (size_t)r * hidden;
        float ss = 0;
        for (size_t i = 0; i < hidden; ++i) {
            const float xv = load1(x, t, base + i);
            ss = fmaf(xv, xv, ss);
        }
        const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
        for (size_t i = 0; i < hidden; ++i) store1(y, t, base + i, load1(x, t, base + i) * inv * load1(w, t, i));
    }
}

/* --------------------------------------------------------------------- RoPE */

static void rope_apply(void* oq, void* ok, const void* iq, const void* ik, const void* co, const void* si, size_t B,
                       size_t S, size_t Q, size_t K, size_t D, size_t R, size_t off, int t, int inverse) {
    const size_t P = R / 2;
#pragma omp parallel for schedule(static)
    for (int64_t z = 0; z < (int64_t)(B * S); ++z) {
        const size_t token = (size_t)z, pos = off + token % S;
        for (int which = 0; which < 2; ++which) {
            const size_t H = which ? K : Q;
            const void* in = which ? ik : iq;
            void* out = which ? ok : oq;
            for (size_t h = 0; h < H; ++h) {
                const size_t base = (token * H + h) * D;
                for (size_t p = 0; p < P; ++p) {
                    const float c = load1(co, t, pos * P + p), s = load1(si, t, pos * P + p);
                    const float x = load1(in, t, base + 2 * p), y = load1(in, t, base + 2 * p + 1);
                    if (inverse) {
                        store1(out, t, base + 2 * p, fmaf(y, s, x * c));
                        store1(out, t, base + 2 * p + 1, fmaf(-x, s, y * c));
                    } else {
                        store1(out, t, base + 2 * p, fmaf(-y, s, x * c));
                        store1(out, t, base + 2 * p + 1, fmaf(x, s, y * c));
                    }
                }
                for (size_t d = R; d < D; ++d) store1(out, t, base + d, load1(in, t, base + d));
            }
        }
    }
}

/* src/ops/cpu/backward/rope_backward_cpu.cpp:110-141. */
void cg_rope_backward_cpu(void* gq, void* gk, const void* rq, const void* rk, const void* co, const void* si, size_t B,
                          size_t S, size_t Q, size_t K, size_t D, size_t R, size_t off, int t) {
    rope_apply(gq, gk, rq, rk, co, si, B, S, Q, K, D, R ? R : D, off, t, 1);
}

/* src/ops/cpu/rope_cpu.cpp:110-120 (scalar branch), in place. */
void cg_rope_forward_cpu(void* q, void* k, const void* co, const void* si, size_t B, size_t S, size_t Q, size_t K,
                         size_t D, size_t R, size_t off, int t) {
    rope_apply(q, k, q, k, co, si, B, S, Q, K, D, R ? R : D, off, t, 0);
}

/* ------------------------------------------------------------------- SwiGLU */

static inline float silu_f(float x) {
    const float s = 1.0f / (1.0f + expf(-x));
    return x * s;
}
static inline float silu_grad_f(float x) {
    const float s = 1.0f / (1.0f + expf(-x));
    return s * (1.0f + x * (1.0f - s));
}

/* src/ops/cpu/backward/swiglu_backward_cpu.cpp:125-141. */
void cg_swiglu_backward_cpu(void* gg, void* gu, const void* go, const void* gate, const void* up, size_t n,
                            int acc_gate, int acc_up, int t) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; ++i) {
        const size_t j = (size_t)i;
        const float g = load1(go, t, j), x = load1(gate, t, j), u = load1(up, t, j);
        const float dg = g * u * silu_grad_f(x), du = g * silu_f(x);
        store1(gg, t, j, dg + (acc_gate ? load1(gg, t, j) : 0));
        store1(gu, t, j, du + (acc_up ? load1(gu, t, j) : 0));
    }
}

/* src/ops/cpu/backward/swiglu_backward_cpu.cpp:161-182: rows of [gate | up]. */
void cg_swiglu_backward_packed_cpu(void* ggu, const void* go, const void* gu, size_t rows, size_t h, int acc, int t) {
    const size_t n = rows * h;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; ++i) {
        const size_t j = (size_t)i, row = j / h, col = j % h;
        const size_t gb = row * 2 * h + col, ub = gb + h;
        const float g = load1(go, t, j), x = load1(gu, t, gb), u = load1(gu, t, ub);
        const float dg = g * u * silu_grad_f(x), du = g * silu_f(x);
        store1(ggu, t, gb, dg + (acc ? load1(ggu, t, gb) : 0));
        store1(ggu, t, ub, du + (acc ? load1(ggu, t, ub) : 0));
    }
}

/* src/ops/cpu/swiglu_cpu.cpp:162 (scalar branch): x/(1+exp(-x))*y. The AVX2
 * branch there (lines 150-160) uses a polynomial exp from
 * include/core/simd_math.h:35-92 that differs from expf by a few ulp. */
void cg_swiglu_forward_cpu(void* out, const void* gate, const void* up, size_t n, int t) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; ++i) {
        const float x = load1(gate, t, (size_t)i), y = load1(up, t, (size_t)i);
        store1(out, t, (size_t)i, x / (1 + expf(-x)) * y);
    }
}

/* ------------------------------------------------------------------- Linear */

/* src/ops/cpu/backward/linear_backward_cpu.cpp:131-165. */
void cg_linear_backward_cpu(void* gi, void* gw, void* gb, const void* go, const void* x, const void* w, size_t rows,
                            size_t I, size_t O, int acc_in, int acc_w, int acc_b, int t) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < (int64_t)rows; ++r) {
        const size_t rb = (size_t)r * I, ob = (size_t)r * O;
        for (size_t i = 0; i < I; ++i) {
            float s = 0;
            for (size_t j = 0; j < O; ++j) s = fmaf(load1(go, t, ob + j), load1(w, t, j * I + i), s);
            store1(gi, t, rb + i, s + (acc_in ? load1(gi, t, rb + i) : 0));
        }
    }
#pragma omp parallel for schedule(static)
    for (int64_t index = 0; index < (int64_t)(O * I); ++index) {
        const size_t z = (size_t)index, j = z / I, i = z % I;
        float s = 0;
        for (size_t r = 0; r < rows; ++r) s = fmaf(load1(go, t, r * O + j), load1(x, t, r * I + i), s);
        store1(gw, t, z, s + (acc_w ? load1(gw, t, z) : 0));
    }
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < (int64_t)O; ++j) {
        float s = 0;
        for (size_t r = 0; r < rows; ++r) s += load1(go, t, r * O + (size_t)j);
        store1(gb, t, (size_t)j, s + (acc_b ? load1(gb, t, (size_t)j) : 0));
    }
}

/* src/ops/cpu/linear_cpu.cpp:205-273: per output, eight FMA lanes over the input
 * dimension, lanes summed 0..7, scalar FMA tail, bias added last; rows > 1 run
 * serially on one thread (lines 271-273). Outputs past the last multiple of
 * eight start from the bias and use a plain FMA chain (lines 259-263). */
void cg_linear_forward_cpu(void* y, const void* x, const void* w, const void* b, size_t rows, size_t I, size_t O,
                           int t) {
    const size_t vec_out = O / 8 * 8;
    for (size_t r = 0; r < rows; ++r) {
        const size_t rb = r * I, ob = r * O;
        for (size_t o = 0; o < vec_out; ++o) {
            float lanes[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            size_t i = 0;
            for (; i + 7 < I; i += 8)
                for (int z = 0; z < 8; ++z) lanes[z] = fmaf(load1(x, t, rb + i + z), load1(w, t, o * I + i + z), lanes[z]);
            float s = 0;
            for (int z = 0; z < 8; ++z) s += lanes[z];
            for (; i < I; ++i) s = fmaf(load1(x, t, rb + i), load1(w, t, o * I + i), s);
            if (b) s += load1(b, t, o);
            store1(y, t, ob + o, s);
        }
        for (size_t o = vec_out; o < O; ++o) {
            float s = b ? load1(b, t, o) : 0;
            for (size_t i = 0; i < I; ++i) s = fmaf(load1(x, t, rb + i), load1(w, t, o * I + i), s);
            store1(y, t, ob + o, s);
        }
    }
}

/* ---------------------------------------------------------------- Embedding */

/* src/ops/cpu/backward/embedding_backward_cpu.cpp:89-114: token order, one
 * rounding to the storage dtype per add; ids >= vocab skipped when checked. */
void cg_embedding_backward_cpu(void* gw, const void* go, const uint32_t* ids, size_t count, size_t vocab, size_t hidden,
                               int bounds_check, int accumulate, int t) {
#pragma omp parallel for schedule(static)
    for (int64_t f = 0; f < (int64_t)hidden; ++f) {
        const size_t feature = (size_t)f;
        if (!accumulate)
            for (size_t row = 0; row < vocab; ++row) store1(gw, t, row * hidden + feature, 0);
        for (size_t token = 0; token < count; ++token) {
            const uint32_t id = ids[token];
            if (bounds_check && id >= vocab) continue;
            const size_t index = (size_t)id * hidden + feature;
            /* The reference reads `old` as 0 when not accumulating (line 109),
             * which drops earlier tokens of a repeated id; its own GPU kernel and
             * test (tests/embedding_test.cu:183-203) sum them, so this follows
             * the sum. */
            const float old = load1(gw, t, index);
            store1(gw, t, index, old + load1(go, t, token * hidden + feature));
        }
    }
}

/* src/ops/cpu/embedding_cpu.cpp: row gather; ids >= vocab give a zero row. */
void cg_embedding_forward_cpu(void* out, const uint32_t* ids, size_t count, const void* w, size_t vocab, size_t hidden,
                              int t) {
    const size_t es = t == CG_F32 ? 4 : 2;
#pragma omp parallel for schedule(static)
    for (int64_t tok = 0; tok < (int64_t)count; ++tok) {
        char* dst = (char*)out + (size_t)tok * hidden * es;
        if (ids[tok] < vocab)
            memcpy(dst, (const char*)w + (size_t)ids[tok] * hidden * es, hidden * es);
        else
            memset(dst, 0, hidden * es);
    }
}

/* ------------------------------------------------------------ Cross entropy */

/* src/ops/cpu/backward/cross_entropy_backward_cpu.cpp:122-148. */
void cg_cross_entropy_forward_backward_cpu(float* loss, void* g, const void* p, const uint32_t* targets, size_t n,
                                           size_t vocab, float scale, int t) {
    float total = 0.0f;
#pragma omp parallel for reduction(+ : total) schedule(static)
    for (int64_t r = 0; r < (int64_t)n; ++r) {
        const size_t base = (size_t)r * vocab;
        float maximum = -INFINITY;
        for (size_t i = 0; i < vocab; ++i) maximum = fmaxf(maximum, load1(p, t, base + i));
        float sum = 0.0f;
        for (size_t i = 0; i < vocab; ++i) sum += expf(load1(p, t, base + i) - maximum);
        const float inv = 1.0f / sum;
        const float factor = scale / (float)n;
        if (targets[r] < vocab) total += logf(sum) + maximum - load1(p, t, base + targets[r]);
        for (size_t i = 0; i < vocab; ++i) {
            float value = expf(load1(p, t, base + i) - maximum) * inv;
            if (targets[r] == i) value -= 1.0f;
            store1(g, t, base + i, value * factor);
        }
    }
    *loss = total / (float)n;
}

/* src/ops/cpu/cross_entropy_cpu.cpp: the loss half of the function above. */
void cg_cross_entropy_forward_cpu(float* loss, const void* p, const uint32_t* targets, size_t n, size_t vocab, int t) {
    float total = 0.0f;
#pragma omp parallel for reduction(+ : total) schedule(static)
    for (int64_t r = 0; r < (int64_t)n; ++r) {
        const size_t base = (size_t)r * vocab;
        float maximum = -INFINITY;
        for (size_t i = 0; i < vocab; ++i) maximum = fmaxf(maximum, load1(p, t, base + i));
        float sum = 0.0f;
        for (size_t i = 0; i < vocab; ++i) sum += expf(load1(p, t, base + i) - maximum);
        if (targets[r] < vocab) total += logf(sum) + maximum - load1(p, t, base + targets[r]);
    }
    *loss = total / (float)n;
}

/* ---------------------------------------------------------------- Attention */

/* src/ops/cpu/attention_cpu.cpp:146-183: per (b, q, h) row, max pass, sum pass,
 * then one pass per output dimension; LSE = log(den) + max. */
void cg_attention_forward_cpu(void* out, float* lse, const void* q, const void* k, const void* v, size_t B, size_t QS,
                              size_t KS, size_t H, size_t KV, size_t D, float attention_scale, int causal, size_t off,
                              int t) {
    const float scale = attention_scale > 0 ? attention_scale : 1.0f / sqrtf((float)D);
#pragma omp parallel for schedule(static)
    for (int64_t task = 0; task < (int64_t)(B * QS * H); ++task) {
        const size_t z = (size_t)task, h = z % H, qi = (z / H) % QS, b = z / (H * QS), kvh = h / (H / KV);
        const size_t qb = ((b * QS + qi) * H + h) * D;
        const size_t last = causal ? (off + qi + 1) : KS;
        float mx = -INFINITY;
        for (size_t kj = 0; kj < last; ++kj) mx = fmaxf(mx, dot8(q, k, t, qb, ((b * KS + kj) * KV + kvh) * D, D) * scale);
        float den = 0;
        for (size_t kj = 0; kj < last; ++kj) den += expf(dot8(q, k, t, qb, ((b * KS + kj) * KV + kvh) * D, D) * scale - mx);
        if (lse) lse[(b * QS + qi) * H + h] = logf(den) + mx;
        for (size_t d = 0; d < D; ++d) {
            float sum = 0;
            for (size_t kj = 0; kj < last; ++kj) {
                const size_t kb = ((b * KS + kj) * KV + kvh) * D;
                sum += expf(dot8(q, k, t, qb, kb, D) * scale - mx) * load1(v, t, kb + d);
            }
            store1(out, t, qb + d, sum / den);
        }
    }
}

/* src/ops/cpu/backward/attention_backward_cpu.cpp:206-280. The softmax row is
 * recomputed for every dK/dV element exactly as there (lines 239-275), which
 * makes the cost cubic in the sequence length. */
void cg_attention_backward_cpu(void* gq, void* gk, void* gv, const void* go, const void* q, const void* k,
                               const void* v, size_t B, size_t QS, size_t KS, size_t H, size_t KV, size_t D,
                               float attention_scale, int causal, size_t off, int acc, int t) {
    const size_t es = t == CG_F32 ? 4 : 2;
    if (!acc) {
        memset(gk, 0, B * KS * KV * D * es);
        memset(gv, 0, B * KS * KV * D * es);
    }
    const float scale = attention_scale > 0 ? attention_scale : 1.0f / sqrtf((float)D);
#pragma omp parallel for schedule(static)
    for (int64_t task = 0; task < (int64_t)(B * QS * H); ++task) {
        const size_t z = (size_t)task, hq = z % H, qi = (z / H) % QS, b = z / (H * QS), kvh = hq / (H / KV);
        const size_t qb = ((b * QS + qi) * H + hq) * D;
        const size_t last = causal ? off + qi + 1 : KS;
        float* p = (float*)malloc(last * sizeof(float));
        float mx = -INFINITY;
        for (size_t kj = 0; kj < last; ++kj) mx = fmaxf(mx, dot8(q, k, t, qb, ((b * KS + kj) * KV + kvh) * D, D) * scale);
        float den = 0;
        for (size_t kj = 0; kj < last; ++kj) {
            p[kj] = expf(dot8(q, k, t, qb, ((b * KS + kj) * KV + kvh) * D, D) * scale - mx);
            den += p[kj];
        }
        for (size_t kj = 0; kj < last; ++kj) p[kj] /= den;
        float delta = 0;
        for (size_t kj = 0; kj < last; ++kj) delta += p[kj] * dot8(go, v, t, qb, ((b * KS + kj) * KV + kvh) * D, D);
        for (size_t d = 0; d < D; ++d) {
            float s = 0;
            for (size_t kj = 0; kj < last; ++kj) {
                const size_t kb = ((b * KS + kj) * KV + kvh) * D;
                const float dp = dot8(go, v, t, qb, kb, D), ds = p[kj] * (dp - delta);
                s += ds * load1(k, t, kb + d);
            }
            store1(gq, t, qb + d, s * scale + (acc ? load1(gq, t, qb + d) : 0));
        }
        free(p);
    }
#pragma omp parallel for schedule(static)
    for (int64_t task = 0; task < (int64_t)(B * KV * KS * D); ++task) {
        const size_t z = (size_t)task, d = z % D, kj = (z / D) % KS, kvh = (z / D / KS) % KV, b = z / (D * KS * KV);
        const size_t kb = ((b * KS + kj) * KV + kvh) * D;
        float dk = 0, dv = 0;
        for (size_t qi = 0; qi < QS; ++qi) {
            const size_t last = causal ? off + qi + 1 : KS;
            if (kj >= last) continue;
            for (size_t hq = kvh * (H / KV); hq < (kvh + 1) * (H / KV); ++hq) {
                const size_t qb = ((b * QS + qi) * H + hq) * D;
                float mx = -INFINITY;
                for (size_t kk = 0; kk < last; ++kk)
                    mx = fmaxf(mx, dot8(q, k, t, qb, ((b * KS + kk) * KV + kvh) * D, D) * scale);
                float den = 0;
                for (size_t kk = 0; kk < last; ++kk)
                    den += expf(dot8(q, k, t, qb, ((b * KS + kk) * KV + kvh) * D, D) * scale - mx);
                const float prob = expf(dot8(q, k, t, qb, kb, D) * scale - mx) / den;
                const float dp = dot8(go, v, t, qb, kb, D);
                float delta = 0;
                for (size_t kk = 0; kk < last; ++kk) {
                    const size_t kkb = ((b * KS + kk) * KV + kvh) * D;
                    const float pp = expf(dot8(q, k, t, qb, kkb, D) * scale - mx) / den;
                    delta += pp * dot8(go, v, t, qb, kkb, D);
                }
                const float ds = prob * (dp - delta);
                dk += ds * load1(q, t, qb + d) * scale;
                dv += prob * load1(go, t, qb + d);
            }
        }
        store1(gk, t, kb + d, dk + (acc ? load1(gk, t, kb + d) : 0));
        store1(gv, t, kb + d, dv + (acc ? load1(gv, t, kb + d) : 0));
    }
}

/* -------------------------------------------------------------------- AdamW */

/* adamw_cpu, src/optim/adamw.cu:193-225, with the host-side bias corrections of
 * adamw_step (lines 413-415: pow in double, cast to float). Parameters and
 * gradients are F32 here as in the reference's CPU branch, which converts other
 * dtypes through copy_to_host first. Returns 0 and changes nothing when a
 * gradient is not finite. */
int cg_adamw_cpu(float* parameter, const float* gradient, float* master, float* m, float* v, size_t n, float lr,
                 float beta1, float beta2, float eps, float wd, float loss_scale, float max_grad_norm,
                 uint64_t next_step) {
    const float bc1 = (float)(1.0 - pow((double)beta1, (double)next_step));
    const float bc2 = (float)(1.0 - pow((double)beta2, (double)next_step));
    double squared_norm = 0.0;
    for (size_t i = 0; i < n; ++i) {
        const float grad = gradient[i] / loss_scale;
        if (!isfinite(grad)) return 0;
        squared_norm += (double)grad * grad;
    }
    const float norm = (float)sqrt(squared_norm);
    const float gradient_scale = norm > max_grad_norm ? max_grad_norm / norm : 1.0f;
    for (size_t i = 0; i < n; ++i) {
        const float grad = gradient[i] / loss_scale * gradient_scale;
        const float first = m[i] = beta1 * m[i] + (1.0f - beta1) * grad;
        const float second = v[i] = beta2 * v[i] + (1.0f - beta2) * grad * grad;
        const float normalized = (first / bc1) / (sqrtf(second / bc2) + eps);
        master[i] = master[i] * (1.0f - lr * wd) - lr * normalized;
        parameter[i] = master[i];
    }
    return 1;
}

/* Same update threaded with OpenMP for the CPU baseline timing only (the
 * reference loop is serial); element results are identical because elements are
 * independent once the norm is known. */
int cg_adamw_cpu_parallel(float* parameter, const float* gradient, float* master, float* m, float* v, size_t n,
                          float lr, float beta1, float beta2, float eps, float wd, float loss_scale,
                          float max_grad_norm, uint64_t next_step) {
    const float bc1 = (float)(1.0 - pow((double)beta1, (double)next_step));
    const float bc2 = (float)(1.0 - pow((double)beta2, (double)next_step));
    double squared_norm = 0.0;
    int bad = 0;
#pragma omp parallel for reduction(+ : squared_norm) reduction(| : bad) schedule(static)
    for (int64_t i = 0; i < (int64_t)n; ++i) {
        const float grad = gradient[i] / loss_scale;
        if (!isfinite(grad)) bad |= 1;
        squared_norm += (double)grad * grad;
    }
    if (bad) return 0;
    const float norm = (float)sqrt(squared_norm);
    const float gradient_scale = norm > max_grad_norm ? max_grad_norm / norm : 1.0f;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; ++i) {
        const float grad = gradient[i] / loss_scale * gradient_scale;
        const float first = m[i] = beta1 * m[i] + (1.0f - beta1) * grad;
        const float second = v[i] = beta2 * v[i] + (1.0f - beta2) * grad * grad;
        const float normalized = (first / bc1) / (sqrtf(second / bc2) + eps);
        master[i] = master[i] * (1.0f - lr * wd) - lr * normalized;
        parameter[i] = master[i];
    }
    return 1;
}

/* Residual add, src/core/generation_cpu.cpp (block composition): out = a + b. */
void cg_add_cpu(void* out, const void* a, const void* b, size_t n, int t) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; ++i) store1(out, t, (size_t)i, load1(a, t, (size_t)i) + load1(b, t, (size_t)i));
}

int cg_max_threads(void) {
#ifdef _OPENMP
    extern int omp_get_max_threads(void);
    return omp_get_max_threads();
#else
    return 1;
#endif
}
