/*
 * gpuk_oracle.c -- plain-C CPU restatement of the two fused paths, independent of torch.
 *
 * TEST INFRASTRUCTURE ONLY.  Only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load the library built from this file.  The
 * product (the HIP kernels behind the C-ABI) never links or calls it.
 *
 * What it restates: the *torch reference* of the reference repository, with its
 * op-by-op rounding sequence spelled out in scalar arithmetic:
 *   add + RMSNorm + fp8 quant : gpuk/__init__.py:147-173 (without dist.all_reduce)
 *   RMSNorm per head          : test/test_fused_rope_rms.py:8-13
 *   rotation                  : test/test_fused_rope_rms.py:16-34
 *   mRoPE axis selection      : test/test_fused_mrope_rms_set_kv.py:16-24 (interleaved),
 *                               :108-115 (chunked); index form src/impl/rope_rms_impl.h:120-153
 *   KV-cache write            : test/test_fused_mrope_rms_set_kv.py:127-129,
 *                               layout src/impl/rope_rms_impl.h:208-231
 *
 * Rounding sequence (T = bf16 or fp16, "rT" = round-to-nearest-even into T):
 *   res  = rT(f32(x) + f32(r))
 *   var  = f32(sum_i f32(res_i)^2) / f32(H)           (sum accumulated in double here;
 *                                                      torch uses a pairwise fp32 sum --
 *                                                      both are within 1 ulp of exact)
 *   rstd = 1.0f / sqrtf(var + eps)                    (both correctly rounded, as torch CPU)
 *   n1   = rT(f32(res) * rstd)
 *   n2   = rT(f32(gamma) * f32(n1))
 *   amax = max |n2| ; scale = amax / fp8_max (fp32 division); scale = 1 if amax == 0
 *   code = e4m3fn_rne(clamp(f32(n2) / scale, +-fp8_max))        (fp32 division)
 *   rope: t = rT(a*c), u = rT(b*s), o = rT(t -/+ u)   (three roundings per output)
 *   fp8 KV: code = e4m3fn(rT(f32(k) / scale))
 *
 * Pinned by tests/test_oracle_formats.py against torch-CPU library routines (exhaustive
 * e4m3fn table over all bf16 patterns, bf16/fp16 rounding over sampled fp32) and by
 * tests/test_oracle_norm_quant.py and tests/test_oracle_rope.py against oracle/torch_oracle.py
 * on seeded inputs.
 *
 * Deviations from torch semantics, both documented in the header of torch_oracle.py:
 * zero rows give scale 1; a cache of the activation dtype is written unscaled.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define GPUK_DT_BF16 0
#define GPUK_DT_FP16 1

/* ------------------------------------------------------------------ scalar formats */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

static inline float bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

static inline uint16_t f32_to_bf16(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0; /* NaN */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

static inline float fp16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0x1f) return bits_f32(sign | 0x7f800000u | (man << 13));
    if (exp == 0) {
        float v = ldexpf((float)man, -24);
        return sign ? -v : v;
    }
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

static inline uint16_t f32_to_fp16(float f) {
    uint32_t u = f32_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to inf */
    float af = bits_f32(a);
    if (a < 0x38800000u) { /* below 2^-14: subnormal half, step 2^-24 */
        float q = nearbyintf(af * 16777216.0f);
        return (uint16_t)(sign | (uint16_t)q);
    }
    uint32_t lsb = (a >> 13) & 1u;
    a += 0xfffu + lsb;
    return (uint16_t)(sign | (uint16_t)((a - 0x38000000u) >> 13));
}

/* OCP e4m3fn, round-to-nearest-even, torch cast semantics: no saturation, anything
 * that would round past 448 becomes NaN (0x7f). */
static inline uint8_t f32_to_e4m3fn(float f) {
    uint32_t u = f32_bits(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    float a = fabsf(f);
    if (!(a == a)) return (uint8_t)(sign | 0x7f);
    if (a < 0.015625f) { /* below 2^-6: subnormal grid of 2^-9 */
        float q = nearbyintf(a * 512.0f);
        return (uint8_t)(sign | (uint8_t)q);
    }
    if (a >= 480.0f) return (uint8_t)(sign | 0x7f);
    int e;
    float m = frexpf(a, &e);          /* a = m * 2^e, m in [0.5, 1) */
    float q = nearbyintf(m * 16.0f);  /* 8..16 */
    if (q == 16.0f) { q = 8.0f; e += 1; }
    int field = e + 6;                /* (e-1) + bias 7 */
    int code = (field << 3) | ((int)q - 8);
    if (code >= 0x7f) return (uint8_t)(sign | 0x7f);
    return (uint8_t)(sign | (uint8_t)code);
}

static inline float e4m3fn_to_f32(uint8_t c) {
    int sign = c & 0x80;
    int e = (c >> 3) & 0xf;
    int m = c & 7;
    float v;
    if (e == 0xf && m == 7) v = NAN;
    else if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf((float)(8 + m), e - 10);
    return sign ? -v : v;
}

static inline float ld(const uint16_t *p, int64_t i, int dt) {
    return dt == GPUK_DT_BF16 ? bf16_to_f32(p[i]) : fp16_to_f32(p[i]);
}
static inline uint16_t rT(float f, int dt) {
    return dt == GPUK_DT_BF16 ? f32_to_bf16(f) : f32_to_fp16(f);
}
static inline float rTf(float f, int dt) { /* round into T and come back to fp32 */
    uint16_t h = rT(f, dt);
    return dt == GPUK_DT_BF16 ? bf16_to_f32(h) : fp16_to_f32(h);
}

/* ------------------------------------------------------------------ exported scalar probes */

uint16_t gpuk_oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }
uint16_t gpuk_oracle_f32_to_fp16(float f) { return f32_to_fp16(f); }
float gpuk_oracle_fp16_to_f32(uint16_t h) { return fp16_to_f32(h); }
uint8_t gpuk_oracle_f32_to_e4m3fn(float f) { return f32_to_e4m3fn(f); }
float gpuk_oracle_e4m3fn_to_f32(uint8_t c) { return e4m3fn_to_f32(c); }

void gpuk_oracle_e4m3fn_table_bf16(uint8_t *out65536) {
    for (uint32_t i = 0; i < 65536; ++i) out65536[i] = f32_to_e4m3fn(bf16_to_f32((uint16_t)i));
}

/* ------------------------------------------------------------------ add + RMSNorm + quant */

/* quant: 0 none (norm_out is T), 1 dynamic per-token e4m3fn (scale[T] written),
 *        3 static per-tensor e4m3fn (scale[0] read).   Returns 0, or 1 on bad arguments. */
int gpuk_oracle_add_rmsnorm_quant(const uint16_t *x, const uint16_t *residual_in, const uint16_t *gamma,
                                  uint16_t *residual_out, void *norm_out, float *scale,
                                  int64_t tokens, int64_t hidden, float eps, int dtype, int quant,
                                  float fp8_max) {
    if (tokens < 0 || hidden <= 0 || (dtype != GPUK_DT_BF16 && dtype != GPUK_DT_FP16)) return 1;
    if (quant != 0 && quant != 1 && quant != 3) return 1;
#pragma omp parallel
    {
        uint16_t *n2 = (uint16_t *)malloc((size_t)hidden * sizeof(uint16_t));
#pragma omp for schedule(static)
        for (int64_t t = 0; t < tokens; ++t) {
            const uint16_t *xr = x + t * hidden, *rr = residual_in + t * hidden;
            uint16_t *ro = residual_out + t * hidden;
            double acc = 0.0;
            for (int64_t i = 0; i < hidden; ++i) {
                uint16_t r = rT(ld(xr, i, dtype) + ld(rr, i, dtype), dtype);
                ro[i] = r;
                float rf = ld(ro, i, dtype);
                acc += (double)(rf * rf);
            }
            float var = (float)acc / (float)hidden;
            float rstd = 1.0f / sqrtf(var + eps);
            float amax = 0.0f;
            for (int64_t i = 0; i < hidden; ++i) {
                float n1 = rTf(ld(ro, i, dtype) * rstd, dtype);
                n2[i] = rT(ld(gamma, i, dtype) * n1, dtype);
                float a = fabsf(ld(n2, i, dtype));
                if (a > amax || a != a) amax = a;
            }
            if (quant == 0) {
                memcpy((uint16_t *)norm_out + t * hidden, n2, (size_t)hidden * sizeof(uint16_t));
                continue;
            }
            float s;
            if (quant == 1) {
                s = amax == 0.0f ? 1.0f : amax / fp8_max;
                scale[t] = s;
            } else {
                s = scale[0];
            }
            uint8_t *qo = (uint8_t *)norm_out + t * hidden;
            for (int64_t i = 0; i < hidden; ++i) {
                float q = ld(n2, i, dtype) / s;
                if (q > fp8_max) q = fp8_max;
                if (q < -fp8_max) q = -fp8_max;
                qo[i] = f32_to_e4m3fn(q);
            }
        }
        free(n2);
    }
    return 0;
}

/* ------------------------------------------------------------------ QK-RMSNorm + RoPE (+ KV write) */

/* Position axis feeding rotary frequency `f` (0 <= f < D/2).
 * Interleaved (rope_rms_impl.h:127-138): axis a = f mod 3 is used when a >= 1 and f < section[a]*3.
 * Chunked (rope_rms_impl.h:139-151): the first a with f < section[0]+...+section[a]. */
static inline int mrope_axis(int64_t f, const int64_t *section, int interleaved) {
    if (interleaved) {
        int a = (int)(f % 3);
        return (a >= 1 && f < section[a] * 3) ? a : 0;
    }
    int64_t end = 0;
    for (int a = 0; a < 3; ++a) {
        end += section[a];
        if (f < end) return a;
    }
    return 2;
}

static void norm_rope_head(const uint16_t *in, const uint16_t *w, const uint16_t *cosr, const uint16_t *sinr,
                           uint16_t *out, int64_t D, float eps, int neox, int dt) {
    /* cosr/sinr: D/2 values already selected for this token */
    double acc = 0.0;
    for (int64_t i = 0; i < D; ++i) { float v = ld(in, i, dt); acc += (double)(v * v); }
    float var = (float)acc / (float)D;
    float rstd = 1.0f / sqrtf(var + eps);
    int64_t half = D / 2;
    for (int64_t f = 0; f < half; ++f) {
        int64_t i1 = neox ? f : 2 * f, i2 = neox ? f + half : 2 * f + 1;
        float x1 = rTf(ld(w, i1, dt) * rTf(ld(in, i1, dt) * rstd, dt), dt);
        float x2 = rTf(ld(w, i2, dt) * rTf(ld(in, i2, dt) * rstd, dt), dt);
        float c = ld(cosr, f, dt), s = ld(sinr, f, dt);
        out[i1] = rT(rTf(x1 * c, dt) - rTf(x2 * s, dt), dt);
        out[i2] = rT(rTf(x2 * c, dt) + rTf(x1 * s, dt), dt);
    }
}

/*
 * One entry point for all variants.
 *   positions: element (axis a, token t) at positions[a*ps_axis + t*ps_token]; n_axes is 1 (RoPE) or 3 (mRoPE).
 *   set_kv == 0: q and k heads are rewritten in place in qkv, V untouched.
 *   set_kv == 1: qkv is read only; q -> q_out[t,h,:], k -> k_cache[kv_loc[t],h,:], v -> v_cache[kv_loc[t],h,:].
 *   kv_fp8 == 0: caches hold T, written unscaled.  kv_fp8 == 1: caches hold e4m3fn codes of rT(x/scale).
 */
int gpuk_oracle_rope_rms(uint16_t *qkv, const uint16_t *qw, const uint16_t *kw, const uint16_t *cos_sin,
                         const int64_t *positions, int64_t ps_axis, int64_t ps_token, int n_axes,
                         int64_t T, int64_t Hq, int64_t Hk, int64_t Hv, int64_t D,
                         int neox, const int64_t *section, int interleaved, float eps, int dtype,
                         int set_kv, uint16_t *q_out, void *k_cache, void *v_cache, const int64_t *kv_loc,
                         float k_scale, float v_scale, int kv_fp8) {
    if (D <= 0 || (D & 1) || (n_axes != 1 && n_axes != 3)) return 1;
    if (dtype != GPUK_DT_BF16 && dtype != GPUK_DT_FP16) return 1;
    int64_t half = D / 2, H = Hq + Hk + Hv;
    if (n_axes == 3 && section[0] + section[1] + section[2] != half) return 1;
#pragma omp parallel
    {
        uint16_t *cs = (uint16_t *)malloc((size_t)D * sizeof(uint16_t));
        uint16_t *tmp = (uint16_t *)malloc((size_t)D * sizeof(uint16_t));
#pragma omp for schedule(static)
        for (int64_t t = 0; t < T; ++t) {
            for (int64_t f = 0; f < half; ++f) {
                int a = n_axes == 3 ? mrope_axis(f, section, interleaved) : 0;
                int64_t p = positions[a * ps_axis + t * ps_token];
                cs[f] = cos_sin[p * D + f];
                cs[half + f] = cos_sin[p * D + half + f];
            }
            uint16_t *tok = qkv + t * H * D;
            for (int64_t h = 0; h < Hq + Hk; ++h) {
                const uint16_t *w = h < Hq ? qw : kw;
                norm_rope_head(tok + h * D, w, cs, cs + half, tmp, D, eps, neox, dtype);
                if (!set_kv) {
                    memcpy(tok + h * D, tmp, (size_t)D * 2);
                } else if (h < Hq) {
                    memcpy(q_out + (t * Hq + h) * D, tmp, (size_t)D * 2);
                } else {
                    int64_t off = (kv_loc[t] * Hk + (h - Hq)) * D;
                    if (!kv_fp8) {
                        memcpy((uint16_t *)k_cache + off, tmp, (size_t)D * 2);
                    } else {
                        for (int64_t i = 0; i < D; ++i)
                            ((uint8_t *)k_cache)[off + i] = f32_to_e4m3fn(rTf(ld(tmp, i, dtype) / k_scale, dtype));
                    }
                }
            }
            if (set_kv) {
                for (int64_t h = 0; h < Hv; ++h) {
                    const uint16_t *v = tok + (Hq + Hk + h) * D;
                    int64_t off = (kv_loc[t] * Hv + h) * D;
                    if (!kv_fp8) {
                        memcpy((uint16_t *)v_cache + off, v, (size_t)D * 2);
                    } else {
                        for (int64_t i = 0; i < D; ++i)
                            ((uint8_t *)v_cache)[off + i] = f32_to_e4m3fn(rTf(ld(v, i, dtype) / v_scale, dtype));
                    }
                }
            }
        }
        free(cs);
        free(tmp);
    }
    return 0;
}

/* Two token streams with their own weights and per-token cos/sin rows, outputs concatenated
 * along the token axis (test/test_fused_rope_rms_2way.py:37-81).
 * q{0,1}: [B, T{0,1}, Hq, D]; k likewise with Hk; cos_sin{0,1}: [T{0,1}, D];
 * out_q: [B, T0+T1, Hq, D]; out_k: [B, T0+T1, Hk, D].  neox = !is_interleaved. */
int gpuk_oracle_rope_rms_2way(const uint16_t *q0, const uint16_t *k0, const uint16_t *q1, const uint16_t *k1,
                              const uint16_t *wq0, const uint16_t *wk0, const uint16_t *wq1, const uint16_t *wk1,
                              const uint16_t *cos_sin0, const uint16_t *cos_sin1,
                              int64_t B, int64_t T0, int64_t T1, int64_t Hq, int64_t Hk, int64_t D,
                              int is_interleaved, float eps, int dtype, uint16_t *out_q, uint16_t *out_k) {
    if (D <= 0 || (D & 1)) return 1;
    int neox = !is_interleaved;
    int64_t half = D / 2, TT = T0 + T1;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t t = 0; t < TT; ++t) {
            int s1 = t >= T0;
            int64_t tl = s1 ? t - T0 : t, Ts = s1 ? T1 : T0;
            const uint16_t *q = (s1 ? q1 : q0) + (b * Ts + tl) * Hq * D;
            const uint16_t *k = (s1 ? k1 : k0) + (b * Ts + tl) * Hk * D;
            const uint16_t *cs = (s1 ? cos_sin1 : cos_sin0) + tl * D;
            for (int64_t h = 0; h < Hq; ++h)
                norm_rope_head(q + h * D, s1 ? wq1 : wq0, cs, cs + half, out_q + ((b * TT + t) * Hq + h) * D, D, eps, neox, dtype);
            for (int64_t h = 0; h < Hk; ++h)
                norm_rope_head(k + h * D, s1 ? wk1 : wk0, cs, cs + half, out_k + ((b * TT + t) * Hk + h) * D, D, eps, neox, dtype);
        }
    }
    return 0;
}

/* Model of the device's reciprocal-based quotient (one multiply, two fused multiply-adds with
 * rcp = RN(1/b), then the device's fix-up step, which restores the sign and hands zero, infinite and NaN
 * numerators the result a division gives them) against the IEEE quotient a/b, for finite b > 0: returns how many of the n pairs differ.  Lets the CPU
 * tests show that the shortcut the HIP kernels take is exact on the operand ranges they guard. */
int64_t gpuk_oracle_count_div_rcp_mismatch(const float *a, const float *b, int64_t n) {
    int64_t bad = 0;
    for (int64_t i = 0; i < n; ++i) {
        float rcp = 1.0f / b[i];
        float q = a[i] * rcp;
        float e = fmaf(-q, b[i], a[i]);
        float q1 = fmaf(e, rcp, q);
        if (a[i] != a[i] || isinf(a[i]) || a[i] == 0.0f) q1 = a[i];  /* NaN, +-inf, +-0 pass through (b > 0) */
        else q1 = copysignf(q1, a[i]);
        float want = a[i] / b[i];
        if (f32_bits(q1) != f32_bits(want) && !(q1 != q1 && want != want)) ++bad;
    }
    return bad;
}

/* Models of the short square-root and reciprocal sequences of the HIP kernels, checked here against the C library
 * over every mantissa.  The device starts from v_sqrt_f32 / v_rcp_f32, which are documented to 1 ULP; the models
 * start from the correctly rounded value moved by `first_guess_ulp` in {-1, 0, +1} ULPs, i.e. from every value the
 * instruction may return, and must reach the correctly rounded result from each.
 *
 * Square root (the sequence LLVM emits for an fp32 sqrt on operands that need no rescaling): with s the first
 * guess, take s-1ulp if v - (s-1ulp)*s <= 0, else s+1ulp if v - (s+1ulp)*s > 0, else s.
 * Returns the number of v = bits first_bits .. first_bits + n - 1 whose result differs from sqrtf(v). */
static inline float next_ulp(float f, int k) { return bits_f32(f32_bits(f) + (uint32_t)k); }

int64_t gpuk_oracle_count_short_sqrt_mismatch(uint32_t first_bits, int64_t n, int first_guess_ulp) {
    int64_t bad = 0;
    for (int64_t i = 0; i < n; ++i) {
        const float v = bits_f32(first_bits + (uint32_t)i);
        const float want = sqrtf(v);
        float s = next_ulp(want, first_guess_ulp);
        const float dn = next_ulp(s, -1), up = next_ulp(s, 1);
        const float r_dn = fmaf(-dn, s, v), r_up = fmaf(-up, s, v);
        if (r_dn <= 0.0f) s = dn;
        else if (r_up > 0.0f) s = up;
        if (f32_bits(s) != f32_bits(want)) ++bad;
    }
    return bad;
}

/* Reciprocal: y the first guess; one Newton step y += y*(1 - s*y); then the quotient correction of 1/s with that
 * reciprocal: q = y, q += y*(1 - s*q).  Returns the number of s whose result differs from 1.0f / s. */
int64_t gpuk_oracle_count_short_rcp_mismatch(uint32_t first_bits, int64_t n, int first_guess_ulp) {
    int64_t bad = 0;
    for (int64_t i = 0; i < n; ++i) {
        const float s = bits_f32(first_bits + (uint32_t)i);
        const float want = 1.0f / s;
        float y = next_ulp(want, first_guess_ulp);
        y = fmaf(fmaf(-s, y, 1.0f), y, y);
        const float q = fmaf(fmaf(-s, y, 1.0f), y, y);
        if (f32_bits(q) != f32_bits(want)) ++bad;
    }
    return bad;
}
