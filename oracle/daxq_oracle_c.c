/*
 * Bit-level C closed forms of the DAX W8A8 linear arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY: built into oracle/libdaxq_oracle_c.so and loaded by
 * tests/ (and by nothing that ships).  It exists so that the torch-CPU oracle
 * (oracle/daxq_oracle.py, which follows the reference op by op) is pinned by a
 * second, independent statement of what the mathematics fixes: every rounding
 * below is done by hand on the bit patterns, no library conversion is used.
 *
 * Reference lines restated (paths relative to the reference checkout):
 *   dax/quant/nn/dynamic/functional.py:124-135   per-token scale
 *   dax/quant/nn/quantized/functional.py:11-20   leaf quantisers
 *   dax/quant/quantization/observer.py:97-134    per-channel weight scale
 *   dax/quant/nn/dynamic/linear.py:214-228       int8 epilogue
 *
 * Build: gcc -O2 -fno-fast-math -ffp-contract=off -shared -fPIC (see oracle/Makefile).
 * -ffp-contract=off matters: every product and sum below must round on its own.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* bf16 bits -> f32 (exact widening) */
float daxo_bf16_to_f32(uint16_t b) { return u2f((uint32_t)b << 16); }

/* f32 -> bf16 bits, round to nearest even; NaN stays NaN (quiet) */
uint16_t daxo_f32_to_bf16(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

/* per-token scale from the row abs-max (bf16 bits, sign already cleared):
 * s = f32( max( bf16_rne( f32(amax) / qmax ), 2^-23 ) ) */
float daxo_act_scale(uint16_t amax_bits, float qmax) {
    float a = daxo_bf16_to_f32(amax_bits);
    float q = a / qmax;                      /* IEEE binary32 division */
    float s = daxo_bf16_to_f32(daxo_f32_to_bf16(q));
    const float eps = 1.1920928955078125e-07f; /* 2^-23, exact in bf16 */
    if (!(s >= eps)) s = (s != s) ? s : eps;   /* clamp(min=eps) keeps NaN */
    return s;
}

/* round half to even of an f32 to an integral f32, by hand */
static float rne_integral(float v) {
    uint32_t u = f2u(v);
    uint32_t e = (u >> 23) & 0xffu;
    if (e >= 150u) return v;                 /* already integral (or inf/nan) */
    uint32_t sign = u & 0x80000000u;
    float a = u2f(u & 0x7fffffffu);
    if (e < 126u) return u2f(sign);          /* |v| < 0.5 -> +-0 */
    float fl = (float)(int64_t)a;            /* trunc, a >= 0 */
    float diff = a - fl;                     /* exact */
    float r;
    if (diff > 0.5f) r = fl + 1.0f;
    else if (diff < 0.5f) r = fl;
    else r = (((int64_t)fl) & 1) ? fl + 1.0f : fl;
    return u2f(f2u(r) | sign);
}

/* int8 leaf quantiser: clamp(rint(f32(x) * (1.0f / s)), -128, 127) */
int8_t daxo_quant_i8(uint16_t x_bits, float s) {
    float inv = 1.0f / s;
    float v = daxo_bf16_to_f32(x_bits) * inv;
    float r = rne_integral(v);
    if (r < -128.0f) r = -128.0f;
    if (r > 127.0f) r = 127.0f;
    return (int8_t)(int32_t)r;
}

/* f32 -> OCP e4m3fn byte, round to nearest even, no saturation:
 * |v| above the largest value that still rounds to 448 (i.e. > 464) and
 * inf/NaN give NaN (0x7f | sign), which is what an IEEE-style RNE cast into a
 * format without infinities does. */
uint8_t daxo_f32_to_e4m3fn(float v) {
    uint32_t u = f2u(v);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t au = u & 0x7fffffffu;
    if (au > 0x7f800000u) return (uint8_t)(sign | 0x7fu);          /* NaN */
    /* 464 = 0x43e80000: midpoint between 448 and the would-be 480; tie goes to
     * even mantissa (448 = 1.110b x 2^8 has even lsb) so 464 itself -> 448 */
    if (au > 0x43e80000u) return (uint8_t)(sign | 0x7fu);
    int32_t e = (int32_t)(au >> 23) - 127;                         /* unbiased */
    uint32_t man = (au & 0x7fffffu) | (au >= 0x00800000u ? 0x800000u : 0u);
    if (au < 0x00800000u) e = -126;                                /* f32 subnormal */
    /* target: value = m * 2^(E) with 3 fraction bits; min normal exp -6,
     * subnormal quantum 2^-9 */
    int32_t shift;                 /* number of low bits of `man` (24-bit, lsb 2^(e-23)) to drop */
    int32_t qexp;                  /* exponent of result quantum */
    if (e >= -6) qexp = e - 3; else qexp = -9;
    shift = qexp - (e - 23);
    uint32_t q;
    if (shift >= 32) q = 0;
    else if (shift > 25) { q = 0; }  /* far below half a quantum (man < 2^24) */
    else {
        uint32_t keep = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (keep & 1u))) keep++;
        q = keep;
    }
    /* q is the integer multiple of 2^qexp */
    if (q == 0) return sign;
    uint8_t out;
    if (e >= -6) {
        /* q in [8,16]; 16 means carry into next exponent */
        int32_t be = e + 7;
        if (q == 16) { q = 8; be += 1; }
        out = (uint8_t)((be << 3) | (q & 7u));
    } else {
        /* subnormal: q in [0,8]; q == 8 is the min normal (be = 1, m = 0) */
        out = (uint8_t)q;          /* q==8 -> 0x08 which is exactly be=1,m=0 */
    }
    return (uint8_t)(sign | out);
}

/* e4m3fn byte -> f32 (exact) */
float daxo_e4m3fn_to_f32(uint8_t b) {
    uint32_t sign = (uint32_t)(b & 0x80u) << 24;
    uint32_t be = (b >> 3) & 0xfu, m = b & 7u;
    float mag;
    if (be == 0xf && m == 7) return u2f(sign | 0x7fc00000u);
    if (be == 0) mag = ldexpf((float)m, -9);
    else mag = ldexpf((float)(8 + m), (int)be - 7 - 3);
    return u2f(f2u(mag) | sign);
}

/* f32 -> OCP e5m2 byte, round to nearest even; e5m2 is IEEE-like (5 exponent bits, bias 15, 2 mantissa
 * bits, infinities and NaNs): values at or above 61440 (the midpoint between 57344 and 65536) round to
 * infinity. */
uint8_t daxo_f32_to_e5m2(float v) {
    uint32_t u = f2u(v);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t au = u & 0x7fffffffu;
    if (au > 0x7f800000u) return (uint8_t)(sign | 0x7fu);            /* NaN */
    if (au >= 0x47700000u) return (uint8_t)(sign | 0x7cu);           /* >= 61440 -> inf (tie goes to even = 65536 = inf) */
    int32_t e = (int32_t)(au >> 23) - 127;
    uint32_t man = (au & 0x7fffffu) | (au >= 0x00800000u ? 0x800000u : 0u);
    if (au < 0x00800000u) e = -126;
    int32_t qexp = (e >= -14) ? e - 2 : -16;                         /* quantum: 2 fraction bits, subnormal 2^-16 */
    int32_t shift = qexp - (e - 23);
    uint32_t q;
    if (shift > 25) q = 0;
    else {
        uint32_t keep = man >> shift, rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (keep & 1u))) keep++;
        q = keep;
    }
    if (q == 0) return sign;
    uint8_t out;
    if (e >= -14) {
        int32_t be = e + 15;
        if (q == 8) { q = 4; be += 1; }
        out = (uint8_t)((be << 2) | (q & 3u));
    } else {
        out = (uint8_t)q;                                            /* q == 4 is the min normal */
    }
    return (uint8_t)(sign | out);
}

float daxo_e5m2_to_f32(uint8_t b) {
    uint32_t sign = (uint32_t)(b & 0x80u) << 24;
    uint32_t be = (b >> 2) & 0x1fu, m = b & 3u;
    if (be == 0x1f) return u2f(sign | (m ? 0x7fc00000u : 0x7f800000u));
    float mag = be == 0 ? ldexpf((float)m, -16) : ldexpf((float)(4 + m), (int)be - 15 - 2);
    return u2f(f2u(mag) | sign);
}

uint8_t daxo_quant_e5m2(uint16_t x_bits, float s) {
    float v = daxo_bf16_to_f32(x_bits) / s;
    if (v < -57344.0f) v = -57344.0f;
    if (v > 57344.0f) v = 57344.0f;
    return daxo_f32_to_e5m2(v);
}

/* fp8 leaf quantiser: e4m3fn_rne(clamp(f32(x) / s, -448, 448)) */
uint8_t daxo_quant_e4m3(uint16_t x_bits, float s) {
    float v = daxo_bf16_to_f32(x_bits) / s;
    if (v < -448.0f) v = -448.0f;
    if (v > 448.0f) v = 448.0f;
    return daxo_f32_to_e4m3fn(v);
}

/* whole rows -------------------------------------------------------------- */
static uint16_t row_amax_bits(const uint16_t* x, int64_t k) {
    uint16_t m = 0;
    for (int64_t i = 0; i < k; ++i) {
        uint16_t a = x[i] & 0x7fffu;
        if (a > m) m = a;
    }
    return m;
}

void daxo_act_quant_i8(const uint16_t* x, int64_t m, int64_t k, int8_t* q, float* scale) {
    for (int64_t r = 0; r < m; ++r) {
        float s = daxo_act_scale(row_amax_bits(x + r * k, k), 127.0f);
        scale[r] = s;
        for (int64_t i = 0; i < k; ++i) q[r * k + i] = daxo_quant_i8(x[r * k + i], s);
    }
}

void daxo_act_quant_e4m3(const uint16_t* x, int64_t m, int64_t k, uint8_t* q, float* scale) {
    for (int64_t r = 0; r < m; ++r) {
        float s = daxo_act_scale(row_amax_bits(x + r * k, k), 448.0f);
        scale[r] = s;
        for (int64_t i = 0; i < k; ++i) q[r * k + i] = daxo_quant_e4m3(x[r * k + i], s);
    }
}

void daxo_act_quant_e5m2(const uint16_t* x, int64_t m, int64_t k, uint8_t* q, float* scale) {
    for (int64_t r = 0; r < m; ++r) {
        float s = daxo_act_scale(row_amax_bits(x + r * k, k), 57344.0f);
        scale[r] = s;
        for (int64_t i = 0; i < k; ++i) q[r * k + i] = daxo_quant_e5m2(x[r * k + i], s);
    }
}

/* per-channel weight scale: max( max(-min, max) / qmax, 2^-23 ) in f32 */
void daxo_weight_scale(const uint16_t* w, int64_t n, int64_t k, float qmax, float* scale) {
    const float eps = 1.1920928955078125e-07f;
    for (int64_t r = 0; r < n; ++r) {
        float lo = daxo_bf16_to_f32(w[r * k]), hi = lo;
        for (int64_t i = 1; i < k; ++i) {
            float v = daxo_bf16_to_f32(w[r * k + i]);
            if (v < lo) lo = v;
            if (v > hi) hi = v;
        }
        float a = (-lo > hi) ? -lo : hi;
        float s = a / qmax;
        scale[r] = (s > eps) ? s : eps;
    }
}

/* exact integer GEMM, a [m,k] . b[n,k]^T -> int32 [m,n] */
void daxo_gemm_i8(const int8_t* a, const int8_t* b, int64_t m, int64_t n, int64_t k, int32_t* c) {
    for (int64_t i = 0; i < m; ++i)
        for (int64_t j = 0; j < n; ++j) {
            int32_t s = 0;
            for (int64_t t = 0; t < k; ++t) s += (int32_t)a[i * k + t] * (int32_t)b[j * k + t];
            c[i * n + j] = s;
        }
}

/* int8 epilogue: bf16( f32(bf16( f32_rne(acc) * sx * sw )) + f32(bias) ) ; bias may be NULL */
void daxo_epilogue_i8(const int32_t* acc, const float* sx, const float* sw, const uint16_t* bias,
                      int64_t m, int64_t n, uint16_t* out) {
    for (int64_t i = 0; i < m; ++i)
        for (int64_t j = 0; j < n; ++j) {
            float y = (float)acc[i * n + j];          /* RNE by the C standard's default mode */
            y = y * sx[i];
            y = y * sw[j];
            uint16_t o = daxo_f32_to_bf16(y);
            if (bias) o = daxo_f32_to_bf16(daxo_bf16_to_f32(o) + daxo_bf16_to_f32(bias[j]));
            out[i * n + j] = o;
        }
}

/* vector helpers used by the exhaustive tests */
void daxo_f32_to_e4m3fn_vec(const float* v, int64_t n, uint8_t* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = daxo_f32_to_e4m3fn(v[i]);
}
void daxo_f32_to_e5m2_vec(const float* v, int64_t n, uint8_t* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = daxo_f32_to_e5m2(v[i]);
}
void daxo_quant_e5m2_vec(const uint16_t* x_bits, int64_t n, float s, uint8_t* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = daxo_quant_e5m2(x_bits[i], s);
}
void daxo_act_scale_vec(const uint16_t* amax_bits, int64_t n, float qmax, float* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = daxo_act_scale(amax_bits[i], qmax);
}
void daxo_quant_i8_vec(const uint16_t* x_bits, int64_t n, float s, int8_t* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = daxo_quant_i8(x_bits[i], s);
}
void daxo_quant_e4m3_vec(const uint16_t* x_bits, int64_t n, float s, uint8_t* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = daxo_quant_e4m3(x_bits[i], s);
}
