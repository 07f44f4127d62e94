/*
 * CPU oracle, part 2 (TEST INFRASTRUCTURE ONLY - never linked into or called by the shipped library):
 * a plain-C restatement of the arithmetic on the routing hot path that does not rely on torch:
 *
 *   oracle_e4m3_from_f32()      IEEE fp32 -> OCP e4m3fn, round-to-nearest-even (the conversion
 *                               deep_ep/utils/math.py:37-38 gets from `.to(torch.float8_e4m3fn)`)
 *   oracle_cast_1x128()         deep_ep/utils/math.py:30-39: per 128 channels, amax clamped at 1e-4,
 *                               payload = e4m3(x * (448 / amax)), scale = amax / 448 (IEEE divisions)
 *   oracle_ordered_sum_bf16()   deep_ep/utils/refs.py:156-174: fp32 running sum in index order on top of
 *                               an initial value, one round-to-nearest-even to bf16
 *
 * The encoder is written from the format definition (1 sign, 4 exponent bits with bias 7, 3 mantissa
 * bits, no infinities, 0x7f = NaN, largest finite 448, smallest subnormal 2^-9) by enumerating the
 * representable magnitudes and picking the nearest, ties to the even code: deliberately a different
 * method from both the library routine and the GPU kernel's bit manipulation.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float e4m3_value(int code /* 0..126 */) {
    const int exp = code >> 3, man = code & 7;
    if (exp == 0) return ldexpf((float)man, -9);             /* subnormal: man * 2^-9 */
    return ldexpf(1.0f + (float)man / 8.0f, exp - 7);
}

uint8_t oracle_e4m3_from_f32(float f) {
    uint32_t bits;
    memcpy(&bits, &f, 4);
    const uint8_t sign = (uint8_t)((bits >> 24) & 0x80);
    const float a = fabsf(f);
    if (!(a == a)) return (uint8_t)(sign | 0x7f);             /* NaN */
    /* 464 is halfway between 448 (code 0x7e) and the first value the format cannot hold (480);
       the tie goes to the even code 0x7e, anything above has no finite neighbour: NaN. */
    if (a > 464.0f) return (uint8_t)(sign | 0x7f);
    int best = 0;
    double best_err = (double)a;                              /* distance to code 0 (value 0) */
    for (int code = 1; code <= 126; ++code) {
        const double err = fabs((double)a - (double)e4m3_value(code));
        if (err < best_err || (err == best_err && (code & 1) == 0)) {
            best = code;
            best_err = err;
        }
    }
    return (uint8_t)(sign | best);
}

static float bf16_to_f32(uint16_t h) {
    uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static uint16_t f32_to_bf16(float f) {
    uint32_t bits;
    memcpy(&bits, &f, 4);
    if (f != f) return 0x7fc0;
    bits += 0x7fffu + ((bits >> 16) & 1u);
    return (uint16_t)(bits >> 16);
}

/* x: bf16 bits [tokens][hidden]; out: e4m3 bytes [tokens][hidden]; scales: [tokens][ceil(hidden/128)] */
void oracle_cast_1x128(const uint16_t* x, int64_t tokens, int64_t hidden, uint8_t* out, float* scales) {
    const int64_t groups = (hidden + 127) / 128;
    for (int64_t t = 0; t < tokens; ++t) {
        for (int64_t g = 0; g < groups; ++g) {
            const int64_t lo = g * 128, hi = lo + 128 < hidden ? lo + 128 : hidden;
            float amax = 0.0f;
            for (int64_t c = lo; c < hi; ++c) {
                const float v = fabsf(bf16_to_f32(x[t * hidden + c]));
                if (v > amax) amax = v;
            }
            if (amax < 1e-4f) amax = 1e-4f;
            const volatile float factor = 448.0f / amax;     /* volatile: keep both divisions in fp32 */
            const volatile float scale = amax / 448.0f;
            scales[t * groups + g] = scale;
            for (int64_t c = lo; c < hi; ++c) {
                const volatile float scaled = bf16_to_f32(x[t * hidden + c]) * factor;
                out[t * hidden + c] = oracle_e4m3_from_f32(scaled);
            }
        }
    }
}

/* rows: bf16 bits [count][hidden]; init: fp32 [hidden] or NULL; out: bf16 bits [hidden] */
void oracle_ordered_sum_bf16(const uint16_t* rows, int64_t count, int64_t hidden, const float* init, uint16_t* out) {
    for (int64_t c = 0; c < hidden; ++c) {
        volatile float acc = init ? init[c] : 0.0f;
        for (int64_t r = 0; r < count; ++r) acc = acc + bf16_to_f32(rows[r * hidden + c]);
        out[c] = f32_to_bf16(acc);
    }
}
