/* Host-side scalar and Q8_0 block codecs on the attention path, bit-exact with
 * src/gguf/quant_scalar.c:40-143 and src/gguf/quant_block.c:160-186,819-833 of the
 * reference.  They are used to build KV caches (quantise on write) and by callers that
 * need the canonical bytes; the kernels decode the same bytes in registers. */
#include "private.h"

#include <math.h>
#include <string.h>

static unsigned int float_bits(float value)
{
    unsigned int bits;
    memcpy(&bits, &value, sizeof(bits));
    return bits;
}

static float bits_float(unsigned int bits)
{
    float value;
    memcpy(&value, &bits, sizeof(value));
    return value;
}

float yvex_quant_bf16_decode(unsigned short bits) { return bits_float((unsigned int)bits << 16); }

/* Round to nearest even; a NaN keeps its upper half with the quiet bit forced. */
unsigned short yvex_quant_bf16_encode(float value)
{
    unsigned int bits = float_bits(value);
    unsigned int round;
    if ((bits & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((bits >> 16) | 0x0040u);
    round = 0x7fffu + ((bits >> 16) & 1u);
    return (unsigned short)((bits + round) >> 16);
}

float yvex_quant_f16_decode(unsigned short bits)
{
    unsigned int sign = ((unsigned int)bits & 0x8000u) << 16;
    unsigned int exponent = ((unsigned int)bits >> 10) & 0x1fu;
    unsigned int mantissa = (unsigned int)bits & 0x03ffu;
    if (exponent == 0x1fu)
        return bits_float(sign | 0x7f800000u | (mantissa << 13) | (mantissa ? 0x00400000u : 0u));
    if (exponent) return bits_float(sign | ((exponent + 112u) << 23) | (mantissa << 13));
    if (!mantissa) return bits_float(sign);
    /* subnormal half: value = mantissa * 2^-24, exact in binary32 */
    return bits_float(sign | float_bits((float)mantissa * 5.9604644775390625e-08f));
}

/* Round to nearest even on the half grid.  Normal range by integer rounding of the
 * mantissa; subnormal range by adding the magic constant whose ulp is the half
 * subnormal step, which makes the FPU perform the same RNE. */
unsigned short yvex_quant_f16_encode(float value)
{
    unsigned int bits = float_bits(value);
    unsigned int sign = (bits >> 16) & 0x8000u;
    unsigned int magnitude = bits & 0x7fffffffu;
    if (magnitude > 0x7f800000u)
        return (unsigned short)(sign | 0x7e00u | ((magnitude >> 13) & 0x01ffu));
    if (magnitude >= 0x47800000u) /* >= 65536, including infinity */
        return (unsigned short)(sign | 0x7c00u);
    if (magnitude >= 0x38800000u) { /* normal half range: 2^-14 .. */
        unsigned int rounded = magnitude - 0x38000000u; /* rebias exponent by 112 */
        unsigned int half = rounded >> 13;
        unsigned int rest = rounded & 0x1fffu;
        if (rest > 0x1000u || (rest == 0x1000u && (half & 1u))) ++half;
        if (half >= 0x7c00u) half = 0x7c00u;
        return (unsigned short)(sign | half);
    }
    if (magnitude < 0x33000000u) return (unsigned short)sign; /* below 2^-25: signed zero */
    {
        /* 0.5f has ulp 2^-24 on [0.5, 1): adding it rounds |value| to a multiple of 2^-24 */
        float shifted = bits_float(magnitude) + 0.5f;
        return (unsigned short)(sign | (float_bits(shifted) - 0x3f000000u));
    }
}

/* src/gguf/quant_block.c:160-186 */
static int q8_0_encode_block(const float *source, unsigned char *encoded)
{
    float maximum = 0.0f, scale, inverse;
    unsigned short half;
    unsigned int index;
    for (index = 0u; index < YVEX_QUANT_Q8_0_ELEMENTS; ++index) {
        float magnitude = fabsf(source[index]);
        if (magnitude > maximum) maximum = magnitude;
    }
    half = yvex_quant_f16_encode(maximum / 127.0f);
    encoded[0] = (unsigned char)(half & 0xffu);
    encoded[1] = (unsigned char)(half >> 8);
    scale = yvex_quant_f16_decode(half);
    if (!isfinite(scale) || scale < 0.0f || (maximum > 0.0f && scale == 0.0f)) return 0;
    inverse = scale != 0.0f ? 1.0f / scale : 0.0f;
    for (index = 0u; index < YVEX_QUANT_Q8_0_ELEMENTS; ++index) {
        float scaled = roundf(source[index] * inverse); /* half away from zero */
        int code = scaled < -127.0f ? -127 : scaled > 127.0f ? 127 : (int)scaled;
        encoded[2u + index] = (unsigned char)(signed char)code;
    }
    return 1;
}

int yvex_rocm_q8_0_encode_row(const float *source, unsigned long long elements,
                              unsigned char *encoded, yvex_error *err)
{
    unsigned long long block;
    if (!source || !encoded || !elements || elements % YVEX_QUANT_Q8_0_ELEMENTS) {
        yvex_error_set(err, YVEX_ERR_INVALID_ARG, "rocm.q8_0.encode",
                       "source, destination and a multiple of 32 elements are required");
        return YVEX_ERR_INVALID_ARG;
    }
    for (block = 0ull; block < elements / YVEX_QUANT_Q8_0_ELEMENTS; ++block)
        if (!q8_0_encode_block(source + block * YVEX_QUANT_Q8_0_ELEMENTS,
                               encoded + block * YVEX_QUANT_Q8_0_BYTES)) {
            yvex_error_set(err, YVEX_ERR_BOUNDS, "rocm.q8_0.encode",
                           "Q8_0 scale is not representable");
            return YVEX_ERR_BOUNDS;
        }
    yvex_error_clear(err);
    return YVEX_OK;
}

/* src/gguf/quant_block.c:819-833 */
int yvex_rocm_q8_0_decode_row(const unsigned char *encoded, unsigned long long elements,
                              float *out, yvex_error *err)
{
    unsigned long long block;
    unsigned int index;
    if (!encoded || !out || !elements || elements % YVEX_QUANT_Q8_0_ELEMENTS) {
        yvex_error_set(err, YVEX_ERR_INVALID_ARG, "rocm.q8_0.decode",
                       "source, destination and a multiple of 32 elements are required");
        return YVEX_ERR_INVALID_ARG;
    }
    for (block = 0ull; block < elements / YVEX_QUANT_Q8_0_ELEMENTS; ++block) {
        const unsigned char *in = encoded + block * YVEX_QUANT_Q8_0_BYTES;
        float scale = yvex_quant_f16_decode((unsigned short)(in[0] | ((unsigned int)in[1] << 8)));
        if (!isfinite(scale) || scale < 0.0f) {
            yvex_error_set(err, YVEX_ERR_FORMAT, "rocm.q8_0.decode",
                           "Q8_0 encoded scale is negative or non-finite");
            return YVEX_ERR_FORMAT;
        }
        for (index = 0u; index < YVEX_QUANT_Q8_0_ELEMENTS; ++index)
            out[block * YVEX_QUANT_Q8_0_ELEMENTS + index] =
                scale * (float)(signed char)in[2u + index];
    }
    yvex_error_clear(err);
    return YVEX_OK;
}
