/* Helpers shared by the oracle's C files (test infrastructure only). */
#ifndef ORACLE_COMMON_H
#define ORACLE_COMMON_H
#include <math.h>
#include <stdint.h>
#include <string.h>

/* Round-to-nearest-even fp32 -> bf16 -> fp32 (value stays in a float). */
static inline float bf16_round(float v)
{
    uint32_t u;
    memcpy(&u, &v, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) { u |= 0x00400000u; u &= 0xffff0000u; }
    else { u += 0x7fffu + ((u >> 16) & 1u); u &= 0xffff0000u; }
    memcpy(&v, &u, 4);
    return v;
}

static inline float silu_f(float v)
{
    /* x / (1 + exp(-x)): J/engine/nn/layer/active/gpu/activeFunction.cu:172-179 */
    return v / (1.0f + (float)exp(-(double)v));
}
#endif
