/*
 * TEST INFRASTRUCTURE ONLY -- see lstm_oracle_impl.h for what this restates
 * and which reference lines each part follows.  Built by oracle/Makefile into
 * oracle/liblstm_oracle.so and loaded (ctypes) by oracle/lstm_oracle.py from
 * tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg only.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* float -> IEEE binary16 -> float, round-to-nearest-even, with subnormals,
 * overflow to inf.  Written out by hand: this gcc has no _Float16 on x86. */
static float round_fp16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint32_t sign = u & 0x80000000u;
    uint32_t a = u & 0x7fffffffu;
    float r;
    if (a >= 0x7f800000u) return f; /* inf / nan */
    if (a >= 0x477ff000u) {         /* >= 65520 rounds to inf */
        a = 0x7f800000u;
    } else if (a < 0x38800000u) { /* below 2^-14: subnormal half, quantum 2^-24 */
        float af;
        memcpy(&af, &a, 4);
        /* adding 0.5f's worth of exponent forces RNE at the 2^-24 quantum */
        const float magic = 0.5f; /* 2^-1: mantissa lsb = 2^-24 */
        af = (af + magic) - magic;
        memcpy(&a, &af, 4);
    } else {
        const uint32_t lsb = (a >> 13) & 1u;
        a += 0x0fffu + lsb;
        a &= ~0x1fffu;
    }
    a |= sign;
    memcpy(&r, &a, 4);
    return r;
}

/* float -> bfloat16 -> float, round-to-nearest-even. */
static float round_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) >= 0x7f800000u) return f;
    const uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    u &= 0xffff0000u;
    float r;
    memcpy(&r, &u, 4);
    return r;
}

static double round_to(double v, int mode) {
    if (mode == 1) return (double)round_fp16((float)v);
    if (mode == 2) return (double)round_bf16((float)v);
    return v;
}

/* exported so the tests can pin the two rounding helpers against numpy/torch */
float oracle_round_fp16(float f) { return round_fp16(f); }
float oracle_round_bf16(float f) { return round_bf16(f); }

#define REAL double
#define SUF f64
#include "lstm_oracle_impl.h"
#undef REAL
#undef SUF

#define REAL float
#define SUF f32
#include "lstm_oracle_impl.h"
#undef REAL
#undef SUF
