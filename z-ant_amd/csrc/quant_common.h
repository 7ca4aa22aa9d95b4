// Device helpers shared by the int8 kernels: the single requantisation sequence and the fused
// Dequantize -> activation -> Quantize step.
#pragma once
#include <cmath>

#include "common.h"

// round-half-to-even (v_rndne_f32), add the zero point as a float (exact), saturate, convert.
__device__ __forceinline__ uint8_t sat_u8_rne(float v, uint8_t zp) {
    float r = __builtin_rintf(v) + float(zp);
    r = __builtin_fmaxf(r, 0.0f);  // NaN -> 0
    r = __builtin_fminf(r, 255.0f);
    return uint8_t(r);
}

// The same for finite inputs (an int32 accumulator times a finite multiplier), as a byte in the low bits of a dword:
// v_cvt_pk_u8_f32 converts with saturation to [0, 255], which replaces the clamp and the conversion.  The value is
// already integral after rint + zero point, so the conversion's own rounding never acts.
__device__ __forceinline__ uint32_t sat_u8_rne_finite(float v, float zp_f) {
    return __builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(v) + zp_f, 0u, 0u);
}

struct QAct {
    int act;            // zant_act
    float alpha;        // LeakyReLU slope
    float in_scale;     // scale / zero point of the tensor the activation reads
    int in_zp;
    float out_scale;    // scale / zero point of the tensor it writes
    uint8_t out_zp;
};

// Quantisation parameters of one QLinearConv as its kernels take them.
struct QConvArgs {
    float x_scale, y_scale;
    int x_zp;
    uint8_t y_zp;
    int n_wscale;       // 1 or K
    int has_act;
    QAct act;
};

__device__ __forceinline__ float act_f32(float v, int act, float alpha) {
    switch (act) {
    case ZANT_ACT_RELU: return v > 0.0f ? v : 0.0f;
    case ZANT_ACT_LEAKY: return v <= 0.0f ? alpha * v : v;
    case ZANT_ACT_RELU6: return __builtin_fminf(__builtin_fmaxf(v, 0.0f), 6.0f);
    default: return v;
    }
}

// q -> sat_u8(rne(act((q - in_zp) * in_scale) / out_scale) + out_zp)
__device__ __forceinline__ uint8_t qact_apply(uint8_t q, const QAct &a) {
    const float v = act_f32(float(int(q) - a.in_zp) * a.in_scale, a.act, a.alpha);
    return sat_u8_rne(v / a.out_scale, a.out_zp);
}

// p / d for 0 <= p < 2^20 and d > 0, with inv = 1.0f / d: the float quotient is off by at most one, which the
// remainder corrects.  Far fewer instructions than the general 32-bit division sequence.
__device__ __forceinline__ int small_div(int p, int d, float inv) {
    int q = int(float(p) * inv);
    const int r = p - q * d;
    q += r >= d ? 1 : 0;
    q -= r < 0 ? 1 : 0;
    return q;
}

// s / y, correctly rounded.  The general f32 division scales its operands against overflow and underflow of the
// intermediate terms, then runs reciprocal refinement and two residual corrections.  When the caller knows that no scaling
// can be needed (|s| and y within 2^+-40), the refined reciprocal r is the same for every element and the rest is five
// instructions with the same correctly rounded result.
__device__ __forceinline__ float div_by(float s, float y, float r, int fast) {
    if (!fast) return s / y;
    const float q0 = s * r;
    const float e0 = __builtin_fmaf(-y, q0, s);
    const float q1 = __builtin_fmaf(e0, r, q0);
    const float e1 = __builtin_fmaf(-y, q1, s);
    return __builtin_fmaf(e1, r, q1);
}

// Host side of div_by: whether the unscaled sequence applies to sums of two dequantised bytes divided by y_scale
// (|sum| <= 256 * (a_scale + b_scale); all scales far inside the range where f32 division needs no operand scaling), and
// the refined reciprocal it takes (a correctly rounded 1 / y as the seed, one Newton step as in the hardware sequence).
static inline bool zant_fast_div_ok(float a_scale, float b_scale, float y_scale) {
    auto tame = [](float v) { return v > 1e-9f && v < 1e9f; };
    return tame(a_scale) && tame(b_scale) && tame(y_scale);
}
static inline float zant_refined_rcp(float y) {
    const volatile float r0 = 1.0f / y;
    return std::fmaf(std::fmaf(-y, r0, 1.0f), r0, r0);
}

// Requantisation followed by a 256-entry byte table that sits at a 256-byte aligned LDS address: the saturating
// conversion writes its byte into the low byte of `table` (its third operand), which makes the result the entry's
// address -- no separate address addition per value.
__device__ __forceinline__ unsigned lds_address(const void *p) {
    return unsigned(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void *) const_cast<void *>(p)));
}
__device__ __forceinline__ uint32_t requant_lookup(float v, float zp_f, unsigned table) {
    const unsigned addr = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(v) + zp_f, 0u, table);
    return *reinterpret_cast<const __attribute__((address_space(3))) uint8_t *>(addr);
}

typedef int zq_i32x4 __attribute__((ext_vector_type(4)));
typedef int zq_i32x16 __attribute__((ext_vector_type(16)));

// LDS reads the compiler does not see, so that it neither serialises them with waits of its own nor reorders them:
// the kernel issues a batch (the nine taps of a position tile, the sixteen table lookups of a requantisation), keeps
// computing, and waits with a counted s_waitcnt that hands the values to their users.  LDS operations complete in
// order; operations the compiler issues in between only make a counted wait stricter.
__device__ __forceinline__ void qb_read128(zq_i32x4 &v, unsigned addr, int imm) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(imm));
}
__device__ __forceinline__ void qb_ready(zq_i32x4 &b, int pending) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(b) : "i"(pending));
}
__device__ __forceinline__ uint32_t qb_read_u8(unsigned addr) {
    uint32_t v;
    asm volatile("ds_read_u8 %0, %1" : "=v"(v) : "v"(addr));
    return v;
}
__device__ __forceinline__ void qb_ready8(uint32_t *v) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]));
}
// Requantises the accumulator values [V0, V0 + 8 * G) of one MFMA tile and looks their bytes up in the activation
// table at `table` (256-byte aligned): all lookups of the batch are issued before the one wait.  d[g] receives the four
// bytes of accumulator registers 4g .. 4g + 3.
template <int G>
__device__ __forceinline__ void qb_requant_lookup(const zq_i32x16 &acc, const float (&mv)[16], float zp_f, unsigned table,
                                                  uint32_t (&d)[4]) {
    uint32_t b[16];
#pragma unroll
    for (int v = 0; v < 4 * G; ++v)
        b[v] = qb_read_u8(__builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(float(acc[v]) * mv[v]) + zp_f, 0u, table));
    qb_ready8(b);
    if (G > 2) qb_ready8(b + 8);
#pragma unroll
    for (int g = 0; g < 4; ++g)
        d[g] = g < G ? (b[4 * g] | (b[4 * g + 1] << 8) | (b[4 * g + 2] << 16) | (b[4 * g + 3] << 24)) : 0u;
}

// The same for NU accumulator tiles at once: every lookup of every tile is issued before the one wait, so the later
// tiles' lookups travel under the first tile's packing.
template <int G, int NU>
__device__ __forceinline__ void qb_requant_lookup_n(const zq_i32x16 (&acc)[NU], const float (&mv)[16], float zp_f, unsigned table,
                                                    uint32_t (&d)[NU][4]) {
    uint32_t b[NU][16];
#pragma unroll
    for (int j = 0; j < NU; ++j)
#pragma unroll
        for (int v = 0; v < 4 * G; ++v)
            b[j][v] = qb_read_u8(__builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(float(acc[j][v]) * mv[v]) + zp_f, 0u, table));
#pragma unroll
    for (int j = 0; j < NU; ++j) {
        qb_ready8(b[j]);
        if (G > 2) qb_ready8(b[j] + 8);
#pragma unroll
        for (int g = 0; g < 4; ++g)
            d[j][g] = g < G ? (b[j][4 * g] | (b[j][4 * g + 1] << 8) | (b[j][4 * g + 2] << 16) | (b[j][4 * g + 3] << 24)) : 0u;
    }
}
