// Shared pieces of the chunked wkv6 kernels (gfx950): constants, the hi/lo bf16 operand format, in-chunk decay factors.
#pragma once
#include "common.h"

namespace rwkv {
namespace {

constexpr int N = 64;
constexpr int L = 32;             // chunk length
constexpr int NW = 8;             // waves per workgroup: two per SIMD (a single wave per SIMD issues VALU ~3x slower)
constexpr int NT = NW * 64;
constexpr int RS = 68;            // row stride (dwords) of [token][channel] operand arrays: 272 B
constexpr int TS = 36;            // row stride (dwords) of [channel][token] hi/lo operand arrays: 144 B
constexpr int VS = 20;            // row stride (dwords) of the bf16 [channel][token] array: 80 B
constexpr int STAGES = 4;         // chunks of input kept in flight
constexpr float RANGE_LIMIT = 60.0f;
constexpr float LOG2E = 1.44269504088896340736f;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

enum { W_EW = 1, W_RAW = 2 };     // wkv6: fp32 ew = -exp(w_raw) [B,T,C];  wkv6_state: raw bf16 w

struct ArgsC {
    int T, C, H;
    const uint16_t *r, *k, *v, *u, *s0;
    const void* w;
    uint16_t* y;
};

struct ArgsB {
    int T, C, H;
    const uint16_t *r, *k, *v, *u, *s0, *gy;
    const void* w;
    uint16_t *gr, *gk, *gv, *gw, *gu, *gs;
    float* rdr;                   // workspace [B,T,C] fp32
};

// Operand format.  An fp32 value x is used as hi = bf16(x), lo = bf16(x - hi).  Along the K axis of an MFMA a lane holds
// 8 slots = 4 consecutive elements e0..e3 as  P = [h0 h1 h2 h3 | l0 l1 l2 l3]  (dwords H01, H23, L01, L23).  With the
// halves exchanged, P~ = [l0 l1 l2 l3 | h0 h1 h2 h3] (a register renaming, no instruction), and Q in the same format,
//     mfma(P, Q) + mfma(P~, Q) = sum_e (h + l)_P (h + l)_Q
// i.e. the full product at ~16 mantissa bits per operand.  An operand that is exact in bf16 (v) is used as
// [v0 v1 v2 v3 | v0 v1 v2 v3], which makes a single mfma(P, .) = sum_e (h + l)_P v.
struct HL { uint32_t h, l; };     // two elements: bf16 pair of the hi parts, bf16 pair of the lo parts
DEVINL uint32_t cvt2(float a, float b) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const bf16x2 p = {static_cast<__bf16>(a), static_cast<__bf16>(b)};
    return __builtin_bit_cast(uint32_t, p);
}
DEVINL HL hilo2(float a, float b) {
    HL r;
    r.h = cvt2(a, b);
    r.l = cvt2(a - __uint_as_float(r.h << 16), b - __uint_as_float(r.h & 0xffff0000u));
    return r;
}
DEVINL bf16x8 as_op(uint32_t a, uint32_t b, uint32_t c, uint32_t d) { return __builtin_bit_cast(bf16x8, make_uint4(a, b, c, d)); }
DEVINL bf16x8 lds_op(const uint32_t* p) { return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p)); }
DEVINL bf16x8 lds_dup(const uint32_t* p) {          // 4 exact bf16 -> [v0..v3 | v0..v3]
    const uint2 x = *reinterpret_cast<const uint2*>(p);
    return as_op(x.x, x.y, x.x, x.y);
}
DEVINL bf16x8 swapped(const bf16x8& a) {
    const uint4 x = __builtin_bit_cast(uint4, a);
    return as_op(x.z, x.w, x.x, x.y);
}
DEVINL f32x4 mfma(bf16x8 a, bf16x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
DEVINL f32x4 mfma_full(bf16x8 a, bf16x8 b, f32x4 c) { return mfma(swapped(a), b, mfma(a, b, c)); }
DEVINL float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// dword position, inside a stored row, of the (H, L) pair of elements (2p, 2p+1): groups of 4 elements are H01 H23 L01 L23
DEVINL int hpos(int p) { return 4 * (p >> 1) + (p & 1); }

DEVINL bf16x8 lds_op_sw(const uint32_t* p) {       // the same cell with its halves exchanged: [l0..l3 | h0..h3]
    const uint2 lo = *reinterpret_cast<const uint2*>(p + 2);
    const uint2 hi = *reinterpret_cast<const uint2*>(p);
    return as_op(lo.x, lo.y, hi.x, hi.y);
}
// full product of two hi/lo cells read from LDS: A (and A with halves exchanged) against B
DEVINL f32x4 mfma_full_lds(const uint32_t* pa, bf16x8 b, f32x4 c) { return mfma(lds_op_sw(pa), b, mfma(lds_op(pa), b, c)); }

// In-chunk exponents, in log2 units, for the two tokens (t0, t0+1) of one channel held by a thread.
// near = sum of lam over the tokens of the same half-chunk that lie between this pair and the middle of the chunk.
//   first half : Ea_t = 2^{-sum_{z=t..15} lam},  Eb_t = 2^{sum_{z=t+1..15} lam}
//   second half: Ea_t = 2^{sum_{z=16..t-1} lam}, Eb_t = 2^{-sum_{z=16..t} lam}
struct Scale { float ea[2], eb[2]; };
DEVINL Scale chunk_scale(bool second_half, float near, float lam0, float lam1) {
    Scale s;
    if (!second_half) {
        const float s1 = lam1 + near, s0 = lam0 + s1;          // suffix sums from t0+1, t0
        s.ea[0] = exp2_fast(-s0); s.ea[1] = exp2_fast(-s1);
        s.eb[0] = exp2_fast(s1);  s.eb[1] = exp2_fast(near);
    } else {
        const float p1 = near + lam0, p2 = p1 + lam1;          // prefix sums up to t0+1, t0+2
        s.ea[0] = exp2_fast(near); s.ea[1] = exp2_fast(p1);
        s.eb[0] = exp2_fast(-p1);  s.eb[1] = exp2_fast(-p2);
    }
    return s;
}

}  // namespace
}  // namespace rwkv
