// wkv6 / wkv6_state, chunked formulation on the matrix cores (gfx950, v_mfma_f32_16x16x32_bf16).
//
// Time is cut into chunks of L = 32 steps.  With lam_t[j] = log w_t[j] <= 0 and the in-chunk
// cumulative sums c_t = sum_{z<t} lam_z (c_0 = 0), everything is referred to the chunk's MIDDLE
// (m = 16) so that neither factor of a product can run away unless 16 consecutive decays shrink a
// channel by more than e^-60 (then the chunk is redone step by step, see `exact`):
//     R'_t = r_t e^{c_t - c_m}        K'_s = k_s e^{c_m - c_{s+1}}
//     Rs_t = r_t e^{c_t}     = R'_t e^{c_m}            (reads the state that entered the chunk)
//     Ke_s = k_s e^{c_L - c_{s+1}} = K'_s e^{c_L - c_m} (carries token s to the end of the chunk)
//     A[t,s] = sum_j R'_t[j] K'_s[j]  (s < t),   A[t,t] = sum_j r_t[j] u[j] k_t[j]
//     Y   = Rs S0^T + A V                               S[i][j]: i value channel, j key channel
//     S_L = S0 diag(e^{c_L}) + V^T Ke
// Every product runs on bf16 MFMA with fp32 accumulation; an fp32 operand x is split into
// hi = bf16(x), lo = bf16(x - hi) (v, gy are exact in bf16 and need no split), which keeps ~16
// mantissa bits per operand -- far below the bf16 rounding of the outputs, which is the error
// the original fp32 kernels have.
//
// The state never leaves the accumulator registers: the accumulator layout of a 16x16 tile
// (lane = column, lane group g and register v = row 4g+v) is used AS IS as the B operand of the
// next chunk's Rs S0^T product, because the K slots of an MFMA may be assigned to channels in any
// order as long as the A operand uses the same order; no transpose is ever needed.
//
// This header: constants, the hi/lo bf16 operand format, in-chunk decay factors, helpers of the wave-specialised kernels.
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
// The decay gradient comes from P_t = sum_i dS_t[i,j] S_t[i,j], which the second sweep carries backwards as
// P_t = P_{t+1} + r_t dr'_t - k_t dk'_t.  The two terms come from different kernels, each good to ~4e-6 (hi/lo bf16
// products), so P random-walks: wkv6's per-token gw is 5 % worse than the reference's at T = 4096 and keeps growing, and
// wkv5, which sums G_t over the whole sequence, collects an error ~T^1.5 (1.5 % at T = 4096 against the reference's
// 0.2 %).  Every PCK chunks (wkv5) or 4 PCK chunks (wkv6) the first sweep therefore stores its state S, and the second
// sweep recomputes P from S and its own dS at that boundary, which bounds the walk to 128 / 512 steps: wkv5's gw error is
// then the reference's at any T, wkv6's within 1 % of it.  The workspace holds a slot for every PCK-th chunk in both cases.
constexpr int PCK = 4;
constexpr int PCK_FLOATS = 64 * 64;      // one stored state: [8 state waves of sweep A][64 lanes][8 values]
constexpr float RANGE_LIMIT = 60.0f;
constexpr float LOG2E = 1.44269504088896340736f;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// A state that the forward saves for the one-sweep backward (wkv6_fwd_f.hip -> wkv6_bwd_f.hip; the two-sweep forward
// writes it for the heads it redoes): 64 x 64 values of 24 bits -- fp32 rounded to 16 significant bits, which is what the
// backward's hi/lo bf16 operands keep of it anyway -- in 12 KB instead of 16: first the upper 16 bits of every value
// (8 KB), then the next 8 bits (4 KB), both in the order in which the backward's state waves take them.  Value channel i,
// key channel j: wave j / 16, lane 16 ((i / 4) % 4) + j % 16, element e = 4 (i / 16) + i % 4; a lane's sixteen elements
// are 16 bytes of upper halves for e < 8, 16 bytes for e >= 8 (1 KB further on) and 16 low bytes.
constexpr int SAVED_LO_B = 2 * N * N, SAVED_STATE_B = 3 * N * N;
DEVINL uint32_t saved_round(const float x) { return __float_as_uint(x) + 0x80u; }    // bits 31..8 are what is kept
// x: value channel i, key channels j .. j + 3 (j a multiple of 4: neighbours in a group of sixteen keys lie 16 bytes apart)
DEVINL void saved_put4(char* state, const int i, const int j, const f32x4 x) {
    const int w = j >> 4, lane = 16 * ((i >> 2) & 3) + (j & 15), e = 4 * (i >> 4) + (i & 3);
    char* hi = state + ((2 * w + (e >> 3)) * 64 + lane) * 16 + 2 * (e & 7);
    char* lo = state + SAVED_LO_B + (w * 64 + lane) * 16 + e;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const uint32_t q = saved_round(x[d]);
        *reinterpret_cast<uint16_t*>(hi + 16 * d) = static_cast<uint16_t>(q >> 16);
        *reinterpret_cast<uint8_t*>(lo + 16 * d) = static_cast<uint8_t>(q >> 8);
    }
}

enum { W_HEAD = 0, W_EW = 1, W_RAW = 2 };   // wkv5: fp32 [H,N] (forward: decay eew, backward: ew = log decay);
                                             // wkv6: fp32 ew = -exp(w_raw) [B,T,C];  wkv6_state: raw bf16 w [B,T,C]

struct ArgsC {
    int T, C, H;
    const uint16_t *r, *k, *v, *u, *s0;
    const void* w;
    uint16_t* y;
    // SPLIT kernels only (see below)
    int cross;
    float* y32;
    // when not null: [B*H][ceil(chunks / 2)] saved states (SAVED_STATE_B bytes each), the state entering every even chunk,
    // for the one-sweep backward (wkv6_bwd_f.hip)
    char* saved;
    // when not null: [B*H][8]; a workgroup runs only if one of its eight words is not zero (see ArgsB)
    const int* only_flagged;
};

struct ArgsB {
    int T, C, H;
    const uint16_t *r, *k, *v, *u, *s0, *gy;
    const void* w;
    uint16_t *gr, *gk, *gv, *gw, *gu, *gs;
    float* rdr;                   // workspace [B,T,C] fp32
    // SPLIT kernels only (see below)
    int cross;
    float *gr32, *gk32, *gv32, *gw32, *gu32;
    // when not null: [B*H][8]; a workgroup runs only if one of its eight words is not zero (the (batch, head) pairs that
    // the one-sweep backward has handed back)
    const int* only_flagged;
    // when not null (sweep B only): out[c] = bf16(sum_b float(in[b][c])), the sum of per-batch-row partials over the batch
    // (torch.sum(gu, 0) of the wrapper), done by the workgroups of batch row 0 before anything else.  `in` must be
    // complete when the kernel starts: sweep B does not write it.
    const uint16_t* sum_in;
    uint16_t* sum_out;
    int sum_B;
};
DEVINL bool skip_unflagged(const int* f, const int bh) {
    if (f == nullptr) return false;
    const int4 x = *reinterpret_cast<const int4*>(f + 8 * bh), y = *reinterpret_cast<const int4*>(f + 8 * bh + 4);
    return (x.x | x.y | x.z | x.w | y.x | y.y | y.z | y.w) == 0;
}

// A head of 128 channels as four heads of 64 (SPLIT = true, wkv5 only).  With the key channels j and the value channels
// i of the head cut into halves J and I, everything the op computes is a sum over blocks of the state S[i in I][j in J]:
//     y_I = sum_J wkv(r_J, k_J, v_I; w_J, u_J)     gv_I = sum_J ...     gr_J, gk_J, gw_J, gu_J = sum_I ...
// and each term is exactly the 64-channel problem.  A launch treats the tensor as 2 H heads of 64: workgroup h takes its
// v, gy (and y, gv) from block h and its r, k, w, u (and gr, gk, gw, gu) from block h ^ cross.  cross = 0 gives the
// diagonal blocks (I = J), cross = 1 the other two, so every output element gets exactly one term from each launch.  The
// first launch writes its terms in fp32 (y32, gr32, ...: [B,T,C] like the tensors, gw32 / gu32 [B,C]); the second
// launch of the forward and of the first sweep reads them back, adds its own and writes the bf16 outputs, while both
// launches of the second sweep write terms that the caller adds.  Either way an output is rounded to bf16 once.

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


// ----------------------------------------------------------------------------------------------------------------------
// Pieces shared by the wave-specialised kernels (forward, both backward sweeps).
constexpr int OS = 40;            // row stride (dwords) of a bf16 [token][channel] plane: 160 B, conflict-free for 16-byte reads
constexpr int FS = 72;            // row stride (dwords) of an fp32 [token][channel] array
constexpr int AS = 24;            // row stride (dwords) of a tile plane [row][32 permuted positions]
constexpr float LN2 = 0.69314718055994530942f;

// The factor that turns G into the raw-decay gradient: gw = lam G with lam = -exp(w_raw) = log(decay).  G comes from the
// P recurrence and carries rounding noise of a few 1e-6 |P| whatever the decay, while its true value is decay * (...).  Once
// the decay is below e^-30 the true gw is under 3e-12 of the other gradients, but lam would amplify the noise without bound
// (w_raw = 15 -> lam = -3e6).  The factor is therefore zero from there on, which is also what the original kernel
// produces, exactly, once its fp32 decay has underflowed.
constexpr float LAM_CUT = -30.0f;
DEVINL float gw_factor(float lam) { return lam < LAM_CUT ? 0.f : lam; }

// A chunk takes the step-by-step path when the mid-point factors of some channel could leave the range that the hi / lo
// bf16 operands are designed for: the decay exponent summed over either half of the chunk beyond RANGE_LIMIT.  Every
// prep wave holds every channel (a lane per channel pair), so each of them takes this decision from the eight partial sums
// by itself and all arrive at the same answer.  other[] = the four partial sums of the half this wave does not prepare.
DEVINL bool chunk_needs_exact_path(const float2 (&own)[4], const float2 (&other)[4]) {
    const float ax = (own[0].x + own[1].x) + (own[2].x + own[3].x), ay = (own[0].y + own[1].y) + (own[2].y + own[3].y);
    const float bx = (other[0].x + other[1].x) + (other[2].x + other[3].x), by = (other[0].y + other[1].y) + (other[2].y + other[3].y);
    const float worst = fminf(fminf(ax, ay), fminf(bx, by));            // exponents are <= 0, in log2 units
    return __ballot(-worst > RANGE_LIMIT * LOG2E) != 0ull;
}

template <int CTRL, int ROW_MASK> DEVINL float dpp_add(float x) {
    return x + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, ROW_MASK, 0xf, true));
}
// sum over lanes 0..31 in lane 31 and over lanes 32..63 in lane 63
DEVINL float half_wave_sum(float x) {
    x = dpp_add<0x118, 0xf>(x);       // row_shr:8
    x = dpp_add<0x114, 0xf>(x);       // row_shr:4
    x = dpp_add<0x112, 0xf>(x);       // row_shr:2
    x = dpp_add<0x111, 0xf>(x);       // row_shr:1   -> lane 15 of every row holds the row sum
    x = dpp_add<0x142, 0xa>(x);       // row_bcast:15 into rows 1 and 3
    return x;
}
// sum over the 16 lanes of a row, valid in lane 15 of the row
DEVINL float row_sum_to_last(float x) {
    x = dpp_add<0x118, 0xf>(x);
    x = dpp_add<0x114, 0xf>(x);
    x = dpp_add<0x112, 0xf>(x);
    x = dpp_add<0x111, 0xf>(x);
    return x;
}
// inclusive suffix sum over the 16 lanes of a row: lane l gets the sum of lanes l..15
DEVINL float row_suffix_sum(float x) {
    x = dpp_add<0x101, 0xf>(x);       // row_shl:1
    x = dpp_add<0x102, 0xf>(x);       // row_shl:2
    x = dpp_add<0x104, 0xf>(x);       // row_shl:4
    x = dpp_add<0x108, 0xf>(x);       // row_shl:8
    return x;
}
DEVINL uint4 one_hot(bool on, int e) {                       // 8 bf16 slots, 1.0 in slot e
    const uint32_t bits = (e & 1) ? 0x3f800000u : 0x00003f80u;
    const int d = e >> 1;
    return make_uint4(on && d == 0 ? bits : 0u, on && d == 1 ? bits : 0u, on && d == 2 ? bits : 0u, on && d == 3 ? bits : 0u);
}
DEVINL bf16x8 op4(const uint4& x) { return __builtin_bit_cast(bf16x8, x); }
// two accumulator tiles (tokens 0..15 and 16..31 down the rows) -> one operand with the tokens along the K slots
DEVINL bf16x8 pack_tokens(const f32x4& z0, const f32x4& z1) {
    return as_op(cvt2(z0[0], z0[1]), cvt2(z0[2], z0[3]), cvt2(z1[0], z1[1]), cvt2(z1[2], z1[3]));
}
// stores at a wave-uniform base plus a 32-bit per-lane byte offset (keeps the address out of the vector registers)
DEVINL void store8(const void* sbase, uint32_t byte_off, const uint2& x) {
    asm volatile("global_store_dwordx2 %0, %1, %2" : : "v"(byte_off), "v"(x), "s"(sbase) : "memory");
}
DEVINL void store16(const void* sbase, uint32_t byte_off, const f32x4& x) {
    asm volatile("global_store_dwordx4 %0, %1, %2" : : "v"(byte_off), "v"(x), "s"(sbase) : "memory");
}
DEVINL void unpack4(const uint2& x, float (&f)[4]) { f[0] = bf_lo(x.x); f[1] = bf_hi(x.x); f[2] = bf_lo(x.y); f[3] = bf_hi(x.y); }

}  // namespace
}  // namespace rwkv
