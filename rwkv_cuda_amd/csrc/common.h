// Shared device helpers and host-side argument checks for librwkv_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <utility>

#include "rwkv_hip.h"

#define DEVINL __device__ __forceinline__

namespace rwkv {

// ----------------------------------------------------------------------------- bf16 <-> f32
DEVINL float bf2f(uint16_t x) { return __uint_as_float(static_cast<uint32_t>(x) << 16); }
DEVINL float bf_lo(uint32_t x) { return __uint_as_float(x << 16); }          // element 0 of a packed pair
DEVINL float bf_hi(uint32_t x) { return __uint_as_float(x & 0xffff0000u); }  // element 1 of a packed pair

// fp32 -> bf16, round to nearest even (v_cvt_pk_bf16_f32 on gfx950; NaN stays NaN)
DEVINL uint16_t f2bf(float f) { return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f)); }
DEVINL uint32_t pack_bf2(float lo, float hi) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const bf16x2_t p = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
    return __builtin_bit_cast(uint32_t, p);
}

DEVINL void unpack8(const uint4& q, float (&f)[8]) {
    f[0] = bf_lo(q.x); f[1] = bf_hi(q.x); f[2] = bf_lo(q.y); f[3] = bf_hi(q.y);
    f[4] = bf_lo(q.z); f[5] = bf_hi(q.z); f[6] = bf_lo(q.w); f[7] = bf_hi(q.w);
}
DEVINL uint4 pack8(const float (&f)[8]) {
    uint4 q;
    q.x = pack_bf2(f[0], f[1]); q.y = pack_bf2(f[2], f[3]);
    q.z = pack_bf2(f[4], f[5]); q.w = pack_bf2(f[6], f[7]);
    return q;
}

// ----------------------------------------------------------------------------- row broadcast
// A wave64 is four DPP rows of 16 lanes.  bc<J>(x) is x of lane (row*16 + J): with a vector
// laid out as x_lane = vec[base + (lane & 15)] this gives vec[base + J] in every lane without
// an LDS read or an SGPR.  The fused forms below put the broadcast inside the VALU op
// (v_fmac_f32_dpp / v_mul_f32_dpp row_newbcast), so a broadcast operand costs nothing.
// The DPP source operand must not have been written by the one or two VALU instructions
// just before (gfx9 DPP read-after-VALU-write hazard); callers only feed it values that come
// straight from LDS or that are loop invariant.
template <int J> DEVINL void fmac_bc(float& acc, float row_vec, float s) {   // acc += row_vec[J] * s
    asm("v_fmac_f32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf"
        : "+v"(acc) : "v"(row_vec), "v"(s), "n"(J));
}
template <int J> DEVINL void mul_bc(float& s, float row_vec) {               // s *= row_vec[J]
    asm("v_mul_f32_dpp %0, %1, %0 row_newbcast:%2 row_mask:0xf bank_mask:0xf"
        : "+v"(s) : "v"(row_vec), "n"(J));
}
template <int J> DEVINL float bc(float row_vec) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, row_vec),
                                                                0x150 + J, 0xf, 0xf, true));
}

template <typename F, int... I> DEVINL void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F> DEVINL void static_for(F&& f) {
    static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

// sum over a group of 2^k consecutive lanes (k <= 6); result valid in every lane of the group
template <int WIDTH> DEVINL float group_sum(float x) {
#pragma unroll
    for (int m = WIDTH / 2; m >= 1; m >>= 1) x += __shfl_xor(x, m, 64);
    return x;
}

// sum over the four 16-lane rows of a wave (lanes l, l^16, l^32, l^48); result in all four.
// Two register-swap steps: permlane16_swap exchanges odd rows of one copy with even rows of
// the other, permlane32_swap exchanges the wave halves; neither touches LDS.  The s_nop
// covers the wait states a swap needs after a VALU write of its operands.
DEVINL float allreduce_rows(float x) {
#if RWKV_ROWSUM_SHFL
    x += __shfl_xor(x, 16, 64);
    x += __shfl_xor(x, 32, 64);
    return x;
#else
    float a = x, b = x;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    float s = a + b;
    a = s; b = s;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return a + b;
#endif
}

// The same two swaps applied to distinct values do more work per instruction.  permlane16_swap(a, b) leaves
// a = [a0, b0, a2, b2] and b = [a1, b1, a3, b3] (by row), permlane32_swap(s, t) leaves s = [s0, s1, t0, t1] and
// t = [s2, s3, t2, t3].

// Row sums of four values in three swaps: row 0 of the result holds sum(a), row 1 sum(b), row 2 sum(c), row 3 sum(d).
DEVINL float reduce4_rows(float a, float b, float c, float d) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\tv_permlane16_swap_b32 %2, %3\n\ts_nop 1"
                 : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    float s = a + b, t = c + d;                   // [a01, b01, a23, b23], [c01, d01, c23, d23]
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(s), "+v"(t));
    return s + t;
}

// Row sums of two values, each result in all four rows, in three swaps instead of four.
DEVINL void allreduce2_rows(float& x, float& y) {
    float a = x, b = y;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    float s = a + b;                              // [x01, y01, x23, y23]
    float t = s;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(s), "+v"(t));
    float u = s + t;                              // [X, Y, X, Y]
    float w = u;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(u), "+v"(w));
    x = u; y = w;                                 // [X, X, X, X], [Y, Y, Y, Y]
}

// ----------------------------------------------------------------------------- host checks
extern thread_local int g_last_hip_error;

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// need_align: the kernels that will run use 16-byte loads and stores (those for other head sizes than 64 do not)
inline int check_ptrs(std::initializer_list<const void*> ps, bool need_align = true) {
    for (const void* p : ps) if (p == nullptr) return RWKV_ERR_NULL;
    if (need_align) for (const void* p : ps) if (!aligned16(p)) return RWKV_ERR_ALIGN;
    return RWKV_OK;
}

inline int launch_status() {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { g_last_hip_error = static_cast<int>(e); return RWKV_ERR_LAUNCH; }
    return RWKV_OK;
}

// ----------------------------------------------------------------------------- internal launchers
// wkv6_chunk.hip: chunked MFMA kernels.  wmode: 1 = fp32 ew [B,T,C], 2 = raw bf16 w.
int launch_wkv6_fwd_chunk(hipStream_t st, int wmode, int B, int T, int C, int H, const uint16_t* r,
                          const uint16_t* k, const uint16_t* v, const void* w, const uint16_t* u,
                          const uint16_t* s0, uint16_t* y, char* saved = nullptr, const int* only_flagged = nullptr);
// wkv6_fwd_f.hip: the forward that goes with wkv6_bwd_f.hip (raw bf16 decay, head size 64): y and the state entering
// every second chunk; flags [B*H][8] names the (batch, head) pairs that have to be redone by the kernel above
// NB > 1: the sequences in NB blocks of TB tokens, one workgroup per (batch, head, block): local states, a scan, the outputs
// (blk_state, s32: [B*H*NB][64][64] floats each, blk_decay: [B*H*NB][64]; flags cleared by the caller)
int launch_wkv6_fwd_fused(hipStream_t st, int B, int T, int C, int H, const uint16_t* r, const uint16_t* k, const uint16_t* v,
                          const uint16_t* w, const uint16_t* u, const uint16_t* s0, uint16_t* y, char* saved, int* flags,
                          int NB = 1, int TB = 0, float* blk_state = nullptr, float* blk_decay = nullptr, float* s32 = nullptr,
                          float* decay_out = nullptr);
int launch_wkv6_scan_reverse(hipStream_t st, int BH, int NB, const float* local, const float* logdec, float* out);
int launch_wkv6_bwd_a_chunk(hipStream_t st, int wmode, int B, int T, int C, int H, const uint16_t* r,
                            const uint16_t* k, const uint16_t* v, const void* w, const uint16_t* u,
                            const uint16_t* s0, const uint16_t* gy, uint16_t* gr, uint16_t* gu, float* rdr,
                            const int* only_flagged = nullptr);
int launch_wkv6_bwd_b_chunk(hipStream_t st, int wmode, int B, int T, int C, int H, const uint16_t* r,
                            const uint16_t* k, const uint16_t* v, const void* w, const uint16_t* u,
                            const uint16_t* s0, const uint16_t* gy, uint16_t* gk, uint16_t* gv, uint16_t* gw,
                            uint16_t* gs, const float* rdr, const int* only_flagged = nullptr,
                            const uint16_t* sum_in = nullptr, uint16_t* sum_out = nullptr);
// wkv6_bwd_f.hip: the whole backward in one reverse sweep from the states the forward saved (raw bf16 decay);
// flags [B*H][8] names the (batch, head) pairs that have to be redone by the two sweeps above
int launch_wkv6_bwd_fused(hipStream_t st, int B, int T, int C, int H, const uint16_t* r, const uint16_t* k, const uint16_t* v,
                          const uint16_t* w, const uint16_t* u, const uint16_t* gy, uint16_t* gr, uint16_t* gk, uint16_t* gv,
                          uint16_t* gw, uint16_t* gu, uint16_t* gs, const char* saved, int* flags,
                          int NB = 1, int TB = 0, float* blk_ds = nullptr, float* blk_decay = nullptr, float* ds32 = nullptr,
                          float* gu32 = nullptr, uint16_t* gwp = nullptr, float* gw32 = nullptr);
// gwp != nullptr: wkv5 (w is the raw decay per channel [H][64]; its gradient per batch row goes to gwp [B][C], gw is not written)
// wkv5 with heads of 128 channels as four heads of 64 (see ArgsB in wkv6_chunk.h): one launch of each kernel per value
// of `cross`.  Forward and first sweep: the first launch (cross = 0) leaves fp32 terms, the second adds them to its own
// and writes the bf16 outputs.  Second sweep: both launches leave fp32 terms (its waves have no registers to spare for
// the first launch's terms), which the caller adds.
int launch_wkv5_fwd_split(hipStream_t st, int cross, int B, int T, int C, int H, const uint16_t* r, const uint16_t* k,
                          const uint16_t* v, const float* eew, const uint16_t* u, float* y32, uint16_t* y);
int launch_wkv5_bwd_a_split(hipStream_t st, int cross, int B, int T, int C, int H, const uint16_t* r, const uint16_t* k,
                            const uint16_t* v, const float* ew, const uint16_t* u, const uint16_t* gy, float* gr32, float* gu32,
                            uint16_t* gr, uint16_t* gu, float* rdr);
int launch_wkv5_bwd_b_split(hipStream_t st, int cross, int B, int T, int C, int H, const uint16_t* r, const uint16_t* k,
                            const uint16_t* v, const float* ew, const uint16_t* u, const uint16_t* gy, float* gk32, float* gv32,
                            float* gw32, const float* rdr);

// rwkv7_chunk.hip: chunked rwkv7 kernels (bf16 I/O); s0, sT, dsT, ds0 may be null
int launch7c_fwd(hipStream_t st, int B, int T, int H, const float* s0, const uint16_t* r, const uint16_t* w, const uint16_t* k,
                 const uint16_t* v, const uint16_t* a, const uint16_t* b, uint16_t* y, float* sT, float* s, float* sa);
int launch7c_bwd(hipStream_t st, int B, int T, int H, const uint16_t* r, const uint16_t* w, const uint16_t* k, const uint16_t* v,
                 const uint16_t* a, const uint16_t* b, const uint16_t* dy, const float* dsT, const float* s, const float* sa,
                 float* ds0, uint16_t* dr, uint16_t* dw, uint16_t* dk, uint16_t* dv, uint16_t* da, uint16_t* db);

}  // namespace rwkv
