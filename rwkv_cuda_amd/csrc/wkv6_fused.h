// Helpers shared by the one-sweep wkv6 kernels (wkv6_fwd_f.hip, wkv6_bwd_f.hip): explicit LDS byte addressing, MFMA
// operand reads from [token][channel] planes, scans inside a 16-lane row.
#pragma once
#include "wkv6_chunk.h"

namespace rwkv {
namespace {

typedef uint32_t lds_t;            // a byte address in the workgroup's LDS
// LDS is addressed with explicit byte addresses: a few per-lane bases (made opaque to the optimiser once per iteration,
// so that it does not keep dozens of base + constant sums in registers across the loop), a wave-uniform part that
// changes with the chunk (slot, tile set, X / Z parity) and a constant that goes into the instruction.
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
template <class T> DEVINL T lds_ld(const lds_t a) { return *(const __attribute__((address_space(3))) T*)(a); }
template <class T> DEVINL void lds_st(const lds_t a, const T v) { *(__attribute__((address_space(3))) T*)(a) = v; }
DEVINL lds_t lds_of(const void* p) { return static_cast<lds_t>(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) char*)p)); }
DEVINL void opaque(lds_t& x) { asm volatile("" : "+v"(x)); }
// a wave-uniform base (a slot, a tile) behind an empty asm: left to itself the compiler merges "(c % 3) * size" of two
// chunks into one induction variable plus constants, some of them negative, and a negative constant cannot ride in the
// offset field of an LDS instruction: every such read then costs an add
DEVINL lds_t uniform_base(lds_t x) { x = __builtin_amdgcn_readfirstlane(x); asm volatile("" : "+s"(x)); return x; }
typedef short v4s __attribute__((ext_vector_type(4)));
typedef v4s __attribute__((address_space(3))) * lds_v4s_ptr;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Operand with the rows of an LDS matrix along K: slot (g, e) <-> row row0 + e (e = 0..7), lane l16 <-> column col + l16.
// a = address of element [row0 + (l16 >> 2)][col + 4 (l16 & 3)] of a bf16 matrix with rows of `row_bytes`; row0 = 8 g for
// a 32-row contraction.
DEVINL bf16x8 ld_tr(const lds_t a, const lds_t row_bytes) {
    const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_ptr)(a));
    const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_ptr)(a + 4 * row_bytes));
    const u32x2 x = __builtin_bit_cast(u32x2, lo), y = __builtin_bit_cast(u32x2, hi);
    return as_op(x[0], x[1], y[0], y[1]);
}
// Operand with channels along K in accumulator order: slot (g, e) <-> channel 32 ks + 16 (e >> 2) + 4 g + (e & 3).
// a = address of channel 32 ks + 4 g of a [token] row of a bf16 plane.
DEVINL bf16x8 ld_acc(const lds_t a) {
    const u32x2 x = lds_ld<u32x2>(a), y = lds_ld<u32x2>(a + 32);
    return as_op(x[0], x[1], y[0], y[1]);
}
DEVINL bf16x8 ld_op(const lds_t a) { return __builtin_bit_cast(bf16x8, lds_ld<u32x4>(a)); }
// inclusive prefix sum over the 16 lanes of a row: lane l gets the sum of lanes 0..l
DEVINL float row_prefix_sum(float x) {
    x = dpp_add<0x111, 0xf>(x);       // row_shr:1
    x = dpp_add<0x112, 0xf>(x);
    x = dpp_add<0x114, 0xf>(x);
    x = dpp_add<0x118, 0xf>(x);
    return x;
}
// value of the next lane of the row (lane 15 gets 0)
DEVINL float row_next(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x101, 0xf, 0xf, true));
}
// hilo2 with the pair of hi parts behind an empty asm (otherwise the compiler converts the first element once more by
// itself to get its rounded value back: one more instruction per pair)
DEVINL HL hilo2k(float a, float b) {
    HL r;
    r.h = cvt2(a, b);
    asm("" : "+v"(r.h));
    r.l = cvt2(a - __uint_as_float(r.h << 16), b - __uint_as_float(r.h & 0xffff0000u));
    return r;
}
DEVINL void split16(const f32x4 (&x)[4], const float s, bf16x8 (&h)[2], bf16x8 (&l)[2]) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        const HL a = hilo2k(x[2 * ks][0] * s, x[2 * ks][1] * s), b = hilo2k(x[2 * ks][2] * s, x[2 * ks][3] * s);
        const HL c = hilo2k(x[2 * ks + 1][0] * s, x[2 * ks + 1][1] * s), d = hilo2k(x[2 * ks + 1][2] * s, x[2 * ks + 1][3] * s);
        h[ks] = as_op(a.h, b.h, c.h, d.h);
        l[ks] = as_op(a.l, b.l, c.l, d.l);
    }
}

// A meeting point for some of the waves of a workgroup (the hardware barrier takes all of them): each wave adds one to a
// counter in LDS when its part of a staging area is written, and reads the area only when the counter says that all have.
// LDS serves the requests of a wave in the order of issue, so whoever sees the count sees the data written before it.
// The counter only grows: the k-th meeting of m waves is complete at k m.  The poll is bounded, so that a mistake in the
// counting ends as a wrong result flagged to the caller and not as a hung GPU.
DEVINL void meet_signal(uint32_t* cnt, const int lane) {
    // (the add is written out: the compiler's own lowering of an atomic counts the active lanes first, five vector
    //  instructions for a wave in which one lane is active by construction; nothing is returned, so no wait depends on it)
    asm volatile("" ::: "memory");
    if (lane == 0) asm volatile("ds_add_u32 %0, %1" : : "v"(lds_of(cnt)), "v"(1u) : "memory");
}
DEVINL bool meet_wait(uint32_t* cnt, const uint32_t target) {
    bool ok = true;
    int polls = 0;
    while (__hip_atomic_load(cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < target) {
        if (++polls > (1 << 16)) { ok = false; break; }
        __builtin_amdgcn_s_sleep(1);
    }
    asm volatile("" ::: "memory");
    return ok;
}

}  // namespace
}  // namespace rwkv
