// wkv6 / wkv6_state forward (gfx950) that keeps the state entering every second chunk for the one-sweep backward
// (wkv6_bwd_f.hip), built like that kernel: wave roles, operands from [token][channel] planes, one barrier per chunk.
//
// Formulas (wkv6_chunk.h for R', K', d1, d2, dec; chunk of L = 32 tokens, factors referred to its middle m = 16):
//     A[t][s] = R'_t . K'_s (s < t),  A[t][t] = sum_j r u k
//     y_t = (S d1) R'_t + sum_{s<=t} A[t][s] v_s              S <- S dec + d2 V^T K'
//
// One workgroup of 16 waves per (batch, head):
//   P  (prep, 8 waves)  channels 8w..8w+7 of r, k, w, v for all 32 tokens of a chunk: lane = 16 * (channel pair) + token.
//                       Writes the bf16 hi / lo planes of R', K' and plain v, the per-channel factors and the diagonal
//                       of A; stores the finished y rows of the chunk three iterations back.
//   S  (state, 4 waves) S[i][j], value channels i = 16w..: lane = i, registers = j.  y, the state update, the saved state.
//   T  (tiles, 3 of 4 waves) the causal tile A of the next chunk, one 16 x 16 quadrant each; the fourth wave moves the
//                       states to be saved from LDS to global memory.
// Pipeline: in iteration `it` the P waves prepare chunk it, the T waves make the tile of chunk it-1, the S waves do the
// products of chunk it-2 and the P waves store the y of chunk it-3.
//
// Global memory is touched in whole 128-byte rows, 16 bytes per lane: the inputs are staged in LDS by whichever prep wave
// loaded them, and y leaves through an LDS tile.
//
// A chunk in which some channel decays by more than e^-60 over either half cannot use the mid-point factors.  Such a
// (batch, head) is flagged in `flags` and the caller reruns it with wkv6_fwd_ws, which has a step-by-step path.
#include "wkv6_fused.h"

namespace rwkv {
namespace {

constexpr int NTQ = 16 * 64;
constexpr int PS = 36;             // bf16 [token][channel] planes: 144 B per row (see wkv6_bwd_f.hip)
constexpr int DEPTH = 4;           // chunks that the prep waves load ahead (a power of two)
constexpr int SS = 68;             // fp32 [value][key] state: 272 B per row

struct alignas(16) SlotQ {
    uint32_t RpH[L][PS], RpL[L][PS], KpH[L][PS], KpL[L][PS], V[L][PS];
    float d1[N], d2[N], dec[N];            // 2^{c_m}, 2^{c_L - c_m}, 2^{c_L}
    float ruk[8][L];                        // sum of r u k over the 8 channels of each prep wave
};
struct alignas(16) TilesQ {
    uint32_t AH[L][AS], AL[L][AS];         // [t][s] bf16 hi / lo
};
struct alignas(16) SmemQ {
    // (the small arrays come first: below 64 KB their addresses are a lane offset plus a constant inside the instruction)
    uint32_t yb[2][L][PS];                  // y of the last two chunks, bf16 [token][channel]
    float sst[N][SS];                       // the state entering an even chunk, on its way to global memory
    uint32_t met[4];                        // [0]: meeting counter of the prep waves
    SlotQ slot[3];
    TilesQ tile[2];
};
constexpr lds_t ROW_B = PS * 4, PLANE_B = L * ROW_B, TROW_B = AS * 4;
constexpr lds_t O_RPH = 0, O_RPL = PLANE_B, O_KPH = 2 * PLANE_B, O_KPL = 3 * PLANE_B, O_V = 4 * PLANE_B;
constexpr lds_t O_D1 = 5 * PLANE_B, O_D2 = O_D1 + 4 * N, O_DEC = O_D2 + 4 * N, O_RUK = O_DEC + 4 * N;
constexpr lds_t SLOT_B = sizeof(SlotQ), SLOT0 = offsetof(SmemQ, slot);
constexpr lds_t T_AH = 0, T_AL = L * TROW_B, TILE_B = sizeof(TilesQ), TILE0 = offsetof(SmemQ, tile), YB0 = offsetof(SmemQ, yb), SST0 = offsetof(SmemQ, sst);
static_assert(offsetof(SlotQ, V) == O_V && offsetof(SlotQ, d1) == O_D1 && offsetof(SlotQ, ruk) == O_RUK && offsetof(TilesQ, AL) == T_AL, "layout");

struct ArgsQ {
    int T, C, H;
    const uint16_t *r, *k, *v, *w, *u, *s0;
    uint16_t* y;
    char* saved;                   // [B*H][ceil(n/2)] saved states (SAVED_STATE_B bytes each): the state entering every even chunk
    int* flags;                    // [B*H][8]
    // Sequences cut into NB blocks of TB tokens (a multiple of 64), one workgroup per (batch, head, block), for shapes with
    // fewer (batch, head) pairs than the chip has CUs.  Three launches: LOCAL = true leaves in blk_state the state that a
    // block builds from nothing and in blk_decay the log2 of its total decay per key channel; wkv6_scan turns these into
    // the state entering every block (s32); LOCAL = false then starts each block from there.  NB = 1: one launch, TB = T.
    int NB, TB;
    const float* s32;              // [B*H][NB][64][64] or null
    float* blk_state;              // [B*H][NB][64][64]
    float* blk_decay;              // [B*H][NB][64]
    bool head_decay;               // wkv5: w is one raw decay per channel, [H][64], the same at every token
    float* decay_out;              // wkv5: [2][C] fp32, exp(-exp(w)) and -exp(w), left for the two-sweep kernels and the backward
    bool first_row;                // this workgroup has batch row 0 (and block 0): it writes decay_out
};

// ---------------------------------------------------------------------------------------------------- P waves
template <bool LOCAL, bool HD>
DEVINL void role_prep(SmemQ& S, const ArgsQ& a, const int lane, const int w, const size_t base, const int h, const size_t bh, const int n, const int nit) {
    int jq = lane >> 4, tp = lane & 15;                 // arithmetic: channel pair, token (and token + 16)
    // Global memory is touched in whole 128-byte rows: eight lanes per row, eight rows per wave and instruction (waves
    // 0..3: r and w, waves 4..7: k and v, rows 8 (w & 3) ..), because the memory system takes requests for pieces of
    // a line, one from each of eight waves, at a much lower rate.  A wave thus stages columns that other waves prepare:
    // the prep waves meet (meet_signal / meet_wait) between the two.
    int rq = lane >> 3, pc = lane & 7;                  // memory: row 8 (w & 3) + rq of the chunk, piece pc of the row
    const int ch0 = 8 * w + 2 * (lane >> 4);
    const int T = a.T, C = a.C;
    const int wq = w & 3;
    const bool lower = w < 4;
    // global addresses: a wave-uniform base and a 32-bit byte offset per lane (row of the chunk + 16 bytes of the row), to
    // which a chunk adds a uniform term; rows past the end of the sequence are clamped to the last one
    const char* __restrict__ pA = reinterpret_cast<const char*>((lower ? a.r : a.k) + base);      // r | k
    // wkv5: the decay row of the head stands in for every token's (the loads stay, they hit the cache)
    // (HD: the decay is one value per channel and read once below; the r waves keep their second load, of the head's decay
    //  row at every token - a cache hit - so that all prep waves run the same loads and the waits count the same)
    const char* __restrict__ pB = reinterpret_cast<const char*>(lower ? (HD ? a.w + h * N : a.w + base) : a.v + base);   // w | v
    const uint32_t bmask = (HD && lower) ? 127u : ~0u;
    const uint32_t row_b = 2u * static_cast<uint32_t>(a.C);                                     // bytes from a token to the next
    uint32_t offA = (8 * (w & 3) + (lane >> 3)) * row_b + 16 * (lane & 7);                      // rows 8 (w & 3) .. +7
    const uint32_t lastA = static_cast<uint32_t>(a.T - 1) * row_b + 16 * (lane & 7);
    // LDS: uniform bases plus a few per-lane byte offsets, constants in the instruction
    const lds_t sb = lds_of(&S);
    lds_t b_row = (8 * (w & 3) + (lane >> 3)) * ROW_B + 16 * (lane & 7);  // [row 8 wq + rq][16 bytes pc] of a plane (staging, stores)
    lds_t b_tp = (lane & 15) * ROW_B + 4 * (4 * w + (lane >> 4));         // [token tp][channel pair 4 w + jq] of a plane
    lds_t b_ch = 4 * (8 * w + 2 * (lane >> 4));                           // channel 8 w + 2 jq of a per-channel array
    lds_t b_l = 4 * (lane & 15);                                          // token tp of a per-token array
    float uj[2];
    {
        const uint32_t x = *reinterpret_cast<const uint32_t*>(a.u + h * N + ch0);
        uj[0] = bf_lo(x); uj[1] = bf_hi(x);
    }
    struct Raw { u32x4 a, b; };
    // Little's law sets the depth: 256 workgroups x 8 waves x 2 KB per chunk are 4 MB, the memory system answers after
    // two to three microseconds under load, and a chunk is to take little more than one.
    Raw ring[DEPTH];                       // DEPTH chunks ahead
    auto fetch = [&](const int c, Raw& x) __attribute__((always_inline)) {
        const uint32_t o = min(static_cast<uint32_t>(c * L) * row_b + offA, lastA);
        x.a = *reinterpret_cast<const u32x4*>(pA + o);
        x.b = *reinterpret_cast<const u32x4*>(pB + (o & bmask));
    };
    // the rows of chunk c into the slot: r, k, w where the R' hi, K' hi, R' lo planes will be (staging), v in place
    auto stage_in = [&](const int c, const Raw& x, auto PARTIAL) __attribute__((always_inline)) {
        const lds_t so = uniform_base(sb + SLOT0 + (c % 3) * SLOT_B);
        const int row = 8 * wq + rq;
        const bool live = !decltype(PARTIAL)::value || c * L + row < T;
        const u32x4 zero = {0u, 0u, 0u, 0u};
        lds_st<u32x4>(so + (lower ? O_RPH : O_KPH) + b_row, live ? x.a : zero);
        if (!(HD && lower)) lds_st<u32x4>(so + (lower ? O_RPL : O_V) + b_row, (live || lower) ? x.b : zero);    // w of a dead row is masked where the decay is formed
        meet_signal(&S.met[0], lane);
    };
    bool any_exact = false, met_ok = true;
    float logdec[2] = {0.f, 0.f};          // LOCAL: log2 of the decay over the whole block
    // HD (wkv5): the decay of a channel is the same at every token, and so are the factors of every whole chunk: the sums
    // along time are products, the exponentials are taken once
    float lamc[2] = {0.f, 0.f}, eac[2][2] = {}, ebc[2][2] = {}, dc[2] = {0.f, 0.f};
    if constexpr (HD) {
        const uint32_t x = *reinterpret_cast<const uint32_t*>(a.w + h * N + ch0);
        lamc[0] = -LOG2E * exp2_fast(LOG2E * bf_lo(x)); lamc[1] = -LOG2E * exp2_fast(LOG2E * bf_hi(x));
#pragma unroll
        for (int z = 0; z < 2; ++z) {
            const float cc0 = -static_cast<float>(16 - tp) * lamc[z], cc1 = static_cast<float>(tp) * lamc[z];
            eac[0][z] = exp2_fast(cc0); eac[1][z] = exp2_fast(cc1);
            ebc[0][z] = exp2_fast(-(cc0 + lamc[z])); ebc[1][z] = exp2_fast(-(cc1 + lamc[z]));
            dc[z] = exp2_fast(16.f * lamc[z]);              // d1 = d2: the decay over half a chunk
        }
        const bool bad = (-16.f * lamc[0] > RANGE_LIMIT * LOG2E) || (-16.f * lamc[1] > RANGE_LIMIT * LOG2E);
        any_exact = __ballot(bad) != 0ull;
        if (!LOCAL && a.first_row && tp == 0) {
            // the wrapper-side transform of wkv5_bf16/run.py:63-64, for whoever needs the decay in that form afterwards
            const float e0 = -expf(bf_lo(x)), e1 = -expf(bf_hi(x));
            *reinterpret_cast<float2*>(a.decay_out + h * N + ch0) = make_float2(expf(e0), expf(e1));
            *reinterpret_cast<float2*>(a.decay_out + a.C + h * N + ch0) = make_float2(e0, e1);
        }
    }
    auto prep = [&](const int c, auto PARTIAL) __attribute__((always_inline)) {
        const lds_t so = uniform_base(sb + SLOT0 + (c % 3) * SLOT_B);
        constexpr bool CONST = HD && !decltype(PARTIAL)::value;      // a whole chunk of a constant decay
        float lam[2][2], rf[2][2], kf[2][2], ea[2][2], eb[2][2];
        uint32_t xr[2], xk[2], xw[2] = {0u, 0u};
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            xr[e] = lds_ld<uint32_t>(so + O_RPH + e * 16 * ROW_B + b_tp);
            xk[e] = lds_ld<uint32_t>(so + O_KPH + e * 16 * ROW_B + b_tp);
            if constexpr (!HD) xw[e] = lds_ld<uint32_t>(so + O_RPL + e * 16 * ROW_B + b_tp);
        }
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            rf[e][0] = bf_lo(xr[e]); rf[e][1] = bf_hi(xr[e]);
            kf[e][0] = bf_lo(xk[e]); kf[e][1] = bf_hi(xk[e]);
        }
        float a0, a1, b0, b1;
        if constexpr (CONST) {
#pragma unroll
            for (int e = 0; e < 2; ++e)
#pragma unroll
                for (int z = 0; z < 2; ++z) { ea[e][z] = eac[e][z]; eb[e][z] = ebc[e][z]; }
            a0 = dc[0]; a1 = dc[1]; b0 = dc[0]; b1 = dc[1];
            if constexpr (LOCAL) { logdec[0] += 32.f * lamc[0]; logdec[1] += 32.f * lamc[1]; }
        } else {
            float cc[2][2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const bool live = !decltype(PARTIAL)::value || c * L + tp + 16 * e < T;
                lam[e][0] = live ? (HD ? lamc[0] : -LOG2E * exp2_fast(LOG2E * bf_lo(xw[e]))) : 0.f;
                lam[e][1] = live ? (HD ? lamc[1] : -LOG2E * exp2_fast(LOG2E * bf_hi(xw[e]))) : 0.f;
            }
            float l1[2], l2[2];
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                const float s0 = row_suffix_sum(lam[0][z]);        // sum over tokens tp..15
                const float p1 = row_prefix_sum(lam[1][z]);        // sum over tokens 16..16+tp
                cc[0][z] = -s0;
                cc[1][z] = p1 - lam[1][z];
                l1[z] = bc<0>(s0);
                l2[z] = bc<15>(p1);
                if constexpr (LOCAL) logdec[z] += l1[z] + l2[z];
            }
            {
                const bool bad = (-l1[0] > RANGE_LIMIT * LOG2E) || (-l2[0] > RANGE_LIMIT * LOG2E) || (-l1[1] > RANGE_LIMIT * LOG2E) || (-l2[1] > RANGE_LIMIT * LOG2E);
                any_exact = any_exact || (__ballot(bad) != 0ull);
            }
            a0 = exp2_fast(l1[0]); a1 = exp2_fast(l1[1]); b0 = exp2_fast(l2[0]); b1 = exp2_fast(l2[1]);
#pragma unroll
            for (int e = 0; e < 2; ++e)
#pragma unroll
                for (int z = 0; z < 2; ++z) { ea[e][z] = exp2_fast(cc[e][z]); eb[e][z] = exp2_fast(-(cc[e][z] + lam[e][z])); }
        }
        if (tp == 0) {
            lds_st<f32x2>(so + O_D1 + b_ch, f32x2{a0, a1});
            lds_st<f32x2>(so + O_D2 + b_ch, f32x2{b0, b1});
            lds_st<f32x2>(so + O_DEC + b_ch, f32x2{a0 * b0, a1 * b1});
        }
        float ruk[2];
        HL r0[2], k0[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const float rp0 = rf[e][0] * ea[e][0], rp1 = rf[e][1] * ea[e][1];
            const float kp0 = kf[e][0] * eb[e][0], kp1 = kf[e][1] * eb[e][1];
            ruk[e] = fmaf(rf[e][0] * uj[0], kf[e][0], rf[e][1] * uj[1] * kf[e][1]);
            r0[e] = hilo2k(rp0, rp1); k0[e] = hilo2k(kp0, kp1);
        }
        // (the stores side by side, with no load between them: the compiler then pairs them, two planes or two rows an instruction)
#pragma unroll
        for (int e = 0; e < 2; ++e) { lds_st<uint32_t>(so + O_RPH + e * 16 * ROW_B + b_tp, r0[e].h); lds_st<uint32_t>(so + O_RPL + e * 16 * ROW_B + b_tp, r0[e].l); }
#pragma unroll
        for (int e = 0; e < 2; ++e) { lds_st<uint32_t>(so + O_KPH + e * 16 * ROW_B + b_tp, k0[e].h); lds_st<uint32_t>(so + O_KPL + e * 16 * ROW_B + b_tp, k0[e].l); }
        allreduce2_rows(ruk[0], ruk[1]);                       // sums over the four channel pairs of this wave
        if (jq == 0) { lds_st<float>(so + O_RUK + w * (4 * L) + b_l, ruk[0]); lds_st<float>(so + O_RUK + w * (4 * L) + 64 + b_l, ruk[1]); }
    };
    // The y rows of chunk c, left in LDS by the S waves in the last iteration: waves 0..3 store eight rows each, eight
    // lanes per 128-byte row, so that the memory system sees whole lines and not the 16-byte pieces of the loads.
    // (A store on every path, masked per lane, so that the waits for the prefetched inputs count the same on all of them.)
    char* __restrict__ pY = reinterpret_cast<char*>(a.y + base);
    auto store_y = [&](const int c, const bool on) __attribute__((always_inline)) {
        const int row = 8 * wq + rq;
        const u32x4 o = lds_ld<u32x4>(sb + YB0 + (c & 1) * PLANE_B + b_row);
        const int tg = c * L + row;
        if (on && lower && tg < T) *reinterpret_cast<u32x4*>(pY + (static_cast<uint32_t>(c * L) * row_b + offA)) = o;
    };

    const std::true_type part{};           // only the last chunk can be cut short
    const std::false_type full{};
    // in the order in which the loop consumes them: its waits are counted from the worst of all the ways into it
    static_for<DEPTH>([&](auto Z) {
        constexpr int z = decltype(Z)::value;
        __builtin_amdgcn_sched_barrier(0);
        fetch(z < n ? z : n - 1, ring[z]);
    });
    __builtin_amdgcn_sched_barrier(0);
    // DEPTH iterations per trip, nothing in them skipped: a way round a stage, or round the second half, would be one more
    // way into the next wait, on which the registers it waits for are the newest loads (the count then covers everything).
    // Past the last chunk the stages run on rows that all count as dead, into a slot nobody reads.
    for (int it0 = 0; it0 < nit; it0 += DEPTH)
        static_for<DEPTH>([&](auto Z) {
            constexpr int z = decltype(Z)::value;
            const int it = it0 + z;
            asm volatile("" : "+v"(jq), "+v"(tp), "+v"(rq), "+v"(pc), "+v"(offA));
            opaque(b_row); opaque(b_tp); opaque(b_ch); opaque(b_l);
            if (it >= n - 1) stage_in(it, ring[z], part); else stage_in(it, ring[z], full);
            __builtin_amdgcn_sched_barrier(0);
            fetch(it + DEPTH < n ? it + DEPTH : n - 1, ring[z]);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (!LOCAL) store_y(it >= 3 ? it - 3 : 0, it >= 3);
            __builtin_amdgcn_sched_barrier(0);
            met_ok = meet_wait(&S.met[0], 8u * (it + 1)) && met_ok;      // all eight waves have staged their rows of chunk it
            if (it >= n - 1) prep(it, part); else prep(it, full);
            __syncthreads();
        });
    // (a meeting that never completed, which the counting excludes, would leave the results of this head to the other kernel)
    // (with several blocks per head the words are cleared by the caller and only ever set)
    const bool flag = any_exact || !met_ok;
    if (lane == 0 && (a.NB == 1 || flag)) a.flags[bh * 8 + w] = flag ? 1 : 0;
    if constexpr (LOCAL) {
        if (tp == 0) *reinterpret_cast<float2*>(a.blk_decay + ch0) = make_float2(logdec[0], logdec[1]);
    }
}

// ---------------------------------------------------------------------------------------------------- S waves
template <bool LOCAL>
DEVINL void role_state(SmemQ& S, const ArgsQ& a, const int lane, const int w, const size_t bh, const int n, const int nit) {
    const int g = lane >> 4, l16 = lane & 15, i = 16 * w + l16;
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    const lds_t sb = lds_of(&S);
    lds_t b_acc = l16 * ROW_B + 8 * g;                                          // [token l16][channel 4 g] of a plane
    lds_t b_tr = ((8 * g + (l16 >> 2)) * PS + 2 * (l16 & 3)) * 4;               // transposing read of a plane, rows 8 g ..
    lds_t b_natt = l16 * TROW_B + 16 * g;                                       // [row l16][position 8 g] of a tile
    lds_t b_g = 16 * g + 4 * (l16 & 3);                                          // channel 4 g + (l16 & 3) of a per-channel array
    const uint32_t b_sv = i * N + 4 * g;                                        // [value channel i][key channel 4 g] of a state
    lds_t b_ss = (i * SS + 4 * g) * 4;                                          // the same in the LDS copy
    f32x4 St[4];                           // S[i = 16w + l16][j = 16 tile + 4g + v]
    if (!LOCAL && a.s32 != nullptr) {
#pragma unroll
        for (int tl = 0; tl < 4; ++tl) St[tl] = *reinterpret_cast<const f32x4*>(a.s32 + b_sv + 16 * tl);
    } else if (!LOCAL && a.s0 != nullptr) {
#pragma unroll
        for (int tl = 0; tl < 4; ++tl) {
            const uint2 x = *reinterpret_cast<const uint2*>(a.s0 + bh * (N * N) + b_sv + 16 * tl);
            St[tl] = f32x4{bf_lo(x.x), bf_hi(x.x), bf_lo(x.y), bf_hi(x.y)};
        }
    } else {
#pragma unroll
        for (int tl = 0; tl < 4; ++tl) St[tl] = zero4;
    }
    __syncthreads();                       // iterations 0 and 1: nothing prepared yet
    __syncthreads();
    // The factors, R' and v of a chunk have been in LDS for a whole iteration when its turn comes: they are asked for at
    // the end of the chunk before, so that the scaling of the state and the first products can start right behind the
    // barrier, when every wave of the workgroup is asking the LDS for something (only the A tile is made that late).
    float dq[4], de[4], d2[4];
    bf16x8 rh[2][2], rl[2][2], vop;
    // (in two parts, each where the registers it fills have had their last use in the current chunk)
    auto ahead_late = [&](const int c) __attribute__((always_inline)) {
        const lds_t so = uniform_base(sb + SLOT0 + (c % 3) * SLOT_B);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            de[q] = lds_ld<float>(so + O_DEC + 64 * q + b_g);
            d2[q] = lds_ld<float>(so + O_D2 + 64 * q + b_g);
        }
        vop = ld_tr(so + O_V + 32 * w + b_tr, ROW_B);                           // lane = value channel 16w + l16, K = tokens
    };
    auto ahead = [&](const int c) __attribute__((always_inline)) {
        const lds_t so = uniform_base(sb + SLOT0 + (c % 3) * SLOT_B);
#pragma unroll
        for (int q = 0; q < 4; ++q) dq[q] = lds_ld<float>(so + O_D1 + 64 * q + b_g);
        if constexpr (!LOCAL) {
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    rh[tt][ks] = ld_acc(so + O_RPH + tt * 16 * ROW_B + 64 * ks + b_acc);
                    rl[tt][ks] = ld_acc(so + O_RPL + tt * 16 * ROW_B + 64 * ks + b_acc);
                }
        }
    };
    ahead(0);
    ahead_late(0);
#pragma unroll 1
    for (int c = 0; c < n; ++c) {
        opaque(b_acc); opaque(b_tr); opaque(b_natt); opaque(b_g); opaque(b_ss);
        const lds_t so = uniform_base(sb + SLOT0 + (c % 3) * SLOT_B), to = uniform_base(sb + TILE0 + (c & 1) * TILE_B);
        if (!LOCAL && !(c & 1)) {
            // The state entering an even chunk goes to LDS and from there, in the next iteration, to global memory through
            // a wave that has nothing else to do: every workgroup writes its 16 KB at about the same moment, the memory
            // system takes a while to accept such a burst, and a state wave that waited for that would hold up the chunk.
#pragma unroll
            for (int tl = 0; tl < 4; ++tl) lds_st<f32x4>(sb + SST0 + 64 * tl + b_ss, St[tl]);
        }
        // ------------------------------------------------------------ batch 1: d1, R' (natural rows), v and the A tile
        // per-channel factors: a lane holds the one of channel 16 tile + 4 g + (l16 & 3), a 4-byte read that all rows of
        // four lanes share; the products below take lane v of the 16-lane row inside the multiply (row_newbcast)
        // (LOCAL: only the state is wanted, everything that serves y is left out)
        // (the A tile by rows: it arrives while the state is scaled and split)
        bf16x8 ah[2], al[2];
#pragma unroll
        for (int tt = 0; tt < (LOCAL ? 0 : 2); ++tt) { ah[tt] = ld_op(to + T_AH + tt * 16 * TROW_B + b_natt); al[tt] = ld_op(to + T_AL + tt * 16 * TROW_B + b_natt); }
        __builtin_amdgcn_sched_barrier(0);
        // ------------------------------------------------------------ y^T[i][t] = (S d1) R'^T + V^T A^T
        bf16x8 sh[2], sl[2];
#pragma unroll
        for (int ks = 0; ks < (LOCAL ? 0 : 2); ++ks) {
            float p[4], q[4];
            static_for<4>([&](auto V) {
                constexpr int v = decltype(V)::value;
                p[v] = St[2 * ks][v]; q[v] = St[2 * ks + 1][v];
                mul_bc<v>(p[v], dq[2 * ks]); mul_bc<v>(q[v], dq[2 * ks + 1]);
            });
            const HL x0 = hilo2k(p[0], p[1]), x1 = hilo2k(p[2], p[3]), x2 = hilo2k(q[0], q[1]), x3 = hilo2k(q[2], q[3]);
            sh[ks] = as_op(x0.h, x1.h, x2.h, x3.h);
            sl[ks] = as_op(x0.l, x1.l, x2.l, x3.l);
        }
        __builtin_amdgcn_sched_barrier(0);
        f32x4 Y[2] = {zero4, zero4};
#pragma unroll
        for (int ks = 0; ks < (LOCAL ? 0 : 2); ++ks)
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                Y[tt] = mfma(sh[ks], rh[tt][ks], Y[tt]);
                Y[tt] = mfma(sh[ks], rl[tt][ks], Y[tt]);
                Y[tt] = mfma(sl[ks], rh[tt][ks], Y[tt]);
            }
        __builtin_amdgcn_sched_barrier(0);
        // ------------------------------------------------------------ batch 3: K' with the tokens along K
        bf16x8 kh[4], kl[4];
#pragma unroll
        for (int tl = 0; tl < 4; ++tl) { kh[tl] = ld_tr(so + O_KPH + 32 * tl + b_tr, ROW_B); kl[tl] = ld_tr(so + O_KPL + 32 * tl + b_tr, ROW_B); }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int tt = 0; tt < (LOCAL ? 0 : 2); ++tt) {
            Y[tt] = mfma(vop, ah[tt], Y[tt]);
            Y[tt] = mfma(vop, al[tt], Y[tt]);
        }
        f32x4 U[4];
#pragma unroll
        for (int tl = 0; tl < 4; ++tl) {
            U[tl] = mfma(kh[tl], vop, zero4);
            U[tl] = mfma(kl[tl], vop, U[tl]);
        }
        __builtin_amdgcn_sched_barrier(0);
        ahead(c + 1);                      // (past the last chunk: a slot that holds something, read for nothing)
        __builtin_amdgcn_sched_barrier(0);
        // y: lane = token, four consecutive value channels in registers
#pragma unroll
        for (int tt = 0; tt < (LOCAL ? 0 : 2); ++tt)
            lds_st<u32x2>(sb + YB0 + (c & 1) * PLANE_B + tt * 16 * ROW_B + 32 * w + b_acc, u32x2{pack_bf2(Y[tt][0], Y[tt][1]), pack_bf2(Y[tt][2], Y[tt][3])});
        // ------------------------------------------------------------ S^T <- S^T dec + d2 K'^T V
#pragma unroll
        for (int tl = 0; tl < 4; ++tl)
            static_for<4>([&](auto V) {
                constexpr int v = decltype(V)::value;
                float x = St[tl][v];
                mul_bc<v>(x, de[tl]);
                fmac_bc<v>(x, d2[tl], U[tl][v]);
                St[tl][v] = x;
            });
        __builtin_amdgcn_sched_barrier(0);
        ahead_late(c + 1);
        __syncthreads();
    }
    for (int it = n + 2; it < nit; ++it) __syncthreads();      // the P waves store the last y
    if constexpr (LOCAL) {
#pragma unroll
        for (int tl = 0; tl < 4; ++tl) *reinterpret_cast<f32x4*>(a.blk_state + b_sv + 16 * tl) = St[tl];
    }
}

// ---------------------------------------------------------------------------------------------------- T waves
template <bool LOCAL>
DEVINL void role_tiles(SmemQ& S, const ArgsQ& a, const int lane, const int w, const size_t bh, const int n, const int nit) {
    const int g = lane >> 4, l16 = lane & 15;
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    const lds_t sb = lds_of(&S);
    lds_t b_nat = l16 * ROW_B + 8 * g;                                          // [token l16][channel 4 g] of a plane
    lds_t b_tw = l16 * TROW_B + 8 * g;                                          // [row l16][position 4 g] of a tile
    lds_t b_l = 4 * l16;
    // wave 0, 1, 2 -> quadrant (t, s) = (0,0) (1,0) (1,1); accumulator rows are s, lanes t
    const int ta = (w == 0) ? 0 : 1, tb = (w == 2) ? 1 : 0;
    // wave 3: the state that the S waves left in LDS in the last iteration, into the saved-state format (wkv6_chunk.h): in
    // step wq the lane gathers the sixteen elements of lane `lane` of the backward's state wave wq (value channels
    // 16 (e / 4) + 4 g + e % 4 of key channel 16 wq + l16: 4-byte reads, a bank per lane) and stores 3 x 16 bytes
    lds_t b_sr = (4 * g * SS + l16) * 4;
    char* __restrict__ sv = a.saved + 16 * lane;
    __syncthreads();                       // iteration 0
#pragma unroll 1
    for (int c = 0; c < nit - 1; ++c) {    // iteration c + 1
        opaque(b_nat); opaque(b_tw); opaque(b_l); opaque(b_sr);
        if (!LOCAL && w == 3 && c >= 2 && c - 2 < n && !(c & 1)) {
            char* dst = sv + static_cast<size_t>((c - 2) >> 1) * SAVED_STATE_B;
#pragma unroll
            for (int wq = 0; wq < 4; ++wq) {
                uint32_t x[16];
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    x[e] = saved_round(lds_ld<float>(sb + SST0 + ((16 * (e >> 2) + (e & 3)) * SS + 16 * wq) * 4 + b_sr));
                u32x4 hi[2], lo;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    // byte selectors: 0..3 from the second operand, 4..7 from the first
                    hi[0][q] = __builtin_amdgcn_perm(x[2 * q + 1], x[2 * q], 0x07060302u);
                    hi[1][q] = __builtin_amdgcn_perm(x[8 + 2 * q + 1], x[8 + 2 * q], 0x07060302u);
                    const uint32_t p01 = __builtin_amdgcn_perm(x[4 * q + 1], x[4 * q], 0x0c0c0501u);
                    const uint32_t p23 = __builtin_amdgcn_perm(x[4 * q + 3], x[4 * q + 2], 0x0c0c0501u);
                    lo[q] = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
                }
                *reinterpret_cast<u32x4*>(dst + wq * 2048) = hi[0];
                *reinterpret_cast<u32x4*>(dst + wq * 2048 + 1024) = hi[1];
                *reinterpret_cast<u32x4*>(dst + SAVED_LO_B + wq * 1024) = lo;
            }
        }
        if (!LOCAL && c < n && w < 3) {
            const lds_t so = uniform_base(sb + SLOT0 + (c % 3) * SLOT_B), to = uniform_base(sb + TILE0 + (c & 1) * TILE_B);
            // (in accumulator order, two 8-byte pieces: any order of the channels serves a contraction over them, and these
            //  reads run at the LDS's rate where 16-byte reads of rows take 1.6 x as long)
            const lds_t ra = so + ta * 16 * ROW_B + b_nat, rb = so + tb * 16 * ROW_B + b_nat;
            bf16x8 kh[2], kl[2], rh[2], rl[2];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                kh[ks] = ld_acc(rb + O_KPH + 64 * ks); kl[ks] = ld_acc(rb + O_KPL + 64 * ks);
                rh[ks] = ld_acc(ra + O_RPH + 64 * ks); rl[ks] = ld_acc(ra + O_RPL + 64 * ks);
            }
            float d = 0.f;
            if (ta == tb) {
                const lds_t ru = so + O_RUK + ta * 64 + b_l;
#pragma unroll
                for (int q = 0; q < 8; ++q) d += lds_ld<float>(ru + q * (4 * L));
            }
            __builtin_amdgcn_sched_barrier(0);
            f32x4 a0 = zero4, a1 = zero4;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                a0 = mfma(kh[ks], rh[ks], a0);
                a1 = mfma(kh[ks], rl[ks], a1);
                a1 = mfma(kl[ks], rh[ks], a1);
            }
            f32x4 am = a0 + a1;                                // [v]: s = 16 tb + 4g + v, t = 16 ta + l16
            if (ta == tb) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int sl = 4 * g + v;
                    am[v] = (sl < l16) ? am[v] : (sl == l16 ? d : 0.f);
                }
            }
            const HL x0 = hilo2k(am[0], am[1]), x1 = hilo2k(am[2], am[3]);
            const lds_t tw = to + ta * 16 * TROW_B + tb * 32 + b_tw;
            lds_st<u32x2>(tw + T_AH, u32x2{x0.h, x1.h});
            lds_st<u32x2>(tw + T_AL, u32x2{x0.l, x1.l});
        }
        __syncthreads();
    }
}

template <bool LOCAL, bool HD>
__global__ __launch_bounds__(NTQ) void wkv6_fwd_fused(const ArgsQ arg) {
    __shared__ SmemQ S;
    const int tid = threadIdx.x;
    // this workgroup's block of the sequence as a problem of its own
    const int bhx = blockIdx.x / arg.NB, blk = blockIdx.x % arg.NB;
    const int b = bhx / arg.H, h = bhx % arg.H;
    const int t0 = blk * arg.TB;
    const size_t base = (static_cast<size_t>(b) * arg.T + t0) * arg.C + static_cast<size_t>(h) * N;
    const size_t bh = bhx, bq = bh * arg.NB + blk;
    ArgsQ a = arg;
    a.T = arg.T - t0 < arg.TB ? arg.T - t0 : arg.TB;
    const int nseg = ((arg.T + L - 1) / L + 1) / 2;                 // saved states of a whole sequence
    a.saved = arg.saved + (bh * nseg + t0 / (2 * L)) * SAVED_STATE_B;
    if (arg.s32 != nullptr) a.s32 = arg.s32 + bq * (N * N);
    if (arg.blk_state != nullptr) { a.blk_state = arg.blk_state + bq * (N * N); a.blk_decay = arg.blk_decay + bq * N; }
    a.first_row = b == 0 && blk == 0;
    const int n = (a.T + L - 1) / L;
    // the quadrant t < 16 <= s of the tiles is never written and must read as zero
    for (int i = tid; i < static_cast<int>(sizeof(S.tile) / 4); i += NTQ) reinterpret_cast<uint32_t*>(&S.tile[0])[i] = 0;
    if (tid == 0) S.met[0] = 0;
    __syncthreads();
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, w = wid & 3;
    const int nit = (n + 2 + DEPTH) & ~(DEPTH - 1);        // iterations of the pipeline: n + 3, in whole trips of the prep loop
    if (wid < 8) role_prep<LOCAL, HD>(S, a, lane, wid, base, h, bh, n, nit);
    else if (wid < 12) role_state<LOCAL>(S, a, lane, w, bh, n, nit);
    else role_tiles<LOCAL>(S, a, lane, w, bh, n, nit);
}

// States entering the blocks from the local results, one workgroup of 256 threads per (batch, head), 16 consecutive key
// channels of one value channel per thread.  Forward (reverse = 0): S = s0; out[blk] = S; S <- S 2^logdec[blk] + local[blk].
// Reverse: the same from the last block down, from zero: what enters a block from above.
__global__ __launch_bounds__(256) void wkv6_scan(const float* __restrict__ local, const float* __restrict__ logdec, const uint16_t* __restrict__ s0,
                                                 float* __restrict__ out, const int NB, const int reverse) {
    const size_t bh = blockIdx.x;
    const int e = threadIdx.x * 16, j0 = e % N;
    float x[16];
#pragma unroll
    for (int q = 0; q < 16; ++q) x[q] = (s0 != nullptr && !reverse) ? bf2f(s0[bh * (N * N) + e + q]) : 0.f;
    for (int i = 0; i < NB; ++i) {
        const int blk = reverse ? NB - 1 - i : i;
        const size_t o = (bh * NB + blk) * (N * N) + e;
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            out[o + q] = x[q];
            x[q] = fmaf(x[q], exp2_fast(logdec[(bh * NB + blk) * N + j0 + q]), local[o + q]);
        }
    }
}

}  // namespace

int launch_wkv6_fwd_fused(hipStream_t st, int B, int T, int C, int H, const uint16_t* r, const uint16_t* k, const uint16_t* v,
                          const uint16_t* w, const uint16_t* u, const uint16_t* s0, uint16_t* y, char* saved, int* flags,
                          int NB, int TB, float* blk_state, float* blk_decay, float* s32, float* decay_out) {
    ArgsQ a{};
    const bool head_decay = decay_out != nullptr;
    a.head_decay = head_decay; a.decay_out = decay_out;
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.s0 = s0; a.y = y; a.saved = saved; a.flags = flags;
    a.NB = 1; a.TB = T;
    if (NB <= 1) {
        if (head_decay) hipLaunchKernelGGL((wkv6_fwd_fused<false, true>), dim3(B * H), dim3(NTQ), 0, st, a);
        else hipLaunchKernelGGL((wkv6_fwd_fused<false, false>), dim3(B * H), dim3(NTQ), 0, st, a);
        return launch_status();
    }
    a.NB = NB; a.TB = TB; a.blk_state = blk_state; a.blk_decay = blk_decay;
    if (head_decay) hipLaunchKernelGGL((wkv6_fwd_fused<true, true>), dim3(B * H * NB), dim3(NTQ), 0, st, a);
    else hipLaunchKernelGGL((wkv6_fwd_fused<true, false>), dim3(B * H * NB), dim3(NTQ), 0, st, a);
    hipLaunchKernelGGL(wkv6_scan, dim3(B * H), dim3(256), 0, st, blk_state, blk_decay, s0, s32, NB, 0);
    a.blk_state = nullptr; a.blk_decay = nullptr; a.s32 = s32;
    if (head_decay) hipLaunchKernelGGL((wkv6_fwd_fused<false, true>), dim3(B * H * NB), dim3(NTQ), 0, st, a);
    else hipLaunchKernelGGL((wkv6_fwd_fused<false, false>), dim3(B * H * NB), dim3(NTQ), 0, st, a);
    return launch_status();
}

// reverse scan for the backward (wkv6_bwd_f.hip): out[blk] = what enters block blk from above
int launch_wkv6_scan_reverse(hipStream_t st, int BH, int NB, const float* local, const float* logdec, float* out) {
    hipLaunchKernelGGL(wkv6_scan, dim3(BH), dim3(256), 0, st, local, logdec, static_cast<const uint16_t*>(nullptr), out, NB, 1);
    return launch_status();
}

}  // namespace rwkv
