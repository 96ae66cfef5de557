// wkv6 / wkv6_state backward in ONE reverse sweep (gfx950), from the chunk states that the forward kernel saved.
//
// Formulas (wkv6_chunk.h for R', K', d1, d2, dec; chunk of L = 32 tokens, factors referred to its middle m = 16):
//     Bm[t][s] = gy_t . v_s (s < t)              A[t][s] = R'_t . K'_s (s < t),  A[t][t] = sum_j r u k
//     X_t = GY_t (S0 d1) + sum_{s<t} Bm[t][s] K'_s            dr'_t = ea_t X_t      gr = dr' + u k_t (v_t . gy_t)
//     Z_s = V_s (dS d2) + sum_{t>s} Bm[t][s] R'_t             dk'_s = eb_s Z_s      gk = dk' + u r_s (v_s . gy_s)
//     gv_s = (dS d2) K'_s + sum_{t>=s} A[t][s] gy_t
//     dS <- dS dec + d1 GY^T R'                               (gradient of the state that enters the chunk)
//     gw_t = lam_t G_t,  G_t = P_{t+1} - k_t dk'_t,  P_t = P_{t+1} + r_t dr'_t - k_t dk'_t,  P = sum_i dS S exactly where a saved state is at hand
// S0 = the forward state entering the chunk: the forward kernel stores it for every second chunk (fp32, [value][key]);
// the state of the odd chunk in between is rebuilt here with one update, S <- S dec + d2 V^T K'.
//
// One workgroup of 16 waves per (batch, head) in three roles: eight P waves with 8 channels each, four SD and four E waves
// with 16 channels each:
//   P  (prep)   channels 8w..8w+7 of r, k, w, v, gy for all 32 tokens of a chunk: lane = 16 * (channel pair) + token,
//               so the time scans of a half-chunk are four DPP adds inside a 16-lane row and no prep wave ever needs
//               another one's sums.  Writes the bf16 hi / lo planes of R', K', plain v, gy; keeps r, k and the exponents
//               cc_t = log2 ea_t of the chunks in flight in registers and, three iterations later, turns the X and Z of
//               that chunk into gr, gk, gw (and gu) and stores them: all elementwise work sits where the inputs are.
//   SD (states) forward state S[i][j] and gradient state dS[i][j], key channels j = 16w..: lane = j, registers = i.
//               X, Z, gs, the dS update, P at the anchors.
//   E  (dstate^T) dS[i][j], value channels i = 16w..: lane = i, registers = j.  gv, dS update, and the causal tiles A, Bm of
//               the next chunk.
// A state is the accumulator of its update product and, as it stands, the A operand of the products that read it
// (K slots <-> channels in accumulator order).  Operands with the tokens along K come from the natural [token][channel]
// planes through ds_read_b64_tr_b16: 16 lanes read a 4 x 16 block and each ends up with one column of it.
// The accumulators of X, Z, gv have lane = token and four consecutive channels in registers -- the layout of the prep
// waves: X and Z cross to the prep waves through LDS, gv is stored from registers.
//
// Pipeline (one barrier per chunk): in iteration `it` the P waves prepare chunk n-1-it, the EW waves make the tiles of
// chunk n-it, the SD and E waves do the products of chunk n+1-it, and the P waves finish chunk n+2-it.
//
// A chunk in which some channel decays by more than e^-60 over either half cannot use the mid-point factors.  Such a
// (batch, head) is flagged in `flags` and the caller reruns it with the two-sweep kernels, which have a step-by-step path.
#include "wkv6_fused.h"

namespace rwkv {
namespace {

constexpr int NTG = 16 * 64;
// Row strides (dwords) measured on the access patterns of this kernel: 36 serves the 8-byte operand reads in accumulator
// order and the prep waves' 4-byte reads at twice the rate of 40, 68 serves the prep waves' reads of X and Z at five
// times the rate of 72 (16-byte reads and the transposing reads do not care).
constexpr int PS = 36;             // bf16 [token][channel] planes: 144 B
constexpr int CS = 68;             // fp32 [token][channel] arrays: 272 B
constexpr int DEPTH = 2;           // chunks that the prep waves load ahead (four would cost the prep waves spills)
constexpr int KEPT = 3;            // iterations between the preparation of a chunk and its finishing
constexpr int TRIP = 6;            // iterations per trip of the prep loop: a multiple of both, so that the registers of the
                                   // loads in flight and of what is kept for the finishing have fixed names (no copies)
constexpr int TQ = 20;             // causal tiles [t][s], 32 bf16 and 16 bytes of padding: 80 B (16-byte reads of 16 rows hit all banks once)

struct alignas(16) SlotG {
    uint32_t RpH[L][PS], RpL[L][PS], KpH[L][PS], KpL[L][PS], V[L][PS], GY[L][PS];
    float d1[N], d2[N], dec[N];            // 2^{c_m}, 2^{c_L - c_m}, 2^{c_L}
    float ruk[8][L];                        // sum of r u k over the 8 channels of each prep wave
};
struct alignas(16) TilesG {
    uint32_t AH[L][TQ], AL[L][TQ], BH[L][TQ], BL[L][TQ];   // [t][s] bf16 hi / lo
};
struct alignas(16) SmemG {
    // (the small arrays come first: below 64 KB their addresses are a lane offset plus a constant inside the instruction)
    uint32_t out[4][L][PS];                 // gr, gk, gw, gv of one chunk, bf16 [token][channel], on their way to global memory
    float vg[3][L];                         // v_t . gy_t of the chunks in flight
    float pex[2][N];                        // P = sum_i dS S at the last two anchors
    uint32_t met[4];                        // meeting counters: inputs staged, results written, gv taken
    SlotG slot[3];
    TilesG tile[2];
    float xz[2][2][L][CS];                  // [chunk parity][X, Z][token][key channel]: from the SD waves to the P waves
};
static_assert(sizeof(SmemG) <= 160 * 1024, "LDS");
constexpr lds_t ROW_B = PS * 4, PLANE_B = L * ROW_B, TROW_B = TQ * 4, XROW_B = CS * 4, XZ_B = L * XROW_B;
constexpr lds_t O_RPH = 0, O_RPL = PLANE_B, O_KPH = 2 * PLANE_B, O_KPL = 3 * PLANE_B, O_V = 4 * PLANE_B, O_GY = 5 * PLANE_B;
constexpr lds_t O_D1 = 6 * PLANE_B, O_D2 = O_D1 + 4 * N, O_DEC = O_D2 + 4 * N, O_RUK = O_DEC + 4 * N;
constexpr lds_t SLOT_B = sizeof(SlotG), SLOT0 = offsetof(SmemG, slot);
constexpr lds_t T_AH = 0, T_AL = L * TROW_B, T_BH = 2 * L * TROW_B, T_BL = 3 * L * TROW_B, TILE_B = sizeof(TilesG), TILE0 = offsetof(SmemG, tile);
constexpr lds_t XZ0 = offsetof(SmemG, xz), VG0 = offsetof(SmemG, vg), PEX0 = offsetof(SmemG, pex), OUT0 = offsetof(SmemG, out);
static_assert(offsetof(SlotG, GY) == O_GY && offsetof(SlotG, d1) == O_D1 && offsetof(SlotG, ruk) == O_RUK && offsetof(TilesG, BL) == T_BL, "layout");


struct ArgsG {
    int T, C, H;
    const uint16_t *r, *k, *v, *u, *gy;
    const void* w;
    uint16_t *gr, *gk, *gv, *gw, *gu, *gs;
    const char* saved;             // [B*H][ceil(n/2)] saved states (SAVED_STATE_B bytes each): the forward state entering every even chunk
    int* flags;                    // [B*H][8]
    // Sequences cut into NB blocks of TB tokens (a multiple of 64), one workgroup per (batch, head, block), see
    // wkv6_fwd_f.hip.  LOCAL = true leaves in blk_ds the gradient state that a block builds from nothing, going down from
    // its end, and in blk_decay the log2 of its total decay; wkv6_scan (reverse) turns these into the gradient state
    // that enters every block from above (ds32); LOCAL = false then starts each block from there.
    int NB, TB;
    const float* ds32;             // [B*H][NB][64][64], [value][key], or null
    float* blk_ds;                 // [B*H][NB][64][64]
    float* blk_decay;              // [B*H][NB][64]
    float* gu32;                   // NB > 1: gu of this (batch, head, block) in fp32 (the blocks are added before rounding)
    bool first, above;             // this is block 0; there is a block above this one
    // wkv5: w is one raw decay per channel, [H][64], and its gradient is summed over the tokens: a row per batch row in
    // gwp (bf16 [B][C]) or, with NB > 1, per block and batch row in gw32 (fp32 [NB][B][C]); gw is not written
    bool head_decay;
    uint16_t* gwp;
    float* gw32;
};

// state entering even chunk e of this (batch, head), in the layout of the SD waves: lane <-> key channel 16w + l16,
// x[tile][v] <-> value channel 16 tile + 4g + v.  p: the state (wave-uniform), lo = byte offset of [4 g][16 w + l16].
// (a uniform base per tile, one 32-bit lane offset and constants: sixteen loads without any address arithmetic)
DEVINL void load_state(const float* __restrict__ p, const uint32_t lo, f32x4 (&x)[4]) {
#pragma unroll
    for (int tl = 0; tl < 4; ++tl) {
        const char* q = reinterpret_cast<const char*>(p + 16 * tl * N) + lo;
#pragma unroll
        for (int v = 0; v < 4; ++v) x[tl][v] = *reinterpret_cast<const float*>(q + v * (4 * N));
    }
}

// A saved state (format: wkv6_chunk.h) in the same layout, for SD wave w: three 16-byte loads per lane (p: the state,
// wave-uniform; lo = 16 * lane), kept as loaded while they are in flight and expanded where the state is first needed.
struct SavedRaw { u32x4 ha, hb, lo; };
DEVINL void fetch_saved(const char* __restrict__ p, const int w, const uint32_t lo, SavedRaw& q) {
    const char* hi = p + 2048 * w, *lw = p + SAVED_LO_B + 1024 * w;
    q.ha = *reinterpret_cast<const u32x4*>(hi + lo);
    q.hb = *reinterpret_cast<const u32x4*>(hi + 1024 + lo);
    q.lo = *reinterpret_cast<const u32x4*>(lw + lo);
}
DEVINL void expand_saved(const SavedRaw& q, f32x4 (&x)[4]) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        // bytes 3, 2: the element's upper half; byte 1: its low byte; byte 0: zero
        constexpr uint32_t ZERO = 0x0cu;
        const uint32_t sel = ((5u + 2u * (e & 1)) << 24) | ((4u + 2u * (e & 1)) << 16) | (static_cast<uint32_t>(e & 3) << 8) | ZERO;
        const uint32_t h = e < 8 ? q.ha[(e & 7) >> 1] : q.hb[(e & 7) >> 1];
        x[e >> 2][e & 3] = __uint_as_float(__builtin_amdgcn_perm(h, q.lo[e >> 2], sel));
    }
}

// ---------------------------------------------------------------------------------------------------- P waves
// wave w (0..7): channels 8w..8w+7; lane = 16 * (channel pair) + token: a thread has two channels of tokens tp and tp + 16
template <int WMODE, bool LOCAL>
DEVINL void role_prep(SmemG& S, const ArgsG& a, const int lane, const int w, const size_t base, const int h, const size_t bh, const int n, const int nit) {
    // jq, tp (and hl, rw below) are redefined behind an empty asm in every iteration, see role_sd
    int jq = lane >> 4, tp = lane & 15;
    const int ch0 = 8 * w + 2 * (lane >> 4);
    const int T = a.T, C = a.C;
    // Global memory is touched in whole 128-byte rows, 16 bytes per lane and eight lanes per row: the memory system takes
    // requests for pieces of a line, one from each of eight waves, at a much lower rate.  Per chunk a wave loads rows
    // 8 (w & 3) .. +7 of two tensors (waves 0..3: r and w, waves 4..7: k and v) and rows 4 w .. +3 of gy, and stores rows
    // 8 (w & 3) .. +7 of two (gr and gw, or gk and gv).  So a wave stages columns that other waves prepare, and stores
    // columns that other waves have finished: the planes of the slot being prepared carry the inputs, `out` the results,
    // and the prep waves meet (meet_signal / meet_wait) between writing and reading them.
    int rq = lane >> 3, pc = lane & 7, rg = (lane & 31) >> 3;
    const int wq = w & 3;
    const bool lower = w < 4;
    // LDS is addressed as in the other roles: uniform bases plus a few per-lane byte offsets, constants in the instruction
    const lds_t sb = lds_of(&S);
    lds_t b_row = (8 * wq + rq) * ROW_B + 16 * pc;                    // [row 8 wq + rq][16 bytes pc] of a plane (staging, stores)
    lds_t b_rowg = (4 * w + rg) * ROW_B + 16 * pc;                    // the same for the rows of gy
    lds_t b_tp = tp * ROW_B + 4 * (4 * w + jq);                       // [token tp][channel pair 4 w + jq] of a plane
    lds_t b_ch = 4 * (8 * w + 2 * jq);                                // channel 8 w + 2 jq of a per-channel array
    lds_t b_l = 4 * tp;                                               // token tp of a per-token array
    lds_t b_x = tp * XROW_B + 4 * (8 * w + 2 * jq);                   // [token tp][channel 8 w + 2 jq] of X / Z
    // global addresses: a wave-uniform base and a 32-bit byte offset per lane (row of the chunk + 16 bytes of the row), to
    // which a chunk adds a uniform term; rows past the end of the sequence are clamped to the last one
    const char* __restrict__ pA = reinterpret_cast<const char*>((lower ? a.r : a.k) + base);                         // r | k
    constexpr bool HD = WMODE == W_HEAD;   // wkv5: one decay per channel, the same at every token
    // (HD: the r waves keep their second load, of the head's decay row at every token - a cache hit - so that all prep waves
    //  run the same loads and the waits count the same; the decay itself is read once, below)
    const char* __restrict__ pB = reinterpret_cast<const char*>(lower ? (HD ? static_cast<const uint16_t*>(a.w) + h * N : static_cast<const uint16_t*>(a.w) + base) : a.v + base);   // w | v
    const uint32_t bmask = (lower && HD) ? 127u : ~0u;
    const char* __restrict__ pC = reinterpret_cast<const char*>(a.gy + base);
    const uint32_t row_b = 2u * static_cast<uint32_t>(a.C);                                     // bytes from a token to the next
    uint32_t offA = (8 * (w & 3) + (lane >> 3)) * row_b + 16 * (lane & 7);                      // rows 8 (w & 3) .. +7
    uint32_t offG = (4 * w + ((lane & 31) >> 3)) * row_b + 16 * (lane & 7);                     // rows 4 w .. +3
    const uint32_t lastA = static_cast<uint32_t>(a.T - 1) * row_b + 16 * (lane & 7);
    float uj[2];
    {
        const uint32_t x = *reinterpret_cast<const uint32_t*>(a.u + h * N + ch0);
        uj[0] = bf_lo(x); uj[1] = bf_hi(x);
    }
    struct Raw { u32x4 a, b, c; };
    Raw ring[DEPTH];                       // DEPTH chunks ahead
    auto fetch = [&](const int c, Raw& x) __attribute__((always_inline)) {
        const uint32_t cb = static_cast<uint32_t>(c * L) * row_b;
        const uint32_t o = min(cb + offA, lastA), og = min(cb + offG, lastA);
        x.a = *reinterpret_cast<const u32x4*>(pA + o);
        x.b = *reinterpret_cast<const u32x4*>(pB + (o & bmask));
        x.c = *reinterpret_cast<const u32x4*>(pC + og);    // (both halves of the wave ask for the same four rows)
    };
    // the rows of chunk c into the slot: r, k, w where the R' hi, K' hi, R' lo planes will be (staging), v and gy in place
    auto stage_in = [&](const int c, const Raw& x, auto PARTIAL) __attribute__((always_inline)) {
        const lds_t so = uniform_base(sb + SLOT0 + ((c + 9) % 3) * SLOT_B);
        const int row = 8 * wq + rq, rowg = 4 * w + rg;
        const bool live = !decltype(PARTIAL)::value || (c >= 0 && c * L + row < T);
        const bool liveg = !decltype(PARTIAL)::value || (c >= 0 && c * L + rowg < T);
        const u32x4 zero = {0u, 0u, 0u, 0u};
        const lds_t da = so + (lower ? O_RPH : O_KPH) + b_row, db = so + (lower ? O_RPL : O_V) + b_row;
        lds_st<u32x4>(da, live ? x.a : zero);
        if (!(HD && lower)) lds_st<u32x4>(db, (live || lower) ? x.b : zero);    // w of a dead row is masked where the decay is formed
        if (lane < 32) lds_st<u32x4>(so + O_GY + b_rowg, liveg ? x.c : zero);
    };
    // what the finishing of a chunk needs from its preparation, three iterations earlier
    // (r, k as loaded; ea = 2^{cc_t}, eb = 2^{-cc_{t+1}}, the factors of R' and K'; lf = d ln w / d w_raw, the decay gradient's factor:
    //  keeping the factors costs twelve registers per chunk in flight and saves the finishing two exponentials per element)
    struct Held { uint32_t r[2], k[2]; float ea[2][2], eb[2][2], lf[2][2]; };
    Held hq[3] = {};
    bool any_exact = false, met_ok = true;
    float logdec[2] = {0.f, 0.f};          // LOCAL: log2 of the decay over the whole block
    float carry[2] = {0.f, 0.f}, gu_acc[2] = {0.f, 0.f}, gw_acc[2] = {0.f, 0.f};
    // HD: the factors of every whole chunk are the same: the sums along time are products, the exponentials are taken once
    float lamc[2] = {0.f, 0.f}, eac[2][2] = {}, ebc[2][2] = {}, dc[2] = {0.f, 0.f}, lfc[2] = {0.f, 0.f};
    if constexpr (HD) {
        const uint32_t x = *reinterpret_cast<const uint32_t*>(static_cast<const uint16_t*>(a.w) + h * N + ch0);
        lamc[0] = -LOG2E * exp2_fast(LOG2E * bf_lo(x)); lamc[1] = -LOG2E * exp2_fast(LOG2E * bf_hi(x));
#pragma unroll
        for (int z = 0; z < 2; ++z) {
            const float cc0 = -static_cast<float>(16 - tp) * lamc[z], cc1 = static_cast<float>(tp) * lamc[z];
            eac[0][z] = exp2_fast(cc0); eac[1][z] = exp2_fast(cc1);
            ebc[0][z] = exp2_fast(-(cc0 + lamc[z])); ebc[1][z] = exp2_fast(-(cc1 + lamc[z]));
            dc[z] = exp2_fast(16.f * lamc[z]);              // d1 = d2: the decay over half a chunk
            lfc[z] = gw_factor(lamc[z] * LN2);
        }
        const bool bad = (-16.f * lamc[0] > RANGE_LIMIT * LOG2E) || (-16.f * lamc[1] > RANGE_LIMIT * LOG2E);
        any_exact = __ballot(bad) != 0ull;
    }
    // Only the last chunk of the sequence can be cut short (PARTIAL): its rows past T carry no input and no decay.

    auto prep = [&](const int c, Held& hd, auto PARTIAL) __attribute__((always_inline)) {
        const lds_t so = uniform_base(sb + SLOT0 + ((c + 9) % 3) * SLOT_B);
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
            hd.r[e] = xr[e]; hd.k[e] = xk[e];
        }
        float a0, a1, b0, b1;
        if constexpr (CONST) {
            // (the finishing takes the constant factors too: nothing but r and k is kept)
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
                const bool live = !decltype(PARTIAL)::value || (c >= 0 && c * L + tp + 16 * e < T);
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
                for (int z = 0; z < 2; ++z) {
                    ea[e][z] = exp2_fast(cc[e][z]);
                    eb[e][z] = exp2_fast(-(cc[e][z] + lam[e][z]));
                    hd.ea[e][z] = ea[e][z]; hd.eb[e][z] = eb[e][z];
                    hd.lf[e][z] = gw_factor(lam[e][z] * LN2);
                }
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

    // gr, gk, gw of chunk c from X, Z (left by the SD waves in the last iteration) and what prep kept
    auto finish = [&](const int c, const Held& hd, auto PARTIAL) __attribute__((always_inline)) {
        constexpr bool CONSTF = HD && !decltype(PARTIAL)::value;
        const lds_t xo = uniform_base(sb + XZ0 + (c & 1) * 2 * XZ_B), vo = uniform_base(sb + VG0 + (c % 3) * (4 * L));
        float q[2][2], kdk[2][2];
        uint32_t ogr[2], ogk[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const f32x2 x2 = lds_ld<f32x2>(xo + e * 16 * XROW_B + b_x);
            const f32x2 z2 = lds_ld<f32x2>(xo + XZ_B + e * 16 * XROW_B + b_x);
            const float X[2] = {x2.x, x2.y}, Z[2] = {z2.x, z2.y};
            const float vg = lds_ld<float>(vo + 64 * e + b_l);
            const float rf[2] = {bf_lo(hd.r[e]), bf_hi(hd.r[e])}, kf[2] = {bf_lo(hd.k[e]), bf_hi(hd.k[e])};
            float gr[2], gk[2];
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                const float drp = (CONSTF ? eac[e][z] : hd.ea[e][z]) * X[z], dkp = (CONSTF ? ebc[e][z] : hd.eb[e][z]) * Z[z];
                const float uvg = uj[z] * vg;
                gr[z] = fmaf(uvg, kf[z], drp);
                gk[z] = fmaf(uvg, rf[z], dkp);
                kdk[e][z] = kf[z] * dkp;
                q[e][z] = fmaf(rf[z], drp, -kdk[e][z]);
                gu_acc[z] = fmaf(rf[z] * kf[z], vg, gu_acc[z]);
            }
            ogr[e] = pack_bf2(gr[0], gr[1]); ogk[e] = pack_bf2(gk[0], gk[1]);
        }
#pragma unroll
        for (int e = 0; e < 2; ++e) { lds_st<uint32_t>(sb + OUT0 + e * 16 * ROW_B + b_tp, ogr[e]); lds_st<uint32_t>(sb + OUT0 + PLANE_B + e * 16 * ROW_B + b_tp, ogk[e]); }
        float gw[2][2];
#pragma unroll
        for (int z = 0; z < 2; ++z) {
            const float s1 = row_suffix_sum(q[1][z]) + carry[z];           // P_t of the second half
            const float s0 = row_suffix_sum(q[0][z]) + bc<0>(s1);
            gw[1][z] = (CONSTF ? lfc[z] : hd.lf[1][z]) * ((s1 - q[1][z]) - kdk[1][z]);        // lam (P_{t+1} - k dk')
            gw[0][z] = (CONSTF ? lfc[z] : hd.lf[0][z]) * ((s0 - q[0][z]) - kdk[0][z]);
            carry[z] = bc<0>(s0);
        }
        if (!(c & 1)) {
            // the chunk began at an anchor: from here on P counts from its exact value there
            const f32x2 p2 = lds_ld<f32x2>(sb + PEX0 + ((c >> 1) & 1) * (4 * N) + b_ch);
            carry[0] = p2.x; carry[1] = p2.y;
        }
        // without an initial state nothing has been accumulated before token 0: its decay has no effect at all
        if (a.gs == nullptr && a.first && c == 0 && tp == 0) { gw[0][0] = 0.f; gw[0][1] = 0.f; }
        if (HD) {
            gw_acc[0] += gw[0][0] + gw[1][0]; gw_acc[1] += gw[0][1] + gw[1][1];
        } else {
#pragma unroll
            for (int e = 0; e < 2; ++e) lds_st<uint32_t>(sb + OUT0 + 2 * PLANE_B + e * 16 * ROW_B + b_tp, pack_bf2(gw[e][0], gw[e][1]));
        }
    };
    const bool cut = (T % L) != 0;         // the last chunk is cut short
    const std::true_type part{};
    const std::false_type full{};
    // in the order in which the loop consumes them: its waits are counted from the worst of all the ways into it
    static_for<DEPTH>([&](auto Z) {
        constexpr int z = decltype(Z)::value;
        __builtin_amdgcn_sched_barrier(0);
        fetch(n - 1 - z >= 0 ? n - 1 - z : 0, ring[z]);
    });
    __builtin_amdgcn_sched_barrier(0);
    // DEPTH iterations per trip, no stage with loads or ring registers skipped: a way round one, or round the second half,
    // would be one more way into the next wait, on which the registers it waits for are the newest loads (the count then
    // covers everything).  Below chunk 0 the stages run on rows that all count as dead, into the planes of a slot that
    // nobody reads any more (c < 0: the slot of chunk c + 3, whose products were done in the iteration before).
    for (int it0 = 0; it0 < nit; it0 += TRIP)
        static_for<TRIP>([&](auto Z) {
            constexpr int z = decltype(Z)::value % DEPTH, zk = decltype(Z)::value % KEPT;
            const int it = it0 + decltype(Z)::value;
            const int cp = n - 1 - it;
            asm volatile("" : "+v"(jq), "+v"(tp), "+v"(rq), "+v"(pc), "+v"(rg), "+v"(offA), "+v"(offG));
            opaque(b_row); opaque(b_rowg); opaque(b_tp); opaque(b_ch); opaque(b_l); opaque(b_x);
            const bool fin = !LOCAL && it >= 3 && cp + 3 >= 0;      // chunk cp + 3 is finished in this iteration
            if ((cut && it == 0) || cp < 0) stage_in(cp, ring[z], part); else stage_in(cp, ring[z], full);
            meet_signal(&S.met[0], lane);
            __builtin_amdgcn_sched_barrier(0);
            fetch(cp >= DEPTH ? cp - DEPTH : 0, ring[z]);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (!LOCAL) {
                if (it == 3 && a.above) {
                    // P at the end of the block, from the gradient state that enters from above and the saved state there
                    const f32x2 p2 = lds_ld<f32x2>(sb + PEX0 + ((n >> 1) & 1) * (4 * N) + b_ch);
                    carry[0] = p2.x; carry[1] = p2.y;
                }
                if (fin) { if (cut && it == 3) finish(cp + 3, hq[zk], part); else finish(cp + 3, hq[zk], full); }
                meet_signal(&S.met[1], lane);
            }
            __builtin_amdgcn_sched_barrier(0);
            met_ok = meet_wait(&S.met[0], 8u * (it + 1)) && met_ok;        // all rows of chunk cp are staged
            if ((cut && it == 0) || cp < 0) prep(cp, hq[zk], part); else prep(cp, hq[zk], full);
            __syncthreads();
        });
    // (a meeting that never completed, which the counting excludes, would leave this head to the two-sweep kernels)
    // (with several blocks per head the words are cleared by the caller and only ever set)
    // (S.met[3]: a meeting of the E waves that never completed; written before the last barrier)
    const bool flag = any_exact || !met_ok || S.met[3] != 0;
    if (lane == 0 && (a.NB == 1 || flag)) a.flags[bh * 8 + w] = flag ? 1 : 0;
    if constexpr (LOCAL) {
        if (tp == 0) *reinterpret_cast<float2*>(a.blk_decay + ch0) = make_float2(logdec[0], logdec[1]);
    } else {
        // gu of this batch row (and block): sum over the tokens (lanes of a row)
#pragma unroll
        for (int z = 0; z < 2; ++z) gu_acc[z] = row_sum_to_last(gu_acc[z]);
        if (tp == 15) {
            if (a.gu32 != nullptr) *reinterpret_cast<float2*>(a.gu32 + ch0) = make_float2(gu_acc[0], gu_acc[1]);
            else *reinterpret_cast<uint32_t*>(a.gu + ch0) = pack_bf2(gu_acc[0], gu_acc[1]);
        }
        if (HD) {
#pragma unroll
            for (int z = 0; z < 2; ++z) gw_acc[z] = row_sum_to_last(gw_acc[z]);
            if (tp == 15) {
                if (a.gw32 != nullptr) *reinterpret_cast<float2*>(a.gw32 + ch0) = make_float2(gw_acc[0], gw_acc[1]);
                else *reinterpret_cast<uint32_t*>(a.gwp + ch0) = pack_bf2(gw_acc[0], gw_acc[1]);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------- SD waves
template <int WMODE, bool LOCAL>
DEVINL void role_sd(SmemG& S, const ArgsG& a, const int lane, const int w, const size_t bh, const int n, const int nit) {
    const int g = lane >> 4, l16 = lane & 15, j = 16 * w + l16;
    const int nseg = (n + 1) / 2;
    const char* __restrict__ sv = a.saved;                                      // the saved states of this block
    if constexpr (LOCAL) {                 // only the E waves have work
        for (int it = 0; it < nit; ++it) __syncthreads();
        return;
    }
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    const lds_t sb = lds_of(&S);
    // per-lane address parts
    uint32_t b_sv = 4 * (4 * g * N + j);                                        // [value channel 4 g][key channel j] of an fp32 state (bytes)
    uint32_t b_q = 16 * lane;                                                   // this lane's pieces of a saved state
    lds_t b_acc = l16 * ROW_B + 8 * g;                                          // [token l16][channel 4 g] of a plane
    lds_t b_tr = ((8 * g + (l16 >> 2)) * PS + 2 * (l16 & 3)) * 4;               // transposing read of a plane, rows 8 g ..
    lds_t b_trt = ((8 * g + (l16 >> 2)) * TQ + 2 * (l16 & 3)) * 4;              // the same of a tile
    lds_t b_natt = l16 * TROW_B + 16 * g;                                       // [row l16][position 8 g] of a tile
    lds_t b_xz = l16 * XROW_B + 16 * g;                                         // [token l16][channel 4 g] of X / Z
    lds_t b_j = 4 * l16;
    f32x4 D[4] = {zero4, zero4, zero4, zero4};
    SavedRaw Sq;                           // the saved state of the segment at hand (chunks 2 sg, 2 sg + 1), as loaded: twelve
                                           // registers instead of sixteen, expanded where a chunk uses it
    float pa = 0.f;                        // P = sum_i dS S of an even chunk, this lane's part

    // Operands are fetched in batches, each issued as a whole before anything waits for it (the scheduling barriers keep
    // the batches apart): a wave then waits for LDS a few times per chunk instead of once per product.
    // X^T[j][t] = (S d1)^T GY^T + K'^T Bm^T for chunk c; S = Sa (even chunk) or one update of it (odd chunk)
    auto part_x = [&](const int c) __attribute__((always_inline)) {
        const lds_t so = uniform_base(sb + SLOT0 + (c % 3) * SLOT_B), to = uniform_base(sb + TILE0 + (c & 1) * TILE_B), xo = uniform_base(sb + XZ0 + (c & 1) * 2 * XZ_B + 64 * w);
        f32x4 Sc[4], Sa[4];
        expand_saved(Sq, Sa);
        if (c & 1) {
            // state entering the odd chunk: S dec + d2 V^T K' with the chunk below
            const lds_t qo = uniform_base(sb + SLOT0 + ((c - 1) % 3) * SLOT_B);
            const float qdec = lds_ld<float>(qo + O_DEC + 64 * w + b_j), qd2 = lds_ld<float>(qo + O_D2 + 64 * w + b_j);
            const bf16x8 qh = ld_tr(qo + O_KPH + 32 * w + b_tr, ROW_B), ql = ld_tr(qo + O_KPL + 32 * w + b_tr, ROW_B);
            bf16x8 vop[4];
#pragma unroll
            for (int tl = 0; tl < 4; ++tl) vop[tl] = ld_tr(qo + O_V + 32 * tl + b_tr, ROW_B);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int tl = 0; tl < 4; ++tl) {
                f32x4 U = mfma(vop[tl], qh, zero4);
                U = mfma(vop[tl], ql, U);
#pragma unroll
                for (int v = 0; v < 4; ++v) Sc[tl][v] = fmaf(Sa[tl][v], qdec, qd2 * U[v]);
            }
        } else {
            // anchor: P = sum_i dS S with the saved state entering this chunk (D has taken the chunk in already)
            pa = 0.f;
#pragma unroll
            for (int tl = 0; tl < 4; ++tl) {
                Sc[tl] = Sa[tl];
#pragma unroll
                for (int v = 0; v < 4; ++v) pa = fmaf(D[tl][v], Sa[tl][v], pa);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        const float d1 = lds_ld<float>(so + O_D1 + 64 * w + b_j);
        bf16x8 gop[2][2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) gop[tt][ks] = ld_acc(so + O_GY + tt * 16 * ROW_B + 64 * ks + b_acc);
        const bf16x8 kh = ld_tr(so + O_KPH + 32 * w + b_tr, ROW_B), kl = ld_tr(so + O_KPL + 32 * w + b_tr, ROW_B);
        bf16x8 bh_[2], bl_[2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) { bh_[tt] = ld_op(to + T_BH + tt * 16 * TROW_B + b_natt); bl_[tt] = ld_op(to + T_BL + tt * 16 * TROW_B + b_natt); }
        __builtin_amdgcn_sched_barrier(0);
        bf16x8 sh[2], sl[2];
        split16(Sc, d1, sh, sl);
        f32x4 X[2] = {zero4, zero4};
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                X[tt] = mfma(sh[ks], gop[tt][ks], X[tt]);
                X[tt] = mfma(sl[ks], gop[tt][ks], X[tt]);
            }
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
            X[tt] = mfma(kh, bh_[tt], X[tt]);
            X[tt] = mfma(kh, bl_[tt], X[tt]);
            X[tt] = mfma(kl, bh_[tt], X[tt]);
        }
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) lds_st<f32x4>(xo + tt * 16 * XROW_B + b_xz, X[tt]);
    };
    // Z^T[j][s] = (dS d2)^T V^T + R'^T Bm, then dS <- dS dec + d1 GY^T R'
    auto part_z = [&](const int c) __attribute__((always_inline)) {
        const lds_t so = uniform_base(sb + SLOT0 + (c % 3) * SLOT_B), to = uniform_base(sb + TILE0 + (c & 1) * TILE_B), xo = uniform_base(sb + XZ0 + (c & 1) * 2 * XZ_B + XZ_B + 64 * w);
        const float d1 = lds_ld<float>(so + O_D1 + 64 * w + b_j), d2 = lds_ld<float>(so + O_D2 + 64 * w + b_j), dec = lds_ld<float>(so + O_DEC + 64 * w + b_j);
        bf16x8 vop[2][2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) vop[tt][ks] = ld_acc(so + O_V + tt * 16 * ROW_B + 64 * ks + b_acc);
        const bf16x8 rh = ld_tr(so + O_RPH + 32 * w + b_tr, ROW_B), rl = ld_tr(so + O_RPL + 32 * w + b_tr, ROW_B);
        bf16x8 bh_[2], bl_[2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) { bh_[tt] = ld_tr(to + T_BH + 32 * tt + b_trt, TROW_B); bl_[tt] = ld_tr(to + T_BL + 32 * tt + b_trt, TROW_B); }
        __builtin_amdgcn_sched_barrier(0);
        bf16x8 dh[2], dl[2];
        split16(D, d2, dh, dl);
        __builtin_amdgcn_sched_barrier(0);
        bf16x8 gop[4];
#pragma unroll
        for (int tl = 0; tl < 4; ++tl) gop[tl] = ld_tr(so + O_GY + 32 * tl + b_tr, ROW_B);
        __builtin_amdgcn_sched_barrier(0);
        f32x4 Z[2] = {zero4, zero4};
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                Z[tt] = mfma(dh[ks], vop[tt][ks], Z[tt]);
                Z[tt] = mfma(dl[ks], vop[tt][ks], Z[tt]);
            }
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
            Z[tt] = mfma(rh, bh_[tt], Z[tt]);
            Z[tt] = mfma(rh, bl_[tt], Z[tt]);
            Z[tt] = mfma(rl, bh_[tt], Z[tt]);
        }
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) lds_st<f32x4>(xo + tt * 16 * XROW_B + b_xz, Z[tt]);
#pragma unroll
        for (int tl = 0; tl < 4; ++tl) {
            f32x4 U = mfma(gop[tl], rh, zero4);
            U = mfma(gop[tl], rl, U);
#pragma unroll
            for (int v = 0; v < 4; ++v) D[tl][v] = fmaf(D[tl][v], dec, d1 * U[v]);
        }
    };

    if (a.ds32 != nullptr) {
        load_state(a.ds32, b_sv, D);       // the gradient state that enters the block from above
        if (a.above) {
            // P there, with the forward state at the end of the block (the first saved state of the block above)
            fetch_saved(sv + static_cast<size_t>(n >> 1) * SAVED_STATE_B, w, b_q, Sq);
            f32x4 Sa[4];
            expand_saved(Sq, Sa);
            float p = 0.f;
#pragma unroll
            for (int tl = 0; tl < 4; ++tl)
#pragma unroll
                for (int v = 0; v < 4; ++v) p = fmaf(D[tl][v], Sa[tl][v], p);
            p = allreduce_rows(p);
            if (g == 0) lds_st<float>(sb + PEX0 + ((n >> 1) & 1) * (4 * N) + 64 * w + b_j, p);
        }
    }
    fetch_saved(sv + static_cast<size_t>(nseg - 1) * SAVED_STATE_B, w, b_q, Sq);
    __syncthreads();                       // iterations 0 and 1: nothing prepared yet
    __syncthreads();
#pragma unroll 1
    for (int c = n - 1; c >= 0; --c) {
        opaque(b_acc); opaque(b_tr); opaque(b_trt); opaque(b_natt); opaque(b_xz); opaque(b_j); opaque(b_q);
        // the state of an odd chunk's segment was asked for at the end of the last iteration: what does not need it goes first
        part_z(c);
        __builtin_amdgcn_sched_barrier(0);
        part_x(c);
        __builtin_amdgcn_sched_barrier(0);
        if (!(c & 1)) {
            const float p = allreduce_rows(pa);
            if (g == 0) lds_st<float>(sb + PEX0 + ((c >> 1) & 1) * (4 * N) + 64 * w + b_j, p);
            // the next segment's state (index clamped: the load is issued on every path, so that waits can count it)
            fetch_saved(sv + static_cast<size_t>(c >= 2 ? (c >> 1) - 1 : 0) * SAVED_STATE_B, w, b_q, Sq);
        }
        __syncthreads();
    }
    for (int it = n + 2; it < nit; ++it) __syncthreads();      // the P waves finish chunk 0
    if (a.gs != nullptr && a.first) {
#pragma unroll
        for (int tl = 0; tl < 4; ++tl)
#pragma unroll
            for (int v = 0; v < 4; ++v) a.gs[(bh * N + 16 * tl + 4 * g + v) * N + j] = f2bf(D[tl][v]);
    }
}

// ---------------------------------------------------------------------------------------------------- E waves
template <int WMODE, bool LOCAL>
DEVINL void role_e(SmemG& S, const ArgsG& a, const int lane, const int w, const size_t base, const int n, const int nit) {
    constexpr bool HD = WMODE == W_HEAD;
    const int g = lane >> 4, l16 = lane & 15;
    const int T = a.T, C = a.C;
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    const lds_t sb = lds_of(&S);
    lds_t b_acc = l16 * ROW_B + 8 * g;                                          // [token l16][channel 4 g] of a plane
    lds_t b_nat = l16 * ROW_B + 16 * g;                                         // [token l16][channel 8 g] of a plane
    lds_t b_tr = ((8 * g + (l16 >> 2)) * PS + 2 * (l16 & 3)) * 4;               // transposing read of a plane, rows 8 g ..
    lds_t b_trt = ((8 * g + (l16 >> 2)) * TQ + 2 * (l16 & 3)) * 4;              // the same of a tile
    lds_t b_tw = l16 * TROW_B + 8 * g;                                          // [row l16][position 4 g] of a tile
    lds_t b_g = 16 * g + 4 * (l16 & 3);                                          // channel 4 g + (l16 & 3) of a per-channel array
    lds_t b_l = 4 * l16;
    // The E waves also carry the results to global memory, in whole 128-byte rows (eight lanes a row, rows 8 w .. +7 of each
    // of the four tensors per wave): the prep waves leave gr, gk, gw of a chunk in `out`, the E waves gv, and meetings
    // (meet_signal / meet_wait) stand between the writing and the reading of a plane.
    lds_t b_row = (8 * w + (lane >> 3)) * ROW_B + 16 * (lane & 7);
    const uint32_t row_b = 2u * static_cast<uint32_t>(C);
    uint32_t offA = (8 * w + (lane >> 3)) * row_b + 16 * (lane & 7);
    char* __restrict__ pgr = reinterpret_cast<char*>(a.gr + base);
    char* __restrict__ pgk = reinterpret_cast<char*>(a.gk + base);
    char* __restrict__ pgv = reinterpret_cast<char*>(a.gv + base);
    char* __restrict__ pgw = reinterpret_cast<char*>(a.gw + base);
    bool met_ok = true;
    f32x4 E[4] = {zero4, zero4, zero4, zero4};     // dS[i = 16w + l16][j = 16 tile + 4g + v]
    const uint32_t b_e = (16 * w + l16) * N + 4 * g;                            // that element of a [value][key] state
    if (!LOCAL && a.ds32 != nullptr) {
#pragma unroll
        for (int tl = 0; tl < 4; ++tl) E[tl] = *reinterpret_cast<const f32x4*>(a.ds32 + b_e + 16 * tl);
    }

    // causal tiles of chunk c, quadrants (t, s) = (0,0) (1,0) (1,1); accumulator rows are s, lanes t.  A = tril(K' R'^T) with
    // the bonus on the diagonal, Bm = tril_strict(V GY^T) (its diagonal goes to vg).  Waves 0 and 2 form the A tile of a
    // diagonal quadrant each, wave 1 both tiles of the full quadrant, wave 3 the Bm tiles of the two diagonal quadrants.
    auto tile_a = [&](const int c, const int ta, const int tb) __attribute__((always_inline)) {
        const lds_t so = uniform_base(sb + SLOT0 + (c % 3) * SLOT_B), to = uniform_base(sb + TILE0 + (c & 1) * TILE_B);
        const lds_t ra = so + ta * 16 * ROW_B + b_nat, rb = so + tb * 16 * ROW_B + b_nat;
        f32x4 a0 = zero4, a1 = zero4;
        bf16x8 kh[2], kl[2], rh[2], rl[2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            kh[ks] = ld_op(rb + O_KPH + 64 * ks); kl[ks] = ld_op(rb + O_KPL + 64 * ks);
            rh[ks] = ld_op(ra + O_RPH + 64 * ks); rl[ks] = ld_op(ra + O_RPL + 64 * ks);
        }
        float d = 0.f;
        if (ta == tb) {
            const lds_t ru = so + O_RUK + ta * 64 + b_l;
#pragma unroll
            for (int q = 0; q < 8; ++q) d += lds_ld<float>(ru + q * (4 * L));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            a0 = mfma(kh[ks], rh[ks], a0);
            a1 = mfma(kh[ks], rl[ks], a1);
            a1 = mfma(kl[ks], rh[ks], a1);
        }
        f32x4 am = a0 + a1;                                    // [v]: s = 16 tb + 4g + v, t = 16 ta + l16
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
    };
    auto tile_b = [&](const int c, const int ta, const int tb) __attribute__((always_inline)) {
        const lds_t so = uniform_base(sb + SLOT0 + (c % 3) * SLOT_B), to = uniform_base(sb + TILE0 + (c & 1) * TILE_B);
        const lds_t ra = so + ta * 16 * ROW_B + b_nat, rb = so + tb * 16 * ROW_B + b_nat;
        f32x4 bm = zero4;
        bf16x8 vo[2], go[2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) { vo[ks] = ld_op(rb + O_V + 64 * ks); go[ks] = ld_op(ra + O_GY + 64 * ks); }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) bm = mfma(vo[ks], go[ks], bm);
        if (ta == tb) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int sl = 4 * g + v;
                if (sl == l16) lds_st<float>(sb + VG0 + (c % 3) * (4 * L) + ta * 64 + b_l, bm[v]);
                bm[v] = (sl < l16) ? bm[v] : 0.f;
            }
        }
        const HL y0 = hilo2k(bm[0], bm[1]), y1 = hilo2k(bm[2], bm[3]);
        const lds_t tw = to + ta * 16 * TROW_B + tb * 32 + b_tw;
        lds_st<u32x2>(tw + T_BH, u32x2{y0.h, y1.h});
        lds_st<u32x2>(tw + T_BL, u32x2{y0.l, y1.l});
    };
    auto tiles = [&](const int c) __attribute__((always_inline)) {
        if (w == 0) tile_a(c, 0, 0);
        else if (w == 2) tile_a(c, 1, 1);
        else if (w == 1) { tile_a(c, 1, 0); tile_b(c, 1, 0); }
        else { tile_b(c, 0, 0); tile_b(c, 1, 1); }
    };

#pragma unroll 1
    for (int it = 0; it < nit; ++it) {
        const int c = n + 1 - it;
        opaque(b_acc); opaque(b_nat); opaque(b_tr); opaque(b_trt); opaque(b_tw); opaque(b_g); opaque(b_l); opaque(b_row);
        asm volatile("" : "+v"(offA));
        if (it >= 2 && c >= 0) {
            const lds_t so = uniform_base(sb + SLOT0 + (c % 3) * SLOT_B), to = uniform_base(sb + TILE0 + (c & 1) * TILE_B);
            // Operands are fetched in batches, each issued as a whole before anything waits for it (the scheduling barriers
            // keep the batches apart): a wave then waits for LDS three times per chunk instead of once per product.
            // ------------------------------------------------------------ batch 1: d2 and K' (natural rows)
            // per-channel factors: a lane holds the one of channel 16 tile + 4 g + (l16 & 3), a 4-byte read that rows of
            // four lanes share; the products below take lane v of the 16-lane row inside the multiply (row_newbcast)
            float dq[4], de[4], d1[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                dq[q] = lds_ld<float>(so + O_D2 + 64 * q + b_g);
                de[q] = lds_ld<float>(so + O_DEC + 64 * q + b_g);
                d1[q] = lds_ld<float>(so + O_D1 + 64 * q + b_g);
            }
            // (LOCAL: only the gradient state is wanted, everything that serves gv is left out)
            bf16x8 kh[2][2], kl[2][2];
#pragma unroll
            for (int tt = 0; tt < (LOCAL ? 0 : 2); ++tt)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    kh[tt][ks] = ld_acc(so + O_KPH + tt * 16 * ROW_B + 64 * ks + b_acc);
                    kl[tt][ks] = ld_acc(so + O_KPL + tt * 16 * ROW_B + 64 * ks + b_acc);
                }
            __builtin_amdgcn_sched_barrier(0);
            // ------------------------------------------------------------ gv^T[i][s] = (dS d2) K'^T + GY^T A
            bf16x8 dh[2], dl[2];
#pragma unroll
            for (int ks = 0; ks < (LOCAL ? 0 : 2); ++ks) {
                float p[4], q[4];
                static_for<4>([&](auto V) {
                    constexpr int v = decltype(V)::value;
                    p[v] = E[2 * ks][v]; q[v] = E[2 * ks + 1][v];
                    mul_bc<v>(p[v], dq[2 * ks]); mul_bc<v>(q[v], dq[2 * ks + 1]);
                });
                const HL x0 = hilo2k(p[0], p[1]), x1 = hilo2k(p[2], p[3]), x2 = hilo2k(q[0], q[1]), x3 = hilo2k(q[2], q[3]);
                dh[ks] = as_op(x0.h, x1.h, x2.h, x3.h);
                dl[ks] = as_op(x0.l, x1.l, x2.l, x3.l);
            }
            __builtin_amdgcn_sched_barrier(0);
            // ------------------------------------------------------------ batch 2: gy and the A tile with the tokens along K
            const bf16x8 gyo = ld_tr(so + O_GY + 32 * w + b_tr, ROW_B);        // lane = value channel 16w + l16, K = tokens
            bf16x8 ah[2], al[2];
#pragma unroll
            for (int tt = 0; tt < (LOCAL ? 0 : 2); ++tt) { ah[tt] = ld_tr(to + T_AH + 32 * tt + b_trt, TROW_B); al[tt] = ld_tr(to + T_AL + 32 * tt + b_trt, TROW_B); }
            __builtin_amdgcn_sched_barrier(0);
            f32x4 G[2] = {zero4, zero4};
#pragma unroll
            for (int ks = 0; ks < (LOCAL ? 0 : 2); ++ks)
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    G[tt] = mfma(dh[ks], kh[tt][ks], G[tt]);
                    G[tt] = mfma(dh[ks], kl[tt][ks], G[tt]);
                    G[tt] = mfma(dl[ks], kh[tt][ks], G[tt]);
                }
            __builtin_amdgcn_sched_barrier(0);
            // ------------------------------------------------------------ batch 3: R' with the tokens along K
            bf16x8 rh[4], rl[4];
#pragma unroll
            for (int tl = 0; tl < 4; ++tl) { rh[tl] = ld_tr(so + O_RPH + 32 * tl + b_tr, ROW_B); rl[tl] = ld_tr(so + O_RPL + 32 * tl + b_tr, ROW_B); }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int tt = 0; tt < (LOCAL ? 0 : 2); ++tt) {
                G[tt] = mfma(gyo, ah[tt], G[tt]);
                G[tt] = mfma(gyo, al[tt], G[tt]);
            }
            f32x4 U[4];
#pragma unroll
            for (int tl = 0; tl < 4; ++tl) {
                U[tl] = mfma(rh[tl], gyo, zero4);
                U[tl] = mfma(rl[tl], gyo, U[tl]);
            }
            __builtin_amdgcn_sched_barrier(0);
            // gv: lane = token, four consecutive value channels in registers (the rows of the last chunk were taken out of
            // `out` before the barrier)
#pragma unroll
            for (int tt = 0; tt < (LOCAL ? 0 : 2); ++tt)
                lds_st<u32x2>(sb + OUT0 + 3 * PLANE_B + tt * 16 * ROW_B + 32 * w + b_acc, u32x2{pack_bf2(G[tt][0], G[tt][1]), pack_bf2(G[tt][2], G[tt][3])});
            // ------------------------------------------------------------ dS^T <- dS^T dec + d1 R'^T GY
#pragma unroll
            for (int tl = 0; tl < 4; ++tl)
                static_for<4>([&](auto V) {
                    constexpr int v = decltype(V)::value;
                    float x = E[tl][v];
                    mul_bc<v>(x, de[tl]);
                    fmac_bc<v>(x, d1[tl], U[tl][v]);
                    E[tl][v] = x;
                });
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!LOCAL) {
            // gv of chunk c, when all four E waves have written their channels
            meet_signal(&S.met[2], lane);
            met_ok = meet_wait(&S.met[2], 4u * (it + 1)) && met_ok;
            const u32x4 o = lds_ld<u32x4>(sb + OUT0 + 3 * PLANE_B + b_row);
            if (it >= 2 && c >= 0 && c * L + 8 * w + (lane >> 3) < T) *reinterpret_cast<u32x4*>(pgv + (static_cast<uint32_t>(c * L) * row_b + offA)) = o;
        }
        __builtin_amdgcn_sched_barrier(0);
        if (!LOCAL && it >= 1 && c - 1 >= 0) tiles(c - 1);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!LOCAL) {
            // gr, gk, gw of chunk c + 1, when all eight prep waves have finished their columns
            met_ok = meet_wait(&S.met[1], 8u * (it + 1)) && met_ok;
            const u32x4 o0 = lds_ld<u32x4>(sb + OUT0 + b_row), o1 = lds_ld<u32x4>(sb + OUT0 + PLANE_B + b_row), o2 = lds_ld<u32x4>(sb + OUT0 + 2 * PLANE_B + b_row);
            if (it >= 3 && c + 1 >= 0 && (c + 1) * L + 8 * w + (lane >> 3) < T) {
                const uint32_t ob = static_cast<uint32_t>((c + 1) * L) * row_b + offA;
                *reinterpret_cast<u32x4*>(pgr + ob) = o0;
                *reinterpret_cast<u32x4*>(pgk + ob) = o1;
                if (!HD) *reinterpret_cast<u32x4*>(pgw + ob) = o2;
            }
        }
        if (!met_ok && lane == 0) S.met[3] = 1;        // (the prep waves read it after the last barrier and flag the head)
        __syncthreads();
    }
    if constexpr (LOCAL) {
#pragma unroll
        for (int tl = 0; tl < 4; ++tl) *reinterpret_cast<f32x4*>(a.blk_ds + b_e + 16 * tl) = E[tl];
    }
}

template <int WMODE, bool LOCAL>
__global__ __launch_bounds__(NTG) void wkv6_bwd_fused(const ArgsG arg) {
    __shared__ SmemG S;
    const int tid = threadIdx.x;
    // this workgroup's block of the sequence as a problem of its own
    const int bhx = blockIdx.x / arg.NB, blk = blockIdx.x % arg.NB;
    const int b = bhx / arg.H, h = bhx % arg.H;
    const int t0 = blk * arg.TB;
    const size_t base = (static_cast<size_t>(b) * arg.T + t0) * arg.C + static_cast<size_t>(h) * N;
    const size_t bh = bhx, bq = bh * arg.NB + blk;
    ArgsG a = arg;
    a.T = arg.T - t0 < arg.TB ? arg.T - t0 : arg.TB;
    const int nsegs = ((arg.T + L - 1) / L + 1) / 2;                // saved states of a whole sequence
    a.saved = arg.saved + (bh * nsegs + t0 / (2 * L)) * SAVED_STATE_B;
    a.first = blk == 0;
    a.above = blk + 1 < arg.NB;
    if (arg.ds32 != nullptr) a.ds32 = arg.ds32 + bq * (N * N);
    if (arg.blk_ds != nullptr) { a.blk_ds = arg.blk_ds + bq * (N * N); a.blk_decay = arg.blk_decay + bq * N; }
    // gu: a row per batch row [B][C], or per block and batch row [NB][B][C] in fp32
    if (arg.gu32 != nullptr) a.gu32 = arg.gu32 + ((static_cast<size_t>(blk) * (gridDim.x / (arg.NB * arg.H)) + b) * arg.H + h) * N;
    else a.gu = arg.gu + bh * N;
    if (arg.gw32 != nullptr) a.gw32 = arg.gw32 + ((static_cast<size_t>(blk) * (gridDim.x / (arg.NB * arg.H)) + b) * arg.H + h) * N;
    else if (arg.gwp != nullptr) a.gwp = arg.gwp + bh * N;
    const int n = (a.T + L - 1) / L;
    // the quadrant t < 16 <= s of the tiles is never written and must read as zero
    for (int i = tid; i < static_cast<int>(sizeof(S.tile) / 4); i += NTG) reinterpret_cast<uint32_t*>(&S.tile[0])[i] = 0;
    if (tid < 4) S.met[tid] = 0;
    __syncthreads();
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, w = wid & 3;
    const int nit = (n + 3 + TRIP - 1) / TRIP * TRIP;      // iterations of the pipeline: n + 3, in whole trips of the prep loop
    if (wid < 8) role_prep<WMODE, LOCAL>(S, a, lane, wid, base, h, bh, n, nit);
    else if (wid < 12) role_sd<WMODE, LOCAL>(S, a, lane, w, bh, n, nit);
    else {
        // The dS waves carry the recurrence and issue little; left at the default priority they are the youngest waves of
        // their SIMDs, get the issue slots that the others leave, and the whole workgroup waits for them at every barrier
        // (measured: 5 % of their time at the barrier against 22..37 % for the others).  Ahead of the others they cost those
        // almost nothing.  (Raising the X/Z waves as well starves the prep waves: slower.)
        __builtin_amdgcn_s_setprio(2);
        role_e<WMODE, LOCAL>(S, a, lane, w, base, n, nit);
    }
}

// gu of a batch row from its blocks: out[b][c] = bf16(sum_blk part[blk][b][c])
__global__ __launch_bounds__(256) void gu_block_sum(const int NB, const size_t n, const float* __restrict__ part, uint16_t* __restrict__ out) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= n) return;
    float x = 0.f;
    for (int blk = 0; blk < NB; ++blk) x += part[blk * n + i];
    out[i] = f2bf(x);
}

}  // namespace

int launch_wkv6_bwd_fused(hipStream_t st, int B, int T, int C, int H, const uint16_t* r, const uint16_t* k, const uint16_t* v,
                          const uint16_t* w, const uint16_t* u, const uint16_t* gy, uint16_t* gr, uint16_t* gk, uint16_t* gv,
                          uint16_t* gw, uint16_t* gu, uint16_t* gs, const char* saved, int* flags,
                          int NB, int TB, float* blk_ds, float* blk_decay, float* ds32, float* gu32, uint16_t* gwp, float* gw32) {
    ArgsG a{};
    a.head_decay = gwp != nullptr; a.gwp = gwp;
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.gy = gy;
    a.gr = gr; a.gk = gk; a.gv = gv; a.gw = gw; a.gu = gu; a.gs = gs; a.saved = saved; a.flags = flags;
    a.NB = 1; a.TB = T;
    const bool hd = a.head_decay;
    if (NB <= 1) {
        if (hd) hipLaunchKernelGGL((wkv6_bwd_fused<W_HEAD, false>), dim3(B * H), dim3(NTG), 0, st, a);
        else hipLaunchKernelGGL((wkv6_bwd_fused<W_RAW, false>), dim3(B * H), dim3(NTG), 0, st, a);
        return launch_status();
    }
    a.NB = NB; a.TB = TB; a.blk_ds = blk_ds; a.blk_decay = blk_decay;
    if (hd) hipLaunchKernelGGL((wkv6_bwd_fused<W_HEAD, true>), dim3(B * H * NB), dim3(NTG), 0, st, a);
    else hipLaunchKernelGGL((wkv6_bwd_fused<W_RAW, true>), dim3(B * H * NB), dim3(NTG), 0, st, a);
    if (int e = launch_wkv6_scan_reverse(st, B * H, NB, blk_ds, blk_decay, ds32)) return e;
    a.blk_ds = nullptr; a.blk_decay = nullptr; a.ds32 = ds32; a.gu32 = gu32;
    if (gwp != nullptr) a.gw32 = gw32;
    if (hd) hipLaunchKernelGGL((wkv6_bwd_fused<W_HEAD, false>), dim3(B * H * NB), dim3(NTG), 0, st, a);
    else hipLaunchKernelGGL((wkv6_bwd_fused<W_RAW, false>), dim3(B * H * NB), dim3(NTG), 0, st, a);
    const size_t n = static_cast<size_t>(B) * C;
    hipLaunchKernelGGL(gu_block_sum, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st, NB, n, gu32, gu);
    if (gwp != nullptr) hipLaunchKernelGGL(gu_block_sum, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st, NB, n, gw32, gwp);
    return launch_status();
}

}  // namespace rwkv
