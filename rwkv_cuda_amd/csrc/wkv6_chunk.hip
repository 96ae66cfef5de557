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
// hi = bf16(x), lo = bf16(x - hi) and the product uses hi*hi + hi*lo + lo*hi (v, gy are exact in
// bf16 and need no split), which keeps ~16 mantissa bits per operand -- far below the bf16
// rounding of the outputs, which is the error the original fp32 kernels have.
//
// Forward: one workgroup of 4 waves per (batch, head); wave q owns value channels [16q, 16q+16):
// its slice of the state lives in 16 accumulator VGPRs as S^T[j][i] (4 tiles of 16 j), and the
// accumulator layout of a 16x16 tile (lane = column i, lane group g and register v = row 4g+v)
// is used AS IS as the B operand of the next chunk's Rs S0^T product: the K slots of an MFMA may
// be any permutation as long as A uses the same one, so operands that multiply the state are
// stored in LDS with their 64 channels permuted (`perm64`) and no transpose is ever needed.
#include "common.h"

namespace rwkv {
namespace {

constexpr int N = 64;
constexpr int L = 32;             // chunk length
constexpr int NW = 4;
constexpr int NT = NW * 64;
constexpr int RS = 72;            // row stride (bf16 elements) of [token][channel] operand arrays: 144 B
constexpr int TS = 40;            // row stride (bf16 elements) of [channel][token] operand arrays:  80 B
constexpr float RANGE_LIMIT = 60.0f;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

enum { W_EW = 1, W_RAW = 2 };     // wkv6: fp32 ew = -exp(w_raw) [B,T,C];  wkv6_state: raw bf16 w

struct ArgsC {
    int T, C, H;
    const uint16_t *r, *k, *v, *u, *s0;
    const void* w;
    uint16_t* y;
};

// position of channel j inside a stored row: j = 32*ks + 16*h + 4*g + e  ->  32*ks + 8*g + 4*h + e, so that the
// eight K slots of lane group g (16 B) are the channels held by accumulator tiles 2ks and 2ks+1, rows 4g..4g+3
DEVINL int perm64(int j) { return (j & 32) | ((j & 12) << 1) | ((j & 16) >> 2) | (j & 3); }

DEVINL uint16_t bfbits(float x) { return __builtin_bit_cast(uint16_t, static_cast<__bf16>(x)); }
DEVINL void split(float x, uint16_t& hi, uint16_t& lo) {
    const __bf16 h = static_cast<__bf16>(x);
    hi = __builtin_bit_cast(uint16_t, h);
    lo = bfbits(x - static_cast<float>(h));
}
DEVINL void split8(const float (&x)[8], bf16x8& hi, bf16x8& lo) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const __bf16 h = static_cast<__bf16>(x[e]);
        hi[e] = h;
        lo[e] = static_cast<__bf16>(x[e] - static_cast<float>(h));
    }
}
DEVINL bf16x8 lds8(const uint16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
DEVINL f32x4 mfma(bf16x8 a, bf16x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
// a (hi,lo) x b (hi,lo), dropping lo*lo
DEVINL f32x4 mfma3(bf16x8 ah, bf16x8 al, bf16x8 bh, bf16x8 bl, f32x4 c) {
    c = mfma(ah, bh, c);
    c = mfma(ah, bl, c);
    return mfma(al, bh, c);
}
DEVINL float wave_sum(float x) {
    x += __shfl_xor(x, 1, 64);
    x += __shfl_xor(x, 2, 64);
    x += __shfl_xor(x, 4, 64);
    x += __shfl_xor(x, 8, 64);
    return allreduce_rows(x);
}

struct alignas(16) SmemFwd {
    uint16_t Rs_hi[L][RS], Rs_lo[L][RS];     // r e^{c_t}               [t][perm j]  A operand of  Rs S0^T
    uint16_t Rp_hi[L][RS], Rp_lo[L][RS];     // r e^{c_t - c_m}         [t][perm j]  A operand of  A = R' K'^T
    uint16_t Kp_hi[L][RS], Kp_lo[L][RS];     // k e^{c_m - c_{t+1}}     [s][perm j]  B operand of  A
    uint16_t Ke_hi[N][TS], Ke_lo[N][TS];     // k e^{c_L - c_{s+1}}     [j][s]       A operand of  S^T += Ke^T V
    uint16_t Vt[N][TS];                      // v                       [i][s]       B operand
    uint16_t Am_hi[L][TS], Am_lo[L][TS];     // A                       [t][s]       A operand of  A V
    float raw[3][L][N];                      // exact path only: r, k, decay as fp32 [t][j]
    float dec[N];                            // e^{c_L}[j]
    float ruk[L];                            // sum_j r u k
    float part[4][N];                        // sum of lam over each quarter of the chunk
    float Y[L][N + 4];                       // output staging
    int exact;                               // chunk must be redone step by step
};

template <int WMODE>
__global__ __launch_bounds__(NT) void wkv6_fwd_chunk(const ArgsC a) {
    __shared__ SmemFwd S;
    const int tid = threadIdx.x, lane = tid & 63, q = tid >> 6, l16 = lane & 15, g = lane >> 4;
    const int b = blockIdx.x / a.H, h = blockIdx.x % a.H;
    const int T = a.T, C = a.C;
    const size_t base = static_cast<size_t>(b) * T * C + static_cast<size_t>(h) * N;
    const size_t bh = static_cast<size_t>(b) * a.H + h;
    // prep coordinates: channel pj (key channel for r,k,w; value channel for v), quarter pq of the chunk
    const int pj = lane, pq = q, pp = perm64(pj);
    const float uj = bf2f(a.u[h * N + pj]);

    // state slice S^T[j][i], i = 16q + l16:  D[mt][v] <-> j = 16 mt + 4 g + v
    f32x4 D[4];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) D[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (a.s0 != nullptr) {
        const uint16_t* s = a.s0 + (bh * N + q * 16 + l16) * N;
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) {
            const uint2 x = *reinterpret_cast<const uint2*>(s + 16 * mt + 4 * g);
            D[mt] = f32x4{bf_lo(x.x), bf_hi(x.x), bf_lo(x.y), bf_hi(x.y)};
        }
    }
    // the upper-right 16x16 tile of A (t < 16 <= s) is never written: keep it zero
    for (int i = tid; i < L * TS; i += NT) { (&S.Am_hi[0][0])[i] = 0; (&S.Am_lo[0][0])[i] = 0; }
    if (tid == 0) S.exact = 0;

    const int nchunks = (T + L - 1) / L;
    // raw bits of the next chunk, converted only when the chunk is prepared so that the loads stay in flight
    uint16_t qr[8], qk[8], pv[8];
    uint32_t qw[8];
    auto prefetch = [&](int c) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int t = c * L + 8 * pq + e;
            const size_t o = base + static_cast<size_t>(t < T ? t : T - 1) * C + pj;
            qr[e] = a.r[o];
            qk[e] = a.k[o];
            pv[e] = a.v[o];
            if constexpr (WMODE == W_RAW) qw[e] = static_cast<const uint16_t*>(a.w)[o];
            else qw[e] = static_cast<const uint32_t*>(a.w)[o];
        }
    };
    prefetch(0);

    for (int c = 0; c < nchunks; ++c) {
        const int c0 = c * L;
        // ------------------------------------------------------------------ prep (thread = channel pj, quarter pq)
        float pr[8], pk[8], plam[8];
        float cs[8];                                   // inclusive sums inside the quarter
        {
            float s = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const bool ok = (c0 + 8 * pq + e) < T;     // rows past T: no input, no decay
                pr[e] = ok ? bf2f(qr[e]) : 0.f;
                pk[e] = ok ? bf2f(qk[e]) : 0.f;
                if (!ok) pv[e] = 0;
                float lam;
                if constexpr (WMODE == W_RAW) lam = -__expf(bf2f(static_cast<uint16_t>(qw[e])));
                else lam = __uint_as_float(qw[e]);
                plam[e] = ok ? lam : 0.f;
                s += plam[e];
                cs[e] = s;
            }
        }
        __syncthreads();                               // previous chunk is done with LDS
        S.part[pq][pj] = cs[7];
        __syncthreads();
        const float p0 = S.part[0][pj], p1 = S.part[1][pj], p2 = S.part[2][pj], p3 = S.part[3][pj];
        const float cm = p0 + p1, cl = cm + (p2 + p3);
        const float pre = (pq == 0) ? 0.f : (pq == 1) ? p0 : (pq == 2) ? cm : cm + p2;
        if (-cm > RANGE_LIMIT || (cm - cl) > RANGE_LIMIT) S.exact = 1;
        const float d1 = __expf(cm), d2 = __expf(cl - cm);
        if (pq == 0) S.dec[pj] = __expf(cl);
        {
            uint16_t keh[8], kel[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int t = 8 * pq + e;
                const float ct = pre + (e == 0 ? 0.f : cs[e - 1]), ct1 = pre + cs[e];
                const float rp = pr[e] * __expf(ct - cm);
                const float kp = pk[e] * __expf(cm - ct1);
                uint16_t hi, lo;
                split(rp, hi, lo);       S.Rp_hi[t][pp] = hi; S.Rp_lo[t][pp] = lo;
                split(rp * d1, hi, lo);  S.Rs_hi[t][pp] = hi; S.Rs_lo[t][pp] = lo;
                split(kp, hi, lo);       S.Kp_hi[t][pp] = hi; S.Kp_lo[t][pp] = lo;
                split(kp * d2, keh[e], kel[e]);
                const float ruk = wave_sum(pr[e] * uj * pk[e]);
                if (lane == 0) S.ruk[t] = ruk;
                S.raw[0][t][pj] = pr[e];
                S.raw[1][t][pj] = pk[e];
                S.raw[2][t][pj] = __expf(plam[e]);
            }
            auto pack = [](const uint16_t (&x)[8]) {
                auto two = [](uint16_t lo, uint16_t hi) { return static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16); };
                return make_uint4(two(x[0], x[1]), two(x[2], x[3]), two(x[4], x[5]), two(x[6], x[7]));
            };
            *reinterpret_cast<uint4*>(&S.Ke_hi[pj][8 * pq]) = pack(keh);
            *reinterpret_cast<uint4*>(&S.Ke_lo[pj][8 * pq]) = pack(kel);
            *reinterpret_cast<uint4*>(&S.Vt[pj][8 * pq]) = pack(pv);
        }
        __syncthreads();
        if (c + 1 < nchunks) prefetch(c + 1);          // global loads fly while the matrix cores work
        const bool exact = S.exact != 0;

        f32x4 Y[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
        if (!exact) {
            // -------------------------------------------------------------- A tiles (waves 0..2)
            if (q < 3) {
                const int ta = (q == 0) ? 0 : 1, tb = (q == 2) ? 1 : 0;          // (0,0) (1,0) (1,1)
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const int o = 32 * ks + 8 * g;
                    acc = mfma3(lds8(&S.Rp_hi[16 * ta + l16][o]), lds8(&S.Rp_lo[16 * ta + l16][o]),
                                lds8(&S.Kp_hi[16 * tb + l16][o]), lds8(&S.Kp_lo[16 * tb + l16][o]), acc);
                }
#pragma unroll
                for (int v = 0; v < 4; ++v) {                                   // row t = 4g+v, column s = l16
                    const int tl = 4 * g + v;
                    float x = acc[v];
                    if (ta == tb) x = (l16 < tl) ? x : (l16 == tl ? S.ruk[16 * ta + tl] : 0.f);
                    uint16_t hi, lo;
                    split(x, hi, lo);
                    S.Am_hi[16 * ta + tl][16 * tb + l16] = hi;
                    S.Am_lo[16 * ta + tl][16 * tb + l16] = lo;
                }
            }
            // -------------------------------------------------------------- Y = Rs S0^T
            {
                bf16x8 sh[2], sl[2];
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const float x[8] = {D[2 * ks][0], D[2 * ks][1], D[2 * ks][2], D[2 * ks][3],
                                        D[2 * ks + 1][0], D[2 * ks + 1][1], D[2 * ks + 1][2], D[2 * ks + 1][3]};
                    split8(x, sh[ks], sl[ks]);
                }
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) {
                        const int o = 32 * ks + 8 * g;
                        Y[mt] = mfma3(lds8(&S.Rs_hi[16 * mt + l16][o]), lds8(&S.Rs_lo[16 * mt + l16][o]), sh[ks], sl[ks], Y[mt]);
                    }
            }
            __syncthreads();                           // A is in LDS
            // -------------------------------------------------------------- Y += A V ;  S^T = S^T diag(dec) + Ke^T V
            const bf16x8 vb = lds8(&S.Vt[16 * q + l16][8 * g]);
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) {
                Y[mt] = mfma(lds8(&S.Am_hi[16 * mt + l16][8 * g]), vb, Y[mt]);
                Y[mt] = mfma(lds8(&S.Am_lo[16 * mt + l16][8 * g]), vb, Y[mt]);
            }
#pragma unroll
            for (int mt = 0; mt < 4; ++mt) {
                const float4 dj = *reinterpret_cast<const float4*>(&S.dec[16 * mt + 4 * g]);
                f32x4 x = {D[mt][0] * dj.x, D[mt][1] * dj.y, D[mt][2] * dj.z, D[mt][3] * dj.w};
                x = mfma(lds8(&S.Ke_hi[16 * mt + l16][8 * g]), vb, x);
                D[mt] = mfma(lds8(&S.Ke_lo[16 * mt + l16][8 * g]), vb, x);
            }
        } else {
            // -------------------------------------------------------------- exact path: 32 sequential steps
            // lane (i = 16q + l16, group g) holds S[i][j] for j = 16 mt + 4 g + v
            for (int t = 0; t < L; ++t) {
                const float vi = bf2f(S.Vt[16 * q + l16][t]);
                float yp = 0.f;
#pragma unroll
                for (int mt = 0; mt < 4; ++mt) {
                    const float4 rr = *reinterpret_cast<const float4*>(&S.raw[0][t][16 * mt + 4 * g]);
                    const float4 kk = *reinterpret_cast<const float4*>(&S.raw[1][t][16 * mt + 4 * g]);
                    const float4 ww = *reinterpret_cast<const float4*>(&S.raw[2][t][16 * mt + 4 * g]);
                    yp = fmaf(rr.x, D[mt][0], yp); yp = fmaf(rr.y, D[mt][1], yp);
                    yp = fmaf(rr.z, D[mt][2], yp); yp = fmaf(rr.w, D[mt][3], yp);
                    D[mt][0] = fmaf(D[mt][0], ww.x, kk.x * vi); D[mt][1] = fmaf(D[mt][1], ww.y, kk.y * vi);
                    D[mt][2] = fmaf(D[mt][2], ww.z, kk.z * vi); D[mt][3] = fmaf(D[mt][3], ww.w, kk.w * vi);
                }
                const float y = allreduce_rows(yp) + S.ruk[t] * vi;
                if (g == 0) S.Y[t][16 * q + l16] = y;
            }
            __syncthreads();                           // keeps the barrier count equal on both paths
        }
        if (!exact) {
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int v = 0; v < 4; ++v) S.Y[16 * mt + 4 * g + v][16 * q + l16] = Y[mt][v];
        }
        __syncthreads();
        if (tid == 0) S.exact = 0;                     // read by everyone before the barrier above
        {
            const int t = tid >> 3, i0 = (tid & 7) * 8;
            if (c0 + t < T) {
                const float4 x0 = *reinterpret_cast<const float4*>(&S.Y[t][i0]);
                const float4 x1 = *reinterpret_cast<const float4*>(&S.Y[t][i0 + 4]);
                const float f[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
                *reinterpret_cast<uint4*>(a.y + base + static_cast<size_t>(c0 + t) * C + i0) = pack8(f);
            }
        }
    }
}

}  // namespace

// Launchers used by wkv56.hip's entry points.
int launch_wkv6_fwd_chunk(hipStream_t st, int wmode, int B, int T, int C, int H, const uint16_t* r,
                          const uint16_t* k, const uint16_t* v, const void* w, const uint16_t* u,
                          const uint16_t* s0, uint16_t* y) {
    ArgsC a{};
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.s0 = s0; a.y = y;
    if (wmode == W_RAW) hipLaunchKernelGGL(wkv6_fwd_chunk<W_RAW>, dim3(B * H), dim3(NT), 0, st, a);
    else hipLaunchKernelGGL(wkv6_fwd_chunk<W_EW>, dim3(B * H), dim3(NT), 0, st, a);
    return launch_status();
}

}  // namespace rwkv
