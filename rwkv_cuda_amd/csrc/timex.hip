// depthwise_conv1d ("TimeX"): causal depthwise convolution with a full-length (T-tap) kernel
// per channel, fp32, gfx950.
//
//   x[b,c,t]  = eps + sum_{u<=t} wr[t-u] k[b,c,u]            wr[d] = w[c, T-1-d]
//   gk[b,c,u] =       sum_{t>=u} wr[t-u] g[b,c,t]
//   gw[b,c,T-1-d] =   sum_{u}    g[b,c,u+d] k[b,c,u]         (per batch; the wrapper sums over b)
//
// conv / corr kernels: one workgroup per (channel, group of BB batch rows).  The reversed
// kernel row wr (with four leading zeros, so taps of negative lag read 0 and the diagonal block
// needs no mask) and the BB input rows sit in LDS; a thread owns 4 consecutive outputs for all
// BB rows and walks the lags 4 at a time: two 16-byte LDS reads give the 7 taps it needs, one
// broadcast 16-byte read per row gives the inputs, 16 FMAs per row follow.
// gw kernel: one workgroup per (b,c) row; a thread owns 4 consecutive lags d.
#include "common.h"

namespace rwkv {
namespace {

constexpr int BB = 8;

// MIRROR = false: out[t] = eps + sum_{u<=t} wr[t-u] in[u]      (forward)
// MIRROR = true : out[u] =       sum_{t>=u} wr[t-u] in[t]      (gk)
template <bool MIRROR>
__global__ __launch_bounds__(1024) void timex_conv(const float* __restrict__ w, const float* __restrict__ in,
                                                  float* __restrict__ out, float eps, int B, int C, int T) {
    extern __shared__ float lds[];
    float* wr = lds;                 // [T + 4], wr[4 + d] = w[c][T-1-d], wr[0..3] = 0
    float* rows = lds + T + 4;       // [BB][T]
    const int c = blockIdx.x, b0 = blockIdx.y * BB, tid = threadIdx.x;
    const int nthr = T >> 2;

    for (int i = tid; i < 4; i += nthr) wr[i] = 0.f;
    for (int d = tid; d < T; d += nthr) wr[4 + d] = w[static_cast<size_t>(c) * T + (T - 1 - d)];
#pragma unroll
    for (int r = 0; r < BB; ++r) {
        const int b = b0 + r;
        float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
        if (b < B) x = *reinterpret_cast<const float4*>(in + (static_cast<size_t>(b) * C + c) * T + 4 * tid);
        *reinterpret_cast<float4*>(rows + r * T + 4 * tid) = x;
    }
    __syncthreads();

    const int o0 = 4 * tid;          // first output index of this thread
    float acc[BB][4];
#pragma unroll
    for (int r = 0; r < BB; ++r)
#pragma unroll
        for (int a = 0; a < 4; ++a) acc[r][a] = MIRROR ? 0.f : eps;

    const int lo = MIRROR ? o0 : 0, hi = MIRROR ? T - 4 : o0;
    for (int s4 = lo; s4 <= hi; s4 += 4) {
        const int d0 = MIRROR ? s4 - o0 : o0 - s4;                   // >= 0, multiple of 4
        const float4 wl = *reinterpret_cast<const float4*>(wr + d0);       // lags d0-4 .. d0-1
        const float4 wh = *reinterpret_cast<const float4*>(wr + d0 + 4);   // lags d0   .. d0+3
        const float wv[8] = {wl.x, wl.y, wl.z, wl.w, wh.x, wh.y, wh.z, wh.w};
#pragma unroll
        for (int r = 0; r < BB; ++r) {
            const float4 x4 = *reinterpret_cast<const float4*>(rows + r * T + s4);
            const float xv[4] = {x4.x, x4.y, x4.z, x4.w};
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    // forward: lag = (o0+a) - (s4+e) = d0 + a - e;  mirror: lag = (s4+e) - (o0+a) = d0 + e - a
                    acc[r][a] = fmaf(wv[4 + (MIRROR ? e - a : a - e)], xv[e], acc[r][a]);
        }
    }
#pragma unroll
    for (int r = 0; r < BB; ++r) {
        const int b = b0 + r;
        if (b < B)
            *reinterpret_cast<float4*>(out + (static_cast<size_t>(b) * C + c) * T + o0) =
                make_float4(acc[r][0], acc[r][1], acc[r][2], acc[r][3]);
    }
}

// gw[row][T-1-d] = sum_u g[row][u+d] k[row][u]
__global__ __launch_bounds__(1024) void timex_gw(const float* __restrict__ k, const float* __restrict__ g,
                                                float* __restrict__ gw, int T) {
    extern __shared__ float lds[];
    float* ks = lds;                 // [T]
    float* gs = lds + T;             // [T + 4], four trailing zeros
    const size_t row = blockIdx.x;
    const int tid = threadIdx.x;
    *reinterpret_cast<float4*>(ks + 4 * tid) = *reinterpret_cast<const float4*>(k + row * T + 4 * tid);
    *reinterpret_cast<float4*>(gs + 4 * tid) = *reinterpret_cast<const float4*>(g + row * T + 4 * tid);
    for (int i = tid; i < 4; i += (T >> 2)) gs[T + i] = 0.f;
    __syncthreads();

    const int d0 = 4 * tid;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int u4 = 0; u4 + d0 < T; u4 += 4) {
        const float4 k4 = *reinterpret_cast<const float4*>(ks + u4);
        const float4 g0 = *reinterpret_cast<const float4*>(gs + u4 + d0);
        const float4 g1 = *reinterpret_cast<const float4*>(gs + u4 + d0 + 4);
        const float kv[4] = {k4.x, k4.y, k4.z, k4.w};
        const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[a] = fmaf(gv[e + a], kv[e], acc[a]);   // g[u4+e + d0+a] k[u4+e]
    }
    // lags d0..d0+3 live at taps T-1-d0 .. T-4-d0
    *reinterpret_cast<float4*>(gw + row * T + (T - 4 - d0)) = make_float4(acc[3], acc[2], acc[1], acc[0]);
}

// ---------------------------------------------------------------------------------------------------- matrix-core path
// For T a multiple of 32 (and short enough for 32 rows to sit in LDS) the convolution of 32 batch rows of one channel is a
// product of the lower-triangular Toeplitz matrix W[t][u] = wr[t-u] with the [T x 32] block of inputs, on 32 x 32 matrix
// instructions (accumulator register v of lane l: row 8 (v/4) + 4 (l>>5) + (v&3), column l & 31).  The kernel row is
// followed by zeros, so a tap of negative lag reads 0 and the diagonal block needs no mask.  Output tile o of 32 time
// steps sums over input tiles 0..o (mirror: o..T/32-1); the tiles are dealt to the eight waves so that their loads are
// about equal.  256 persistent workgroups; a unit is one channel x 32 batch rows, and the next unit's rows are
// loaded into registers under the products of the current one.
typedef float f32x16 __attribute__((ext_vector_type(16)));
constexpr int MROWS = 32;              // batch rows per workgroup = columns of the product
constexpr int T_MFMA_MAX = 1024;
constexpr int TXW = 8;                 // waves per workgroup: two per SIMD, one reads LDS while the other runs MFMAs
constexpr int TXT = 64 * TXW;
constexpr int NCU = 256;               // workgroups of the persistent kernels: one per CU

// ------------------------------------------------------------------------------------ fp32 accuracy from fp16 x 2 products
// Every fp32 operand x is cut into two fp16 terms, x 2^s = h + l (h the nearest fp16, l the nearest fp16 of what h
// leaves: 22 mantissa bits together), and
//     x y = (h h' + h l' + l h') 2^-(s+s')                    (the term left out is below 2^-22 of the product)
// on v_mfma_f32_32x32x16_f16: three instructions of 16 matrix passes where v_mfma_f32_32x32x2_f32 needs eight of 16 passes
// for the same 32 x 32 x 16 block, i.e. 5.3 times the arithmetic rate at fp32 accuracy (accumulation is fp32 either way).
// fp16 has five exponent bits: the power of two 2^s brings the largest magnitude of a unit's rows (and of the kernel row)
// to [2^14, 2^15), computed for every unit from the rows themselves.  Elements more than 2^28 below that lose bits (fp16
// subnormals: absolute error 2^-25 on that scale, 2^-40 of the largest element), which a sum that contains the large
// elements does not see; the accumulators are scaled back exactly.
// Operand layout of the instruction: lane = (row or column l & 31, K half l >> 5) holds the eight consecutive K slots
// 8 (l >> 5) .. + 7; accumulator as above.  K slot s of a step is input step 16 ks + s of the 32-step tile.
//   rows : two planes [32 batch rows][T + 16] fp16; a lane's eight slots are 16 aligned bytes.
//   taps : the A operand of row t and slot u is line[base(t) + u] for a line that depends only on the direction
//          (forward: the kernel row in tap order followed by zeros; mirror: 31 zeros, then the reversed kernel row), so a
//          lane reads eight consecutive bf16 starting at an arbitrary element.  Two copies of every plane, the second
//          shifted by one element, make that four aligned dwords whatever the parity of the start.
// LDS: 2 x 32 x (T + 16) x 2 + 4 x (T + 96) x 2 + 64 bytes = 142 144 of 163 840 at T = 1024, the longest T this form takes.
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
constexpr int T_H2_MAX = 1024;
constexpr int T_H2_MID = 768;          // up to here a lane holds 3 pieces (16 bytes each) of each of its four rows while they are in flight, beyond 4
__host__ __device__ inline int h2_row_stride(int T) { return T + 16; }           // elements; (T + 16) / 2 dwords = 8 or 24 mod 32
__host__ __device__ inline int h2_line_len(int T) { return T + ((T & 32) ? 64 : 96); }    // half of it = 16 mod 32 dwords: the shifted copy sits 16 banks away
__host__ __device__ inline size_t h2_lds_bytes(int T) {
    return (2 * static_cast<size_t>(MROWS) * h2_row_stride(T) + 4 * static_cast<size_t>(h2_line_len(T))) * sizeof(uint16_t) + 16 * sizeof(float);
}
// x (already scaled) = h + l: h the nearest fp16, l the nearest fp16 of the exact remainder
struct H2 { uint16_t h, l; };
DEVINL H2 split2(float x) {
    const _Float16 h = static_cast<_Float16>(x);
    const _Float16 l = static_cast<_Float16>(x - static_cast<float>(h));
    H2 r;
    r.h = __builtin_bit_cast(uint16_t, h);
    r.l = __builtin_bit_cast(uint16_t, l);
    return r;
}
// the same for four elements times a power of two (the scaling is exact, so the remainder may be formed from x up in one
// fused operation): four multiplications, four fused multiply-adds and four packed conversions
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
struct H2x4 { uint2 h, l; };
DEVINL H2x4 split2x4(const float4& v, const float up) {
    const f32x2 a = {v.x * up, v.y * up}, b = {v.z * up, v.w * up};
    const f16x2 ha = __builtin_convertvector(a, f16x2), hb = __builtin_convertvector(b, f16x2);
    const f32x2 ra = a - __builtin_convertvector(ha, f32x2), rb = b - __builtin_convertvector(hb, f32x2);
    const f16x2 la = __builtin_convertvector(ra, f16x2), lb = __builtin_convertvector(rb, f16x2);
    H2x4 r;
    r.h = make_uint2(__builtin_bit_cast(uint32_t, ha), __builtin_bit_cast(uint32_t, hb));
    r.l = make_uint2(__builtin_bit_cast(uint32_t, la), __builtin_bit_cast(uint32_t, lb));
    return r;
}
// 2^s with m 2^s in [2^14, 2^15) for a magnitude m (s = 0 for zero, subnormal or infinite m), and 2^-s
struct Pow2 { float up, down; };
DEVINL Pow2 scale_for(float m) {
    const int e = static_cast<int>((__float_as_uint(m) >> 23) & 255u);
    int sft = 14 + 127 - e;
    sft = sft < -100 ? -100 : (sft > 100 ? 100 : sft);
    if (e == 0 || e == 255) sft = 0;
    Pow2 r;
    r.up = __uint_as_float(static_cast<uint32_t>(127 + sft) << 23);
    r.down = __uint_as_float(static_cast<uint32_t>(127 - sft) << 23);
    return r;
}
DEVINL float wave_max(float m) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    return m;
}
DEVINL float max_abs4(float m, const float4& v) { return fmaxf(fmaxf(m, fmaxf(fabsf(v.x), fabsf(v.y))), fmaxf(fabsf(v.z), fabsf(v.w))); }

// NI: 16-byte pieces of a row per lane, 64 lanes a row: 3 up to T = 768, 4 beyond
template <bool MIRROR, int NI>
__global__ __launch_bounds__(TXT) void timex_conv_h2(const float* __restrict__ w, const float* __restrict__ in,
                                                      float* __restrict__ out, float eps, int B, int C, int T) {
    extern __shared__ float lds[];
    const int rs = h2_row_stride(T), xl = h2_line_len(T);
    uint16_t* rp = reinterpret_cast<uint16_t*>(lds);                    // [2][32][rs]
    uint16_t* al = rp + 2 * MROWS * rs;                                 // [2 planes][2 copies][xl]
    float* red = reinterpret_cast<float*>(al + 4 * xl);                 // [2][8]: every wave's largest magnitude of the rows / of the kernel row
    const int tid = threadIdx.x, lane = tid & 63, wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ln = lane & 31, kh = lane >> 5;
    const int q4n = T >> 2, nt = T >> 5;
    const int nbg = (B + MROWS - 1) / MROWS, nunits = C * nbg;
    // Staging: wave wv takes rows 4 wv .. 4 wv + 3 of the unit, lane l the 16-byte pieces l, l + 64, ... of each: a row's
    // address is wave-uniform, the rest is the lane number times 16 and a constant, in global memory and in LDS alike.
    float4 x[4][NI];
    float wr[2];
    // (in NI parts, piece i of the four rows each, the kernel row with part 0: asked for all at once by every workgroup of
    //  the chip at the same moment, the loads queue up in the memory system and the waves stall issuing them; the parts
    //  are spread over the products of the unit before)
    auto fetch_part = [&](const int unit, const int i) __attribute__((always_inline)) {
        const int c = unit / nbg, b0 = (unit - c * nbg) * MROWS;
        const int q4 = min(lane + 64 * i, q4n - 1);
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            // (a row past the batch is read as the batch's last row and counts as zero later)
            const int b = min(b0 + 4 * wv + rr, B - 1);
            x[rr][i] = *reinterpret_cast<const float4*>(in + (static_cast<size_t>(b) * C + c) * T + 4 * q4);
        }
        if (i == 0) {
#pragma unroll
            for (int s = 0; s < 2; ++s) wr[s] = w[static_cast<size_t>(c) * T + min(s * TXT + tid, T - 1)];
        }
    };
    // the largest magnitudes of the unit, this wave's part (pieces past a row's end repeat its last piece)
    auto unit_max = [&]() __attribute__((always_inline)) {
        float mx = 0.f;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr)
#pragma unroll
            for (int i = 0; i < NI; ++i) mx = max_abs4(mx, x[rr][i]);
        mx = wave_max(mx);
        const float mw = wave_max(fmaxf(fabsf(wr[0]), fabsf(wr[1])));
        if (lane == 0) { red[wv] = mx; red[8 + wv] = mw; }
    };
    float unscale = 1.f;
    auto store_unit = [&](const int unit) __attribute__((always_inline)) {
        const int c = unit / nbg, b0 = (unit - c * nbg) * MROWS;
        float mx = 0.f, mw = 0.f;
#pragma unroll
        for (int i = 0; i < TXW; ++i) { mx = fmaxf(mx, red[i]); mw = fmaxf(mw, red[8 + i]); }
        const Pow2 sx = scale_for(mx), sw = scale_for(mw);
        unscale = sx.down * sw.down;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const int r = 4 * wv + rr;
            const float up = b0 + r < B ? sx.up : 0.f;
            uint16_t* d = rp + r * rs + 4 * lane;
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                if (lane + 64 * i < q4n) {
                    const H2x4 y = split2x4(x[rr][i], up);
                    *reinterpret_cast<uint2*>(d + 256 * i) = y.h;
                    *reinterpret_cast<uint2*>(d + 256 * i + MROWS * rs) = y.l;
                }
            }
        }
        // tap tau of the kernel row sits at line position tau (forward) or 31 + (T - 1 - tau) (mirror); the rest is zero
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int tau = s * TXT + tid;
            if (tau < T) {
                const H2 a = split2(wr[s] * sw.up);
                const int pos = MIRROR ? 31 + (T - 1 - tau) : tau;
                const uint16_t pl[2] = {a.h, a.l};
#pragma unroll
                for (int p = 0; p < 2; ++p) {
                    al[(2 * p) * xl + pos] = pl[p];
                    if (pos >= 1) al[(2 * p + 1) * xl + pos - 1] = pl[p];
                }
            }
        }
        (void)c;
    };
    // the zero parts of the line never change: clear everything once (the taps are rewritten for every unit)
    for (int i = tid; i < 4 * xl; i += TXT) al[i] = 0;
    __syncthreads();
    int unit = blockIdx.x;
    if (unit < nunits) {
#pragma unroll
        for (int i = 0; i < NI; ++i) fetch_part(unit, i);
    }
    static_assert(T_H2_MAX / 64 <= 2 * TXW, "a wave takes at most two pairs of tiles per unit");

    for (; unit < nunits; unit += gridDim.x) {
        const int c = unit / nbg, b0 = (unit - c * nbg) * MROWS;
        unit_max();
        __syncthreads();
        store_unit(unit);
        __syncthreads();
        const int next = unit + static_cast<int>(gridDim.x);
        const bool more = next < nunits;
        if (more) fetch_part(next, 0);
        // Output tile ot sums over ot + 1 input tiles (mirror: T/32 - ot).  A wave works on two neighbouring output tiles at a
        // time, because they share operands: a step is 16 input steps (K = 16), and with
        //   forward: row t = 32 ot + ln, slot u: tap T-1-(t-u)            -> line[T-1-32 ot-ln + u],  rows[u]
        //   mirror : row u = 32 ot + ln, slot t: lag 32 (it-ot) + slot-ln -> line[31-ln + 32 (it-ot) + slot],  rows[32 ot + slot]
        // step j of both tiles takes the same rows (forward) or the same taps (mirror), and the other operand of the
        // shorter tile at step j is that of the longer one (forward: tile ot + 1, mirror: tile ot) at step j + 2.  So a
        // step reads one operand of each kind from LDS (4 KB per wave) for six matrix instructions instead of three: the
        // "carried" operand C(j) enters the shorter tile at once and the longer tile two steps later, from registers.
        // The pairs are dealt to the waves in the order of decreasing work, back and forth (waves 0..7, then 7..0): at most
        // two pairs a wave.
        const int npairs = (nt + 1) >> 1;
        auto do_pair = [&](const int ts, auto&& halfway) __attribute__((always_inline)) {
            {
                const int m = MIRROR ? ts : npairs - 1 - ts;
                // the longer tile and the shorter one (absent when T/32 is odd and this is the last tile)
                const bool both = 2 * m + 1 < nt;
                const int tl = MIRROR ? 2 * m : (both ? 2 * m + 1 : 2 * m), tsh = MIRROR ? 2 * m + 1 : 2 * m;
                const int n_long = 2 * (MIRROR ? nt - tl : tl + 1), n_short = n_long - 2;
                f32x16 accl, accs;                             // the two tiles' instructions alternate: consecutive ones are independent
#pragma unroll
                for (int v = 0; v < 16; ++v) { accl[v] = 0.f; accs[v] = 0.f; }
                const int start0 = (MIRROR ? 31 - ln : T - 1 - 32 * tl - ln) + 8 * kh;
                const uint32_t* ap0 = reinterpret_cast<const uint32_t*>(al + (start0 & 1) * xl) + (start0 >> 1);
                const uint16_t* bp0 = rp + ln * rs + (MIRROR ? 32 * tl : 0) + 8 * kh;
                auto taps = [&](int j, f16x8 (&f)[2]) __attribute__((always_inline)) {
#pragma unroll
                    for (int pq = 0; pq < 2; ++pq) {
                        const uint32_t* a4 = ap0 + 8 * j + pq * xl;    // a plane is 2 xl elements = xl dwords
                        f[pq] = __builtin_bit_cast(f16x8, make_uint4(a4[0], a4[1], a4[2], a4[3]));
                    }
                };
                auto rows = [&](int j, f16x8 (&f)[2]) __attribute__((always_inline)) {
#pragma unroll
                    for (int pq = 0; pq < 2; ++pq) f[pq] = __builtin_bit_cast(f16x8, *reinterpret_cast<const uint4*>(bp0 + 16 * j + pq * MROWS * rs));
                };
                auto carried = [&](int j, f16x8 (&f)[2]) __attribute__((always_inline)) { if constexpr (MIRROR) rows(j, f); else taps(j, f); };
                auto shared = [&](int j, f16x8 (&f)[2]) __attribute__((always_inline)) { if constexpr (MIRROR) taps(j, f); else rows(j, f); };
                // term number `term` of the product of a carried and a shared operand: h h', h l', l h'
                auto product = [&](f32x16& acc, const int term, const f16x8 (&cc)[2], const f16x8 (&sh)[2]) __attribute__((always_inline)) {
                    const f16x8 (&fa)[2] = MIRROR ? sh : cc;
                    const f16x8 (&fb)[2] = MIRROR ? cc : sh;
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[term == 2 ? 1 : 0], fb[term == 1 ? 1 : 0], acc, 0, 0, 0);
                };
                // (a last tile without a partner computes a second tile all the same and does not store it)
                auto step = [&](const f16x8 (&cl)[2], const f16x8 (&cs)[2], const f16x8 (&sh)[2]) __attribute__((always_inline)) {
#pragma unroll
                    for (int term = 0; term < 3; ++term) { product(accl, term, cl, sh); product(accs, term, cs, sh); }
                };
                // Two pairs of carried operands, P and Q, change roles every two steps (the longer tile reads what the shorter
                // one read two steps earlier), the shared operand alternates between two sets: no register is ever copied.
                // Every read is issued one step ahead; the fences keep it in front of the products of the current step.
                // (C(j) is asked for up to j = n_long - 1 only, S(j) likewise: nothing outside the tiles' own steps is read.)
                f16x8 P[2][2], Q[2][2], se[2], so[2];
                carried(0, P[0]); carried(1, P[1]); carried(n_long > 2 ? 2 : 1, Q[0]); shared(0, se);
                // (one way into every loop body and one way out: with an exit in the middle of a body the compiler keeps two
                //  versions of the accumulators and copies all 32 registers between them in every pass of the loop, after waiting for
                //  the matrix pipeline to drain)
                auto block_pq = [&](const int j) __attribute__((always_inline)) {      // steps j, j + 1: longer tile from P, shorter from Q
                    carried(j + 3, Q[1]); shared(j + 1, so);
                    __builtin_amdgcn_sched_barrier(0);
                    step(P[0], Q[0], se);
                    __builtin_amdgcn_sched_barrier(0);
                    carried(min(j + 4, n_long - 1), P[0]); shared(j + 2, se);
                    __builtin_amdgcn_sched_barrier(0);
                    step(P[1], Q[1], so);
                    __builtin_amdgcn_sched_barrier(0);
                };
                auto block_qp = [&](const int j) __attribute__((always_inline)) {      // the same with the roles of P and Q exchanged
                    carried(j + 3, P[1]); shared(j + 1, so);
                    __builtin_amdgcn_sched_barrier(0);
                    step(Q[0], P[0], se);
                    __builtin_amdgcn_sched_barrier(0);
                    carried(min(j + 4, n_long - 1), Q[0]); shared(j + 2, se);
                    __builtin_amdgcn_sched_barrier(0);
                    step(Q[1], P[1], so);
                    __builtin_amdgcn_sched_barrier(0);
                };
                int j = 0;
                const int half = (n_short >> 1) & ~3;
                for (; j < half; j += 4) { block_pq(j); block_qp(j + 2); }
                halfway();
                for (; j + 4 <= n_short; j += 4) { block_pq(j); block_qp(j + 2); }
                if (j < n_short) {                              // (two steps left: afterwards the longer tile's operands are in Q)
                    block_pq(j);
#pragma unroll
                    for (int q = 0; q < 2; ++q) { P[0][q] = Q[0][q]; P[1][q] = Q[1][q]; }
                }
                // the last two steps belong to the longer tile alone
                shared(n_short + 1, so);
#pragma unroll
                for (int term = 0; term < 3; ++term) product(accl, term, P[0], se);
#pragma unroll
                for (int term = 0; term < 3; ++term) product(accl, term, P[1], so);
                auto put_tile = [&](f32x16& acc, const int ot) __attribute__((always_inline)) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[v] = fmaf(acc[v], unscale, MIRROR ? 0.f : eps);
                    if (b0 + ln < B) {
                        float* o = out + (static_cast<size_t>(b0 + ln) * C + c) * T + 32 * ot + 4 * kh;
#pragma unroll
                        for (int v4 = 0; v4 < 4; ++v4)
                            *reinterpret_cast<float4*>(o + 8 * v4) = make_float4(acc[4 * v4], acc[4 * v4 + 1], acc[4 * v4 + 2], acc[4 * v4 + 3]);
                    }
                };
                put_tile(accl, tl);
                if (both) put_tile(accs, tsh);
            }
        };
        if (wv < npairs) do_pair(wv, [&]() __attribute__((always_inline)) { if (more) fetch_part(next, 1); });
        else if (more) fetch_part(next, 1);
        if (more) fetch_part(next, 2);
        if (2 * TXW - 1 - wv < npairs) do_pair(2 * TXW - 1 - wv, []() __attribute__((always_inline)) {});
        if constexpr (NI > 3) { if (more) fetch_part(next, 3); }
        __syncthreads();               // every wave is done with this unit's rows
    }
}

// Kernel gradient summed over the batch: gws[c][T-1-lag] = sum_b sum_t g[b,c,t] k[b,c,t-lag], i.e. the sum of the lag-th
// sub-diagonal of M = G^T K (contraction over the batch), with the two-term fp16 products of timex_conv_h2.  Batch rows
// are staged 16 at a time (a pass; both tensors scaled by a power of two of their own per pass): one
// v_mfma_f32_32x32x16_f16 block per pair of tiles and product, K = the 16 batch rows.  A wave owns whole lag tiles d (all
// tile pairs (d + i, i) accumulate into the same registers); no atomics, every fp32 sum in a fixed order.
// The planes keep the tensors' own layout, [16 rows][T + 16 .. 112] fp16 (staged like the convolution's rows: a wave takes two
// rows of each tensor, wave-uniform row addresses, 8-byte LDS stores).  Both operands need the batch rows along K and a
// lane per step: ds_read_b64_tr_b16 delivers exactly that -- within 16 lanes, four rows of 16 consecutive steps come back
// with a lane per step and the four rows in its registers; two such reads are a lane's eight K slots.
// Two neighbouring lag tiles per wave at a time: tile pair i of lag tile d + 1 takes the same k tile as pair i of lag
// tile d, and its g tile is the one that lag tile d takes at pair i + 1.  So a pair reads one g tile and one k tile
// from LDS for six matrix instructions; the g operand enters lag tile d + 1 at once and lag tile d one pair later.
// A finished tile's diagonals are summed in registers: lane p of a half-wave collects, for every row t it holds, the
// element of column (t - p) mod 32 (one ds_bpermute per accumulator register), which belongs to diagonal p if t >= p and
// to diagonal p - 32 otherwise.
// LDS: 2 x 2 x 16 x (T + 16) x 2 + 2 T x 4 + 64 bytes = 141 376 at T = 1024.
constexpr int GH2_ROWS = 16;
typedef short v4s __attribute__((ext_vector_type(4)));
typedef v4s __attribute__((address_space(3))) * lds_v4s_ptr;
// elements; = 16 mod 128, i.e. 8 banks mod 64: the 16 lanes of a transposing read take four rows x four 8-byte pieces, and
// with rows 8 banks apart the sixteen pieces fall on different banks
__host__ __device__ inline int gw_row_stride(int T) { return T + ((144 - (T & 127)) & 127); }
__host__ __device__ inline size_t gw_h2_lds_bytes(int T) {
    return 4 * static_cast<size_t>(GH2_ROWS) * gw_row_stride(T) * sizeof(uint16_t) + (2 * static_cast<size_t>(T) + 16) * sizeof(float);
}

// NI: 16-byte pieces of a row per lane, 64 lanes a row: 3 up to T = 768, 4 beyond
template <int NI>
__global__ __launch_bounds__(TXT) void timex_gw_sum_h2(const float* __restrict__ k, const float* __restrict__ g,
                                                        float* __restrict__ gws, int B, int C, int T) {
    extern __shared__ float lds[];
    const int rsg = gw_row_stride(T);
    const int plane = GH2_ROWS * rsg;                          // elements
    uint16_t* gp = reinterpret_cast<uint16_t*>(lds);           // [2][16][rsg]
    uint16_t* kp = gp + 2 * plane;                             // [2][16][rsg]
    float* diag = reinterpret_cast<float*>(kp + 2 * plane);    // [T/32 lag tiles][64]: entry l of tile d is the sum for lag 32 d + l - 31
    float* red = diag + 2 * T;                                 // [2][8]: every wave's largest magnitude of g / of k in this pass
    const int tid = threadIdx.x, lane = tid & 63, wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ln = lane & 31, kh = lane >> 5, l16 = lane & 15;
    const int nt = T >> 5, q4n = T >> 2;
    const int npass = (B + GH2_ROWS - 1) / GH2_ROWS;
    const int nmine = (C > static_cast<int>(blockIdx.x) ? (C - 1 - static_cast<int>(blockIdx.x)) / static_cast<int>(gridDim.x) + 1 : 0) * npass;
    // Staging: wave wv takes rows 2 wv and 2 wv + 1 of the pass, of both tensors; lane l the 16-byte pieces l, l + 64, ...
    float4 xg[2][NI], xk[2][NI];
    // (in NI parts, piece i of both rows and both tensors each: asked for all at once by every workgroup of the chip at the
    //  same moment, the loads queue up in the memory system and the waves stall issuing them while the matrix cores wait;
    //  the parts are spread over the products of the pass before)
    const int nblk = gridDim.x;
    auto fetch_part = [&](const int u, const int i) __attribute__((always_inline)) {
        const int c = blockIdx.x + (u / npass) * nblk, b0 = (u % npass) * GH2_ROWS;
        const int q4 = min(lane + 64 * i, q4n - 1);
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
            // (a row past the batch is read as the batch's last row and counts as zero later)
            const size_t row = (static_cast<size_t>(min(b0 + 2 * wv + rr, B - 1)) * C + c) * T;
            xg[rr][i] = *reinterpret_cast<const float4*>(g + row + 4 * q4);
            xk[rr][i] = *reinterpret_cast<const float4*>(k + row + 4 * q4);
        }
    };
    // the largest magnitudes of the pass, this wave's part (pieces past a row's end repeat its last piece)
    auto unit_max = [&]() __attribute__((always_inline)) {
        float mg = 0.f, mk = 0.f;
#pragma unroll
        for (int rr = 0; rr < 2; ++rr)
#pragma unroll
            for (int i = 0; i < NI; ++i) { mg = max_abs4(mg, xg[rr][i]); mk = max_abs4(mk, xk[rr][i]); }
        mg = wave_max(mg); mk = wave_max(mk);
        if (lane == 0) { red[wv] = mg; red[8 + wv] = mk; }
    };
    float unscale = 1.f;
    auto store_unit = [&](const int u) __attribute__((always_inline)) {
        const int b0 = (u % npass) * GH2_ROWS;
        float mg = 0.f, mk = 0.f;
#pragma unroll
        for (int i = 0; i < TXW; ++i) { mg = fmaxf(mg, red[i]); mk = fmaxf(mk, red[8 + i]); }
        const Pow2 sg = scale_for(mg), sk = scale_for(mk);
        unscale = sg.down * sk.down;
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
            const int r = 2 * wv + rr;
            const bool real = b0 + r < B;
            const float ug = real ? sg.up : 0.f, uk = real ? sk.up : 0.f;
            uint16_t* dg = gp + r * rsg + 4 * lane;
            uint16_t* dk = kp + r * rsg + 4 * lane;
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                if (lane + 64 * i < q4n) {
                    const H2x4 yg = split2x4(xg[rr][i], ug), yk = split2x4(xk[rr][i], uk);
                    *reinterpret_cast<uint2*>(dg + 256 * i) = yg.h;
                    *reinterpret_cast<uint2*>(dg + 256 * i + plane) = yg.l;
                    *reinterpret_cast<uint2*>(dk + 256 * i) = yk.h;
                    *reinterpret_cast<uint2*>(dk + 256 * i + plane) = yk.l;
                }
            }
        }
    };
    // operand of tile tt of a tensor: lane (ln, kh) <-> step 32 tt + ln, K slot 8 kh + e <-> batch row 8 kh + e.  Within its
    // group of 16 lanes a lane points at [row 8 kh + (l16 >> 2)][step 32 tt + 16 (ln >> 4) + 4 (l16 & 3)]; the second read
    // is four rows further on.
    const uint32_t tr0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) char*)gp))
                       + 2u * static_cast<uint32_t>((8 * kh + (l16 >> 2)) * rsg + 16 * (ln >> 4) + 4 * (l16 & 3));
    const uint32_t k_off = 2u * 2u * static_cast<uint32_t>(plane), row4 = 2u * 4u * static_cast<uint32_t>(rsg), pl_b = 2u * static_cast<uint32_t>(plane);
    auto operand = [&](const uint32_t base, const int tt, f16x8 (&f)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int pq = 0; pq < 2; ++pq) {
            const uint32_t a = base + 64u * static_cast<uint32_t>(tt) + pq * pl_b;
            const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_ptr)(a));
            const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_ptr)(a + row4));
            const uint2 x = __builtin_bit_cast(uint2, lo), y = __builtin_bit_cast(uint2, hi);
            f[pq] = __builtin_bit_cast(f16x8, make_uint4(x.x, x.y, y.x, y.y));
        }
    };
    if (nmine > 0) {
#pragma unroll
        for (int i = 0; i < NI; ++i) fetch_part(0, i);
    }
    static_assert(T_H2_MAX / 64 <= 2 * TXW, "a wave takes at most two pairs of lag tiles per pass");

    for (int u = 0; u < nmine; ++u) {
        const int pass = u % npass;
        if (pass == 0)
            for (int i = tid; i < 2 * T; i += TXT) diag[i] = 0.f;
        unit_max();
        __syncthreads();
        store_unit(u);
        __syncthreads();
        const bool more = u + 1 < nmine;
        if (more) fetch_part(u + 1, 0);
        // lag tile d has T/32 - d tile pairs; the lag tiles go to the waves two at a time (2 m, 2 m + 1), in the order of
        // decreasing work, back and forth (waves 0..7, then 7..0): at most two pairs a wave
        const int npairs = (nt + 1) >> 1;
        auto do_pair = [&](const int m, auto&& halfway) __attribute__((always_inline)) {
            const int dl = 2 * m, n = nt - dl;                 // the longer lag tile and its tile pairs; the shorter one, dl + 1, has n - 1
            f32x16 accl, accs;
#pragma unroll
            for (int v = 0; v < 16; ++v) { accl[v] = 0.f; accs[v] = 0.f; }
            // term number `term` of the product of a g and a k operand: h h', h l', l h'
            auto product = [&](f32x16& acc, const int term, const f16x8 (&fa)[2], const f16x8 (&fb)[2]) __attribute__((always_inline)) {
                acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[term == 2 ? 1 : 0], fb[term == 1 ? 1 : 0], acc, 0, 0, 0);
            };
            auto both = [&](const f16x8 (&al_)[2], const f16x8 (&as_)[2], const f16x8 (&fb)[2]) __attribute__((always_inline)) {
                // (the longer tile's first two terms go first: the shorter tile's g operand is the read issued last)
                product(accl, 0, al_, fb); product(accl, 1, al_, fb);
                product(accs, 0, as_, fb); product(accl, 2, al_, fb);
                product(accs, 1, as_, fb); product(accs, 2, as_, fb);
            };
            auto last = [&](const f16x8 (&al_)[2], const f16x8 (&fb)[2]) __attribute__((always_inline)) {
#pragma unroll
                for (int term = 0; term < 3; ++term) product(accl, term, al_, fb);
            };
            // Pair i: the longer lag tile takes g tile dl + i, the shorter one g tile dl + 1 + i, both k tile i.  Two sets of g
            // operands change roles every pair, two sets of k operands alternate; a set is read again as soon as its last
            // product has been issued, one pair ahead of its use.
            f16x8 P[2], Q[2], be[2], bo[2];
            operand(tr0, dl, P); operand(tr0 + k_off, 0, be); operand(tr0, min(dl + 1, nt - 1), Q);
            // (one way into the loop body and one way out, see timex_conv_h2)
            auto two_pairs = [&](const int i) __attribute__((always_inline)) {
                operand(tr0 + k_off, i + 1, bo);
                __builtin_amdgcn_sched_barrier(0);
                both(P, Q, be);
                __builtin_amdgcn_sched_barrier(0);
                operand(tr0, min(dl + 2 + i, nt - 1), P);
                operand(tr0 + k_off, i + 2, be);
                __builtin_amdgcn_sched_barrier(0);
                both(Q, P, bo);
                __builtin_amdgcn_sched_barrier(0);
                operand(tr0, min(dl + 3 + i, nt - 1), Q);
            };
            int i = 0;
            const int half = ((n - 1) >> 1) & ~1;
            for (; i < half; i += 2) two_pairs(i);
            halfway();
            for (; i + 2 <= n - 1; i += 2) two_pairs(i);
            if (i < n - 1) {                                    // one pair with both tiles left, then the longer tile's last pair
                operand(tr0 + k_off, i + 1, bo);
                __builtin_amdgcn_sched_barrier(0);
                both(P, Q, be);
                __builtin_amdgcn_sched_barrier(0);
                last(Q, bo);
            } else last(P, be);
            // accumulator v: t = 8 (v/4) + 4 kh + (v&3), u = ln, of tiles d apart
            auto diagonals = [&](const f32x16& acc, const int d) __attribute__((always_inline)) {
                float pos = 0.f, neg = 0.f;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int t = 8 * (v >> 2) + 4 * kh + (v & 3);
                    const float y = __shfl(acc[v], (kh << 5) | ((t - ln) & 31), 64);
                    if (t >= ln) pos += y; else neg += y;
                }
                pos += __shfl_xor(pos, 32, 64);
                neg += __shfl_xor(neg, 32, 64);
                if (kh == 0) diag[64 * d + 31 + ln] += pos * unscale;    // lag tile d belongs to this wave alone
                else if (ln >= 1) diag[64 * d + ln - 1] += neg * unscale;
            };
            diagonals(accl, dl);
            if (dl + 1 < nt) diagonals(accs, dl + 1);
        };
        if (wv < npairs) do_pair(wv, [&]() __attribute__((always_inline)) { if (more) fetch_part(u + 1, 1); });
        else if (more) fetch_part(u + 1, 1);
        if (more) fetch_part(u + 1, 2);
        if (2 * TXW - 1 - wv < npairs) do_pair(2 * TXW - 1 - wv, []() __attribute__((always_inline)) {});
        if constexpr (NI > 3) { if (more) fetch_part(u + 1, 3); }
        __syncthreads();
        if (pass == npass - 1) {
            const int c = blockIdx.x + (u / npass) * gridDim.x;
            for (int x = tid; x < T; x += TXT) {        // lag = 32 d + e comes from tile d (diagonal e) and tile d + 1 (diagonal e - 32)
                const int lag = T - 1 - x, d = lag >> 5, e = lag & 31;
                gws[static_cast<size_t>(c) * T + x] = diag[64 * d + 31 + e] + (d + 1 < nt ? diag[64 * (d + 1) + e - 1] : 0.f);
            }
            __syncthreads();           // diag is cleared for the next channel only after it has been read
        }
    }
}

constexpr int T_MAX = 4096;

int check_tx(int B, int C, int T) {
    if (B <= 0 || C <= 0 || T <= 0) return RWKV_ERR_SHAPE;
    if (T % 4 != 0 || T > T_MAX) return RWKV_ERR_SHAPE;
    if ((B + BB - 1) / BB > 65535) return RWKV_ERR_SHAPE;
    return RWKV_OK;
}

// The matrix-core path pays off once the 32 columns of a product are mostly real batch rows.
bool use_mfma(int B, int T) { return T % 32 == 0 && T <= T_MFMA_MAX && B >= 8; }
int conv_grid(int B, int C) {
    const long long units = static_cast<long long>(C) * ((B + MROWS - 1) / MROWS);
    return static_cast<int>(units < NCU ? units : NCU);
}

template <typename K> int raise_lds_limit(K kernel, size_t bytes) {
    if (bytes <= 48 * 1024) return RWKV_OK;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes));
    if (e != hipSuccess) { g_last_hip_error = static_cast<int>(e); return RWKV_ERR_LAUNCH; }
    return RWKV_OK;
}

}  // namespace
}  // namespace rwkv

using namespace rwkv;

// gk = the mirrored convolution of gwk with w.
int launch_gk(void* stream, const float* w, const float* gwk, float* gk, int B, int C, int T) {
    if (use_mfma(B, T)) {
        const size_t lds = h2_lds_bytes(T);
        auto kernel = T <= T_H2_MID ? timex_conv_h2<true, T_H2_MID / 256> : timex_conv_h2<true, T_H2_MAX / 256>;
        if (int e = raise_lds_limit(kernel, lds)) return e;
        hipLaunchKernelGGL(kernel, dim3(conv_grid(B, C)), dim3(TXT), lds, static_cast<hipStream_t>(stream), w, gwk, gk, 0.0f, B, C, T);
    } else {
        const size_t lds = (static_cast<size_t>(BB + 1) * T + 4) * sizeof(float);
        if (int e = raise_lds_limit(timex_conv<true>, lds)) return e;
        hipLaunchKernelGGL(timex_conv<true>, dim3(C, (B + BB - 1) / BB), dim3(T / 4), lds,
                           static_cast<hipStream_t>(stream), w, gwk, gk, 0.0f, B, C, T);
    }
    return RWKV_OK;
}

extern "C" {

int rwkv_timex_forward(void* stream, const float* w, const float* k, float* x, float eps, int B, int C, int T) {
    if (int e = check_tx(B, C, T)) return e;
    if (int e = check_ptrs({w, k, x})) return e;
    if (use_mfma(B, T)) {
        const size_t lds = h2_lds_bytes(T);
        auto kernel = T <= T_H2_MID ? timex_conv_h2<false, T_H2_MID / 256> : timex_conv_h2<false, T_H2_MAX / 256>;
        if (int e = raise_lds_limit(kernel, lds)) return e;
        hipLaunchKernelGGL(kernel, dim3(conv_grid(B, C)), dim3(TXT), lds, static_cast<hipStream_t>(stream), w, k, x, eps, B, C, T);
        return launch_status();
    }
    const size_t lds = (static_cast<size_t>(BB + 1) * T + 4) * sizeof(float);
    if (int e = raise_lds_limit(timex_conv<false>, lds)) return e;
    hipLaunchKernelGGL(timex_conv<false>, dim3(C, (B + BB - 1) / BB), dim3(T / 4), lds,
                       static_cast<hipStream_t>(stream), w, k, x, eps, B, C, T);
    return launch_status();
}

int rwkv_timex_backward(void* stream, const float* w, const float* k, const float* gwk, float* gw, float* gk,
                        int B, int C, int T) {
    if (int e = check_tx(B, C, T)) return e;
    if (int e = check_ptrs({w, k, gwk, gw, gk})) return e;
    if (static_cast<long long>(B) * C > 0x7fffffffLL) return RWKV_ERR_SHAPE;
    if (int e = launch_gk(stream, w, gwk, gk, B, C, T)) return e;
    hipLaunchKernelGGL(timex_gw, dim3(B * C), dim3(T / 4), (2 * static_cast<size_t>(T) + 4) * sizeof(float),
                       static_cast<hipStream_t>(stream), k, gwk, gw, T);
    return launch_status();
}

int rwkv_timex_backward_sum(void* stream, const float* w, const float* k, const float* gwk, float* gw_sum, float* gk,
                            int B, int C, int T) {
    if (int e = check_tx(B, C, T)) return e;
    if (T % 32 != 0 || T > T_MFMA_MAX) return RWKV_ERR_SHAPE;
    if (int e = check_ptrs({w, k, gwk, gw_sum, gk})) return e;
    if (int e = launch_gk(stream, w, gwk, gk, B, C, T)) return e;
    // (any batch size: a pass takes 16 rows, rows past the batch count as zero)
    const size_t lds_gw = gw_h2_lds_bytes(T);
    auto kernel = T <= T_H2_MID ? timex_gw_sum_h2<T_H2_MID / 256> : timex_gw_sum_h2<T_H2_MAX / 256>;
    if (int e = raise_lds_limit(kernel, lds_gw)) return e;
    hipLaunchKernelGGL(kernel, dim3(C < NCU ? C : NCU), dim3(TXT), lds_gw, static_cast<hipStream_t>(stream), k, gwk, gw_sum, B, C, T);
    return launch_status();
}

}  // extern "C"
