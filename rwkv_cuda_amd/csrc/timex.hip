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
// product of the lower-triangular Toeplitz matrix W[t][u] = wr[t-u] with the [T x 32] block of inputs, done in fp32 on
// v_mfma_f32_32x32x2_f32 (lane = (row or column l & 31, K slot half l >> 5); accumulator register v: row 8 (v/4) + 4 (l>>5)
// + (v&3), column l & 31).  The kernel row is stored in tap order followed by 32 zeros, so a tap of negative lag reads 0
// and the diagonal block needs no mask.  Output tile o of 32 time steps sums over input tiles 0..o (mirror: o..T/32-1);
// wave p takes tiles p and T/32-1-p (and p + 8, ...), which balances the triangle.  K slot (half, kk) is input step 16 half + kk of the
// tile, so a lane reads its 16 B operands as four 16-byte LDS reads.
typedef float f32x16 __attribute__((ext_vector_type(16)));
constexpr int MROWS = 32;              // batch rows per workgroup = columns of the product
constexpr int T_MFMA_MAX = 1024;
constexpr int TXW = 8;                 // waves per workgroup: two per SIMD, one reads LDS while the other runs MFMAs
constexpr int TXT = 64 * TXW;
constexpr int STG = 4;
constexpr int PFQ = MROWS * (T_MFMA_MAX / 4) / TXT;     // 16-byte pieces of a unit's rows per thread, at the longest T
constexpr int NCU = 256;               // workgroups of the persistent kernels: one per CU                 // 16-byte global loads in flight per thread while staging

template <bool MIRROR>
__global__ __launch_bounds__(TXT) void timex_conv_mfma(const float* __restrict__ w, const float* __restrict__ in,
                                                       float* __restrict__ out, float eps, int B, int C, int T) {
    extern __shared__ float lds[];
    float* wp = lds;                   // [T + 32]: wp[x] = w[c][x] (tap order), 0 for x >= T
    float* rows = lds + T + 32;        // [32][T + 4]
    const int rs = T + 4;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int ln = lane & 31, kh = lane >> 5;
    const int q4n = T >> 2, total = MROWS * q4n, nt = T >> 5;
    // A workgroup walks over units (channel, group of 32 batch rows).  One workgroup fills a CU, so nothing else hides the
    // HBM latency of staging: the rows of the next unit are fetched into registers before the MFMA loop of the current
    // one and written to LDS after it.  Loads are unconditional (clamped addresses), rows past B are zeroed on the way in.
    const int nbg = (B + MROWS - 1) / MROWS, nunits = C * nbg;
    float4 x[PFQ];
    float wr[2];
    auto fetch_unit = [&](const int unit) __attribute__((always_inline)) {
        const int c = unit / nbg, b0 = (unit - c * nbg) * MROWS;
#pragma unroll
        for (int s = 0; s < PFQ; ++s) {
            const int idx = s * TXT + tid, r = idx / q4n, q4 = idx - r * q4n;
            const bool live = idx < total && b0 + r < B;
            x[s] = *reinterpret_cast<const float4*>(in + (static_cast<size_t>(live ? b0 + r : b0) * C + c) * T + (live ? 4 * q4 : 0));
        }
#pragma unroll
        for (int s = 0; s < 2; ++s) wr[s] = w[static_cast<size_t>(c) * T + min(s * TXT + tid, T - 1)];
    };
    auto store_unit = [&](const int unit) __attribute__((always_inline)) {
        const int c = unit / nbg, b0 = (unit - c * nbg) * MROWS;
#pragma unroll
        for (int s = 0; s < PFQ; ++s) {
            const int idx = s * TXT + tid, r = idx / q4n, q4 = idx - r * q4n;
            if (idx < total) *reinterpret_cast<float4*>(rows + r * rs + 4 * q4) = b0 + r < B ? x[s] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int s = 0; s < 2; ++s)
            if (s * TXT + tid < T) wp[s * TXT + tid] = wr[s];
    };
    if (tid < 32) wp[T + tid] = 0.f;
    int unit = blockIdx.x;
    if (unit < nunits) fetch_unit(unit);

    const float* brow = rows + ln * rs + 16 * kh;
    for (; unit < nunits; unit += gridDim.x) {
        const int c = unit / nbg, b0 = (unit - c * nbg) * MROWS;
        store_unit(unit);
        __syncthreads();
        if (unit + static_cast<int>(gridDim.x) < nunits) fetch_unit(unit + gridDim.x);
        // (handing tiles out longest-first from an LDS counter was slower: the older wave of a SIMD wins the matrix core,
        // drains the queue, and the younger one is left alone with a long tile)
        for (int p = wv; 2 * p < nt; p += TXW) {
#pragma unroll 1
            for (int side = 0; side < 2; ++side) {
                const int ot = side == 0 ? p : nt - 1 - p;
                if (side == 1 && ot == p) break;
                f32x16 acc, acc1;                              // even / odd K steps: consecutive MFMAs are independent
#pragma unroll
                for (int v = 0; v < 16; ++v) { acc[v] = MIRROR ? 0.f : eps; acc1[v] = 0.f; }
                const int n_in = MIRROR ? nt - ot : ot + 1;
                // operands of step j + 1 are read while the MFMAs of step j run
                float a[16], b[16];
                auto fetch = [&](int j, float (&fa)[16], float (&fb)[16]) {
                    const int it = MIRROR ? ot + j : j;            // input tile
                    const int d = MIRROR ? j : ot - j;             // lag in tiles, >= 0
                    // A[row][K slot]: forward row = t, slot = u: tap T-1-(t-u);  mirror row = u, slot = t: tap T-1-(t-u)
                    const float* ap = wp + (MIRROR ? T - 1 - 32 * d - 16 * kh + ln : T - 1 - 32 * d - ln + 16 * kh);
#pragma unroll
                    for (int kk = 0; kk < 16; ++kk) fa[kk] = MIRROR ? ap[-kk] : ap[kk];
#pragma unroll
                    for (int z = 0; z < 4; ++z) {
                        const float4 y = *reinterpret_cast<const float4*>(brow + 32 * it + 4 * z);
                        fb[4 * z] = y.x; fb[4 * z + 1] = y.y; fb[4 * z + 2] = y.z; fb[4 * z + 3] = y.w;
                    }
                };
                fetch(0, a, b);
                for (int j = 0; j < n_in; ++j) {
                    float an[16], bn[16];
                    fetch(j + 1 < n_in ? j + 1 : j, an, bn);
#pragma unroll
                    for (int kk = 0; kk < 16; kk += 2) {
                        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kk], b[kk], acc, 0, 0, 0);
                        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kk + 1], b[kk + 1], acc1, 0, 0, 0);
                    }
#pragma unroll
                    for (int kk = 0; kk < 16; ++kk) { a[kk] = an[kk]; b[kk] = bn[kk]; }
                }
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[v] += acc1[v];
                if (b0 + ln < B) {
                    float* o = out + (static_cast<size_t>(b0 + ln) * C + c) * T + 32 * ot + 4 * kh;
#pragma unroll
                    for (int v4 = 0; v4 < 4; ++v4)
                        *reinterpret_cast<float4*>(o + 8 * v4) = make_float4(acc[4 * v4], acc[4 * v4 + 1], acc[4 * v4 + 2], acc[4 * v4 + 3]);
                }
            }
        }
        __syncthreads();               // every wave is done with this unit's rows
    }
}

// ------------------------------------------------------------------------------------ matrix-core path, bf16 x 3 products
// The same product with every fp32 operand x cut into three bf16 terms, x = h + m + l (24 mantissa bits together), and
//     x y = h h' + h m' + m h' + m m' + h l' + l h'          (the terms left out are below 2^-24 of the product)
// on v_mfma_f32_32x32x16_bf16: six instructions of 16 matrix passes where the fp32 instruction needs eight of 16 passes
// for the same 32 x 32 x 16 block, i.e. 2.7 times the arithmetic rate at fp32 accuracy (accumulation is fp32 either way).
// Operand layout of the instruction: lane = (row or column l & 31, K half l >> 5) holds the eight consecutive K slots
// 8 (l >> 5) .. + 7; accumulator as above.  K slot s of a step is input step 16 ks + s of the 32-step tile.
//   rows : three planes [32 batch rows][T + 16] bf16; a lane's eight slots are 16 aligned bytes.
//   taps : the A operand of row t and slot u is line[base(t) + u] for a line that depends only on the direction
//          (forward: the kernel row in tap order followed by zeros; mirror: 31 zeros, then the reversed kernel row), so a
//          lane reads eight consecutive bf16 starting at an arbitrary element.  Two copies of every plane, the second
//          shifted by one element, make that four aligned dwords whatever the parity of the start.
// LDS: 3 x 32 x (T + 16) x 2 + 6 x (T + 96) x 2 bytes = 160 896 of 163 840 at T = 768, the longest T this form takes.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
constexpr int T_BF3_MAX = 768;
constexpr int PFQ3 = MROWS * (T_BF3_MAX / 4) / TXT;
__host__ __device__ inline int bf3_row_stride(int T) { return T + 16; }          // elements; (T + 16) / 2 dwords = 8 or 24 mod 32
__host__ __device__ inline int bf3_line_len(int T) { return T + ((T & 32) ? 64 : 96); }   // half of it = 16 mod 32 dwords: the shifted copy sits 16 banks away
__host__ __device__ inline size_t bf3_lds_bytes(int T) {
    return (3 * static_cast<size_t>(MROWS) * bf3_row_stride(T) + 6 * static_cast<size_t>(bf3_line_len(T))) * sizeof(uint16_t);
}
// x = h + m + l with each term the leading eight mantissa bits of what the terms before it leave (truncation: two AND and
// two exact subtractions; what l drops is below 2^-24 |x|)
struct Bf3 { uint16_t h, m, l; };
DEVINL Bf3 split3(float x) {
    const uint32_t hb = __float_as_uint(x) & 0xffff0000u;
    const float x1 = x - __uint_as_float(hb);
    const uint32_t mb = __float_as_uint(x1) & 0xffff0000u;
    const float x2 = x1 - __uint_as_float(mb);
    Bf3 r;
    r.h = static_cast<uint16_t>(hb >> 16);
    r.m = static_cast<uint16_t>(mb >> 16);
    r.l = static_cast<uint16_t>(__float_as_uint(x2) >> 16);
    return r;
}

template <bool MIRROR>
__global__ __launch_bounds__(TXT) void timex_conv_bf3(const float* __restrict__ w, const float* __restrict__ in,
                                                      float* __restrict__ out, float eps, int B, int C, int T) {
    extern __shared__ float lds[];
    const int rs = bf3_row_stride(T), xl = bf3_line_len(T);
    uint16_t* rp = reinterpret_cast<uint16_t*>(lds);                    // [3][32][rs]
    uint16_t* al = rp + 3 * MROWS * rs;                                 // [3 planes][2 copies][xl]
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int ln = lane & 31, kh = lane >> 5;
    const int q4n = T >> 2, total = MROWS * q4n, nt = T >> 5;
    const int nbg = (B + MROWS - 1) / MROWS, nunits = C * nbg;
    float4 x[PFQ3];
    float wr[2];
    // piece s of this thread is 16-byte piece idx = s TXT + tid of the unit's rows, (row, piece in the row) = (idx / q4n,
    // idx % q4n): one division here, then steps of TXT
    const int r_first = tid / q4n, q_first = tid - r_first * q4n, r_step = TXT / q4n, q_step = TXT - r_step * q4n;
    auto fetch_unit = [&](const int unit) __attribute__((always_inline)) {
        const int c = unit / nbg, b0 = (unit - c * nbg) * MROWS;
        int r = r_first, q4 = q_first;
#pragma unroll
        for (int s = 0; s < PFQ3; ++s) {
            const bool live = s * TXT + tid < total && b0 + r < B;
            x[s] = *reinterpret_cast<const float4*>(in + (static_cast<size_t>(live ? b0 + r : b0) * C + c) * T + (live ? 4 * q4 : 0));
            r += r_step; q4 += q_step;
            if (q4 >= q4n) { q4 -= q4n; ++r; }
        }
#pragma unroll
        for (int s = 0; s < 2; ++s) wr[s] = w[static_cast<size_t>(c) * T + min(s * TXT + tid, T - 1)];
    };
    auto store_unit = [&](const int unit) __attribute__((always_inline)) {
        const int c = unit / nbg, b0 = (unit - c * nbg) * MROWS;
        int r = r_first, q4 = q_first;
#pragma unroll
        for (int s = 0; s < PFQ3; ++s) {
            if (s * TXT + tid < total) {
                const float4 v = b0 + r < B ? x[s] : make_float4(0.f, 0.f, 0.f, 0.f);
                const Bf3 a0 = split3(v.x), a1 = split3(v.y), a2 = split3(v.z), a3 = split3(v.w);
                uint16_t* d = rp + r * rs + 4 * q4;
                *reinterpret_cast<uint2*>(d) = make_uint2(a0.h | (static_cast<uint32_t>(a1.h) << 16), a2.h | (static_cast<uint32_t>(a3.h) << 16));
                *reinterpret_cast<uint2*>(d + MROWS * rs) = make_uint2(a0.m | (static_cast<uint32_t>(a1.m) << 16), a2.m | (static_cast<uint32_t>(a3.m) << 16));
                *reinterpret_cast<uint2*>(d + 2 * MROWS * rs) = make_uint2(a0.l | (static_cast<uint32_t>(a1.l) << 16), a2.l | (static_cast<uint32_t>(a3.l) << 16));
            }
            r += r_step; q4 += q_step;
            if (q4 >= q4n) { q4 -= q4n; ++r; }
        }
        // tap tau of the kernel row sits at line position tau (forward) or 31 + (T - 1 - tau) (mirror); the rest is zero
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int tau = s * TXT + tid;
            if (tau < T) {
                const Bf3 a = split3(wr[s]);
                const int pos = MIRROR ? 31 + (T - 1 - tau) : tau;
                const uint16_t pl[3] = {a.h, a.m, a.l};
#pragma unroll
                for (int p = 0; p < 3; ++p) {
                    al[(2 * p) * xl + pos] = pl[p];
                    if (pos >= 1) al[(2 * p + 1) * xl + pos - 1] = pl[p];
                }
            }
        }
        (void)c;
    };
    // the zero parts of the line never change: clear everything once (the taps are rewritten for every unit)
    for (int i = tid; i < 6 * xl; i += TXT) al[i] = 0;
    __syncthreads();
    int unit = blockIdx.x;
    if (unit < nunits) fetch_unit(unit);

    for (; unit < nunits; unit += gridDim.x) {
        const int c = unit / nbg, b0 = (unit - c * nbg) * MROWS;
        store_unit(unit);
        __syncthreads();
        if (unit + static_cast<int>(gridDim.x) < nunits) fetch_unit(unit + gridDim.x);
        for (int p = wv; 2 * p < nt; p += TXW) {
#pragma unroll 1
            for (int side = 0; side < 2; ++side) {
                const int ot = side == 0 ? p : nt - 1 - p;
                if (side == 1 && ot == p) break;
                f32x16 acc, acc1;                              // two chains: consecutive MFMAs are independent
#pragma unroll
                for (int v = 0; v < 16; ++v) { acc[v] = MIRROR ? 0.f : eps; acc1[v] = 0.f; }
                const int n_in = MIRROR ? nt - ot : ot + 1;
                // A step is 16 input steps: the six products of one K block.  From one step to the next both operands move on
                // by 16 elements: the tap window because the lag falls by 16 (forward) or grows by 16 (mirror) together with
                // the slot base, the rows because the input step does.
                //   forward: row t = 32 ot + ln, slot u: tap T-1-(t-u)            -> line[T-1-32 ot-ln + u]
                //   mirror : row u = 32 ot + ln, slot t: lag 32 (it-ot) + slot-ln -> line[31-ln + 32 (it-ot) + slot]
                const int start0 = (MIRROR ? 31 - ln : T - 1 - 32 * ot - ln) + 8 * kh;
                const uint32_t* ap0 = reinterpret_cast<const uint32_t*>(al + (start0 & 1) * xl) + (start0 >> 1);
                const uint16_t* bp0 = rp + ln * rs + (MIRROR ? 32 * ot : 0) + 8 * kh;
                auto fetch = [&](int j2, bf16x8 (&fa)[3], bf16x8 (&fb)[3]) __attribute__((always_inline)) {
#pragma unroll
                    for (int pq = 0; pq < 3; ++pq) {
                        const uint32_t* a4 = ap0 + 8 * j2 + pq * xl;   // a plane is 2 xl elements = xl dwords
                        fa[pq] = __builtin_bit_cast(bf16x8, make_uint4(a4[0], a4[1], a4[2], a4[3]));
                        fb[pq] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(bp0 + 16 * j2 + pq * MROWS * rs));
                    }
                };
                auto products = [&](const bf16x8 (&fa)[3], const bf16x8 (&fb)[3]) __attribute__((always_inline)) {
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[0], fb[0], acc, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[0], fb[1], acc1, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[1], fb[0], acc, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[1], fb[1], acc1, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[0], fb[2], acc, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[2], fb[0], acc1, 0, 0, 0);
                };
                // two register sets take turns; the step after the last one is fetched too and never used (it lies inside
                // the workgroup's LDS: the line has at least 64 spare elements, the rows are followed by the line)
                bf16x8 a[3], b[3], a2[3], b2[3];
                fetch(0, a, b);
                // (the fences keep the reads of the next step in front of the products of this one: left to itself the
                // scheduler sinks them behind the products and then waits for them at once)
                for (int j2 = 0; j2 < 2 * n_in; j2 += 2) {
                    fetch(j2 + 1, a2, b2);
                    __builtin_amdgcn_sched_barrier(0);
                    products(a, b);
                    __builtin_amdgcn_sched_barrier(0);
                    fetch(j2 + 2, a, b);
                    __builtin_amdgcn_sched_barrier(0);
                    products(a2, b2);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[v] += acc1[v];
                if (b0 + ln < B) {
                    float* o = out + (static_cast<size_t>(b0 + ln) * C + c) * T + 32 * ot + 4 * kh;
#pragma unroll
                    for (int v4 = 0; v4 < 4; ++v4)
                        *reinterpret_cast<float4*>(o + 8 * v4) = make_float4(acc[4 * v4], acc[4 * v4 + 1], acc[4 * v4 + 2], acc[4 * v4 + 3]);
                }
            }
        }
        __syncthreads();               // every wave is done with this unit's rows
    }
}

// Kernel gradient summed over the batch: gws[c][T-1-lag] = sum_b sum_t g[b,c,t] k[b,c,t-lag], i.e. the sum of the lag-th
// sub-diagonal of M = G^T K (contraction over the batch).  Batch rows are staged ROWS at a time; MFMA number kk contracts
// rows 2kk and 2kk+1 (K slot = l >> 5), even and odd kk into separate accumulators so that consecutive MFMAs are
// independent.  A wave owns whole lag tiles d (all tile pairs (tt, tt-d) accumulate into the same registers; d and
// T/32-1-d together balance the triangle).  A finished tile goes through a per-wave LDS tile, from which lane l sums
// diagonal l - 31 in row order and adds it to entry l of lag tile d, which no other wave touches: no atomics, every fp32
// sum in a fixed order.
constexpr int DIAG_STRIDE = 33;
constexpr int T_GW_WIDE = 768;         // up to here 16 batch rows per pass fit in LDS, beyond 8
__host__ __device__ inline int gw_row_stride(int T) { return T + 32 - (T & 63); }      // = 32 mod 64: the two K halves of a read use different banks
__host__ __device__ inline size_t gw_lds_floats(int T, int rows) {
    return 2 * static_cast<size_t>(rows) * gw_row_stride(T) + 2 * static_cast<size_t>(T) + TXW * 32 * DIAG_STRIDE;
}

template <int ROWS>
__global__ __launch_bounds__(TXT) void timex_gw_sum_mfma(const float* __restrict__ k, const float* __restrict__ g,
                                                         float* __restrict__ gws, int B, int C, int T) {
    extern __shared__ float lds[];
    const int rs = gw_row_stride(T);
    float* gr = lds;                           // [ROWS][rs]
    float* kr = gr + ROWS * rs;                // [ROWS][rs]
    float* diag = kr + ROWS * rs;              // [T/32 lag tiles][64]: entry l of tile d is the sum for lag 32 d + l - 31
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int ln = lane & 31, kh = lane >> 5;
    const int nt = T >> 5, q4n = T >> 2, total = ROWS * q4n;
    float* tile = diag + 2 * T + wv * (32 * DIAG_STRIDE);         // [32 t][33]: one finished product tile

    // A workgroup walks over its channels (blockIdx.x, + gridDim.x, ...) and, per channel, over passes of ROWS batch rows;
    // the rows of the next pass are fetched into registers before the MFMA loop of the current one (see timex_conv_mfma).
    constexpr int PF = ROWS * ((ROWS == 16 ? T_GW_WIDE : T_MFMA_MAX) / 4) / TXT;
    const int npass = (B + ROWS - 1) / ROWS;
    const int nmine = (C > static_cast<int>(blockIdx.x) ? (C - 1 - static_cast<int>(blockIdx.x)) / static_cast<int>(gridDim.x) + 1 : 0) * npass;
    float4 xg[PF], xk[PF];
    auto fetch_unit = [&](const int u) __attribute__((always_inline)) {
        const int c = blockIdx.x + (u / npass) * gridDim.x, b0 = (u % npass) * ROWS;
#pragma unroll
        for (int s = 0; s < PF; ++s) {
            const int idx = s * TXT + tid, r = idx / q4n, q4 = idx - r * q4n;
            const bool live = idx < total && b0 + r < B;
            const size_t off = (static_cast<size_t>(live ? b0 + r : b0) * C + c) * T + (live ? 4 * q4 : 0);
            xg[s] = *reinterpret_cast<const float4*>(g + off);
            xk[s] = *reinterpret_cast<const float4*>(k + off);
        }
    };
    auto store_unit = [&](const int u) __attribute__((always_inline)) {
        const int b0 = (u % npass) * ROWS;
#pragma unroll
        for (int s = 0; s < PF; ++s) {
            const int idx = s * TXT + tid, r = idx / q4n, q4 = idx - r * q4n;
            if (idx < total) {
                const bool real = b0 + r < B;
                *reinterpret_cast<float4*>(gr + r * rs + 4 * q4) = real ? xg[s] : make_float4(0.f, 0.f, 0.f, 0.f);
                *reinterpret_cast<float4*>(kr + r * rs + 4 * q4) = real ? xk[s] : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    };
    if (nmine > 0) fetch_unit(0);

    const float* ga = gr + kh * rs + ln;
    const float* kb = kr + kh * rs + ln;
    for (int u = 0; u < nmine; ++u) {
        const int pass = u % npass;
        if (pass == 0)
            for (int i = tid; i < 2 * T; i += TXT) diag[i] = 0.f;
        store_unit(u);
        __syncthreads();
        if (u + 1 < nmine) fetch_unit(u + 1);
        for (int p = wv; 2 * p < nt; p += TXW) {
#pragma unroll 1
            for (int side = 0; side < 2; ++side) {
                const int d = side == 0 ? p : nt - 1 - p;
                if (side == 1 && d == p) break;
                f32x16 acc0, acc1;
#pragma unroll
                for (int v = 0; v < 16; ++v) acc0[v] = acc1[v] = 0.f;
                constexpr int NK = ROWS / 2;
                float a[NK], b[NK];
                auto fetch = [&](int tt, float (&fa)[NK], float (&fb)[NK]) {
#pragma unroll
                    for (int kk = 0; kk < NK; ++kk) {
                        fa[kk] = ga[2 * kk * rs + 32 * tt];
                        fb[kk] = kb[2 * kk * rs + 32 * (tt - d)];
                    }
                };
                fetch(d, a, b);
                for (int tt = d; tt < nt; ++tt) {
                    float an[NK], bn[NK];
                    fetch(tt + 1 < nt ? tt + 1 : tt, an, bn);
#pragma unroll
                    for (int kk = 0; kk < NK; kk += 2) {
                        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kk], b[kk], acc0, 0, 0, 0);
                        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kk + 1], b[kk + 1], acc1, 0, 0, 0);
                    }
#pragma unroll
                    for (int kk = 0; kk < NK; ++kk) { a[kk] = an[kk]; b[kk] = bn[kk]; }
                }
                // accumulator v: t = 8 (v/4) + 4 kh + (v&3), u = ln, of tiles d apart
#pragma unroll
                for (int v = 0; v < 16; ++v) tile[(8 * (v >> 2) + 4 * kh + (v & 3)) * DIAG_STRIDE + ln] = acc0[v] + acc1[v];
                const int dl = lane - 31;                   // diagonal t - u of this lane
                float sum = 0.f;
#pragma unroll
                for (int t = 0; t < 32; ++t) {
                    const int uu = t - dl;
                    const float y = tile[t * DIAG_STRIDE + (uu & 31)];
                    sum += (uu >= 0 && uu < 32) ? y : 0.f;
                }
                diag[64 * d + lane] += sum;                 // lag tile d belongs to this wave alone
            }
        }
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

// The same sum with three-term bf16 products (see timex_conv_bf3), 16 batch rows per pass: one v_mfma_f32_32x32x16_bf16
// block per pair of tiles and product.  Both operands hold eight consecutive batch rows per lane, so the planes are kept
// transposed, [step][16 rows] bf16: 32 bytes per step, and the 64 lanes of an operand read cover one contiguous KiB.
// A finished tile's diagonals are summed in registers: lane p of a half-wave collects, for every row t it holds, the
// element of column (t - p) mod 32 (one ds_bpermute per accumulator register), which belongs to diagonal p if t >= p and
// to diagonal p - 32 otherwise.
// LDS: 2 x 3 x T x 32 + 2 T x 4 bytes = 153 600 at T = 768.
constexpr int GB3_ROWS = 16;
__host__ __device__ inline size_t gw_bf3_lds_bytes(int T) { return 6 * static_cast<size_t>(T) * GB3_ROWS * sizeof(uint16_t) + 2 * static_cast<size_t>(T) * sizeof(float); }

__global__ __launch_bounds__(TXT) void timex_gw_sum_bf3(const float* __restrict__ k, const float* __restrict__ g,
                                                        float* __restrict__ gws, int B, int C, int T) {
    extern __shared__ float lds[];
    uint16_t* gp = reinterpret_cast<uint16_t*>(lds);           // [3][T][16]
    uint16_t* kp = gp + 3 * T * GB3_ROWS;                      // [3][T][16]
    float* diag = reinterpret_cast<float*>(kp + 3 * T * GB3_ROWS);   // [T/32 lag tiles][64]: entry l of tile d is the sum for lag 32 d + l - 31
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int ln = lane & 31, kh = lane >> 5;
    const int nt = T >> 5, q4n = T >> 2;
    const int plane = T * GB3_ROWS;                            // elements

    // Staging: thread (row r = tid & 15, piece q = tid >> 4, + 32 per round) reads 16 bytes of its row.  The bank of a
    // step's cell depends on the step within its group of four and on the row only, so the cells of a group are stored
    // rotated by the group number: step 4 q + e sits in cell 4 q + ((e + q) & 3), and the lanes of a store instruction
    // (one e, many q) spread over all banks.  A reading lane applies the same rotation to its step, once.
    constexpr int PF = GB3_ROWS * (T_BF3_MAX / 4) / TXT;       // pieces per thread and tensor: 6
    const int npass = (B + GB3_ROWS - 1) / GB3_ROWS;
    const int nmine = (C > static_cast<int>(blockIdx.x) ? (C - 1 - static_cast<int>(blockIdx.x)) / static_cast<int>(gridDim.x) + 1 : 0) * npass;
    const int r_own = tid & 15, q_own = tid >> 4;
    float4 xg[PF], xk[PF];
    auto fetch_unit = [&](const int u) __attribute__((always_inline)) {
        const int c = blockIdx.x + (u / npass) * gridDim.x, b0 = (u % npass) * GB3_ROWS;
#pragma unroll
        for (int s = 0; s < PF; ++s) {
            const int q4 = s * 32 + q_own;
            const bool live = q4 < q4n && b0 + r_own < B;
            const size_t off = (static_cast<size_t>(live ? b0 + r_own : b0) * C + c) * T + (live ? 4 * q4 : 0);
            xg[s] = *reinterpret_cast<const float4*>(g + off);
            xk[s] = *reinterpret_cast<const float4*>(k + off);
        }
    };
    auto put = [&](uint16_t* dst, const float4& x4, const int q4, const bool real) __attribute__((always_inline)) {
        const float xs[4] = {real ? x4.x : 0.f, real ? x4.y : 0.f, real ? x4.z : 0.f, real ? x4.w : 0.f};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const Bf3 y = split3(xs[e]);
            uint16_t* d = dst + (4 * q4 + ((e + q4) & 3)) * GB3_ROWS + r_own;
            d[0] = y.h; d[plane] = y.m; d[2 * plane] = y.l;
        }
    };
    auto store_unit = [&](const int u) __attribute__((always_inline)) {
        const int b0 = (u % npass) * GB3_ROWS;
        const bool real = b0 + r_own < B;
#pragma unroll
        for (int s = 0; s < PF; ++s) {
            const int q4 = s * 32 + q_own;
            if (q4 < q4n) { put(gp, xg[s], q4, real); put(kp, xk[s], q4, real); }
        }
    };
    if (nmine > 0) fetch_unit(0);

    for (int u = 0; u < nmine; ++u) {
        const int pass = u % npass;
        if (pass == 0)
            for (int i = tid; i < 2 * T; i += TXT) diag[i] = 0.f;
        store_unit(u);
        __syncthreads();
        if (u + 1 < nmine) fetch_unit(u + 1);
        for (int p = wv; 2 * p < nt; p += TXW) {
#pragma unroll 1
            for (int side = 0; side < 2; ++side) {
                const int d = side == 0 ? p : nt - 1 - p;
                if (side == 1 && d == p) break;
                f32x16 acc0, acc1;
#pragma unroll
                for (int v = 0; v < 16; ++v) acc0[v] = acc1[v] = 0.f;
                // tile tt of g against tile tt - d of k: both move on by one tile (32 steps of 32 bytes) per iteration
                const int cell = (ln & ~3) | (((ln & 3) + (ln >> 2)) & 3);     // where step ln of a tile sits (8 groups per tile)
                const uint16_t* ga0 = gp + (32 * d + cell) * GB3_ROWS + 8 * kh;
                const uint16_t* kb0 = kp + cell * GB3_ROWS + 8 * kh;
                auto fetch = [&](int i, bf16x8 (&fa)[3], bf16x8 (&fb)[3]) __attribute__((always_inline)) {
#pragma unroll
                    for (int pq = 0; pq < 3; ++pq) {
                        fa[pq] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(ga0 + i * 32 * GB3_ROWS + pq * plane));
                        fb[pq] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(kb0 + i * 32 * GB3_ROWS + pq * plane));
                    }
                };
                auto products = [&](const bf16x8 (&fa)[3], const bf16x8 (&fb)[3]) __attribute__((always_inline)) {
                    acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[0], fb[0], acc0, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[0], fb[1], acc1, 0, 0, 0);
                    acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[1], fb[0], acc0, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[1], fb[1], acc1, 0, 0, 0);
                    acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[0], fb[2], acc0, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[2], fb[0], acc1, 0, 0, 0);
                };
                const int n = nt - d;                          // tile pairs of this lag tile
                // one register set: the other wave of the SIMD runs its products while this one waits for its operands (a
                // second set, with the next unit's rows held across this loop, does not fit in 256 registers)
                for (int i = 0; i < n; ++i) {
                    bf16x8 a[3], b[3];
                    fetch(i, a, b);
                    products(a, b);
                }
                // accumulator v: t = 8 (v/4) + 4 kh + (v&3), u = ln, of tiles d apart
                float pos = 0.f, neg = 0.f;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int t = 8 * (v >> 2) + 4 * kh + (v & 3);
                    const float y = __shfl(acc0[v] + acc1[v], (kh << 5) | ((t - ln) & 31), 64);
                    if (t >= ln) pos += y; else neg += y;
                }
                pos += __shfl_xor(pos, 32, 64);
                neg += __shfl_xor(neg, 32, 64);
                if (kh == 0) diag[64 * d + 31 + ln] += pos;    // lag tile d belongs to this wave alone
                else if (ln >= 1) diag[64 * d + ln - 1] += neg;
            }
        }
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
bool use_bf3(int B, int T) { return use_mfma(B, T) && T <= T_BF3_MAX; }
int conv_grid(int B, int C) {
    const long long units = static_cast<long long>(C) * ((B + MROWS - 1) / MROWS);
    return static_cast<int>(units < NCU ? units : NCU);
}
size_t mfma_lds_bytes(int T) { return (static_cast<size_t>(T) + 32 + static_cast<size_t>(MROWS) * (T + 4)) * sizeof(float); }

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
    if (use_bf3(B, T)) {
        const size_t lds = bf3_lds_bytes(T);
        if (int e = raise_lds_limit(timex_conv_bf3<true>, lds)) return e;
        hipLaunchKernelGGL(timex_conv_bf3<true>, dim3(conv_grid(B, C)), dim3(TXT), lds,
                           static_cast<hipStream_t>(stream), w, gwk, gk, 0.0f, B, C, T);
    } else if (use_mfma(B, T)) {
        const size_t lds = mfma_lds_bytes(T);
        if (int e = raise_lds_limit(timex_conv_mfma<true>, lds)) return e;
        hipLaunchKernelGGL(timex_conv_mfma<true>, dim3(conv_grid(B, C)), dim3(TXT), lds,
                           static_cast<hipStream_t>(stream), w, gwk, gk, 0.0f, B, C, T);
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
    if (use_bf3(B, T)) {
        const size_t lds = bf3_lds_bytes(T);
        if (int e = raise_lds_limit(timex_conv_bf3<false>, lds)) return e;
        hipLaunchKernelGGL(timex_conv_bf3<false>, dim3(conv_grid(B, C)), dim3(TXT), lds,
                           static_cast<hipStream_t>(stream), w, k, x, eps, B, C, T);
        return launch_status();
    }
    if (use_mfma(B, T)) {
        const size_t lds = mfma_lds_bytes(T);
        if (int e = raise_lds_limit(timex_conv_mfma<false>, lds)) return e;
        hipLaunchKernelGGL(timex_conv_mfma<false>, dim3(conv_grid(B, C)), dim3(TXT), lds,
                           static_cast<hipStream_t>(stream), w, k, x, eps, B, C, T);
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
    if (use_bf3(B, T)) {
        const size_t lds_gw = gw_bf3_lds_bytes(T);
        if (int e = raise_lds_limit(timex_gw_sum_bf3, lds_gw)) return e;
        hipLaunchKernelGGL(timex_gw_sum_bf3, dim3(C < NCU ? C : NCU), dim3(TXT), lds_gw, static_cast<hipStream_t>(stream), k, gwk, gw_sum, B, C, T);
        return launch_status();
    }
    const bool wide = T <= T_GW_WIDE;
    const size_t lds_gw = gw_lds_floats(T, wide ? 16 : 8) * sizeof(float);
    auto kernel = wide ? timex_gw_sum_mfma<16> : timex_gw_sum_mfma<8>;
    if (int e = raise_lds_limit(kernel, lds_gw)) return e;
    hipLaunchKernelGGL(kernel, dim3(C < NCU ? C : NCU), dim3(TXT), lds_gw, static_cast<hipStream_t>(stream), k, gwk, gw_sum, B, C, T);
    return launch_status();
}

}  // extern "C"
