// Prefill quantise-and-pack for gfx950, and the unfused quant()/encode()
// operators of the reference surface.
//
// Per-channel statistics need a column reduction over the token axis, so the
// work is three launches on one stream:
//   1. partial min/max per (batch, head, token chunk, channel)  - reads x once
//   2. statistics: combine the chunks, run the storage-dtype op chain
//      and, per channel, the input thresholds at which the code steps up
//   3. emit: re-read x, compare against the thresholds, pack the codes
// Every arithmetic step that the reference performs as a separate torch op on
// a 16-bit tensor is rounded to that dtype here (rnd<DT>), and divisions are
// IEEE (__fdiv_rn); contraction is off so no multiply-add is fused.
//
// For a positive finite scale the code is a non-decreasing step function of the
// input (division by a positive number, adding a constant, rounding, clamping are
// all monotone), so it is fixed by L thresholds per channel: the smallest storage
// value that yields code k.  The statistics kernel finds them by bisection over
// the ordered 16-bit values, evaluating the exact op chain, and the emit kernel
// only compares - the per-element IEEE division would otherwise bound the pass.
#include "cq_common.h"

#include <atomic>

#include <mutex>
#include <vector>

#pragma clang fp contract(off)

namespace cq {

constexpr int kQThreads = 256;
constexpr int kQUnroll = 4;   // rows in flight per thread in the chunked kernels

struct QuantGeom {
    int B, T, H, D;
    int64_t sb, st, sh;   // element strides of x
    int nchunk, chunk;    // token chunks
    FastDiv dT, dH;       // divisors T and H of a flat (b, h, t) row index (per-token quantiser)
    FastDiv dTB;          // per-token quantiser: blocks of 16 tokens per (batch, head)
    int shared_stats;     // non-zero: one row of statistics / thresholds serves every (batch, head) (whole-tensor mode)
    // One-pass kernel on a token axis that is longer than a workgroup's registers hold (SPLIT): 2^parts_log2
    // workgroups share a slice, `part_rows` rows each, and exchange their channel minima / maxima through `rec`
    // inside the launch: [virtual slice][channel][2] 64-bit records, the float's bits below the call's epoch, so a
    // record is valid by itself and nothing has to be cleared.  The wait for the other parts is bounded
    // (spin_limit polls); a lane that gives up sets *status (pinned host memory).
    int parts_log2, part_rows;
    int wide_map;         // one-pass kernel: which (batch, head) pairs share a die, see slice_of()
    unsigned long long* rec;
    uint32_t epoch;
    int spin_limit;
    int* status;
};

static inline int pick_chunks(int B, int T, int H) {
    int64_t bh = static_cast<int64_t>(B) * H;
    int64_t want = (4096 + bh - 1) / bh;
    int64_t cap = T / 64 > 1 ? T / 64 : 1;
    int64_t n = want < cap ? want : cap;
    if (n > 256) n = 256;
    if (n < 1) n = 1;
    return static_cast<int>(n);
}

// ---- 1. partial min / max -------------------------------------------------
// grid (nchunk, H, B), 256 threads.  A row of D elements is covered by D/8
// adjacent lanes with one 16-byte load each; 256/(D/8) rows per iteration.
template <typename DT>
__global__ __launch_bounds__(kQThreads) void minmax_partial_kernel(const uint16_t* __restrict__ x, QuantGeom g,
                                                                  float* __restrict__ part) {
    const int lpr = g.D >> 3;
    const int rows_per_iter = kQThreads / lpr;
    const int lane = threadIdx.x % lpr;
    const int row = threadIdx.x / lpr;
    const int c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int t0 = c * g.chunk;
    const int t1 = min(g.T, t0 + g.chunk);
    const uint16_t* base = x + b * g.sb + h * g.sh + lane * 8;

    float mn[8], mx[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { mn[i] = INFINITY; mx[i] = -INFINITY; }
    // four rows in flight per thread; rows past the chunk re-read its last row (harmless for min / max)
    for (int tb = t0 + row; tb < t1; tb += kQUnroll * rows_per_iter) {
        uint4 v[kQUnroll];
#pragma unroll
        for (int u = 0; u < kQUnroll; ++u)
            v[u] = *reinterpret_cast<const uint4*>(base + min(tb + u * rows_per_iter, t1 - 1) * g.st);
#pragma unroll
        for (int u = 0; u < kQUnroll; ++u) {
            float f[8];
            unpack8<DT>(v[u], f);
#pragma unroll
            for (int i = 0; i < 8; ++i) { mn[i] = fminf(mn[i], f[i]); mx[i] = fmaxf(mx[i], f[i]); }
        }
    }
    __shared__ float smn[kQThreads * 8];
    __shared__ float smx[kQThreads * 8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        smn[(row * lpr + lane) * 8 + i] = mn[i];
        smx[(row * lpr + lane) * 8 + i] = mx[i];
    }
    __syncthreads();
    // thread d (< D) folds the rows_per_iter partial rows of channel d
    for (int d = threadIdx.x; d < g.D; d += kQThreads) {
        float a = INFINITY, z = -INFINITY;
        for (int r = 0; r < rows_per_iter; ++r) {
            a = fminf(a, smn[r * g.D + d]);
            z = fmaxf(z, smx[r * g.D + d]);
        }
        float* o = part + ((static_cast<int64_t>(b) * g.H + h) * g.nchunk + c) * 2 * g.D;
        o[d] = a;
        o[g.D + d] = z;
    }
}

// One element of calibquant.py:36: round(clamp(x / scale + zero_point, 0, L)).
// Returns the rounded value; NaN stays NaN (the reference's LUT search then
// finds no match and yields index 0).
template <typename DT>
__device__ __forceinline__ float quant_value(float x, float s, float zp, float levels) {
    float y = rnd<DT>(__fdiv_rn(x, s));
    y = rnd<DT>(y + zp);
    if (y != y) return y;
    y = fminf(fmaxf(y, 0.0f), levels);
    return rintf(y);
}

// Monotone map between the 16-bit storage patterns and integers: order of the keys =
// order of the values (-inf lowest, +inf highest; NaN patterns lie outside [kKeyLo, kKeyHi]).
template <typename DT> struct Keys;
template <> struct Keys<BF16> { static constexpr int lo = -0x7f80, hi = 0x7f80; };
template <> struct Keys<FP16> { static constexpr int lo = -0x7c00, hi = 0x7c00; };
template <typename DT>
__device__ __forceinline__ float key_value(int key) {   // key >= 0: pattern key; key < 0: sign bit + (-key)
    const uint32_t bits = key >= 0 ? static_cast<uint32_t>(key) : (0x8000u | static_cast<uint32_t>(-key));
    return Cvt<DT>::to_float(bits);
}

// ---- 2. statistics ---------------------------------------------------------
// grid (B*H), 1024 threads = 1024/D parts x D channels: thread (p, d) folds every (1024/D)-th chunk
// partial of channel d; after the fold, part 0 writes the statistics and parts 1..3 search one
// threshold each.
// The op chain of calibquant.py:27-34 with one rounding per op; `tensor / python_scalar` is
// a multiply by the fp32 reciprocal, as torch's device kernel does.
constexpr int kStatThreads = 1024;
template <typename DT>
__global__ void stats_kernel(const float* __restrict__ part, QuantGeom g, float clip, float levels,
                             uint16_t* __restrict__ scale, uint16_t* __restrict__ zero, float* __restrict__ thr) {
    const int bh = blockIdx.x;
    const int d = threadIdx.x % g.D;
    const int pt = threadIdx.x / g.D;
    const int nparts = kStatThreads / g.D;   // >= 4 for D <= 256
    __shared__ float sh[2 * kStatThreads];   // [part][2][D]
    float a = INFINITY, z = -INFINITY;
    const float* p = part + static_cast<int64_t>(bh) * g.nchunk * 2 * g.D;
#pragma unroll 4
    for (int c = pt; c < g.nchunk; c += nparts) {   // independent loads: four pairs in flight
        a = fminf(a, p[c * 2 * g.D + d]);
        z = fmaxf(z, p[c * 2 * g.D + g.D + d]);
    }
    sh[(pt * 2) * g.D + d] = a;
    sh[(pt * 2 + 1) * g.D + d] = z;
    __syncthreads();
    for (int q = 0; q < nparts; ++q) {
        a = fminf(a, sh[(q * 2) * g.D + d]);
        z = fmaxf(z, sh[(q * 2 + 1) * g.D + d]);
    }
    const float x_min = rnd<DT>(a * clip);
    const float x_max = rnd<DT>(z * clip);
    const float diff = rnd<DT>(x_max - x_min);
    const float inv_levels = __fdiv_rn(1.0f, levels);
    const float s = rnd<DT>(diff * inv_levels);
    const float zp = rnd<DT>(__fdiv_rn(-x_min, s));
    // thresholds thr[k-1] = smallest storage value whose code is >= k (k = 1..L), kept as
    // [k][channel].  NaN in thr[0]: the step-function argument does not hold for this channel
    // (scale not positive and finite, or zero-point NaN) and emit evaluates the chain itself.
    float* o = thr + static_cast<int64_t>(bh) * 3 * g.D + d;
    const bool monotone = s > 0.0f && s < INFINITY && zp == zp;
    if (pt == 0) {
        scale[static_cast<int64_t>(bh) * g.D + d] = static_cast<uint16_t>(Cvt<DT>::from_float(s));
        zero[static_cast<int64_t>(bh) * g.D + d] = static_cast<uint16_t>(Cvt<DT>::from_float(zp));
        return;
    }
    if (pt > 3) return;
    const int nlev = static_cast<int>(levels);
    const int k = pt;   // this thread's level
    float t = NAN;      // no value reaches code k
    if (monotone && k <= nlev) {
        int lo = Keys<DT>::lo, hi = Keys<DT>::hi;   // invariant: code(lo) < k (or lo is the floor), answer in (lo, hi]
        if (quant_value<DT>(key_value<DT>(hi), s, zp, levels) >= static_cast<float>(k)) {
            if (quant_value<DT>(key_value<DT>(lo), s, zp, levels) >= static_cast<float>(k)) {
                hi = lo;
            } else {
                while (hi - lo > 1) {
                    const int mid = lo + (hi - lo) / 2;
                    if (quant_value<DT>(key_value<DT>(mid), s, zp, levels) >= static_cast<float>(k)) hi = mid;
                    else lo = mid;
                }
            }
            t = key_value<DT>(hi);
        }
    }
    // thr[1] distinguishes "not monotone" (non-NaN) from "code 1 unreachable" (NaN)
    if (!monotone) t = (k == 2) ? 1.0f : NAN;
    o[(k - 1) * g.D] = t;
}

// Whole-tensor statistics (`per_channel=False`, calibquant.py:29-31: x.min() * scale, x.max() * scale):
// one 1024-thread workgroup folds every chunk partial into a single (min, max), runs the same op chain
// and threshold search as above, and writes one row of D identical statistics / thresholds that the
// emit kernel reads for every (batch, head), plus the two scalars the caller gets back.
template <typename DT>
__global__ __launch_bounds__(kStatThreads) void tensor_stats_kernel(const float* __restrict__ part, int64_t npairs, int D,
                                                                    float clip, float levels,
                                                                    uint16_t* __restrict__ scale_row,
                                                                    uint16_t* __restrict__ zero_row,
                                                                    float* __restrict__ thr_row,
                                                                    uint16_t* __restrict__ scale1,
                                                                    uint16_t* __restrict__ zero1) {
    __shared__ float smn[kStatThreads / kWave], smx[kStatThreads / kWave];
    __shared__ float st[2 + 3];   // scale, zero-point, thresholds
    const int tid = threadIdx.x;
    float a = INFINITY, z = -INFINITY;
    const int64_t n = npairs * 2 * D;
    for (int64_t e = tid; e < n; e += kStatThreads) {
        const float v = part[e];
        if ((e / D) & 1) z = fmaxf(z, v); else a = fminf(a, v);   // [pair][min row | max row][D]
    }
    a = wave_min(a);
    z = wave_max(z);
    if ((tid & 63) == 0) { smn[tid >> 6] = a; smx[tid >> 6] = z; }
    __syncthreads();
    if (tid == 0) {
        for (int w = 0; w < kStatThreads / kWave; ++w) { a = fminf(a, smn[w]); z = fmaxf(z, smx[w]); }
        const float x_min = rnd<DT>(a * clip);
        const float x_max = rnd<DT>(z * clip);
        const float diff = rnd<DT>(x_max - x_min);
        const float s = rnd<DT>(diff * __fdiv_rn(1.0f, levels));
        st[0] = s;
        st[1] = rnd<DT>(__fdiv_rn(-x_min, s));
    }
    __syncthreads();
    const float s = st[0], zp = st[1];
    const bool monotone = s > 0.0f && s < INFINITY && zp == zp;
    const int nlev = static_cast<int>(levels);
    if (tid < 3) {
        const int k = tid + 1;
        float t = NAN;
        if (monotone && k <= nlev) {
            int lo = Keys<DT>::lo, hi = Keys<DT>::hi;
            if (quant_value<DT>(key_value<DT>(hi), s, zp, levels) >= static_cast<float>(k)) {
                if (quant_value<DT>(key_value<DT>(lo), s, zp, levels) >= static_cast<float>(k)) {
                    hi = lo;
                } else {
                    while (hi - lo > 1) {
                        const int mid = lo + (hi - lo) / 2;
                        if (quant_value<DT>(key_value<DT>(mid), s, zp, levels) >= static_cast<float>(k)) hi = mid;
                        else lo = mid;
                    }
                }
                t = key_value<DT>(hi);
            }
        }
        if (!monotone) t = (k == 2) ? 1.0f : NAN;   // same marker as stats_kernel: emit evaluates the chain itself
        st[2 + tid] = t;
    }
    __syncthreads();
    for (int d = tid; d < D; d += kStatThreads) {
        scale_row[d] = static_cast<uint16_t>(Cvt<DT>::from_float(s));
        zero_row[d] = static_cast<uint16_t>(Cvt<DT>::from_float(zp));
        thr_row[d] = st[2];
        thr_row[D + d] = st[3];
        thr_row[2 * D + d] = st[4];
    }
    if (tid == 0) {
        scale1[0] = static_cast<uint16_t>(Cvt<DT>::from_float(s));
        zero1[0] = static_cast<uint16_t>(Cvt<DT>::from_float(zp));
    }
}

// ---- 3. emit -----------------------------------------------------------------
// XQ = false: packed codes (B, H, T, D*BITS/8).  XQ = true: the unpacked code
// values as storage-dtype numbers in a contiguous (B, T, H, D) tensor.
template <typename DT, int BITS, bool XQ>
__global__ __launch_bounds__(kQThreads) void emit_kernel(const uint16_t* __restrict__ x, QuantGeom g,
                                                        const uint16_t* __restrict__ scale,
                                                        const uint16_t* __restrict__ zero,
                                                        const float* __restrict__ thr,
                                                        uint8_t* __restrict__ codes, uint16_t* __restrict__ xq) {
    const int lpr = g.D >> 3;
    const int rows_per_iter = kQThreads / lpr;
    const int lane = threadIdx.x % lpr;
    const int row = threadIdx.x / lpr;
    // chunks are walked in the reverse order of the min / max launch: what that launch read last is
    // still in the memory-side cache when this one starts
    const int c = gridDim.x - 1 - blockIdx.x, h = gridDim.y - 1 - blockIdx.y, b = gridDim.z - 1 - blockIdx.z;
    const int t0 = c * g.chunk;
    const int t1 = min(g.T, t0 + g.chunk);
    const uint16_t* base = x + b * g.sb + h * g.sh + lane * 8;
    const int64_t bh = static_cast<int64_t>(b) * g.H + h;
    const int64_t sbh = g.shared_stats ? 0 : bh;   // row of the statistics / threshold arrays
    constexpr float levels = static_cast<float>((1 << BITS) - 1);

    float s[8], zp[8];
    {
        uint4 sv = *reinterpret_cast<const uint4*>(scale + sbh * g.D + lane * 8);
        uint4 zv = *reinterpret_cast<const uint4*>(zero + sbh * g.D + lane * 8);
        unpack8<DT>(sv, s);
        unpack8<DT>(zv, zp);
    }
    // thresholds of this lane's 8 channels (all three levels are loaded, as vectors, whatever BITS is);
    // `slow`: a channel without the step-function property
    float th[3][8];
    bool slow = false;
    {
        const float4* tp = reinterpret_cast<const float4*>(thr + sbh * 3 * g.D + lane * 8);
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const float4 a = tp[k * (g.D >> 2)], c4 = tp[k * (g.D >> 2) + 1];
            th[k][0] = a.x; th[k][1] = a.y; th[k][2] = a.z; th[k][3] = a.w;
            th[k][4] = c4.x; th[k][5] = c4.y; th[k][6] = c4.z; th[k][7] = c4.w;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) slow = slow | ((th[0][i] != th[0][i]) & (th[1][i] == th[1][i]));
    }
    const int nb = g.D * BITS / 8;  // bytes per packed row
    // dword stores: the lanes of a quad sit in one row (16 or 32 lanes per row) and combine their bytes
    const bool wide = !XQ && (lpr % 4) == 0 && (reinterpret_cast<uintptr_t>(codes) & 3u) == 0;
    const int64_t step = rows_per_iter * g.st;
    const uint16_t* rp = base + (t0 + row) * g.st;
    const uint16_t* last = base + (t1 - 1) * g.st;   // rows past the chunk re-read its last row
    for (int tb = t0 + row; tb < t1; tb += kQUnroll * rows_per_iter, rp += kQUnroll * step) {
        uint4 v[kQUnroll];   // four rows in flight per thread
#pragma unroll
        for (int u = 0; u < kQUnroll; ++u)
            v[u] = *reinterpret_cast<const uint4*>(tb + u * rows_per_iter < t1 ? rp + u * step : last);
#pragma unroll
        for (int u = 0; u < kQUnroll; ++u) {
            const int t = tb + u * rows_per_iter;
            if (t >= t1) break;   // uniform over the lanes of a row
            float f[8];
            unpack8<DT>(v[u], f);
            if constexpr (XQ) {
                float qv[8];
                if (!slow) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        qv[i] = (f[i] >= th[0][i]) ? 1.0f : 0.0f;
                        if constexpr (BITS == 2) {
                            qv[i] += (f[i] >= th[1][i]) ? 1.0f : 0.0f;
                            qv[i] += (f[i] >= th[2][i]) ? 1.0f : 0.0f;
                        }
                        qv[i] = (f[i] != f[i]) ? f[i] : qv[i];   // a NaN input stays NaN in x_q
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) qv[i] = quant_value<DT>(f[i], s[i], zp[i], levels);
                }
                uint32_t w[4];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    w[i] = Cvt<DT>::from_float(qv[2 * i]) | (Cvt<DT>::from_float(qv[2 * i + 1]) << 16);
                uint16_t* o = xq + ((static_cast<int64_t>(b) * g.T + t) * g.H + h) * g.D + lane * 8;
                *reinterpret_cast<uint4*>(o) = make_uint4(w[0], w[1], w[2], w[3]);
            } else {
                uint32_t code[8];
                if (!slow) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) {   // a NaN input compares false: code 0
                        code[i] = (f[i] >= th[0][i]) ? 1u : 0u;
                        if constexpr (BITS == 2) {
                            code[i] += (f[i] >= th[1][i]) ? 1u : 0u;
                            code[i] += (f[i] >= th[2][i]) ? 1u : 0u;
                        }
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const float qv = quant_value<DT>(f[i], s[i], zp[i], levels);
                        code[i] = (qv != qv) ? 0u : static_cast<uint32_t>(qv);
                    }
                }
                uint8_t* o = codes + (bh * g.T + t) * nb;
                if constexpr (BITS == 1) {
                    uint32_t byte = 0;
#pragma unroll
                    for (int i = 0; i < 8; ++i) byte |= code[i] << (7 - i);
                    if (wide) {
                        int w = static_cast<int>(byte << (8 * (lane & 3)));
                        w |= dpp_move_i<0xB1>(w, 0);
                        w |= dpp_move_i<0x4E>(w, 0);
                        if ((lane & 3) == 0) *reinterpret_cast<uint32_t*>(o + lane) = static_cast<uint32_t>(w);
                    } else {
                        o[lane] = static_cast<uint8_t>(byte);
                    }
                } else {
                    const uint32_t b0 = (code[0] << 6) | (code[1] << 4) | (code[2] << 2) | code[3];
                    const uint32_t b1 = (code[4] << 6) | (code[5] << 4) | (code[6] << 2) | code[7];
                    const uint32_t half = b0 | (b1 << 8);
                    if (wide) {
                        int w = static_cast<int>(half << (16 * (lane & 1)));
                        w |= dpp_move_i<0xB1>(w, 0);
                        if ((lane & 1) == 0) *reinterpret_cast<uint32_t*>(o + 2 * lane) = static_cast<uint32_t>(w);
                    } else {
                        reinterpret_cast<uint16_t*>(o)[lane] = static_cast<uint16_t>(half);
                    }
                }
            }
        }
    }
}

// ---- one-pass quantise and pack ------------------------------------------------------------
// A 1024-thread workgroup owns (batch, head, quarter of the channels): 32 channels = 64 bytes of
// every token row, T <= 3328 tokens, which is 16 bytes x up to 13 rows per thread - the slice
// stays in registers between the min/max and the emit, so x is read from HBM once.
// thread = (row r = tid / 4 of a 256-row pass, 16-byte piece q = tid % 4).
constexpr int kFThreads = 1024;
constexpr int kFRows = 13;                  // rows per thread at most (13 x 256 = 12 tiles + thumbnail of 256 tokens)
constexpr int kFMaxT = kFRows * (kFThreads / 4);
constexpr int kFGridDefault = 256;          // workgroups of the persistent launch when no device can be asked: a whole MI355X
// rows per thread of the next slice that are staged in LDS (16 KB each for the workgroup)
// (not with the rotary embedding fused in: that instantiation has no registers to spare for the addresses).
// The staged loads are assembly that the compiler does not see (m0, their own wait count): building with
// -DCQ_NO_LDS_STAGE refills every row from memory through registers instead, for a toolchain that breaks them.
#ifdef CQ_NO_LDS_STAGE
constexpr int fused_stage_rows(int, bool) { return 0; }
#else
constexpr int fused_stage_rows(int nr, bool rope) { return (nr > 8 && !rope) ? 8 : 0; }
#endif

// Rotary embedding fused into the pass (ROPE): x is the un-rotated key block; every row is rotated as it
// arrives - rnd(rnd(x * cos) + rotate_half(x) * sin), the arithmetic of the ops the reference runs on the
// whole key tensor before it quantises the image slice (patch_internvl.py:125-134, 258-260, 295-297) - the
// rotated row is written out once (the prefill attention and the caller's cache need it) and quantised from
// the registers.  A channel d pairs with d + 64, so the 32 channels of a slice are then 16 of the lower half
// and the matching 16 of the upper half (pieces 0, 1 / 2, 3 of a row's four lanes): the partner's raw values
// are two lanes away, no second read of x.
struct RopeArgs {
    const uint16_t* cos;      // (table_rows, 128) in the storage dtype
    const uint16_t* sin;
    const int64_t* pos;       // position id of (b, t) at pos[b * pos_sb + t * pos_st]; NULL: pos0 + t
    int64_t pos_sb, pos_st, pos0, table_rows;
    uint16_t* out;            // rotated rows, (B, T, H, 128) through element strides
    int64_t ob, ot, oh;
    // cq_rope_rows_grouped: every head is a group of `gn` rows, `gs` elements apart in x and `og` in out
    int gn = 1;
    int64_t gs = 0, og = 0;
};

// SPLIT: the token axis is longer than NR * 256 rows: 2^g.parts_log2 workgroups share a slice, each with g.part_rows
// of its rows (<= NR * 256) in registers, and exchange their channels' min / max before the statistics - x is still
// read once.  The parts of a slice are consecutive ids, i.e. they are worked on by different workgroups of the
// persistent launch in the same step of their walks (the grid is a multiple of the part count), all of them
// resident: whoever waits, waits for workgroups that are running.
template <typename DT, int BITS, int NR, bool ROPE = false, bool SPLIT = false>   // NR: rows per thread (T <= NR * 256)
__global__ __launch_bounds__(kFThreads) void fused_pack_kernel(const uint16_t* __restrict__ x, QuantGeom g, float clip,
                                                              uint16_t* __restrict__ scale,
                                                              uint16_t* __restrict__ zero,
                                                              uint8_t* __restrict__ codes, RopeArgs ra) {
    constexpr int L = (1 << BITS) - 1;
    constexpr float levels = static_cast<float>(L);
    __shared__ __attribute__((aligned(16))) float part_mn[32][kFThreads / 16];   // [channel][wave * 4 + row of 16 lanes]
    __shared__ __attribute__((aligned(16))) float part_mx[32][kFThreads / 16];
    __shared__ float s_s[32], s_z[32], s_thr[3][32];
    // NP rows per thread of the NEXT slice travel through LDS: they are requested as soon as this slice's min / max
    // fold has read the registers - global-to-LDS loads that need no register to land in - so HBM stays busy
    // through the statistics and threshold phases, in which nothing else is in flight; the emit then refills those
    // rows' registers from LDS and only the other NR - NP rows from memory.
    constexpr int NP = fused_stage_rows(NR, ROPE);
    extern __shared__ __attribute__((aligned(16))) unsigned char stage[];   // [NP][thread][16 bytes]
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int q4 = tid & 3, row = tid >> 2;
    // A workgroup walks slices blockIdx.x, blockIdx.x + gridDim.x, ... (gridDim.x is a multiple
    // of 32).  The four quarters of one (batch, head) sit on one XCD (slice ids 8 apart), so the
    // four 4-byte pieces of a packed row meet in one L2.  While a slice's rows are emitted, every
    // row's registers are refilled with the same row of the next slice: its loads are in flight
    // during the emit and its min / max pass starts without a wait.
    const int plog = SPLIT ? g.parts_log2 : 0;
    const int64_t nbh = static_cast<int64_t>(g.B) * g.H;
    // Slice vb -> (quarter, (batch, head) pair).  Workgroup l of the launch runs on die l % 8 and its ids are a
    // multiple of 8 apart, so the low three bits of an id are the die: of an unsplit slice the low three bits of vb,
    // of a slice split four ways the part and the lowest bit of vb.  The four quarters of a pair always share a
    // die (their 4-byte pieces of a packed row meet in one L2, and two quarters share every 128-byte line of x).
    // Narrow map: the low bits of vb are the low bits of the pair index - with eight heads, of the head.  Wide
    // map: they select among eight runs of eight consecutive pairs - with eight heads, among batch rows - and the
    // place in the run comes from bits 5-7.  For split slices of a contiguous (B, T, H, D) tensor the wide map
    // puts all heads of a token row (one contiguous 2 KB) on one die, where the narrow one spreads them over two
    // or more; the host picks it there (measured, see wide_map_for()).
    const int wide = g.wide_map;
    const int nslice = (wide ? static_cast<int>((nbh + 63) / 64) * 256 : static_cast<int>((nbh + 7) / 8) * 32) << plog;   // ids: slice * parts + part
    auto slice_of = [&](int vb, int& quarter) -> int64_t {
        if (wide) {
            quarter = (vb >> 3) & 3;
            return (static_cast<int64_t>(vb >> 8) * 8 + (vb & 7)) * 8 + ((vb >> 5) & 7);
        }
        quarter = (vb >> 3) & 3;
        return static_cast<int64_t>(vb >> 5) * 8 + (vb & 7);
    };
    auto part_first = [&](int id) { return SPLIT ? (id & ((1 << plog) - 1)) * g.part_rows : 0; };        // first row of the id's part
    auto part_len = [&](int id) { return SPLIT ? min(g.T - part_first(id), g.part_rows) : g.T; };       // rows of it
    // The slice's base is the same for the whole workgroup and a row's piece sits at a 32-bit byte
    // offset from it (the host checks T * row stride < 2^24 bytes): a load takes its address as
    // scalar base + vector offset, one 24-bit multiply-add per row.
    auto slice_base = [&](int id) -> const unsigned char* {   // slices past the last (batch, head) alias the last one
        const int vb = id >> plog;
        int quarter;
        const uint32_t bh = static_cast<uint32_t>(min(slice_of(vb, quarter), nbh - 1));
        const uint32_t b = g.dH.quot(bh), h = bh - b * g.dH.div;   // B * H < 2^31 on this path
        return reinterpret_cast<const unsigned char*>(x + static_cast<int64_t>(b) * g.sb + static_cast<int64_t>(h) * g.sh +
                                                      static_cast<int64_t>(part_first(id)) * g.st + quarter * (ROPE ? 16 : 32));
    };
    // first channel of the thread's piece, less the slice's own offset (quarter * 32, or quarter * 16 with ROPE)
    const int chan_t = ROPE ? (q4 >> 1) * 64 + (q4 & 1) * 8 : q4 * 8;
    const uint32_t st_bytes = static_cast<uint32_t>(g.st) * 2u, q_bytes = static_cast<uint32_t>(chan_t) * 2u;
    auto row_offset = [&](int t, int len) -> uint32_t {   // byte offset of the thread's piece of row min(t, len - 1) of a slice (part)
        return static_cast<uint32_t>(__umul24(static_cast<uint32_t>(min(t, len - 1)), st_bytes)) + q_bytes;
    };
    typedef uint32_t U4 __attribute__((ext_vector_type(4)));
    U4 v[NR];
    {
        const unsigned char* base = slice_base(blockIdx.x);
        const int len0 = part_len(blockIdx.x);
#pragma unroll
        for (int i = 0; i < NR; ++i)   // rows past T re-read row T-1: min / max unchanged, never written
            v[i] = *reinterpret_cast<const U4*>(base + row_offset(i * (kFThreads / 4) + row, len0));
    }
    for (int id = blockIdx.x; id < nslice; id += gridDim.x) {
    const int vb = id >> plog;
    int quarter;
    const int64_t bh = slice_of(vb, quarter);
    const bool live = bh < nbh;                         // a padding slice computes and writes nothing
    const bool has_next = id + static_cast<int>(gridDim.x) < nslice;
    const int next_id = has_next ? id + gridDim.x : id;
    const unsigned char* next_base = slice_base(next_id);
    const int t_first = part_first(id), t_len = part_len(id), next_len = part_len(next_id);
    int row_i = row;   // opaque per iteration: the row offsets below are recomputed, not kept in registers across the loop
    asm volatile("" : "+v"(row_i));
    if constexpr (ROPE) {
        const uint32_t bhc = static_cast<uint32_t>(min(bh, nbh - 1));
        const uint32_t bb = g.dH.quot(bhc), hh = bhc - bb * g.dH.div;
        const int chan0 = quarter * 16 + chan_t;
        uint16_t* orow = ra.out + static_cast<int64_t>(bb) * ra.ob + static_cast<int64_t>(hh) * ra.oh + chan0;
        const bool upper = (q4 >> 1) != 0;
        const int64_t* pos_p = ra.pos ? ra.pos + static_cast<int64_t>(bb) * ra.pos_sb : reinterpret_cast<const int64_t*>(ra.cos);
        const int64_t pos_st = ra.pos ? ra.pos_st : 0;
        const int64_t trow_max = ra.table_rows - 1;
        const uint32_t ysign = upper ? 0u : 0x80008000u;   // rotate_half(x) = (-x2, x1): the lower half takes minus its partner
        // the table rows of GR rows at a time are requested before the first of them is used: every request
        // is a round trip to the L2, and one row after the other would make a slice wait for NR of them in turn
        constexpr int GR = 2;
#pragma unroll
        for (int i0 = 0; i0 < NR; i0 += GR) {
            U4 cw[GR], sw[GR];
#pragma unroll
            for (int k = 0; k < GR; ++k) {
                if (i0 + k < NR) {
                    const int t = min((i0 + k) * (kFThreads / 4) + row_i, g.T - 1);
                    // no control flow around the loads (the compiler then requests a group's rows side by side):
                    // without a position tensor the load reads a valid dummy and the select takes pos0 + t
                    const int64_t pv = pos_p[static_cast<int64_t>(t) * pos_st];
                    const int64_t pl = ra.pos ? pv : ra.pos0 + t;
                    // clamped to the table in 32 bits (the host checks table_rows < 2^24)
                    const uint32_t ps = static_cast<uint32_t>(pl < 0 ? 0 : (pl > trow_max ? trow_max : pl));
                    cw[k] = *reinterpret_cast<const U4*>(ra.cos + __umul24(ps, 128u) + chan0);
                    sw[k] = *reinterpret_cast<const U4*>(ra.sin + __umul24(ps, 128u) + chan0);
                }
            }
#pragma unroll
            for (int k = 0; k < GR; ++k) {
                if (i0 + k < NR) {
                    const int i = i0 + k;
                    const int t = min(i * (kFThreads / 4) + row_i, g.T - 1);
                    U4 pw;   // the partner's raw piece: the lane two away holds channel d +- 64 of the same row
#pragma unroll
                    for (int w = 0; w < 4; ++w)
                        pw[w] = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v[i][w]), 0x4E, 0xf, 0xf, true)) ^ ysign;
                    U4 r4;
#pragma unroll
                    for (int w = 0; w < 4; ++w) {   // a word (two elements) at a time: few values live at once
                        const float x0 = Cvt<DT>::lo(v[i][w]), x1 = Cvt<DT>::hi(v[i][w]);
                        const float y0 = Cvt<DT>::lo(pw[w]), y1 = Cvt<DT>::hi(pw[w]);
                        const float c0 = Cvt<DT>::lo(cw[k][w]), c1 = Cvt<DT>::hi(cw[k][w]);
                        const float s0 = Cvt<DT>::lo(sw[k][w]), s1 = Cvt<DT>::hi(sw[k][w]);
                        const uint32_t o0 = Cvt<DT>::from_float(rnd<DT>(x0 * c0) + y0 * s0);   // y carries the sign of rotate_half
                        const uint32_t o1 = Cvt<DT>::from_float(rnd<DT>(x1 * c1) + y1 * s1);
                        r4[w] = o0 | (o1 << 16);
                    }
                    v[i] = r4;
                    // unconditional store: a row past T repeats row T - 1 and a padding slice repeats the last
                    // (batch, head), so whatever is written twice is written with the same bits
                    *reinterpret_cast<U4*>(orow + static_cast<int64_t>(t) * ra.ot) = r4;
                }
            }
        }
    }
    // Both storage types are sign-magnitude, so the extremes of a column follow from three packed
    // 16-bit integer folds of the raw words, two elements per instruction and no unpacking: as
    // signed integers the non-negative values are in value order (the signed maximum is the
    // largest of them, if there is one); as unsigned integers the negative values lie above every
    // non-negative one, in order of magnitude (the unsigned maximum is the most negative value,
    // if there is one; the unsigned minimum is the smallest non-negative value, or with negatives
    // only the one nearest to zero).  -0 counts as negative and orders below +0.
    typedef short S2 __attribute__((ext_vector_type(2)));
    typedef unsigned short US2 __attribute__((ext_vector_type(2)));
    uint32_t k_smax[4], k_umin[4], k_umax[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) { k_smax[w] = 0x80008000u; k_umin[w] = 0xffffffffu; k_umax[w] = 0u; }
#pragma unroll
    for (int i = 0; i < NR; ++i) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const uint32_t r = v[i][w];
            k_smax[w] = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(S2, k_smax[w]), __builtin_bit_cast(S2, r)));
            k_umin[w] = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(US2, k_umin[w]), __builtin_bit_cast(US2, r)));
            k_umax[w] = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(US2, k_umax[w]), __builtin_bit_cast(US2, r)));
        }
    }
    if constexpr (NP > 0) {
        if (has_next) {
            // lane l of a wave lands at the wave's base + 16 l: thread tid's piece of row i at stage[i][tid].
            // Written as assembly: the compiler waits for a global-to-LDS load it knows of before the next LDS
            // instruction of any kind, which would take the loads out of flight again at once.  The fold's
            // results are operands of the first statement only to place the loads after the fold, i.e. after the
            // compiler's own wait for the rows that came through registers; unknown to the compiler, the loads
            // can only make its later vector-memory waits stricter, never weaker, and the wait before the
            // staged pieces are read back is written out below.  (m0, the LDS base of such a load, has no other
            // use in this kernel; the compiler reserves it and does not accept it as a clobber.)
            const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(stage)) +
                                  static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(wv)) * 1024u;
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const uint32_t off = row_offset(i * (kFThreads / 4) + row_i, next_len);
                const uint32_t ldsa = lds0 + static_cast<uint32_t>(i) * (kFThreads * 16);
                if (i == 0)
                    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %2"
                                 :
                                 : "v"(off), "s"(ldsa), "s"(next_base), "v"(k_smax[0]), "v"(k_smax[1]), "v"(k_smax[2]),
                                   "v"(k_smax[3]), "v"(k_umin[0]), "v"(k_umin[1]), "v"(k_umin[2]), "v"(k_umin[3]),
                                   "v"(k_umax[0]), "v"(k_umax[1]), "v"(k_umax[2]), "v"(k_umax[3])
                                 : "memory");
                else
                    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %2"
                                 :
                                 : "v"(off), "s"(ldsa), "s"(next_base)
                                 : "memory");
            }
        }
    }
    float mn[8], mx[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int sh = 16 * (j & 1);
        const uint32_t smax = (k_smax[j >> 1] >> sh) & 0xffffu, umin = (k_umin[j >> 1] >> sh) & 0xffffu,
                       umax = (k_umax[j >> 1] >> sh) & 0xffffu;
        mn[j] = Cvt<DT>::to_float((umax & 0x8000u) ? umax : umin);
        mx[j] = Cvt<DT>::to_float((smax & 0x8000u) ? umin : smax);
    }
    // lanes l, l+4, l+8, l+12 of a row of 16 lanes hold the same channels: two rotations fold them
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        mn[j] = fminf(mn[j], dpp_move<0x124>(mn[j], INFINITY));   // row_ror:4
        mn[j] = fminf(mn[j], dpp_move<0x128>(mn[j], INFINITY));   // row_ror:8
        mx[j] = fmaxf(mx[j], dpp_move<0x124>(mx[j], -INFINITY));
        mx[j] = fmaxf(mx[j], dpp_move<0x128>(mx[j], -INFINITY));
    }
    if ((lane & 15) < 4) {
        const int p = wv * 4 + (lane >> 4);
#pragma unroll
        for (int j = 0; j < 8; ++j) { part_mn[q4 * 8 + j][p] = mn[j]; part_mx[q4 * 8 + j][p] = mx[j]; }
    }
    __syncthreads();
    // channel c of the quarter: 16 lanes fold its 64 partials (four each, then across the row),
    // the first of them runs the statistics chain
    if (tid < 32 * 16) {
        const int c = tid >> 4, p16 = tid & 15;
        const float4 a4 = *reinterpret_cast<const float4*>(&part_mn[c][4 * p16]);
        const float4 z4 = *reinterpret_cast<const float4*>(&part_mx[c][4 * p16]);
        float a = fminf(fminf(a4.x, a4.y), fminf(a4.z, a4.w));
        float z = fmaxf(fmaxf(z4.x, z4.y), fmaxf(z4.z, z4.w));
        a = row_reduce(a, OpMin(), INFINITY);
        z = row_reduce(z, OpMax(), -INFINITY);
        if constexpr (SPLIT) {
            if (p16 == 0 && live) {
                // This part's extremes of channel c go out as two self-validating records; then the records of all
                // parts of the slice are polled (device-scope loads, a bounded number of times) and folded.  The
                // other parts are being worked on right now by other workgroups of this launch.
                const unsigned long long tag = static_cast<unsigned long long>(g.epoch) << 32;
                unsigned long long* mine = g.rec + (static_cast<int64_t>(id) * 32 + c) * 2;
                __hip_atomic_store(mine, tag | __float_as_uint(a), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(mine + 1, tag | __float_as_uint(z), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const int nparts = 1 << plog;
                const unsigned long long* first = g.rec + (static_cast<int64_t>(id & ~(nparts - 1)) * 32 + c) * 2;
                bool ok = false;
                float fa = a, fz = z;
                for (int it = 0; it < g.spin_limit && !ok; ++it) {
                    ok = true;
                    fa = a; fz = z;
                    for (int pp = 0; pp < nparts; ++pp) {
                        const unsigned long long lo = __hip_atomic_load(first + pp * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        const unsigned long long hi = __hip_atomic_load(first + pp * 64 + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        ok = ok && static_cast<uint32_t>(lo >> 32) == g.epoch && static_cast<uint32_t>(hi >> 32) == g.epoch;
                        // (a NaN extreme of any part stays one, as it does inside a part)
                        const float pa = __uint_as_float(static_cast<uint32_t>(lo)), pz = __uint_as_float(static_cast<uint32_t>(hi));
                        fa = (fa != fa || pa != pa) ? NAN : fminf(fa, pa);
                        fz = (fz != fz || pz != pz) ? NAN : fmaxf(fz, pz);
                    }
                    if (!ok) __builtin_amdgcn_s_sleep(2);
                }
                if (ok) { a = fa; z = fz; }
                else if (g.status) __hip_atomic_store(g.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);   // this call's result is not valid
            }
        }
        if (p16 == 0 && live) {
            const float x_min = rnd<DT>(a * clip);
            const float x_max = rnd<DT>(z * clip);
            const float diff = rnd<DT>(x_max - x_min);
            const float sc = rnd<DT>(diff * __fdiv_rn(1.0f, levels));
            const float zp = rnd<DT>(__fdiv_rn(-x_min, sc));
            const int64_t o = bh * g.D + (ROPE ? (c >> 4) * 64 + quarter * 16 + (c & 15) : quarter * 32 + c);
            if (!SPLIT || t_first == 0) {   // (one of the parts writes them)
                scale[o] = static_cast<uint16_t>(Cvt<DT>::from_float(sc));
                zero[o] = static_cast<uint16_t>(Cvt<DT>::from_float(zp));
            }
            s_s[c] = sc;
            s_z[c] = zp;
        }
    }
    __syncthreads();
    // thresholds (see the statistics kernel): one 16-ary search per (channel, level) and group of
    // 16 lanes, four rounds narrow the 2^16 ordered storage values down to one; a wave runs four
    // searches side by side.  The code is a non-decreasing function of x for every (scale,
    // zero-point) the chain can produce - also for scale 0 (x / 0 is -inf, NaN, +inf in that order
    // and NaN maps to code 0) and for NaN statistics (every code 0) - so the search runs for
    // every channel.
    {
        const int grp = lane >> 4, l16 = lane & 15;
        for (int sid0 = wv * 4; sid0 < 32 * L; sid0 += kFThreads / 16) {
            const int sid = min(sid0 + grp, 32 * L - 1);   // a group past the end repeats the last search
            const int c = sid / L, k = sid % L + 1;
            const float sc = s_s[c], zp = s_z[c];
            int lo = Keys<DT>::lo - 1, hi = Keys<DT>::hi;   // code(lo) < k (lo may be the virtual floor), answer in (lo, hi]
            bool reach = true;
#pragma unroll
            for (int round = 0; round < 4; ++round) {
                const int step = (hi - lo + 15) / 16;
                const int key = min(lo + (l16 + 1) * step, hi);
                const bool pred = quant_value<DT>(key_value<DT>(key), sc, zp, levels) >= static_cast<float>(k);
                const unsigned long long m = __ballot(pred);
                const uint32_t mg = static_cast<uint32_t>(m >> (16 * grp)) & 0xffffu;   // the group's lanes
                reach = reach && mg != 0;
                const int f = mg ? __builtin_ctz(mg) : 0;
                hi = min(lo + (f + 1) * step, hi);
                lo = lo + f * step;
            }
            // stays NaN if no value reaches code k
            if (l16 == 0 && sid0 + grp < 32 * L) s_thr[k - 1][c] = reach ? key_value<DT>(hi) : NAN;
        }
    }
    __syncthreads();
    float th[L][8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int k = 0; k < L; ++k) th[k][j] = s_thr[k][q4 * 8 + j];
    constexpr int nb = 128 * BITS / 8;   // bytes per packed row
#pragma unroll
    for (int e = 0; e < NR; ++e) {
        // the rows refilled from memory go first (their loads then have the rest of the emit to land), the
        // staged rows after them
        const int i = (e + NP) % NR;
        if constexpr (NP > 0) {
            if (e == NR - NP) {
                // Every staged piece has landed once at most NR - NP younger memory operations are outstanding
                // (the refills just issued; stores issued since only make the wait stricter).  A thread reads
                // back exactly the bytes its own lane requested, so no barrier is needed.
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NR - NP) : "memory");
            }
        }
        const int t = i * (kFThreads / 4) + row_i;
        // (the empty statement keeps the compiler from carrying the unpacked floats of the
        // min/max pass over to here: that would double the registers the slice needs)
        asm volatile("" : "+v"(v[i]));
        float f[8];
        unpack8<DT>(v[i], f);
        uint32_t code[8];
        if constexpr (BITS == 2) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                code[j] = ((f[j] >= th[0][j]) ? 1u : 0u) + ((f[j] >= th[1][j]) ? 1u : 0u) + ((f[j] >= th[2][j]) ? 1u : 0u);
        }
        // ROPE: the quad's bytes are two pairs, the lower-half pair at quarter * nb / 8 and the upper-half pair nb / 2 further
        uint8_t* o = codes + (min(bh, nbh - 1) * g.T + t_first + min(t, t_len - 1)) * nb + (ROPE ? quarter * (nb / 8) : quarter * (nb / 4));
        if constexpr (BITS == 1) {
            // The byte is built by eight add-with-carry steps, w = w + w + (f[j] >= th[j]): each
            // comparison leaves its lane mask in a scalar register pair of its own and the add
            // takes it as the carry-in (two instructions per element; a compare, a select and an
            // OR otherwise).  The compares come first, so every mask is read at least two
            // instructions after it is written, as this chip requires of a vector instruction
            // that reads a scalar register written by another.
            uint32_t w = 0;
            unsigned long long m0, m1, m2, m3, m4, m5, m6, m7;
            asm volatile(
                "v_cmp_le_f32_e64 %[m0], %[t0], %[f0]\n\t"
                "v_cmp_le_f32_e64 %[m1], %[t1], %[f1]\n\t"
                "v_cmp_le_f32_e64 %[m2], %[t2], %[f2]\n\t"
                "v_cmp_le_f32_e64 %[m3], %[t3], %[f3]\n\t"
                "v_cmp_le_f32_e64 %[m4], %[t4], %[f4]\n\t"
                "v_cmp_le_f32_e64 %[m5], %[t5], %[f5]\n\t"
                "v_cmp_le_f32_e64 %[m6], %[t6], %[f6]\n\t"
                "v_cmp_le_f32_e64 %[m7], %[t7], %[f7]\n\t"
                "v_addc_co_u32_e64 %[w], %[m0], %[w], %[w], %[m0]\n\t"
                "v_addc_co_u32_e64 %[w], %[m1], %[w], %[w], %[m1]\n\t"
                "v_addc_co_u32_e64 %[w], %[m2], %[w], %[w], %[m2]\n\t"
                "v_addc_co_u32_e64 %[w], %[m3], %[w], %[w], %[m3]\n\t"
                "v_addc_co_u32_e64 %[w], %[m4], %[w], %[w], %[m4]\n\t"
                "v_addc_co_u32_e64 %[w], %[m5], %[w], %[w], %[m5]\n\t"
                "v_addc_co_u32_e64 %[w], %[m6], %[w], %[w], %[m6]\n\t"
                "v_addc_co_u32_e64 %[w], %[m7], %[w], %[w], %[m7]"
                : [w] "+v"(w), [m0] "=&s"(m0), [m1] "=&s"(m1), [m2] "=&s"(m2), [m3] "=&s"(m3),
                  [m4] "=&s"(m4), [m5] "=&s"(m5), [m6] "=&s"(m6), [m7] "=&s"(m7)
                : [t0] "v"(th[0][0]), [t1] "v"(th[0][1]), [t2] "v"(th[0][2]), [t3] "v"(th[0][3]),
                  [t4] "v"(th[0][4]), [t5] "v"(th[0][5]), [t6] "v"(th[0][6]), [t7] "v"(th[0][7]),
                  [f0] "v"(f[0]), [f1] "v"(f[1]), [f2] "v"(f[2]), [f3] "v"(f[3]),
                  [f4] "v"(f[4]), [f5] "v"(f[5]), [f6] "v"(f[6]), [f7] "v"(f[7]));
            w <<= 8 * q4;
            w |= static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(w), 0xB1, 0xf, 0xf, true));
            w |= static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(w), 0x4E, 0xf, 0xf, true));
            if constexpr (ROPE) {
                if ((q4 & 1) == 0 && t < t_len && live)
                    *reinterpret_cast<uint16_t*>(o + (q4 >> 1) * (nb / 2)) = static_cast<uint16_t>(w >> (8 * q4));
            } else {
                if (q4 == 0 && t < t_len && live) *reinterpret_cast<uint32_t*>(o) = w;
            }
        } else {
            const uint32_t b0 = (code[0] << 6) | (code[1] << 4) | (code[2] << 2) | code[3];
            const uint32_t b1 = (code[4] << 6) | (code[5] << 4) | (code[6] << 2) | code[7];
            const uint32_t half = b0 | (b1 << 8);
            const uint32_t other = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(half), 0xB1, 0xf, 0xf, true));
            if constexpr (ROPE) {
                if ((q4 & 1) == 0 && t < t_len && live) *reinterpret_cast<uint32_t*>(o + (q4 >> 1) * (nb / 2)) = half | (other << 16);
            } else {
                if ((q4 & 1) == 0 && t < t_len && live) reinterpret_cast<uint32_t*>(o)[q4 >> 1] = half | (other << 16);
            }
        }
        // the row is packed: its registers take the same row of the next slice
        if (has_next) {
            if (i < NP) v[i] = *reinterpret_cast<const U4*>(stage + (i * kFThreads + tid) * 16);
            else v[i] = *reinterpret_cast<const U4*>(next_base + row_offset(t, next_len));
        }
    }
    }
}

// Raises a kernel's dynamic-LDS limit (the default stops at 64 KB); asked of the runtime once per kernel and device.
static int allow_dynamic_lds(const void* kernel, int bytes) {
    struct Done { const void* k; uint64_t devices; };
    static std::mutex mu;
    static std::vector<Done> done;
    int dev = 0;
    CQ_HIP_CHECK(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(mu);
    for (auto& d : done)
        if (d.k == kernel) {
            if (d.devices >> (dev & 63) & 1) return CQ_OK;
            CQ_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
            d.devices |= 1ull << (dev & 63);
            return CQ_OK;
        }
    CQ_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    done.push_back({kernel, 1ull << (dev & 63)});
    return CQ_OK;
}

template <typename DT, int BITS, int NR, bool ROPE, bool SPLIT = false>
static int launch_fused(dim3 grid, hipStream_t st, const uint16_t* xp, const QuantGeom& g, float clip, uint16_t* sp,
                        uint16_t* zp, uint8_t* codes, const RopeArgs& ra) {
    constexpr int lds = fused_stage_rows(NR, ROPE) * kFThreads * 16;
    auto kf = fused_pack_kernel<DT, BITS, NR, ROPE, SPLIT>;
    if (lds) {
        const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kf), lds);
        if (rc != CQ_OK) return rc;
    }
    hipLaunchKernelGGL(kf, grid, dim3(kFThreads), lds, st, xp, g, clip, sp, zp, codes, ra);
    return CQ_OK;
}

// true if the shape goes through the one-pass kernel (x read once, slice by slice in registers)
// Compute units of the current device, asked once per process.
static int persistent_units() {
    static std::atomic<int> cached{0};
    int n = cached.load(std::memory_order_relaxed);
    if (n > 0) return n;
    int dev = 0, cu = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cu < 1) {
        (void)hipGetLastError();   // not an error of the caller's
        cu = kFGridDefault;
    }
    cached.store(cu, std::memory_order_relaxed);
    return cu;
}

// ---- a token axis longer than one workgroup's registers: several workgroups per slice (SPLIT) ----------------
// Parts per slice (a power of two up to 32, so that it divides the persistent grid), rows per part and per thread:
// the choice that loads the fewest rows (a thread's rows past its part's end repeat the part's last row).  Only with
// more than eight rows per thread, the instantiations that stage the next slice's rows through LDS: measured against
// the three launches (partial min / max, statistics, emit - whose second read of x comes from the memory-side cache)
// on one device, 1 bit, (batch, tokens, 8 heads): strided view of a fused projection (16, 9 984) 105 against 126 us,
// (64, 5 000) 224 against 263 us, contiguous (16, 9 984) 123 against 123 us; with eight rows per thread and no
// staging (8, 32 768) 265 against 205 us.
struct SplitPlan { int plog, part_rows, nr; };
static bool split_plan(int T, SplitPlan* sp) {
    static const int kRowOptions[2] = {10, 13};
    int64_t best = -1;
    for (int plog = 1; plog <= 5; ++plog) {
        const int parts = 1 << plog;
        const int rows = (T + parts - 1) / parts;
        if (rows > kFMaxT || static_cast<int64_t>(parts - 1) * rows >= T) continue;
        const int need = (rows + kFThreads / 4 - 1) / (kFThreads / 4);
        int nr = 0;
        for (int o : kRowOptions) if (!nr && o >= need) nr = o;
        if (need <= 8) continue;   // (would be the unstaged instantiation)
        const int64_t cost = static_cast<int64_t>(nr) * parts;
        if (best < 0 || cost < best) { best = cost; sp->plog = plog; sp->part_rows = rows; sp->nr = nr; }
    }
    return best >= 0;
}
static size_t split_records_bytes(int B, int H, int plog) {   // (for the map with more ids)
    return ((static_cast<size_t>(B) * H + 63) / 64 * 256 << plog) * 32 * 2 * sizeof(unsigned long long);
}
// Which slices share a die (see slice_of() in the kernel).  Measured, 1 bit, batch 16 x 9 984 tokens x 8 heads split
// four ways: contiguous (B, T, H, D) 122 -> 110 us with the wide map, the strided view of a fused projection 104 ->
// 106 us; unsplit slices (batch 64 x 3 328) are indifferent to it (129 / 130 us contiguous, 106 / 106 us strided).
// (the wide map pads the (batch, head) pairs to a multiple of 64: only where there are at least that many)
static int wide_map_for(const QuantGeom& g, bool split) {
    return (split && g.sh == g.D && static_cast<int64_t>(g.B) * g.H >= 64) ? 1 : 0;
}

// The wait of a part for the others is bounded; a lane that gives up sets a word of pinned host memory (one per
// device, allocated at the first such call outside a stream capture, never freed).  The next call on the device
// finds it, reports CQ_ERR_LAUNCH once, and the process goes on with the three-launch path.
constexpr int kQMaxDevices = 64;
static std::atomic<int*> g_qstatus[kQMaxDevices];
static std::atomic<bool> g_split_off{false};
static std::atomic<uint32_t> g_qepoch{0x51ab0000u};
static std::atomic<int> g_qspin{1 << 18};

static int* split_status_word(hipStream_t st) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kQMaxDevices) return nullptr;
    int* p = g_qstatus[dev].load(std::memory_order_acquire);
    if (p) return p;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;   // not while the stream is being recorded
    if (hipStreamIsCapturing(st, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return nullptr;
    }
    void* raw = nullptr;
    if (hipHostMalloc(&raw, 64, hipHostMallocDefault) != hipSuccess || !raw) {
        (void)hipGetLastError();
        return nullptr;
    }
    *static_cast<volatile int*>(raw) = 0;
    int* expected = nullptr;
    if (!g_qstatus[dev].compare_exchange_strong(expected, static_cast<int*>(raw), std::memory_order_acq_rel)) {
        (void)hipHostFree(raw);   // another host thread was first
        return expected;
    }
    return static_cast<int*>(raw);
}

static bool one_pass_shape(const QuantGeom& g, const uint8_t* codes) {
    return g.D == 128 && g.T <= kFMaxT && (reinterpret_cast<uintptr_t>(codes) & 3u) == 0 &&
           static_cast<int64_t>(g.B) * g.H < (static_cast<int64_t>(1) << 31) && g.st > 0 && g.st * 2 < (1 << 24) &&
           static_cast<int64_t>(g.T) * g.st * 2 < (static_cast<int64_t>(1) << 31);   // 32-bit row offsets
}

template <typename DT>
static int run_quant(const void* x, QuantGeom g, int bits, float clip, uint8_t* codes, void* xq, void* scale,
                     void* zero, float* ws, hipStream_t st, const RopeArgs* rope = nullptr) {
    dim3 grid(g.nchunk, g.H, g.B);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    uint16_t* sp = static_cast<uint16_t*>(scale);
    uint16_t* zp = static_cast<uint16_t*>(zero);
    if (rope && (xq || !one_pass_shape(g, codes))) return CQ_ERR_UNSUPPORTED;
    if (!xq && one_pass_shape(g, codes)) {
        // x fits a workgroup's registers slice by slice: one pass
        const int64_t bh8 = (static_cast<int64_t>(g.B) * g.H + 7) / 8;
        // persistent: at most one workgroup per compute unit and a multiple of 32 of them
        g.wide_map = wide_map_for(g, false);
        const int64_t nsl = g.wide_map ? (static_cast<int64_t>(g.B) * g.H + 63) / 64 * 256 : bh8 * 32;
        // (the compute-unit count of the current device - a partitioned device reports its own share -
        // rounded down to the multiple of 32 the slice walk needs)
        const int cu = persistent_units();
        const int64_t fmax = cu >= 32 ? cu / 32 * 32 : 32;
        const dim3 fgrid(static_cast<unsigned>(nsl < fmax ? nsl : fmax));
        const int nr = (g.T + kFThreads / 4 - 1) / (kFThreads / 4);
        const RopeArgs ra = rope ? *rope : RopeArgs{};
#define CQ_FUSED(B_, N_)                                                                          \
        do {                                                                                      \
            const int rc = rope ? launch_fused<DT, B_, N_, true>(fgrid, st, xp, g, clip, sp, zp, codes, ra)   \
                                : launch_fused<DT, B_, N_, false>(fgrid, st, xp, g, clip, sp, zp, codes, ra); \
            if (rc != CQ_OK) return rc;                                                           \
        } while (0)
        if (bits == 1) {
            if (nr <= 4) CQ_FUSED(1, 4); else if (nr <= 8) CQ_FUSED(1, 8); else CQ_FUSED(1, 13);
        } else {
            if (nr <= 4) CQ_FUSED(2, 4); else if (nr <= 8) CQ_FUSED(2, 8); else CQ_FUSED(2, 13);
        }
#undef CQ_FUSED
        CQ_LAUNCH_CHECK();
        return CQ_OK;
    }
    SplitPlan spl;
    // (the slice walk pads the (batch, head) pairs to a multiple of 8 and a padding slice costs what a live one does:
    // measured, a single pair of 40 000 tokens takes 33 us split and 25 us in three launches, six pairs of 13 000
    // tokens 19.5 against 25.7 us)
    if (!xq && !rope && g.D == 128 && g.T > kFMaxT && static_cast<int64_t>(g.B) * g.H >= 4 && split_plan(g.T, &spl) &&
        !g_split_off.load(std::memory_order_relaxed) &&
        (reinterpret_cast<uintptr_t>(codes) & 3u) == 0 && static_cast<int64_t>(g.B) * g.H < (static_cast<int64_t>(1) << 26) &&
        g.st > 0 && g.st * 2 < (1 << 24) && static_cast<int64_t>(spl.part_rows) * g.st * 2 < (static_cast<int64_t>(1) << 31)) {
        // Still one pass over x: the slices are split along the token axis between workgroups of one persistent
        // launch, which exchange their channel min / max inside it.
        int* status = split_status_word(st);
        if (status) {
            if (*static_cast<volatile int*>(status) != 0) {
                *static_cast<volatile int*>(status) = 0;
                g_split_off.store(true, std::memory_order_relaxed);
                return CQ_ERR_LAUNCH;   // an earlier split pass did not complete: its output is not valid
            }
            g.wide_map = wide_map_for(g, true);
            const int64_t nids = (g.wide_map ? (static_cast<int64_t>(g.B) * g.H + 63) / 64 * 256
                                             : (static_cast<int64_t>(g.B) * g.H + 7) / 8 * 32) << spl.plog;
            const int cu = persistent_units();
            const int64_t fmax = cu >= 32 ? cu / 32 * 32 : 32;
            const dim3 fgrid(static_cast<unsigned>(nids < fmax ? nids : fmax));
            g.parts_log2 = spl.plog;
            g.part_rows = spl.part_rows;
            g.rec = reinterpret_cast<unsigned long long*>(ws);
            uint32_t ep = g_qepoch.fetch_add(1, std::memory_order_relaxed) + 1;
            g.epoch = ep ? ep : g_qepoch.fetch_add(1, std::memory_order_relaxed) + 1;
            g.spin_limit = g_qspin.load(std::memory_order_relaxed);
            g.status = status;
            const RopeArgs ra{};
            int rc = CQ_OK;
#define CQ_SPLIT(B_, N_) rc = launch_fused<DT, B_, N_, false, true>(fgrid, st, xp, g, clip, sp, zp, codes, ra)
            if (bits == 1) {
                if (spl.nr == 10) CQ_SPLIT(1, 10); else CQ_SPLIT(1, 13);
            } else {
                if (spl.nr == 10) CQ_SPLIT(2, 10); else CQ_SPLIT(2, 13);
            }
#undef CQ_SPLIT
            if (rc != CQ_OK) return rc;
            CQ_LAUNCH_CHECK();
            return CQ_OK;
        }
    }
    hipLaunchKernelGGL(minmax_partial_kernel<DT>, grid, dim3(kQThreads), 0, st, xp, g, ws);
    CQ_LAUNCH_CHECK();
    const float levels = static_cast<float>((1 << bits) - 1);
    float* thr = ws + static_cast<size_t>(g.B) * g.H * g.nchunk * 2 * g.D;
    hipLaunchKernelGGL(stats_kernel<DT>, dim3(g.B * g.H), dim3(kStatThreads), 0, st, ws, g, clip, levels, sp, zp, thr);
    CQ_LAUNCH_CHECK();
    uint16_t* xqp = static_cast<uint16_t*>(xq);
    if (xq) {
        if (bits == 1)
            hipLaunchKernelGGL((emit_kernel<DT, 1, true>), grid, dim3(kQThreads), 0, st, xp, g, sp, zp, thr, codes, xqp);
        else
            hipLaunchKernelGGL((emit_kernel<DT, 2, true>), grid, dim3(kQThreads), 0, st, xp, g, sp, zp, thr, codes, xqp);
    } else {
        if (bits == 1)
            hipLaunchKernelGGL((emit_kernel<DT, 1, false>), grid, dim3(kQThreads), 0, st, xp, g, sp, zp, thr, codes, xqp);
        else
            hipLaunchKernelGGL((emit_kernel<DT, 2, false>), grid, dim3(kQThreads), 0, st, xp, g, sp, zp, thr, codes, xqp);
    }
    CQ_LAUNCH_CHECK();
    return CQ_OK;
}

// quant(per_channel=False): partial min / max, whole-tensor statistics, emit of the unpacked codes.
template <typename DT>
static int run_quant_tensor(const void* x, QuantGeom g, int bits, float clip, void* xq, void* scale1, void* zero1,
                            float* ws, hipStream_t st) {
    dim3 grid(g.nchunk, g.H, g.B);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    hipLaunchKernelGGL(minmax_partial_kernel<DT>, grid, dim3(kQThreads), 0, st, xp, g, ws);
    CQ_LAUNCH_CHECK();
    const float levels = static_cast<float>((1 << bits) - 1);
    const int64_t npairs = static_cast<int64_t>(g.B) * g.H * g.nchunk;
    float* thr = ws + static_cast<size_t>(npairs) * 2 * g.D;            // 3 * D thresholds
    uint16_t* srow = reinterpret_cast<uint16_t*>(thr + 3 * g.D);         // D scales, then D zero-points
    uint16_t* zrow = srow + g.D;
    hipLaunchKernelGGL(tensor_stats_kernel<DT>, dim3(1), dim3(kStatThreads), 0, st, ws, npairs, g.D, clip, levels, srow,
                       zrow, thr, static_cast<uint16_t*>(scale1), static_cast<uint16_t*>(zero1));
    CQ_LAUNCH_CHECK();
    g.shared_stats = 1;
    uint16_t* xqp = static_cast<uint16_t*>(xq);
    if (bits == 1)
        hipLaunchKernelGGL((emit_kernel<DT, 1, true>), grid, dim3(kQThreads), 0, st, xp, g, srow, zrow, thr, nullptr, xqp);
    else
        hipLaunchKernelGGL((emit_kernel<DT, 2, true>), grid, dim3(kQThreads), 0, st, xp, g, srow, zrow, thr, nullptr, xqp);
    CQ_LAUNCH_CHECK();
    return CQ_OK;
}

static int quant_entry(const void* x, int dtype, int B, int T, int H, int D, int64_t sb, int64_t st, int64_t sh,
                       int bits, float clip, uint8_t* codes, void* xq, void* scale, void* zero, void* ws,
                       size_t ws_bytes, cq_stream_t stream, const RopeArgs* rope = nullptr) {
    if (!x || !scale || !zero || (!codes && !xq)) return CQ_ERR_NULL;
    if (dtype != CQ_BF16 && dtype != CQ_FP16) return CQ_ERR_DTYPE;
    if (bits != 1 && bits != 2) return CQ_ERR_UNSUPPORTED;
    if (B < 1 || T < 1 || H < 1 || (D != 64 && D != 128 && D != 256)) return CQ_ERR_SHAPE;
    if (H > 65535 || B > 65535) return CQ_ERR_SHAPE;
    if ((sb % 8) || (st % 8) || (sh % 8) || !aligned16(x) || !aligned16(scale) || !aligned16(zero) ||
        (xq && !aligned16(xq)) || (codes && (reinterpret_cast<uintptr_t>(codes) & 1u)))
        return CQ_ERR_ALIGN;
    const size_t need = cq_quantize_pack_workspace(B, T, H, D);
    if (!ws || ws_bytes < need || !aligned16(ws)) return CQ_ERR_WORKSPACE;
    QuantGeom g = {};
    g.B = B; g.T = T; g.H = H; g.D = D;
    g.sb = sb; g.st = st; g.sh = sh;
    g.nchunk = pick_chunks(B, T, H);
    g.chunk = (T + g.nchunk - 1) / g.nchunk;
    g.dT.set(static_cast<uint32_t>(T));
    g.dH.set(static_cast<uint32_t>(H));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == CQ_BF16)
        return run_quant<BF16>(x, g, bits, clip, codes, xq, scale, zero, static_cast<float*>(ws), s, rope);
    return run_quant<FP16>(x, g, bits, clip, codes, xq, scale, zero, static_cast<float*>(ws), s, rope);
}

// Rotary embedding of the rows of a (B, T, H, 128) view, the same arithmetic as above: one thread per
// (row, head, 8 channels of the lower half and the matching 8 of the upper half).
template <typename DT>
__global__ __launch_bounds__(256) void rope_rows_kernel(const uint16_t* __restrict__ x, QuantGeom g, RopeArgs ra) {
    typedef uint32_t U4 __attribute__((ext_vector_type(4)));
    const int64_t gid = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t total = static_cast<int64_t>(g.B) * g.T * g.H * ra.gn * 8;
    if (gid >= total) return;
    const int p8 = static_cast<int>(gid & 7);
    int64_t r = gid >> 3;
    const int gq = static_cast<int>(r % ra.gn); r /= ra.gn;
    const int h = static_cast<int>(r % g.H); r /= g.H;
    const int t = static_cast<int>(r % g.T);
    const int b = static_cast<int>(r / g.T);
    const uint16_t* xr = x + b * g.sb + static_cast<int64_t>(t) * g.st + static_cast<int64_t>(h) * g.sh + gq * ra.gs + p8 * 8;
    int64_t ps = ra.pos ? ra.pos[b * ra.pos_sb + static_cast<int64_t>(t) * ra.pos_st] : ra.pos0 + t;
    ps = ps < 0 ? 0 : (ps >= ra.table_rows ? ra.table_rows - 1 : ps);
    const U4 lo = *reinterpret_cast<const U4*>(xr), hi = *reinterpret_cast<const U4*>(xr + 64);
    const U4 cl = *reinterpret_cast<const U4*>(ra.cos + ps * 128 + p8 * 8), ch = *reinterpret_cast<const U4*>(ra.cos + ps * 128 + 64 + p8 * 8);
    const U4 sl = *reinterpret_cast<const U4*>(ra.sin + ps * 128 + p8 * 8), sh = *reinterpret_cast<const U4*>(ra.sin + ps * 128 + 64 + p8 * 8);
    float x1[8], x2[8], c1[8], c2[8], s1[8], s2[8];
    unpack8<DT>(lo, x1); unpack8<DT>(hi, x2); unpack8<DT>(cl, c1); unpack8<DT>(ch, c2); unpack8<DT>(sl, s1); unpack8<DT>(sh, s2);
    uint32_t o1[8], o2[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        o1[j] = Cvt<DT>::from_float(rnd<DT>(x1[j] * c1[j]) + (-x2[j]) * s1[j]);
        o2[j] = Cvt<DT>::from_float(rnd<DT>(x2[j] * c2[j]) + x1[j] * s2[j]);
    }
    U4 r1, r2;
#pragma unroll
    for (int w = 0; w < 4; ++w) { r1[w] = o1[2 * w] | (o1[2 * w + 1] << 16); r2[w] = o2[2 * w] | (o2[2 * w + 1] << 16); }
    uint16_t* orow = ra.out + b * ra.ob + static_cast<int64_t>(t) * ra.ot + static_cast<int64_t>(h) * ra.oh + gq * ra.og + p8 * 8;
    *reinterpret_cast<U4*>(orow) = r1;
    *reinterpret_cast<U4*>(orow + 64) = r2;
}

static int check_rope(const void* cos_table, const void* sin_table, int64_t table_rows, const int64_t* pos,
                      void* out, int64_t ob, int64_t ot, int64_t oh, int D) {
    if (!cos_table || !sin_table || !out) return CQ_ERR_NULL;
    if (D != 128) return CQ_ERR_UNSUPPORTED;
    if (table_rows < 1 || table_rows >= (1 << 24)) return CQ_ERR_SHAPE;
    if (!aligned16(cos_table) || !aligned16(sin_table) || !aligned16(out) || (ob % 8) || (ot % 8) || (oh % 8) ||
        (pos && (reinterpret_cast<uintptr_t>(pos) & 7u)))
        return CQ_ERR_ALIGN;
    return CQ_OK;
}

// ---- per-token value quantiser --------------------------------------------------------
// The reference's `triton_quantize_and_pack_along_last_dim` (qjl/new_pack.py:53-82): for every
// token and every group of 32 consecutive channels min and max, scale = (max - min) / L,
// code = round(clamp((x - min) / scale, 0, L)), every op rounded to the storage dtype
// (`tensor / python int` multiplies by the fp32 reciprocal; `div_` by the scale tensor is an
// IEEE division), 32/BITS codes per int32 word with the first code in the lowest bits.
// 16 lanes cover a row of 128 channels with one 16-byte load each; the four lanes of a
// quad are one group.  One pass over x.
template <typename DT> struct BF16Like { static constexpr bool value = false; };
template <> struct BF16Like<BF16> { static constexpr bool value = true; };

template <typename DT, int BITS>
__global__ __launch_bounds__(kQThreads) void token_pack_kernel(const uint16_t* __restrict__ x, QuantGeom g,
                                                               int32_t* __restrict__ words,
                                                               uint16_t* __restrict__ scale,
                                                               uint16_t* __restrict__ mins) {
    constexpr float levels = static_cast<float>((1 << BITS) - 1);
    const int l16 = threadIdx.x & 15, q4 = threadIdx.x & 3, grp = l16 >> 2;
    const float inv_levels = __fdiv_rn(1.0f, levels);
    // A workgroup pass is 16 consecutive tokens of one (batch, head).  Consecutive workgroups take the heads of the
    // same 16 tokens, then the next 16 tokens: what is in flight on the device at any moment then covers whole token
    // rows of x.  (Walking the output order (b, h, t) instead, everything in flight reads the same 256-byte column of
    // its token rows - one head - and a contiguous (B, T, H, D) input then keeps a fraction of the memory channels
    // busy.)
    const uint32_t ntb = g.dTB.div;                                   // 16-token blocks per (batch, head)
    const int64_t nblk = static_cast<int64_t>(g.B) * g.H * ntb;      // (the host keeps this below 2^31)
    for (int64_t blk = blockIdx.x; blk < nblk; blk += gridDim.x) {
        const uint32_t b32 = static_cast<uint32_t>(blk);
        const uint32_t bt = g.dH.quot(b32);                           // (b, token block)
        const int h = static_cast<int>(b32 - bt * g.dH.div);
        const uint32_t bq = g.dTB.quot(bt);
        const int b = static_cast<int>(bq);
        const int t = static_cast<int>(bt - bq * ntb) * (kQThreads / 16) + static_cast<int>(threadIdx.x >> 4);
        if (t >= g.T) continue;   // (the 16 lanes of a row leave together)
        const int64_t row = (static_cast<int64_t>(b) * g.H + h) * g.T + t;   // output row order (b, h, t)
        const uint4 v = *reinterpret_cast<const uint4*>(x + b * g.sb + t * g.st + h * g.sh + l16 * 8);
        float f[8];
        unpack8<DT>(v, f);
        float mn = f[0], mx = f[0];
#pragma unroll
        for (int i = 1; i < 8; ++i) { mn = fminf(mn, f[i]); mx = fmaxf(mx, f[i]); }
        mn = quad_reduce(mn, OpMin(), INFINITY);
        mx = quad_reduce(mx, OpMax(), -INFINITY);
        const float s = rnd<DT>(rnd<DT>(mx - mn) * inv_levels);
        // bf16: the code steps up where y = bf16(fp32(d / s)), d = bf16(x - min), crosses
        // 0.5 (exclusive), 1.5 (inclusive), 2.5 (exclusive) under round-half-even, i.e. where
        // fp32(d / s) crosses the midpoint m to the neighbouring bf16 value.  d and s have 8
        // significant bits and m at most 10, so s * m is exact in fp32 and d / s is either
        // exactly m or further from it than fp32 rounding can move it: the comparison
        // d > s * m (or >=) decides exactly what the division would, without dividing.
        const bool by_compare = BF16Like<DT>::value && s > 0.0f && s < INFINITY;
        const float m1 = s * (0.5f + 0.001953125f);      // 0.5 + 2^-9
        const float m2 = s * (1.5f - 0.00390625f);       // 1.5 - 2^-8
        const float m3 = s * (2.5f + 0.0078125f);        // 2.5 + 2^-7
        // ... and d = bf16(y), y = fp32(x - min) >= 0, is a monotone function of y, so each of those comparisons is
        // one comparison of y itself: with u the smallest bf16 value that satisfies it (the one above m for ">", m
        // rounded up for ">="), bf16(y) >= u exactly when y lies above the midpoint between u and the bf16 value
        // below it, or on it if u is the even one of the two (round-half-even).  In the bit patterns of positive
        // floats that midpoint is u - 0x8000, also across a power of two.  One subtraction and one comparison per
        // element instead of a subtraction, a rounding and a comparison.
        auto from = [](float m, bool inclusive) -> float {
            const uint32_t mb = __float_as_uint(m);
            const uint32_t ub = inclusive ? ((mb + 0xffffu) & 0xffff0000u) : ((mb & 0xffff0000u) + 0x10000u);
            const uint32_t mid = ub - 0x8000u;
            return __uint_as_float((ub & 0x10000u) ? mid + 1u : mid);
        };
        const float y1 = from(m1, false), y2 = from(m2, true), y3 = from(m3, false);
        uint32_t packed = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float y = f[i] - mn;
            uint32_t code = 0;
            if (by_compare) {
                code = (y >= y1) ? 1u : 0u;
                if constexpr (BITS == 2) code += ((y >= y2) ? 1u : 0u) + ((y >= y3) ? 1u : 0u);
            } else {
                const float q = rnd<DT>(__fdiv_rn(rnd<DT>(y), s));
                if (q == q) code = static_cast<uint32_t>(rintf(fminf(fmaxf(q, 0.0f), levels)));
            }
            packed |= code << (BITS * i);
        }
        const int64_t gidx = row * (g.D / 32) + grp;
        if constexpr (BITS == 1) {
            // 8 bits per lane, 32 per quad: one word
            uint32_t w = packed << (8 * q4);
            w |= static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(w), 0xB1, 0xf, 0xf, true));   // lane ^ 1
            w |= static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(w), 0x4E, 0xf, 0xf, true));   // lane ^ 2
            if (q4 == 0) words[gidx] = static_cast<int32_t>(w);
        } else {
            // 16 bits per lane: lanes (0,1) and (2,3) of the quad make the group's two words
            const uint32_t other = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(packed), 0xB1, 0xf, 0xf, true));
            if ((q4 & 1) == 0) words[gidx * 2 + (q4 >> 1)] = static_cast<int32_t>(packed | (other << 16));
        }
        if (q4 == 0) {
            scale[gidx] = static_cast<uint16_t>(Cvt<DT>::from_float(s));
            mins[gidx] = static_cast<uint16_t>(Cvt<DT>::from_float(mn));
        }
    }
}

// ---- encode() ---------------------------------------------------------------------
template <typename IT>
__device__ __forceinline__ uint32_t index_of(const IT* p, int64_t i);
template <> __device__ __forceinline__ uint32_t index_of<int64_t>(const int64_t* p, int64_t i) { return static_cast<uint32_t>(p[i]); }
template <> __device__ __forceinline__ uint32_t index_of<int32_t>(const int32_t* p, int64_t i) { return static_cast<uint32_t>(p[i]); }
template <> __device__ __forceinline__ uint32_t index_of<uint8_t>(const uint8_t* p, int64_t i) { return p[i]; }
struct Bf16Tag { uint16_t v; };
struct Fp16Tag { uint16_t v; };
template <> __device__ __forceinline__ uint32_t index_of<Bf16Tag>(const Bf16Tag* p, int64_t i) {
    float f = bf16_bits_to_float(p[i].v);
    return (f != f) ? 0u : static_cast<uint32_t>(static_cast<int>(f));
}
template <> __device__ __forceinline__ uint32_t index_of<Fp16Tag>(const Fp16Tag* p, int64_t i) {
    float f = fp16_bits_to_float(p[i].v);
    return (f != f) ? 0u : static_cast<uint32_t>(static_cast<int>(f));
}

template <typename IT, int BITS>
__global__ void encode_kernel(const IT* __restrict__ idx, int64_t nbytes, uint8_t* __restrict__ out) {
    constexpr int dpe = 8 / BITS;
    constexpr uint32_t m = (1u << BITS) - 1u;
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < nbytes;
         i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        uint32_t byte = 0;
#pragma unroll
        for (int k = 0; k < dpe; ++k) byte |= (index_of<IT>(idx, i * dpe + k) & m) << (BITS * (dpe - 1 - k));
        out[i] = static_cast<uint8_t>(byte);
    }
}

template <typename IT>
static int run_encode(const void* idx, int64_t nbytes, int bits, uint8_t* out, hipStream_t st) {
    int64_t blocks = (nbytes + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (bits == 1)
        hipLaunchKernelGGL((encode_kernel<IT, 1>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st,
                           static_cast<const IT*>(idx), nbytes, out);
    else
        hipLaunchKernelGGL((encode_kernel<IT, 2>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st,
                           static_cast<const IT*>(idx), nbytes, out);
    CQ_LAUNCH_CHECK();
    return CQ_OK;
}

}  // namespace cq

extern "C" {

size_t cq_quantize_pack_workspace(int B, int T, int H, int D) {
    if (B < 1 || T < 1 || H < 1 || D < 1) return 0;
    // partial min / max per chunk, then three thresholds per channel (+ one row of statistics in the
    // storage dtype for the whole-tensor mode of cq_quant_tensor)
    size_t need = (static_cast<size_t>(B) * H * (static_cast<size_t>(cq::pick_chunks(B, T, H)) * 2 + 3) + 4) * D * sizeof(float);
    // (the records that the parts of a split slice exchange, when the one-pass kernel takes a long token axis)
    cq::SplitPlan spl;
    if (D == 128 && T > cq::kFMaxT && cq::split_plan(T, &spl)) {
        const size_t rec = cq::split_records_bytes(B, H, spl.plog);
        if (rec > need) need = rec;
    }
    return need;
}

int cq_quantize_pack_wait_polls(int polls) {
    const int before = cq::g_qspin.load(std::memory_order_relaxed);
    if (polls >= 0) {
        cq::g_qspin.store(polls, std::memory_order_relaxed);
        cq::g_split_off.store(false, std::memory_order_relaxed);
    }
    return before;
}

int cq_quantize_pack(const void* x, int dtype, int B, int T, int H, int D, int64_t stride_b, int64_t stride_t,
                     int64_t stride_h, int bits, float clip, uint8_t* codes, void* scale, void* zero,
                     void* workspace, size_t workspace_bytes, cq_stream_t stream) {
    if (!codes) return CQ_ERR_NULL;
    return cq::quant_entry(x, dtype, B, T, H, D, stride_b, stride_t, stride_h, bits, clip, codes, nullptr, scale,
                           zero, workspace, workspace_bytes, stream);
}

int cq_rope_quantize_pack(const void* x, int dtype, int B, int T, int H, int D, int64_t stride_b, int64_t stride_t,
                          int64_t stride_h, const void* cos_table, const void* sin_table, int64_t table_rows,
                          const int64_t* pos, int64_t pos_stride_b, int64_t pos_stride_t, int64_t pos0,
                          void* x_rot, int64_t rot_stride_b, int64_t rot_stride_t, int64_t rot_stride_h,
                          int bits, float clip, uint8_t* codes, void* scale, void* zero,
                          void* workspace, size_t workspace_bytes, cq_stream_t stream) {
    if (!codes) return CQ_ERR_NULL;
    int rc = cq::check_rope(cos_table, sin_table, table_rows, pos, x_rot, rot_stride_b, rot_stride_t, rot_stride_h, D);
    if (rc != CQ_OK) return rc;
    cq::RopeArgs ra;
    ra.cos = static_cast<const uint16_t*>(cos_table); ra.sin = static_cast<const uint16_t*>(sin_table);
    ra.pos = pos; ra.pos_sb = pos_stride_b; ra.pos_st = pos_stride_t; ra.pos0 = pos0; ra.table_rows = table_rows;
    ra.out = static_cast<uint16_t*>(x_rot); ra.ob = rot_stride_b; ra.ot = rot_stride_t; ra.oh = rot_stride_h;
    return cq::quant_entry(x, dtype, B, T, H, D, stride_b, stride_t, stride_h, bits, clip, codes, nullptr, scale,
                           zero, workspace, workspace_bytes, stream, &ra);
}

int cq_rope_rows(const void* x, int dtype, int B, int T, int H, int D, int64_t stride_b, int64_t stride_t,
                 int64_t stride_h, const void* cos_table, const void* sin_table, int64_t table_rows,
                 const int64_t* pos, int64_t pos_stride_b, int64_t pos_stride_t, int64_t pos0,
                 void* x_rot, int64_t rot_stride_b, int64_t rot_stride_t, int64_t rot_stride_h, cq_stream_t stream) {
    return cq_rope_rows_grouped(x, dtype, B, T, H, 1, D, stride_b, stride_t, stride_h, 0, cos_table, sin_table, table_rows,
                                pos, pos_stride_b, pos_stride_t, pos0, x_rot, rot_stride_b, rot_stride_t, rot_stride_h, 0,
                                stream);
}

int cq_rope_rows_grouped(const void* x, int dtype, int B, int T, int H, int G, int D, int64_t stride_b, int64_t stride_t,
                         int64_t stride_h, int64_t stride_g, const void* cos_table, const void* sin_table,
                         int64_t table_rows, const int64_t* pos, int64_t pos_stride_b, int64_t pos_stride_t, int64_t pos0,
                         void* x_rot, int64_t rot_stride_b, int64_t rot_stride_t, int64_t rot_stride_h,
                         int64_t rot_stride_g, cq_stream_t stream) {
    if (!x) return CQ_ERR_NULL;
    if (dtype != CQ_BF16 && dtype != CQ_FP16) return CQ_ERR_DTYPE;
    if (B < 1 || T < 1 || H < 1 || G < 1) return CQ_ERR_SHAPE;
    int rc = cq::check_rope(cos_table, sin_table, table_rows, pos, x_rot, rot_stride_b, rot_stride_t, rot_stride_h, D);
    if (rc != CQ_OK) return rc;
    if ((stride_b % 8) || (stride_t % 8) || (stride_h % 8) || (stride_g % 8) || (rot_stride_g % 8) || !cq::aligned16(x))
        return CQ_ERR_ALIGN;
    cq::QuantGeom g = {};
    g.B = B; g.T = T; g.H = H; g.D = D; g.sb = stride_b; g.st = stride_t; g.sh = stride_h;
    cq::RopeArgs ra;
    ra.cos = static_cast<const uint16_t*>(cos_table); ra.sin = static_cast<const uint16_t*>(sin_table);
    ra.pos = pos; ra.pos_sb = pos_stride_b; ra.pos_st = pos_stride_t; ra.pos0 = pos0; ra.table_rows = table_rows;
    ra.out = static_cast<uint16_t*>(x_rot); ra.ob = rot_stride_b; ra.ot = rot_stride_t; ra.oh = rot_stride_h;
    ra.gn = G; ra.gs = stride_g; ra.og = rot_stride_g;
    const int64_t total = static_cast<int64_t>(B) * T * H * G * 8;
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffff) return CQ_ERR_SHAPE;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    if (dtype == CQ_BF16) hipLaunchKernelGGL(cq::rope_rows_kernel<cq::BF16>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, xp, g, ra);
    else hipLaunchKernelGGL(cq::rope_rows_kernel<cq::FP16>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, xp, g, ra);
    CQ_LAUNCH_CHECK();
    return CQ_OK;
}

int cq_quantize_pack_token(const void* x, int dtype, int B, int T, int H, int D, int64_t stride_b, int64_t stride_t,
                           int64_t stride_h, int bits, int group_size, int32_t* words, void* scale, void* mins,
                           cq_stream_t stream) {
    if (!x || !words || !scale || !mins) return CQ_ERR_NULL;
    if (dtype != CQ_BF16 && dtype != CQ_FP16) return CQ_ERR_DTYPE;
    if ((bits != 1 && bits != 2) || group_size != 32 || D != 128) return CQ_ERR_UNSUPPORTED;
    if (B < 1 || T < 1 || H < 1) return CQ_ERR_SHAPE;
    if ((stride_b % 8) || (stride_t % 8) || (stride_h % 8) || !cq::aligned16(x) ||
        (reinterpret_cast<uintptr_t>(words) & 3u) || (reinterpret_cast<uintptr_t>(scale) & 1u) ||
        (reinterpret_cast<uintptr_t>(mins) & 1u))
        return CQ_ERR_ALIGN;
    cq::QuantGeom g = {};
    g.B = B; g.T = T; g.H = H; g.D = D;
    g.sb = stride_b; g.st = stride_t; g.sh = stride_h;
    g.nchunk = 1; g.chunk = T;
    g.dT.set(static_cast<uint32_t>(T));
    g.dH.set(static_cast<uint32_t>(H));
    const int64_t ntb = (static_cast<int64_t>(T) + cq::kQThreads / 16 - 1) / (cq::kQThreads / 16);
    g.dTB.set(static_cast<uint32_t>(ntb));
    const int64_t nblk = static_cast<int64_t>(B) * H * ntb;
    if (nblk > 0x7fffffff) return CQ_ERR_SHAPE;
    int64_t blocks = nblk;
    if (blocks > (1 << 20)) blocks = 1 << 20;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    uint16_t* sp = static_cast<uint16_t*>(scale);
    uint16_t* mp = static_cast<uint16_t*>(mins);
    const dim3 grid(static_cast<unsigned>(blocks)), block(cq::kQThreads);
    if (dtype == CQ_BF16) {
        if (bits == 1) hipLaunchKernelGGL((cq::token_pack_kernel<cq::BF16, 1>), grid, block, 0, st, xp, g, words, sp, mp);
        else hipLaunchKernelGGL((cq::token_pack_kernel<cq::BF16, 2>), grid, block, 0, st, xp, g, words, sp, mp);
    } else {
        if (bits == 1) hipLaunchKernelGGL((cq::token_pack_kernel<cq::FP16, 1>), grid, block, 0, st, xp, g, words, sp, mp);
        else hipLaunchKernelGGL((cq::token_pack_kernel<cq::FP16, 2>), grid, block, 0, st, xp, g, words, sp, mp);
    }
    CQ_LAUNCH_CHECK();
    return CQ_OK;
}

int cq_quant(const void* x, int dtype, int B, int T, int H, int D, int64_t stride_b, int64_t stride_t,
             int64_t stride_h, int bits, float clip, void* x_q, void* scale, void* zero, void* workspace,
             size_t workspace_bytes, cq_stream_t stream) {
    if (!x_q) return CQ_ERR_NULL;
    return cq::quant_entry(x, dtype, B, T, H, D, stride_b, stride_t, stride_h, bits, clip, nullptr, x_q, scale,
                           zero, workspace, workspace_bytes, stream);
}

int cq_quant_tensor(const void* x, int dtype, int B, int T, int H, int D, int64_t stride_b, int64_t stride_t,
                    int64_t stride_h, int bits, float clip, void* x_q, void* scale1, void* zero1, void* workspace,
                    size_t workspace_bytes, cq_stream_t stream) {
    if (!x || !x_q || !scale1 || !zero1) return CQ_ERR_NULL;
    if (dtype != CQ_BF16 && dtype != CQ_FP16) return CQ_ERR_DTYPE;
    if (bits != 1 && bits != 2) return CQ_ERR_UNSUPPORTED;
    if (B < 1 || T < 1 || H < 1 || (D != 64 && D != 128 && D != 256)) return CQ_ERR_SHAPE;
    if (H > 65535 || B > 65535) return CQ_ERR_SHAPE;
    if ((stride_b % 8) || (stride_t % 8) || (stride_h % 8) || !cq::aligned16(x) || !cq::aligned16(x_q) ||
        (reinterpret_cast<uintptr_t>(scale1) & 1u) || (reinterpret_cast<uintptr_t>(zero1) & 1u))
        return CQ_ERR_ALIGN;
    const size_t need = cq_quantize_pack_workspace(B, T, H, D);
    if (!workspace || workspace_bytes < need || !cq::aligned16(workspace)) return CQ_ERR_WORKSPACE;
    cq::QuantGeom g = {};
    g.B = B; g.T = T; g.H = H; g.D = D;
    g.sb = stride_b; g.st = stride_t; g.sh = stride_h;
    g.nchunk = cq::pick_chunks(B, T, H);
    g.chunk = (T + g.nchunk - 1) / g.nchunk;
    g.dT.set(static_cast<uint32_t>(T));
    g.dH.set(static_cast<uint32_t>(H));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == CQ_BF16)
        return cq::run_quant_tensor<cq::BF16>(x, g, bits, clip, x_q, scale1, zero1, static_cast<float*>(workspace), s);
    return cq::run_quant_tensor<cq::FP16>(x, g, bits, clip, x_q, scale1, zero1, static_cast<float*>(workspace), s);
}

int cq_encode(const void* idx, int idx_dtype, int64_t rows, int D, int bits, uint8_t* out, cq_stream_t stream) {
    if (!idx || !out) return CQ_ERR_NULL;
    if (bits != 1 && bits != 2) return CQ_ERR_UNSUPPORTED;
    if (rows < 0 || D < 1 || (D % (8 / bits)) != 0) return CQ_ERR_SHAPE;
    if (rows == 0) return CQ_OK;
    const int64_t nbytes = rows * (D * bits / 8);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (idx_dtype) {
        case CQ_I64: return cq::run_encode<int64_t>(idx, nbytes, bits, out, s);
        case CQ_I32: return cq::run_encode<int32_t>(idx, nbytes, bits, out, s);
        case CQ_U8: return cq::run_encode<uint8_t>(idx, nbytes, bits, out, s);
        case CQ_BF16: return cq::run_encode<cq::Bf16Tag>(idx, nbytes, bits, out, s);
        case CQ_FP16: return cq::run_encode<cq::Fp16Tag>(idx, nbytes, bits, out, s);
        default: return CQ_ERR_DTYPE;
    }
}

}  // extern "C"
