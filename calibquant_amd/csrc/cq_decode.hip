// Fused decode attention over bit-packed K/V for gfx950 (MI355X).
//
// One workgroup owns one (batch, kv-head, head-group, token-chunk) unit and
// runs the whole step for HPB query heads that share the kv-head:
//
//   K side   q.s_k is folded into a byte-indexed partial-sum table in LDS
//            (one entry per byte position and byte value, HPB floats wide,
//            zero-point folded in).  A token's logits are NB table look-ups
//            and adds; the fp16/bf16 K tensor is never materialised.
//   stats    min / max of the image logits (calibration), then e = exp(w' - M)
//            in place in LDS.
//   V side   tokens are taken four at a time: a 16-entry table of subset sums
//            of their e values is built once per group, every byte column of
//            the packed V rows is bit-transposed with a 256-entry spread
//            table, and each of the 8 bit lanes of the column adds one table
//            entry.  Scale / zero-point are applied once at the end.
//   residual the full-precision rows run as an ordinary online-softmax
//            flash-decode in the same workgroup and are merged at the end.
//
// When the chunk does not cover all T tokens (long context or small batch)
// a first launch publishes the per-chunk logit min / max, the main launch
// recomputes its chunk's logits against the global min / max and writes an
// (m, l, acc) partial, and a merge launch combines the partials.
//
// Everything here is HBM / LDS / VALU work; no matrix-core instructions.
#include "cq_common.h"

#include <atomic>

namespace cq {

constexpr int kD = 128;
constexpr int kNT = 512;          // threads per workgroup
constexpr int kNW = kNT / kWave;  // waves per workgroup
constexpr int kVSub = 1024;       // V tokens staged in LDS at a time
constexpr int kResTile = kNT / 8; // residual rows per tile (8 lanes per row)
constexpr int kLdsMax = 160 * 1024;

template <int N> struct alignas(N * 4) Vec { float v[N]; };

struct DecodeGeom {
    const void* q;
    const uint8_t* ck;
    const uint8_t* cv;
    const void *ks, *kz, *vs, *vz;
    const void *kres, *vres;
    int64_t rs_b, rs_h, rs_r;
    const float* mask;
    int64_t mask_sb;
    void* out;
    float* mm;    // [B][Hq][nsplit][2] chunk logit min / max
    float* part;  // [B][Hq][nx][kD + 2] partials (m, l, acc)
    int B, Hq, Hkv, T, R, S;
    int nsplit, chunk, nx;
    int calib;
    float off_max, off_min;
    int cap;      // logits capacity of the LDS layout, tokens
};

template <int BITS, int HPB> struct Lay {
    static constexpr int NB = 16 * BITS;            // bytes per packed row
    static constexpr int PC = NB * 8;               // bit lanes per row
    static constexpr int GPW = kWave / NB;          // 4-token groups per wave pass
    static constexpr int TPW = 4 * GPW;             // tokens per wave pass
    static constexpr int KT = NB * 256 * HPB * 4;   // K table bytes
    static constexpr int SPREAD = 256 * 8;
    static constexpr int WTAB = kNW * GPW * 16 * HPB * 4;
    static constexpr int VSTAGE = kVSub * NB;
    static constexpr int VNEED = SPREAD + WTAB + VSTAGE;
    static constexpr int RED = kNW * PC * HPB * 4;
    static constexpr int RED2 = kNW * kD * HPB * 4;
    static constexpr int A0 = KT > VNEED ? KT : VNEED;
    static constexpr int A1 = RED > RED2 ? RED : RED2;
    static constexpr int REGION_A = A0 > A1 ? A0 : A1;
    // fixed small region (floats)
    static constexpr int F_WBIT = 0;                          // NB*8*HPB
    static constexpr int F_ZSUM = F_WBIT + NB * 8 * HPB;      // NB*HPB
    static constexpr int F_QF = F_ZSUM + NB * HPB;            // HPB*kD
    static constexpr int F_QSZ = F_QF + HPB * kD;             // HPB*kD
    static constexpr int F_RED = F_QSZ + HPB * kD;            // kNW*HPB*2
    static constexpr int F_BC = F_RED + kNW * HPB * 2;        // 4*HPB broadcast slots
    static constexpr int F_SRES = F_BC + 4 * HPB;             // kResTile*HPB
    static constexpr int F_PRES = F_SRES + kResTile * HPB;    // kResTile*HPB
    static constexpr int F_END = F_PRES + kResTile * HPB;
    static constexpr int FIXED = ((F_END * 4 + 15) / 16) * 16;
    static constexpr int max_chunk() { return ((kLdsMax - REGION_A - FIXED) / (HPB * 4)) / 64 * 64; }
    static constexpr int lds_bytes(int cap) { return REGION_A + FIXED + cap * HPB * 4; }
};

__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Block-wide reduction of HPB values with `op`; result broadcast to all threads.
template <int HPB, typename Op>
__device__ __forceinline__ void block_reduce(float* v, float* red, Op op, float identity) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
    for (int h = 0; h < HPB; ++h) {
        float x = v[h];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) x = op(x, __shfl_xor(x, o, kWave));
        if (lane == 0) red[w * HPB + h] = x;
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < HPB; ++h) {
        float x = identity;
#pragma unroll
        for (int i = 0; i < kNW; ++i) x = op(x, red[i * HPB + h]);
        v[h] = x;
    }
    __syncthreads();
}

struct OpMin { __device__ float operator()(float a, float b) const { return fminf(a, b); } };
struct OpMax { __device__ float operator()(float a, float b) const { return fmaxf(a, b); } };
struct OpSum { __device__ float operator()(float a, float b) const { return a + b; } };

// Unit decomposition of a 1-D grid.  Consecutive work ids share packed codes
// (head groups of one kv-head), so when the grid is a multiple of the 8 XCDs
// the hardware's round-robin placement is undone to keep them on one L2.
__device__ __forceinline__ int virtual_block_id() {
    const int n = gridDim.x;
    const int l = blockIdx.x;
    if ((n & 7) == 0) return (l & 7) * (n >> 3) + (l >> 3);
    return l;
}

template <int BITS, int HPB, typename DT, bool MINMAX_ONLY>
__global__ __launch_bounds__(kNT) void decode_kernel(DecodeGeom g) {
    using L = Lay<BITS, HPB>;
    using V = Vec<HPB>;
    constexpr int NB = L::NB;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char* regA = smem;
    float* fx = reinterpret_cast<float*>(smem + L::REGION_A);
    V* logits = reinterpret_cast<V*>(smem + L::REGION_A + L::FIXED);
    float* wbit = fx + L::F_WBIT;
    float* zsum = fx + L::F_ZSUM;
    float* qf = fx + L::F_QF;
    float* qsz = fx + L::F_QSZ;
    float* red = fx + L::F_RED;
    float* bc = fx + L::F_BC;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = tid >> 6;
    const int G = g.Hq / g.Hkv;
    const int NG = G / HPB;

    int vb = virtual_block_id();
    const int hg = vb % NG; vb /= NG;
    const int split = vb % g.nx; vb /= g.nx;
    const int hkv = vb % g.Hkv;
    const int b = vb / g.Hkv;
    const int hq0 = hkv * G + hg * HPB;
    const int64_t bh = static_cast<int64_t>(b) * g.Hkv + hkv;

    const bool img_unit = split < g.nsplit && g.T > 0;
    const bool do_res = !MINMAX_ONLY && g.R > 0 && (g.nsplit == 1 || split == g.nsplit);
    const int t0 = img_unit ? split * g.chunk : 0;
    const int n = img_unit ? min(g.T, t0 + g.chunk) - t0 : 0;
    const float inv_sqrt_d = 0.08838834764831845f;  // 1/sqrt(128)

    // ---- phase 0: q, per-bit weights, zero-point sums ------------------------
    if (tid < HPB * kD) {
        const int h = tid / kD, d = tid % kD;
        const float qv = load_elem<DT>(g.q, (static_cast<int64_t>(b) * g.Hq + hq0 + h) * kD + d) * inv_sqrt_d;
        qf[h * kD + d] = qv;
        if (n > 0) {
            const float s = load_elem<DT>(g.ks, bh * kD + d);
            const float z = load_elem<DT>(g.kz, bh * kD + d);
            const float qs = qv * s;
            qsz[h * kD + d] = qs * z;
            if constexpr (BITS == 1) {
                wbit[((d >> 3) * 8 + (7 - (d & 7))) * HPB + h] = qs;
            } else {
                const int sh = 6 - 2 * (d & 3);
                wbit[((d >> 2) * 8 + sh) * HPB + h] = qs;
                wbit[((d >> 2) * 8 + sh + 1) * HPB + h] = 2.0f * qs;
            }
        }
    }
    __syncthreads();

    float mn[HPB], mx[HPB];
#pragma unroll
    for (int h = 0; h < HPB; ++h) { mn[h] = INFINITY; mx[h] = -INFINITY; }

    if (n > 0) {
        if (tid < NB * HPB) {
            const int j = tid / HPB, h = tid % HPB;
            constexpr int cpb = 8 / BITS;
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < cpb; ++i) s += qsz[h * kD + j * cpb + i];
            zsum[j * HPB + h] = s;
        }
        __syncthreads();

        // ---- phase 1: byte table.  Thread = (byte position, high nibble);
        // the 16 low-nibble values are walked in Gray-code order so each entry
        // costs one add per head.
        V* ktab = reinterpret_cast<V*>(regA);
        for (int pr = tid; pr < NB * 16; pr += kNT) {
            const int j = pr >> 4, vhi = pr & 15;
            const V* wb = reinterpret_cast<const V*>(wbit) + j * 8;
            V acc;
            const V zs = reinterpret_cast<const V*>(zsum)[j];
#pragma unroll
            for (int h = 0; h < HPB; ++h) acc.v[h] = -zs.v[h];
#pragma unroll
            for (int bt = 0; bt < 4; ++bt) {
                const V wv4 = wb[4 + bt];
                const float f = static_cast<float>((vhi >> bt) & 1);
#pragma unroll
                for (int h = 0; h < HPB; ++h) acc.v[h] += f * wv4.v[h];
            }
            V wlo[4];
#pragma unroll
            for (int bt = 0; bt < 4; ++bt) wlo[bt] = wb[bt];
            V* dst = ktab + j * 256 + vhi * 16;
            dst[0] = acc;
#pragma unroll
            for (int k = 1; k < 16; ++k) {
                const int gray = k ^ (k >> 1);
                const int bt = __builtin_ctz(k);
                const bool set = (gray >> bt) & 1;
#pragma unroll
                for (int h = 0; h < HPB; ++h) acc.v[h] = set ? acc.v[h] + wlo[bt].v[h] : acc.v[h] - wlo[bt].v[h];
                dst[gray] = acc;
            }
        }
        __syncthreads();

        // ---- phase 2: logits of the chunk ------------------------------------
        const uint8_t* ckb = g.ck + (bh * g.T + t0) * NB;
        for (int tt = tid; tt < n; tt += kNT) {
            const uint4* cp = reinterpret_cast<const uint4*>(ckb + static_cast<int64_t>(tt) * NB);
            uint32_t wds[4 * BITS];
#pragma unroll
            for (int i = 0; i < BITS; ++i) {
                const uint4 c = cp[i];
                wds[4 * i + 0] = c.x; wds[4 * i + 1] = c.y; wds[4 * i + 2] = c.z; wds[4 * i + 3] = c.w;
            }
            V acc;
#pragma unroll
            for (int h = 0; h < HPB; ++h) acc.v[h] = 0.f;
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const uint32_t byte = (wds[j >> 2] >> (8 * (j & 3))) & 0xffu;
                const V e = ktab[j * 256 + byte];
#pragma unroll
                for (int h = 0; h < HPB; ++h) acc.v[h] += e.v[h];
            }
            if constexpr (!MINMAX_ONLY) logits[tt] = acc;
#pragma unroll
            for (int h = 0; h < HPB; ++h) { mn[h] = fminf(mn[h], acc.v[h]); mx[h] = fmaxf(mx[h], acc.v[h]); }
        }
        block_reduce<HPB>(mn, red, OpMin(), INFINITY);
        block_reduce<HPB>(mx, red, OpMax(), -INFINITY);
    }

    if constexpr (MINMAX_ONLY) {
        if (n > 0 && tid < HPB) {
            float* o = g.mm + ((static_cast<int64_t>(b) * g.Hq + hq0 + tid) * g.nsplit + split) * 2;
            o[0] = mn[tid];
            o[1] = mx[tid];
        }
        return;
    } else {
        // ---- phase 3: calibration + exp -------------------------------------------
        float m_img[HPB], l_img[HPB];
#pragma unroll
        for (int h = 0; h < HPB; ++h) { m_img[h] = -INFINITY; l_img[h] = 0.f; }
        float o_img = 0.f;  // thread (h, d) = (tid / kD, tid % kD) for tid < HPB*kD

        if (n > 0) {
            if (g.nsplit > 1) {
#pragma unroll
                for (int h = 0; h < HPB; ++h) {
                    const float* p = g.mm + (static_cast<int64_t>(b) * g.Hq + hq0 + h) * g.nsplit * 2;
                    float a = INFINITY, z = -INFINITY;
                    for (int s = 0; s < g.nsplit; ++s) { a = fminf(a, p[2 * s]); z = fmaxf(z, p[2 * s + 1]); }
                    mn[h] = a; mx[h] = z;
                }
            }
            float slope[HPB], tmin[HPB];
#pragma unroll
            for (int h = 0; h < HPB; ++h) {
                if (g.calib) {
                    const float tgt_max = mx[h] + g.off_max;
                    tmin[h] = mn[h] + g.off_min;
                    slope[h] = (tgt_max - tmin[h]) / (mx[h] - mn[h] + 1e-8f);
                } else {
                    tmin[h] = mn[h];
                    slope[h] = 1.0f;
                }
            }
            const int npad = (n + L::TPW - 1) / L::TPW * L::TPW;
            if (g.mask) {
                const float* mk = g.mask + b * g.mask_sb + g.S + t0;
                float lm[HPB];
#pragma unroll
                for (int h = 0; h < HPB; ++h) lm[h] = -INFINITY;
                for (int tt = tid; tt < n; tt += kNT) {
                    V w = logits[tt];
                    const float mv = mk[tt];
#pragma unroll
                    for (int h = 0; h < HPB; ++h) {
                        w.v[h] = (w.v[h] - mn[h]) * slope[h] + tmin[h] + mv;
                        lm[h] = fmaxf(lm[h], w.v[h]);
                    }
                    logits[tt] = w;
                }
                block_reduce<HPB>(lm, red, OpMax(), -INFINITY);
#pragma unroll
                for (int h = 0; h < HPB; ++h) { m_img[h] = lm[h]; slope[h] = 1.0f; tmin[h] = 0.f; mn[h] = 0.f; }
            } else {
#pragma unroll
                for (int h = 0; h < HPB; ++h) m_img[h] = fmaxf(tmin[h], (mx[h] - mn[h]) * slope[h] + tmin[h]);
            }
            float ls[HPB];
#pragma unroll
            for (int h = 0; h < HPB; ++h) ls[h] = 0.f;
            for (int tt = tid; tt < npad; tt += kNT) {
                V w;
                if (tt < n) {
                    w = logits[tt];
#pragma unroll
                    for (int h = 0; h < HPB; ++h) {
                        const float x = (w.v[h] - mn[h]) * slope[h] + tmin[h];
                        const float e = (m_img[h] == -INFINITY) ? 0.f : __expf(x - m_img[h]);
                        w.v[h] = e;
                        ls[h] += e;
                    }
                } else {
#pragma unroll
                    for (int h = 0; h < HPB; ++h) w.v[h] = 0.f;
                }
                logits[tt] = w;
            }
            block_reduce<HPB>(ls, red, OpSum(), 0.f);
#pragma unroll
            for (int h = 0; h < HPB; ++h) l_img[h] = ls[h];

            // ---- phase 4: packed V ----------------------------------------------------
            uint2* spread = reinterpret_cast<uint2*>(regA);
            V* wtab = reinterpret_cast<V*>(regA + L::SPREAD) + wv * (L::GPW * 16);
            unsigned char* vst = regA + L::SPREAD + L::WTAB;
            if (tid < 256) {
                uint32_t lo = 0, hi = 0;
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    lo |= ((tid >> (7 - m)) & 1u) << (8 * m);
                    hi |= ((tid >> (3 - m)) & 1u) << (8 * m);
                }
                spread[tid] = make_uint2(lo, hi);
            }
            const int j = lane % NB, gs = lane / NB;
            const int bg = lane >> 4, be = lane & 15;   // table build: group, entry
            float bsel[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) bsel[i] = static_cast<float>((be >> i) & 1);
            V acc[8];
#pragma unroll
            for (int m = 0; m < 8; ++m)
#pragma unroll
                for (int h = 0; h < HPB; ++h) acc[m].v[h] = 0.f;
            const uint8_t* cvb = g.cv + (bh * g.T + t0) * NB;

            for (int vs0 = 0; vs0 < npad; vs0 += kVSub) {
                const int vn = min(kVSub, npad - vs0);
                __syncthreads();  // previous sub-chunk consumed (and spread written)
                for (int u = tid; u < vn * NB / 16; u += kNT) {
                    const int tok = vs0 + u * 16 / NB;
                    uint4 c = make_uint4(0, 0, 0, 0);
                    if (tok < n) c = reinterpret_cast<const uint4*>(cvb + static_cast<int64_t>(vs0) * NB)[u];
                    reinterpret_cast<uint4*>(vst)[u] = c;
                }
                __syncthreads();
                for (int u = wv; u * L::TPW < vn; u += kNW) {
                    const int tl = u * L::TPW;        // token offset inside the sub-chunk
                    if (bg < L::GPW) {
                        V val;
#pragma unroll
                        for (int h = 0; h < HPB; ++h) val.v[h] = 0.f;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const V e = logits[vs0 + tl + 4 * bg + i];
#pragma unroll
                            for (int h = 0; h < HPB; ++h) val.v[h] += bsel[i] * e.v[h];
                        }
                        wtab[bg * 16 + be] = val;
                    }
                    wave_lds_fence();
                    uint32_t xlo = 0, xhi = 0;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const uint32_t c = vst[(tl + 4 * gs + i) * NB + j];
                        const uint2 sp = spread[c];
                        xlo |= sp.x << i;
                        xhi |= sp.y << i;
                    }
                    const V* tb = wtab + gs * 16;
#pragma unroll
                    for (int m = 0; m < 8; ++m) {
                        const uint32_t x = m < 4 ? xlo : xhi;
                        const V e = tb[(x >> (8 * (m & 3))) & 15u];
#pragma unroll
                        for (int h = 0; h < HPB; ++h) acc[m].v[h] += e.v[h];
                    }
                    wave_lds_fence();
                }
            }
            // fold the group slots of the wave, then the waves
#pragma unroll
            for (int o = NB; o < kWave; o <<= 1)
#pragma unroll
                for (int m = 0; m < 8; ++m)
#pragma unroll
                    for (int h = 0; h < HPB; ++h) acc[m].v[h] += __shfl_xor(acc[m].v[h], o, kWave);
            __syncthreads();
            V* redv = reinterpret_cast<V*>(regA);  // [wave][PC]
            if (gs == 0) {
#pragma unroll
                for (int m = 0; m < 8; ++m) redv[wv * L::PC + j * 8 + m] = acc[m];
            }
            __syncthreads();
            if (tid < HPB * kD) {
                const int h = tid / kD, d = tid % kD;
                float a = 0.f;
                if constexpr (BITS == 1) {
#pragma unroll
                    for (int w = 0; w < kNW; ++w) a += redv[w * L::PC + d].v[h];
                } else {
#pragma unroll
                    for (int w = 0; w < kNW; ++w)
                        a += 2.0f * redv[w * L::PC + 2 * d].v[h] + redv[w * L::PC + 2 * d + 1].v[h];
                }
                const float s = load_elem<DT>(g.vs, bh * kD + d);
                const float z = load_elem<DT>(g.vz, bh * kD + d);
                // pick this thread's head out of the per-head sums
                float lh = l_img[0];
#pragma unroll
                for (int k = 1; k < HPB; ++k) lh = (h == k) ? l_img[k] : lh;
                o_img = s * (a - z * lh);
            }
            __syncthreads();
        }

        // ---- phase 5: full-precision residual rows, online softmax ----------------
        float m_res[HPB], l_res[HPB];
#pragma unroll
        for (int h = 0; h < HPB; ++h) { m_res[h] = -INFINITY; l_res[h] = 0.f; }
        float o_res = 0.f;
        if (do_res) {
            float* sres = fx + L::F_SRES;
            float* pres = fx + L::F_PRES;
            const int l8 = tid & 7, row = tid >> 3;
            const int ds = tid & 15, rslot = tid >> 4;
            float qa[HPB][16];
#pragma unroll
            for (int h = 0; h < HPB; ++h)
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    qa[h][k] = qf[h * kD + l8 * 8 + k];
                    qa[h][8 + k] = qf[h * kD + 64 + l8 * 8 + k];
                }
            float accv[8][HPB];
#pragma unroll
            for (int k = 0; k < 8; ++k)
#pragma unroll
                for (int h = 0; h < HPB; ++h) accv[k][h] = 0.f;
            const uint16_t* kb = static_cast<const uint16_t*>(g.kres) + b * g.rs_b + hkv * g.rs_h;
            const uint16_t* vbp = static_cast<const uint16_t*>(g.vres) + b * g.rs_b + hkv * g.rs_h;
            const float* mk = g.mask ? g.mask + b * g.mask_sb : nullptr;

            for (int r0 = 0; r0 < g.R; r0 += kResTile) {
                const int r = r0 + row;
                float dot[HPB];
#pragma unroll
                for (int h = 0; h < HPB; ++h) dot[h] = 0.f;
                if (r < g.R) {
                    const uint16_t* kp = kb + r * g.rs_r;
                    const uint4 v0 = *reinterpret_cast<const uint4*>(kp + l8 * 8);
                    const uint4 v1 = *reinterpret_cast<const uint4*>(kp + 64 + l8 * 8);
                    float f[16];
                    unpack8<DT>(v0, f);
                    unpack8<DT>(v1, f + 8);
#pragma unroll
                    for (int h = 0; h < HPB; ++h)
#pragma unroll
                        for (int k = 0; k < 16; ++k) dot[h] += qa[h][k] * f[k];
                }
#pragma unroll
                for (int h = 0; h < HPB; ++h) {
                    dot[h] += __shfl_xor(dot[h], 1, kWave);
                    dot[h] += __shfl_xor(dot[h], 2, kWave);
                    dot[h] += __shfl_xor(dot[h], 4, kWave);
                }
                if (l8 == 0) {
                    float mv = 0.f;
                    if (mk && r < g.R) mv = mk[r < g.S ? r : g.T + r];
#pragma unroll
                    for (int h = 0; h < HPB; ++h) sres[row * HPB + h] = (r < g.R) ? dot[h] + mv : -INFINITY;
                }
                __syncthreads();
                float alpha[HPB];
#pragma unroll
                for (int h = 0; h < HPB; ++h) {
                    const float s = sres[lane * HPB + h];
                    const float mt = wave_max(s);
                    const float mnew = fmaxf(m_res[h], mt);
                    float p = 0.f;
                    alpha[h] = 1.0f;
                    if (mnew != -INFINITY) {
                        p = __expf(s - mnew);
                        alpha[h] = __expf(m_res[h] - mnew);
                    }
                    const float lt = wave_sum(p);
                    l_res[h] = l_res[h] * alpha[h] + lt;
                    m_res[h] = mnew;
                    if (wv == 0) pres[lane * HPB + h] = p;
                }
                __syncthreads();
#pragma unroll
                for (int k = 0; k < 8; ++k)
#pragma unroll
                    for (int h = 0; h < HPB; ++h) accv[k][h] *= alpha[h];
#pragma unroll
                for (int rep = 0; rep < kResTile / (kNT / 16); ++rep) {
                    const int rr = rslot + rep * (kNT / 16);
                    const int r2 = r0 + rr;
                    if (r2 < g.R) {
                        const uint4 vv = *reinterpret_cast<const uint4*>(vbp + r2 * g.rs_r + ds * 8);
                        float f[8];
                        unpack8<DT>(vv, f);
                        const V p = reinterpret_cast<const V*>(pres)[rr];
#pragma unroll
                        for (int k = 0; k < 8; ++k)
#pragma unroll
                            for (int h = 0; h < HPB; ++h) accv[k][h] += p.v[h] * f[k];
                    }
                }
            }
            // fold the row slots: 4 per wave (lane bits 4,5), then the waves
#pragma unroll
            for (int k = 0; k < 8; ++k)
#pragma unroll
                for (int h = 0; h < HPB; ++h) {
                    accv[k][h] += __shfl_xor(accv[k][h], 16, kWave);
                    accv[k][h] += __shfl_xor(accv[k][h], 32, kWave);
                }
            __syncthreads();
            float* red2 = reinterpret_cast<float*>(regA);  // [wave][kD][HPB]
            if (lane < 16) {
#pragma unroll
                for (int k = 0; k < 8; ++k)
#pragma unroll
                    for (int h = 0; h < HPB; ++h) red2[(wv * kD + ds * 8 + k) * HPB + h] = accv[k][h];
            }
            __syncthreads();
            if (tid < HPB * kD) {
                const int h = tid / kD, d = tid % kD;
#pragma unroll
                for (int w = 0; w < kNW; ++w) o_res += red2[(w * kD + d) * HPB + h];
            }
        }

        // ---- phase 6: merge / write -------------------------------------------------
        if (tid < HPB * kD) {
            const int h = tid / kD, d = tid % kD;
            float mi = m_img[0], li = l_img[0], mr = m_res[0], lr = l_res[0];
#pragma unroll
            for (int k = 1; k < HPB; ++k) {
                mi = (h == k) ? m_img[k] : mi; li = (h == k) ? l_img[k] : li;
                mr = (h == k) ? m_res[k] : mr; lr = (h == k) ? l_res[k] : lr;
            }
            const int64_t row = static_cast<int64_t>(b) * g.Hq + hq0 + h;
            if (g.nsplit == 1) {
                const float mf = fmaxf(mi, mr);
                const float wi = (mi == -INFINITY) ? 0.f : __expf(mi - mf);
                const float wr = (mr == -INFINITY) ? 0.f : __expf(mr - mf);
                const float num = o_img * wi + o_res * wr;
                const float den = li * wi + lr * wr;
                store_elem<DT>(g.out, row * kD + d, num / den);
            } else {
                float* p = g.part + (row * g.nx + split) * (kD + 2);
                const bool is_img = split < g.nsplit;
                if (d == 0) { p[0] = is_img ? mi : mr; p[1] = is_img ? li : lr; }
                p[2 + d] = is_img ? o_img : o_res;
            }
        }
        (void)bc;
    }
}

// Combine the (m, l, acc) partials of one (batch, q-head) row.  grid (B*Hq), kD threads.
template <typename DT>
__global__ void merge_kernel(const float* __restrict__ part, int nx, void* __restrict__ out) {
    const int64_t row = blockIdx.x;
    const int d = threadIdx.x;
    const float* p = part + row * nx * (kD + 2);
    float m = -INFINITY;
    for (int s = 0; s < nx; ++s) m = fmaxf(m, p[s * (kD + 2)]);
    float num = 0.f, den = 0.f;
    for (int s = 0; s < nx; ++s) {
        const float ms = p[s * (kD + 2)];
        const float w = (ms == -INFINITY) ? 0.f : __expf(ms - m);
        den += p[s * (kD + 2) + 1] * w;
        num += p[s * (kD + 2) + 2 + d] * w;
    }
    store_elem<DT>(out, row * kD + d, num / den);
}

struct Plan {
    int hpb, nsplit, chunk, nx, cap, lds;
    size_t ws_mm, ws_part;
};

template <int BITS, int HPB>
static void plan_for(const cq_decode_args* a, Plan* p) {
    using L = Lay<BITS, HPB>;
    const int G = a->Hq / a->Hkv;
    const int64_t units = static_cast<int64_t>(a->B) * a->Hkv * (G / HPB);
    const int maxc = L::max_chunk();
    int nsplit = 1;
    if (a->T > 0) {
        const int need = (a->T + maxc - 1) / maxc;
        nsplit = need;
        if (a->force_splits > 0) {
            nsplit = a->force_splits > need ? a->force_splits : need;
        } else if (units < 192) {
            int64_t want = (512 + units - 1) / units;
            int64_t most = a->T / 1024 > 1 ? a->T / 1024 : 1;
            if (want > most) want = most;
            if (want > nsplit) nsplit = static_cast<int>(want);
        }
    }
    int chunk = a->T > 0 ? ((a->T + nsplit - 1) / nsplit + 63) / 64 * 64 : 64;
    if (chunk > maxc) chunk = maxc;
    nsplit = a->T > 0 ? (a->T + chunk - 1) / chunk : 1;
    p->hpb = HPB;
    p->nsplit = nsplit;
    p->chunk = chunk;
    p->nx = nsplit + ((nsplit > 1 && a->R > 0) ? 1 : 0);
    p->cap = a->T > 0 ? chunk : 64;
    p->lds = L::lds_bytes(p->cap);
    const size_t rows = static_cast<size_t>(a->B) * a->Hq;
    p->ws_mm = nsplit > 1 ? ((rows * nsplit * 2 * sizeof(float) + 255) / 256 * 256) : 0;
    p->ws_part = nsplit > 1 ? rows * p->nx * (kD + 2) * sizeof(float) : 0;
}

static int make_plan(const cq_decode_args* a, Plan* p) {
    if (!a) return CQ_ERR_NULL;
    if (a->dtype != CQ_BF16 && a->dtype != CQ_FP16) return CQ_ERR_DTYPE;
    if (a->bits != 1 && a->bits != 2) return CQ_ERR_UNSUPPORTED;
    if (a->D != kD) return CQ_ERR_UNSUPPORTED;
    if (a->B < 1 || a->Hq < 1 || a->Hkv < 1 || a->Hq % a->Hkv) return CQ_ERR_SHAPE;
    if (a->T < 0 || a->R < 0 || (a->T == 0 && a->R == 0)) return CQ_ERR_SHAPE;
    if (a->sprompt_len < 0 || a->sprompt_len > a->R) return CQ_ERR_SHAPE;
    const int G = a->Hq / a->Hkv;
    if (a->bits == 1) {
        if (G % 4 == 0) plan_for<1, 4>(a, p);
        else if (G % 2 == 0) plan_for<1, 2>(a, p);
        else plan_for<1, 1>(a, p);
    } else {
        if (G % 2 == 0) plan_for<2, 2>(a, p);
        else plan_for<2, 1>(a, p);
    }
    const int64_t blocks = static_cast<int64_t>(a->B) * a->Hkv * (G / p->hpb) * p->nx;
    if (blocks > 0x7fffffff) return CQ_ERR_SHAPE;
    return CQ_OK;
}

template <int BITS, int HPB, typename DT>
static int launch(const DecodeGeom& g, const Plan& p, hipStream_t st) {
    const int G = g.Hq / g.Hkv;
    const unsigned units = static_cast<unsigned>(g.B) * g.Hkv * (G / HPB);
    auto kmain = decode_kernel<BITS, HPB, DT, false>;
    auto kmm = decode_kernel<BITS, HPB, DT, true>;
    // raise the dynamic-LDS limit once per device for this instantiation
    static std::atomic<uint32_t> attr_done{0};
    int dev = 0;
    CQ_HIP_CHECK(hipGetDevice(&dev));
    const uint32_t bit = 1u << (dev & 31);
    if (!(attr_done.load(std::memory_order_acquire) & bit)) {
        CQ_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kmain),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, kLdsMax));
        CQ_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kmm),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, kLdsMax));
        attr_done.fetch_or(bit, std::memory_order_release);
    }
    if (g.nsplit > 1) {
        DecodeGeom g1 = g;
        g1.nx = g.nsplit;  // the min/max pass has no residual unit
        const int lds_mm = Lay<BITS, HPB>::lds_bytes(0);
        hipLaunchKernelGGL(kmm, dim3(units * g.nsplit), dim3(kNT), lds_mm, st, g1);
        CQ_LAUNCH_CHECK();
    }
    hipLaunchKernelGGL(kmain, dim3(units * g.nx), dim3(kNT), p.lds, st, g);
    CQ_LAUNCH_CHECK();
    if (g.nsplit > 1) {
        hipLaunchKernelGGL(merge_kernel<DT>, dim3(static_cast<unsigned>(g.B) * g.Hq), dim3(kD), 0, st, g.part, g.nx,
                           g.out);
        CQ_LAUNCH_CHECK();
    }
    return CQ_OK;
}

template <typename DT>
static int dispatch(const DecodeGeom& g, const Plan& p, int bits, hipStream_t st) {
    if (bits == 1) {
        if (p.hpb == 4) return launch<1, 4, DT>(g, p, st);
        if (p.hpb == 2) return launch<1, 2, DT>(g, p, st);
        return launch<1, 1, DT>(g, p, st);
    }
    if (p.hpb == 2) return launch<2, 2, DT>(g, p, st);
    return launch<2, 1, DT>(g, p, st);
}

}  // namespace cq

extern "C" {

size_t cq_decode_attn_workspace(const cq_decode_args* args) {
    cq::Plan p;
    if (cq::make_plan(args, &p) != CQ_OK) return 0;
    return p.ws_mm + p.ws_part;
}

int cq_decode_attn(const cq_decode_args* a, cq_stream_t stream) {
    cq::Plan p;
    int rc = cq::make_plan(a, &p);
    if (rc != CQ_OK) return rc;
    if (!a->q || !a->out) return CQ_ERR_NULL;
    if (a->T > 0 && (!a->codes_k || !a->codes_v || !a->k_scale || !a->k_zero || !a->v_scale || !a->v_zero))
        return CQ_ERR_NULL;
    if (a->R > 0 && (!a->k_res || !a->v_res)) return CQ_ERR_NULL;
    if (a->T > 0 && (!cq::aligned16(a->codes_k) || !cq::aligned16(a->codes_v))) return CQ_ERR_ALIGN;
    if (a->R > 0 && (!cq::aligned16(a->k_res) || !cq::aligned16(a->v_res) || (a->res_stride_b % 8) ||
                     (a->res_stride_h % 8) || (a->res_stride_r % 8)))
        return CQ_ERR_ALIGN;
    const size_t need = p.ws_mm + p.ws_part;
    if (need && (!a->workspace || a->workspace_bytes < need || !cq::aligned16(a->workspace))) return CQ_ERR_WORKSPACE;

    cq::DecodeGeom g;
    g.q = a->q; g.ck = a->codes_k; g.cv = a->codes_v;
    g.ks = a->k_scale; g.kz = a->k_zero; g.vs = a->v_scale; g.vz = a->v_zero;
    g.kres = a->k_res; g.vres = a->v_res;
    g.rs_b = a->res_stride_b; g.rs_h = a->res_stride_h; g.rs_r = a->res_stride_r;
    g.mask = a->mask; g.mask_sb = a->mask_stride_b;
    g.out = a->out;
    g.mm = static_cast<float*>(a->workspace);
    g.part = need ? reinterpret_cast<float*>(static_cast<char*>(a->workspace) + p.ws_mm) : nullptr;
    g.B = a->B; g.Hq = a->Hq; g.Hkv = a->Hkv; g.T = a->T; g.R = a->R; g.S = a->sprompt_len;
    g.nsplit = p.nsplit; g.chunk = p.chunk; g.nx = p.nx;
    g.calib = a->calibrate; g.off_max = a->calib_off_max; g.off_min = a->calib_off_min;
    g.cap = p.cap;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (a->dtype == CQ_BF16) return cq::dispatch<cq::BF16>(g, p, a->bits, st);
    return cq::dispatch<cq::FP16>(g, p, a->bits, st);
}

}  // extern "C"
