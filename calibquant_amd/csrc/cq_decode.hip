// Fused decode attention over bit-packed K/V for gfx950 (MI355X).
//
// One workgroup (1024 threads, or 512 threads with two workgroups resident per compute
// unit when there are more units than compute units) owns one (batch, kv-head,
// head-group, token-chunk) unit and runs the whole step for HPB query heads that share
// the kv-head:
//
//   loads    the packed K rows are requested at kernel entry, the first block of
//            packed V rows behind them (half before the logits, half as the K
//            registers free up), the first tile of residual K/V rows when the
//            packed-V phase ends: each stream is in flight while the phase before
//            its consumer runs, and no phase starts behind a queue of requests
//            it does not need.
//   K side   q.s_k is folded into a byte-indexed partial-sum table in LDS
//            (one entry per byte position and byte value, HPB floats wide,
//            zero-point folded in).  A token's logits are NB table look-ups
//            and adds; the fp16/bf16 K tensor is never materialised.
//   stats    min / max of the image logits (calibration), then e = exp(w' - M)
//            in place in LDS.
//   V side   tokens are taken four at a time: a 16-entry table of subset sums
//            of their e values is built once per group, every byte column of
//            the packed V rows is staged byte-transposed (the 4 tokens' bytes of a
//            column in one dword), a 4-byte dot product turns each bit lane of the
//            column into a table offset, and the lane adds that table entry.  Scale /
//            zero-point are applied once at the end.
//   residual the full-precision rows run last as an online-softmax flash-decode in
//            the same workgroup (packed dot2 for q.K) and are merged at the end.
//
// When the chunk does not cover all T tokens (long context or small batch)
// a first launch computes every chunk's logits and publishes the per-chunk min / max;
// the main launch recomputes its chunk's logits (or, where the packed K row is more
// bytes than the logits - 2 bits, or fewer than four heads per unit - reads back what
// the first launch left in a buffer, fp32, instead of building the table and doing the
// look-ups again), exponentiates against the global min / max and writes an (m, l, acc)
// partial; the last workgroup of a unit to get there combines the unit's partials.
//
// Everything here is HBM / LDS / VALU work; no matrix-core instructions.
#include "cq_common.h"

// The kernels below lean on behaviour of this architecture family that the HIP memory model does not
// promise (see the in-launch merge of the chunked step) and on its LDS size, DPP controls and
// instruction set: refuse to build device code for anything else.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__) && !defined(__gfx942__)
#error "cq_decode.hip is written for gfx950 (validated on gfx950 only; gfx942 shares the memory behaviour relied on)"
#endif

#include <atomic>
#include <cstdlib>
#include <type_traits>

namespace cq {

constexpr int kD = 128;
constexpr int kPF = 4;             // 16-byte loads kept in flight per thread and stream
constexpr int kLdsMax = 160 * 1024;
constexpr int kDefaultUnits = 256; // compute units of a whole MI355X, assumed when no device can be asked
constexpr int kRegPair = 8;        // rounds of logits a thread of a 512-thread workgroup keeps in registers (4 096 tokens)
constexpr int kRegTwoBit = 4;      // ... of the 2-bit kernel with four heads per unit (4 096 tokens)
constexpr int kRegLong = 10;       // ... of a 1024-thread workgroup that holds a long chunk in one launch (10 240 tokens)
constexpr float kLog2e = 1.4426950408889634f;

// Profiling build (-DCQ_PHASE_STOPS, `python -m calibquant_amd.build --phase-stops`; only the headline
// instantiation is compiled): a launch can be told to end at a phase boundary (environment variable
// CQ_DECODE_PHASE_STOP = k, read per call), so that whole-launch hardware counters of runs with successive
// k give per-phase counts by subtraction.  The shipped library has none of this.
#ifdef CQ_PHASE_STOPS
#define CQ_PHASE(k) do { if (g.stop == (k)) return; } while (0)
#else
#define CQ_PHASE(k) do { } while (0)
#endif


template <int N> struct alignas(N * 4) Vec { float v[N]; };
// native 16-byte vector: copies are single vector moves (HIP's uint4 struct copies lower to memcpy)
typedef uint32_t U4 __attribute__((ext_vector_type(4)));

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
    const int32_t* r_dev;   // optional: residual row count read at run time (R is then the capacity)
    float* mm;    // [B][Hq][nsplit][2] chunk logit min / max
    float* part;  // [B][Hq][nx][kD + 2] partials (m, l, acc)
    float* lgt;   // chunked launch: [unit][T][HPB] logits, written by the min/max launch and read by the main
                  // launch instead of its own K look-ups; NULL: the main launch recomputes them
    int* cnt;     // chunked launch: [unit] count of the unit's chunks (+ residual unit) that have written their
                  // partial; the one that finds all the others done merges them
    // Chunked step in ONE launch (every chunk's workgroup resident at once): the chunks of a unit exchange their
    // logit min / max inside the launch.  rec: [unit][head][chunk][2] 64-bit records, a float (min, then max)
    // in the lower half and the call's epoch in the upper half - a record is valid by itself, so a chunk
    // publishes with plain write-through stores and waits for nothing, and the others poll the records
    // (whatever an earlier call or an uninitialised workspace left there has another epoch).  done64: [unit]
    // partials written, tagged with the epoch the same way.  status: host-visible word that a workgroup sets
    // when it gives up waiting (spin_limit polls); NULL: nowhere to report.
    unsigned long long* rec;
    unsigned long long* done64;
    int* status;
    uint32_t epoch;
    int fused;
    int spin_limit;
#ifdef CQ_PHASE_STOPS
    int stop;     // phase boundary at which the launch ends (-1: runs to the end)
#endif
    int B, Hq, Hkv, T, R, S;
    int nsplit, chunk, nx;
    int calib;
    float off_max, off_min;
    int cap;      // logits capacity of the LDS layout, tokens
    FastDiv d_ng, d_nx, d_hkv;   // divisors of the unit decomposition: head groups, chunks (+ residual unit), kv heads
    int G;        // query heads per kv head
    int ncu;      // paired launch whose workgroups are all resident from the start (at most two per compute unit):
                  // the number of compute units (the two workgroups of a unit are told apart by it); else 0
    float one;    // 1.0f, opaque to the compiler: keeps f16 -> f32 accumulation in one mixed-precision FMA
};

constexpr int cmax(int a, int b) { return a > b ? a : b; }
constexpr int cmin(int a, int b) { return a < b ? a : b; }

// VTOK: values quantised per token and per group of 32 channels (scale * code + minimum,
// codes in little-endian 32-bit words, first channel in the lowest bits) instead of per
// channel.  A token slot then also carries the token's group scales, and every channel
// group has its own subset-sum tables.
// REGL > 0: a thread keeps the logits of its tokens (at most REGL rounds of kNT tokens) in registers
// until the block's min / max are known and writes only e = exp(.) to the token slots, as packed fp16:
// the slots take half the bytes, which is what lets two 512-thread workgroups share a compute unit's
// LDS (with the K table built for half of the byte positions at a time), or one 1024-thread workgroup
// hold a chunk of 9 984 tokens.
template <int BITS, int HPB, bool VTOK = false, int NT_ = 1024, int REGL = 0> struct Lay {
    static constexpr int kNT = NT_;                 // threads per workgroup
    static constexpr int kNW = kNT / kWave;         // waves per workgroup
    // residual window: tiles of 128 rows for either workgroup size - a 512-thread workgroup puts 4 lanes on a
    // row (32 channels each), a 1024-thread one 8 (16 channels each)
    static constexpr int LPR = kNT / 128;           // lanes per residual row
    static constexpr int kResTile = kNT / LPR;      // residual rows per tile
    static constexpr int NKP = 16 / LPR;            // 16-byte pieces of a row per lane
    static constexpr int RPW = kResTile / kNW;      // rows of a tile whose values one wave multiplies
    static constexpr int NB = 16 * BITS;            // bytes per packed row
    static constexpr int PC = NB * 8;               // bit lanes per row
    static constexpr int GPW = kWave / NB;          // 4-token groups per wave pass
    static constexpr int MPL = 8 / GPW;             // bit lanes of a byte column handled by one lane
    static constexpr int TPW = 4 * GPW;             // tokens per wave pass
    static constexpr int ESZ = HPB * 4;             // bytes per fp32 table entry / logits slot
    static constexpr int HW = HPB >= 2 ? HPB / 2 : 1;   // 32-bit words per packed-fp16 entry
    static constexpr int ESZH = HW * 4;             // bytes per packed-fp16 table entry
    // The byte-indexed K table covers NBP byte positions at a time: all of them when that fits the
    // table's share of the LDS (64 KB; 32 KB for a 512-thread workgroup), else half of them in each of
    // two (or a quarter in each of four) passes over the chunk's rows, the earlier passes' partial logits
    // waiting in the token slots or, with REGL, in registers.
    // INA (512-thread workgroup with the logits in registers): nothing else lives in LDS while the K table is
    // in use, so the table takes all 64 KB of region A and the token slots, written only after the last
    // look-up, sit in that region as well, behind the staged V block - one table pass at 1 bit (two at 2 bits)
    // with 256-byte rows, i.e. single-permute look-up addresses, inside the 80 KB a paired workgroup may use.
    // The table is then built straight from the per-bit weights (no nibble tables to find room for).
    static constexpr bool INA = (NT_ == 512 && REGL > 0);
    static constexpr int KTMAX = ((NT_ == 512 && !INA) ? 32 : 64) * 1024;
    static constexpr int KPASS = (NB * 256 * ESZ > 2 * KTMAX) ? 4 : (NB * 256 * ESZ > KTMAX) ? 2 : 1;
    static constexpr int NBP = NB / KPASS;          // byte positions per pass
    static constexpr int WPP = NBP / 4;             // 32-bit words of a row per pass
    static constexpr int PCS = (WPP + 3) / 4;       // 16-byte pieces of a row a pass looks at
    static constexpr int KT = NBP * 256 * ESZ;      // K table bytes
    static_assert(NB * 256 * ESZ <= 4 * KTMAX, "at most four table passes");
    static_assert(!(REGL > 0 && VTOK), "logits in registers: per-channel values only");
    static constexpr int SLOT = VTOK ? 16 : (REGL > 0 ? ESZH : ESZ);   // bytes per token slot: logits, later e (+ 4 group scales)
    static constexpr int NGRP = VTOK ? kD / 32 : 1; // channel groups with tables of their own
    static constexpr int WTAB = kNW * NGRP * GPW * 16 * ESZH;
    static constexpr int RW = cmax(3 * HPB, VTOK ? (NGRP + 1) * HPB : 0);   // per-wave partials: min/max + masked max, or the closing sums
    static constexpr int VSUB = kNT * kPF / BITS;   // V tokens staged at a time
    static constexpr int KR = kPF / BITS;           // K token rounds in flight per thread
    static constexpr int RED = kNW * PC * ESZ;
    static constexpr int RED2 = kNW * kD * ESZ;
    // fixed small region (floats)
    static constexpr int F_WBIT = 0;                          // NB*8*HPB
    static constexpr int F_QSZ = F_WBIT + NB * 8 * HPB;       // NB*HPB: zero-point sum per byte position and head
    static constexpr int F_QRAW = F_QSZ + NB * HPB;           // HPB*kD raw 16-bit q
    static constexpr int F_RED = F_QRAW + HPB * kD / 2;       // kNW*HPB
    static constexpr int F_STAT = F_RED + kNW * RW;           // 8*HPB: per-head softmax state
    static constexpr int F_VSZ = F_STAT + 8 * HPB;            // 2*kD: value scale, zero-point (VTOK: NGRP*HPB minimum terms)
    static constexpr int F_NIB = F_VSZ + 2 * kD;              // NB*32*HPB: nibble tables
    // (REGL: the nibble tables live in the token slots, which are first written after the last table pass;
    // INA: there are none)
    static constexpr int NIBF = NB * 32 * HPB;
    static constexpr int F_SRES = F_NIB + (REGL > 0 ? 0 : NIBF);  // kResTile*HPB
    static constexpr int F_PRES = F_SRES + kResTile * HPB;    // kResTile*HPB
    static constexpr int F_END = F_PRES + kResTile * HPB;
    static constexpr int FIXED = ((F_END * 4 + 255) / 256) * 256;
    // byte offset of the token slots: behind the fixed region, or (INA) inside region A behind the staged V block
    static constexpr int slots_in_a(int cap) { return WTAB + cmin(VSUB, cap) * NB; }
    static constexpr int region_a(int cap) {
        return (cmax(cmax(KT, slots_in_a(cap) + (INA ? cap * SLOT : 0)), cmax(RED, RED2)) + 255) / 256 * 256;
    }
    static constexpr int lds_bytes(int cap) {
        return region_a(cap) + FIXED + (INA ? 0 : cmax(cap * SLOT, REGL > 0 ? NIBF * 4 : 0));
    }
    // largest chunk whose layout fits: the whole LDS for a 1024-thread workgroup, half of it for a
    // 512-thread workgroup (two are meant to be resident per compute unit)
    static constexpr int max_chunk() {
        int best = 64;
        for (int c = 64; c <= 16384; c += 64)
            if (lds_bytes(c) <= (kNT == 512 ? kLdsMax / 2 : kLdsMax) && (REGL == 0 || c <= REGL * kNT)) best = c;
        return best;
    }
};

// One exchange step of an integer-key maximum, N values side by side: the N chains are
// independent, so the cross-lane moves of one fill the wait states of the others.
template <int N, int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ void max_step(int* k) {
    constexpr int lo = static_cast<int>(0x80000000u);
    int t[N];
#pragma unroll
    for (int h = 0; h < N; ++h) t[h] = dpp_move_i<CTRL, ROW_MASK>(k[h], lo);
#pragma unroll
    for (int h = 0; h < N; ++h) k[h] = max(k[h], t[h]);
}

// Block-wide maximum of N values (integer keys, see float_key); result wave-uniform.
// One barrier; `red`: N words that hold the smallest key when the first wave gets here.
template <int N, int kNW>
__device__ __forceinline__ void block_max(float* v, float* red) {
    const int lane = threadIdx.x & 63;
    int* redi = reinterpret_cast<int*>(red);
    int k[N];
#pragma unroll
    for (int h = 0; h < N; ++h) k[h] = float_key(v[h]);
    max_step<N, 0xB1>(k);
    max_step<N, 0x4E>(k);
    max_step<N, 0x141>(k);
    max_step<N, 0x140>(k);
    max_step<N, 0x142, 0xa>(k);
    max_step<N, 0x143, 0xc>(k);
    // second stage: the waves' maxima meet in N words of LDS (set to the smallest key before the last barrier
    // ahead of this call) through one atomic per wave and value
    if (lane == 63) {   // the last lane holds the wave's maxima
#pragma unroll
        for (int h = 0; h < N; ++h) __hip_atomic_fetch_max(redi + h, k[h], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < N; ++h) v[h] = key_float(__builtin_amdgcn_readfirstlane(redi[h]));
}

// Unit decomposition of a 1-D grid.  Consecutive work ids share packed codes
// (head groups of one kv-head), so when the grid is a multiple of the 8 XCDs
// the hardware's round-robin placement is undone to keep them on one L2.
__device__ __forceinline__ int virtual_block_id() {
    const int n = gridDim.x;
    const int l = blockIdx.x;
    if ((n & 7) == 0) return (l & 7) * (n >> 3) + (l >> 3);
    return l;
}

// Two-element dot product with fp32 accumulation on raw 16-bit pairs.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
template <typename DT> __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c);
template <> __device__ __forceinline__ float dot2<BF16>(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c, false);
}
template <> __device__ __forceinline__ float dot2<FP16>(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a), __builtin_bit_cast(f16x2_t, b), c, false);
}

template <int N> struct alignas(N * 4) Words { uint32_t w[N]; };

// N dwords at an absolute LDS byte address (N-dword aligned): one ds_read of that width.
template <int N> __device__ __forceinline__ Words<N> lds_words(uint32_t addr) {
    typedef uint32_t VT __attribute__((ext_vector_type(N)));
    const VT v = *(const __attribute__((address_space(3))) VT*)(static_cast<uintptr_t>(addr));
    Words<N> r;
#pragma unroll
    for (int k = 0; k < N; ++k) r.w[k] = v[k];
    return r;
}

// N floats at an absolute LDS byte address.
template <int N> __device__ __forceinline__ Vec<N> lds_floats(uint32_t addr) {
    typedef float VT __attribute__((ext_vector_type(N)));
    const VT v = *(const __attribute__((address_space(3))) VT*)(static_cast<uintptr_t>(addr));
    Vec<N> r;
#pragma unroll
    for (int k = 0; k < N; ++k) r.v[k] = v[k];
    return r;
}

// A float handed from one workgroup to another inside a launch: device-scope atomic store.
__device__ __forceinline__ void publish(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One more arrival at an epoch-tagged counter; returns the arrivals of this epoch including this one.
// Measured on this device: an atomic read-modify-write is executed at the memory side whatever scope it names
// (about 2 us a round trip, those on one address one after the other), so such counters are for counting once
// per workgroup, never for polling.
// peek64: the current value of a 64-bit word as the memory side holds it, a compare-and-swap of 0 for 0.  (Not a
// read-modify-write that changes nothing, such as OR 0: the compiler turns those into plain loads, which a
// compute unit's own cache may answer with what it read earlier.)
template <int SCOPE>
__device__ __forceinline__ unsigned long long peek64(unsigned long long* c) {
    unsigned long long v = 0ull;
    __hip_atomic_compare_exchange_strong(c, &v, 0ull, __ATOMIC_RELAXED, __ATOMIC_RELAXED, SCOPE);
    return v;
}

template <int SCOPE>
__device__ __forceinline__ uint32_t arrive(unsigned long long* c, uint32_t epoch) {
    unsigned long long old = peek64<SCOPE>(c);
    for (;;) {   // every failed exchange is another workgroup's success: at most as many rounds as workgroups
        const unsigned long long want = (static_cast<uint32_t>(old >> 32) == epoch)
                                            ? old + 1 : ((static_cast<unsigned long long>(epoch) << 32) | 1u);
        if (__hip_atomic_compare_exchange_strong(c, &old, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED, SCOPE))
            return static_cast<uint32_t>(want);
    }
}

// The single-launch chunked step's records and arrival counter of one unit back to empty: by the unit's last
// workgroup, once every other one is past both.
template <int HPB, int NT>
__device__ __forceinline__ void clear_handover(const DecodeGeom& g, int64_t unit, int tid) {
    for (int i = tid; i < HPB * g.nsplit * 2; i += NT)
        __hip_atomic_store(g.rec + unit * HPB * g.nsplit * 2 + i, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid == 0) __hip_atomic_store(g.done64 + unit, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ uint32_t pack_f16(float a, float b) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {a, b};
    const f16x2_t h = __builtin_convertvector(v, f16x2_t);   // one packed conversion, round to nearest even
    return __builtin_bit_cast(uint32_t, h);
}

// CHUNKED: the launch is one of the two of a chunked step (the min/max launch always is); a single launch carries
// none of their code.  EXTRAS: an additive mask or a residual row count read from device memory may be present; a
// call with neither runs an instantiation without their code (32.6-32.8 against 33.5-34.0 us at the benchmark shape:
// the kernel sits at the register limit of its occupancy, and code that never runs still costs registers).
// NH: query heads a unit serves, at most HPB.  Tables, slots and partials are laid out HPB heads wide either way
// (16-byte entries at HPB = 4); with NH = 3 the fourth lane of every entry is dead and the arithmetic on it is
// left out - six query heads per kv-head (InternLM2-20B) make two exact units of three instead of two units of
// four that carry two padding heads between them.
template <int BITS, int HPB, typename DT, bool MINMAX_ONLY, bool VTOK = false, int NT = 1024, int REGL = 0,
          bool CHUNKED = MINMAX_ONLY, bool EXTRAS = !MINMAX_ONLY, int NH = HPB>
// (four waves per SIMD - at most 128 VGPRs - for either workgroup size: two 512-thread workgroups per compute
// unit are only resident together within that)
__global__ __launch_bounds__(NT, 4) void decode_kernel(DecodeGeom g) {
    using L = Lay<BITS, HPB, VTOK, NT, REGL>;
    using V = Vec<HPB>;
    constexpr int NB = L::NB;
    constexpr int kNT = L::kNT, kNW = L::kNW, kResTile = L::kResTile;
    extern __shared__ __attribute__((aligned(256))) unsigned char smem[];
    const int reg_a = L::region_a(g.cap);
    unsigned char* regA = smem;
    float* fx = reinterpret_cast<float*>(smem + reg_a);
    unsigned char* slots = L::INA ? smem + L::slots_in_a(g.cap) : smem + reg_a + L::FIXED;   // one slot per token of the chunk
    auto slot = [&](int t) { return slots + t * L::SLOT; };
    float* wbit = fx + L::F_WBIT;
    float* qsz = fx + L::F_QSZ;
    float* red = fx + L::F_RED;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = tid >> 6;
    const int G = g.G;
    // Wave priorities of the paired launch (two 512-thread workgroups per compute unit, all of them
    // resident from the first cycle).  Left to the hardware's own arbitration the workgroup that was
    // dispatched first gets most of the issue slots: it ends after about 56 K cycles and the other one
    // after 77 K, the last 20 K alone on the unit with too few waves to hide its own latencies.  With the
    // short, latency-bound phases (set-up, table build, reductions, staging, exp) above the throughput
    // phases, the first workgroup ahead in the K look-ups and the second ahead in the packed-V loop,
    // both end together (measured at the benchmark shape: 36.0 -> 33.8 us, same results).  Launches with
    // more workgroups than fit at once start their later workgroups as earlier ones end, which staggers
    // them by itself; there the priorities are left alone (with them: 66 -> 84 us at batch 128).
    // `second`: the workgroup that shares its unit with an older one (workgroups are handed out unit by
    // unit, g.ncu at a time).
    const bool prio_on = NT == 512 && g.ncu > 0;
    const bool second = prio_on && blockIdx.x >= static_cast<unsigned>(g.ncu);
    auto phase_priority = [&](auto phase_c) {
        constexpr int PH = decltype(phase_c)::value;   // 0 set-up and tables, 1 K look-ups, 2 min/max .. exp, 3 packed V, 4 folds, window, merge
        if constexpr (NT == 512) {
            if (prio_on) {
                if constexpr (PH == 0 || PH == 2) __builtin_amdgcn_s_setprio(2);
                else if constexpr (PH == 1) { if (second) __builtin_amdgcn_s_setprio(0); else __builtin_amdgcn_s_setprio(1); }
                else if constexpr (PH == 3) { if (second) __builtin_amdgcn_s_setprio(2); else __builtin_amdgcn_s_setprio(1); }
                else __builtin_amdgcn_s_setprio(0);
            }
        }
    };
    // (unconditional at entry - with no later change every wave simply runs at this priority - so that no branch
    // on a kernel argument stands between the wave's start and the loads of the other arguments: all of them are
    // then requested in one go instead of in two round trips)
    if constexpr (NT == 512) __builtin_amdgcn_s_setprio(2);

    uint32_t vb = static_cast<uint32_t>(virtual_block_id());
    uint32_t qn = g.d_ng.quot(vb);
    const int hg = static_cast<int>(vb - qn * g.d_ng.div); vb = qn;
    qn = g.d_nx.quot(vb);
    const int split = static_cast<int>(vb - qn * g.d_nx.div); vb = qn;
    qn = g.d_hkv.quot(vb);
    const int hkv = static_cast<int>(vb - qn * g.d_hkv.div);
    const int b = static_cast<int>(qn);
    static_assert(NH >= 1 && NH <= HPB, "heads per unit");
    const int hq0 = hkv * G + hg * NH;
    const int nh = min(NH, G - hg * NH);   // query heads of this unit; the rest of its NH heads are padding
    const int64_t bh = static_cast<int64_t>(b) * g.Hkv + hkv;

    const bool img_unit = split < g.nsplit && g.T > 0;
    const int R = (EXTRAS && g.r_dev) ? min(*g.r_dev, g.R) : g.R;   // rows in the residual window
    const bool do_res = !MINMAX_ONLY && R > 0 && (!CHUNKED || split == g.nsplit);
    const int t0 = img_unit ? split * g.chunk : 0;
    const int n = img_unit ? min(g.T, t0 + g.chunk) - t0 : 0;
    const int npad = (n + L::TPW - 1) / L::TPW * L::TPW;
    const float inv_sqrt_d = 0.08838834764831845f;  // 1/sqrt(128)

    // ---- entry: the few elements phase 0 needs are requested first; the packed K rows follow
    // phase 0, packed V rows and the residual tile later still (see the file header).
    // Loads are unconditional with clamped (always valid) addresses: no divergent
    // control flow around them, so the compiler can wait on exactly the counter value
    // each consumer needs.
    // A unit without packed tokens or without residual rows aims the unused streams
    // at q (always mapped, at least 256 bytes) and never looks at what comes back.
    const bool has_img = n > 0;
    // chunked launch with a logits buffer: the min/max launch leaves this chunk's logits there and the main
    // launch takes them from there - no packed K rows, no table, no look-ups of its own
    const int64_t unit = bh * static_cast<int64_t>(g.d_ng.div) + hg;
    V* gl = reinterpret_cast<V*>(g.lgt) + (unit * g.T + t0);
    const bool from_gl = !MINMAX_ONLY && CHUNKED && g.lgt != nullptr && has_img;
    const bool k_rows = has_img && !from_gl;
    uint32_t q_raw, s_raw, z_raw;
    constexpr bool kVSep = (HPB * kD > kNT - kD);
    uint32_t vs_raw = 0, vz_raw = 0;
    {
        const int h = min(min(tid / kD, HPB - 1), nh - 1), d = tid % kD;   // a padding head repeats the last real one
        const uint16_t* qp = static_cast<const uint16_t*>(g.q) + (static_cast<int64_t>(b) * g.Hq + hq0) * kD;
        q_raw = qp[h * kD + d];
        // the last kD threads fetch the value statistics, unless they are q threads as well
        // (then the first kD threads fetch them with two loads of their own, below)
        const bool vstat = tid >= kNT - kD && !kVSep;
        const uint16_t* sp = has_img ? static_cast<const uint16_t*>((vstat && !VTOK) ? g.vs : g.ks) + bh * kD : qp;
        const uint16_t* zp = has_img ? static_cast<const uint16_t*>((vstat && !VTOK) ? g.vz : g.kz) + bh * kD : qp;
        s_raw = sp[d];
        z_raw = zp[d];
        if constexpr (kVSep && !VTOK) {
            vs_raw = (has_img ? static_cast<const uint16_t*>(g.vs) + bh * kD : qp)[d];
            vz_raw = (has_img ? static_cast<const uint16_t*>(g.vz) + bh * kD : qp)[d];
        }
    }
    const int64_t code_off = has_img ? (bh * g.T + t0) * NB : 0;   // one offset for both code streams
    const uint4* ckp = reinterpret_cast<const uint4*>(k_rows ? g.ck + code_off : static_cast<const uint8_t*>(g.q));
    const uint4* cvp = reinterpret_cast<const uint4*>((has_img ? g.cv : static_cast<const uint8_t*>(g.q)) + code_off);
    const U4* cvp4 = reinterpret_cast<const U4*>(cvp);
    const int last_u = has_img ? n * NB / 16 - 1 : 0;   // last valid 16-byte unit of either stream
    const int last_uk = k_rows ? last_u : 0;
    // residual tile: K slice (row = tid / LPR, 128 / LPR elements); V: a wave owns RPW rows of the tile and a
    // lane one channel pair of each of them, so the value products need no fold inside the wave
    constexpr int LPR = L::LPR, NKP = L::NKP, RPW = L::RPW;
    const int lq = tid % LPR, krow = tid / LPR;
    const int wvr = __builtin_amdgcn_readfirstlane(wv);   // wave-uniform: scalar row arithmetic
    // (the strides are read where the other kernel arguments are, not behind the branch that needs them: one
    // round trip to the argument block instead of one more)
    // (a single launch: every workgroup has a window; of a chunked launch only the residual units do)
    int64_t arg_rs_b = g.rs_b, arg_rs_h = g.rs_h, arg_rs_r = g.rs_r;
    if constexpr (!CHUNKED) asm volatile("" : "+s"(arg_rs_b), "+s"(arg_rs_h), "+s"(arg_rs_r));
    const int64_t res_off = do_res ? b * arg_rs_b + hkv * arg_rs_h : 0;   // one offset for both windows
    const uint16_t* kb = static_cast<const uint16_t*>(do_res ? g.kres : g.q) + res_off;
    const uint16_t* vbp = static_cast<const uint16_t*>(do_res ? g.vres : g.q) + res_off;
    const int last_r = do_res ? R - 1 : 0;
    const int64_t rs_r = do_res ? arg_rs_r : 0;
    uint4 rk[NKP];
    uint32_t rv[RPW];
    auto load_res_k = [&](int r0, uint4* k2) {   // rows past R re-read row R-1 (their logit is masked)
        const uint16_t* kp = kb + min(r0 + krow, last_r) * rs_r + lq * 8;
#pragma unroll
        for (int i = 0; i < NKP; ++i) k2[i] = *reinterpret_cast<const uint4*>(kp + i * (LPR * 8));   // piece i * LPR + lq
    };
    auto load_res_v = [&](int r0, uint32_t* v8) {   // rows past R re-read row R-1 (their weight is 0)
#pragma unroll
        for (int i = 0; i < RPW; ++i) {
            const int r2 = min(r0 + wvr * RPW + i, last_r);
            v8[i] = *reinterpret_cast<const uint32_t*>(vbp + r2 * rs_r + 2 * lane);
        }
    };

    CQ_PHASE(1);   // prologue, requests of q and the statistics
    // ---- phase 0: q, per-bit weights ---------------------------------------------------
    if (tid < HPB * kD) {
        const int h = tid / kD, d = tid % kD;
        const float qraw = Cvt<DT>::to_float(q_raw);
        reinterpret_cast<uint16_t*>(fx + L::F_QRAW)[h * kD + d] = static_cast<uint16_t>(q_raw);
        const float qv = qraw * inv_sqrt_d;
        if (n > 0) {
            const float s = Cvt<DT>::to_float(s_raw);
            const float z = Cvt<DT>::to_float(z_raw);
            const float qs = qv * s;
            // zero-point term of the byte position: sum of q s z over the channels of one byte
            // (consecutive lanes), kept [byte position][head]
            constexpr int cpb0 = 8 / BITS;
            const float zsum = (cpb0 == 8) ? oct_reduce(qs * z, OpSum(), 0.f) : quad_reduce(qs * z, OpSum(), 0.f);
            if (d % cpb0 == 0) qsz[(d / cpb0) * HPB + h] = zsum;
            if constexpr (BITS == 1) {
                wbit[((7 - (d & 7)) * NB + (d >> 3)) * HPB + h] = qs;   // [bit][byte position][head]
            } else {
                const int sh = 6 - 2 * (d & 3);
                wbit[(sh * NB + (d >> 2)) * HPB + h] = qs;
                wbit[((sh + 1) * NB + (d >> 2)) * HPB + h] = 2.0f * qs;
            }
        }
    }
    if constexpr (kVSep) {
        if (!VTOK && n > 0 && tid < kD) {
            fx[L::F_VSZ + tid] = Cvt<DT>::to_float(vs_raw);
            fx[L::F_VSZ + kD + tid] = Cvt<DT>::to_float(vz_raw);
        }
    } else if (!VTOK && n > 0 && tid >= kNT - kD) {
        const int d = tid - (kNT - kD);
        fx[L::F_VSZ + d] = Cvt<DT>::to_float(s_raw);
        fx[L::F_VSZ + kD + d] = Cvt<DT>::to_float(z_raw);
    }
    if (tid < 3 * HPB) reinterpret_cast<int*>(red)[tid] = static_cast<int>(0x80000000u);   // block_max's meeting words
    // The packed K rows are requested only now: a wave that has to queue 64 KB of requests
    // first gets to phase 0 thousands of cycles later, and the table build below covers
    // their latency anyway.
    // (requested any later - after the table build, or all but the first round - the launch is slower;
    // requested at kernel entry, ahead of q, as well)
    uint4 kc[L::KR][BITS];
#pragma unroll
    for (int r = 0; r < L::KR; ++r) {
#pragma unroll
        for (int i = 0; i < BITS; ++i) kc[r][i] = ckp[min((tid + r * kNT) * BITS + i, last_uk)];
    }
    // Chunked launch: the chunks' logit min / max, lane s the pair of chunk s for every head (all in flight
    // together; they are folded across the wave where the calibration needs them), and - with a logits
    // buffer and the logits in registers - this thread's logits.
    struct alignas(8) MinMax { float lo, hi; };
    MinMax mraw[HPB];
    // REGL: the logits of this thread's tokens, round r = token tid + r * kNT
    V lg[REGL > 0 ? REGL : 1];
    if constexpr (!MINMAX_ONLY) {
        if (CHUNKED && has_img && !g.fused) {
#pragma unroll
            for (int h = 0; h < HPB; ++h) {
                const MinMax* p = reinterpret_cast<const MinMax*>(g.mm) +
                                  (static_cast<int64_t>(b) * g.Hq + hq0 + min(h, nh - 1)) * g.nsplit;
                mraw[h] = p[min(lane, g.nsplit - 1)];
            }
        }
        if constexpr (REGL > 0) {
            if (from_gl) {
#pragma unroll
                for (int rd = 0; rd < REGL; ++rd) lg[rd] = gl[min(tid + rd * kNT, n - 1)];
            }
        }
    }
    __syncthreads();

    float* stat = fx + L::F_STAT;   // [alpha | m_res | l_res | m_img | l_img][HPB]
    float o_res = 0.f;
    float mn[HPB], mx[HPB];
#pragma unroll
    for (int h = 0; h < HPB; ++h) { mn[h] = h < NH ? INFINITY : 0.f; mx[h] = h < NH ? -INFINITY : 0.f; }
    // logits (later: calibrated, masked logits) of a token: in its slot, or in the thread's registers
    auto load_logits = [&](int rd, int tt) {
        if constexpr (REGL > 0) return lg[rd];
        else return *reinterpret_cast<const V*>(slot(tt));
    };
    auto store_logits = [&](int rd, int tt, const V& w) {
        if constexpr (REGL > 0) lg[rd] = w;
        else *reinterpret_cast<V*>(slot(tt)) = w;
    };
    // f(round, token) for the thread's tokens below lim; with REGL the rounds are unrolled so that
    // lg[] is indexed by constants
    auto for_my_tokens = [&](int lim, auto&& f) {
        if constexpr (REGL > 0) {
#pragma unroll
            for (int rd = 0; rd < REGL; ++rd) {
                const int tt = tid + rd * kNT;
                if (tt < lim) f(rd, tt);
            }
        } else {
            for (int tt = tid; tt < lim; tt += kNT) f(0, tt);
        }
    };
    // First block of packed V rows: half of it is requested here, behind the packed K rows, the
    // rest as the K registers free up, so it has arrived when the logits are done.
    U4 vc[kPF];
    auto request_v = [&](int r) { vc[r] = cvp4[min((tid + (r / BITS) * kNT) * BITS + r % BITS, last_u)]; };
    constexpr int kVEarly = kPF / 2;
    if constexpr (!MINMAX_ONLY) {
#pragma unroll
        for (int r = 0; r < kVEarly; ++r) request_v(r);
    }

    if (from_gl) {
        // (the look-up rounds, which request the rest of the first packed V block as they go, do not run)
#pragma unroll
        for (int r = kVEarly; r < kPF; ++r) request_v(r);
        if constexpr (REGL == 0) for_my_tokens(n, [&](int rd, int tt) { store_logits(rd, tt, gl[tt]); });
    }
    CQ_PHASE(2);   // q, per-bit weights, first packed K rows requested
    if (k_rows) {
        // ---- phase 2: byte table = high-nibble table + low-nibble table ----------------
        // nibble tables: entry (j, half, v) = sum of the per-bit weights v selects; the
        // zero-point sum of the byte position is folded into the high half.
        V* nib = REGL > 0 ? reinterpret_cast<V*>(slots) : reinterpret_cast<V*>(fx + L::F_NIB);   // [half*16 + value][byte position]
        V* ktab = reinterpret_cast<V*>(regA);           // [byte value][byte position]
        if constexpr (!L::INA)
        for (int e = tid; e < NB * 32; e += kNT) {
            const int j = e % NB, half = (e / NB) >> 4, v = (e / NB) & 15;
            // position-fastest: the lanes of a wave read consecutive entries
            const V* wb = reinterpret_cast<const V*>(wbit) + half * 4 * NB + j;
            V acc;
            const V zs = reinterpret_cast<const V*>(qsz)[j];
#pragma unroll
            for (int h = 0; h < HPB; ++h) acc.v[h] = half ? -zs.v[h] : 0.f;
#pragma unroll
            for (int bt = 0; bt < 4; ++bt) {
                const V w4 = wb[bt * NB];
                const float f = static_cast<float>((v >> bt) & 1);
#pragma unroll
                for (int h = 0; h < HPB; ++h) acc.v[h] += f * w4.v[h];
            }
            nib[e] = acc;
        }
        if constexpr (!L::INA) __syncthreads();

        phase_priority(std::integral_constant<int, 1>{});
        // ---- phase 3: logits of the chunk ------------------------------------------------
        // Lane l walks the byte positions of a pass in the order k ^ (l mod NBP): in every step
        // the lanes that the LDS serves together read NBP distinct positions of the
        // position-fastest table, i.e. distinct banks whatever the byte values are.  The
        // row is permuted by the same XOR once, so step k finds its byte at a fixed place.
        // The NBP terms are added as a balanced binary tree over k; an XOR of the leaf index
        // only swaps the two children of some tree levels, so every lane gets bit-identical
        // logits for identical rows.
        constexpr int NBP = L::NBP;
        constexpr int NW32 = NBP / 4;
        const int skew = lane % NBP;
        // byte i of a word <- byte i ^ (skew & 3)
        const uint32_t bsel = (0x03020100u ^ (0x01010101u * (skew & 3)));
        uint32_t pofs[NBP];   // byte offset of position k ^ skew inside a table row
#pragma unroll
        for (int k = 0; k < NBP; ++k) pofs[k] = (k ^ skew) * L::ESZ;
        const unsigned char* ktab_b = regA;
        // With 256-byte table rows the address of a look-up is two bytes side by side, the
        // byte value above the position offset: one byte permute builds it from the row word
        // and a word holding four position offsets.
        constexpr bool kPermAddr = (NBP * L::ESZ == 256);
        uint32_t pofs4[NBP / 4];
#pragma unroll
        for (int i = 0; i < NBP / 4; ++i)
            pofs4[i] = pofs[4 * i] | (pofs[4 * i + 1] << 8) | (pofs[4 * i + 2] << 16) | (pofs[4 * i + 3] << 24);
        // c: the L::PCS 16-byte pieces of the row that pass P looks at; rd: the token's round (REGL)
        // kLateMM (one table pass, logits in registers): a wave works out a round's logits for all its lanes as soon
        // as its first lane has a token - the lanes past the chunk's end hold a copy of its last row (clamped
        // request) and get that token's logits - so the min / max can be taken afterwards over the registers, two
        // rounds per instruction, with no lane left out.
        constexpr bool kLateMM = L::KPASS == 1 && REGL > 0 && !MINMAX_ONLY;
        // a table entry: the NH live floats of it (12 bytes at three heads)
        auto lds_entry = [&](uint32_t addr) {
            V r;
            if constexpr (NH == HPB) {
                r = lds_floats<HPB>(addr);
            } else {
                typedef float VT __attribute__((ext_vector_type(NH)));
                const VT v = *(const __attribute__((address_space(3))) VT*)(static_cast<uintptr_t>(addr));
#pragma unroll
                for (int k = 0; k < HPB; ++k) r.v[k] = k < NH ? v[k < NH ? k : 0] : 0.f;
            }
            return r;
        };
        auto token_logits = [&](auto pass_c, int rd, int tt, const uint4* c) {
            constexpr int P = decltype(pass_c)::value;
            if (kLateMM ? (__builtin_amdgcn_readfirstlane(tt) < n) : (tt < n)) {
                constexpr int WO = (P * L::WPP) % 4;   // the pass's first word inside its first piece
                uint32_t w[NW32];
#pragma unroll
                for (int i = 0; i < NW32; ++i) {
                    const uint4& pc = c[(WO + i) / 4];
                    const int k4 = (WO + i) % 4;
                    w[i] = k4 == 0 ? pc.x : k4 == 1 ? pc.y : k4 == 2 ? pc.z : pc.w;
                }
#pragma unroll
                for (int st = 0; (1 << st) < NW32; ++st) {   // word i <- word i ^ (skew / 4)
                    const bool on = ((skew >> 2) >> st) & 1;
                    uint32_t t[NW32];
#pragma unroll
                    for (int i = 0; i < NW32; ++i) t[i] = w[i ^ (1 << st)];
#pragma unroll
                    for (int i = 0; i < NW32; ++i) w[i] = on ? t[i] : w[i];
                }
                uint32_t wds[NW32];
#pragma unroll
                for (int i = 0; i < NW32; ++i) wds[i] = __builtin_amdgcn_perm(w[i], w[i], bsel);
                // balanced-tree sum with a small stack of partial sums (level l holds 2^l terms)
                V part[6];
#pragma unroll
                for (int k = 0; k < NBP; ++k) {
                    V cur;
                    if constexpr (kPermAddr) {
                        const uint32_t sel = static_cast<uint32_t>(k & 3) | (static_cast<uint32_t>(4 + (k & 3)) << 8) | 0x0c0c0000u;
                        // The kernel's only LDS object is the dynamic array, so it starts at LDS
                        // address 0 and the K table with it (the host checks that the kernel has no
                        // static LDS before the first launch): the permute result is the address.
                        cur = lds_entry(__builtin_amdgcn_perm(wds[k >> 2], pofs4[k >> 2], sel));
                    } else {
                        const uint32_t byte = (wds[k >> 2] >> (8 * (k & 3))) & 0xffu;
                        cur = *reinterpret_cast<const V*>(ktab_b + byte * (NBP * L::ESZ) + pofs[k]);
                    }
#pragma unroll
                    for (int l = 0; l < 6; ++l) {
                        if ((k >> l) & 1) {
#pragma unroll
                            for (int h = 0; h < NH; ++h) cur.v[h] += part[l].v[h];
                        } else {
                            part[l] = cur;
                            break;
                        }
                    }
                    if (k == NBP - 1) part[5] = cur;
                    // keep at most 8 look-ups in flight: bounds the registers this loop needs
                    if ((k & 7) == 7) __builtin_amdgcn_sched_barrier(0);
                }
                V acc = part[5];
                if constexpr (P > 0) {   // add the earlier pass's partial
                    const V prev = load_logits(rd, tt);
#pragma unroll
                    for (int h = 0; h < NH; ++h) acc.v[h] += prev.v[h];
                }
#pragma unroll
                for (int h = NH; h < HPB; ++h) acc.v[h] = 0.f;   // dead lanes of the entry
                if constexpr (!MINMAX_ONLY || P + 1 < L::KPASS) store_logits(rd, tt, acc);
                if constexpr (MINMAX_ONLY && P + 1 == L::KPASS) {
                    if (g.lgt) gl[tt] = acc;   // for the main launch
                }
                if constexpr (P + 1 == L::KPASS && !kLateMM) {
#pragma unroll
                    for (int h = 0; h < NH; ++h) { mn[h] = fminf(mn[h], acc.v[h]); mx[h] = fmaxf(mx[h], acc.v[h]); }
                }
            }
        };
        // The min/max launch has no value rows, tables or sums to keep: with the logits in registers it also keeps
        // the packed K rows of all its tokens there across the table passes instead of requesting, in every pass, the
        // 16-byte piece that pass looks at (at 2 bits, four passes: 214 MB fetched for 67 MB of rows at batch 8 x
        // 32 768 - the rows of the 512 workgroups in flight do not fit the L2s between two passes).
        constexpr bool kKeepRows = MINMAX_ONLY && REGL > 0 && L::KPASS > 1;
        uint4 kall[kKeepRows ? REGL : 1][BITS];
        // Two table passes in a paired workgroup (2 bits): the first pass requests whole rows and keeps the
        // 16-byte piece the second pass looks at in registers - requested one piece per pass, every 32-byte row
        // would cross the memory system twice (a piece is half a row, and memory is fetched by the row or more).
        constexpr bool kKeepHalf = !MINMAX_ONLY && L::INA && L::KPASS == 2 && BITS == 2 && !kKeepRows;
        uint4 khalf[kKeepHalf ? REGL : 1];
        auto k_pass = [&](auto pass_c) {
            constexpr int P = decltype(pass_c)::value;
            constexpr int kP0 = (P * L::WPP) / 4;   // first 16-byte piece of a row the pass looks at
            if constexpr (L::INA) {
                // Straight from the per-bit weights: a thread owns (position, high nibble, bit 3) and writes the
                // eight entries of the low three bits - the part common to all eight first, then one or two adds
                // per entry; a wave writes four whole 256-byte rows at a time.
                static_assert(!L::INA || (NBP == 16 && kNT == 512), "thread mapping of the direct table build");
                const int pos = tid & 15, hv = (tid >> 4) & 15, b3 = tid >> 8;
                const V* wb = reinterpret_cast<const V*>(wbit) + P * NBP + pos;
                const V zs = reinterpret_cast<const V*>(qsz)[P * NBP + pos];
                V base;
#pragma unroll
                for (int h = 0; h < HPB; ++h) base.v[h] = -zs.v[h];
#pragma unroll
                for (int bt = 3; bt < 8; ++bt) {
                    const V w4 = wb[bt * NB];
                    const float f = static_cast<float>(bt == 3 ? b3 : (hv >> (bt - 4)) & 1);
#pragma unroll
                    for (int h = 0; h < HPB; ++h) base.v[h] += f * w4.v[h];
                }
                const V w0 = wb[0], w1 = wb[NB], w2 = wb[2 * NB];
                V hp[2], p01;
#pragma unroll
                for (int h = 0; h < HPB; ++h) {
                    hp[0].v[h] = base.v[h];
                    hp[1].v[h] = base.v[h] + w2.v[h];
                    p01.v[h] = w0.v[h] + w1.v[h];
                }
                V* row = ktab + (hv * 16 + b3 * 8) * NBP + pos;
#pragma unroll
                for (int l = 0; l < 8; ++l) {
                    V o = hp[l >> 2];
                    if ((l & 3) != 0) {
                        const V& ad = (l & 3) == 1 ? w0 : (l & 3) == 2 ? w1 : p01;
#pragma unroll
                        for (int h = 0; h < HPB; ++h) o.v[h] += ad.v[h];
                    }
                    row[l * NBP] = o;
                }
            } else {
            // byte table of the pass's positions = high-nibble table + low-nibble table
            for (int e = tid; e < NBP * 256; e += kNT) {
                const int j = P * NBP + e % NBP, v = e / NBP;
                const V hi = nib[(16 + (v >> 4)) * NB + j];
                const V lo = nib[(v & 15) * NB + j];
                V o;
#pragma unroll
                for (int h = 0; h < HPB; ++h) o.v[h] = hi.v[h] + lo.v[h];
                ktab[e] = o;
            }
            }
            __syncthreads();
            // One table pass, logits in registers: the rows stream through the KR row registers - when a
            // round's row has been looked up its registers take the row of KR rounds later, so KR rounds
            // are in flight while one is worked on and no batch of rows is waited for as a whole.
            constexpr bool kRotate = L::KPASS == 1 && REGL > 0;
            if constexpr (kRotate) {
                static_assert(!kRotate || BITS == 1, "one 16-byte piece per row");
#pragma unroll
                for (int rd = 0; rd < REGL; ++rd) {
                    token_logits(pass_c, rd, tid + rd * kNT, kc[rd % L::KR]);
                    if (rd + L::KR < REGL) kc[rd % L::KR][0] = ckp[min(tid + (rd + L::KR) * kNT, last_uk)];
                    if constexpr (!MINMAX_ONLY) {
                        if (rd < kPF - kVEarly) request_v(kVEarly + rd);   // the rest of the first packed V block
                    }
                }
                if constexpr (kLateMM) {
                    const int t0w = __builtin_amdgcn_readfirstlane(tid);   // the wave's first token of round 0
#pragma unroll
                    for (int rd = 0; rd < REGL; rd += 2) {
                        if (rd + 1 < REGL && t0w + (rd + 1) * kNT < n) {
#pragma unroll
                            for (int h = 0; h < NH; ++h) {
                                mn[h] = fminf(mn[h], fminf(lg[rd].v[h], lg[rd + 1].v[h]));
                                mx[h] = fmaxf(mx[h], fmaxf(lg[rd].v[h], lg[rd + 1].v[h]));
                            }
                        } else if (t0w + rd * kNT < n) {
#pragma unroll
                            for (int h = 0; h < NH; ++h) { mn[h] = fminf(mn[h], lg[rd].v[h]); mx[h] = fmaxf(mx[h], lg[rd].v[h]); }
                        }
                    }
                }
                return;
            }
            // first batch: rows already in registers; each consumed round of the last pass frees
            // registers that take the first block of packed V rows
            // (written out round by round with constant indices so vc stays in registers)
#define CQ_K_ROUND(R)                                                                         \
            if constexpr (L::KR > (R)) {                                                      \
                token_logits(pass_c, (R), tid + (R) * kNT, kc[(R)] + kP0);                    \
                if constexpr (!MINMAX_ONLY && P + 1 == L::KPASS) {                            \
                    if constexpr (kVEarly + (R) * BITS < kPF) request_v(kVEarly + (R) * BITS);    \
                    if constexpr (BITS == 2 && kVEarly + (R) * BITS + 1 < kPF) request_v(kVEarly + (R) * BITS + 1); \
                }                                                                             \
            }
            CQ_K_ROUND(0)
            CQ_K_ROUND(1)
            CQ_K_ROUND(2)
            CQ_K_ROUND(3)
#undef CQ_K_ROUND
            static_assert(L::KR <= 4, "rounds are written out up to 4");
            uint4 kx[L::KR][L::PCS];   // rows beyond the first batch: this pass's pieces only
            if constexpr (kKeepRows) {
                // whole rows, requested in the first pass and kept for the later ones
#pragma unroll
                for (int ob = 1; ob < (REGL + L::KR - 1) / L::KR; ++ob) {
                    const int tb = ob * kNT * L::KR;
                    if (tb < n) {
                        if constexpr (P == 0) {
#pragma unroll
                            for (int r = 0; r < L::KR; ++r) {
                                const int tt = min(tb + tid + r * kNT, n - 1);
#pragma unroll
                                for (int i = 0; i < BITS; ++i)
                                    if (ob * L::KR + r < REGL) kall[ob * L::KR + r][i] = ckp[static_cast<int64_t>(tt) * BITS + i];
                            }
                        }
#pragma unroll
                        for (int r = 0; r < L::KR; ++r)
                            if (ob * L::KR + r < REGL)
                                token_logits(pass_c, ob * L::KR + r, tb + tid + r * kNT, kall[ob * L::KR + r] + kP0);
                    }
                }
            } else if constexpr (REGL > 0) {
                // batches written out, so that the logits' registers are indexed by constants
#pragma unroll
                for (int ob = 1; ob < (REGL + L::KR - 1) / L::KR; ++ob) {
                    const int tb = ob * kNT * L::KR;
                    if (tb < n) {
#pragma unroll
                        for (int r = 0; r < L::KR; ++r) {
                            const int tt = min(tb + tid + r * kNT, n - 1);
                            if constexpr (kKeepHalf) {
                                static_assert(!kKeepHalf || L::PCS == 1, "a pass looks at one piece of the row");
                                if constexpr (P == 0) {
                                    kx[r][0] = ckp[static_cast<int64_t>(tt) * BITS];
                                    if (ob * L::KR + r < REGL) khalf[ob * L::KR + r] = ckp[static_cast<int64_t>(tt) * BITS + 1];
                                } else {
                                    if (ob * L::KR + r < REGL) kx[r][0] = khalf[ob * L::KR + r];
                                }
                                continue;
                            }
#pragma unroll
                            for (int i = 0; i < L::PCS; ++i) kx[r][i] = ckp[static_cast<int64_t>(tt) * BITS + kP0 + i];
                        }
#pragma unroll
                        for (int r = 0; r < L::KR; ++r)
                            if (ob * L::KR + r < REGL) token_logits(pass_c, ob * L::KR + r, tb + tid + r * kNT, kx[r]);
                    }
                }
            } else {
                for (int tb = kNT * L::KR; tb < n; tb += kNT * L::KR) {
#pragma unroll
                    for (int r = 0; r < L::KR; ++r) {
                        const int tt = min(tb + tid + r * kNT, n - 1);
#pragma unroll
                        for (int i = 0; i < L::PCS; ++i) kx[r][i] = ckp[static_cast<int64_t>(tt) * BITS + kP0 + i];
                    }
#pragma unroll
                    for (int r = 0; r < L::KR; ++r) token_logits(pass_c, 0, tb + tid + r * kNT, kx[r]);
                }
            }
        };
        k_pass(std::integral_constant<int, 0>{});
        if constexpr (L::KPASS >= 2) {
            __syncthreads();   // every wave is done with the previous pass's table
            k_pass(std::integral_constant<int, 1>{});
        }
        if constexpr (L::KPASS == 4) {
            __syncthreads();
            k_pass(std::integral_constant<int, 2>{});
            __syncthreads();
            k_pass(std::integral_constant<int, 3>{});
        }
    }
    CQ_PHASE(3);   // K table and look-ups
    phase_priority(std::integral_constant<int, 2>{});
    if (k_rows) {   // one reduction for both: max of (-min, max)
        float mm2[2 * HPB];
#pragma unroll
        for (int h = 0; h < HPB; ++h) { mm2[h] = -mn[h]; mm2[HPB + h] = mx[h]; }
        block_max<2 * HPB, kNW>(mm2, red);
#pragma unroll
        for (int h = 0; h < HPB; ++h) { mn[h] = -mm2[h]; mx[h] = mm2[HPB + h]; }
    }

    CQ_PHASE(4);   // block min / max
    if constexpr (MINMAX_ONLY) {
#pragma unroll
        for (int h = 0; h < HPB; ++h) {
            if (n > 0 && tid == h && h < nh) {
                float* o = g.mm + ((static_cast<int64_t>(b) * g.Hq + hq0 + h) * g.nsplit + split) * 2;
                o[0] = mn[h];
                o[1] = mx[h];
            }
        }
        if (split == 0 && tid == 0) g.cnt[unit] = 0;   // the main launch counts the unit's partials from 0
        return;
    } else {
        float m_img[HPB];
#pragma unroll
        for (int h = 0; h < HPB; ++h) m_img[h] = -INFINITY;
        float o_img = 0.f;  // thread (h, d) = (tid / kD, tid % kD) for tid < HPB*kD

        if constexpr (CHUNKED) {
            // One launch: this chunk's min / max go out now (write-through stores, waited for, then the arrival
            // count); the other chunks' are collected further down, after the staging of the first V block.
            if (g.fused && k_rows && tid == 0) {
                unsigned long long* o = g.rec + ((unit * HPB) * g.nsplit + split) * 2;
                const unsigned long long tag = static_cast<unsigned long long>(g.epoch) << 32;
#pragma unroll
                for (int h = 0; h < HPB; ++h) {
                    __hip_atomic_store(o + h * g.nsplit * 2, tag | __float_as_uint(mn[h]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(o + h * g.nsplit * 2 + 1, tag | __float_as_uint(mx[h]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }

        if (n > 0) {
            // The K table is dead: stage the first block of packed V rows in its place
            // (ordered by the barrier of block_max).  Layout: [unit of TPW tokens]
            // [byte column][token], so the 4 bytes that the 4 tokens of a group have in one
            // column form one dword.  A quad of lanes holds a group (tokens are
            // lane-consecutive): per dword of its 16-byte piece the quad transposes a 4 x 4 byte
            // block in two exchange steps (lane ^ 1, then lane ^ 2), a byte permute after each,
            // and lane i ends up with the 4 tokens' bytes of column 4 q + i.
            unsigned char* vst = regA + L::WTAB;
            const int qi = lane & 3;
            // step 1, operands (partner, own): bytes qi and qi ^ 2 of the even and of the odd lane
            const uint32_t b0 = static_cast<uint32_t>(qi), b2 = static_cast<uint32_t>(qi ^ 2);
            const uint32_t sel1 = (qi & 1) ? ((4 + b0) | (b0 << 8) | ((4 + b2) << 16) | (b2 << 24))
                                           : (b0 | ((4 + b0) << 8) | (b2 << 16) | ((4 + b2) << 24));
            // step 2, operands (partner, own): own low half and the partner's high half, pair 0 first
            const uint32_t sel2 = (qi & 2) ? 0x01000706u : 0x07060100u;
            auto stage_piece = [&](U4 c, int tok, int piece, bool write) {
                const uint32_t w[4] = {c.x, c.y, c.z, c.w};
                const int base = ((tok / L::TPW) * NB + 16 * piece + qi) * L::TPW + ((tok % L::TPW) & ~3);
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t p1 = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(w[q]), 0xB1, 0xf, 0xf, true));
                    const uint32_t a = __builtin_amdgcn_perm(p1, w[q], sel1);
                    const uint32_t p2 = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(a), 0x4E, 0xf, 0xf, true));
                    const uint32_t t4 = __builtin_amdgcn_perm(p2, a, sel2);
                    if (write) *reinterpret_cast<uint32_t*>(vst + base + 4 * q * L::TPW) = t4;
                }
            };
            {
                const int vn0 = min(L::VSUB, npad);
#pragma unroll
                for (int r = 0; r < kPF; ++r) {
                    const int tok = tid + (r / BITS) * kNT;
                    stage_piece(vc[r], tok, r % BITS, tok < vn0);
                }
            }
            // The registers of a staged block take the next block's rows (clamped addresses when there is none):
            // the block is in flight while the current one is multiplied, instead of being asked for behind a
            // barrier when the loop gets there.  (The first residual tile requested here as well measured slower.)
            constexpr bool kVAhead = L::INA;
            auto request_v_block = [&](int vs0) {
#pragma unroll
                for (int r = 0; r < kPF; ++r) vc[r] = cvp4[min((vs0 + tid + (r / BITS) * kNT) * BITS + r % BITS, last_u)];
            };

            CQ_PHASE(5);   // staging of the first packed V block
            // ---- phase 4: calibration + exp ---------------------------------------------
            if constexpr (CHUNKED) {
                if (g.fused) {
                    // Wait until every chunk of the unit has published: the first wave polls the records, lane s
                    // those of chunk s, a bounded number of times (workgroups that are not all resident together -
                    // a smaller device than planned for - must not spin for ever; giving up ends this workgroup
                    // without a result and tells the host), folds them and leaves the unit's min / max in LDS.
                    float* fold = red + 4 * HPB;           // 2 * HPB floats, then whether the wait succeeded
                    int* flag = reinterpret_cast<int*>(fold + 2 * HPB);
                    if (wv == 0) {
                        const unsigned long long* pr = g.rec + ((unit * HPB) * g.nsplit + min(lane, g.nsplit - 1)) * 2;
                        float mm2[2 * HPB];
                        bool ok = false;
                        for (int it = 0; it < g.spin_limit && !ok; ++it) {
                            bool valid = true;
#pragma unroll
                            for (int h = 0; h < HPB; ++h) {
                                const unsigned long long lo = __hip_atomic_load(pr + h * g.nsplit * 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                const unsigned long long hi = __hip_atomic_load(pr + h * g.nsplit * 2 + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                valid = valid && static_cast<uint32_t>(lo >> 32) == g.epoch && static_cast<uint32_t>(hi >> 32) == g.epoch;
                                mm2[h] = -__uint_as_float(static_cast<uint32_t>(lo));
                                mm2[HPB + h] = __uint_as_float(static_cast<uint32_t>(hi));
                            }
                            ok = __builtin_amdgcn_ballot_w64(!valid) == 0;
                            if (!ok) __builtin_amdgcn_s_sleep(2);
                        }
                        wave_reduce_n<2 * HPB>(mm2, OpMax(), -INFINITY);
                        if (lane == 0) {
#pragma unroll
                            for (int i = 0; i < 2 * HPB; ++i) fold[i] = mm2[i];
                            *flag = ok ? 1 : 0;
                            if (!ok && g.status) __hip_atomic_store(g.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                        }
                    }
                    __syncthreads();
                    if (!*flag) {
                        // Given up: no result from this workgroup, but it is still counted, so that the unit's
                        // last workgroup - this one or another - leaves the records and the counter empty and a
                        // replay of this very launch (same epoch) does not take this launch's records for its own.
                        int* last = reinterpret_cast<int*>(red);
                        if (tid == 0) *last = arrive<__HIP_MEMORY_SCOPE_AGENT>(g.done64 + unit, g.epoch) == static_cast<uint32_t>(g.nx);
                        __syncthreads();
                        if (*last) clear_handover<HPB, kNT>(g, unit, tid);
                        return;
                    }
#pragma unroll
                    for (int h = 0; h < HPB; ++h) { mn[h] = -fold[h]; mx[h] = fold[HPB + h]; }
                } else {
                // one fold for both: max of (-min, max) over the chunks
                float mm2[2 * HPB];
#pragma unroll
                for (int h = 0; h < HPB; ++h) {
                    mm2[h] = -mraw[h].lo;
                    mm2[HPB + h] = mraw[h].hi;
                    const MinMax* p = reinterpret_cast<const MinMax*>(g.mm) +
                                      (static_cast<int64_t>(b) * g.Hq + hq0 + min(h, nh - 1)) * g.nsplit;
                    for (int s = lane + 64; s < g.nsplit; s += 64) {   // (more than 64 chunks)
                        const MinMax v = p[s];
                        mm2[h] = fmaxf(mm2[h], -v.lo);
                        mm2[HPB + h] = fmaxf(mm2[HPB + h], v.hi);
                    }
                }
                wave_reduce_n<2 * HPB>(mm2, OpMax(), -INFINITY);
#pragma unroll
                for (int h = 0; h < HPB; ++h) { mn[h] = -mm2[h]; mx[h] = mm2[HPB + h]; }
                }
            }
            float slope[HPB], tmin[HPB];
#pragma unroll
            for (int h = 0; h < HPB; ++h) {
                if (g.calib) {
                    const float tgt_max = mx[h] + g.off_max;
                    tmin[h] = mn[h] + g.off_min;
                    // (the hardware reciprocal, one unit in the last place: far inside the tolerance of the map)
                    slope[h] = (tgt_max - tmin[h]) * __builtin_amdgcn_rcpf(mx[h] - mn[h] + 1e-8f);
                } else {
                    tmin[h] = mn[h];
                    slope[h] = 1.0f;
                }
            }
            if (EXTRAS && g.mask) {
                const float* mk = g.mask + b * g.mask_sb + g.S + t0;
                float lm[HPB];
#pragma unroll
                for (int h = 0; h < HPB; ++h) lm[h] = -INFINITY;
                for_my_tokens(n, [&](int rd, int tt) {
                    V w = load_logits(rd, tt);
                    const float mv = mk[tt];
#pragma unroll
                    for (int h = 0; h < HPB; ++h) {
                        w.v[h] = (w.v[h] - mn[h]) * slope[h] + tmin[h] + mv;
                        lm[h] = fmaxf(lm[h], w.v[h]);
                    }
                    store_logits(rd, tt, w);
                });
                block_max<HPB, kNW>(lm, red + 2 * HPB);   // words of its own
#pragma unroll
                for (int h = 0; h < HPB; ++h) { m_img[h] = lm[h]; slope[h] = 1.0f; tmin[h] = 0.f; mn[h] = 0.f; }
            } else {
#pragma unroll
                for (int h = 0; h < HPB; ++h) m_img[h] = fmaxf(tmin[h], (mx[h] - mn[h]) * slope[h] + tmin[h]);
            }
            float ls[HPB];
#pragma unroll
            for (int h = 0; h < HPB; ++h) ls[h] = 0.f;
            // e = exp(x - M) with x = (w - mn) * slope + tmin, as exp2((w - mn) * ea + ec)
            float ea[HPB], ec[HPB];
#pragma unroll
            for (int h = 0; h < HPB; ++h) {
                const bool dead = (m_img[h] == -INFINITY);   // every position masked out
                ea[h] = dead ? 0.f : slope[h] * kLog2e;
                ec[h] = dead ? -INFINITY : (tmin[h] - m_img[h]) * kLog2e;
            }
            using HWv = Words<L::HW>;
            // per-token value statistics (VTOK): (T, NGRP) scales and minima of this kv-head
            const uint16_t* tsc = static_cast<const uint16_t*>(g.vs) + (bh * g.T + t0) * L::NGRP;
            const uint16_t* tmn = static_cast<const uint16_t*>(g.vz) + (bh * g.T + t0) * L::NGRP;
            float cma[VTOK ? L::NGRP * HPB : 1];   // sum_t e[t][h] * minimum[t][group], kept [group][head]
#pragma unroll
            for (int i = 0; i < (VTOK ? L::NGRP * HPB : 1); ++i) cma[i] = 0.f;
            // With a slope of ordinary size the subtraction folds into the constant: exp2(w * ea + (ec - mn * ea)), one
            // FMA per logit.  A degenerate logit range makes the slope ~1e8, and only the exact zero of (w - mn)
            // keeps the product finite: those units take the two-step form.
            float ec2[HPB];
            bool plain = true;
#pragma unroll
            for (int h = 0; h < HPB; ++h) {
                ec2[h] = ec[h] - mn[h] * ea[h];
                if (h < NH) plain = plain && fabsf(ea[h]) <= 4.0f;
            }
            auto exp_tokens = [&](auto fused_c) {
            constexpr bool kFused = decltype(fused_c)::value;
            for_my_tokens(npad, [&](int rd, int tt) {
                float e[4] = {0.f, 0.f, 0.f, 0.f};
                uint32_t sc2[2] = {0u, 0u};   // the token's group scales as fp16
                if (tt < n) {
                    const V w = load_logits(rd, tt);
#pragma unroll
                    for (int h = 0; h < NH; ++h) {
                        if constexpr (kFused) e[h] = __builtin_amdgcn_exp2f(__builtin_fmaf(w.v[h], ea[h], ec2[h]));
                        else e[h] = __builtin_amdgcn_exp2f((w.v[h] - mn[h]) * ea[h] + ec[h]);
                        ls[h] += e[h];
                    }
                    if constexpr (VTOK) {
                        const uint2 sr = *reinterpret_cast<const uint2*>(tsc + tt * L::NGRP);
                        const uint2 mr = *reinterpret_cast<const uint2*>(tmn + tt * L::NGRP);
                        sc2[0] = pack_f16(Cvt<DT>::lo(sr.x), Cvt<DT>::hi(sr.x));
                        sc2[1] = pack_f16(Cvt<DT>::lo(sr.y), Cvt<DT>::hi(sr.y));
                        const float mg[4] = {Cvt<DT>::lo(mr.x), Cvt<DT>::hi(mr.x), Cvt<DT>::lo(mr.y), Cvt<DT>::hi(mr.y)};
#pragma unroll
                        for (int gi = 0; gi < L::NGRP; ++gi)
#pragma unroll
                            for (int h = 0; h < HPB; ++h) cma[gi * HPB + h] += e[h] * mg[gi];
                    }
                }
                // e as packed fp16 in the first bytes of the token's slot (read by the V tables)
                HWv hw;
                hw.w[0] = pack_f16(e[0], e[1]);
                if constexpr (L::HW == 2) hw.w[1] = pack_f16(e[2], e[3]);
                *reinterpret_cast<HWv*>(slot(tt)) = hw;
                if constexpr (VTOK) *reinterpret_cast<uint2*>(slot(tt) + 8) = make_uint2(sc2[0], sc2[1]);
            });
            };
            if (plain) exp_tokens(std::true_type{});
            else exp_tokens(std::false_type{});
            // The sums of e (and of e * minimum) are only needed at the very end: each thread
            // keeps its partial through the packed-V phase and the fold rides on that phase's
            // closing barriers.
            __syncthreads();   // publishes e and vst
            CQ_PHASE(6);   // calibration and exponentials
            // (requested here, not right after the staging: the logits' registers are free now)
            if constexpr (kVAhead) request_v_block(L::VSUB);

            // ---- phase 5: packed V ----------------------------------------------------------
            // lane = (byte column j, slice c of its 8 bit lanes); a wave pass covers TPW tokens
            unsigned char* wtab = regA + wv * (L::NGRP * L::GPW * 16 * L::ESZH);   // [channel group][token group][16]
            const int j = lane / L::GPW, cs = lane % L::GPW;
            const int wvu = __builtin_amdgcn_readfirstlane(wv);
            const int bg = lane >> 4, be = lane & 15;   // table build: group, entry
            f16x2_t bsel[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const _Float16 f = static_cast<_Float16>(static_cast<float>((be >> i) & 1));
                bsel[i] = f16x2_t{f, f};
            }
            float acc[L::MPL][HPB];
#pragma unroll
            for (int m = 0; m < L::MPL; ++m)
#pragma unroll
                for (int h = 0; h < HPB; ++h) acc[m][h] = 0.f;
            const float one = g.one;
            // Bit lane m of a byte is bit 7 - m; table offset = sum_i bit(token i) * ESZH * 2^i.
            // The lane's MPL bit lanes sit in one nibble: the dword is shifted by 4 * (m < 4) once,
            // each lane masks its bit in place (value 2^s per byte) and the dot-product
            // multiplier carries the 2^-s: ESZH * 2^i >> s stays integral for s <= 3, ESZH = 8;
            // with 4-byte entries the multiplier is kept whole and s = 0 (bit moved down first).
            constexpr bool kInPlace = (L::ESZH == 8);
            const uint32_t nib_shift = (cs * L::MPL < 4) ? 4u : 0u;
            uint32_t bmask[L::MPL], bmult[L::MPL], bshr[L::MPL];
#pragma unroll
            for (int m = 0; m < L::MPL; ++m) {
                const uint32_t sft = 3 - ((cs * L::MPL + m) & 3);   // bit position inside the nibble
                bmask[m] = kInPlace ? (0x01010101u << sft) : 0x01010101u;
                bmult[m] = kInPlace ? ((L::ESZH * 0x08040201u) >> sft) & 0x7f7f7f7fu : L::ESZH * 0x08040201u;
                bshr[m] = kInPlace ? 0u : sft;
            }
            using WG = Words<L::GPW>;   // the GPW dwords of one (unit, column)
            // channel group of the lane's byte column (32 channels = 4*BITS columns): lane / 16 for both widths
            const int cgrp = VTOK ? (lane >> 4) : 0;
            // absolute LDS address of the wave's tables (the dot product's addend)
            const uint32_t wtab_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
                (__attribute__((address_space(3))) unsigned char*)wtab));

            phase_priority(std::integral_constant<int, 3>{});
            for (int vs0 = 0; vs0 < npad; vs0 += L::VSUB) {
                const int vn = min(L::VSUB, npad - vs0);
                if (vs0 > 0) {
                    __syncthreads();  // previous block consumed
                    if constexpr (!kVAhead) request_v_block(vs0);
#pragma unroll
                    for (int r = 0; r < kPF; ++r) {
                        const int tok = tid + (r / BITS) * kNT;
                        stage_piece(vc[r], tok, r % BITS, tok < vn);
                    }
                    if constexpr (kVAhead) request_v_block(vs0 + L::VSUB);
                    __syncthreads();
                }
                // One pass over the TPW tokens of unit u: the sum of the entries each of the lane's bit lanes picks,
                // as packed fp16 (GPW entries of at most 4 terms each, added pairwise).
                struct PreV { HWv e[4]; WG cw; };
                auto load_pre = [&](int u, PreV& p) {
                    const int tl = u * L::TPW;
#pragma unroll
                    for (int i = 0; i < 4; ++i) p.e[i] = *reinterpret_cast<const HWv*>(slot(vs0 + tl + 4 * bg + i));
                    p.cw = *reinterpret_cast<const WG*>(vst + (u * NB + j) * L::TPW);
                };
                // A pass in three steps, so that two passes can be woven together: the table of the second is built and
                // written while the look-ups of the first are in flight (the LDS executes a wave's instructions in
                // order: the second table's write lands after the first pass's reads).
                auto v_build = [&](int u, const PreV& pre) {
                    const int tl = u * L::TPW;        // token offset inside the block
                    (void)tl;
                    if (bg < L::GPW) {
                        f16x2_t val[L::NGRP][L::HW];
#pragma unroll
                        for (int gi = 0; gi < L::NGRP; ++gi)
#pragma unroll
                            for (int k = 0; k < L::HW; ++k) val[gi][k] = f16x2_t{0, 0};
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const unsigned char* sl = slot(vs0 + tl + 4 * bg + i);
                            const HWv e = VTOK ? *reinterpret_cast<const HWv*>(sl) : pre.e[i];
                            if constexpr (VTOK) {
                                const uint2 sc = *reinterpret_cast<const uint2*>(sl + 8);
                                const f16x2_t s01 = __builtin_bit_cast(f16x2_t, sc.x), s23 = __builtin_bit_cast(f16x2_t, sc.y);
                                const _Float16 sg[4] = {s01.x, s01.y, s23.x, s23.y};
#pragma unroll
                                for (int gi = 0; gi < L::NGRP; ++gi) {
                                    const f16x2_t w2 = bsel[i] * f16x2_t{sg[gi], sg[gi]};
#pragma unroll
                                    for (int k = 0; k < L::HW; ++k) val[gi][k] += __builtin_bit_cast(f16x2_t, e.w[k]) * w2;
                                }
                            } else {
#pragma unroll
                                for (int k = 0; k < L::HW; ++k) val[0][k] += __builtin_bit_cast(f16x2_t, e.w[k]) * bsel[i];
                            }
                        }
#pragma unroll
                        for (int gi = 0; gi < L::NGRP; ++gi) {
                            HWv o;
#pragma unroll
                            for (int k = 0; k < L::HW; ++k) o.w[k] = __builtin_bit_cast(uint32_t, val[gi][k]);
                            reinterpret_cast<HWv*>(wtab)[(gi * L::GPW + bg) * 16 + be] = o;
                        }
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                };
                auto v_lookups = [&](const WG& cw, f16x2_t (&pk)[L::MPL][L::GPW][L::HW]) {
#pragma unroll
                    for (int gq = 0; gq < L::GPW; ++gq) {
                        const uint32_t tbase = wtab_addr + static_cast<uint32_t>((cgrp * L::GPW + gq) * 16 * L::ESZH);
                        const uint32_t wsh = cw.w[gq] >> nib_shift;
#pragma unroll
                        for (int m = 0; m < L::MPL; ++m) {
                            const uint32_t bits = (kInPlace ? wsh : (wsh >> bshr[m])) & bmask[m];
                            const uint32_t off = __builtin_amdgcn_udot4(bits, bmult[m], tbase, false);
                            const HWv e = lds_words<L::HW>(off);
#pragma unroll
                            for (int k = 0; k < L::HW; ++k) pk[m][gq][k] = __builtin_bit_cast(f16x2_t, e.w[k]);
                        }
                    }
                };
                auto v_reduce = [&](f16x2_t (&pk)[L::MPL][L::GPW][L::HW], f16x2_t (&sum)[L::MPL][L::HW]) {
#pragma unroll
                    for (int m = 0; m < L::MPL; ++m) {
#pragma unroll
                        for (int st = 1; st < L::GPW; st *= 2)
#pragma unroll
                            for (int gq = 0; gq + st < L::GPW; gq += 2 * st)
#pragma unroll
                                for (int k = 0; k < L::HW; ++k) pk[m][gq][k] += pk[m][gq + st][k];
#pragma unroll
                        for (int k = 0; k < L::HW; ++k) sum[m][k] = pk[m][0][k];
                    }
                };
                auto v_pass = [&](int u, f16x2_t (&sum)[L::MPL][L::HW], const PreV& pre, auto&& after_lookups) {
                    f16x2_t pk[L::MPL][L::GPW][L::HW];
                    v_build(u, pre);
                    v_lookups(pre.cw, pk);
                    after_lookups();
                    v_reduce(pk, sum);
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                };
                // one mixed-precision FMA per head moves a packed sum into the fp32 accumulators
                auto v_flush = [&](const f16x2_t (&sum)[L::MPL][L::HW]) {
#pragma unroll
                    for (int m = 0; m < L::MPL; ++m)
#pragma unroll
                        for (int h = 0; h < NH; ++h) {
                            const f16x2_t pr = sum[m][h >> 1];
                            const _Float16 hv = (h & 1) ? pr.y : pr.x;
                            acc[m][h] = __builtin_fmaf(static_cast<float>(hv), one, acc[m][h]);
                        }
                };
                int u = wvu;   // wave-uniform loop control
                // the slot entries and code words of a pass are read while the pass before it waits for its look-ups
                PreV cur, nxt;
                if (u * L::TPW < vn) load_pre(u, cur);
                {
                    // two passes per fp32 accumulation: the sums of 2 * TPW tokens meet as packed fp16 first
                    for (; (u + kNW) * L::TPW < vn; u += 2 * kNW) {
                        f16x2_t s0[L::MPL][L::HW], s1[L::MPL][L::HW];
                        f16x2_t pk0[L::MPL][L::GPW][L::HW], pk1[L::MPL][L::GPW][L::HW];
                        v_build(u, cur);
                        v_lookups(cur.cw, pk0);
                        load_pre(u + kNW, nxt);
                        v_build(u + kNW, nxt);           // (its table write queues behind the look-ups above)
                        v_lookups(nxt.cw, pk1);
                        if ((u + 2 * kNW) * L::TPW < vn) load_pre(u + 2 * kNW, cur);
                        v_reduce(pk0, s0);
                        v_reduce(pk1, s1);
                        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                        __builtin_amdgcn_wave_barrier();
#pragma unroll
                        for (int m = 0; m < L::MPL; ++m)
#pragma unroll
                            for (int k = 0; k < L::HW; ++k) s0[m][k] += s1[m][k];
                        v_flush(s0);
                    }
                }
                for (; u * L::TPW < vn; u += kNW) {
                    f16x2_t s0[L::MPL][L::HW];
                    v_pass(u, s0, cur, [&]() { if ((u + kNW) * L::TPW < vn) load_pre(u + kNW, cur); });
                    v_flush(s0);
                }
            }
            CQ_PHASE(7);   // packed-V loop (tables, look-ups, sums; staging of the later blocks)
            phase_priority(std::integral_constant<int, 4>{});
            load_res_k(0, rk);   // first residual tile's K rows: in flight during the fold below
            // per-wave partial sums of e (and of e * minimum), folded by the output threads below
            constexpr int kSums = VTOK ? (L::NGRP + 1) * HPB : HPB;
            wave_reduce_n<HPB>(ls, OpSum(), 0.f);
            if constexpr (VTOK) {
#pragma unroll
                for (int gi = 0; gi < L::NGRP; ++gi) wave_reduce_n<HPB>(cma + gi * HPB, OpSum(), 0.f);
            }
            if (lane == 0) {
#pragma unroll
                for (int h = 0; h < HPB; ++h) red[wv * kSums + h] = ls[h];
                if constexpr (VTOK) {
#pragma unroll
                    for (int i = 0; i < L::NGRP * HPB; ++i) red[wv * kSums + HPB + i] = cma[i];
                }
            }
            __syncthreads();
            // head-major, so that the fold below reads consecutive words with consecutive lanes
            float* redv = reinterpret_cast<float*>(regA);  // [wave][head][bit lane]
#pragma unroll
            for (int h = 0; h < HPB; ++h) {
                Vec<L::MPL> a4;
#pragma unroll
                for (int m = 0; m < L::MPL; ++m) a4.v[m] = acc[m][h];
                *reinterpret_cast<Vec<L::MPL>*>(redv + (wv * HPB + h) * L::PC + j * 8 + cs * L::MPL) = a4;
            }
            __syncthreads();
            if (tid < HPB * kD) {
                const int h = tid / kD, d = tid % kD;
                float a = 0.f;
                // bit lanes of channel d.  Per-channel codes: first channel of a byte in its top
                // bits; per-token codes: first channel in the lowest bits.
                const int per = 8 / BITS;                       // channels per byte
                const int cb = d / per * 8, c = d % per;
                const int lane_hi = VTOK ? cb + 8 - BITS * (c + 1) : cb + BITS * c;   // bit lane of the code's top bit
                if constexpr (BITS == 1) {
#pragma unroll
                    for (int w = 0; w < kNW; ++w) a += redv[(w * HPB + h) * L::PC + lane_hi];
                } else {
#pragma unroll
                    for (int w = 0; w < kNW; ++w)
                        a += 2.0f * redv[(w * HPB + h) * L::PC + lane_hi] + redv[(w * HPB + h) * L::PC + lane_hi + 1];
                }
                float lh = 0.f;   // sum of e of this thread's head
#pragma unroll
                for (int w = 0; w < kNW; ++w) lh += red[w * kSums + h];
                if constexpr (VTOK) {
                    float cm = 0.f;   // sum_t e * minimum of the channel's group
#pragma unroll
                    for (int w = 0; w < kNW; ++w) cm += red[w * kSums + HPB + (d >> 5) * HPB + h];
                    o_img = a + cm;
                } else {
                    const float s = fx[L::F_VSZ + d];
                    const float z = fx[L::F_VSZ + kD + d];
                    o_img = s * (a - z * lh);
                }
                if (d == 0) stat[4 * HPB + h] = lh;
            }
            __syncthreads();
        }

        if (n == 0) load_res_k(0, rk);
        CQ_PHASE(8);   // fold of the packed part
        // ---- phase 6: full-precision residual rows, online softmax.  Runs last: its first
        // tile is requested when the packed-V phase ends and arrives during that phase's fold.
#pragma unroll
        for (int h = 0; h < HPB; ++h) {
            if (tid == h) {
                stat[HPB + h] = -INFINITY;
                stat[2 * HPB + h] = 0.f;
            }
        }
        if (do_res) {
            float m_run = -INFINITY, l_run = 0.f;
            float* sres = fx + L::F_SRES;
            float* pres = fx + L::F_PRES;
            // raw 16-bit q, [head][kD], read per head as two 16-byte LDS loads
            const uint4* q128 = reinterpret_cast<const uint4*>(fx + L::F_QRAW);
            float accv[2][HPB];   // the lane's channel pair
#pragma unroll
            for (int k = 0; k < 2; ++k)
#pragma unroll
                for (int h = 0; h < HPB; ++h) accv[k][h] = 0.f;
            const float* mk = (EXTRAS && g.mask) ? g.mask + b * g.mask_sb : nullptr;

            for (int r0 = 0; r0 < R; r0 += kResTile) {
                const bool more = r0 + kResTile < R;
                const int r = r0 + krow;
                load_res_v(r0, rv);   // the tile's value words: in flight while its logits and weights are worked out
                float dot[HPB];
#pragma unroll
                for (int h = NH; h < HPB; ++h) dot[h] = 0.f;
#pragma unroll
                for (int h = 0; h < NH; ++h) {
                    float a = 0.f;
#pragma unroll
                    for (int i = 0; i < NKP; ++i) {
                        const uint4 qa = q128[h * (kD / 8) + i * LPR + lq];
                        a = dot2<DT>(qa.x, rk[i].x, a); a = dot2<DT>(qa.y, rk[i].y, a);
                        a = dot2<DT>(qa.z, rk[i].z, a); a = dot2<DT>(qa.w, rk[i].w, a);
                    }
                    dot[h] = (LPR == 4 ? quad_reduce(a, OpSum(), 0.f) : oct_reduce(a, OpSum(), 0.f)) * inv_sqrt_d;
                    // one head's q pieces at a time: all of them side by side would not fit the registers
                    if constexpr (NKP > 2) __builtin_amdgcn_sched_barrier(0);
                }
                if (more) load_res_k(r0 + kResTile, rk);   // next tile's K slice, in place
                if (lq == 0) {
                    float mv = 0.f;
                    if (mk && r < R) mv = mk[r < g.S ? r : g.T + r];
#pragma unroll
                    for (int h = 0; h < HPB; ++h) sres[krow * HPB + h] = (r < R) ? dot[h] + mv : -INFINITY;
                }
                __syncthreads();
                if (wv < NH) {   // wave h keeps the running softmax state of head h
                    const int h = wv;
                    constexpr int kRL = kResTile / kWave;   // tile rows per lane
                    float sv[kRL], smax = -INFINITY;
#pragma unroll
                    for (int i = 0; i < kRL; ++i) {
                        sv[i] = sres[(lane + i * kWave) * HPB + h];
                        smax = fmaxf(smax, sv[i]);
                    }
                    const float mnew = fmaxf(m_run, wave_max(smax));
                    const bool dead = (mnew == -INFINITY);
                    float psum = 0.f;
#pragma unroll
                    for (int i = 0; i < kRL; ++i) {
                        const float pi = dead ? 0.f : __expf(sv[i] - mnew);
                        pres[(lane + i * kWave) * HPB + h] = pi;
                        psum += pi;
                    }
                    const float al = dead ? 1.0f : __expf(m_run - mnew);
                    l_run = l_run * al + wave_sum(psum);
                    m_run = mnew;
                    if (lane == 0) { stat[h] = al; stat[HPB + h] = m_run; stat[2 * HPB + h] = l_run; }
                }
                __syncthreads();
                if (r0 > 0) {
#pragma unroll
                    for (int h = 0; h < NH; ++h) {
                        const float al = stat[h];
                        accv[0][h] *= al;
                        accv[1][h] *= al;
                    }
                }
#pragma unroll
                for (int i = 0; i < RPW; ++i) {
                    const float f0 = Cvt<DT>::lo(rv[i]), f1 = Cvt<DT>::hi(rv[i]);
                    const V p = reinterpret_cast<const V*>(pres)[wvr * RPW + i];   // the row's weights (0 past R), one address per wave
#pragma unroll
                    for (int h = 0; h < NH; ++h) {
                        accv[0][h] = __builtin_fmaf(p.v[h], f0, accv[0][h]);
                        accv[1][h] = __builtin_fmaf(p.v[h], f1, accv[1][h]);
                    }
                }
            }
            __syncthreads();
            float* red2 = reinterpret_cast<float*>(regA);  // [wave][head][kD]: the fold reads consecutive words
#pragma unroll
            for (int h = 0; h < HPB; ++h) {
                Vec<2> a2;
                a2.v[0] = accv[0][h]; a2.v[1] = accv[1][h];
                *reinterpret_cast<Vec<2>*>(red2 + (wv * HPB + h) * kD + 2 * lane) = a2;
            }
            __syncthreads();
            if (tid < HPB * kD) {
                const int h = tid / kD, d = tid % kD;
#pragma unroll
                for (int w = 0; w < kNW; ++w) o_res += red2[(w * HPB + h) * kD + d];
            }
        }

#pragma unroll
        for (int h = 0; h < HPB; ++h) {
            if (tid == h) {
                stat[3 * HPB + h] = m_img[h];
                if (n == 0) stat[4 * HPB + h] = 0.f;
            }
        }
        CQ_PHASE(9);   // residual window
        // ---- phase 7: merge / write ---------------------------------------------------------
        __syncthreads();
        if (tid < nh * kD) {
            const int h = tid / kD, d = tid % kD;
            const float mr = stat[HPB + h], lr = stat[2 * HPB + h];
            const float mi = stat[3 * HPB + h], li = stat[4 * HPB + h];
            const int64_t row = static_cast<int64_t>(b) * g.Hq + hq0 + h;
            if constexpr (!CHUNKED) {
                const float mf = fmaxf(mi, mr);
                const float wi = (mi == -INFINITY) ? 0.f : __expf(mi - mf);
                const float wr = (mr == -INFINITY) ? 0.f : __expf(mr - mf);
                const float num = o_img * wi + o_res * wr;
                const float den = li * wi + lr * wr;
                store_elem<DT>(g.out, row * kD + d, num * __builtin_amdgcn_rcpf(den));
            } else {
                float* p = g.part + (row * g.nx + split) * (kD + 2);
                const bool is_img = split < g.nsplit;
                if (d == 0) { publish(p, is_img ? mi : mr); publish(p + 1, is_img ? li : lr); }
                publish(p + 2 + d, is_img ? o_img : o_res);
            }
        }
        if constexpr (CHUNKED) {
            // The unit's chunks (and its residual unit) each leave an (m, l, acc) partial; the workgroup that
            // finds all the others' already counted combines them.  The partials are device-scope atomic stores
            // (written through to the level all compute units share, so no cache has to be written back as a
            // whole): every thread waits for its own stores to complete, the barrier collects the workgroup,
            // then one thread counts.
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            int* last = reinterpret_cast<int*>(red);
            if (tid == 0) {
                if (g.fused) *last = arrive<__HIP_MEMORY_SCOPE_AGENT>(g.done64 + unit, g.epoch) == static_cast<uint32_t>(g.nx);
                else *last = __hip_atomic_fetch_add(g.cnt + unit, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == g.nx - 1;
            }
            __syncthreads();
            if (*last) {
                // the reader: one acquire drops this compute unit's and this die's cached copies of what other
                // dies wrote, after which ordinary loads (issued together, unlike atomic ones) see the partials
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
                if (tid < nh * kD) {
                    const int h = tid / kD, d = tid % kD;
                    const int64_t row = static_cast<int64_t>(b) * g.Hq + hq0 + h;
                    const float* p = g.part + row * g.nx * (kD + 2);
                    // eight partials at a time, their loads in flight together; running (m, num, den)
                    float m = -INFINITY, num = 0.f, den = 0.f;
                    for (int s0 = 0; s0 < g.nx; s0 += 8) {
                        float ms[8], ls[8], as[8];
#pragma unroll
                        for (int k = 0; k < 8; ++k) {
                            const float* q = p + min(s0 + k, g.nx - 1) * (kD + 2);
                            ms[k] = q[0]; ls[k] = q[1]; as[k] = q[2 + d];
                        }
                        float mb = m;
#pragma unroll
                        for (int k = 0; k < 8; ++k) mb = fmaxf(mb, (s0 + k < g.nx) ? ms[k] : -INFINITY);
                        const float keep = (m == -INFINITY) ? 0.f : __expf(m - mb);
                        num *= keep; den *= keep;
#pragma unroll
                        for (int k = 0; k < 8; ++k) {
                            const float w = (s0 + k < g.nx && ms[k] != -INFINITY) ? __expf(ms[k] - mb) : 0.f;
                            den += ls[k] * w;
                            num += as[k] * w;
                        }
                        m = mb;
                    }
                    store_elem<DT>(g.out, row * kD + d, num / den);
                }
                // every other workgroup of the unit is past both counters: leave them empty for a replay of this
                // very launch (a recorded step comes back with the same epoch)
                if (g.fused) clear_handover<HPB, kNT>(g, unit, tid);
            }
        }
    }
}

// ---- the chunked step in one launch: host side ------------------------------------------------------
// A word of pinned host memory per device that a workgroup sets when it gives up waiting for the other
// chunks of its unit (allocated once, at the first such call on the device; never freed).  The next chunked
// call on that device finds it set, reports CQ_ERR_LAUNCH once and the process goes on with two launches.
constexpr int kMaxDevices = 64;
static std::atomic<int*> g_status[kMaxDevices];
static std::atomic<bool> g_fused_off{false};      // set by a give-up; cleared by cq_decode_attn_wait_polls
static std::atomic<bool> g_fused_wanted{true};    // cq_decode_attn_single_launch
static std::atomic<uint32_t> g_epoch{0x5eed0000u};
static std::atomic<int> g_spin_limit{1 << 18};   // polls of about a microsecond each

// Compute units of the current device (a partitioned device reports its own share), asked once per
// process; kDefaultUnits when there is no device to ask (a host that only plans).
static int pair_units() {
    static std::atomic<int> cached{0};
    int n = cached.load(std::memory_order_relaxed);
    if (n > 0) return n;
    int dev = 0, cu = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cu < 1) {
        (void)hipGetLastError();   // not an error of the caller's
        cu = kDefaultUnits;
    }
    cached.store(cu, std::memory_order_relaxed);
    return cu;
}

// head groups per kv head; the last one may be partly padding (its spare heads repeat its last query head
// and write nothing)
static inline int ngroups(int G, int hpb) { return (G + hpb - 1) / hpb; }

struct Plan {
    int hpb, nh, nt, regl, nsplit, chunk, nx, cap, lds;   // hpb: heads an entry is wide; nh: heads a unit serves
    bool fused;   // chunked step in one launch: every chunk's workgroup fits the device at once
    size_t ws_mm, ws_part, ws_cnt, ws_lgt;   // chunked launch: min / max, partials, counters; logits (optional)
};

template <int BITS, int HPB, bool VTOK, int NT = 1024, int REGL = 0>
static void plan_for(const cq_decode_args* a, Plan* p, int nh = HPB) {
    using L = Lay<BITS, HPB, VTOK, NT, REGL>;
    const int G = a->Hq / a->Hkv;
    const int64_t units = static_cast<int64_t>(a->B) * a->Hkv * ngroups(G, nh);
    const int maxc = L::max_chunk();
    int nsplit = 1;
    if (a->T > 0) {
        const int need = (a->T + maxc - 1) / maxc;
        nsplit = need;
        if (a->force_splits > 0) {
            nsplit = a->force_splits > need ? a->force_splits : need;
        } else if (units < 192 && need > 1) {
            // too few units to fill the device and T does not fit one unit anyway: more, smaller chunks.
            // (A T that fits one unit is never chunked: the min/max launch's second pass over the packed
            // K rows and the merge cost more than the idle compute units, at any batch size.)
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
    p->nh = nh;
    p->nt = NT;
    p->regl = REGL;
    p->nsplit = nsplit;
    p->chunk = chunk;
    p->nx = nsplit + ((nsplit > 1 && a->R > 0) ? 1 : 0);
    p->cap = a->T > 0 ? chunk : 64;
    p->lds = L::lds_bytes(p->cap);
    const size_t rows = static_cast<size_t>(a->B) * a->Hq;
    p->ws_mm = nsplit > 1 ? ((rows * nsplit * 2 * sizeof(float) + 255) / 256 * 256) : 0;
    p->ws_part = nsplit > 1 ? (rows * p->nx * (kD + 2) * sizeof(float) + 255) / 256 * 256 : 0;
    // counters: [unit] partials written (4 or 8 bytes), then the min / max records of the single-launch step
    p->ws_cnt = nsplit > 1 ? (static_cast<size_t>(units) * sizeof(unsigned long long) + 255) / 256 * 256 +
                                 static_cast<size_t>(units) * HPB * nsplit * 16 : 0;
    p->fused = false;
    // The logits go through a buffer where that is less traffic than the main launch reading the packed K rows
    // again (4 bytes per head and token against the row's 16 or 32 bytes).  Measured at batch 8 x 32 768 tokens,
    // four heads per unit: 2 bits 108.6 -> 90.9 us with the buffer, 1 bit (equal bytes) 52.3 -> 54.0 us.
    const bool hand_over = nsplit > 1 && 16 * BITS > 4 * HPB;
    p->ws_lgt = hand_over ? static_cast<size_t>(units) * a->T * HPB * sizeof(float) : 0;
}

static int make_plan(const cq_decode_args* a, Plan* p) {
    if (!a) return CQ_ERR_NULL;
    const int kPairUnits = pair_units();
    if (a->dtype != CQ_BF16 && a->dtype != CQ_FP16) return CQ_ERR_DTYPE;
    if (a->bits != 1 && a->bits != 2) return CQ_ERR_UNSUPPORTED;
    if (a->D != kD) return CQ_ERR_UNSUPPORTED;
    if (a->B < 1 || a->Hq < 1 || a->Hkv < 1 || a->Hq % a->Hkv) return CQ_ERR_SHAPE;
    if (a->T < 0 || a->R < 0 || (a->T == 0 && a->R == 0)) return CQ_ERR_SHAPE;
    if (a->sprompt_len < 0 || a->sprompt_len > a->R) return CQ_ERR_SHAPE;
    const int G = a->Hq / a->Hkv;
    if (a->v_mode != CQ_V_PER_CHANNEL && a->v_mode != CQ_V_PER_TOKEN) return CQ_ERR_UNSUPPORTED;
    const bool vtok = a->v_mode == CQ_V_PER_TOKEN;
    // heads a unit with four-wide entries serves: three when that divides the group exactly and four does not
    // (G = 3, 6, 9: exact units instead of a padded last one; per-channel values only)
    const int nh4 = (!vtok && G % 3 == 0 && G % 4 != 0) ? 3 : 4;
    if (a->bits == 1) {
        // G = 3, 5, 6, 7, ...: units of four heads with the last one partly padding (two units per kv head at
        // G = 6) do less work than units of two heads or one (three or six of them, each walking all the packed rows)
        const bool pad4 = G % 4 != 0 && G > 2;
        if (G % 4 == 0 || pad4) vtok ? plan_for<1, 4, true>(a, p) : plan_for<1, 4, false>(a, p, nh4);
        else if (G % 2 == 0) vtok ? plan_for<1, 2, true>(a, p) : plan_for<1, 2, false>(a, p);
        else vtok ? plan_for<1, 1, true>(a, p) : plan_for<1, 1, false>(a, p);
        // More units than compute units: 512-thread workgroups, two resident per compute unit, need fewer
        // instructions per unit than one 1024-thread workgroup after the other (half as many waves pay
        // the per-wave set-up, reductions and folds) - when a unit's whole layout fits half the LDS.
        // Four heads per unit, enough units to fill the device, and T beyond the layout with fp32 logits in
        // the token slots: with the logits in registers (half the bytes per token slot) the layout may still
        // hold all T tokens in one launch, which saves the min/max launch's second pass over the packed K rows.
        if (p->hpb == 4 && !vtok && a->force_splits == 0 && p->nsplit > 1 &&
            static_cast<int64_t>(a->B) * a->Hkv * ngroups(G, nh4) >= kPairUnits * 3 / 4) {
            Plan q;
            plan_for<1, 4, false, 1024, kRegLong>(a, &q, nh4);
            if (q.nsplit == 1) *p = q;
        }
        // Single launch: only if the 512-thread layout also holds all T tokens.  Chunked launch (four heads
        // per unit): the chunks are units of their own.
        const int64_t units = static_cast<int64_t>(a->B) * a->Hkv * ngroups(G, p->nh);
        if (!vtok && a->force_splits == 0 && p->hpb >= 2) {
            Plan q;
            if (p->hpb == 4) plan_for<1, 4, false, 512, kRegPair>(a, &q, nh4); else plan_for<1, 2, false, 512, 0>(a, &q);
            const bool single = p->nsplit == 1 && q.nsplit == 1 && units > kPairUnits;
            const bool chunked = p->hpb == 4 && p->nsplit > 1 && q.nsplit > 1 && units * q.nsplit > kPairUnits;
            if ((single || chunked) && q.lds <= kLdsMax / 2) *p = q;
        }
    } else {
        // four heads per unit need the two-pass K table; with per-token values their LDS layout
        // would not hold a 3 328-token chunk, so that mode keeps two heads per unit
        // (the first pass's partial logits wait in registers, four tokens per thread: -3 % against the token slots)
        if ((G % 4 == 0 || G > 2) && !vtok) {
            plan_for<2, 4, false, 1024, kRegTwoBit>(a, p, nh4);
            // more units than compute units: two 512-thread workgroups per compute unit (K table in two passes)
            const int64_t units = static_cast<int64_t>(a->B) * a->Hkv * ngroups(G, nh4);
            if (a->force_splits == 0) {
                Plan q;
                plan_for<2, 4, false, 512, kRegPair>(a, &q, nh4);
                const bool single = p->nsplit == 1 && q.nsplit == 1 && units > kPairUnits;
                const bool chunked = p->nsplit > 1 && q.nsplit > 1 && units * q.nsplit > kPairUnits;
                if ((single || chunked) && q.lds <= kLdsMax / 2) *p = q;
            }
        }
        else if (G >= 2) vtok ? plan_for<2, 2, true>(a, p) : plan_for<2, 2, false>(a, p);   // (per-token values: two heads per unit, padded for odd G)
        else vtok ? plan_for<2, 1, true>(a, p) : plan_for<2, 1, false>(a, p);
    }
    // A handful of units leave most compute units idle, and a launch then lasts as long as one unit: fewer
    // heads per unit make the units cheaper (18.8 / 15.5 / 14.2 us for four / two / one head at 3 328 + 128 tokens)
    // and there are compute units for two or four times as many of them.
    if (a->force_splits == 0 && p->nsplit == 1 && p->hpb == 4) {
        const int64_t u4 = static_cast<int64_t>(a->B) * a->Hkv * ngroups(G, p->nh);
        const int h = u4 <= 32 ? 1 : (u4 <= 64 && G % 2 == 0) ? 2 : 4;
        Plan q = *p;
        if (a->bits == 1) {
            if (h == 1) vtok ? plan_for<1, 1, true>(a, &q) : plan_for<1, 1, false>(a, &q);
            if (h == 2) vtok ? plan_for<1, 2, true>(a, &q) : plan_for<1, 2, false>(a, &q);
        } else {
            if (h == 1) vtok ? plan_for<2, 1, true>(a, &q) : plan_for<2, 1, false>(a, &q);
            if (h == 2) vtok ? plan_for<2, 2, true>(a, &q) : plan_for<2, 2, false>(a, &q);
        }
        if (q.nsplit == 1) *p = q;
    }
    const int64_t blocks = static_cast<int64_t>(a->B) * a->Hkv * ngroups(G, p->nh) * p->nx;
    if (blocks > 0x7fffffff) return CQ_ERR_SHAPE;
    // Chunked, and every chunk's workgroup resident at once (two 512-thread workgroups per compute unit, one of
    // 1024): one launch, the chunks exchange their min / max inside it and keep their logits - no second read of
    // the packed K rows, no logits buffer.  (The residual units wait for nobody and make room as they end.)
    if (p->nsplit > 1) {
        const int64_t waiting = static_cast<int64_t>(a->B) * a->Hkv * ngroups(G, p->nh) * p->nsplit;
        const int64_t room = static_cast<int64_t>(kPairUnits) * ((p->nt == 512 && p->lds <= kLdsMax / 2) ? 2 : 1);
        // (one lane per chunk polls)
        if (waiting <= room && p->nsplit <= 64 && g_fused_wanted.load(std::memory_order_relaxed)) p->fused = true;
    }
    return CQ_OK;
}

template <int BITS, int HPB, typename DT, bool VTOK, int NT = 1024, int REGL = 0, int NH = HPB>
static int launch(const DecodeGeom& g, const Plan& p, hipStream_t st) {
    const int G = g.Hq / g.Hkv;
    const unsigned units = static_cast<unsigned>(g.B) * g.Hkv * ngroups(G, NH);
    const bool extras = g.mask != nullptr || g.r_dev != nullptr;
    auto kmain = g.nsplit > 1 ? (extras ? decode_kernel<BITS, HPB, DT, false, VTOK, NT, REGL, true, true, NH>
                                        : decode_kernel<BITS, HPB, DT, false, VTOK, NT, REGL, true, false, NH>)
                              : (extras ? decode_kernel<BITS, HPB, DT, false, VTOK, NT, REGL, false, true, NH>
                                        : decode_kernel<BITS, HPB, DT, false, VTOK, NT, REGL, false, false, NH>);
    auto kmm = decode_kernel<BITS, HPB, DT, true, false, NT, REGL, true, false, NH>;   // the min/max pass never looks at values
    // raise the dynamic-LDS limit once per device for this instantiation
    static std::atomic<uint32_t> attr_done{0};
    int dev = 0;
    CQ_HIP_CHECK(hipGetDevice(&dev));
    const uint32_t bit = 1u << (dev & 31);
    if (!(attr_done.load(std::memory_order_acquire) & bit)) {
        // the K look-ups address the table absolutely: the dynamic LDS array must start at 0
        const void* kernels[5] = {reinterpret_cast<const void*>(decode_kernel<BITS, HPB, DT, false, VTOK, NT, REGL, false, false, NH>),
                                  reinterpret_cast<const void*>(decode_kernel<BITS, HPB, DT, false, VTOK, NT, REGL, false, true, NH>),
                                  reinterpret_cast<const void*>(decode_kernel<BITS, HPB, DT, false, VTOK, NT, REGL, true, false, NH>),
                                  reinterpret_cast<const void*>(decode_kernel<BITS, HPB, DT, false, VTOK, NT, REGL, true, true, NH>),
                                  reinterpret_cast<const void*>(kmm)};
        for (const void* k : kernels) {
            hipFuncAttributes fa;
            CQ_HIP_CHECK(hipFuncGetAttributes(&fa, k));
            if (fa.sharedSizeBytes != 0) return CQ_ERR_LAUNCH;
            CQ_HIP_CHECK(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsMax));
        }
        attr_done.fetch_or(bit, std::memory_order_release);
    }
    DecodeGeom gm = g;
    gm.G = G;
    // (a main launch that reads its logits back has no look-up phase for the first workgroup to get ahead in:
    // with the priorities the second one would hold the packed-V loop to itself)
    gm.ncu = (NT == 512 && !g.lgt && !g.fused && static_cast<int64_t>(units) * g.nx <= 2 * static_cast<int64_t>(pair_units())) ? pair_units() : 0;
    gm.d_ng.set(static_cast<uint32_t>(ngroups(G, NH)));
    gm.d_nx.set(static_cast<uint32_t>(g.nx));
    gm.d_hkv.set(static_cast<uint32_t>(g.Hkv));
    if (g.nsplit > 1 && !g.fused) {
        DecodeGeom g1 = gm;
        g1.nx = g.nsplit;  // the min/max pass has no residual unit
        g1.d_nx.set(static_cast<uint32_t>(g.nsplit));
        // ... and keeps no logits, unless the table takes two passes (partial logits wait in the slots)
        g1.cap = (Lay<BITS, HPB, false, NT, REGL>::KPASS > 1 && REGL == 0) ? p.cap : 0;
        const int lds_mm = Lay<BITS, HPB, false, NT, REGL>::lds_bytes(g1.cap);
        hipLaunchKernelGGL(kmm, dim3(units * g.nsplit), dim3(NT), lds_mm, st, g1);
        CQ_LAUNCH_CHECK();
    }
    hipLaunchKernelGGL(kmain, dim3(units * g.nx), dim3(NT), p.lds, st, gm);
    CQ_LAUNCH_CHECK();
    return CQ_OK;
}

template <typename DT, bool VTOK>
static int dispatch(const DecodeGeom& g, const Plan& p, int bits, hipStream_t st) {
#ifdef CQ_PHASE_STOPS
    if constexpr (!VTOK && std::is_same<DT, BF16>::value) {
        if (bits == 1 && p.hpb == 4 && p.nh == 4 && p.nt == 512) return launch<1, 4, DT, false, 512, kRegPair>(g, p, st);
    }
    return CQ_ERR_UNSUPPORTED;
#else
    if constexpr (!VTOK) {
        if (p.nh == 3 && p.hpb == 4) {   // exact units of three heads
            if (bits == 1) {
                if (p.nt == 512) return launch<1, 4, DT, false, 512, kRegPair, 3>(g, p, st);
                if (p.regl) return launch<1, 4, DT, false, 1024, kRegLong, 3>(g, p, st);
                return launch<1, 4, DT, false, 1024, 0, 3>(g, p, st);
            }
            if (p.nt == 512) return launch<2, 4, DT, false, 512, kRegPair, 3>(g, p, st);
            return launch<2, 4, DT, false, 1024, kRegTwoBit, 3>(g, p, st);
        }
    }
    if (bits == 1) {
        if constexpr (!VTOK) {
            if (p.hpb == 4 && p.nt == 512) return launch<1, 4, DT, false, 512, kRegPair>(g, p, st);
            if (p.hpb == 4 && p.regl) return launch<1, 4, DT, false, 1024, kRegLong>(g, p, st);
            if (p.hpb == 2 && p.nt == 512) return launch<1, 2, DT, false, 512, 0>(g, p, st);
        }
        if (p.hpb == 4) return launch<1, 4, DT, VTOK>(g, p, st);
        if (p.hpb == 2) return launch<1, 2, DT, VTOK>(g, p, st);
        return launch<1, 1, DT, VTOK>(g, p, st);
    }
    if constexpr (!VTOK) {
        if (p.hpb == 4 && p.nt == 512) return launch<2, 4, DT, false, 512, kRegPair>(g, p, st);
        if (p.hpb == 4) return launch<2, 4, DT, false, 1024, kRegTwoBit>(g, p, st);
    }
    if (p.hpb == 2) return launch<2, 2, DT, VTOK>(g, p, st);
    return launch<2, 1, DT, VTOK>(g, p, st);
#endif
}

// ---- static scratch for callers that cannot allocate --------------------------------------------
// The chunked path's workspace (per-chunk logit min / max, flash-decoding partials) in a file-scope
// device array: every GPU the library runs on holds its own copy, at its own address, until the
// process ends.  Host code never uses the array's name as an address: the device address is asked
// for once per device (with that device current) and kept.
constexpr size_t kScratchBytes = static_cast<size_t>(8) << 20;
// (`used`: no kernel names the array - they get its address as an argument - so nothing else keeps it in the code object)
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[kScratchBytes];

static std::atomic<void*> g_scratch_ptr[kMaxDevices];

static int scratch_address(void** out) {
    int dev = 0;
    CQ_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return CQ_ERR_UNSUPPORTED;
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        CQ_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return CQ_ERR_LAUNCH;
        g_scratch_ptr[dev].store(p, std::memory_order_release);   // every caller on this device gets the same address
    }
    *out = p;
    return CQ_OK;
}

static int* fused_status_word(hipStream_t st) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    int* p = g_status[dev].load(std::memory_order_acquire);
    if (p) return p;
    // not while the stream is being recorded: an allocation would end the recording
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
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
    if (!g_status[dev].compare_exchange_strong(expected, static_cast<int*>(raw), std::memory_order_acq_rel)) {
        (void)hipHostFree(raw);   // another host thread was first
        return expected;
    }
    return static_cast<int*>(raw);
}

static int decode_entry(const cq_decode_args* a, void* workspace, size_t workspace_bytes, bool static_scratch,
                        cq_stream_t stream) {
    Plan p;
    int rc = make_plan(a, &p);
    if (rc != CQ_OK) return rc;
    if (!a->q || !a->out) return CQ_ERR_NULL;
    if (a->T > 0 && (!a->codes_k || !a->codes_v || !a->k_scale || !a->k_zero || !a->v_scale || !a->v_zero))
        return CQ_ERR_NULL;
    if (a->R > 0 && (!a->k_res || !a->v_res)) return CQ_ERR_NULL;
    if (a->r_dev && a->mask) return CQ_ERR_UNSUPPORTED;   // the mask's length would have to follow the count
    if (a->r_dev && (reinterpret_cast<uintptr_t>(a->r_dev) & 3)) return CQ_ERR_ALIGN;
    if (a->T > 0 && (!aligned16(a->codes_k) || !aligned16(a->codes_v))) return CQ_ERR_ALIGN;
    if (a->R > 0 && (!aligned16(a->k_res) || !aligned16(a->v_res) || (a->res_stride_b % 8) ||
                     (a->res_stride_h % 8) || (a->res_stride_r % 8)))
        return CQ_ERR_ALIGN;
    // the logits buffer is the last part of the workspace; the static scratch does without it when it
    // does not fit (the main launch then recomputes the logits)
    const size_t need_min = p.ws_mm + p.ws_part + p.ws_cnt;
    // One launch when the plan allows it, the caller's own workspace is used (the static entry point allocates
    // nothing, not even the status word) and no earlier launch of this process gave up waiting.
    int* status = nullptr;
    bool fused = p.fused && !static_scratch && !g_fused_off.load(std::memory_order_relaxed);
    if (fused) {
        status = fused_status_word(static_cast<hipStream_t>(stream));
        if (!status) {
            fused = false;
        } else if (*static_cast<volatile int*>(status) != 0) {
            *static_cast<volatile int*>(status) = 0;
            g_fused_off.store(true, std::memory_order_relaxed);
            return CQ_ERR_LAUNCH;   // an earlier single-launch step did not complete: its output is not valid
        }
    }
    bool with_logits = !fused && p.ws_lgt > 0;
    if (static_scratch && need_min + p.ws_lgt > kScratchBytes) with_logits = false;
    // (a plan for one launch sizes the caller's workspace without the logits buffer)
    if (!static_scratch && p.fused && workspace_bytes < need_min + p.ws_lgt) with_logits = false;
    const size_t need = need_min + (with_logits ? p.ws_lgt : 0);
    if (static_scratch) {
        if (need > kScratchBytes) return CQ_ERR_SCRATCH_LIMIT;
        workspace = nullptr;
        if (need) {
            rc = scratch_address(&workspace);
            if (rc != CQ_OK) return rc;
        }
    } else if (need && (!workspace || workspace_bytes < need || !aligned16(workspace))) {
        return CQ_ERR_WORKSPACE;
    }

    DecodeGeom g;
    g.q = a->q; g.ck = a->codes_k; g.cv = a->codes_v;
    g.ks = a->k_scale; g.kz = a->k_zero; g.vs = a->v_scale; g.vz = a->v_zero;
    g.kres = a->k_res; g.vres = a->v_res;
    g.rs_b = a->res_stride_b; g.rs_h = a->res_stride_h; g.rs_r = a->res_stride_r;
    g.mask = a->mask; g.mask_sb = a->mask_stride_b;
    g.r_dev = a->r_dev;
    g.out = a->out;
    g.mm = static_cast<float*>(workspace);
    g.part = need ? reinterpret_cast<float*>(static_cast<char*>(workspace) + p.ws_mm) : nullptr;
    g.cnt = need ? reinterpret_cast<int*>(static_cast<char*>(workspace) + p.ws_mm + p.ws_part) : nullptr;
    {
        const int G = a->Hq / a->Hkv;
        const size_t units = static_cast<size_t>(a->B) * a->Hkv * ngroups(G, p.nh);
        char* c0 = reinterpret_cast<char*>(g.cnt);
        g.done64 = reinterpret_cast<unsigned long long*>(c0);
        g.rec = reinterpret_cast<unsigned long long*>(c0 + (units * sizeof(unsigned long long) + 255) / 256 * 256);
    }
#ifdef CQ_PHASE_STOPS
    {
        const char* e = getenv("CQ_DECODE_PHASE_STOP");
        g.stop = e ? atoi(e) : -1;
    }
#endif
    g.fused = fused ? 1 : 0;
    g.status = status;
    g.spin_limit = g_spin_limit.load(std::memory_order_relaxed);
    uint32_t ep = g_epoch.fetch_add(1, std::memory_order_relaxed) + 1;
    g.epoch = ep ? ep : g_epoch.fetch_add(1, std::memory_order_relaxed) + 1;   // 0 marks an empty counter
    g.lgt = with_logits ? reinterpret_cast<float*>(static_cast<char*>(workspace) + need_min) : nullptr;
    g.B = a->B; g.Hq = a->Hq; g.Hkv = a->Hkv; g.T = a->T; g.R = a->R; g.S = a->sprompt_len;
    g.nsplit = p.nsplit; g.chunk = p.chunk; g.nx = p.nx;
    g.calib = a->calibrate; g.off_max = a->calib_off_max; g.off_min = a->calib_off_min;
    g.cap = p.cap;
    g.one = 1.0f;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool vtok = a->v_mode == CQ_V_PER_TOKEN;
    if (a->dtype == CQ_BF16)
        return vtok ? dispatch<BF16, true>(g, p, a->bits, st) : dispatch<BF16, false>(g, p, a->bits, st);
    return vtok ? dispatch<FP16, true>(g, p, a->bits, st) : dispatch<FP16, false>(g, p, a->bits, st);
}

}  // namespace cq

extern "C" {

size_t cq_decode_attn_workspace(const cq_decode_args* args) {
    cq::Plan p;
    if (cq::make_plan(args, &p) != CQ_OK) return 0;
    return p.ws_mm + p.ws_part + p.ws_cnt + (p.fused ? 0 : p.ws_lgt);
}

int cq_decode_attn_single_launch(int enable) {
    const int before = cq::g_fused_wanted.load(std::memory_order_relaxed) ? 1 : 0;
    if (enable >= 0) cq::g_fused_wanted.store(enable != 0, std::memory_order_relaxed);
    return before;
}

int cq_decode_attn_gave_up(void) {
    for (int dev = 0; dev < cq::kMaxDevices; ++dev) {
        const int* p = cq::g_status[dev].load(std::memory_order_acquire);
        if (p && *static_cast<const volatile int*>(p) != 0) return 1;
    }
    return 0;
}

int cq_decode_attn_wait_polls(int polls) {
    const int before = cq::g_spin_limit.load(std::memory_order_relaxed);
    if (polls >= 0) {
        cq::g_spin_limit.store(polls, std::memory_order_relaxed);
        cq::g_fused_off.store(false, std::memory_order_relaxed);
    }
    return before;
}

int cq_decode_attn_plan(const cq_decode_args* args, cq_decode_plan* plan) {
    if (!plan) return CQ_ERR_NULL;
    cq::Plan p;
    const int rc = cq::make_plan(args, &p);
    if (rc != CQ_OK) return rc;
    plan->threads = p.nt;
    plan->heads_per_unit = p.nh;
    plan->chunks = p.nsplit;
    plan->chunk_tokens = args->T > 0 ? p.chunk : 0;
    plan->launches = (p.nsplit > 1 && !p.fused) ? 2 : 1;
    plan->lds_bytes = p.lds;
    plan->register_logits = p.regl;
    return CQ_OK;
}

int cq_decode_attn(const cq_decode_args* a, cq_stream_t stream) {
    if (!a) return CQ_ERR_NULL;
    return cq::decode_entry(a, a->workspace, a->workspace_bytes, false, stream);
}

size_t cq_decode_attn_static_limit(void) { return cq::kScratchBytes; }

int cq_decode_attn_static(const cq_decode_args* a, cq_stream_t stream) {
    if (!a) return CQ_ERR_NULL;
    return cq::decode_entry(a, nullptr, 0, true, stream);
}

}  // extern "C"
