// The two look-up-table vec-mat operators of the reference surface
// (fused_kernel / fused_kernel_wv), for callers that keep the unfused call
// sequence.  Any table contents are honoured (the fused decode kernel assumes
// the identity table instead), and a table shorter than 2^bits entries - the
// reference builds it from the levels seen in the first 10 000 codes
// (patch_internvl.py:318-329) - is never read past its end: a code without an
// entry contributes 0.  fp32 accumulation, fp16 output.
#include "cq_common.h"

namespace cq {

__device__ __forceinline__ float load_any(const void* p, int dtype, int64_t i) {
    switch (dtype) {
        case CQ_BF16: return bf16_bits_to_float(static_cast<const uint16_t*>(p)[i]);
        case CQ_FP16: return fp16_bits_to_float(static_cast<const uint16_t*>(p)[i]);
        default: return static_cast<const float*>(p)[i];
    }
}

constexpr int kVmThreads = 256;

// Table entry v, or 0 past the end of the table.
__device__ __forceinline__ float lut_entry(const void* lut, int lut_dtype, int lut_len, int v) {
    return v < lut_len ? load_any(lut, lut_dtype, v) : 0.f;
}

// c[m, t] = sum_d a[m, d] * lut[code[m, t, d]].  grid (M, token tiles); one
// thread per token, the row a[m, :] pre-multiplied into per-code weights in LDS:
// w[d][v] = a[d] * lut[v].
template <int BITS>
__global__ __launch_bounds__(kVmThreads) void vecmat_qk_kernel(const void* __restrict__ lut, int lut_dtype, int lut_len,
                                                               const void* __restrict__ a, int a_dtype,
                                                               const uint8_t* __restrict__ enc, int T, int D,
                                                               uint16_t* __restrict__ out) {
    constexpr int NV = 1 << BITS;
    constexpr int dpe = 8 / BITS;
    extern __shared__ float w[];  // D * NV
    const int64_t m = blockIdx.x;
    for (int i = threadIdx.x; i < D * NV; i += kVmThreads)
        w[i] = load_any(a, a_dtype, m * D + i / NV) * lut_entry(lut, lut_dtype, lut_len, i % NV);
    __syncthreads();
    const int t = blockIdx.y * kVmThreads + threadIdx.x;
    if (t >= T) return;
    const int nb = D / dpe;
    const uint8_t* row = enc + (m * T + t) * nb;
    float acc = 0.f;
    for (int j = 0; j < nb; ++j) {
        const uint32_t byte = row[j];
#pragma unroll
        for (int k = 0; k < dpe; ++k) {
            const uint32_t v = (byte >> (BITS * (dpe - 1 - k))) & (NV - 1);
            acc += w[(j * dpe + k) * NV + v];
        }
    }
    out[m * T + t] = static_cast<uint16_t>(float_to_fp16_bits(acc));
}

// c[m, d] = sum_t a[m, t] * lut[code[m, t, d]].  grid (M); thread = (byte
// column j, token slot); partial sums folded through LDS.
template <int BITS>
__global__ __launch_bounds__(kVmThreads) void vecmat_pv_kernel(const void* __restrict__ lut, int lut_dtype, int lut_len,
                                                               const void* __restrict__ a, int a_dtype,
                                                               const uint8_t* __restrict__ enc, int T, int D,
                                                               uint16_t* __restrict__ out) {
    constexpr int NV = 1 << BITS;
    constexpr int dpe = 8 / BITS;
    extern __shared__ float red[];  // slots * D
    const int64_t m = blockIdx.x;
    const int nb = D / dpe;
    const int slots = kVmThreads / nb;
    const int j = threadIdx.x % nb;
    const int slot = threadIdx.x / nb;
    float lv[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) lv[v] = lut_entry(lut, lut_dtype, lut_len, v);
    float acc[dpe];
#pragma unroll
    for (int k = 0; k < dpe; ++k) acc[k] = 0.f;
    if (slot < slots) {
        for (int t = slot; t < T; t += slots) {
            const float p = load_any(a, a_dtype, m * T + t);
            const uint32_t byte = enc[(m * T + t) * nb + j];
#pragma unroll
            for (int k = 0; k < dpe; ++k) {
                const uint32_t v = (byte >> (BITS * (dpe - 1 - k))) & (NV - 1);
                float val = lv[0];
#pragma unroll
                for (int u = 1; u < NV; ++u) val = (v == u) ? lv[u] : val;
                acc[k] += p * val;
            }
        }
#pragma unroll
        for (int k = 0; k < dpe; ++k) red[slot * D + j * dpe + k] = acc[k];
    }
    __syncthreads();
    for (int d = threadIdx.x; d < D; d += kVmThreads) {
        float s = 0.f;
        for (int r = 0; r < slots; ++r) s += red[r * D + d];
        out[m * D + d] = static_cast<uint16_t>(float_to_fp16_bits(s));
    }
}

static int check_vm(const void* lut, int lut_dtype, int lut_len, const void* a, int a_dtype, const uint8_t* enc, int64_t M,
                    int T, int D, int bits, void* out) {
    if (!lut || !a || !enc || !out) return CQ_ERR_NULL;
    if (lut_len < 1) return CQ_ERR_SHAPE;
    if (bits != 1 && bits != 2) return CQ_ERR_UNSUPPORTED;
    if (lut_dtype < CQ_BF16 || lut_dtype > CQ_FP32 || a_dtype < CQ_BF16 || a_dtype > CQ_FP32) return CQ_ERR_DTYPE;
    if (M < 1 || M > 0x7fffffff || T < 1 || D < 8 || D > 1024 || (D % 8) != 0) return CQ_ERR_SHAPE;
    return CQ_OK;
}

}  // namespace cq

extern "C" {

int cq_lut_vecmat_qk(const void* lut, int lut_dtype, int lut_len, const void* a, int a_dtype, const uint8_t* enc,
                     int64_t M, int T, int D, int bits, void* out_fp16, cq_stream_t stream) {
    int rc = cq::check_vm(lut, lut_dtype, lut_len, a, a_dtype, enc, M, T, D, bits, out_fp16);
    if (rc != CQ_OK) return rc;
    const int tiles = (T + cq::kVmThreads - 1) / cq::kVmThreads;
    if (tiles > 65535) return CQ_ERR_SHAPE;   // rows on grid.x (up to 2^31 - 1), token tiles on grid.y
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid(static_cast<unsigned>(M), tiles);
    const size_t lds = static_cast<size_t>(D) * (1 << bits) * sizeof(float);
    uint16_t* o = static_cast<uint16_t*>(out_fp16);
    if (bits == 1)
        hipLaunchKernelGGL((cq::vecmat_qk_kernel<1>), grid, dim3(cq::kVmThreads), lds, s, lut, lut_dtype, lut_len, a,
                           a_dtype, enc, T, D, o);
    else
        hipLaunchKernelGGL((cq::vecmat_qk_kernel<2>), grid, dim3(cq::kVmThreads), lds, s, lut, lut_dtype, lut_len, a,
                           a_dtype, enc, T, D, o);
    CQ_LAUNCH_CHECK();
    return CQ_OK;
}

int cq_lut_vecmat_pv(const void* lut, int lut_dtype, int lut_len, const void* a, int a_dtype, const uint8_t* enc,
                     int64_t M, int T, int D, int bits, void* out_fp16, cq_stream_t stream) {
    int rc = cq::check_vm(lut, lut_dtype, lut_len, a, a_dtype, enc, M, T, D, bits, out_fp16);
    if (rc != CQ_OK) return rc;
    const int nb = D * bits / 8;
    if (nb > cq::kVmThreads) return CQ_ERR_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int slots = cq::kVmThreads / nb;
    const size_t lds = static_cast<size_t>(slots) * D * sizeof(float);
    uint16_t* o = static_cast<uint16_t*>(out_fp16);
    if (bits == 1)
        hipLaunchKernelGGL((cq::vecmat_pv_kernel<1>), dim3(static_cast<unsigned>(M)), dim3(cq::kVmThreads), lds, s,
                           lut, lut_dtype, lut_len, a, a_dtype, enc, T, D, o);
    else
        hipLaunchKernelGGL((cq::vecmat_pv_kernel<2>), dim3(static_cast<unsigned>(M)), dim3(cq::kVmThreads), lds, s,
                           lut, lut_dtype, lut_len, a, a_dtype, enc, T, D, o);
    CQ_LAUNCH_CHECK();
    return CQ_OK;
}

}  // extern "C"
