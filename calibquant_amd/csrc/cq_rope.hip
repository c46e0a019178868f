// Decode-step glue around the attention kernel: the (h gs d) de-interleave of the
// fused wqkv projection, rotary embedding of the query and key heads, and the append
// of the new key / value row to the full-precision window, in one launch.
//
// The reference does this with a chain of torch ops per layer and token
// (patch_internvl.py:219-234 split, :258-260 and :119-138 rotary embedding,
// :264-266 torch.cat append).  Arithmetic follows the chain that runs there op for op:
// `copy_().mul_(cos)` rounds x * cos to the storage dtype, then `addcmul_(rotate_half(x), sin)`
// adds the product rotate_half(x) * sin in fp32 and rounds once (patch_internvl.py:125-128):
// rnd(rnd(x * cos) + rot * sin).  The product of two 16-bit values is exact in fp32, so a
// fused or an unfused multiply-add give the same bits.
#include "cq_common.h"

#pragma clang fp contract(off)

namespace cq {

struct RopeGeom {
    const uint16_t* qkv;   // (B, Hkv, G + 2, D)
    const uint16_t* cos;   // (rows, D)
    const uint16_t* sin;
    const int64_t* pos;    // position id of sample b at pos[b * pos_stride]
    int64_t pos_stride;
    int64_t table_rows;
    uint16_t* q_out;       // (B, Hkv * G, D)
    uint16_t* k_win;       // (B, Hkv, capacity, D) through strides
    uint16_t* v_win;
    int64_t ws_b, ws_h, ws_r;
    const int64_t* row_dev;   // window row that receives the new key / value
    int capacity;
    int Hkv, G;
};

constexpr int kRD = 128;   // head_dim

// grid (B * Hkv), block (G + 2) * 64: thread = (slot s of the group, pair (d, d + 64))
template <typename DT>
__global__ void rope_append_kernel(RopeGeom g) {
    const int s = threadIdx.x >> 6, d = threadIdx.x & 63;
    const int hkv = blockIdx.x % g.Hkv, b = blockIdx.x / g.Hkv;
    const uint16_t* x = g.qkv + ((static_cast<int64_t>(b) * g.Hkv + hkv) * (g.G + 2) + s) * kRD;
    const uint32_t lo = x[d], hi = x[d + 64];
    const int64_t row = *g.row_dev;
    const bool room = row >= 0 && row < g.capacity;
    if (s == g.G + 1) {   // value: copied as it is
        if (room) {
            uint16_t* o = g.v_win + b * g.ws_b + hkv * g.ws_h + row * g.ws_r;
            o[d] = static_cast<uint16_t>(lo);
            o[d + 64] = static_cast<uint16_t>(hi);
        }
        return;
    }
    int64_t p = g.pos[b * g.pos_stride];
    p = p < 0 ? 0 : (p >= g.table_rows ? g.table_rows - 1 : p);
    const uint16_t* c = g.cos + p * kRD;
    const uint16_t* sn = g.sin + p * kRD;
    const float x1 = Cvt<DT>::to_float(lo), x2 = Cvt<DT>::to_float(hi);
    // rnd(rnd(x * cos) + rotate_half(x) * sin) with rotate_half(x) = (-x2, x1); the second product stays fp32
    const float o1 = rnd<DT>(rnd<DT>(x1 * Cvt<DT>::to_float(c[d])) + (-x2 * Cvt<DT>::to_float(sn[d])));
    const float o2 = rnd<DT>(rnd<DT>(x2 * Cvt<DT>::to_float(c[d + 64])) + (x1 * Cvt<DT>::to_float(sn[d + 64])));
    uint16_t* o;
    if (s < g.G) {
        o = g.q_out + ((static_cast<int64_t>(b) * g.Hkv + hkv) * g.G + s) * kRD;
    } else {
        if (!room) return;
        o = g.k_win + b * g.ws_b + hkv * g.ws_h + row * g.ws_r;
    }
    o[d] = static_cast<uint16_t>(Cvt<DT>::from_float(o1));
    o[d + 64] = static_cast<uint16_t>(Cvt<DT>::from_float(o2));
}

}  // namespace cq

extern "C" int cq_rope_append(const void* qkv, int dtype, int B, int Hq, int Hkv, int D,
                              const void* cos_table, const void* sin_table, int64_t table_rows,
                              const int64_t* pos, int64_t pos_stride, void* q_out,
                              void* k_win, void* v_win, int64_t win_stride_b, int64_t win_stride_h,
                              int64_t win_stride_r, int capacity, const int64_t* row_dev, cq_stream_t stream) {
    if (!qkv || !cos_table || !sin_table || !pos || !q_out || !k_win || !v_win || !row_dev) return CQ_ERR_NULL;
    if (dtype != CQ_BF16 && dtype != CQ_FP16) return CQ_ERR_DTYPE;
    if (D != cq::kRD) return CQ_ERR_UNSUPPORTED;
    if (B < 1 || Hq < 1 || Hkv < 1 || Hq % Hkv || table_rows < 1 || capacity < 1) return CQ_ERR_SHAPE;
    const int G = Hq / Hkv;
    if ((G + 2) * 64 > 1024) return CQ_ERR_UNSUPPORTED;
    if (static_cast<int64_t>(B) * Hkv > 0x7fffffff) return CQ_ERR_SHAPE;
    cq::RopeGeom g;
    g.qkv = static_cast<const uint16_t*>(qkv);
    g.cos = static_cast<const uint16_t*>(cos_table);
    g.sin = static_cast<const uint16_t*>(sin_table);
    g.pos = pos; g.pos_stride = pos_stride; g.table_rows = table_rows;
    g.q_out = static_cast<uint16_t*>(q_out);
    g.k_win = static_cast<uint16_t*>(k_win);
    g.v_win = static_cast<uint16_t*>(v_win);
    g.ws_b = win_stride_b; g.ws_h = win_stride_h; g.ws_r = win_stride_r;
    g.row_dev = row_dev; g.capacity = capacity; g.Hkv = Hkv; g.G = G;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid(static_cast<unsigned>(B) * Hkv), block((G + 2) * 64);
    if (dtype == CQ_BF16) hipLaunchKernelGGL(cq::rope_append_kernel<cq::BF16>, grid, block, 0, st, g);
    else hipLaunchKernelGGL(cq::rope_append_kernel<cq::FP16>, grid, block, 0, st, g);
    CQ_LAUNCH_CHECK();
    return CQ_OK;
}
