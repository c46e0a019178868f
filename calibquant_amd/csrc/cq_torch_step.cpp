// Host shim between PyTorch and the C-ABI library for the steady-state decode step of one
// attention layer: the bookkeeping the eager path does per layer and token (allocate the
// query and output rows, grow the full-precision window, aim the two launches at this step's
// tensors, take torch's current stream) in one C++ call instead of ~40 lines of Python and two
// ctypes calls.  It owns no kernels: it calls `cq_rope_append` and `cq_decode_attn` with the
// same arguments the Python path passes, so the results are the same bits.
//
// What it replaces in the reference is the per-token torch op chain of one layer's decode
// branch: the (h gs d) split, `apply_rotary_pos_emb`, the `torch.cat` window growth and the
// attention over the packed state (patch_internvl.py:214-266, 304-392).
#include <torch/extension.h>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <algorithm>
#include <cstring>
#include <stdexcept>
#include <string>

#include "calibquant_hip.h"

namespace {

void check(int rc, const char* what) {
    if (rc != CQ_OK) throw std::runtime_error(std::string(what) + ": " + cq_strerror(rc));
}

class LayerStep {
  public:
    // `decode_args_addr`, `decode_args_bytes`: address and size of a filled `cq_decode_args` (the prepared call of the Python
    // path, no mask, no device row count; a chunked call brings its workspace, whose size depends on the packed
    // tokens only); it is copied.  The caller keeps the tensors it points at (packed codes, statistics,
    // workspace) alive for the life of this object.
    // cos, sin: rotary tables (rows, D) in the storage dtype.  k_win, v_win: the window buffers
    // (B, Hkv, capacity, D) whose first `len` rows are filled.  ramp: int64 device vector whose
    // cell i holds i (the row index is read on the device).
    LayerStep(uintptr_t decode_args_addr, size_t decode_args_bytes, at::Tensor cos, at::Tensor sin, at::Tensor k_win, at::Tensor v_win,
              int64_t len, at::Tensor ramp)
        : cos_(std::move(cos)), sin_(std::move(sin)), k_(std::move(k_win)), v_(std::move(v_win)),
          ramp_(std::move(ramp)), len_(len) {
        TORCH_CHECK(decode_args_bytes == sizeof(a_), "LayerStep: argument block of ", decode_args_bytes,
                    " bytes, the library's is ", sizeof(a_));
        std::memcpy(&a_, reinterpret_cast<const void*>(decode_args_addr), sizeof(a_));
        TORCH_CHECK(a_.mask == nullptr && a_.r_dev == nullptr && (a_.workspace_bytes == 0 || a_.workspace != nullptr),
                    "LayerStep: the prepared call must need no mask or device row count");
        dtype_ = a_.dtype == CQ_BF16 ? at::kBFloat16 : at::kHalf;
        TORCH_CHECK(k_.is_cuda() && k_.dim() == 4 && k_.sizes() == v_.sizes() && k_.strides() == v_.strides() &&
                        k_.stride(3) == 1 && k_.size(0) == a_.B && k_.size(1) == a_.Hkv && k_.size(3) == a_.D &&
                        k_.scalar_type() == dtype_ && v_.scalar_type() == dtype_,
                    "LayerStep: window buffers do not match the prepared call");
        TORCH_CHECK(cos_.is_cuda() && cos_.is_contiguous() && sin_.is_contiguous() && cos_.sizes() == sin_.sizes() &&
                        cos_.dim() == 2 && cos_.size(1) == a_.D && cos_.scalar_type() == dtype_ &&
                        sin_.scalar_type() == dtype_,
                    "LayerStep: rotary tables do not match the prepared call");
        TORCH_CHECK(ramp_.is_cuda() && ramp_.scalar_type() == at::kLong && ramp_.is_contiguous() && ramp_.dim() == 1,
                    "LayerStep: the row ramp must be a contiguous int64 device vector");
        TORCH_CHECK(len_ >= 0 && len_ <= k_.size(2) && a_.sprompt_len <= len_, "LayerStep: bad window length");
    }

    // One token: qkv is the fused projection output of the step (B, 1, (Hq + 2 Hkv) D) (any view of
    // that contiguous block), pos the int64 device positions (B,) or (B, 1), past_k the key window
    // the caller holds.  Returns None - and does nothing - when the step is not the steady-state one
    // (the caller then takes the general path): another window than the one this object handed out,
    // tables or ramp too short, other dtype / device / shape.  Otherwise (out (B, 1, Hq D), K, V)
    // with K, V the windows (B, Hkv, len + 1, D).
    py::object step(const at::Tensor& qkv, const at::Tensor& pos, const at::Tensor& past_k) {
        const int64_t B = a_.B, Hq = a_.Hq, Hkv = a_.Hkv, D = a_.D;
        const int64_t R = len_ + 1;
        if (pos.dim() < 1 || !qkv.is_cuda() || qkv.scalar_type() != dtype_ || !qkv.is_contiguous() ||
            qkv.numel() != B * (Hq + 2 * Hkv) * D || qkv.device() != k_.device())
            return py::none();
        if (!pos.is_cuda() || pos.scalar_type() != at::kLong || pos.device() != k_.device() || pos.size(0) != B ||
            !(pos.dim() == 1 || (pos.dim() == 2 && pos.size(1) == 1)))
            return py::none();
        if (past_k.data_ptr() != k_.data_ptr() || past_k.dim() != 4 || past_k.size(2) != len_) return py::none();
        if (R + a_.T > cos_.size(0) || R > ramp_.numel()) return py::none();
        c10::hip::HIPGuardMasqueradingAsCUDA guard(k_.device());
        if (R > k_.size(2)) grow(R);
        auto opts = qkv.options();
        at::Tensor q1 = at::empty({B, Hq, D}, opts);
        at::Tensor out = at::empty({B, 1, Hq * D}, opts);
        hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(k_.device().index()).stream();
        check(cq_rope_append(qkv.data_ptr(), a_.dtype, a_.B, a_.Hq, a_.Hkv, a_.D, cos_.data_ptr(), sin_.data_ptr(),
                             cos_.size(0), pos.data_ptr<int64_t>(), pos.stride(0), q1.data_ptr(), k_.data_ptr(),
                             v_.data_ptr(), k_.stride(0), k_.stride(1), k_.stride(2), static_cast<int>(k_.size(2)),
                             ramp_.data_ptr<int64_t>() + len_, stream),
              "cq_rope_append");
        a_.q = q1.data_ptr();
        a_.out = out.data_ptr();
        a_.k_res = k_.data_ptr();
        a_.v_res = v_.data_ptr();
        a_.R = static_cast<int>(R);
        a_.res_stride_b = k_.stride(0);
        a_.res_stride_h = k_.stride(1);
        a_.res_stride_r = k_.stride(2);
        check(cq_decode_attn(&a_, stream), "cq_decode_attn");
        len_ = R;
        ++steps_;
        return py::make_tuple(out, k_.narrow(2, 0, R), v_.narrow(2, 0, R));
    }

    int64_t length() const { return len_; }
    int64_t steps() const { return steps_; }
    int64_t capacity() const { return k_.size(2); }

  private:
    // New buffers with head-room; the rows held so far are copied once (the reference copies the
    // whole window on every step, patch_internvl.py:264-266).
    void grow(int64_t need) {
        const int64_t cap = need + std::max<int64_t>(256, need / 8);
        at::Tensor k = at::empty({k_.size(0), k_.size(1), cap, k_.size(3)}, k_.options());
        at::Tensor v = at::empty_like(k);
        if (len_ > 0) {
            k.narrow(2, 0, len_).copy_(k_.narrow(2, 0, len_));
            v.narrow(2, 0, len_).copy_(v_.narrow(2, 0, len_));
        }
        k_ = std::move(k);
        v_ = std::move(v);
    }

    cq_decode_args a_;
    at::ScalarType dtype_;
    at::Tensor cos_, sin_, k_, v_, ramp_;
    int64_t len_;
    int64_t steps_ = 0;
};

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "steady-state decode step of one attention layer over the calibquant C-ABI library";
    py::class_<LayerStep>(m, "LayerStep")
        .def(py::init<uintptr_t, size_t, at::Tensor, at::Tensor, at::Tensor, at::Tensor, int64_t, at::Tensor>())
        .def("step", &LayerStep::step)
        .def_property_readonly("length", &LayerStep::length)
        .def_property_readonly("steps", &LayerStep::steps)
        .def_property_readonly("capacity", &LayerStep::capacity);
    m.def("library_version", []() { return cq_version(); });
}
