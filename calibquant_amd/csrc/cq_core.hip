// Library-level entry points: version, error strings, last HIP error.
#include "cq_common.h"

namespace cq {
thread_local int g_last_hip_error = 0;
}

extern "C" {

int cq_version(void) { return 105; }   // 105: chunked decode in two launches (merge inside the main launch; workspace holds counters and, where used, logits); 104: cq_rope_quantize_pack, cq_rope_rows; 103: cq_decode_attn_static; 102: lut_len argument of the look-up vec-mats, cq_quant_tensor

const char* cq_strerror(int status) {
    switch (status) {
        case CQ_OK: return "ok";
        case CQ_ERR_NULL: return "required pointer is NULL";
        case CQ_ERR_SHAPE: return "dimension out of the supported range";
        case CQ_ERR_DTYPE: return "dtype not accepted by this entry point";
        case CQ_ERR_ALIGN: return "pointer or stride not 16-byte aligned";
        case CQ_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case CQ_ERR_LAUNCH: return "HIP runtime error (see cq_last_hip_error)";
        case CQ_ERR_UNSUPPORTED: return "request not covered by this build";
        case CQ_ERR_SCRATCH_LIMIT: return "request needs more scratch than the library's static device buffer holds (cq_decode_attn_static_limit)";
        default: return "unknown status";
    }
}

int cq_last_hip_error(void) { return cq::g_last_hip_error; }

}  // extern "C"
