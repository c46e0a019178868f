/* calibquant_hip.h - C ABI of the MI355X (gfx950) CalibQuant kernels.
 *
 * Plain pointers and sizes only.  All pointers are device pointers unless the
 * comment says otherwise.  No function allocates, frees or synchronises; every
 * launch goes to `stream` (a hipStream_t passed as an opaque pointer, NULL =
 * the default stream).  Return value: CQ_OK (0) or a negative CQ_ERR_* code;
 * cq_strerror() names it and cq_last_hip_error() returns the hipError_t of the
 * last failed runtime call made on the calling host thread.
 *
 * Storage dtypes: CQ_BF16 or CQ_FP16 (16-bit).  "Storage-dtype arithmetic"
 * means fp32 compute with a round-to-nearest-even cast after every operation,
 * which is how the reference's torch op chains behave on 16-bit tensors.
 *
 * Each entry point names the reference interface it replaces
 * (paths relative to the reference checkout).
 */
#ifndef CALIBQUANT_HIP_H
#define CALIBQUANT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* cq_stream_t; /* hipStream_t */

enum cq_dtype { CQ_BF16 = 0, CQ_FP16 = 1, CQ_FP32 = 2, CQ_I64 = 3, CQ_I32 = 4, CQ_U8 = 5 };

enum cq_status {
    CQ_OK = 0,
    CQ_ERR_NULL = -1,        /* a required pointer is NULL */
    CQ_ERR_SHAPE = -2,       /* a dimension is out of the supported range */
    CQ_ERR_DTYPE = -3,       /* dtype code not accepted by this entry point */
    CQ_ERR_ALIGN = -4,       /* pointer or stride not 16-byte aligned */
    CQ_ERR_WORKSPACE = -5,   /* workspace missing or too small */
    CQ_ERR_LAUNCH = -6,      /* the HIP runtime reported an error */
    CQ_ERR_UNSUPPORTED = -7, /* valid request that this build does not cover */
    CQ_ERR_SCRATCH_LIMIT = -8 /* cq_decode_attn_static: the request needs more scratch than the static buffer holds */
};

int cq_version(void);
const char* cq_strerror(int status);
int cq_last_hip_error(void);

/* ------------------------------------------------------------------------
 * Prefill: per-channel min-max quantise + bit-pack of one K or V tensor.
 * Replaces the chain quant() -> LUT/index build -> encode():
 *   calibquant.py:24-42 (quant, per_channel=True, post_scale=True),
 *   patch_internvl.py:292,297 (call sites), :318-329 (LUT indices),
 *   calibquant.py:114-137 (encode), patch_internvl.py:332,339.
 *
 * x      (B, T, H, D) view in storage dtype; element strides stride_b/t/h,
 *        D contiguous.  D in {64, 128, 256}; strides multiples of 8.
 * bits   1 or 2.  clip = the reference's SCALE_K / SCALE_V factor.
 * codes  uint8 (B, H, T, D*bits/8), first channel in the most significant bits.
 * scale, zero   storage dtype, (B, H, D); bit-identical to the reference's
 *        storage-dtype arithmetic, including scale 0 / zero -inf|NaN for a
 *        constant channel (whose codes are 0, as in the reference).
 * workspace     cq_quantize_pack_workspace(B, T, H, D) bytes, 16-byte aligned.
 * Inputs must not contain NaN. */
size_t cq_quantize_pack_workspace(int B, int T, int H, int D);
int cq_quantize_pack(const void* x, int dtype, int B, int T, int H, int D,
                     int64_t stride_b, int64_t stride_t, int64_t stride_h,
                     int bits, float clip,
                     uint8_t* codes, void* scale, void* zero,
                     void* workspace, size_t workspace_bytes, cq_stream_t stream);

/* With D = 128 and more than 3 328 tokens (what one workgroup's registers hold of a slice of 32 channels),
 * cq_quantize_pack still reads x once: two to thirty-two workgroups of its persistent launch share a slice along
 * the token axis and exchange the channels' minima and maxima through the workspace inside the launch.  The wait
 * for the other parts is bounded: after `polls` polls (about a microsecond each; default 262 144) a workgroup goes
 * on with what it has and sets a word of pinned host memory (64 bytes per device, allocated at the first such
 * call outside a stream capture and kept until the process ends).  The next such call on that device then returns
 * CQ_ERR_LAUNCH once (the previous call's output is not valid) and the process goes on with three launches per
 * tensor (partial min / max, statistics, emit; x read twice).  This call sets the bound (polls >= 0; it also
 * re-enables the single launch after a give-up) and returns the previous one; polls < 0 only queries.  No
 * counterpart in the reference, whose quant() is a chain of whole-tensor torch ops (calibquant.py:24-42). */
int cq_quantize_pack_wait_polls(int polls);

/* ------------------------------------------------------------------------
 * Prefill, keys: rotary embedding fused into the quantise-and-pack pass.
 * Replaces, for the image slice of the key tensor, the rotary embedding of
 * the whole key tensor (patch_internvl.py:258-260 with :119-138) followed by
 * cq_quantize_pack's chain (:295-297, 325-339): x is the UN-rotated key
 * block (B, T, H, 128) of the fused projection output; every row is rotated
 * as it arrives, rnd(rnd(x*cos) + rotate_half(x)*sin) with the product added
 * in fp32 (the arithmetic of `copy_().mul_()` + `addcmul_`, :125-128), the
 * rotated row is written once to x_rot (the prefill attention and the cache
 * of the remaining tokens need it) and quantised from the registers: the keys
 * are read from HBM once and nothing is read back.
 * cos_table, sin_table: (table_rows, 128), storage dtype, 16-byte aligned.
 * pos: device int64, position id of (b, t) at pos[b*pos_stride_b +
 * t*pos_stride_t] (clamped to the table), or NULL for positions pos0 + t.
 * x_rot: (B, T, H, 128) through element strides (multiples of 8).
 * codes / scale / zero / workspace as for cq_quantize_pack; the results are
 * bit-identical to cq_quantize_pack on the rotated tensor.
 * Shapes outside the one-pass path (T > 3 328, D != 128) return
 * CQ_ERR_UNSUPPORTED: rotate with cq_rope_rows, then cq_quantize_pack. */
int cq_rope_quantize_pack(const void* x, int dtype, int B, int T, int H, int D,
                          int64_t stride_b, int64_t stride_t, int64_t stride_h,
                          const void* cos_table, const void* sin_table, int64_t table_rows,
                          const int64_t* pos, int64_t pos_stride_b, int64_t pos_stride_t, int64_t pos0,
                          void* x_rot, int64_t rot_stride_b, int64_t rot_stride_t, int64_t rot_stride_h,
                          int bits, float clip, uint8_t* codes, void* scale, void* zero,
                          void* workspace, size_t workspace_bytes, cq_stream_t stream);

/* The rotary embedding alone, same arithmetic, for the rows that are not
 * quantised (queries; system-prompt and text keys): x (B, T, H, 128) through
 * strides -> x_rot (B, T, H, 128) through strides; one launch instead of the
 * reference's chain of torch ops over the whole tensor
 * (patch_internvl.py:119-138). */
int cq_rope_rows(const void* x, int dtype, int B, int T, int H, int D,
                 int64_t stride_b, int64_t stride_t, int64_t stride_h,
                 const void* cos_table, const void* sin_table, int64_t table_rows,
                 const int64_t* pos, int64_t pos_stride_b, int64_t pos_stride_t, int64_t pos0,
                 void* x_rot, int64_t rot_stride_b, int64_t rot_stride_t, int64_t rot_stride_h,
                 cq_stream_t stream);
/* The same over x (B, T, H, G, 128): every head a group of G rows `stride_g` elements apart
 * (`rot_stride_g` in x_rot) - the query block of the fused projection output, (h gs d) with the
 * G query heads of a kv head side by side (patch_internvl.py:219-234), in one launch. */
int cq_rope_rows_grouped(const void* x, int dtype, int B, int T, int H, int G, int D,
                         int64_t stride_b, int64_t stride_t, int64_t stride_h, int64_t stride_g,
                         const void* cos_table, const void* sin_table, int64_t table_rows,
                         const int64_t* pos, int64_t pos_stride_b, int64_t pos_stride_t, int64_t pos0,
                         void* x_rot, int64_t rot_stride_b, int64_t rot_stride_t, int64_t rot_stride_h,
                         int64_t rot_stride_g, cq_stream_t stream);

/* ------------------------------------------------------------------------
 * Per-token value quantiser: the reference's
 * triton_quantize_and_pack_along_last_dim(data, group_size, bit)
 * (qjl/new_pack.py:53-82), the source of the `v_mode = token` layout that
 * cq_decode_attn reads with CQ_V_PER_TOKEN.  x: (B, T, H, D) through element
 * strides (D contiguous, D = 128, group_size = 32); for every token and group
 * of 32 channels: minimum, scale = (max - min) / (2^bits - 1), code =
 * round(clamp((x - min) / scale, 0, 2^bits - 1)), each op rounded to the
 * storage dtype; 32/bits codes per int32 word, first code in the lowest bits
 * (new_pack.py:7-28).  Outputs in (b, h, t) row order: words
 * (B, H, T, D*bits/32), scale and mins (B, H, T, D/32) in the storage dtype.
 * A value is scale*code + min (quantization.cu:116-117). */
int cq_quantize_pack_token(const void* x, int dtype, int B, int T, int H, int D, int64_t stride_b,
                           int64_t stride_t, int64_t stride_h, int bits, int group_size, int32_t* words,
                           void* scale, void* mins, cq_stream_t stream);

/* quant() itself, for callers that keep the reference's unfused call sequence
 * (calibquant.py:24-42 with per_channel=True, post_scale=True).  x_q is a
 * contiguous (B, T, H, D) tensor of storage dtype holding the integer codes
 * (NaN where the reference yields NaN); scale, zero as above. */
int cq_quant(const void* x, int dtype, int B, int T, int H, int D,
             int64_t stride_b, int64_t stride_t, int64_t stride_h,
             int bits, float clip,
             void* x_q, void* scale, void* zero,
             void* workspace, size_t workspace_bytes, cq_stream_t stream);

/* quant() with per_channel=False (calibquant.py:29-31): one minimum and one
 * maximum over the whole tensor (`x.min() * scale`, `x.max() * scale`), then
 * the same op chain as above.  x and x_q as for cq_quant; scale1 and zero1
 * receive a single storage-dtype element each (the reference returns 0-d
 * tensors).  Not called by the attention path (patch_internvl.py:181,187 pass
 * per_channel=True); provided so that the operator's whole signature works.
 * workspace: cq_quantize_pack_workspace(B, T, H, D) bytes. */
int cq_quant_tensor(const void* x, int dtype, int B, int T, int H, int D,
                    int64_t stride_b, int64_t stride_t, int64_t stride_h,
                    int bits, float clip,
                    void* x_q, void* scale1, void* zero1,
                    void* workspace, size_t workspace_bytes, cq_stream_t stream);

/* encode(): pack `rows` rows of D integer indices, 8/bits per byte,
 * first index in the most significant bits (calibquant.py:114-137).
 * idx_dtype: CQ_I64, CQ_I32, CQ_U8, or CQ_BF16/CQ_FP16 numbers holding
 * integers.  Only the low `bits` bits of each index are kept. */
int cq_encode(const void* idx, int idx_dtype, int64_t rows, int D, int bits,
              uint8_t* out, cq_stream_t stream);

/* fused_kernel(): c[m, t] = sum_d a[m, d] * lut[code[m, t, d]], fp32
 * accumulation, fp16 output (calibquant.py:54-111).  a: (M, D) in a_dtype
 * (CQ_BF16/CQ_FP16/CQ_FP32); enc: (M, T, D*bits/8); lut: lut_len entries in
 * lut_dtype (the reference's table holds the levels found in the first
 * 10 000 codes, patch_internvl.py:318-329, so it may be shorter than 2^bits:
 * a code without an entry contributes 0 and nothing past the table is read);
 * out: (M, T) fp16.  M < 2^31, T <= 65 535 * 256. */
int cq_lut_vecmat_qk(const void* lut, int lut_dtype, int lut_len, const void* a, int a_dtype,
                     const uint8_t* enc, int64_t M, int T, int D, int bits,
                     void* out_fp16, cq_stream_t stream);

/* fused_kernel_wv(): c[m, d] = sum_t a[m, t] * lut[code[m, t, d]], fp32
 * accumulation, fp16 output (calibquant.py:192-276).  a: (M, T);
 * enc: (M, T, D*bits/8); out: (M, D) fp16. */
int cq_lut_vecmat_pv(const void* lut, int lut_dtype, int lut_len, const void* a, int a_dtype,
                     const uint8_t* enc, int64_t M, int T, int D, int bits,
                     void* out_fp16, cq_stream_t stream);

/* value quantisation layouts understood by cq_decode_attn (cq_decode_args.v_mode) */
enum cq_v_mode { CQ_V_PER_CHANNEL = 0, CQ_V_PER_TOKEN = 1 };

/* ------------------------------------------------------------------------
 * Decode: one fused attention step over packed image K/V plus the
 * full-precision residual window.  Replaces the whole decode branch
 * patch_internvl.py:344-436: repeat_kv copies (:352-353, 361-362), residual
 * logits (:365-366), post-scaled image logits through fused_kernel
 * (:369-373), calibration (:376-385), concatenation [sys | image | text]
 * (:388), additive mask (:404-410), softmax (:413), fused_kernel_wv and value
 * post-scaling (:418-425), residual outputs and their sum (:428-436).
 * Arithmetic is fp32 with one final rounding to the storage dtype. */
typedef struct cq_decode_args {
    /* query, (B, Hq, D) contiguous, storage dtype; D must be 128 */
    const void* q;
    /* packed codes, uint8 (B, Hkv, T, D*bits/8) contiguous */
    const uint8_t* codes_k;
    const uint8_t* codes_v;
    /* per-channel statistics, storage dtype, (B, Hkv, D) contiguous */
    const void* k_scale;
    const void* k_zero;
    const void* v_scale;
    const void* v_zero;
    /* residual window, storage dtype, (B, Hkv, R, D) with element strides
     * res_stride_b/h/r (D contiguous; strides multiples of 8).  Rows
     * [0, sprompt_len) precede the image block, the rest follow it. */
    const void* k_res;
    const void* v_res;
    int64_t res_stride_b, res_stride_h, res_stride_r;
    /* optional additive mask, fp32, row b at mask + b*mask_stride_b, indexed
     * over the [sys | image | text] order (length sprompt_len + T + R - sprompt_len) */
    const float* mask;
    int64_t mask_stride_b;
    /* output, (B, Hq, D) contiguous, storage dtype */
    void* out;
    /* cq_decode_attn_workspace() bytes, 16-byte aligned; may be NULL if that is 0 */
    void* workspace;
    size_t workspace_bytes;
    int dtype;          /* CQ_BF16 or CQ_FP16 */
    int B, Hq, Hkv, D;
    int T;              /* packed (image) tokens, may be 0 */
    int R;              /* residual rows, may be 0 (T + R > 0) */
    int sprompt_len;    /* 0 <= sprompt_len <= R */
    int bits;           /* 1 or 2 */
    int calibrate;      /* non-zero: apply the logit calibration */
    float calib_off_max;   /* reference: -3 */
    float calib_off_min;   /* reference:  0 */
    int force_splits;   /* 0 = choose; >0 = split the T axis into this many chunks */
    /* Optional: device pointer to the number of residual rows.  When not NULL
     * the kernels read the row count from it at run time (0 <= *r_dev <= R,
     * sprompt_len <= *r_dev) and R above is only the capacity of the window
     * buffers.  A caller that replays a recorded launch (a HIP graph of a
     * decode step) grows the window this way without changing the launch:
     * the reference re-reads the window's length from the tensor shape on
     * every step (patch_internvl.py:246-251,265-266), which a recorded
     * launch cannot.  Must be NULL when a mask is given. */
    const int32_t* r_dev;
    /* How the values were quantised (enum cq_v_mode).  CQ_V_PER_CHANNEL (0):
     * CalibQuant's per-channel statistics, fields as described above.
     * CQ_V_PER_TOKEN: the per-token layout of cq_quantize_pack_token (the
     * reference's qjl/new_pack.py:53-82, consumed by quantization.cu:67-132):
     * codes_v then holds int32 words (B, Hkv, T, D*bits/32), first channel in
     * the lowest bits; v_scale and v_zero hold the scale and the minimum,
     * storage dtype, (B, Hkv, T, D/32); a value is scale*code + minimum. */
    int v_mode;
} cq_decode_args;

size_t cq_decode_attn_workspace(const cq_decode_args* args);
int cq_decode_attn(const cq_decode_args* args, cq_stream_t stream);

/* cq_decode_attn for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * It has no counterpart in the reference, whose operators allocate their
 * outputs and temporaries with torch on every call.  Same arguments and the
 * same kernels as cq_decode_attn, except that args->workspace /
 * workspace_bytes are ignored: the scratch of the chunked path (per-chunk
 * logit min / max, the flash-decoding partials and their counters, and - where
 * the plan hands the first launch's logits to the second through a buffer
 * (2 bits, or fewer than four heads per unit) and it fits beside them - those)
 * lives in a static device array of cq_decode_attn_static_limit() bytes
 * (8 MiB) inside the library; every GPU the library runs on holds its own
 * copy until the process ends.  When the logits do not fit, the second launch
 * recomputes them (same results, more work).  A request whose plan needs more
 * than the limit even so returns CQ_ERR_SCRATCH_LIMIT and launches nothing
 * (batch 8 x 32 768 tokens needs 1.2 MiB; at 2 bits 33 MiB more with the logits).
 * The call allocates and frees nothing and does not synchronise.  Nothing in
 * the scratch has to start at zero: every word a launch reads was written by
 * an earlier launch of the same call (the first launch clears the counters).  All calls on one GPU share that GPU's array, so two calls that
 * may overlap on one GPU (different streams, or one stream per host thread)
 * race on it: keep them on one stream, or give the overlapping ones
 * cq_decode_attn with workspaces of their own. */
size_t cq_decode_attn_static_limit(void);
int cq_decode_attn_static(const cq_decode_args* args, cq_stream_t stream);

/* What cq_decode_attn would launch for these arguments (pointers are not
 * looked at; nothing is launched - the only device call is a query of the
 * current device's compute-unit count, made once per process; a whole MI355X,
 * 256 units, is assumed when there is no device).  No counterpart in the reference,
 * whose Triton kernels re-autotune per shape (calibquant.py:54-76,192-218):
 * here the choice is a pure function of the shape, and a caller can read it. */
typedef struct cq_decode_plan {
    int threads;          /* threads per workgroup: 1024, or 512 with two workgroups per compute unit */
    int heads_per_unit;   /* query heads served by one workgroup (they share a kv head) */
    int chunks;           /* token chunks per (batch, kv head, head group); > 1: the chunks' logit min / max are exchanged
                           * and their partial results merged - in a launch of their own ahead of the main one (launches == 2),
                           * or inside a single launch when every chunk's workgroup fits the device at once (launches == 1) */
    int chunk_tokens;     /* packed tokens per chunk */
    int launches;         /* 1 or 2 (what the plan asks for; see cq_decode_attn_wait_polls for when one becomes two) */
    int lds_bytes;        /* dynamic LDS of the main launch */
    int register_logits;  /* > 0: a thread keeps the logits of up to this many of its tokens in registers (fp32)
                           * and the token slots in LDS hold only exp(.) as fp16; 0: fp32 logits wait in the slots */
} cq_decode_plan;
int cq_decode_attn_plan(const cq_decode_args* args, cq_decode_plan* plan);

/* The single-launch chunked step (plan: chunks > 1, launches == 1) makes the workgroups of a unit wait for each
 * other's logit min / max inside the launch.  That is only sound while they are all resident together, which the
 * plan works out from the device's compute-unit count; the wait is therefore bounded: after `polls` polls (about a
 * microsecond each; default 262 144) a workgroup gives up, ends without a result and sets a word of pinned host
 * memory (64 bytes per device, allocated at the first such call outside a stream capture - the one allocation
 * this library makes - and kept until the process ends).  The next chunked cq_decode_attn on that device then
 * returns CQ_ERR_LAUNCH once (the previous step's output is not valid) and the process goes on with two launches
 * per step.  cq_decode_attn_static always takes two launches.  This call sets the bound (polls >= 0; it also
 * re-enables the single launch after a give-up) and returns the previous one; polls < 0 only queries.
 * No counterpart in the reference (its kernels never split the token axis). */
int cq_decode_attn_wait_polls(int polls);
/* 1 while a give-up is flagged on some device and no cq_decode_attn call has reported it yet, else 0; a read
 * of host memory, no device call.  For callers that replay a recorded single-launch step (a HIP graph) and so
 * never pass through the check inside cq_decode_attn: ask after synchronising with the replays.  A launch
 * whose workgroups gave up leaves the workspace as a finished one does, so later replays are not affected by
 * it.  No counterpart in the reference. */
int cq_decode_attn_gave_up(void);
/* Process-wide switch for the single-launch chunked step (enable != 0: plans may ask for it, the default;
 * 0: chunked shapes always take two launches - for a process that shares the GPU's compute units with
 * other work, e.g. through compute-unit masks the plan cannot see; enable < 0 only queries).  Returns the
 * previous setting.  cq_decode_attn_plan / cq_decode_attn_workspace follow it: size the workspace after
 * the last change.  No counterpart in the reference. */
int cq_decode_attn_single_launch(int enable);

/* ------------------------------------------------------------------------
 * Decode-step glue, one launch per layer and token: the (h gs d) split of
 * the fused wqkv output (patch_internvl.py:219-234), rotary embedding of the
 * query and key heads (patch_internvl.py:119-138, 258-260) with the rounding
 * of the ops that run there: x*cos rounded to the storage dtype
 * (`copy_().mul_()`, :125), then rotate_half(x)*sin added in fp32 and the sum
 * rounded once (`addcmul_`, :127) - not the two-rounding form of the
 * commented-out line :123 - and the append of the new key / value row to the
 * full-precision window (the reference's torch.cat, patch_internvl.py:264-266).
 * qkv: (B, Hkv, Hq/Hkv + 2, D) contiguous, one token per sample; cos_table,
 * sin_table: (table_rows, D) in the storage dtype; pos: device int64,
 * sample b at pos[b*pos_stride] (a position outside [0, table_rows) is
 * clamped to the nearest table row without an error: the caller sizes the
 * tables to cover the positions it passes); q_out: (B, Hq, D)
 * contiguous; k_win, v_win: (B, Hkv, capacity, D) through element strides;
 * row_dev: device int64, the window row that receives the new key / value
 * (if it is outside [0, capacity) the key / value row is dropped without an
 * error: the caller keeps the row inside the window).  Position and row are
 * read on the device, so a recorded launch can be replayed. */
int cq_rope_append(const void* qkv, int dtype, int B, int Hq, int Hkv, int D,
                   const void* cos_table, const void* sin_table, int64_t table_rows,
                   const int64_t* pos, int64_t pos_stride, void* q_out,
                   void* k_win, void* v_win, int64_t win_stride_b, int64_t win_stride_h,
                   int64_t win_stride_r, int capacity, const int64_t* row_dev, cq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* CALIBQUANT_HIP_H */
