/*
 * C ABI of the MI355X (gfx950) flash-attention library.
 *
 * Every entry point is extern "C", takes plain pointers / sizes / strides and
 * returns an int that carries a hipError_t value.  No C++ or torch types cross
 * this boundary.  Each declaration names the reference interface it stands in
 * for (paths relative to the reference tree).
 *
 * Conventions kept from the reference:
 *   - tensors are views: device pointer + sizes + strides (in elements) + dtype
 *     (include/aotriton/util.h:77-158); the last stride must be 1;
 *   - philox seed/offset and the persistent counter are DEVICE pointers
 *     (include/aotriton/flash.h:113-120);
 *   - launches are asynchronous on the caller's stream, nothing is synchronised;
 *   - device memory comes from the caller, directly or through its lazy-tensor
 *     callbacks (include/aotriton/util.h:224-246).
 * One departure from the last point: the library keeps one workspace buffer per device
 * (fa_set_bwd_workspace_limit below: what it is for, how it is bounded, how to switch it
 * off).  Calls on a stream under capture and fa_attn_bwd_noalloc never touch it.
 */
#ifndef AOTRITON_AMD_FLASH_H
#define AOTRITON_AMD_FLASH_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define FA_API __attribute__((visibility("default")))
#else
#define FA_API
#endif

/* include/aotriton/dtypes.h:12-25 -- same integer values. */
enum fa_dtype {
  FA_DTYPE_UNKNOWN = 0,
  FA_DTYPE_FLOAT32 = 1,
  FA_DTYPE_FLOAT16 = 2,
  FA_DTYPE_BFLOAT16 = 3,
  FA_DTYPE_INT8 = 10,
  FA_DTYPE_INT16 = 11,
  FA_DTYPE_INT32 = 12,
  FA_DTYPE_INT64 = 13,
  FA_DTYPE_UINT8 = 20,
  FA_DTYPE_UINT16 = 21,
  FA_DTYPE_UINT32 = 22,
  FA_DTYPE_UINT64 = 23,
};

/* hipError_t values this library returns (include/hip/hip_runtime_api.h); the
 * meaning of each follows python/codegen/template/shim.cc:72-100 and
 * modules/flash/csrc/attn_fwd.cc:53-55. */
enum fa_error {
  FA_SUCCESS = 0,
  FA_ERROR_INVALID_VALUE = 1,             /* null / inconsistent tensor views            */
  FA_ERROR_OUT_OF_MEMORY = 2,             /* fa_attn_bwd_noalloc: more rows than its array holds */
  FA_ERROR_INVALID_SYMBOL = 13,           /* params_version mismatch                     */
  FA_ERROR_NO_BINARY_FOR_GPU = 209,       /* device is not gfx950                        */
  FA_ERROR_PEER_ACCESS_UNSUPPORTED = 217, /* a forced backend cannot take this input     */
  FA_ERROR_NOT_SUPPORTED = 801,           /* functional not built (head dim > 512, stride, ..) */
};

/* TensorView<4|2|1|0>, include/aotriton/util.h:77-210. */
typedef struct fa_tensor4 {
  void* ptr;
  uint64_t sizes[4];
  uint64_t strides[4];
  int32_t dtype;
} fa_tensor4;

typedef struct fa_tensor2 {
  void* ptr;
  uint64_t sizes[2];
  uint64_t strides[2];
  int32_t dtype;
} fa_tensor2;

typedef struct fa_tensor1 {
  void* ptr;
  uint64_t sizes[1];
  uint64_t strides[1];
  int32_t dtype;
} fa_tensor1;

typedef struct fa_tensor0 {
  void* ptr;
  int32_t dtype;
} fa_tensor0;

/* LazyTensor<2|4>, include/aotriton/util.h:224-246.  `eager.ptr != NULL` means
 * the caller already owns the buffer; otherwise `acquire` is called at most once
 * and only if the chosen backend reads the tensor; `dispose` is called before the
 * entry point returns iff `acquire` ran (modules/flash/csrc/attn_bwd.cc:157-158).
 * acquire fills *out and returns 0 on success. */
typedef struct fa_lazy_tensor2 {
  void* cookie;
  int (*acquire)(struct fa_lazy_tensor2* self, fa_tensor2* out);
  void (*dispose)(struct fa_lazy_tensor2* self);
  fa_tensor2 eager;
} fa_lazy_tensor2;

typedef struct fa_lazy_tensor4 {
  void* cookie;
  int (*acquire)(struct fa_lazy_tensor4* self, fa_tensor4* out);
  void (*dispose)(struct fa_lazy_tensor4* self);
  fa_tensor4 eager;
} fa_lazy_tensor4;

/* attn_options, include/aotriton/flash.h:38-41.
 * Backward backends: 0 = split (the reference's preprocess + dK/dV + dQ; here dQ,
 * which also computes delta and writes it to params->D, then dK/dV; fp32 tensors and
 * head dims above 256 launch a delta kernel first), 1 = fused single launch
 * (modules/flash/aot/__init__.py:83-85).  Index 2 (prebuilt assembly
 * backend of the reference) does not exist here and is rejected with
 * FA_ERROR_PEER_ACCESS_UNSUPPORTED.  Forward has backend 0 only. */
typedef struct fa_options {
  int32_t force_backend_index; /* -1 = library's choice */
  int32_t deterministic;       /* every backend here is deterministic */
} fa_options;

/* include/aotriton/flash.h:72-94 */
#define FA_CAUSAL_NONE 0
#define FA_CAUSAL_WINDOWED 3
#define FA_WINDOW_TOP_LEFT (-2147483647)
#define FA_WINDOW_BOTTOM_RIGHT (-2147483646)
#define FA_VARLEN_NONE 0
#define FA_VARLEN_COMPACT 1
#define FA_VARLEN_PADDED 2
#define FA_VARLEN_STRIDED 3

#define FA_FWD_PARAMS_VERSION 3 /* attn_fwd_params::kVersion, flash.h:128 */
#define FA_BWD_PARAMS_VERSION 6 /* attn_bwd_params::kVersion, flash.h:172 */

/* attn_fwd_params, include/aotriton/flash.h:96-130 (same members, same order). */
typedef struct fa_fwd_params {
  fa_tensor4 Q;   /* (B, Hq, Sq, D)   compact varlen: (1, Hq, total_q, D) */
  fa_tensor4 K;   /* (B, Hk, Sk, D) */
  fa_tensor4 V;   /* (B, Hk, Sk, Dv) */
  fa_tensor4 B;   /* additive bias (B, Hq, Sq, Sk) or null */
  fa_tensor2 A;   /* alibi slopes: unused, must be null */
  float Sm_scale;
  fa_tensor2 L;   /* fp32 log-sum-exp (B*Hq, Sq) | varlen (Hq, total_q); may be null */
  fa_tensor4 Out; /* (B, Hq, Sq, Dv) */
  fa_tensor1 cu_seqlens_q; /* int32[num_seqlens+1] or null */
  fa_tensor1 cu_seqlens_k;
  int32_t Max_seqlen_q;
  int32_t Max_seqlen_k;
  fa_tensor1 seq_strides_q; /* strided varlen only */
  fa_tensor1 seq_strides_k;
  float dropout_p;
  fa_tensor0 philox_seed_ptr; /* device uint64 */
  fa_tensor0 philox_offset1;  /* device uint64 */
  uint64_t philox_offset2;
  fa_tensor0 philox_seed_output;   /* nullable */
  fa_tensor0 philox_offset_output; /* nullable */
  fa_tensor4 encoded_softmax;      /* nullable; filled with +-0.5 keep mask */
  fa_tensor0 persistent_atomic_counter; /* device int32, zero on entry; optional here */
  int8_t causal_type;
  int8_t varlen_type;
  int32_t window_left;
  int32_t window_right;
} fa_fwd_params;

/* attn_bwd_params, include/aotriton/flash.h:138-174. */
typedef struct fa_bwd_params {
  fa_tensor4 Q;
  fa_tensor4 K;
  fa_tensor4 V;
  fa_tensor4 B;
  float Sm_scale;
  fa_tensor4 Out;
  fa_tensor4 DO;
  fa_tensor4 DK;
  fa_tensor4 DV;
  fa_tensor4 DQ;
  fa_tensor4 DB; /* nullable */
  fa_tensor2 L;
  fa_lazy_tensor2 D; /* delta; read/written by the split backend only */
  fa_tensor1 cu_seqlens_q;
  fa_tensor1 cu_seqlens_k;
  int32_t Max_seqlen_q;
  int32_t Max_seqlen_k;
  fa_tensor1 seq_strides_q;
  fa_tensor1 seq_strides_k;
  float dropout_p;
  fa_tensor0 philox_seed_ptr;
  fa_tensor0 philox_offset1;
  uint64_t philox_offset2;
  int8_t causal_type;
  int8_t varlen_type;
  int32_t window_left;
  int32_t window_right;
  fa_lazy_tensor4 DQ_ACC; /* never acquired: the dQ path has a single owner per tile */
} fa_bwd_params;

/* What the compile-time tile table selected for a call; stands in for peeking at
 * the reference's debug log (modules/flash/csrc/attn_fwd.cc:15-17). */
typedef struct fa_kernel_config {
  int32_t block_m;
  int32_t block_n;
  int32_t num_waves;
  int32_t lds_bytes;
  int32_t grid[3];
  int32_t backend_index;
  int32_t head_dim;
  int32_t flags; /* bit0 causal/windowed, bit1 bias, bit2 dropout, bit3 varlen, bit4 (backward) dS kept in HBM, bit5 runs on packed copies */
} fa_kernel_config;

/* The MFMA kernels read rows made of aligned 16-byte pieces; the test is the same for every element
 * type: head dims and strides that are multiples of 8 ELEMENTS and 16-byte aligned bases (for fp32
 * that is stricter than 16 bytes: an fp32 head dim of 12 or 36 fails it).  A call with a tensor that
 * fails it runs on packed copies (contiguous, head dim rounded up to a multiple of 8 with zeros) that
 * the library makes in its workspace (fa_set_bwd_workspace_limit below), results copied back: the
 * MFMA kernels plus one pass over each tensor.  Without workspace (limit too small or 0, a stream
 * under capture, fa_attn_bwd_kernel, fa_attn_bwd_noalloc) it runs on element-wise vector-ALU
 * kernels: same results, a few TFLOP/s.  fa_query_*_config sets bit 5 of `flags` for the former. */
/* v2::flash::check_gpu -- modules/flash/csrc/attn_check.cc:36-46.
 * FA_SUCCESS on gfx950, FA_ERROR_NO_BINARY_FOR_GPU otherwise. */
FA_API int fa_check_gpu(void* hip_stream);

/* v3::flash::attn_fwd -- include/aotriton/flash.h:132-136,
 * modules/flash/csrc/attn_fwd.cc:48-149.
 * Head dims 1..512 (Dqk of Q and K, Dv of V and Out may differ), rounded up to a built one with the
 * excess columns masked (attn_fwd.cc:76-82).  Tensors whose rows are made of aligned 16-byte pieces
 * (head dims and strides multiples of 8 elements, 16-byte aligned bases) run on the MFMA kernels as
 * they are, anything else through packed copies or on element-wise kernels (see above).  A bias is
 * (batch of Q, Hq, Max_seqlen_q, Max_seqlen_k); with cu_seqlens its batch index is the sequence for
 * the padded layout and 0 for packed tokens, rows and columns count from the sequence's start
 * (modules/flash/kernel/fwd_kernel.py:393-395). */
FA_API int fa_attn_fwd(const fa_fwd_params* params, int32_t params_version,
                       void* hip_stream, const fa_options* options);

/* v3::flash::attn_bwd -- include/aotriton/flash.h:176-180,
 * modules/flash/csrc/attn_bwd.cc:55-160.
 * Same tensors as the forward.  Single-launch kernels (backend 1) exist for fp16/bf16 up to head dim
 * 256.  For fp32 tensors and head dims above 256 backend 1 runs the split kernels: with params->D when
 * the caller brings one, else with delta in the library's workspace; tensors whose rows are not aligned
 * 16-byte pieces reach either backend through packed copies in the workspace.  A call for backend 1
 * that would need the workspace and cannot have it (limit, stream capture) answers
 * FA_ERROR_PEER_ACCESS_UNSUPPORTED when the backend is forced or no delta buffer is there, and runs the
 * split backend otherwise.  DB with packed tokens is rejected (FA_ERROR_NOT_SUPPORTED): all sequences
 * share one bias there. */
FA_API int fa_attn_bwd(const fa_bwd_params* params, int32_t params_version,
                       void* hip_stream, const fa_options* options);

/* The positional v2 API: v2::flash::attn_fwd, attn_fwd_compact_varlen, attn_bwd, attn_bwd_fused,
 * attn_bwd_compact_varlen.  These are not in the reference tree (0.14 keeps only the v3 params
 * entry points); their signatures are those of AOTriton 0.11's include/aotriton/v2/flash.h:31-141
 * as shipped inside PyTorch, with views passed by pointer (null = the reference's empty view),
 * bool as int32 and the extra-arguments pointer dropped.  Each fills the v3 params: is_causal
 * becomes causal_type 3 with the top-left sentinels, cu_seqlens make varlen_type 1.  attn_bwd runs
 * the split backend, attn_bwd_fused the single-launch backend. */
FA_API int fa_v2_attn_fwd(const fa_tensor4* q, const fa_tensor4* k, const fa_tensor4* v,
                          const fa_tensor4* b, float sm_scale, const fa_tensor2* softmax_lse,
                          const fa_tensor4* out, float dropout_p, const fa_tensor0* philox_seed,
                          const fa_tensor0* philox_offset1, int64_t philox_offset2,
                          const fa_tensor0* philox_seed_output,
                          const fa_tensor0* philox_offset_output,
                          const fa_tensor4* encoded_softmax, int32_t is_causal,
                          const fa_tensor0* atomic_for_causal, void* hip_stream);
FA_API int fa_v2_attn_fwd_compact_varlen(
    const fa_tensor4* q, const fa_tensor4* k, const fa_tensor4* v, const fa_tensor4* b,
    const fa_tensor1* cu_seqlens_q, const fa_tensor1* cu_seqlens_k, int32_t max_seqlen_q,
    int32_t max_seqlen_k, float sm_scale, const fa_tensor2* softmax_lse, const fa_tensor4* out,
    float dropout_p, const fa_tensor0* philox_seed, const fa_tensor0* philox_offset1,
    int64_t philox_offset2, const fa_tensor0* philox_seed_output,
    const fa_tensor0* philox_offset_output, const fa_tensor4* encoded_softmax, int32_t is_causal,
    const fa_tensor0* atomic_for_causal, void* hip_stream);
FA_API int fa_v2_attn_bwd(const fa_tensor4* q, const fa_tensor4* k, const fa_tensor4* v,
                          const fa_tensor4* b, float sm_scale, const fa_tensor4* out,
                          const fa_tensor4* dout, const fa_tensor4* dq, const fa_tensor4* dk,
                          const fa_tensor4* dv, const fa_tensor4* db, const fa_tensor2* softmax_lse,
                          const fa_tensor2* delta, float dropout_p, const fa_tensor0* philox_seed,
                          const fa_tensor0* philox_offset1, int64_t philox_offset2,
                          int32_t is_causal, void* hip_stream);
FA_API int fa_v2_attn_bwd_fused(const fa_tensor4* q, const fa_tensor4* k, const fa_tensor4* v,
                                const fa_tensor4* b, float sm_scale, const fa_tensor4* out,
                                const fa_tensor4* dout, const fa_tensor4* dq, const fa_tensor4* dk,
                                const fa_tensor4* dv, const fa_tensor4* db,
                                const fa_tensor2* softmax_lse, float dropout_p,
                                const fa_tensor0* philox_seed, const fa_tensor0* philox_offset1,
                                int64_t philox_offset2, int32_t is_causal, void* hip_stream);
FA_API int fa_v2_attn_bwd_compact_varlen(
    const fa_tensor4* q, const fa_tensor4* k, const fa_tensor4* v, const fa_tensor1* cu_seqlens_q,
    const fa_tensor1* cu_seqlens_k, int32_t max_seqlen_q, int32_t max_seqlen_k, const fa_tensor4* b,
    float sm_scale, const fa_tensor4* out, const fa_tensor4* dout, const fa_tensor4* dq,
    const fa_tensor4* dk, const fa_tensor4* dv, const fa_tensor4* db, const fa_tensor2* softmax_lse,
    const fa_tensor2* delta, float dropout_p, const fa_tensor0* philox_seed,
    const fa_tensor0* philox_offset1, int64_t philox_offset2, int32_t is_causal, void* hip_stream);

/* The split backward for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): same inputs, outputs and
 * results as fa_attn_bwd with backend 0, but delta lives in a device array that belongs to
 * the library (FA_NOALLOC_MAX_ROWS floats = 16 MiB per GPU the library runs on, held until the
 * process ends); params->D is ignored and nothing is allocated or freed.  It has no
 * counterpart in the reference.  Needs batch * Hq * max_seqlen_q (packed sequences: Hq * tokens)
 * <= FA_NOALLOC_MAX_ROWS, else FA_ERROR_OUT_OF_MEMORY before any launch.  All calls on one GPU
 * share the array: calls that overlap on one GPU (two streams, two threads) race.  The first call
 * on a device looks up the device's properties and the array's address (hipGetDeviceProperties,
 * hipGetSymbolAddress), which a stream capture does not allow: before capturing, call
 * fa_check_gpu on a stream of that device (it does both lookups) or this entry point once. */
#define FA_NOALLOC_MAX_ROWS (4 * 1024 * 1024)
FA_API int fa_attn_bwd_noalloc(const fa_bwd_params* params, int32_t params_version,
                               void* hip_stream);

/* Workspace of the split backward.  For 16-bit tensors at head dims up to 256 (dense batches, no dB,
 * not under stream capture; up to head dim 64 only with dropout or a bias, where it pays) fa_attn_bwd keeps dS in HBM between its dK/dV and dQ kernels instead of
 * recomputing S and dP in the dQ kernel (5 GEMMs instead of 7; delta kernel, dK/dV kernel writing dS,
 * dQ = dS K kernel): 2 bytes per (batch, q-head, query, key) plus 8 bytes per (batch, q-head, query),
 * in a buffer per device that belongs to the library, is allocated on first use, only grows and is
 * reused by every later call (calls on one device take turns: a call on another stream than the last
 * one waits on the GPU for the last one's kernels).  A call that would need more than the limit
 * recomputes instead, with the same results up to fp32 summation order.  The limit is, in this
 * order: the last fa_set_bwd_workspace_limit(bytes >= 0); AOTRITON_AMD_BWD_WORKSPACE_MB of the
 * environment; an eighth of the device's memory.  0 switches the workspace off, a negative value
 * forgets the last call.  fa_query_bwd_config sets bit 4 of `flags` when a call would use it.  fa_trim_workspace
 * waits for the devices and frees the buffers.  Neither has a counterpart in the reference, whose
 * split backward always recomputes (modules/flash/kernel/bwd_kernel_dq.py:45-389). */
FA_API void fa_set_bwd_workspace_limit(int64_t bytes);
FA_API int fa_trim_workspace(void);

/* One kernel of the backward only: kernel_slot 0 = delta (bwd_preprocess), 1 = dK/dV
 * (reads delta), 2 = dQ (16-bit types up to head dim 256: computes delta and writes it;
 * otherwise reads it), 3 = fused; of the backward that keeps dS in the library's workspace (calls
 * that qualify for it, else FA_ERROR_NOT_SUPPORTED): 4 = delta and the prepared row statistics,
 * 5 = dK/dV writing dS, 6 = dQ from the stored dS (what slot 5 left in the workspace).  All slots
 * but 3 need an eager delta buffer in params->D.  Stands in
 * for the per-kernel selection of the reference's tuning interface
 * (attn_options::KernelSlot, include/aotriton/flash.h:46-60; include/aotriton/cpp_tune.h)
 * and is what the benchmark uses to time kernels one at a time. */
FA_API int fa_attn_bwd_kernel(const fa_bwd_params* params, int32_t params_version,
                              void* hip_stream, int32_t kernel_slot);

/* v2::flash::debug_simulate_encoded_softmax -- include/aotriton/flash.h:18-24,
 * modules/flash/csrc/attn_debug.cc:30-69.  r is (B, H, max_seqlen_q, max_seqlen_k). */
FA_API int fa_debug_simulate_encoded_softmax(const fa_tensor4* r, float dropout_p,
                                             const fa_tensor0* philox_seed,
                                             const fa_tensor0* philox_offset1,
                                             uint64_t philox_offset2, void* hip_stream);

/* Pure host argument checks that fa_attn_fwd / fa_attn_bwd run before any HIP
 * call (version gate attn_fwd.cc:53-55; functional availability
 * python/codegen/template/shim.cc:72-100). */
FA_API int fa_validate_fwd(const fa_fwd_params* params, int32_t params_version,
                           const fa_options* options);
FA_API int fa_validate_bwd(const fa_bwd_params* params, int32_t params_version,
                           const fa_options* options);

/* Tile/grid the library would use (host only, num_cu = CU count to assume; the backward
 * query assumes 256 CUs). */
FA_API int fa_query_fwd_config(const fa_fwd_params* params, int32_t num_cu,
                               fa_kernel_config* out);
FA_API int fa_query_bwd_config(const fa_bwd_params* params, const fa_options* options,
                               int32_t kernel_slot, fa_kernel_config* out);

/* K-block interval algebra used by the kernels for one Q tile (host mirror of the
 * device function; modules/flash/kernel/masked_load_store.py:43-210).
 * window_left/right are the raw parameters (sentinels allowed).  out[6] =
 * {left-masked lo,hi, full lo,hi, right-masked lo,hi}, closed, empty if lo>hi. */
FA_API int fa_tile_intervals(int32_t causal_type, int32_t window_left, int32_t window_right,
                             int32_t start_m, int32_t seqlen_q, int32_t seqlen_k,
                             int32_t block_m, int32_t block_n, int32_t out[6]);

/* int32 keep threshold the kernels compare Philox words against
 * (modules/flash/kernel/fwd_kernel.py:195). */
FA_API int32_t fa_dropout_threshold(float dropout_p);

/* pyaotriton.get_name_suffix -- bindings/module.cc:89-99. */
FA_API const char* fa_get_name_suffix(void);
FA_API const char* fa_version(void);

/* v_archname / CU count -- v3src/util.cc:65-113.  buf receives e.g. "gfx950". */
FA_API int fa_get_arch(void* hip_stream, char* buf, int32_t buflen);
FA_API int fa_get_multiprocessor_count(void* hip_stream);
/* hipDeviceProp_t::clockRate (kHz) of the stream's device: the clock the "% of peak" figures
 * of a benchmark assume, printed next to the CU count (python/tune/gpu_utils.py:293-370 is the
 * reference's timing method; it reads the device properties the same way). */
FA_API int fa_get_clock_rate_khz(void* hip_stream);

/* bindings/hipruntime.cc:11-95 */
FA_API int fa_hip_get_last_error(void);
FA_API int fa_hip_device_synchronize(void);

#ifdef __cplusplus
}
#endif
#endif /* AOTRITON_AMD_FLASH_H */
