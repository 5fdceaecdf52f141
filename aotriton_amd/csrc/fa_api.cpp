// Operator entry points of the C ABI: argument checks (pure host, before any HIP
// call), shape derivation, tile-table lookup, launch.  Mirrors the hand-written
// operator layer of the reference (modules/flash/csrc/attn_fwd.cc:48-149,
// attn_bwd.cc:55-160, attn_debug.cc:30-69, attn_check.cc:36-46); the generated
// dispatch / kernel-image runtime underneath it is replaced by direct launches of
// kernels linked into this library.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "aotriton_amd/flash.h"
#include "aotriton_amd/probe.h"
#include "fa_args.h"
#include "fa_intervals.h"
#include "fa_kernels.h"

namespace {

// AOTRITON_DEBUG_LEVEL=0..5 -> stderr (include/aotriton/_internal/log.h:56-65)
int log_level() {
  static int level = [] {
    const char* e = std::getenv("AOTRITON_DEBUG_LEVEL");
    return e ? std::atoi(e) : 0;
  }();
  return level;
}
#define FA_LOG(lvl, ...)                                  \
  do {                                                    \
    if (log_level() >= (lvl)) {                           \
      std::fprintf(stderr, "[aotriton_amd] " __VA_ARGS__); \
      std::fputc('\n', stderr);                           \
    }                                                     \
  } while (0)

constexpr int kMaxDevices = 64;
struct DeviceInfo {
  std::atomic<int> state{0};   // 0 unknown, 1 filled
  bool is_gfx950 = false;
  int num_cu = 0;
  int clock_khz = 0;
  char arch[32] = {0};
};
DeviceInfo g_devices[kMaxDevices];
std::mutex g_device_mutex;

// v3src/util.cc:65-113: arch name up to ':' and CU count, memoised per device.
const DeviceInfo* device_of_stream(hipStream_t stream) {
  int dev = 0;
  hipError_t e = hipErrorUnknown;
  if (stream != nullptr) e = hipStreamGetDevice(stream, &dev);
  if (e != hipSuccess) e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  DeviceInfo& d = g_devices[dev];
  if (d.state.load(std::memory_order_acquire) == 1) return &d;
  std::lock_guard<std::mutex> lock(g_device_mutex);
  if (d.state.load(std::memory_order_relaxed) == 1) return &d;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return nullptr;
  size_t n = 0;
  while (prop.gcnArchName[n] && prop.gcnArchName[n] != ':' && n + 1 < sizeof(d.arch)) {
    d.arch[n] = prop.gcnArchName[n];
    ++n;
  }
  d.arch[n] = 0;
  d.is_gfx950 = std::strcmp(d.arch, "gfx950") == 0;
  d.num_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 40;
  d.clock_khz = prop.clockRate;
  d.state.store(1, std::memory_order_release);
  return &d;
}

int device_index(const DeviceInfo* d) { return (int)(d - g_devices); }

// Delta buffer of fa_attn_bwd_noalloc: device memory that belongs to the library, one copy
// per GPU the library runs on, held until the process ends.  In host code the array's name
// is only a handle for hipGetSymbolAddress; the address the kernels get is looked up once
// per device (with that device current) and kept in g_scratch_ptr.
constexpr int64_t kScratchFloats = FA_NOALLOC_MAX_ROWS;
__device__ __align__(256) static float scratch[kScratchFloats];
float* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

hipError_t scratch_of_device(int dev, float** out) {
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    int cur = -1;
    hipError_t e = hipGetDevice(&cur);
    if (e != hipSuccess) return e;
    if (cur != dev && (e = hipSetDevice(dev)) != hipSuccess) return e;
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (cur != dev) (void)hipSetDevice(cur);
    if (e != hipSuccess) return e;
    if (ptr == nullptr) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = static_cast<float*>(ptr);
  }
  *out = g_scratch_ptr[dev];
  return hipSuccess;
}

// Workspace of the backward that keeps dS in HBM between its two kernels: one buffer per device
// that belongs to the library and only grows (hipMalloc once, then reused: a stream-ordered pool
// allocation made the host wait for the GPU on every call).  Calls on one device share it: the
// device's mutex covers the enqueue, and every call first waits (on the GPU) for the event recorded
// behind the last use (no work when that was on the same stream; stream handles are not compared:
// a destroyed stream's handle can come back).  fa_trim_workspace frees the buffers.
std::atomic<int64_t> g_ws_limit{-1};        // bytes; -1: not set (environment, then default)
struct Workspace {
  void* ptr = nullptr;
  size_t bytes = 0;
  hipEvent_t done = nullptr;
  bool used = false;
  std::mutex mutex;
};
Workspace g_ws[kMaxDevices];

int64_t ws_limit_bytes(int dev) {
  int64_t v = g_ws_limit.load(std::memory_order_relaxed);
  if (v >= 0) return v;
  static const int64_t from_env = [] {
    const char* e = std::getenv("AOTRITON_AMD_BWD_WORKSPACE_MB");
    return e ? (int64_t)std::atoll(e) << 20 : (int64_t)-1;
  }();
  if (from_env >= 0) return from_env;
  // default: an eighth of the device's memory (36 GB of 288)
  static std::atomic<int64_t> dflt[kMaxDevices];
  int64_t d = dflt[dev].load(std::memory_order_relaxed);
  if (d == 0) {
    hipDeviceProp_t prop;
    d = hipGetDeviceProperties(&prop, dev) == hipSuccess ? (int64_t)(prop.totalGlobalMem / 8) : ((int64_t)1 << 30);
    dflt[dev].store(d, std::memory_order_relaxed);
  }
  return d;
}

// Returns with the device's mutex held when it succeeds; ws_release drops it.
hipError_t ws_acquire(int dev, size_t need, hipStream_t stream, void** out) {
  Workspace& w = g_ws[dev];
  w.mutex.lock();
  hipError_t e = hipSuccess;
  if (w.bytes < need || w.done == nullptr) {
    int cur = -1;
    e = hipGetDevice(&cur);
    if (e == hipSuccess && cur != dev) e = hipSetDevice(dev);
    if (e == hipSuccess && w.done == nullptr) e = hipEventCreateWithFlags(&w.done, hipEventDisableTiming);
    if (e == hipSuccess && w.bytes < need) {
      // (hipFree waits for the device: nothing uses the old buffer any more)
      if (w.ptr != nullptr) (void)hipFree(w.ptr);
      w.ptr = nullptr; w.bytes = 0; w.used = false;
      size_t grow = need + need / 8;
      e = hipMalloc(&w.ptr, grow);
      if (e != hipSuccess) {      // no room for the margin: exactly what this call needs
        (void)hipGetLastError();
        grow = need;
        e = hipMalloc(&w.ptr, grow);
      }
      if (e == hipSuccess) w.bytes = grow; else w.ptr = nullptr;
    }
    if (cur >= 0 && cur != dev) (void)hipSetDevice(cur);
  }
  if (e == hipSuccess && w.used) e = hipStreamWaitEvent(stream, w.done, 0);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    w.mutex.unlock();
    return e;
  }
  *out = w.ptr;
  return hipSuccess;
}

void ws_release(int dev, hipStream_t stream) {
  Workspace& w = g_ws[dev];
  if (hipEventRecord(w.done, stream) == hipSuccess) {
    w.used = true;
  } else {
    // without the event the next call cannot order itself behind this one
    (void)hipGetLastError();
    (void)hipStreamSynchronize(stream);
    w.used = false;
  }
  w.mutex.unlock();
}

// A call that holds the workspace (the repacking layer below) hands a part of it to the call it
// makes: that call must neither lock nor grow the buffer.
struct NestedWorkspace { bool active = false; void* ptr = nullptr; size_t bytes = 0; };
thread_local NestedWorkspace t_ws_nested;

bool stream_is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  return hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone;
}

bool is_16bit(int dt) { return dt == FA_DTYPE_FLOAT16 || dt == FA_DTYPE_BFLOAT16; }

// ---- packed copies of tensors whose rows are not made of aligned 16-byte pieces ----------------
// (a head dim or a stride that is no multiple of 8 elements, a base that is not 16-byte aligned).
// The reference runs any head dim on its tuned kernels by padding it inside them
// (modules/flash/csrc/attn_fwd.cc:76-82,109, kernel/composed_tensors.py:60-93).  Here such a call
// gets contiguous copies with the head dim rounded up to a multiple of 8 (zeros in the excess
// columns, which add nothing to any dot product) in the library's workspace, runs on the MFMA
// kernels and has its results copied back; without workspace (limit, stream capture) it runs on
// the element-wise vector-ALU kernels.
int elem_bytes_of(int dt) { return dt == FA_DTYPE_FLOAT32 ? 4 : 2; }

size_t packed_bytes(const fa_tensor4& t) {
  const uint64_t dp = (t.sizes[3] + 7) / 8 * 8;
  const uint64_t n = t.sizes[0] * t.sizes[1] * t.sizes[2] * dp * (uint64_t)elem_bytes_of(t.dtype);
  return (size_t)((n + 255) & ~(uint64_t)255);
}

fa_tensor4 packed_view(const fa_tensor4& t, void* ptr) {
  fa_tensor4 v = t;
  const uint64_t dp = (t.sizes[3] + 7) / 8 * 8;
  v.ptr = (t.sizes[0] * t.sizes[1] * t.sizes[2]) != 0 ? ptr : nullptr;
  v.sizes[3] = dp;
  v.strides[3] = 1;
  v.strides[2] = dp;
  v.strides[1] = t.sizes[2] * dp;
  v.strides[0] = t.sizes[1] * t.sizes[2] * dp;
  return v;
}

hipError_t repack(const fa_tensor4& strided, const fa_tensor4& packed, bool unpack, hipStream_t stream) {
  if (packed.ptr == nullptr || strided.ptr == nullptr) return hipSuccess;
  fa::RepackArgs a{};
  a.strided = strided.ptr; a.packed = packed.ptr;
  a.s0 = (int64_t)strided.strides[0]; a.s1 = (int64_t)strided.strides[1]; a.s2 = (int64_t)strided.strides[2];
  a.n0 = (int32_t)strided.sizes[0]; a.n1 = (int32_t)strided.sizes[1]; a.n2 = (int32_t)strided.sizes[2];
  a.d = (int32_t)strided.sizes[3]; a.dp = (int32_t)packed.sizes[3];
  return fa::run_repack(elem_bytes_of(strided.dtype), unpack, a, stream);
}

// bytes of packed copies a call on the element-wise kernels would need instead
size_t fwd_copies_bytes(const fa_fwd_params* p) {
  return packed_bytes(p->Q) + packed_bytes(p->K) + packed_bytes(p->V) + packed_bytes(p->Out);
}
size_t bwd_copies_bytes(const fa_bwd_params* p) {
  size_t n = 0;
  for (const fa_tensor4* t : {&p->Q, &p->K, &p->V, &p->Out, &p->DO, &p->DQ, &p->DK, &p->DV}) n += packed_bytes(*t);
  return n;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int64_t kMaxRowStride = 1 << 21;   // elements; 256 rows of it stay below 2^31 bytes at 4 bytes per element

// rank-4 activation tensor: non-null unless it has no element, unit last stride.  *pieces is cleared
// when its rows are not made of aligned 16-byte pieces (a head dim or a stride that is no multiple
// of 8 elements, a base address that is not 16-byte aligned): such tensors run on the kernels that
// move single elements (the reference masks the excess columns of any head dim, attn_fwd.cc:76-82).
int check_act(const fa_tensor4& t, int dtype, bool* pieces) {
  const bool empty = (t.sizes[0] == 0 || t.sizes[1] == 0 || t.sizes[2] == 0) && t.sizes[3] > 0;
  if (t.ptr == nullptr && !empty) return FA_ERROR_INVALID_VALUE;
  if (t.dtype != dtype) return FA_ERROR_INVALID_VALUE;
  if (t.strides[3] != 1) return FA_ERROR_NOT_SUPPORTED;
  if (!aligned16(t.ptr) || t.sizes[3] % 8 != 0) *pieces = false;
  // strides travel as unsigned 64-bit numbers; one above 2^63 is a negative stride
  for (int i = 0; i < 3; ++i) {
    if (t.sizes[i] > 1 && (int64_t)t.strides[i] < 0) return FA_ERROR_NOT_SUPPORTED;
    if (t.sizes[i] > 1 && (t.strides[i] % 8) != 0) *pieces = false;
  }
  // a tile's rows are addressed with 32-bit byte offsets from the tile's first row
  if (t.sizes[2] > 1 && (int64_t)t.strides[2] > kMaxRowStride) return FA_ERROR_NOT_SUPPORTED;
  return FA_SUCCESS;
}

// L and delta: fp32, contiguous, one value per (sequence or batch element, query head, query row)
// in the layout the kernels index ((batch * Hq, max_seqlen_q) for rank-4 batches, (Hq, tokens)
// for packed sequences; modules/flash/kernel/fwd_kernel_inner.py:38-43).
int check_row_stats(const fa_tensor2& t, int64_t need) {
  if (t.dtype != FA_DTYPE_FLOAT32) return FA_ERROR_INVALID_VALUE;
  if (t.sizes[1] > 1 && t.strides[1] != 1) return FA_ERROR_NOT_SUPPORTED;
  if (t.sizes[0] > 1 && t.strides[0] != t.sizes[1]) return FA_ERROR_NOT_SUPPORTED;
  if ((int64_t)t.sizes[0] * (int64_t)t.sizes[1] < need) return FA_ERROR_INVALID_VALUE;
  return FA_SUCCESS;
}

// a contiguous fp32 (1, n) view for delta
fa_tensor2 row_stats_view(void* ptr, int64_t n) {
  fa_tensor2 t{};
  t.ptr = ptr;
  t.sizes[0] = 1; t.sizes[1] = (uint64_t)n;
  t.strides[0] = (uint64_t)n; t.strides[1] = 1;
  t.dtype = FA_DTYPE_FLOAT32;
  return t;
}

fa::Strides3 strides3(const fa_tensor4& t) {
  return fa::Strides3{(int64_t)t.strides[0], (int64_t)t.strides[1], (int64_t)t.strides[2]};
}

struct Shape {
  int batch, hq, hk, d, d_qk, d_v, max_sq, max_sk, num_seqlens;  // d: compiled head dim; d_qk, d_v: the tensors'; num_seqlens signed as in attn_fwd.cc:99
  bool windowed, bias, dropout;
  bool elementwise;       // some activation tensor is not made of aligned 16-byte pieces
  bool fused_as_split;    // backend 1 asked for where no single-launch kernel exists (fp32, head dims above 256)
  int64_t row_stats;      // elements of L and of delta
};

// Shared by forward and backward: everything that only depends on
// Q/K/V/B, the varlen descriptors and the scalar options.
int check_common(const fa_tensor4& Q, const fa_tensor4& K, const fa_tensor4& V, const fa_tensor4& B,
                 const fa_tensor1& cu_q, const fa_tensor1& cu_k, const fa_tensor1& ss_q,
                 const fa_tensor1& ss_k, int32_t max_sq, int32_t max_sk, int varlen_type,
                 int causal_type, float dropout_p, const fa_tensor0& seed, Shape* out) {
  const int dtype = Q.dtype;
  if (dtype != FA_DTYPE_FLOAT16 && dtype != FA_DTYPE_BFLOAT16 && dtype != FA_DTYPE_FLOAT32)
    return FA_ERROR_INVALID_VALUE;
  int e;
  bool pieces = true;
  if ((e = check_act(Q, dtype, &pieces)) != FA_SUCCESS) return e;
  if ((e = check_act(K, dtype, &pieces)) != FA_SUCCESS) return e;
  if ((e = check_act(V, dtype, &pieces)) != FA_SUCCESS) return e;
  Shape s{};
  s.elementwise = !pieces;
  s.batch = (int)Q.sizes[0];
  s.hq = (int)Q.sizes[1];
  s.hk = (int)K.sizes[1];
  const int dqk = (int)Q.sizes[3], dv = (int)V.sizes[3];
  if ((int)K.sizes[3] != dqk) return FA_ERROR_INVALID_VALUE;
  if (s.hk <= 0 || s.hq <= 0 || s.hq % s.hk != 0 || (int)V.sizes[1] != s.hk) return FA_ERROR_INVALID_VALUE;
  if (K.sizes[0] != Q.sizes[0] || V.sizes[0] != Q.sizes[0]) return FA_ERROR_INVALID_VALUE;
  if (K.sizes[2] != V.sizes[2]) return FA_ERROR_INVALID_VALUE;
  // Head dims are rounded up to a compiled one and the excess columns are masked in
  // the kernels (PADDED_HEAD, attn_fwd.cc:76-82,109); 16-byte granularity.  Dqk and Dv
  // may differ: both run on the compiled head dim that holds the larger one.
  if (dqk <= 0 || dqk > 512 || dv <= 0 || dv > 512) return FA_ERROR_NOT_SUPPORTED;
  s.d_qk = dqk;
  s.d_v = dv;
  const int dmax = dqk > dv ? dqk : dv;
  s.d = dmax <= 64 ? 64 : (dmax <= 128 ? 128 : (dmax <= 256 ? 256 : 512));   // 512: vector-ALU kernels
  s.max_sq = (int)Q.sizes[2];
  s.max_sk = (int)K.sizes[2];
  s.num_seqlens = 0;
  if (varlen_type < FA_VARLEN_NONE || varlen_type > FA_VARLEN_STRIDED) return FA_ERROR_INVALID_VALUE;
  if (cu_q.ptr != nullptr) {
    if (cu_k.ptr == nullptr || varlen_type == FA_VARLEN_NONE) return FA_ERROR_INVALID_VALUE;
    if (cu_q.dtype != FA_DTYPE_INT32 || cu_k.dtype != FA_DTYPE_INT32) return FA_ERROR_INVALID_VALUE;
    if (cu_q.sizes[0] < 2 || cu_k.sizes[0] != cu_q.sizes[0]) return FA_ERROR_INVALID_VALUE;
    if (max_sq <= 0 || max_sk <= 0) return FA_ERROR_INVALID_VALUE;
    const int n = (int)cu_q.sizes[0] - 1;
    s.num_seqlens = varlen_type == FA_VARLEN_PADDED ? -n : n;
    s.max_sq = max_sq;
    s.max_sk = max_sk;
    if (varlen_type == FA_VARLEN_STRIDED) {
      if (ss_q.ptr == nullptr || ss_k.ptr == nullptr) return FA_ERROR_INVALID_VALUE;
      if (ss_q.sizes[0] != cu_q.sizes[0] || ss_k.sizes[0] != cu_q.sizes[0]) return FA_ERROR_INVALID_VALUE;
    }
    if (varlen_type != FA_VARLEN_PADDED && s.batch != 1) return FA_ERROR_INVALID_VALUE;
    if (varlen_type == FA_VARLEN_PADDED && s.batch != n) return FA_ERROR_INVALID_VALUE;
  } else if (varlen_type != FA_VARLEN_NONE) {
    return FA_ERROR_INVALID_VALUE;
  }
  s.row_stats = s.num_seqlens > 0 ? (int64_t)s.hq * (int64_t)Q.sizes[2]
                                  : (int64_t)s.batch * s.hq * (int64_t)s.max_sq;
  if (causal_type != FA_CAUSAL_NONE && causal_type != FA_CAUSAL_WINDOWED) return FA_ERROR_NOT_SUPPORTED;
  s.windowed = causal_type != FA_CAUSAL_NONE;
  if (!(dropout_p >= 0.0f) || !(dropout_p < 1.0f)) return FA_ERROR_INVALID_VALUE;
  s.dropout = dropout_p > 0.0f;   // attn_fwd.cc:110
  if (s.dropout && seed.ptr == nullptr) return FA_ERROR_INVALID_VALUE;
  s.bias = B.ptr != nullptr;      // attn_fwd.cc:122
  if (s.bias) {
    if (B.dtype != dtype) return FA_ERROR_INVALID_VALUE;
    // Sequences of a varlen batch index the bias like the reference's kernels do
    // (modules/flash/kernel/fwd_kernel.py:393-395): batch stride times the batch index, which is the
    // sequence for the padded layout and 0 for packed tokens (one bias shared by all sequences), rows
    // and columns counted from the sequence's start; hence sizes (batch of Q, Hq, Max_seqlen_q, Max_seqlen_k).
    if ((int)B.sizes[0] != s.batch || (int)B.sizes[1] != s.hq || (int)B.sizes[2] != s.max_sq ||
        (int)B.sizes[3] != s.max_sk)
      return FA_ERROR_INVALID_VALUE;
    for (int i = 0; i < 4; ++i)
      if ((int64_t)B.strides[i] < 0) return FA_ERROR_NOT_SUPPORTED;
    // bias rows of a tile are addressed with 32-bit byte offsets, like the activations'
    if ((int64_t)B.strides[2] > kMaxRowStride || (int64_t)B.strides[3] > kMaxRowStride) return FA_ERROR_NOT_SUPPORTED;
  }
  *out = s;
  return FA_SUCCESS;
}

fa::SeqArgs seq_args(const Shape& s, const fa_tensor1& cu_q, const fa_tensor1& cu_k,
                     const fa_tensor1& ss_q, const fa_tensor1& ss_k, int varlen_type) {
  fa::SeqArgs r{};
  r.cu_q = static_cast<const int32_t*>(cu_q.ptr);
  r.cu_k = static_cast<const int32_t*>(cu_k.ptr);
  const bool strided = varlen_type == FA_VARLEN_STRIDED;
  r.ss_q = strided ? static_cast<const int32_t*>(ss_q.ptr) : nullptr;
  r.ss_k = strided ? static_cast<const int32_t*>(ss_k.ptr) : nullptr;
  r.num_seqlens = s.num_seqlens;
  r.max_seqlen_q = s.max_sq;
  r.max_seqlen_k = s.max_sk;
  return r;
}

int validate_fwd(const fa_fwd_params* p, int32_t version, const fa_options* opt, Shape* shape) {
  if (p == nullptr) return FA_ERROR_INVALID_VALUE;
  if (version != FA_FWD_PARAMS_VERSION) return FA_ERROR_INVALID_SYMBOL;   // attn_fwd.cc:53-55
  Shape s{};
  int e = check_common(p->Q, p->K, p->V, p->B, p->cu_seqlens_q, p->cu_seqlens_k, p->seq_strides_q,
                       p->seq_strides_k, p->Max_seqlen_q, p->Max_seqlen_k, p->varlen_type,
                       p->causal_type, p->dropout_p, p->philox_seed_ptr, &s);
  if (e != FA_SUCCESS) return e;
  bool pieces = !s.elementwise;
  if ((e = check_act(p->Out, p->Q.dtype, &pieces)) != FA_SUCCESS) return e;
  s.elementwise = !pieces;
  for (int i = 0; i < 4; ++i)
    if (p->Out.sizes[i] != (i == 3 ? p->V.sizes[3] : p->Q.sizes[i])) return FA_ERROR_INVALID_VALUE;
  if (p->A.ptr != nullptr) return FA_ERROR_NOT_SUPPORTED;   // alibi: USE_ALIBI=false in attn_fwd.cc:123
  if (p->L.ptr != nullptr && (e = check_row_stats(p->L, s.row_stats)) != FA_SUCCESS) return e;
  if (p->encoded_softmax.ptr != nullptr) {
    const fa_tensor4& r = p->encoded_softmax;
    if (r.strides[3] != 1) return FA_ERROR_NOT_SUPPORTED;
    if ((int)r.sizes[1] != s.hq || (int)r.sizes[2] != s.max_sq || (int)r.sizes[3] != s.max_sk)
      return FA_ERROR_INVALID_VALUE;
  }
  // a forced backend that does not exist cannot take the input (template/op.cc:57-70)
  if (opt != nullptr && opt->force_backend_index > 0) return FA_ERROR_PEER_ACCESS_UNSUPPORTED;
  if (shape) *shape = s;
  return FA_SUCCESS;
}

int bwd_backend(const fa_bwd_params* p, const fa_options* opt) {
  if (opt != nullptr && opt->force_backend_index >= 0) return opt->force_backend_index;
  if (opt != nullptr && opt->deterministic) return 0;   // attn_bwd.cc:147-148
  // without a delta buffer only the fused backend can run
  if (p->D.eager.ptr == nullptr && p->D.acquire == nullptr) return 1;
  return 0;
}

int validate_bwd(const fa_bwd_params* p, int32_t version, const fa_options* opt, Shape* shape,
                 int* backend) {
  if (p == nullptr) return FA_ERROR_INVALID_VALUE;
  if (version != FA_BWD_PARAMS_VERSION) return FA_ERROR_INVALID_SYMBOL;   // attn_bwd.cc:60-62
  Shape s{};
  int e = check_common(p->Q, p->K, p->V, p->B, p->cu_seqlens_q, p->cu_seqlens_k, p->seq_strides_q,
                       p->seq_strides_k, p->Max_seqlen_q, p->Max_seqlen_k, p->varlen_type,
                       p->causal_type, p->dropout_p, p->philox_seed_ptr, &s);
  if (e != FA_SUCCESS) return e;
  const int dt = p->Q.dtype;
  bool pieces = !s.elementwise;
  if ((e = check_act(p->Out, dt, &pieces)) != FA_SUCCESS) return e;
  if ((e = check_act(p->DO, dt, &pieces)) != FA_SUCCESS) return e;
  if ((e = check_act(p->DQ, dt, &pieces)) != FA_SUCCESS) return e;
  if ((e = check_act(p->DK, dt, &pieces)) != FA_SUCCESS) return e;
  if ((e = check_act(p->DV, dt, &pieces)) != FA_SUCCESS) return e;
  s.elementwise = !pieces;
  for (int i = 0; i < 4; ++i) {
    const auto o_i = i == 3 ? p->V.sizes[3] : p->Q.sizes[i];
    if (p->Out.sizes[i] != o_i || p->DO.sizes[i] != o_i ||
        p->DQ.sizes[i] != p->Q.sizes[i] || p->DK.sizes[i] != p->K.sizes[i] ||
        p->DV.sizes[i] != p->V.sizes[i])
      return FA_ERROR_INVALID_VALUE;
  }
  // without a query row L and delta hold nothing and may be null
  const bool no_query = p->Q.sizes[0] == 0 || p->Q.sizes[2] == 0;
  if (p->L.ptr == nullptr && !no_query) return FA_ERROR_INVALID_VALUE;
  if (p->L.ptr != nullptr && (e = check_row_stats(p->L, s.row_stats)) != FA_SUCCESS) return e;
  if (p->DB.ptr != nullptr) {
    if (!s.bias) return FA_ERROR_INVALID_VALUE;
    if (s.num_seqlens > 0) return FA_ERROR_NOT_SUPPORTED;   // packed tokens share one bias: every sequence would write the same dB rows
    if (p->DB.dtype != dt) return FA_ERROR_INVALID_VALUE;
    for (int i = 0; i < 4; ++i)
      if (p->DB.sizes[i] != p->B.sizes[i] || (int64_t)p->DB.strides[i] < 0) return FA_ERROR_INVALID_VALUE;
  }
  int be = bwd_backend(p, opt);
  if (be < 0 || be > 1) return FA_ERROR_PEER_ACCESS_UNSUPPORTED;   // e.g. the assembly backend 2
  // fp32 tensors and head dims above 256 have no single-launch kernel: backend 1 runs the split kernels
  // for them, with the caller's delta buffer when there is one and with one in the library's workspace
  // otherwise (whether the call gets that is known at launch: attn_bwd_impl)
  s.fused_as_split = be == 1 && (!is_16bit(dt) || s.d > 256);
  if (s.fused_as_split && p->D.eager.ptr != nullptr && (e = check_row_stats(p->D.eager, s.row_stats)) != FA_SUCCESS)
    return e;
  // (the fused backend on tensors whose rows are not aligned 16-byte pieces runs on packed copies; whether
  // the call gets the workspace for them is known at launch: fused_without_copies below)
  if (be == 0) {
    if (p->D.eager.ptr == nullptr && p->D.acquire == nullptr) return FA_ERROR_INVALID_VALUE;
    if (p->D.eager.ptr != nullptr && (e = check_row_stats(p->D.eager, s.row_stats)) != FA_SUCCESS) return e;
  }
  if (shape) *shape = s;
  if (backend) *backend = be;
  return FA_SUCCESS;
}

hipError_t run_fwd(int dtype, int d, const fa::FwdArgs& a, const Shape& s, hipStream_t stream) {
  if (s.elementwise) return fa::run_fwd_valu(dtype, d, a, stream);
  if (dtype == FA_DTYPE_FLOAT32)
    return fa::run_fwd_f32(d, a, s.windowed, s.bias, s.dropout, stream);
  if (d > 256) return fa::run_fwd_d512(dtype, a, s.windowed, s.bias, s.dropout, stream);
  const bool padded = a.head_dim != d || a.head_dim_v != d;   // head dim rounded up: the copies that mask the excess columns
  switch (d) {
    case 64: return (padded ? fa::run_fwd_d64_padded : fa::run_fwd_d64)(dtype, a, s.windowed, s.bias, s.dropout, stream);
    case 128: return (padded ? fa::run_fwd_d128_padded : fa::run_fwd_d128)(dtype, a, s.windowed, s.bias, s.dropout, stream);
    case 256: return (padded ? fa::run_fwd_d256_padded : fa::run_fwd_d256)(dtype, a, s.windowed, s.bias, s.dropout, stream);
  }
  return hipErrorNotSupported;
}

fa::DropoutArgs dropout_args(float p, const fa_tensor0& seed, const fa_tensor0& off1, uint64_t off2) {
  fa::DropoutArgs d{};
  d.p = p;
  d.seed_ptr = static_cast<const uint64_t*>(seed.ptr);
  d.offset1_ptr = static_cast<const uint64_t*>(off1.ptr);
  d.offset2 = off2;
  return d;
}

// Bytes of workspace with which the split backward keeps dS in HBM, 0 when this call recomputes S
// and dP in its dQ kernel instead (anything but the 16-bit MFMA kernels of the 128-column build,
// packed sequences, dB wanted, an empty tensor).  *ds_bytes / *stat_bytes: the parts of the buffer.
int64_t ds_workspace_need(const fa_bwd_params* p, const Shape& s, int* ntq, int* ntk, int64_t* ds_bytes,
                          int64_t* stat_bytes) {
  if (s.elementwise || !is_16bit(p->Q.dtype) || (s.d != 64 && s.d != 128 && s.d != 256) || s.num_seqlens != 0 || p->DB.ptr != nullptr ||
      s.batch <= 0 || s.max_sq <= 0 || s.max_sk <= 0)
    return 0;
  // the 64-column build: 2 bytes per pair are too many for its little GEMM work unless the dQ kernel is
  // spared a bias or the Philox arithmetic (same box, stored / recomputing: 1.05-1.14 plain, 0.69-0.81 with either)
  if (s.d == 64 && !s.dropout && !s.bias) return 0;
  int64_t tile_bytes = 0;
  fa::ds_tile_counts(p->Q.dtype, s.d, s.max_sq, s.max_sk, ntq, ntk, &tile_bytes);
  *ds_bytes = (int64_t)s.batch * s.hq * *ntq * *ntk * tile_bytes;
  *stat_bytes = (s.row_stats * 4 + 255) & ~(int64_t)255;
  return *ds_bytes + 2 * *stat_bytes;
}

}  // namespace

extern "C" {

const char* fa_get_name_suffix(void) { return "_amd_gfx950"; }
const char* fa_version(void) { return "0.1.0"; }

int fa_get_arch(void* hip_stream, char* buf, int32_t buflen) {
  const DeviceInfo* d = device_of_stream(static_cast<hipStream_t>(hip_stream));
  if (d == nullptr || buf == nullptr || buflen <= 0) return FA_ERROR_INVALID_VALUE;
  std::snprintf(buf, (size_t)buflen, "%s", d->arch);
  return FA_SUCCESS;
}

int fa_get_multiprocessor_count(void* hip_stream) {
  const DeviceInfo* d = device_of_stream(static_cast<hipStream_t>(hip_stream));
  return d ? d->num_cu : 40;   // v3src/util.cc:95-112 falls back to 40
}

int fa_get_clock_rate_khz(void* hip_stream) {
  const DeviceInfo* d = device_of_stream(static_cast<hipStream_t>(hip_stream));
  return d ? d->clock_khz : 0;
}

int fa_probe_mfma_rate(int32_t random_operands, int32_t num_workgroups, int32_t iters, float* out,
                       uint64_t* clocks, void* hip_stream) {
  if (out == nullptr || clocks == nullptr || num_workgroups <= 0 || iters <= 0) return FA_ERROR_INVALID_VALUE;
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  const DeviceInfo* d = device_of_stream(stream);
  if (d == nullptr || !d->is_gfx950) return FA_ERROR_NO_BINARY_FOR_GPU;
  return (int)fa::run_mfma_rate(random_operands != 0, num_workgroups, iters, out,
                                reinterpret_cast<unsigned long long*>(clocks), stream);
}

int fa_hip_get_last_error(void) { return (int)hipGetLastError(); }
int fa_hip_device_synchronize(void) { return (int)hipDeviceSynchronize(); }

int32_t fa_dropout_threshold(float dropout_p) { return fa::dropout_threshold(dropout_p); }

int fa_tile_intervals(int32_t causal_type, int32_t window_left, int32_t window_right, int32_t start_m,
                      int32_t seqlen_q, int32_t seqlen_k, int32_t block_m, int32_t block_n,
                      int32_t out[6]) {
  if (out == nullptr || block_m <= 0 || block_n <= 0) return FA_ERROR_INVALID_VALUE;
  const bool windowed = causal_type != 0;
  fa::Window w{0, 0};
  if (windowed) w = fa::parse_window(causal_type, window_left, window_right, seqlen_q, seqlen_k);
  const fa::BlockRanges r = fa::block_ranges(windowed, w.left, w.right, start_m, seqlen_q, seqlen_k,
                                             block_m, block_n);
  out[0] = r.lb_lo; out[1] = r.lb_hi; out[2] = r.fb_lo; out[3] = r.fb_hi; out[4] = r.rb_lo; out[5] = r.rb_hi;
  return FA_SUCCESS;
}

int fa_check_gpu(void* hip_stream) {
  const DeviceInfo* d = device_of_stream(static_cast<hipStream_t>(hip_stream));
  if (d == nullptr || !d->is_gfx950) return FA_ERROR_NO_BINARY_FOR_GPU;
  // the address of fa_attn_bwd_noalloc's array is looked up here as well: a first call of that
  // entry point under stream capture then finds it and makes no call that a capture forbids
  float* unused = nullptr;
  (void)scratch_of_device(device_index(d), &unused);
  return FA_SUCCESS;
}

int fa_validate_fwd(const fa_fwd_params* params, int32_t params_version, const fa_options* options) {
  return validate_fwd(params, params_version, options, nullptr);
}

int fa_validate_bwd(const fa_bwd_params* params, int32_t params_version, const fa_options* options) {
  return validate_bwd(params, params_version, options, nullptr, nullptr);
}

int fa_query_fwd_config(const fa_fwd_params* params, int32_t num_cu, fa_kernel_config* out) {
  if (out == nullptr) return FA_ERROR_INVALID_VALUE;
  Shape s{};
  int e = validate_fwd(params, FA_FWD_PARAMS_VERSION, nullptr, &s);
  if (e != FA_SUCCESS) return e;
  // the vector-ALU kernels (3-D grid), the fp32 kernels and the split-head-dim kernels (above 256)
  const bool valu = params->Q.dtype == FA_DTYPE_FLOAT32 || s.d > 256 || s.elementwise;
  const fa::TileShape t = s.elementwise ? fa::TileShape{32, 1, 4, 0}
                          : params->Q.dtype == FA_DTYPE_FLOAT32 ? fa::f32_tile_shape(s.d, -1)
                          : s.d > 256 ? fa::d512_tile_shape(-1)
                                      : fa::fwd_tile_shape(params->Q.dtype, s.d, s.windowed);
  out->block_m = t.block_m; out->block_n = t.block_n; out->num_waves = t.num_waves;
  out->lds_bytes = t.lds_bytes;
  if (valu) {
    const int nz = s.num_seqlens != 0 ? std::abs(s.num_seqlens) : s.batch;
    const int mt = (s.max_sq + t.block_m - 1) / t.block_m;
    if (s.elementwise) {      // vector-ALU kernels: 3-D grid
      out->grid[0] = mt; out->grid[1] = s.hq; out->grid[2] = nz;
    } else {      // one workgroup per tile, the tiles of a kv-head's group back to back on one XCD
      out->grid[0] = fa::kNumXcd * ((nz * s.hk + fa::kNumXcd - 1) / fa::kNumXcd) * (s.hq / s.hk) * mt;
      out->grid[1] = 1; out->grid[2] = 1;
    }
  } else {
    const int nz = s.num_seqlens != 0 ? std::abs(s.num_seqlens) : s.batch;
    const int zh_per_xcd = (nz * s.hq + fa::kNumXcd - 1) / fa::kNumXcd;
    const int ratio = s.hq / s.hk;
    const int zg = ratio > 2 ? (ratio > 8 ? 8 : ratio) : 2;
    const int groups = (zh_per_xcd + zg - 1) / zg;
    // persistent workgroups: one per CU, at most one per Q tile
    const int items = groups * zg * ((s.max_sq + t.block_m - 1) / t.block_m);
    int workers = (num_cu > 0 ? num_cu : 256) / fa::kNumXcd;
    workers = workers < 1 ? 1 : (workers > items ? items : workers);
    out->grid[0] = fa::kNumXcd * workers;
    out->grid[1] = 1;
    out->grid[2] = 1;
  }
  out->backend_index = 0;
  out->head_dim = s.d;
  out->flags = (s.windowed ? 1 : 0) | (s.bias ? 2 : 0) | (s.dropout ? 4 : 0) | (s.num_seqlens != 0 ? 8 : 0);
  // 32: fa_attn_fwd would run this call on packed copies in the workspace of the current device (the
  // tile and grid above are those of the element-wise kernels it runs on otherwise)
  int dev = 0;
  if (s.elementwise && hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices &&
      (int64_t)fwd_copies_bytes(params) <= ws_limit_bytes(dev))
    out->flags |= 32;
  return FA_SUCCESS;
}

int fa_query_bwd_config(const fa_bwd_params* params, const fa_options* options, int32_t kernel_slot,
                        fa_kernel_config* out) {
  if (out == nullptr || kernel_slot < 0 || kernel_slot > 3) return FA_ERROR_INVALID_VALUE;
  Shape s{};
  int be = 0;
  int e = validate_bwd(params, FA_BWD_PARAMS_VERSION, options, &s, &be);
  if (e != FA_SUCCESS) return e;
  const bool valu = params->Q.dtype == FA_DTYPE_FLOAT32 || s.d > 256 || s.elementwise;   // vector-ALU kernels: 32 rows per workgroup
  if (valu && kernel_slot == 3) return FA_ERROR_PEER_ACCESS_UNSUPPORTED;
  const bool split_d = !s.elementwise && params->Q.dtype != FA_DTYPE_FLOAT32 && s.d > 256 && kernel_slot != 0;
  const bool f32_mfma = !s.elementwise && params->Q.dtype == FA_DTYPE_FLOAT32 && kernel_slot != 0;
  const fa::TileShape t = f32_mfma ? fa::f32_tile_shape(s.d, kernel_slot)
                          : split_d ? fa::d512_tile_shape(kernel_slot)
                          : valu  ? (kernel_slot == 1 ? fa::TileShape{1, 32, 4, 0} : fa::TileShape{32, 1, 4, 0})
                                  : fa::bwd_tile_shape(params->Q.dtype, s.d, s.windowed, kernel_slot);
  const int nz = s.num_seqlens != 0 ? std::abs(s.num_seqlens) : s.batch;
  out->block_m = t.block_m; out->block_n = t.block_n; out->num_waves = t.num_waves;
  out->lds_bytes = t.lds_bytes;
  const int mt = (s.max_sq + t.block_m - 1) / t.block_m, nt = (s.max_sk + t.block_n - 1) / t.block_n;
  // 1-D work lists of the main kernels: 8 XCDs x (heads per XCD, rounded up to whole groups) x
  // items per head.  The fused kernel launches one workgroup per item, and so do dK/dV and dQ
  // with a bias or at D = 256; otherwise they run persistent workgroups, one per CU (256 CUs assumed
  // here) and at most one per item.
  auto grid1d = [&](int heads, int zg, int items) {
    const int per_xcd = (nz * heads + fa::kNumXcd - 1) / fa::kNumXcd;
    return fa::kNumXcd * ((per_xcd + zg - 1) / zg) * zg * items;
  };
  auto persistent = [&](int items_total) {
    const int per_xcd = items_total / fa::kNumXcd;
    return s.bias || s.d >= 256 ? items_total : fa::kNumXcd * (per_xcd < 32 ? per_xcd : 32);
  };
  const int ratio = s.hq / s.hk;
  out->grid[1] = 1;
  out->grid[2] = 1;
  if (f32_mfma || split_d) {      // one workgroup per tile, the tiles of a kv-head back to back on one XCD
    out->grid[0] = fa::kNumXcd * ((nz * s.hk + fa::kNumXcd - 1) / fa::kNumXcd) * (kernel_slot == 1 ? nt : ratio * mt);
  } else if (valu) {
    out->grid[0] = kernel_slot == 1 ? nt : mt;
    out->grid[1] = kernel_slot == 1 ? s.hk : s.hq;
    out->grid[2] = nz;
  } else switch (kernel_slot) {
    case 0: out->grid[0] = mt; out->grid[1] = s.hq; out->grid[2] = nz; break;
    case 1: out->grid[0] = persistent(grid1d(s.hk, 2, nt)); break;
    case 2: out->grid[0] = persistent(grid1d(s.hq, ratio > 2 ? (ratio > 8 ? 8 : ratio) : 2, mt)); break;
    default: out->grid[0] = persistent(grid1d(s.hk, 2, nt + mt * ratio)); break;
  }
  out->backend_index = be;
  out->head_dim = s.d;
  out->flags = (s.windowed ? 1 : 0) | (s.bias ? 2 : 0) | (s.dropout ? 4 : 0) | (s.num_seqlens != 0 ? 8 : 0);
  // 16: fa_attn_bwd would keep dS in HBM for this call on the current device (workspace within the
  // limit; a call under stream capture recomputes all the same)
  if (be == 0) {
    int ntq = 0, ntk = 0, dev = 0;
    int64_t ds_bytes = 0, stat_bytes = 0;
    const int64_t need = ds_workspace_need(params, s, &ntq, &ntk, &ds_bytes, &stat_bytes);
    if (need > 0 && hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices && need <= ws_limit_bytes(dev))
      out->flags |= 16;
  }
  // 32: fa_attn_bwd would run this call on packed copies in the workspace
  int dev = 0;
  if (s.elementwise && hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices &&
      (int64_t)bwd_copies_bytes(params) <= ws_limit_bytes(dev))
    out->flags |= 32;
  return FA_SUCCESS;
}

int fa_debug_simulate_encoded_softmax(const fa_tensor4* r, float dropout_p, const fa_tensor0* philox_seed,
                                      const fa_tensor0* philox_offset1, uint64_t philox_offset2,
                                      void* hip_stream) {
  if (r == nullptr || r->ptr == nullptr || philox_seed == nullptr || philox_offset1 == nullptr)
    return FA_ERROR_INVALID_VALUE;
  if (r->dtype != FA_DTYPE_FLOAT16 && r->dtype != FA_DTYPE_BFLOAT16 && r->dtype != FA_DTYPE_FLOAT32)
    return FA_ERROR_INVALID_VALUE;
  if (r->strides[3] != 1) return FA_ERROR_NOT_SUPPORTED;
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  const DeviceInfo* d = device_of_stream(stream);
  if (d == nullptr || !d->is_gfx950) return FA_ERROR_NO_BINARY_FOR_GPU;
  fa::EncodedSoftmaxArgs a{};
  a.r = r->ptr;
  a.s_z = (int64_t)r->strides[0]; a.s_h = (int64_t)r->strides[1]; a.s_m = (int64_t)r->strides[2];
  a.batch = (int)r->sizes[0]; a.heads = (int)r->sizes[1];      // attn_debug.cc:40-42
  a.seqlen_q = (int)r->sizes[2]; a.seqlen_k = (int)r->sizes[3];
  a.dtype = r->dtype;
  a.drop = dropout_args(dropout_p, *philox_seed, *philox_offset1, philox_offset2);
  return (int)fa::run_encoded_softmax(a, stream);
}

int fa_attn_fwd(const fa_fwd_params* p, int32_t params_version, void* hip_stream,
                const fa_options* options) {
  Shape s{};
  int e = validate_fwd(p, params_version, options, &s);
  if (e != FA_SUCCESS) return e;
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  const DeviceInfo* dev = device_of_stream(stream);
  if (dev == nullptr || !dev->is_gfx950) return FA_ERROR_NO_BINARY_FOR_GPU;

  if (s.elementwise && !t_ws_nested.active && !stream_is_capturing(stream)) {
    // packed copies of Q, K, V and Out in the workspace, the MFMA kernels on those, Out copied back
    const fa_tensor4* in[3] = {&p->Q, &p->K, &p->V};
    const size_t need = fwd_copies_bytes(p);
    void* base = nullptr;
    if ((int64_t)need <= ws_limit_bytes(device_index(dev)) && ws_acquire(device_index(dev), need, stream, &base) == hipSuccess) {
      fa_fwd_params p2 = *p;
      char* at = static_cast<char*>(base);
      fa_tensor4* to[3] = {&p2.Q, &p2.K, &p2.V};
      hipError_t err = hipSuccess;
      for (int i = 0; i < 3 && err == hipSuccess; ++i) {
        *to[i] = packed_view(*in[i], at);
        at += packed_bytes(*in[i]);
        err = repack(*in[i], *to[i], false, stream);
      }
      p2.Out = packed_view(p->Out, at);
      int rc = (int)err;
      if (err == hipSuccess) {
        t_ws_nested = NestedWorkspace{true, nullptr, 0};
        rc = fa_attn_fwd(&p2, params_version, hip_stream, options);
        t_ws_nested = NestedWorkspace{};
      }
      if (rc == FA_SUCCESS) rc = (int)repack(p->Out, p2.Out, true, stream);
      ws_release(device_index(dev), stream);
      return rc;
    }
  }

  fa::FwdArgs a{};
  a.q = p->Q.ptr; a.k = p->K.ptr; a.v = p->V.ptr; a.bias = p->B.ptr;
  a.out = p->Out.ptr;
  a.lse = static_cast<float*>(p->L.ptr);
  a.sq = strides3(p->Q); a.sk = strides3(p->K); a.sv = strides3(p->V); a.so = strides3(p->Out);
  if (s.bias) {
    a.sb_z = (int64_t)p->B.strides[0]; a.sb_h = (int64_t)p->B.strides[1];
    a.sb_m = (int64_t)p->B.strides[2]; a.sb_n = (int64_t)p->B.strides[3];
  }
  a.batch = s.batch; a.hq = s.hq; a.hk = s.hk; a.head_dim = s.d_qk; a.head_dim_v = s.d_v;
  a.elementwise = s.elementwise ? 1 : 0;
  a.sm_scale = p->Sm_scale;
  a.seq = seq_args(s, p->cu_seqlens_q, p->cu_seqlens_k, p->seq_strides_q, p->seq_strides_k, p->varlen_type);
  a.mask = fa::MaskArgs{p->causal_type, p->window_left, p->window_right};
  a.drop = dropout_args(p->dropout_p, p->philox_seed_ptr, p->philox_offset1, p->philox_offset2);
  a.seed_out = static_cast<uint64_t*>(p->philox_seed_output.ptr);
  a.offset_out = static_cast<uint64_t*>(p->philox_offset_output.ptr);
  a.atomic_counter = static_cast<int32_t*>(p->persistent_atomic_counter.ptr);
  a.num_cu = dev->num_cu;

  const fa::TileShape t = (p->Q.dtype == FA_DTYPE_FLOAT32 || s.d > 256 || s.elementwise) ? fa::TileShape{32, 1, 4, 0} : fa::fwd_tile_shape(p->Q.dtype, s.d, s.windowed);
  FA_LOG(4, "attn_fwd: D=%d BLOCK_M=%d BLOCK_N=%d waves=%d lds=%d windowed=%d bias=%d dropout=%d nseq=%d",
         s.d, t.block_m, t.block_n, t.num_waves, t.lds_bytes, (int)s.windowed, (int)s.bias,
         (int)s.dropout, s.num_seqlens);
  hipError_t err = run_fwd(p->Q.dtype, s.d, a, s, stream);
  if (err != hipSuccess) return (int)err;
  if (p->encoded_softmax.ptr != nullptr) {
    // the forward metro chains the mask dump (modules/flash/aot/__init__.py:40-41)
    fa_tensor4 r = p->encoded_softmax;
    return fa_debug_simulate_encoded_softmax(&r, p->dropout_p, &p->philox_seed_ptr, &p->philox_offset1,
                                             p->philox_offset2, hip_stream);
  }
  return FA_SUCCESS;
}

// kernel_slot < 0: the whole backward of the chosen backend; otherwise only that
// kernel (0 delta, 1 dK/dV, 2 dQ, 3 fused; 4-6 the three kernels of the backward that keeps dS).
// own_delta: the split backend with delta in the library's own per-device array (params->D is
// not looked at).
static int attn_bwd_impl(const fa_bwd_params* p_in, int32_t params_version, void* hip_stream,
                         const fa_options* options, int kernel_slot, bool own_delta = false) {
  Shape s{};
  int backend = 0;
  fa_options forced{};
  const fa_bwd_params* p = p_in;
  fa_bwd_params with_delta;
  if (own_delta) {
    if (p_in == nullptr) return FA_ERROR_INVALID_VALUE;
    if (params_version != FA_BWD_PARAMS_VERSION) return FA_ERROR_INVALID_SYMBOL;
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    const DeviceInfo* dv = device_of_stream(st);
    if (dv == nullptr || !dv->is_gfx950) return FA_ERROR_NO_BINARY_FOR_GPU;
    float* ptr = nullptr;
    hipError_t se = scratch_of_device(device_index(dv), &ptr);
    if (se != hipSuccess) return (int)se;
    with_delta = *p_in;
    with_delta.D = fa_lazy_tensor2{};
    with_delta.D.eager.ptr = ptr;
    // sized for the check of the tensors below; the limit of the array is tested right after
    with_delta.D.eager.sizes[0] = 1; with_delta.D.eager.sizes[1] = (uint64_t)1 << 60;
    with_delta.D.eager.strides[0] = (uint64_t)1 << 60; with_delta.D.eager.strides[1] = 1;
    with_delta.D.eager.dtype = FA_DTYPE_FLOAT32;
    p = &with_delta;
    forced.force_backend_index = 0;
    forced.deterministic = 0;
    options = &forced;
    Shape probe{};
    const int pe = validate_bwd(p, params_version, options, &probe, nullptr);
    if (pe != FA_SUCCESS) return pe;
    // one delta value per (batch element or token, query head, query row)
    if (probe.row_stats > kScratchFloats) {
      FA_LOG(1, "attn_bwd_noalloc: %lld delta values needed, the library's array holds %lld",
             (long long)probe.row_stats, (long long)kScratchFloats);
      return FA_ERROR_OUT_OF_MEMORY;
    }
  }
  if (kernel_slot >= 0) {
    forced.force_backend_index = kernel_slot == 3 ? 1 : 0;   // (slots 4-6 belong to the split backend too)
    forced.deterministic = 0;
    options = &forced;
  }
  int e = validate_bwd(p, params_version, options, &s, &backend);
  if (e != FA_SUCCESS) return e;
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  const DeviceInfo* dev = device_of_stream(stream);
  if (dev == nullptr || !dev->is_gfx950) return FA_ERROR_NO_BINARY_FOR_GPU;

  if (s.elementwise && kernel_slot < 0 && !own_delta && !t_ws_nested.active && !stream_is_capturing(stream)) {
    // packed copies of the eight activation tensors, the MFMA kernels on those, dQ, dK, dV copied back;
    // the packed call gets the rest of the buffer for its own use (dS)
    const fa_tensor4* all[8] = {&p->Q, &p->K, &p->V, &p->Out, &p->DO, &p->DQ, &p->DK, &p->DV};
    // (a call for backend 1 that will run the split kernels and brings no delta buffer gets one here)
    const bool lib_delta = backend == 1 && s.fused_as_split && p->D.eager.ptr == nullptr && p->D.acquire == nullptr;
    const size_t delta_bytes = lib_delta ? (((size_t)s.row_stats * 4 + 255) & ~(size_t)255) : 0;
    const size_t copies = bwd_copies_bytes(p) + delta_bytes;
    fa_bwd_params p2 = *p;
    fa_tensor4* to[8] = {&p2.Q, &p2.K, &p2.V, &p2.Out, &p2.DO, &p2.DQ, &p2.DK, &p2.DV};
    for (int i = 0; i < 8; ++i) *to[i] = packed_view(*all[i], reinterpret_cast<void*>(uintptr_t(256)));   // shapes first
    Shape s2{};
    int be2 = 0;
    int64_t inner = 0;
    if (validate_bwd(&p2, params_version, options, &s2, &be2) == FA_SUCCESS && be2 == 0) {
      int ntq = 0, ntk = 0;
      int64_t ds_bytes = 0, stat_bytes = 0;
      inner = ds_workspace_need(&p2, s2, &ntq, &ntk, &ds_bytes, &stat_bytes);
      if ((int64_t)copies + inner > ws_limit_bytes(device_index(dev))) inner = 0;
    }
    const size_t need = copies + (size_t)inner;
    void* base = nullptr;
    if ((int64_t)need <= ws_limit_bytes(device_index(dev)) && ws_acquire(device_index(dev), need, stream, &base) == hipSuccess) {
      char* at = static_cast<char*>(base);
      hipError_t err = hipSuccess;
      for (int i = 0; i < 8; ++i) {
        *to[i] = packed_view(*all[i], at);
        at += packed_bytes(*all[i]);
        if (i < 5 && err == hipSuccess) err = repack(*all[i], *to[i], false, stream);
      }
      if (lib_delta) {
        p2.D = fa_lazy_tensor2{};
        p2.D.eager = row_stats_view(at, s.row_stats);
        at += delta_bytes;
      }
      int rc = (int)err;
      if (err == hipSuccess) {
        t_ws_nested = NestedWorkspace{true, inner > 0 ? at : nullptr, (size_t)inner};
        rc = attn_bwd_impl(&p2, params_version, hip_stream, options, kernel_slot, false);
        t_ws_nested = NestedWorkspace{};
      }
      for (int i = 5; i < 8 && rc == FA_SUCCESS; ++i) rc = (int)repack(*all[i], *to[i], true, stream);
      ws_release(device_index(dev), stream);
      return rc;
    }
  }
  if (backend == 1 && s.fused_as_split) {
    // the split kernels: with the caller's delta buffer, or with one in the workspace
    if (kernel_slot == 3) return FA_ERROR_PEER_ACCESS_UNSUPPORTED;      // there is no such kernel to run alone
    if (p->D.eager.ptr != nullptr || p->D.acquire != nullptr) {
      backend = 0;
    } else {
      const size_t bytes = ((size_t)s.row_stats * 4 + 255) & ~(size_t)255;
      void* base = nullptr;
      if (kernel_slot >= 0 || t_ws_nested.active || stream_is_capturing(stream) ||
          (int64_t)bytes > ws_limit_bytes(device_index(dev)) ||
          ws_acquire(device_index(dev), bytes, stream, &base) != hipSuccess)
        return FA_ERROR_PEER_ACCESS_UNSUPPORTED;
      fa_bwd_params p2 = *p;
      p2.D = fa_lazy_tensor2{};
      p2.D.eager = row_stats_view(base, s.row_stats);
      fa_options split = options != nullptr ? *options : fa_options{};
      split.force_backend_index = 0;
      t_ws_nested = NestedWorkspace{true, nullptr, 0};
      const int rc = attn_bwd_impl(&p2, params_version, hip_stream, &split, -1, false);
      t_ws_nested = NestedWorkspace{};
      ws_release(device_index(dev), stream);
      return rc;
    }
  }
  if (s.elementwise && backend == 1) {
    // fused_without_copies: the element-wise kernels have the split backend only
    const bool forced = options != nullptr && options->force_backend_index >= 0;
    if (forced || (p->D.eager.ptr == nullptr && p->D.acquire == nullptr)) return FA_ERROR_PEER_ACCESS_UNSUPPORTED;
    if (p->D.eager.ptr != nullptr && (e = check_row_stats(p->D.eager, s.row_stats)) != FA_SUCCESS) return e;
    backend = 0;
  }

  fa::BwdArgs a{};
  a.q = p->Q.ptr; a.k = p->K.ptr; a.v = p->V.ptr; a.bias = p->B.ptr;
  a.out = p->Out.ptr; a.dout = p->DO.ptr;
  a.dq = p->DQ.ptr; a.dk = p->DK.ptr; a.dv = p->DV.ptr; a.db = p->DB.ptr;
  a.lse = static_cast<const float*>(p->L.ptr);
  a.sq = strides3(p->Q); a.sk = strides3(p->K); a.sv = strides3(p->V); a.so = strides3(p->Out);
  a.sdo = strides3(p->DO); a.sdq = strides3(p->DQ); a.sdk = strides3(p->DK); a.sdv = strides3(p->DV);
  if (s.bias) {
    a.sb_z = (int64_t)p->B.strides[0]; a.sb_h = (int64_t)p->B.strides[1];
    a.sb_m = (int64_t)p->B.strides[2]; a.sb_n = (int64_t)p->B.strides[3];
  }
  if (p->DB.ptr != nullptr) {
    a.sdb_z = (int64_t)p->DB.strides[0]; a.sdb_h = (int64_t)p->DB.strides[1];
    a.sdb_m = (int64_t)p->DB.strides[2]; a.sdb_n = (int64_t)p->DB.strides[3];
  }
  a.batch = s.batch; a.hq = s.hq; a.hk = s.hk; a.head_dim = s.d_qk; a.head_dim_v = s.d_v;
  a.elementwise = s.elementwise ? 1 : 0;
  a.sm_scale = p->Sm_scale;
  a.seq = seq_args(s, p->cu_seqlens_q, p->cu_seqlens_k, p->seq_strides_q, p->seq_strides_k, p->varlen_type);
  a.mask = fa::MaskArgs{p->causal_type, p->window_left, p->window_right};
  a.drop = dropout_args(p->dropout_p, p->philox_seed_ptr, p->philox_offset1, p->philox_offset2);
  a.num_cu = dev->num_cu;

  const int dt = p->Q.dtype;
  FA_LOG(4, "attn_bwd: backend=%d slot=%d D=%d windowed=%d bias=%d dropout=%d nseq=%d", backend,
         kernel_slot, s.d, (int)s.windowed, (int)s.bias, (int)s.dropout, s.num_seqlens);
  hipError_t err = hipSuccess;
  if (backend == 0) {
    // split: delta, then dK/dV, then dQ (modules/flash/aot/__init__.py:52-59)
    fa_lazy_tensor2* lazy = const_cast<fa_lazy_tensor2*>(&p->D);
    fa_tensor2 delta = p->D.eager;
    bool acquired = false;
    if (delta.ptr == nullptr) {
      const bool no_query = p->Q.sizes[0] == 0 || p->Q.sizes[2] == 0;
      if (lazy->acquire(lazy, &delta) != 0 || (delta.ptr == nullptr && !no_query)) return FA_ERROR_INVALID_VALUE;
      acquired = true;
      if (delta.ptr != nullptr && check_row_stats(delta, s.row_stats) != FA_SUCCESS) {
        if (lazy->dispose != nullptr) lazy->dispose(lazy);
        return FA_ERROR_INVALID_VALUE;
      }
    }
    a.delta = static_cast<float*>(delta.ptr);
    const bool slow = s.elementwise;              // rows moved element by element: vector-ALU kernels
    const bool f32 = !slow && dt == FA_DTYPE_FLOAT32;      // fp32 MFMA kernels
    const bool big = !slow && !f32 && s.d > 256;  // head dim split over the waves
    // fp32 and the head dims above 256 take delta from the vector-ALU kernel.  The dQ kernel of the
    // 16-bit types up to head dim 256 computes delta from the O and dO rows it holds and writes it
    // out; the dK/dV kernel runs after it and reads it, so the whole backward is two launches
    // (kernel_slot 0 still launches the preprocess kernel on its own).
    const bool delta_launch = f32 || big || slow;
    // The 16-bit kernels up to head dim 256 can keep dS in HBM instead of recomputing S and dP in
    // the dQ kernel (5 GEMMs instead of 7): delta first, then dK/dV writing dS, then dQ = dS K.  It
    // takes 2 bytes per (query, key) pair of workspace; when that is above the limit, under stream
    // capture, for packed sequences or with dB the kernels recompute.  (Measured at S4096, 16384 tokens:
    // head dim 128 gains 5 %, 256 gains 16 %; head dim 64, where a pair costs half the arithmetic and
    // the same bytes, loses 12 % unless the dQ kernel is spared dropout or a bias: then it gains 20-30 %.)
    void* ds_ws = nullptr;
    int ntq = 0, ntk = 0;
    int64_t ds_bytes = 0, stat_bytes = 0;
    // (kernel_slot 4, 5, 6: one kernel of this backward only; the buffer keeps its content between calls)
    const int ds_slot = kernel_slot >= 4 ? kernel_slot - 4 : -1;
    const int64_t need = (kernel_slot < 0 || ds_slot >= 0) && !own_delta
                             ? ds_workspace_need(p, s, &ntq, &ntk, &ds_bytes, &stat_bytes) : 0;
    if (ds_slot >= 0 && (need == 0 || need > ws_limit_bytes(device_index(dev)))) {
      if (acquired && lazy->dispose != nullptr) lazy->dispose(lazy);
      return FA_ERROR_NOT_SUPPORTED;
    }
    const bool nested = t_ws_nested.active;
    if (nested) {
      // (the caller holds the buffer and has set a part of it aside)
      if (need > 0 && (size_t)need <= t_ws_nested.bytes) {
        ds_ws = t_ws_nested.ptr;
        a.ds_ntq = ntq;
        a.ds_ntk = ntk;
        a.lse_scaled = reinterpret_cast<const float*>(static_cast<char*>(ds_ws) + ds_bytes);
        a.delta_prep = reinterpret_cast<const float*>(static_cast<char*>(ds_ws) + ds_bytes + stat_bytes);
      }
    } else if (need > 0 && need <= ws_limit_bytes(device_index(dev))) {
      if (!stream_is_capturing(stream)) {
        if (ws_acquire(device_index(dev), (size_t)need, stream, &ds_ws) == hipSuccess) {
          a.ds_ntq = ntq;
          a.ds_ntk = ntk;
          a.lse_scaled = reinterpret_cast<const float*>(static_cast<char*>(ds_ws) + ds_bytes);
          a.delta_prep = reinterpret_cast<const float*>(static_cast<char*>(ds_ws) + ds_bytes + stat_bytes);
        } else {
          ds_ws = nullptr;
          FA_LOG(2, "attn_bwd: no workspace of %lld bytes for dS, recomputing instead", (long long)need);
        }
      }
    }
    if (ds_slot >= 0 && ds_ws == nullptr) {
      if (acquired && lazy->dispose != nullptr) lazy->dispose(lazy);
      return FA_ERROR_NOT_SUPPORTED;          // under stream capture, or no memory
    }
    if (ds_ws != nullptr) {
      if (ds_slot < 0 || ds_slot == 0) err = fa::run_bwd_preprocess(dt, s.d, a, stream);
      a.ds_ws = ds_ws;
      if (err == hipSuccess && (ds_slot < 0 || ds_slot == 1))
        err = fa::run_bwd_dkdv(dt, s.d, a, s.windowed, s.bias, s.dropout, stream);
      if (err == hipSuccess && (ds_slot < 0 || ds_slot == 2)) err = fa::run_bwd_dqs(dt, s.d, a, stream);
      if (!nested) ws_release(device_index(dev), stream);
      if (acquired && lazy->dispose != nullptr) lazy->dispose(lazy);
      return (int)err;
    }
    if (kernel_slot == 0 || (kernel_slot < 0 && delta_launch))
      err = delta_launch ? fa::run_bwd_valu(dt, s.d, 0, a, stream) : fa::run_bwd_preprocess(dt, s.d, a, stream);
    const int order[2] = {delta_launch ? 1 : 2, delta_launch ? 2 : 1};
    for (int i = 0; i < 2 && err == hipSuccess; ++i) {
      const int slot = order[i];
      if (kernel_slot >= 0 && kernel_slot != slot) continue;
      if (slow)
        err = fa::run_bwd_valu(dt, s.d, slot, a, stream);
      else if (f32)
        err = fa::run_bwd_f32(s.d, slot, a, s.windowed, s.bias, s.dropout, stream);
      else if (big)
        err = fa::run_bwd_d512(dt, slot, a, s.windowed, s.bias, s.dropout, stream);
      else
        err = slot == 1 ? fa::run_bwd_dkdv(dt, s.d, a, s.windowed, s.bias, s.dropout, stream)
                        : fa::run_bwd_dq(dt, s.d, a, s.windowed, s.bias, s.dropout, stream);
    }
    if (acquired && lazy->dispose != nullptr) lazy->dispose(lazy);   // attn_bwd.cc:157
  } else {
    a.delta = nullptr;
    err = fa::run_bwd_fused(dt, s.d, a, s.windowed, s.bias, s.dropout, stream);
  }
  return (int)err;
}

int fa_attn_bwd(const fa_bwd_params* p, int32_t params_version, void* hip_stream,
                const fa_options* options) {
  return attn_bwd_impl(p, params_version, hip_stream, options, -1);
}

// ---- v2 positional entry points ------------------------------------------------------------
// Thin fills of the v3 params: is_causal -> windowed with the top-left sentinels, compact
// packed sequences -> varlen_type 1 (the reference's Python layer does the same,
// modules/flash/tests/aotriton_flash.py:141-196,277-335).

extern "C++" {
namespace {
template <typename V> V view_or_null(const V* t) { return t ? *t : V{}; }

void set_causal(bool is_causal, int8_t* type, int32_t* left, int32_t* right) {
  *type = is_causal ? FA_CAUSAL_WINDOWED : FA_CAUSAL_NONE;
  *left = *right = is_causal ? FA_WINDOW_TOP_LEFT : 0;
}

int v2_fwd(const fa_tensor4* q, const fa_tensor4* k, const fa_tensor4* v, const fa_tensor4* b,
           const fa_tensor1* cu_q, const fa_tensor1* cu_k, int32_t max_sq, int32_t max_sk, float sm_scale,
           const fa_tensor2* lse, const fa_tensor4* out, float dropout_p, const fa_tensor0* seed,
           const fa_tensor0* off1, int64_t off2, const fa_tensor0* seed_out, const fa_tensor0* off_out,
           const fa_tensor4* encoded_softmax, int32_t is_causal, const fa_tensor0* atomic, void* stream) {
  if (q == nullptr || k == nullptr || v == nullptr || out == nullptr) return FA_ERROR_INVALID_VALUE;
  fa_fwd_params p{};
  p.Q = *q; p.K = *k; p.V = *v; p.B = view_or_null(b);
  p.Sm_scale = sm_scale;
  p.L = view_or_null(lse);
  p.Out = *out;
  p.cu_seqlens_q = view_or_null(cu_q); p.cu_seqlens_k = view_or_null(cu_k);
  p.Max_seqlen_q = max_sq; p.Max_seqlen_k = max_sk;
  p.varlen_type = cu_q != nullptr ? FA_VARLEN_COMPACT : FA_VARLEN_NONE;
  p.dropout_p = dropout_p;
  p.philox_seed_ptr = view_or_null(seed); p.philox_offset1 = view_or_null(off1);
  p.philox_offset2 = (uint64_t)off2;
  p.philox_seed_output = view_or_null(seed_out); p.philox_offset_output = view_or_null(off_out);
  p.encoded_softmax = view_or_null(encoded_softmax);
  p.persistent_atomic_counter = view_or_null(atomic);
  set_causal(is_causal != 0, &p.causal_type, &p.window_left, &p.window_right);
  return fa_attn_fwd(&p, FA_FWD_PARAMS_VERSION, stream, nullptr);
}

int v2_bwd(const fa_tensor4* q, const fa_tensor4* k, const fa_tensor4* v, const fa_tensor4* b,
           const fa_tensor1* cu_q, const fa_tensor1* cu_k, int32_t max_sq, int32_t max_sk, float sm_scale,
           const fa_tensor4* out, const fa_tensor4* dout, const fa_tensor4* dq, const fa_tensor4* dk,
           const fa_tensor4* dv, const fa_tensor4* db, const fa_tensor2* lse, const fa_tensor2* delta,
           float dropout_p, const fa_tensor0* seed, const fa_tensor0* off1, int64_t off2, int32_t is_causal,
           int backend, void* stream) {
  if (q == nullptr || k == nullptr || v == nullptr || out == nullptr || dout == nullptr || dq == nullptr ||
      dk == nullptr || dv == nullptr || lse == nullptr)
    return FA_ERROR_INVALID_VALUE;
  fa_bwd_params p{};
  p.Q = *q; p.K = *k; p.V = *v; p.B = view_or_null(b);
  p.Sm_scale = sm_scale;
  p.Out = *out; p.DO = *dout; p.DQ = *dq; p.DK = *dk; p.DV = *dv; p.DB = view_or_null(db);
  p.L = *lse;
  p.D.eager = view_or_null(delta);
  p.cu_seqlens_q = view_or_null(cu_q); p.cu_seqlens_k = view_or_null(cu_k);
  p.Max_seqlen_q = max_sq; p.Max_seqlen_k = max_sk;
  p.varlen_type = cu_q != nullptr ? FA_VARLEN_COMPACT : FA_VARLEN_NONE;
  p.dropout_p = dropout_p;
  p.philox_seed_ptr = view_or_null(seed); p.philox_offset1 = view_or_null(off1);
  p.philox_offset2 = (uint64_t)off2;
  set_causal(is_causal != 0, &p.causal_type, &p.window_left, &p.window_right);
  fa_options opt{backend, 0};
  return fa_attn_bwd(&p, FA_BWD_PARAMS_VERSION, stream, &opt);
}
}  // namespace
}  // extern "C++"

int fa_v2_attn_fwd(const fa_tensor4* q, const fa_tensor4* k, const fa_tensor4* v, const fa_tensor4* b,
                   float sm_scale, const fa_tensor2* softmax_lse, const fa_tensor4* out, float dropout_p,
                   const fa_tensor0* philox_seed, const fa_tensor0* philox_offset1, int64_t philox_offset2,
                   const fa_tensor0* philox_seed_output, const fa_tensor0* philox_offset_output,
                   const fa_tensor4* encoded_softmax, int32_t is_causal, const fa_tensor0* atomic_for_causal,
                   void* hip_stream) {
  return v2_fwd(q, k, v, b, nullptr, nullptr, 0, 0, sm_scale, softmax_lse, out, dropout_p, philox_seed,
                philox_offset1, philox_offset2, philox_seed_output, philox_offset_output, encoded_softmax,
                is_causal, atomic_for_causal, hip_stream);
}

int fa_v2_attn_fwd_compact_varlen(const fa_tensor4* q, const fa_tensor4* k, const fa_tensor4* v,
                                  const fa_tensor4* b, const fa_tensor1* cu_seqlens_q,
                                  const fa_tensor1* cu_seqlens_k, int32_t max_seqlen_q, int32_t max_seqlen_k,
                                  float sm_scale, const fa_tensor2* softmax_lse, const fa_tensor4* out,
                                  float dropout_p, const fa_tensor0* philox_seed,
                                  const fa_tensor0* philox_offset1, int64_t philox_offset2,
                                  const fa_tensor0* philox_seed_output, const fa_tensor0* philox_offset_output,
                                  const fa_tensor4* encoded_softmax, int32_t is_causal,
                                  const fa_tensor0* atomic_for_causal, void* hip_stream) {
  if (cu_seqlens_q == nullptr || cu_seqlens_k == nullptr) return FA_ERROR_INVALID_VALUE;
  return v2_fwd(q, k, v, b, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, sm_scale, softmax_lse, out,
                dropout_p, philox_seed, philox_offset1, philox_offset2, philox_seed_output, philox_offset_output,
                encoded_softmax, is_causal, atomic_for_causal, hip_stream);
}

int fa_v2_attn_bwd(const fa_tensor4* q, const fa_tensor4* k, const fa_tensor4* v, const fa_tensor4* b,
                   float sm_scale, const fa_tensor4* out, const fa_tensor4* dout, const fa_tensor4* dq,
                   const fa_tensor4* dk, const fa_tensor4* dv, const fa_tensor4* db,
                   const fa_tensor2* softmax_lse, const fa_tensor2* delta, float dropout_p,
                   const fa_tensor0* philox_seed, const fa_tensor0* philox_offset1, int64_t philox_offset2,
                   int32_t is_causal, void* hip_stream) {
  if (delta == nullptr) return FA_ERROR_INVALID_VALUE;
  return v2_bwd(q, k, v, b, nullptr, nullptr, 0, 0, sm_scale, out, dout, dq, dk, dv, db, softmax_lse, delta,
                dropout_p, philox_seed, philox_offset1, philox_offset2, is_causal, 0, hip_stream);
}

int fa_v2_attn_bwd_fused(const fa_tensor4* q, const fa_tensor4* k, const fa_tensor4* v, const fa_tensor4* b,
                         float sm_scale, const fa_tensor4* out, const fa_tensor4* dout, const fa_tensor4* dq,
                         const fa_tensor4* dk, const fa_tensor4* dv, const fa_tensor4* db,
                         const fa_tensor2* softmax_lse, float dropout_p, const fa_tensor0* philox_seed,
                         const fa_tensor0* philox_offset1, int64_t philox_offset2, int32_t is_causal,
                         void* hip_stream) {
  return v2_bwd(q, k, v, b, nullptr, nullptr, 0, 0, sm_scale, out, dout, dq, dk, dv, db, softmax_lse, nullptr,
                dropout_p, philox_seed, philox_offset1, philox_offset2, is_causal, 1, hip_stream);
}

int fa_v2_attn_bwd_compact_varlen(const fa_tensor4* q, const fa_tensor4* k, const fa_tensor4* v,
                                  const fa_tensor1* cu_seqlens_q, const fa_tensor1* cu_seqlens_k,
                                  int32_t max_seqlen_q, int32_t max_seqlen_k, const fa_tensor4* b, float sm_scale,
                                  const fa_tensor4* out, const fa_tensor4* dout, const fa_tensor4* dq,
                                  const fa_tensor4* dk, const fa_tensor4* dv, const fa_tensor4* db,
                                  const fa_tensor2* softmax_lse, const fa_tensor2* delta, float dropout_p,
                                  const fa_tensor0* philox_seed, const fa_tensor0* philox_offset1,
                                  int64_t philox_offset2, int32_t is_causal, void* hip_stream) {
  if (cu_seqlens_q == nullptr || cu_seqlens_k == nullptr || delta == nullptr) return FA_ERROR_INVALID_VALUE;
  return v2_bwd(q, k, v, b, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, sm_scale, out, dout, dq, dk,
                dv, db, softmax_lse, delta, dropout_p, philox_seed, philox_offset1, philox_offset2, is_causal, 0,
                hip_stream);
}

void fa_set_bwd_workspace_limit(int64_t bytes) { g_ws_limit.store(bytes, std::memory_order_relaxed); }

int fa_trim_workspace(void) {
  hipError_t err = hipSuccess;
  for (int d = 0; d < kMaxDevices; ++d) {
    std::lock_guard<std::mutex> lock(g_ws[d].mutex);
    if (g_ws[d].ptr != nullptr) {
      const hipError_t e = hipFree(g_ws[d].ptr);      // waits for the device first
      g_ws[d].ptr = nullptr; g_ws[d].bytes = 0; g_ws[d].used = false;
      if (err == hipSuccess) err = e;
    }
  }
  return (int)err;
}

int fa_attn_bwd_noalloc(const fa_bwd_params* p, int32_t params_version, void* hip_stream) {
  return attn_bwd_impl(p, params_version, hip_stream, nullptr, -1, true);
}

int fa_attn_bwd_kernel(const fa_bwd_params* p, int32_t params_version, void* hip_stream,
                       int32_t kernel_slot) {
  if (kernel_slot < 0 || kernel_slot > 6) return FA_ERROR_INVALID_VALUE;
  return attn_bwd_impl(p, params_version, hip_stream, nullptr, kernel_slot);
}

}  // extern "C"
