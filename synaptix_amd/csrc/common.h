// Shared device helpers for the gfx950 kernels: types, conversions, wave and block
// reductions, and the error channel of the C entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <mutex>

#define SYN_WAVE 64
#define SYN_PAGE 64  // tokens per cache page; the host side asserts the same number

typedef __bf16 bf16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

// ---- error channel: every entry point returns 0, or a code after syn_set_error ----
// One translation unit of each library places SYN_DEFINE_ERROR_CHANNEL at file scope.
#define SYN_EXPORT extern "C" __attribute__((visibility("default")))
SYN_EXPORT const char* syn_last_error();
void syn_set_error(const char* fmt, ...);
#define SYN_DEFINE_ERROR_CHANNEL                                   \
  static thread_local char syn_error_text[512];                    \
  SYN_EXPORT const char* syn_last_error() { return syn_error_text; } \
  void syn_set_error(const char* fmt, ...) {                       \
    va_list ap;                                                    \
    va_start(ap, fmt);                                             \
    vsnprintf(syn_error_text, sizeof(syn_error_text), fmt, ap);    \
    va_end(ap);                                                    \
  }
#define SYN_CHECK(cond, ...)            \
  do {                                  \
    if (!(cond)) {                      \
      syn_set_error(__VA_ARGS__);       \
      return 1;                         \
    }                                   \
  } while (0)
#define SYN_LAUNCH_CHECK(name)                                          \
  do {                                                                  \
    hipError_t e_ = hipGetLastError();                                  \
    if (e_ != hipSuccess) {                                             \
      syn_set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
      return 2;                                                         \
    }                                                                   \
  } while (0)

// ---- once on each device ----
// What has to happen once on a device before a kernel's first launch there (raising its limit of dynamic LDS,
// looking up a device symbol): the flags are kept per device under a lock, so that two threads or two GPUs
// neither skip the step nor run it twice.
#define SYN_MAX_DEVICES 64
struct OncePerDevice {
  std::mutex lock;
  bool done[SYN_MAX_DEVICES] = {};
};
template <typename F>
static inline hipError_t once_per_device(OncePerDevice& once, F&& step) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= SYN_MAX_DEVICES) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> hold(once.lock);
  if (once.done[dev]) return hipSuccess;
  e = step();
  if (e == hipSuccess) once.done[dev] = true;
  return e;
}

// Compute units of the current device (256 on an MI355X), asked once a device: what the hosts' rules for tiles and
// splits fill.  (The Python rules ask the same number: kernels/ops.py, compute_units.)
static inline int syn_compute_units() {
  static int of_device[SYN_MAX_DEVICES];
  static OncePerDevice once;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= SYN_MAX_DEVICES) return 256;
  const hipError_t e = once_per_device(once, [&] {
    int n = 0;
    const hipError_t r = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    of_device[dev] = (r == hipSuccess && n > 0) ? n : 256;
    return hipSuccess;
  });
  return e == hipSuccess ? of_device[dev] : 256;
}

// ---- conversions ----
template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16>(bf16 v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return (bf16)v; }

// a weight vector that is bf16 or float, chosen at run time
__device__ __forceinline__ float load_gain(const void* w, int is_f32, int i) {
  return is_f32 ? ((const float*)w)[i] : (float)((const bf16*)w)[i];
}

// the gain of a norm: w[i], or offset + w[i] for checkpoints that store the gain as a difference from one
__device__ __forceinline__ float load_gain(const void* w, int is_f32, int i, float offset) {
  return offset + load_gain(w, is_f32, i);
}

// ---- the activation of a gated feed-forward: act(gate) * up, on 32-bit sums ----
// One place for every kernel that applies it (the epilogues of the gated products, the activation kernel
// of the 32-bit path).  `act` is a code that the host checks against SYN_ACT_COUNT before any launch;
// another activation is another case here and another name in the host's table.
#define SYN_ACT_SILU 0
#define SYN_ACT_COUNT 1
__device__ __forceinline__ float gate_activation(int act, float g) {
  switch (act) {
    default:  // SYN_ACT_SILU: z / (1 + e^-z)
      return g / (1.f + expf(-g));
  }
}
__device__ __forceinline__ float gated(int act, float gate, float up) { return gate_activation(act, gate) * up; }

// ---- what an attention kernel may do to a scaled score before the mask and the softmax ----
// A soft cap, cap * tanh(score / cap), and a penalty in the distance between query and key, - slope[head] * (q - k)
// (the linear bias of crates/synaptix-ops/src/pos/alibi.rs:47-66 for keys at or before the query).  Neither is set
// by the one architecture built here (slopes == nullptr, cap == 0: the kernels then run the code they ran before
// these arguments existed); they are what a position scheme that acts on the scores, or a capped attention, needs.
struct ScoreTerms {
  const float* slopes;   // [n_heads] or nullptr
  float softcap;         // 0: none
};
__device__ __forceinline__ bool score_terms_on(const ScoreTerms& t) { return t.slopes != nullptr || t.softcap > 0.f; }
// v: the scaled score in natural units; slope: of the query's head (0 without slopes)
__device__ __forceinline__ float score_with_terms(float v, float slope, float cap, int q_pos, int key) {
  if (cap > 0.f) v = cap * tanhf(v / cap);
  return v - slope * (float)(q_pos - key);
}

// ---- reductions over the 64 lanes of a wave ----
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, SYN_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, SYN_WAVE));
  return v;
}

// sum over a block of up to 1024 threads; `red` holds 16 floats of LDS; all threads get the result
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE;
  const int nw = (blockDim.x + SYN_WAVE - 1) / SYN_WAVE;
  __syncthreads();  // `red` may still be read from an earlier call
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += red[i];
  return t;
}

// ---- the order of V inside a bf16 cache page ----
// A bf16 V page of one kv head holds hd x 64 values (dims x tokens of the page) in the order in which
// the decode kernel's MFMA takes them: for each half h of the tokens and each 16 dims dt, the 64 lanes'
// 8 values (lane = 16 * ((token % 32) / 8) + dim % 16, element = token % 8) lie together, so that a
// fragment is one contiguous 1 KB load.  (A float page is plain [hd][64].)
__host__ __device__ __forceinline__ int v_page_offset(int hd, int d, int token) {
  return ((((token >> 5) * (hd >> 4) + (d >> 4)) * 64 + ((token >> 3) & 3) * 16 + (d & 15)) << 3) + (token & 7);
}

// ---- loads through a buffer descriptor, straight into LDS ----
// A base and a size in scalar registers, a 32-bit offset a lane, a further offset as a scalar: a load
// into LDS is then two instructions (LDS address into M0, the load), where a 64-bit address a lane
// costs vector adds and takes longer to issue.
struct BufferView {
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass of the compiler has no such type
  __amdgpu_buffer_rsrc_t r;
#endif
};
__device__ __forceinline__ BufferView buffer_view(const void* base, size_t bytes) {
  BufferView v;
#if defined(__HIP_DEVICE_COMPILE__)
  v.r = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, (int)(bytes > 0xffffffffull ? 0xffffffffull : bytes), 0x00020000);
#endif
  return v;
}
// 16 bytes a lane from base + lane_bytes + uniform_bytes to lds + 16 * lane (lds is the same for all lanes).
// STREAMED: the load is marked non-temporal, for data that is read once (a decode step's keys).
template <bool STREAMED = false>
__device__ __forceinline__ void buffer_to_lds16(const BufferView& v, void* lds, unsigned lane_bytes, int uniform_bytes) {
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_raw_ptr_buffer_load_lds(v.r, (__attribute__((address_space(3))) void*)lds, 16, lane_bytes, uniform_bytes, 0,
                                           STREAMED ? 2 : 0);
#endif
}
