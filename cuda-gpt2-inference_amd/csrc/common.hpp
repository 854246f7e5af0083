// Shared host/device helpers for the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "gpt2_mi355x.h"

namespace g2 {

// ---- host-side error plumbing --------------------------------------------
char* last_error_buffer();  // thread-local, 512 bytes (defined in gpt2.hip)

// The stream every launcher of the calling thread uses (gpt2hip_set_stream); the null
// stream until set.  Defined in gpt2.hip.
hipStream_t& stream_slot();
inline hipStream_t stream() { return stream_slot(); }

// The K-split workspace that matmul_forward / matmul_forward_gelu of the calling thread use
// (gpt2hip_set_workspace); none until set.  Defined in gpt2.hip.
struct ThreadWorkspace {
  void* ptr = nullptr;
  size_t bytes = 0;
};
ThreadWorkspace& workspace_slot();

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

#define G2_HIP(expr)                                                                       \
  do {                                                                                     \
    hipError_t e_ = (expr);                                                                \
    if (e_ != hipSuccess)                                                                  \
      return g2::fail(GPT2HIP_EHIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), \
                      __FILE__, __LINE__);                                                 \
  } while (0)

// After a kernel launch: picks up launch-configuration errors without syncing.
#define G2_LAUNCH_CHECK(name)                                                            \
  do {                                                                                   \
    hipError_t e_ = hipGetLastError();                                                   \
    if (e_ != hipSuccess)                                                                \
      return g2::fail(GPT2HIP_EHIP, "launch of %s failed: %s", name, hipGetErrorString(e_)); \
  } while (0)

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

[[noreturn]] inline void die(const char* what) {
  fprintf(stderr, "[gpt2_mi355x] %s: %s\n", what, last_error_buffer());
  abort();
}

constexpr int kWave = 64;

#if defined(__HIPCC__)
// ---- device helpers --------------------------------------------------------
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Data-parallel-primitive move: value of `v` from the lane selected by CTRL.
template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// All-lanes sum over a 64-wide wavefront: four DPP steps inside each row of 16
// lanes (quad swaps, half-row mirror, row mirror), then two cross-row exchanges.
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp<0x141>(v);  // row_half_mirror
  v += dpp<0x140>(v);  // row_mirror
  v += __shfl_xor(v, 16, 64);
  v += __shfl_xor(v, 32, 64);
  return v;
}

// Sum over each row of 16 lanes (all 16 lanes of the row receive it).
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp<0x141>(v);  // row_half_mirror
  v += dpp<0x140>(v);  // row_mirror
  return v;
}

// (value, index) combination of an argmax: the larger value wins, the smaller index
// among equal values.  NaN never wins (every comparison with it is false).
// Written with selects: as branches, a chain of these turns into divergent control flow.
__device__ __forceinline__ void argmax_combine(float& v, int& i, float ov, int oi) {
  const bool take = (ov > v) | ((ov == v) & (oi < i));
  v = take ? ov : v;
  i = take ? oi : i;
}

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp<0xB1>(v));
  v = fmaxf(v, dpp<0x4E>(v));
  v = fmaxf(v, dpp<0x141>(v));
  v = fmaxf(v, dpp<0x140>(v));
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  v = fmaxf(v, __shfl_xor(v, 32, 64));
  return v;
}

// ---- cache-bypassing accesses for data that other workgroups wrote in this launch ---------
// The eight XCDs' L2 caches are not coherent with each other; data handed from one workgroup
// to another inside a launch is written and read with the sc0 sc1 policy (served by the
// memory side) instead of fencing the whole L2.  128-bit accesses go through buffer
// instructions, whose builtins take the cache policy and leave the bookkeeping of loads in
// flight to the compiler.
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
constexpr int kBypass = 0x11;  // sc0 | sc1
struct Bypass {
  __amdgpu_buffer_rsrc_t rsrc;
  __device__ __forceinline__ Bypass(const float* base, size_t floats)
      : rsrc(__builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, (int)(floats * sizeof(float)),
                                               0x00020000)) {}
  // float_index: this lane's first float (reads past `floats` return zero)
  __device__ __forceinline__ f32x4 load4(int float_index) const {
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, float_index * 4, 0, kBypass));
  }
  __device__ __forceinline__ void store4(int float_index, f32x4 v) const {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), rsrc, float_index * 4, 0, kBypass);
  }
};
__device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(0)" : : : "memory"); }
__device__ __forceinline__ float load_bypass(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_bypass(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// tanh-GELU, 0.5x(1+tanh(u)) with u = sqrt(2/pi)(x + 0.044715x^3), the formula of
// reference 9_matmul_async_cg_tf32_gelu.cuh:5-11, evaluated through the identity
// 0.5(1+tanh(u)) = 1/(1+exp(-2u)): one hardware exp2 and one reciprocal, and no
// cancellation in 1+tanh(u) for negative x.
__device__ __forceinline__ float gelu_tanh(float x) {
  const float k = 0.7978845608028654f;            // sqrt(2/pi)
  const float c = -2.0f * 1.4426950408889634f * k;  // -2 log2(e) sqrt(2/pi)
  const float u = x + 0.044715f * x * x * x;
  const float e = __builtin_amdgcn_exp2f(c * u);  // exp(-2u); +inf for very negative x
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}
#endif

// The <= 16-row GEMM with optional fused input layernorm (ln_w, ln_b: over K) and fused
// residual add (resid, may alias out): out = resid + act(LN(inp) . weight^T + bias).
bool skinny_supported(int M, int K, bool ln, const void* inp, const void* weight);
int skinny_launch(float* out, const float* inp, const float* weight, const float* bias,
                  const float* ln_w, const float* ln_b, const float* resid, int M, int K, int N,
                  bool gelu);

// Decode-step attention of one new position per sequence against the key/value cache
// (kc, vc: (B, NH, maxT, hs)); appends the new key/value at `pos`.  qkv is (B, 3C).
int attention_decode_launch(float* out, const float* qkv, float* kc, float* vc, int B, int pos,
                            int maxT, int C, int NH);
// Copies a prompt's keys and values from packed qkv (B, T, 3C) into the cache.
int kv_store_launch(float* kc, float* vc, const float* qkv, int B, int T, int maxT, int C, int NH);

// One decode step as a single persistent kernel (decode.hip): every pointer is device memory.
constexpr int kDecodeMaxBatch = 16;  // sequences the persistent decode-step kernel takes
constexpr int kDecodeMaxSplits = 4;  // ranges of positions per (sequence, head) in its attention phase
struct DecodeStep {
  const float *wte, *wpe_row, *ln1w, *ln1b, *qkvw, *qkvb, *attprojw, *attprojb, *ln2w, *ln2b, *fcw,
      *fcb, *fcprojw, *fcprojb, *lnfw, *lnfb;
  const int* ids;      // (B) new token of every sequence
  float* kv;           // keys of layer l at kv + 2*l*plane, values at kv + (2*l+1)*plane: (B, NH, maxT, 64)
  size_t plane;
  // handed between workgroups: qkv (B,3C) row-major; x, atty (16,C) and h (16,4C) in granules
  // of 4 sequences x 4 channels (see decode.hip)
  float *x, *qkv, *atty, *h;
  // attention in att_splits > 1 ranges per (sequence, head): their unnormalised outputs
  // (att_splits x the layout of atty) and (maximum, sum) pairs
  float *att_part, *att_ml;
  int att_splits;
  float* logits;              // (B,V)
  unsigned* flags;            // [gridDim.x * FLAG_STRIDE] epochs, then the error word
  unsigned* error_host;       // pinned host word (device address) that receives the error word too
  unsigned epoch0;            // flags hold values below epoch0 + 1 when the kernel starts
  unsigned spin_limit;
  // optional probe: 100 MHz wall clock of every workgroup g of the G = 256 when it has finished
  // phase p's work (trace[(2p) * G + g]) and when it has passed the barrier after it
  // (trace[(2p+1) * G + g])
  unsigned long long* trace;
  int B, C, L, NH, V, pos, maxT;
};
// Whether the persistent kernel takes the model at B sequences on this device; the bytes of
// its flag array (zero-filled by the owner before the first step); the launch itself, which
// uses barrier epochs step.epoch0 + 1 .. step.epoch0 + 5 * L.
bool decode_step_supported(const GPT2Config& c, int B, int device);
size_t decode_step_flag_bytes(int device);
size_t decode_step_activation_floats(const GPT2Config& c);      // DecodeStep::x .. att_ml, one buffer
int decode_step_attention_splits(const GPT2Config& c, int B, int pos);  // DecodeStep::att_splits
size_t decode_step_probe_slots(int num_layers);  // clock slots DecodeStep::trace needs
int decode_step_launch(const DecodeStep& step, const GPT2Config& c, int device);

// encoder_forward with an optional on-device check of the token ids against the
// vocabulary size V (V = 0: ids are trusted, as the reference trusts them).
int encoder_launch(float* out, const int* inp, const float* wte, const float* wpe, int B, int T,
                   int C, int V);

}  // namespace g2
