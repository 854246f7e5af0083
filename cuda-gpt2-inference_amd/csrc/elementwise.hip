// Bandwidth-bound launchers: encoder_forward, residual_forward, gelu_forward,
// argmax_forward.  One pass over HBM each, 128-bit accesses where alignment
// allows, scalar tails otherwise.
#include "common.hpp"

namespace g2 {

constexpr int kBlock = 256;

// ---- encoder: out[b,t,:] = wte[ids[b,t],:] + wpe[t,:] ----------------------
// One thread per float4 of the output; the token id is a broadcast load.  With V > 0 an
// id outside [0, V) is not dereferenced: its row is filled with NaN instead, which shows
// in everything computed from it.
__global__ __launch_bounds__(kBlock) void encoder_vec_kernel(
    f32x4* __restrict__ out, const int* __restrict__ ids, const f32x4* __restrict__ wte,
    const f32x4* __restrict__ wpe, int T, int C4, size_t total4, int V) {
  const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= total4) return;
  const size_t bt = i / C4;
  const int c = (int)(i - bt * C4);
  const int t = (int)(bt % T);
  const int id = ids[bt];
  if (V > 0 && (unsigned)id >= (unsigned)V) {
    const float q = __builtin_nanf("");
    out[i] = f32x4{q, q, q, q};
    return;
  }
  out[i] = wte[(size_t)id * C4 + c] + wpe[(size_t)t * C4 + c];
}

__global__ __launch_bounds__(kBlock) void encoder_scalar_kernel(
    float* __restrict__ out, const int* __restrict__ ids, const float* __restrict__ wte,
    const float* __restrict__ wpe, int T, int C, size_t total, int V) {
  const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= total) return;
  const size_t bt = i / C;
  const int c = (int)(i - bt * C);
  const int t = (int)(bt % T);
  const int id = ids[bt];
  if (V > 0 && (unsigned)id >= (unsigned)V) {
    out[i] = __builtin_nanf("");
    return;
  }
  out[i] = wte[(size_t)id * C + c] + wpe[(size_t)t * C + c];
}

// ---- residual / gelu -----------------------------------------------------
// Each thread handles UNROLL float4, block-strided so that every load
// instruction of a wave covers 1 KiB of consecutive addresses.  Loads and stores are
// streaming (non-temporal): with ordinary stores residual moved 75 % and gelu 68 % of HBM
// peak, with streaming stores 81 % and 73 %.
constexpr int kUnroll = 4;

template <bool GELU>
__global__ __launch_bounds__(kBlock) void map_vec_kernel(f32x4* out, const f32x4* inp1,
                                                          const f32x4* inp2, size_t n4) {
  const size_t base = (size_t)blockIdx.x * (kBlock * kUnroll) + threadIdx.x;
  f32x4 a[kUnroll];
#pragma unroll
  for (int j = 0; j < kUnroll; j++) {
    const size_t i = base + (size_t)j * kBlock;
    if (i < n4) {
      a[j] = __builtin_nontemporal_load(inp1 + i);
      if (!GELU) a[j] += __builtin_nontemporal_load(inp2 + i);
    }
  }
#pragma unroll
  for (int j = 0; j < kUnroll; j++) {
    const size_t i = base + (size_t)j * kBlock;
    if (i < n4) {
      if (GELU) {
        f32x4 r;
        r.x = gelu_tanh(a[j].x);
        r.y = gelu_tanh(a[j].y);
        r.z = gelu_tanh(a[j].z);
        r.w = gelu_tanh(a[j].w);
        __builtin_nontemporal_store(r, out + i);
      } else {
        __builtin_nontemporal_store(a[j], out + i);
      }
    }
  }
}

template <bool GELU>
__global__ __launch_bounds__(kBlock) void map_scalar_kernel(float* out, const float* inp1,
                                                             const float* inp2, size_t start,
                                                             size_t n) {
  const size_t i = start + (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  out[i] = GELU ? gelu_tanh(inp1[i]) : inp1[i] + inp2[i];
}

template <bool GELU>
static int launch_map(const char* name, float* out, const float* inp1, const float* inp2, int N) {
  if (N < 0) return fail(GPT2HIP_EINVAL, "%s: N=%d", name, N);
  if (N == 0) return GPT2HIP_OK;
  if (!out || !inp1 || (!GELU && !inp2)) return fail(GPT2HIP_EINVAL, "%s: null pointer", name);
  const size_t n = (size_t)N;
  size_t done = 0;
  if (aligned16(out) && aligned16(inp1) && (GELU || aligned16(inp2))) {
    const size_t n4 = n / 4;
    if (n4) {
      const size_t per_block = (size_t)kBlock * kUnroll;
      const unsigned grid = (unsigned)((n4 + per_block - 1) / per_block);
      hipLaunchKernelGGL((map_vec_kernel<GELU>), dim3(grid), dim3(kBlock), 0, stream(),
                         reinterpret_cast<f32x4*>(out), reinterpret_cast<const f32x4*>(inp1),
                         reinterpret_cast<const f32x4*>(inp2), n4);
      G2_LAUNCH_CHECK(name);
    }
    done = n4 * 4;
  }
  if (done < n) {
    const unsigned grid = (unsigned)((n - done + kBlock - 1) / kBlock);
    hipLaunchKernelGGL((map_scalar_kernel<GELU>), dim3(grid), dim3(kBlock), 0, stream(), out, inp1, inp2,
                       done, n);
    G2_LAUNCH_CHECK(name);
  }
  return GPT2HIP_OK;
}

// ---- argmax ----------------------------------------------------------------
// One 256-thread block per row.  Every thread scans a strided subset in
// ascending index order (so "first maximum" is kept with a strict >), then
// (value, index) pairs are reduced with "larger value, or equal value and
// smaller index".
__global__ __launch_bounds__(kBlock) void argmax_rows_kernel(int* __restrict__ ids,
                                                              const float* __restrict__ logits,
                                                              int V) {
  const float* x = logits + (size_t)blockIdx.x * V;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  int c = threadIdx.x;
  for (; c + 3 * kBlock < V; c += 4 * kBlock) {
    const float a0 = x[c], a1 = x[c + kBlock], a2 = x[c + 2 * kBlock], a3 = x[c + 3 * kBlock];
    if (a0 > best) { best = a0; bi = c; }
    if (a1 > best) { best = a1; bi = c + kBlock; }
    if (a2 > best) { best = a2; bi = c + 2 * kBlock; }
    if (a3 > best) { best = a3; bi = c + 3 * kBlock; }
  }
  for (; c < V; c += kBlock) {
    const float a = x[c];
    if (a > best) { best = a; bi = c; }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float ov = __shfl_xor(best, off, 64);
    const int oi = __shfl_xor(bi, off, 64);
    argmax_combine(best, bi, ov, oi);
  }
  __shared__ float sv[kBlock / kWave];
  __shared__ int si[kBlock / kWave];
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    sv[wave] = best;
    si[wave] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kBlock / kWave; w++) argmax_combine(best, bi, sv[w], si[w]);
    // a row of all -inf / NaN never beats the initial value: report index 0
    ids[blockIdx.x] = (bi == 0x7fffffff) ? 0 : bi;
  }
}

// V > 0: token ids are checked against the vocabulary size on the device (see the kernels).
int encoder_launch(float* out, const int* inp, const float* wte, const float* wpe, int B, int T,
                   int C, int V) {
  if (B < 0 || T < 0 || C < 1) return fail(GPT2HIP_EINVAL, "encoder_forward: bad shape B=%d T=%d C=%d", B, T, C);
  const size_t total = (size_t)B * T * C;
  if (total == 0) return GPT2HIP_OK;
  if (!out || !inp || !wte || !wpe) return fail(GPT2HIP_EINVAL, "encoder_forward: null pointer");
  if (C % 4 == 0 && aligned16(out) && aligned16(wte) && aligned16(wpe)) {
    const size_t total4 = total / 4;
    hipLaunchKernelGGL(encoder_vec_kernel, dim3((unsigned)((total4 + kBlock - 1) / kBlock)),
                       dim3(kBlock), 0, stream(), reinterpret_cast<f32x4*>(out), inp,
                       reinterpret_cast<const f32x4*>(wte), reinterpret_cast<const f32x4*>(wpe), T,
                       C / 4, total4, V);
  } else {
    hipLaunchKernelGGL(encoder_scalar_kernel, dim3((unsigned)((total + kBlock - 1) / kBlock)),
                       dim3(kBlock), 0, stream(), out, inp, wte, wpe, T, C, total, V);
  }
  G2_LAUNCH_CHECK("encoder_forward");
  return GPT2HIP_OK;
}

}  // namespace g2

extern "C" {

int encoder_forward_status(float* out, const int* inp, const float* wte, const float* wpe, int B,
                           int T, int C) {
  return g2::encoder_launch(out, inp, wte, wpe, B, T, C, 0);
}

void encoder_forward(float* out, const int* inp, const float* wte, const float* wpe, int B, int T,
                     int C) {
  if (encoder_forward_status(out, inp, wte, wpe, B, T, C)) g2::die("encoder_forward");
}

int residual_forward_status(float* out, const float* inp1, const float* inp2, int N) {
  return g2::launch_map<false>("residual_forward", out, inp1, inp2, N);
}

void residual_forward(float* out, const float* inp1, const float* inp2, int N) {
  if (residual_forward_status(out, inp1, inp2, N)) g2::die("residual_forward");
}

int gelu_forward_status(float* out, const float* inp, int N) {
  return g2::launch_map<true>("gelu_forward", out, inp, nullptr, N);
}

void gelu_forward(float* out, const float* inp, int N) {
  if (gelu_forward_status(out, inp, N)) g2::die("gelu_forward");
}

int argmax_forward_status(int* ids, const float* logits, int N, int V) {
  using namespace g2;
  if (N < 0 || V < 1) return fail(GPT2HIP_EINVAL, "argmax_forward: bad shape N=%d V=%d", N, V);
  if (N == 0) return GPT2HIP_OK;
  if (!ids || !logits) return fail(GPT2HIP_EINVAL, "argmax_forward: null pointer");
  hipLaunchKernelGGL(argmax_rows_kernel, dim3(N), dim3(kBlock), 0, stream(), ids, logits, V);
  G2_LAUNCH_CHECK("argmax_forward");
  return GPT2HIP_OK;
}

void argmax_forward(int* ids, const float* logits, int N, int V) {
  if (argmax_forward_status(ids, logits, N, V)) g2::die("argmax_forward");
}

}  // extern "C"
