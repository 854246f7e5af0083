// layernorm_forward and fused_residual_layernorm_forward for gfx950.
//
// One 64-lane wavefront owns one row.  The row (or the sum of the two input
// rows) is read once with 128-bit loads and kept in registers; mean and
// variance are two passes over those registers (llm.c's two-pass arithmetic,
// not the E[x^2]-m^2 shortcut of reference 3_layernorm_warp.cuh:49-50), reduced
// across the wave with DPP; the normalised row and, for the fused form, the
// residual sum are written with 128-bit stores.  HBM traffic is the compulsory
// one pass: 2 reads + 2 writes of the row for the fused form.
#include "common.hpp"

namespace g2 {

constexpr int kWavesPerBlock = 4;  // 256 threads

// One (N, C) array as a buffer: 128-bit accesses at a 32-bit byte offset, loads non-temporal,
// stores non-temporal or plain.
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
struct Stream {
  __amdgpu_buffer_rsrc_t rsrc;
  __device__ __forceinline__ Stream(const float* base, int N, int C)
      : rsrc(__builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, (int)((size_t)N * C * 4), 0x00020000)) {}
  __device__ __forceinline__ f32x4 load(int byte) const {
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte, 0, 2));
  }
  template <bool NT>
  __device__ __forceinline__ void store(int byte, f32x4 v) const {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), rsrc, byte, 0, NT ? 2 : 0);
  }
};

// NV float4 per lane cover C <= 256*NV.  FUSED adds inp2 and stores the sum.  A wave
// owns ROWS consecutive rows and issues all of their loads before it touches any of
// them: at N = 8192 four rows per wave (a quarter of the waves, four times the bytes
// in flight per wave) moved 71 % of HBM peak against 62-67 % for one row per wave, and at
// C = 1024 eight rows per wave 75 % against 70.6 % for four (at C = 768 eight change
// nothing).  The plain form, with half the traffic per row, does best with two rows per
// wave and streaming (non-temporal) stores: 68 / 72 % at C = 768 / 1024 against 65 / 63 %.
// EXACT (C == 256*NV and N % ROWS == 0, true for GPT-2) removes every bounds check, so
// that the loads are issued as one unconditional batch.
// NTS: non-temporal stores.
// BY_STREAM (fused, exact form only): the wave requests all its rows of inp1 and then all its
// rows of inp2 -- two runs of ROWS*C*4 consecutive bytes -- instead of alternating between
// the two arrays every kilobyte.  With streaming stores this moved C = 768 from 17.8 to 16.9 us
// per launch at N = 8192 (70.6 -> 74.6 % of HBM peak); at C = 1024 with eight rows per wave
// neither change pays (22.2 us = 75.6 % as it is, 22.4-23.6 us with either or both).
// BUF (fused, exact form only): the four big arrays are addressed as buffers (a scalar
// descriptor and one 32-bit byte offset per lane, the row and chunk as immediates) instead
// of 64-bit pointers: fewer address instructions ahead of the first load, 17.3 -> 16.8 us
// at C = 768 (at C = 1024 with eight rows per wave it changes nothing: 22.5 / 22.7 us).
// Needs N*C*4 < 2^31.
template <int NV, int ROWS, bool FUSED, bool EXACT, bool NTS, bool BY_STREAM = false,
          bool BUF = false>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void layernorm_rows_kernel(
    float* res_out, float* out, float* __restrict__ mean, float* __restrict__ rstd,
    const float* inp1, const float* inp2, const float* __restrict__ weight,
    const float* __restrict__ bias, int N, int C) {
  const int lane = threadIdx.x & (kWave - 1);
  const int row0 = (blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6)) * ROWS;
  if (row0 >= N) return;
  const int C4 = C >> 2;

  f32x4 v[ROWS][NV];
  [[maybe_unused]] const int lane_byte = row0 * C * 4 + lane * 16;  // BUF: this lane's first chunk
  [[maybe_unused]] const Stream X1(inp1, N, C), X2(inp2, N, C), RO(res_out, N, C), O(out, N, C);
  if constexpr (BUF) {
    static_assert(FUSED && EXACT, "BUF is a form of the fused kernel without bounds checks");
    const int row_bytes = C * 4;
    if constexpr (BY_STREAM) {
      f32x4 u[ROWS][NV];
#pragma unroll
      for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int j = 0; j < NV; j++) v[r][j] = X1.load(lane_byte + r * row_bytes + j * 1024);
#pragma unroll
      for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int j = 0; j < NV; j++) u[r][j] = X2.load(lane_byte + r * row_bytes + j * 1024);
#pragma unroll
      for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int j = 0; j < NV; j++) v[r][j] += u[r][j];
    } else {
#pragma unroll
      for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int j = 0; j < NV; j++)
          v[r][j] = X1.load(lane_byte + r * row_bytes + j * 1024) + X2.load(lane_byte + r * row_bytes + j * 1024);
    }
  } else if constexpr (BY_STREAM) {
    static_assert(FUSED && EXACT, "BY_STREAM is a form of the fused kernel without bounds checks");
    const f32x4* x1 = reinterpret_cast<const f32x4*>(inp1) + (size_t)row0 * C4 + lane;
    const f32x4* x2 = reinterpret_cast<const f32x4*>(inp2) + (size_t)row0 * C4 + lane;
    f32x4 u[ROWS][NV];
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
      for (int j = 0; j < NV; j++) v[r][j] = __builtin_nontemporal_load(x1 + r * C4 + j * kWave);
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
      for (int j = 0; j < NV; j++) u[r][j] = __builtin_nontemporal_load(x2 + r * C4 + j * kWave);
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
      for (int j = 0; j < NV; j++) v[r][j] += u[r][j];
  } else {
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
      // rows past N: reloaded, never stored
      const size_t base = (size_t)(EXACT ? row0 + r : min(row0 + r, N - 1)) * C4;
      const f32x4* x1 = reinterpret_cast<const f32x4*>(inp1) + base;
      const f32x4* x2 = FUSED ? reinterpret_cast<const f32x4*>(inp2) + base : nullptr;
#pragma unroll
      for (int j = 0; j < NV; j++) {
        const int c = lane + j * kWave;
        f32x4 a = {0.f, 0.f, 0.f, 0.f};
        if (EXACT || c < C4) {
          a = __builtin_nontemporal_load(x1 + c);
          if (FUSED) a += __builtin_nontemporal_load(x2 + c);
        }
        v[r][j] = a;
      }
    }
  }

  const f32x4* w4 = reinterpret_cast<const f32x4*>(weight);
  const f32x4* b4 = reinterpret_cast<const f32x4*>(bias);
  float my_mean = 0.f, my_rstd = 0.f;  // lane r keeps the statistics of the wave's row r
#pragma unroll
  for (int r = 0; r < ROWS; r++) {
    const int row = row0 + r;
    if (!EXACT && row >= N) break;
    const size_t base = (size_t)row * C4;
    if (FUSED) {
      f32x4* ro = reinterpret_cast<f32x4*>(res_out) + base;
#pragma unroll
      for (int j = 0; j < NV; j++) {
        const int c = lane + j * kWave;
        if (EXACT || c < C4) {
          if constexpr (BUF)
            RO.template store<NTS>(lane_byte + r * C * 4 + j * 1024, v[r][j]);
          else if (NTS)
            __builtin_nontemporal_store(v[r][j], ro + c);
          else
            ro[c] = v[r][j];
        }
      }
    }

    float s = 0.f;
#pragma unroll
    for (int j = 0; j < NV; j++) s += (v[r][j].x + v[r][j].y) + (v[r][j].z + v[r][j].w);
    const float m = wave_sum(s) / (float)C;

    float q = 0.f;
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int c = lane + j * kWave;
      if (EXACT || c < C4) {
        const f32x4 d = v[r][j] - m;
        q += (d.x * d.x + d.y * d.y) + (d.z * d.z + d.w * d.w);
      }
    }
    const float var = wave_sum(q) / (float)C;
    const float rs = 1.0f / sqrtf(var + 1e-5f);

    if (FUSED) {
      if (lane == r) {
        my_mean = m;
        my_rstd = rs;
      }
    } else if (lane == 0) {
      if (mean) mean[row] = m;
      if (rstd) rstd[row] = rs;
    }

    f32x4* o = reinterpret_cast<f32x4*>(out) + base;
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int c = lane + j * kWave;
      if (EXACT || c < C4) {
        const f32x4 n = (v[r][j] - m) * rs;
        if constexpr (BUF)
          O.template store<NTS>(lane_byte + r * C * 4 + j * 1024, n * w4[c] + b4[c]);
        else if (NTS)
          __builtin_nontemporal_store(n * w4[c] + b4[c], o + c);
        else
          o[c] = n * w4[c] + b4[c];
      }
    }
  }
  // fused form: one store of ROWS consecutive floats per wave and array instead of one per
  // row (77 % of HBM peak against 75-76 % at C = 1024; the plain form, with two rows per
  // wave, was slower with it)
  if (FUSED && lane < ROWS && (EXACT || row0 + lane < N)) {
    if (mean) mean[row0 + lane] = my_mean;
    if (rstd) rstd[row0 + lane] = my_rstd;
  }
}

constexpr int kRowsPerBlock = kWavesPerBlock;  // generic kernel: one row per wave

// Any C, any alignment: one wave per row, three passes over global memory.
template <bool FUSED>
__global__ __launch_bounds__(kRowsPerBlock* kWave) void layernorm_rows_generic_kernel(
    float* res_out, float* out, float* mean, float* rstd, const float* inp1, const float* inp2,
    const float* weight, const float* bias, int N, int C) {
  const int lane = threadIdx.x & (kWave - 1);
  const int row = blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  if (row >= N) return;
  const float* x1 = inp1 + (size_t)row * C;
  const float* x2 = FUSED ? inp2 + (size_t)row * C : nullptr;
  float* ro = FUSED ? res_out + (size_t)row * C : nullptr;
  float s = 0.f;
  for (int c = lane; c < C; c += kWave) {
    float a = x1[c];
    if (FUSED) {
      a += x2[c];
      ro[c] = a;  // each lane re-reads only what it wrote itself
    }
    s += a;
  }
  const float* x = FUSED ? ro : x1;
  const float m = wave_sum(s) / (float)C;
  float q = 0.f;
  for (int c = lane; c < C; c += kWave) {
    const float d = x[c] - m;
    q += d * d;
  }
  const float rs = 1.0f / sqrtf(wave_sum(q) / (float)C + 1e-5f);
  if (lane == 0) {
    if (mean) mean[row] = m;
    if (rstd) rstd[row] = rs;
  }
  float* o = out + (size_t)row * C;
  for (int c = lane; c < C; c += kWave) o[c] = ((x[c] - m) * rs) * weight[c] + bias[c];
}

template <bool FUSED>
static int launch_layernorm(float* res_out, float* out, float* mean, float* rstd,
                            const float* inp1, const float* inp2, const float* weight,
                            const float* bias, int B, int T, int C) {
  const char* name = FUSED ? "fused_residual_layernorm_forward" : "layernorm_forward";
  if (B < 0 || T < 0 || C < 1) return fail(GPT2HIP_EINVAL, "%s: bad shape B=%d T=%d C=%d", name, B, T, C);
  const long long N64 = (long long)B * T;
  if (N64 > 0x7fffffffLL) return fail(GPT2HIP_EINVAL, "%s: B*T too large", name);
  const int N = (int)N64;
  if (N == 0) return GPT2HIP_OK;
  if (!out || !inp1 || !weight || !bias || (FUSED && (!res_out || !inp2)))
    return fail(GPT2HIP_EINVAL, "%s: null pointer", name);
  const dim3 block(kWavesPerBlock * kWave);
  const bool vec = (C % 4 == 0) && C <= 4096 && aligned16(out) && aligned16(inp1) &&
                   aligned16(weight) && aligned16(bias) &&
                   (!FUSED || (aligned16(res_out) && aligned16(inp2)));
  // Several rows per wave once there are enough rows to still fill the chip.  The fused form,
  // timed over N = 512 .. 8192 at C = 768 and 1024 (us; rows per wave 1 / 2 / 4 / 8):
  //   C = 768:  N = 8192: 18.4 / 18.2 / 16.6 / 18.3;  4096: 10.4 / 8.8 / 9.2 / 11.4;
  //             2048: 5.5 / 5.3 / 7.2 / 9.9;  1024: 3.7 / 4.3 / 6.6 / 9.3
  //   C = 1024: N = 8192: 24.3 / 23.6 / 22.3 / 21.5;  4096: 14.0 / 11.6 / 12.4 / 14.4;
  //             2048: 7.5 / 6.4 / 7.6 / 13.4;  1024: 4.9 / 5.0 / 6.8 / 12.3
  // (eight rows at N = 4096 are 128 workgroups: half the chip idle).  The plain form takes two rows
  // per wave from 4096 rows on and one below, always without bounds checks where C is a multiple of
  // 256 and N of 8 (one row with bounds checks had been the form below 4096 rows: 6.9 -> 5.3 us at
  // 3072 x 1024, 6.3 -> 5.5 at 2048 x 1280).
  const bool wide = N >= 4096;
#define G2_LN(NV, ROWS, EXACT, NTS, ...)                                                        \
  hipLaunchKernelGGL((layernorm_rows_kernel<NV, ROWS, FUSED, EXACT, NTS, ##__VA_ARGS__>),       \
                     dim3((N + kWavesPerBlock * ROWS - 1) / (kWavesPerBlock * ROWS)), block, 0, stream(), \
                     res_out, out, mean, rstd, inp1, inp2, weight, bias, N, C)
#define G2_LN_ROWS(NV)                                              \
  if (C == 256 * NV && N % 8 == 0 && (long long)N * C * 4 < (1LL << 31)) { \
    if (!FUSED && wide) {                                           \
      G2_LN(NV, 2, true, true);                                     \
    } else if (!FUSED) {                                            \
      G2_LN(NV, 1, true, true);                                     \
    } else if (NV == 4 && N >= 8192) {                              \
      G2_LN(NV, 8, true, false);                                    \
    } else if (N >= 8192) {                                         \
      G2_LN(NV, 4, true, true, FUSED, FUSED);                       \
    } else if (N >= 2048) {                                         \
      G2_LN(NV, 2, true, true, FUSED, FUSED);                       \
    } else if (NV == 4) {                                           \
      G2_LN(NV, 1, true, false);                                    \
    } else {                                                        \
      G2_LN(NV, 1, true, true, FUSED, FUSED);                       \
    }                                                               \
  } else if (wide) {                                                \
    G2_LN(NV, 4, false, false);                                     \
  } else {                                                          \
    G2_LN(NV, 1, false, false);                                     \
  }
  if (!vec) {
    hipLaunchKernelGGL((layernorm_rows_generic_kernel<FUSED>),
                       dim3((N + kRowsPerBlock - 1) / kRowsPerBlock), block, 0, stream(), res_out, out,
                       mean, rstd, inp1, inp2, weight, bias, N, C);
  } else if (C <= 256) {
    G2_LN_ROWS(1)
  } else if (C <= 512) {
    G2_LN_ROWS(2)
  } else if (C <= 768) {
    G2_LN_ROWS(3)
  } else if (C <= 1024) {
    G2_LN_ROWS(4)
  } else if (C <= 1280) {
    G2_LN_ROWS(5)  // GPT-2 large
  } else if (C <= 1792) {
    G2_LN_ROWS(7)  // GPT-2 XL (1600 channels: 6.25 chunks per lane, the form with bounds checks)
  } else if (C <= 2048) {
    G2_LN_ROWS(8)
  } else {
    G2_LN(16, 1, false, false);
  }
#undef G2_LN_ROWS
#undef G2_LN
  G2_LAUNCH_CHECK(name);
  return GPT2HIP_OK;
}

}  // namespace g2

extern "C" {

int layernorm_forward_status(float* out, float* mean, float* rstd, const float* inp,
                             const float* weight, const float* bias, int B, int T, int C) {
  return g2::launch_layernorm<false>(nullptr, out, mean, rstd, inp, nullptr, weight, bias, B, T, C);
}

void layernorm_forward(float* out, float* mean, float* rstd, const float* inp, const float* weight,
                       const float* bias, int B, int T, int C) {
  if (layernorm_forward_status(out, mean, rstd, inp, weight, bias, B, T, C)) g2::die("layernorm_forward");
}

int fused_residual_layernorm_forward_status(float* res_out, float* layernorm_out, float* mean,
                                            float* rstd, const float* inp1, const float* inp2,
                                            const float* weight, const float* bias, int B, int T,
                                            int C) {
  return g2::launch_layernorm<true>(res_out, layernorm_out, mean, rstd, inp1, inp2, weight, bias, B,
                                    T, C);
}

void fused_residual_layernorm_forward(float* res_out, float* layernorm_out, float* mean,
                                      float* rstd, const float* inp1, const float* inp2,
                                      const float* weight, const float* bias, int B, int T, int C) {
  if (fused_residual_layernorm_forward_status(res_out, layernorm_out, mean, rstd, inp1, inp2,
                                              weight, bias, B, T, C))
    g2::die("fused_residual_layernorm_forward");
}

}  // extern "C"
