// attention_forward for gfx950: causal multi-head self-attention read straight
// from the packed qkv activations (B,T,3C) and written as (B,T,C) — the op of
// reference 3_flash_attention_permute.cuh:346-355 — as one flash-style kernel
// on the fp32 matrix cores.  The T x T scores never leave registers.
//
// Shape of the computation (head size 64).  A workgroup of 4 waves owns 128
// consecutive queries of one (batch, head); each wave owns 32 of them.  Keys
// and values are staged through LDS in tiles of 64 keys (fetched into
// registers one tile ahead, two LDS buffers, one barrier per tile); a wave
// consumes a tile as two sub-tiles of 32 keys.
//
// Per sub-tile a wave computes, with v_mfma_f32_32x32x2_f32,
//     S^T (32 keys x 32 queries) = K_sub (32 x 64) . Q^T (64 x 32)
// so that lane l owns query l%32 and holds 16 of that query's 32 scores
// (keys 8*(v/4) + 4*(l/32) + v%4, v = 0..15); lane l^32 holds the other 16.
// Row maxima and sums are therefore register reductions plus one exchange
// with lane l^32.  The probabilities are then used IN PLACE as the B operand of
//     O^T (64 x 32 queries) += V_sub^T (64 x 32 keys) . P^T (32 keys x 32 queries)
// because the accumulator layout of S^T is exactly a valid B-operand layout
// once the k index of each MFMA is read as "key 8*(v/4)+v%4 for lanes 0..31,
// that key + 4 for lanes 32..63"; the matching V rows are picked by address.
// (The reference bounces P through shared memory for this step,
// 2_flash_attention.cuh:227-240.)
//
// Q is held in registers for the whole kernel in the same k-permuted form the
// GEMM uses (lane half h holds hs = 8g+4h..+3 of group g), K tiles are stored
// with the same XOR chunk swizzle, and V rows are read as 64-bit pairs so that
// accumulator a (0/1) of lane l, register v holds output feature
// 16*(v/4) + 8*(l/32) + 2*(v%4) + a: eight consecutive floats per v/4, stored
// as two 128-bit writes.
#include "common.hpp"

namespace g2 {

constexpr int HS = 64;          // head size this kernel is built for
constexpr int BQ = 128;         // queries per workgroup (4 waves x 32)
constexpr int BKV = 64;         // keys per LDS tile
constexpr int KV_CH = HS / 4;   // 16-byte chunks per K/V row
constexpr int ATT_THREADS = 256;
constexpr int KV_PER = BKV * KV_CH / ATT_THREADS;  // chunks per thread per tensor = 4

__global__ __launch_bounds__(ATT_THREADS) void attention_flash_kernel(
    float* __restrict__ out, const float* __restrict__ qkv, int T, int NH, int nqt,
    float scale_log2e) {
  __shared__ f32x4 k_lds[2][BKV * KV_CH];
  __shared__ f32x4 v_lds[2][BKV * KV_CH];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int h32 = lane >> 5;
  const int l32 = lane & 31;

  // heaviest query tiles (most keys) are launched first
  const int bid = blockIdx.x;
  const int per_tile = gridDim.x / nqt;  // = B*NH
  const int qtile = nqt - 1 - bid / per_tile;
  const int bh = bid % per_tile;
  const int b = bh / NH, head = bh % NH;

  const int C = NH * HS;
  const size_t row_stride = (size_t)3 * C;
  const float* base = qkv + (size_t)b * T * row_stride + head * HS;
  const float* kbase = base + C;
  const float* vbase = base + 2 * C;

  const int q0 = qtile * BQ;          // first query of the workgroup
  const int qw = q0 + wave * 32;      // first query of this wave
  const int myq = qw + l32;           // this lane's query
  const int kv_end = min(T, q0 + BQ); // keys the workgroup needs: [0, kv_end)
  const int ntile = (kv_end + BKV - 1) / BKV;

  // ---- Q in registers: qreg[g] = Q[myq][8g+4h .. +3] --------------------
  f32x4 qreg[8];
  {
    const int qr = min(myq, T - 1);  // clamp: out-of-range queries compute garbage, never stored
    const f32x4* qp = reinterpret_cast<const f32x4*>(base + (size_t)qr * row_stride);
#pragma unroll
    for (int g = 0; g < 8; g++) qreg[g] = qp[2 * g + h32];
  }

  // ---- K/V staging ---------------------------------------------------------
  f32x4 kst[KV_PER], vst[KV_PER];
  int st_row[KV_PER], st_chunk[KV_PER];
#pragma unroll
  for (int j = 0; j < KV_PER; j++) {
    const int q = tid + j * ATT_THREADS;
    st_row[j] = q >> 4;
    st_chunk[j] = q & 15;
  }
  auto fetch = [&](int tile) {
#pragma unroll
    for (int j = 0; j < KV_PER; j++) {
      const int key = tile * BKV + st_row[j];
      f32x4 kk = {0.f, 0.f, 0.f, 0.f}, vv = {0.f, 0.f, 0.f, 0.f};
      if (key < kv_end) {
        const size_t off = (size_t)key * row_stride + st_chunk[j] * 4;
        kk = *reinterpret_cast<const f32x4*>(kbase + off);
        vv = *reinterpret_cast<const f32x4*>(vbase + off);
      }
      kst[j] = kk;
      vst[j] = vv;
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int j = 0; j < KV_PER; j++) {
      const int r = st_row[j], c = st_chunk[j];
      k_lds[buf][r * KV_CH + (c ^ (r & 7))] = kst[j];
      v_lds[buf][r * KV_CH + c] = vst[j];
    }
  };

  f32x16 o0, o1;
#pragma unroll
  for (int v = 0; v < 16; v++) {
    o0[v] = 0.f;
    o1[v] = 0.f;
  }
  float m_run = -INFINITY;  // running max of raw (unscaled) scores of this lane's query
  float l_run = 0.f;        // this lane's share of the running denominator

  fetch(0);
  stash(0);
  __syncthreads();

  for (int tile = 0; tile < ntile; tile++) {
    const int buf = tile & 1;
    if (tile + 1 < ntile) fetch(tile + 1);

#pragma unroll
    for (int sub = 0; sub < 2; sub++) {
      const int k0 = tile * BKV + sub * 32;  // first key of the sub-tile
      if (k0 > qw + 31 || k0 >= T) continue; // wave-uniform: nothing at or below the diagonal

      // S^T = K_sub . Q^T
      f32x16 s;
#pragma unroll
      for (int v = 0; v < 16; v++) s[v] = 0.f;
      const f32x4* krow = &k_lds[buf][(sub * 32 + l32) * KV_CH];
      const int sw = lane & 7;
#pragma unroll
      for (int g = 0; g < 8; g++) {
        const f32x4 kk = krow[(2 * g + h32) ^ sw];
#pragma unroll
        for (int e = 0; e < 4; e++)
          s = __builtin_amdgcn_mfma_f32_32x32x2f32(kk[e], qreg[g][e], s, 0, 0, 0);
      }

      // causal mask on the diagonal sub-tile
      if (k0 + 31 > qw) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int key = k0 + 8 * (v >> 2) + 4 * h32 + (v & 3);
          if (key > myq) s[v] = -INFINITY;
        }
      }

      // online softmax for this lane's query
      float mx = s[0];
#pragma unroll
      for (int v = 1; v < 16; v++) mx = fmaxf(mx, s[v]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run, mx);  // finite: key k0 <= every query of the wave
      const float alpha = exp2f((m_run - m_new) * scale_log2e);
      m_run = m_new;
      float psum = 0.f;
#pragma unroll
      for (int v = 0; v < 16; v++) {
        s[v] = exp2f((s[v] - m_new) * scale_log2e);
        psum += s[v];
      }
      l_run = l_run * alpha + psum;
#pragma unroll
      for (int v = 0; v < 16; v++) {
        o0[v] *= alpha;
        o1[v] *= alpha;
      }

      // O^T += V_sub^T . P^T
      const f32x2* vrow = reinterpret_cast<const f32x2*>(&v_lds[buf][0]);
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int key = sub * 32 + 8 * (v >> 2) + 4 * h32 + (v & 3);
        const f32x2 vv = vrow[key * (HS / 2) + l32];
        o0 = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.x, s[v], o0, 0, 0, 0);
        o1 = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.y, s[v], o1, 0, 0, 0);
      }
    }

    if (tile + 1 < ntile) stash(buf ^ 1);
    __syncthreads();
  }

  // ---- normalise and store -------------------------------------------------
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv = 1.0f / l_tot;
  if (myq < T) {
    float* op = out + ((size_t)b * T + myq) * C + head * HS + 8 * h32;
#pragma unroll
    for (int q4 = 0; q4 < 4; q4++) {
      f32x4 lo = {o0[4 * q4 + 0], o1[4 * q4 + 0], o0[4 * q4 + 1], o1[4 * q4 + 1]};
      f32x4 hi = {o0[4 * q4 + 2], o1[4 * q4 + 2], o0[4 * q4 + 3], o1[4 * q4 + 3]};
      *reinterpret_cast<f32x4*>(op + 16 * q4) = lo * inv;
      *reinterpret_cast<f32x4*>(op + 16 * q4 + 4) = hi * inv;
    }
  }
}

// Any head size / alignment: one wave per (b, head, query), scores streamed in
// chunks of 64 keys with an online softmax.  Slow path for shapes the MFMA
// kernel is not built for.
__global__ __launch_bounds__(256) void attention_generic_kernel(float* out, const float* qkv,
                                                                 int B, int T, int NH, int hs,
                                                                 float scale) {
  const int lane = threadIdx.x & 63;
  const long long w = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= (long long)B * NH * T) return;
  const int t = (int)(w % T);
  const int head = (int)((w / T) % NH);
  const int b = (int)(w / ((long long)T * NH));
  const int C = NH * hs;
  const size_t rs = (size_t)3 * C;
  const float* base = qkv + (size_t)b * T * rs + head * hs;
  const float* q = base + (size_t)t * rs;
  float m = -INFINITY, l = 0.f;
  // each lane accumulates output features lane, lane+64, ... (up to 4 => hs <= 256)
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 <= t; k0 += 64) {
    const int key = k0 + lane;
    float sc = -INFINITY;
    if (key <= t) {
      const float* kp = base + C + (size_t)key * rs;
      float d = 0.f;
      for (int i = 0; i < hs; i++) d += q[i] * kp[i];
      sc = d * scale;
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float alpha = expf(m - m_new);
    const float p = (key <= t) ? expf(sc - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int j = 0; j < 4; j++) acc[j] *= alpha;
    const int nk = min(64, t + 1 - k0);
    for (int kk = 0; kk < nk; kk++) {
      const float pk = __shfl(p, kk, 64);
      const float* vp = base + 2 * C + (size_t)(k0 + kk) * rs;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int f = lane + 64 * j;
        if (f < hs) acc[j] += pk * vp[f];
      }
    }
  }
  float* o = out + ((size_t)b * T + t) * C + head * hs;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int f = lane + 64 * j;
    if (f < hs) o[f] = acc[j] / l;
  }
}

}  // namespace g2

extern "C" {

int attention_forward_status(float* out, float* qkvr, float* att, const float* inp, int B, int T,
                             int C, int NH) {
  using namespace g2;
  (void)qkvr;
  (void)att;
  if (B < 0 || T < 0 || C < 1 || NH < 1 || C % NH != 0)
    return fail(GPT2HIP_EINVAL, "attention_forward: bad shape B=%d T=%d C=%d NH=%d", B, T, C, NH);
  if (B == 0 || T == 0) return GPT2HIP_OK;
  if (!out || !inp) return fail(GPT2HIP_EINVAL, "attention_forward: null pointer");
  const int hs = C / NH;
  if (hs == HS && aligned16(inp) && aligned16(out)) {
    const int nqt = (T + BQ - 1) / BQ;
    const long long blocks = (long long)nqt * B * NH;
    if (blocks > 0x7fffffffLL) return fail(GPT2HIP_EINVAL, "attention_forward: grid too large");
    const float scale_log2e = (1.0f / sqrtf((float)hs)) * 1.4426950408889634f;
    hipLaunchKernelGGL(attention_flash_kernel, dim3((unsigned)blocks), dim3(ATT_THREADS), 0, 0, out,
                       inp, T, NH, nqt, scale_log2e);
  } else {
    if (hs > 256) return fail(GPT2HIP_EINVAL, "attention_forward: head size %d > 256", hs);
    const long long waves = (long long)B * NH * T;
    const long long blocks = (waves + 3) / 4;
    if (blocks > 0x7fffffffLL) return fail(GPT2HIP_EINVAL, "attention_forward: grid too large");
    hipLaunchKernelGGL(attention_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, 0, out, inp,
                       B, T, NH, hs, 1.0f / sqrtf((float)hs));
  }
  G2_LAUNCH_CHECK("attention_forward");
  return GPT2HIP_OK;
}

void attention_forward(float* out, float* qkvr, float* att, const float* inp, int B, int T, int C,
                       int NH) {
  if (attention_forward_status(out, qkvr, att, inp, B, T, C, NH)) g2::die("attention_forward");
}

}  // extern "C"
