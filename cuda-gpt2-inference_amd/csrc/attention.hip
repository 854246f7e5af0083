// attention_forward for gfx950: causal multi-head self-attention read straight
// from the packed qkv activations (B,T,3C) and written as (B,T,C) — the op of
// reference 3_flash_attention_permute.cuh:346-355 — as one flash-style kernel
// on the fp32 matrix cores.  The T x T scores never leave registers.
//
// Shape of the computation (head size 64).  A workgroup of 4 waves owns 64
// consecutive queries of one (batch, head) as two groups of 32, each shared by a
// PAIR of waves that split the keys between them (P = 2), or -- when that would
// leave compute units without work -- one group of 32 queries split four ways (P = 4).
// A wave takes every P-th sub-tile of 32 keys, with its own running maximum, sum
// and output; the partial results of a group are merged once at the end.  Splitting
// keys rather than queries keeps the waves of a workgroup equally busy under the
// causal mask (they differ by at most one sub-tile, on the diagonal), which a split
// by queries does not: with 128 queries per workgroup and one group per wave,
// non-causal attention ran at 80 % of the matrix peak and causal attention at 60 %.
//
// The waves of a workgroup share nothing inside the loop, so there is no barrier in
// it.  A wave's K sub-tile (8 KiB) goes from global memory straight into the wave's
// own LDS region (buffer_load ... lds); as soon as the wave has read it into
// registers it requests the next one into the same region, which then has a whole
// sub-tile of matrix work to arrive.  V needs no transposition (a lane wants two
// neighbouring features of one key: a wave load is two 256-byte rows) and goes
// straight from global memory to registers, requested before the scores and used
// after the softmax.  34 KiB of LDS and 160 registers per lane leave room for three
// workgroups per compute unit, which is what hides a workgroup's start (first
// loads) and end (merge, stores) behind the matrix work of the others: the earlier
// form (keys and values of 64-key tiles shared through 64 KiB of LDS by the four
// waves, one barrier per tile, two workgroups per compute unit) ran the benchmark
// shape B=8, T=1024, NH=12 in 128.8 us where this one takes 121.0 in the same harness.
// Addresses are buffer addresses (scalar base + scalar row offset + a fixed lane offset):
// no vector address arithmetic in the loop.  Only a sequence's ragged last sub-tile (T not a
// multiple of 32) carries its rows in the lane offset, clamped to the sequence's last row.
//
#include <algorithm>
#include <type_traits>

#include "common.hpp"

namespace g2 {

constexpr int HS = 64;          // head size this kernel is built for
constexpr int ATT_THREADS = 256;
constexpr int ATT_WAVES = ATT_THREADS / kWave;
constexpr int WAVE_LDS_BYTES = 34 * kWave * 4;    // a wave's region: its K sub-tile, later its parked partial state
constexpr float LAZY_LOG2 = 8.0f;  // allowed growth of 2^x above the current shift

typedef __attribute__((address_space(3))) void lds_void_t;
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

// Exchange between lanes l and l^32: v_permlane32_swap swaps lanes 32..63 of its
// first operand with lanes 0..31 of its second.  Fed two copies of x it leaves
// {x[0..31], x[0..31]} in one and {x[32..63], x[32..63]} in the other, so either
// reduction of the two registers is the l / l^32 pair reduction, in every lane.
// Written as inline assembly so that both results are kept as distinct registers.
__device__ __forceinline__ void pair_split(float x, float& lo, float& hi) {
  lo = x;
  hi = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
}
__device__ __forceinline__ float pair_max(float x) {
  float lo, hi;
  pair_split(x, lo, hi);
  return fmaxf(lo, hi);
}
__device__ __forceinline__ float pair_sum(float x) {
  float lo, hi;
  pair_split(x, lo, hi);
  return lo + hi;
}

// P = waves that split the keys of one group of 32 queries; a workgroup of 4 waves holds
// 4 / P such groups.
// RAGGED: T is not a multiple of 32, so a sequence's last sub-tile of keys reaches past its
// rows; that instantiation carries the test for it in its loop, the other one does not.
template <int P, bool RAGGED>
__global__ __launch_bounds__(ATT_THREADS) __attribute__((amdgpu_waves_per_eu(3, 3)))
void attention_flash_kernel(float* __restrict__ out, const float* __restrict__ qkv, int T, int NH,
                            int nqb, float scale_log2e, int snake) {
  constexpr int QG = ATT_WAVES / P;  // query groups per workgroup
  constexpr int BQ = 32 * QG;        // queries per workgroup
  __shared__ __attribute__((aligned(16))) char lds_all[ATT_WAVES * WAVE_LDS_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h32 = lane >> 5;
  const int l32 = lane & 31;

  // Heaviest query blocks (most keys) first.  The first three workgroups per compute unit are
  // resident at once and not handed out dynamically: the dispatcher deals workgroup ids breadth
  // first, ids i, i + CUs, i + 2 CUs to the same compute unit, which in descending order of weight
  // gives one unit the heaviest of every third and another the lightest (17 against 10 sub-tiles
  // at B=8, T=256, NH=12).  `snake` (the number of compute units, or 0) deals the second of those
  // three rows of ids in reverse instead, as one deals out cards by strength.  (Later workgroups
  // go wherever one has finished; with the first three rows dealt this way a launch of 1536
  // workgroups, B=8, T=1024, NH=12, still gains 1.5 %: 111.0 -> 109.3 us.)
  int bid = blockIdx.x;
  if (snake > 0 && bid < 3 * snake) {
    const int row = bid / snake, first = row * snake;
    if (row & 1) bid = first + (min(snake, (int)gridDim.x - first) - 1 - (bid - first));
  }
  const int per_block = gridDim.x / nqb;  // = B*NH
  const int qblock = nqb - 1 - bid / per_block;
  const int bh = bid % per_block;
  const int b = bh / NH, head = bh % NH;

  const int C = NH * HS;
  const int row_bytes = 3 * C * 4;
  const int qgroup = wave / P;        // which 32 queries of the workgroup
  const int part = wave % P;          // which sub-tiles of 32 keys: part, part + P, ...
  const int qw = qblock * BQ + qgroup * 32;  // first query of this wave
  const int myq = qw + l32;                  // this lane's query
  const int diag = qw >> 5;                  // the sub-tile that holds the diagonal; the last one needed
  const bool live = qw < T;                  // a group entirely past T has nothing to do

  // One sequence's packed rows as a buffer: offsets are 32-bit.  Rows at or past T are never
  // addressed: the ragged forms below clamp them (keys there only meet masked or unstored queries).
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(qkv) + (size_t)b * T * 3 * C, 0, T * row_bytes, 0x00020000);
  const int q_col = head * (HS * 4), k_col = q_col + C * 4, v_col = q_col + 2 * C * 4;

  char* const my_lds = lds_all + wave * WAVE_LDS_BYTES;

  // ---- K sub-tile: global -> LDS by DMA, 8 instructions of 4 rows x 256 bytes --------
  // Lane l lands at slot l of the instruction's KiB: row l/16, chunk position l%16, and
  // fetches logical chunk (l%16) ^ (row & 7) (the swizzle is applied on the global side).
  // row & 7 = 4*(i&1) + l/16 for instruction i, so two lane offsets cover all eight.
  const int dma_lane[2] = {(lane >> 4) * row_bytes + (((lane & 15) ^ (lane >> 4)) << 4),
                           (lane >> 4) * row_bytes + (((lane & 15) ^ (4 + (lane >> 4))) << 4)};
  // The scalar offset of a buffer access is NOT range-checked (only the lane offset is), so a
  // sub-tile that reaches past T -- the last one of a sequence whose length is not a multiple
  // of 32 -- takes the form below it: the row goes into the lane offset, clamped to the last
  // row of the sequence (finite data, and every key there is masked for every stored query).
  auto dma_k = [&](int sub) {
    if (!RAGGED || (sub + 1) * 32 <= T) {
      const int s0 = sub * 32 * row_bytes + k_col;
#pragma unroll
      for (int i = 0; i < 8; i++)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_t*)(my_lds + i * 1024), 16, dma_lane[i & 1],
                                                 s0 + 4 * i * row_bytes, 0, 0);
    } else {
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const int row = min(sub * 32 + 4 * i + (lane >> 4), T - 1);
        const int chunk = ((lane & 15) ^ (4 * (i & 1) + (lane >> 4))) << 4;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_t*)(my_lds + i * 1024), 16,
                                                 row * row_bytes + chunk, k_col, 0, 0);
      }
    }
  };

  int sub = part;
  if (live && sub <= diag) dma_k(sub);

  // ---- Q in registers: qreg[g] = Q[myq][8g+4h .. +3] --------------------
  f32x4 qreg[8];
  {
    // queries at or past T (RAGGED only; never stored) read the sequence's last row
    const int qv = (RAGGED ? min(myq, T - 1) : l32) * row_bytes + h32 * 16;
    const int qs = (RAGGED ? 0 : qw * row_bytes) + q_col;
#pragma unroll
    for (int g = 0; g < 8; g++)
      qreg[g] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, qv, qs + g * 32, 0));
  }

  f32x16 o0, o1;
#pragma unroll
  for (int v = 0; v < 16; v++) {
    o0[v] = 0.f;
    o1[v] = 0.f;
  }
  float m_used = -INFINITY;  // current shift, in raw (unscaled) score units
  float mc = 0.f;            // m_used * scale_log2e (unused while m_used is -inf)
  float l_run = 0.f;         // this lane's share of the running denominator
  const float lazy_raw = LAZY_LOG2 / scale_log2e;

  // LDS read addresses of the K operand: row l32, chunk (2g+h) ^ (l32 & 7); chunks of g and
  // g + 4 are 128 bytes apart
  const char* k_addr[4];
#pragma unroll
  for (int g = 0; g < 4; g++) k_addr[g] = my_lds + (l32 * 16 + ((2 * g + h32) ^ (lane & 7))) * 16;
  // V straight from global memory: register v pairs with key 8*(v/4) + 4*h32 + v%4 of the
  // sub-tile, this lane's two features are 2*l32, 2*l32+1
  const int v_lane = 4 * h32 * row_bytes + l32 * 8;

  if (live) {
    for (; sub <= diag; sub += P) {
      const int k0 = sub * 32;
      // K of this sub-tile has landed (requested one sub-tile ago)
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      f32x4 kreg[8];
#pragma unroll
      for (int g = 0; g < 8; g++)
        kreg[g] = *reinterpret_cast<const f32x4*>(k_addr[g & 3] + (g >> 2) * 128);
      // V of this sub-tile: needed after the scores and the softmax
      f32x2 vreg[16];
      if (!RAGGED || k0 + 32 <= T) {
        const int vs = k0 * row_bytes + v_col;
#pragma unroll
        for (int v = 0; v < 16; v++)
          vreg[v] = __builtin_bit_cast(
              f32x2, __builtin_amdgcn_raw_buffer_load_b64(rsrc, v_lane, vs + (8 * (v >> 2) + (v & 3)) * row_bytes, 0));
      } else {
        // the sequence's ragged last sub-tile: rows clamped in the lane offset (see dma_k); the
        // clamped rows are finite and meet softmax weights that are exactly zero
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int row = min(k0 + 8 * (v >> 2) + (v & 3) + 4 * h32, T - 1);
          vreg[v] = __builtin_bit_cast(
              f32x2, __builtin_amdgcn_raw_buffer_load_b64(rsrc, row * row_bytes + l32 * 8, v_col, 0));
        }
      }
      // the K region is free once its reads have returned: request the next sub-tile
      if (sub + P <= diag) {
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
        dma_k(sub + P);
      }

      // S^T = K_sub . Q^T
      f32x16 s;
#pragma unroll
      for (int v = 0; v < 16; v++) s[v] = 0.f;
#pragma unroll
      for (int g = 0; g < 8; g++)
#pragma unroll
        for (int e = 0; e < 4; e++)
          s = __builtin_amdgcn_mfma_f32_32x32x2f32(kreg[g][e], qreg[g][e], s, 0, 0, 0);

      // causal mask on the diagonal sub-tile (keys at or past T are beyond every stored query)
      if (sub == diag) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int key = k0 + 8 * (v >> 2) + 4 * h32 + (v & 3);
          if (key > myq) s[v] = -INFINITY;
        }
      }

      // lazy online softmax for this lane's query
      float mx = fmaxf(fmaxf(s[0], s[1]), s[2]);
#pragma unroll
      for (int v = 3; v < 15; v += 2) mx = fmaxf(fmaxf(mx, s[v]), s[v + 1]);
      mx = pair_max(fmaxf(mx, s[15]));  // finite: key k0 <= every query of the wave
      if (__builtin_amdgcn_ballot_w64(mx > m_used + lazy_raw) != 0) {
        const float m_new = fmaxf(m_used, mx);
        const float alpha = __builtin_amdgcn_exp2f((m_used - m_new) * scale_log2e);  // 0 at first
        m_used = m_new;
        mc = m_new * scale_log2e;
        l_run *= alpha;
#pragma unroll
        for (int v = 0; v < 16; v++) {
          o0[v] *= alpha;
          o1[v] *= alpha;
        }
      }
      float psum = 0.f;
#pragma unroll
      for (int v = 0; v < 16; v++) {
        s[v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], scale_log2e, -mc));
        psum += s[v];
      }
      l_run += psum;

      // O^T += V_sub^T . P^T
#pragma unroll
      for (int v = 0; v < 16; v++) {
        o0 = __builtin_amdgcn_mfma_f32_32x32x2f32(vreg[v].x, s[v], o0, 0, 0, 0);
        o1 = __builtin_amdgcn_mfma_f32_32x32x2f32(vreg[v].y, s[v], o1, 0, 0, 0);
      }
    }
  }

  // ---- merge the P key parts of each query group --------------------------
  // Every wave's K region is idle once its own loop has ended; parts 1 .. P-1 park their
  // partial state there, one float per (register, lane).
  float* const park = reinterpret_cast<float*>(my_lds) + lane;
  if (part != 0 && live && part <= diag) {
#pragma unroll
    for (int v = 0; v < 16; v++) {
      park[v * kWave] = o0[v];
      park[(16 + v) * kWave] = o1[v];
    }
    park[32 * kWave] = m_used;
    park[33 * kWave] = l_run;
  }
  __syncthreads();
  if (part == 0 && live) {
    // m_used is finite: key 0 is visible to every query, and sub-tile 0 belongs to part 0
#pragma unroll
    for (int p = 1; p < P; p++) {
      if (p <= diag) {
        const float* other = reinterpret_cast<const float*>(lds_all + (wave + p) * WAVE_LDS_BYTES) + lane;
        const float m1 = other[32 * kWave], l1 = other[33 * kWave];
        const float m = fmaxf(m_used, m1);
        const float a0 = __builtin_amdgcn_exp2f((m_used - m) * scale_log2e);
        const float a1 = __builtin_amdgcn_exp2f((m1 - m) * scale_log2e);
#pragma unroll
        for (int v = 0; v < 16; v++) {
          o0[v] = o0[v] * a0 + other[v * kWave] * a1;
          o1[v] = o1[v] * a0 + other[(16 + v) * kWave] * a1;
        }
        l_run = l_run * a0 + l1 * a1;
        m_used = m;
      }
    }
    const float inv = 1.0f / pair_sum(l_run);
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

// ---- one new position per sequence against a key/value cache ---------------------
// Keys and values of past positions live in kc / vc, (B, NH, maxT, hs) each -- the rows of one
// (sequence, head) are consecutive in memory, so that a step streams them as one block --
// written by kv_store_kernel (a whole prompt) and by this kernel (the new position).  One workgroup
// of 16 waves per (sequence, head): it appends the new key and value, computes the pos+1
// scores one wave per position (lanes over the head dimension, DPP reduction), turns them
// into softmax weights in LDS, and accumulates the weighted values with each wave taking
// every 16th position; the 16 partial outputs are summed in wave order.  The cache rows
// are read exactly once: the kernel is bound by that stream of (pos+1) * 2 * hs * 4 bytes.
constexpr int DEC_WAVES = 16;

__global__ __launch_bounds__(DEC_WAVES* kWave) void attention_decode_kernel(
    float* __restrict__ out, const float* __restrict__ qkv, float* __restrict__ kc,
    float* __restrict__ vc, int pos, int maxT, int NH, int hs, float scale) {
  extern __shared__ float dec_lds[];  // scores [pos+1 rounded up to 64] | partial outputs [16][hs]
  __shared__ float red[2 * DEC_WAVES];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = blockIdx.x / NH, head = blockIdx.x % NH;
  const int C = NH * hs;
  float* const sc = dec_lds;
  float* const part = dec_lds + ((pos + 64) & ~63);
  const float* qrow = qkv + (size_t)b * 3 * C + head * hs;
  float* const kb = kc + (size_t)blockIdx.x * maxT * hs;
  float* const vb = vc + (size_t)blockIdx.x * maxT * hs;

  for (int d = tid; d < hs; d += DEC_WAVES * kWave) {
    kb[(size_t)pos * hs + d] = qrow[C + d];
    vb[(size_t)pos * hs + d] = qrow[2 * C + d];
  }
  float qv[4];
#pragma unroll
  for (int j = 0; j < 4; j++) qv[j] = (lane + 64 * j < hs) ? qrow[lane + 64 * j] : 0.f;
  __syncthreads();  // the appended row is visible to the whole workgroup

  // scores
  float mx = -INFINITY;
  for (int t0 = wave; t0 <= pos; t0 += 4 * DEC_WAVES) {
    float p[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const int t = min(t0 + u * DEC_WAVES, pos);
      const float* kr = kb + (size_t)t * hs;
      p[u] = 0.f;
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (lane + 64 * j < hs) p[u] += qv[j] * kr[lane + 64 * j];
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const int t = t0 + u * DEC_WAVES;
      const float s = wave_sum(p[u]) * scale;
      if (t <= pos) {
        if (lane == 0) sc[t] = s;
        mx = fmaxf(mx, s);
      }
    }
  }
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  float m = red[0];
#pragma unroll
  for (int w = 1; w < DEC_WAVES; w++) m = fmaxf(m, red[w]);  // finite: position 0 always exists

  // softmax weights (unnormalised) and their sum
  float sum = 0.f;
  for (int t = tid; t <= pos; t += DEC_WAVES * kWave) {
    const float e = expf(sc[t] - m);
    sc[t] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  if (lane == 0) red[DEC_WAVES + wave] = sum;
  __syncthreads();
  float l = 0.f;
#pragma unroll
  for (int w = 0; w < DEC_WAVES; w++) l += red[DEC_WAVES + w];

  // weighted values: wave w takes positions w, w + 16, ...
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int t0 = wave; t0 <= pos; t0 += 4 * DEC_WAVES) {
    float vv[4][4], pw[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const int t = t0 + u * DEC_WAVES;
      pw[u] = (t <= pos) ? sc[t] : 0.f;
      const float* vr = vb + (size_t)min(t, pos) * hs;
#pragma unroll
      for (int j = 0; j < 4; j++) vv[u][j] = (lane + 64 * j < hs) ? vr[lane + 64 * j] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 4; u++)
#pragma unroll
      for (int j = 0; j < 4; j++) acc[j] += pw[u] * vv[u][j];
  }
#pragma unroll
  for (int j = 0; j < 4; j++)
    if (lane + 64 * j < hs) part[wave * hs + lane + 64 * j] = acc[j];
  __syncthreads();
  for (int d = tid; d < hs; d += DEC_WAVES * kWave) {
    float o = 0.f;
#pragma unroll
    for (int w = 0; w < DEC_WAVES; w++) o += part[w * hs + d];
    out[(size_t)b * C + head * hs + d] = o / l;
  }
}

// Head size 64 with 16-byte aligned rows: 16 lanes cover one cache row with 128-bit loads,
// so a wave instruction brings four positions (1 KiB) and a wave keeps DEC_UNROLL of them
// in flight; position t = 4 * (wave + 16 * i) + lane / 16.
constexpr int DEC_UNROLL = 8;

// WAVES: waves per workgroup.  Sixteen keep the most rows in flight for one (sequence, head); with
// more of those than the device holds such workgroups at once (two per compute unit), eight-wave
// workgroups are all resident together instead of queueing for a second round.
template <int WAVES>
__global__ __launch_bounds__(WAVES* kWave) void attention_decode64_kernel(
    float* __restrict__ out, const float* __restrict__ qkv, float* __restrict__ kc,
    float* __restrict__ vc, int pos, int maxT, int NH, float scale) {
  extern __shared__ float dec_lds[];  // scores [pos+1 rounded up to 64] | partial outputs [16][64]
  __shared__ float red[2 * WAVES];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int p4 = lane >> 4, sub = lane & 15;
  const int b = blockIdx.x / NH, head = blockIdx.x % NH;
  const int C = NH * 64;
  float* const sc = dec_lds;
  float* const part = dec_lds + ((pos + 64) & ~63);
  const float* qrow = qkv + (size_t)b * 3 * C + head * 64;
  float* const kb = kc + (size_t)blockIdx.x * maxT * 64 + 4 * sub;
  float* const vb = vc + (size_t)blockIdx.x * maxT * 64 + 4 * sub;

  if (tid < 16) {
    *reinterpret_cast<f32x4*>(kb + (size_t)pos * 64) = *reinterpret_cast<const f32x4*>(qrow + C + 4 * sub);
    *reinterpret_cast<f32x4*>(vb + (size_t)pos * 64) =
        *reinterpret_cast<const f32x4*>(qrow + 2 * C + 4 * sub);
  }
  const f32x4 q4 = *reinterpret_cast<const f32x4*>(qrow + 4 * sub);
  __syncthreads();  // the appended row is visible to the whole workgroup

  float mx = -INFINITY;
  for (int g0 = wave; 4 * g0 <= pos; g0 += DEC_UNROLL * WAVES) {
    f32x4 kf[DEC_UNROLL];
#pragma unroll
    for (int u = 0; u < DEC_UNROLL; u++) {
      const int t = min(4 * (g0 + u * WAVES) + p4, pos);
      kf[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(kb + (size_t)t * 64));
    }
#pragma unroll
    for (int u = 0; u < DEC_UNROLL; u++) {
      const int t = 4 * (g0 + u * WAVES) + p4;
      const f32x4 pr = q4 * kf[u];
      const float s = row16_sum((pr[0] + pr[1]) + (pr[2] + pr[3])) * scale;
      if (t <= pos) {
        if (sub == 0) sc[t] = s;
        mx = fmaxf(mx, s);
      }
    }
  }
  mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
  mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  float m = red[0];
#pragma unroll
  for (int w = 1; w < WAVES; w++) m = fmaxf(m, red[w]);  // finite: position 0 always exists

  float sum = 0.f;
  for (int t = tid; t <= pos; t += WAVES * kWave) {
    const float e = expf(sc[t] - m);
    sc[t] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  if (lane == 0) red[WAVES + wave] = sum;
  __syncthreads();
  float l = 0.f;
#pragma unroll
  for (int w = 0; w < WAVES; w++) l += red[WAVES + w];

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int g0 = wave; 4 * g0 <= pos; g0 += DEC_UNROLL * WAVES) {
    f32x4 vf[DEC_UNROLL];
    float pw[DEC_UNROLL];
#pragma unroll
    for (int u = 0; u < DEC_UNROLL; u++) {
      const int t = 4 * (g0 + u * WAVES) + p4;
      pw[u] = (t <= pos) ? sc[t] : 0.f;
      vf[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(vb + (size_t)min(t, pos) * 64));
    }
#pragma unroll
    for (int u = 0; u < DEC_UNROLL; u++) acc += pw[u] * vf[u];
  }
#pragma unroll
  for (int e = 0; e < 4; e++) {
    acc[e] += __shfl_xor(acc[e], 16, 64);
    acc[e] += __shfl_xor(acc[e], 32, 64);
  }
  if (p4 == 0) *reinterpret_cast<f32x4*>(part + wave * 64 + 4 * sub) = acc;
  __syncthreads();
  if (tid < 64) {
    float o = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; w++) o += part[w * 64 + tid];
    out[(size_t)b * C + head * 64 + tid] = o / l;
  }
}

// Copies the key and value thirds of a prompt's packed qkv (B, T, 3C) into the cache
// (B, NH, maxT, hs each) at positions 0..T-1.
__global__ __launch_bounds__(256) void kv_store_kernel(float* __restrict__ kc, float* __restrict__ vc,
                                                        const float* __restrict__ qkv, int T,
                                                        int maxT, int C, int hs, size_t total) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const size_t bt = i / C;
  const int c = (int)(i - bt * C);
  const size_t b = bt / T, t = bt - b * T;
  const float* src = qkv + bt * 3 * C + C + c;
  const int head = c / hs, d = c - head * hs;
  const size_t dst = ((b * (size_t)(C / hs) + head) * maxT + t) * hs + d;
  kc[dst] = src[0];
  vc[dst] = src[C];
}

int attention_decode_launch(float* out, const float* qkv, float* kc, float* vc, int B, int pos,
                            int maxT, int C, int NH) {
  if (B < 1 || C < 1 || NH < 1 || C % NH != 0 || pos < 0 || pos >= maxT)
    return fail(GPT2HIP_EINVAL, "attention_decode: bad shape B=%d C=%d NH=%d pos=%d maxT=%d", B, C,
                NH, pos, maxT);
  if (!out || !qkv || !kc || !vc) return fail(GPT2HIP_EINVAL, "attention_decode: null pointer");
  const int hs = C / NH;
  if (hs > 256) return fail(GPT2HIP_EINVAL, "attention_decode: head size %d > 256", hs);
  const size_t lds = ((size_t)((pos + 64) & ~63) + (size_t)DEC_WAVES * hs) * sizeof(float);
  if (lds > 60 * 1024)
    return fail(GPT2HIP_EINVAL, "attention_decode: position %d needs %zu bytes of LDS", pos, lds);
  if (hs == 64 && aligned16(qkv) && aligned16(kc) && aligned16(vc))
    if (B * NH > 512)
      hipLaunchKernelGGL(attention_decode64_kernel<8>, dim3((unsigned)(B * NH)), dim3(8 * kWave), lds, stream(), out,
                         qkv, kc, vc, pos, maxT, NH, 1.0f / sqrtf(64.f));
    else
      hipLaunchKernelGGL(attention_decode64_kernel<DEC_WAVES>, dim3((unsigned)(B * NH)), dim3(DEC_WAVES * kWave), lds,
                         stream(), out, qkv, kc, vc, pos, maxT, NH, 1.0f / sqrtf(64.f));
  else
    hipLaunchKernelGGL(attention_decode_kernel, dim3((unsigned)(B * NH)), dim3(DEC_WAVES * kWave), lds,
                       stream(), out, qkv, kc, vc, pos, maxT, NH, hs, 1.0f / sqrtf((float)hs));
  G2_LAUNCH_CHECK("attention_decode");
  return GPT2HIP_OK;
}

int kv_store_launch(float* kc, float* vc, const float* qkv, int B, int T, int maxT, int C, int NH) {
  const size_t total = (size_t)B * T * C;
  if (total == 0) return GPT2HIP_OK;
  if (NH < 1 || C % NH != 0) return fail(GPT2HIP_EINVAL, "kv_store: bad shape C=%d NH=%d", C, NH);
  hipLaunchKernelGGL(kv_store_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream(), kc,
                     vc, qkv, T, maxT, C, C / NH, total);
  G2_LAUNCH_CHECK("kv_store");
  return GPT2HIP_OK;
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
  if (hs == HS && aligned16(inp) && aligned16(out) && (long long)T * 3 * C * 4 < (1LL << 31)) {
    // Two query groups per workgroup (64 queries, keys split two ways) when there are enough
    // of them: 768 are resident at once, and a launch is as long as its heaviest workgroup
    // (T / 64 sub-tiles per wave) unless several rounds of them even that out.  Below that,
    // one group per workgroup with the keys split four ways: twice the workgroups, each half as
    // long, at the price of reading every key and value twice as often and a four-way merge.
    // Both forms timed over T = 256 .. 1024, B = 1 .. 16 and 12, 16, 20, 25 heads (with the first
    // 768 workgroups dealt in alternating direction, see the kernel): the four-way split wins, by
    // up to 40 %, below 384 / 500 / 650 / 780 workgroups of 64 queries at T = 256 / 512 / 768 /
    // 1024 -- at T = 256 that is where its own workgroups stop being resident all at once -- and
    // loses 3-28 % beyond; the line below is within 2.8 % of the better form at each of the 144
    // shapes timed, 0.2 % on average.
    const long long wide = (long long)((T + 63) / 64) * B * NH;
    const long long four_way_below = (long long)(0.47 * T + 265.0);
    const int P = wide < four_way_below ? 4 : 2;
    const int bq = 32 * (ATT_WAVES / P);
    const int nqb = (T + bq - 1) / bq;
    const long long blocks = (long long)nqb * B * NH;
    if (blocks > 0x7fffffffLL) return fail(GPT2HIP_EINVAL, "attention_forward: grid too large");
    const float scale_log2e = (1.0f / sqrtf((float)hs)) * 1.4426950408889634f;
    const bool ragged = T % 32 != 0;
    auto kfn = P == 2 ? (ragged ? attention_flash_kernel<2, true> : attention_flash_kernel<2, false>)
                      : (ragged ? attention_flash_kernel<4, true> : attention_flash_kernel<4, false>);
    // the first three workgroups per compute unit are resident at once: see the kernel's `snake`
    int cus = 0, dev = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
      cus = 0;
    const int snake = cus > 0 ? cus : 0;
    hipLaunchKernelGGL(kfn, dim3((unsigned)blocks), dim3(ATT_THREADS), 0, stream(), out, inp, T, NH, nqb,
                       scale_log2e, snake);
  } else {
    if (hs > 256) return fail(GPT2HIP_EINVAL, "attention_forward: head size %d > 256", hs);
    const long long waves = (long long)B * NH * T;
    const long long blocks = (waves + 3) / 4;
    if (blocks > 0x7fffffffLL) return fail(GPT2HIP_EINVAL, "attention_forward: grid too large");
    hipLaunchKernelGGL(attention_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, stream(), out, inp,
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
