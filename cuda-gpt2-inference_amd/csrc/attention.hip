// attention_forward for gfx950: causal multi-head self-attention read straight
// from the packed qkv activations (B,T,3C) and written as (B,T,C) — the op of
// reference 3_flash_attention_permute.cuh:346-355 — as one flash-style kernel
// on the fp32 matrix cores.  The T x T scores never leave registers.
//
// Shape of the computation (head size 64).  A workgroup of 4 waves owns 64
// consecutive queries of one (batch, head): two groups of 32 queries, each shared
// by a PAIR of waves that split the keys between them.  Keys and values go from
// global memory straight into LDS (global_load_lds_dwordx4, two buffers of 64
// keys, one barrier per tile); of every tile the first wave of a pair takes the
// first 32 keys and the second wave the last 32, each with its own running
// maximum, sum and output, and the two partial results are merged once at the
// end.  Splitting keys rather than queries keeps the four waves of a workgroup
// equally busy under the causal mask (they differ by at most one sub-tile, on the
// diagonal), which a split by queries does not: with 128 queries per workgroup and
// one group per wave, non-causal attention ran at 80 % of the matrix peak and
// causal attention at 60 %.
//
// Per sub-tile a wave computes, with v_mfma_f32_32x32x2_f32,
//     S^T (32 keys x 32 queries) = K_sub (32 x 64) . Q^T (64 x 32)
// so that lane l owns query l%32 and holds 16 of that query's 32 scores
// (keys 8*(v/4) + 4*(l/32) + v%4, v = 0..15); lane l^32 holds the other 16.
// Row maxima and sums are therefore register reductions plus one exchange
// with lane l^32 (v_permlane32_swap).  The probabilities are then used IN PLACE
// as the B operand of
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
//
// Every VALU instruction takes issue time from the matrix pipe on this chip, so
// the softmax is kept lean: hardware exp2 on a fused multiply-add, and a LAZY
// running maximum — the shift m only moves when some score exceeds it by more
// than 2^8 after scaling, so the rescaling of O and of the running sum is a rare,
// wave-uniform branch.  Softmax is invariant to the shift, so this is exact;
// probabilities are merely allowed to reach 2^8 instead of 1 before normalisation.
// (The branch is taken per group of 32 queries, so the ROUNDING of a query's result
// can depend on the other queries of its group; its value cannot.)
#include <type_traits>

#include "common.hpp"

namespace g2 {

constexpr int HS = 64;          // head size this kernel is built for
constexpr int BQ = 64;          // queries per workgroup (2 groups of 32, 2 waves each)
constexpr int BKV = 64;         // keys per LDS tile
constexpr int KV_CH = HS / 4;   // 16-byte chunks per K/V row
constexpr int ATT_THREADS = 256;
constexpr int ATT_WAVES = ATT_THREADS / kWave;
constexpr int KV_TILE_BYTES = BKV * HS * 4;                 // 16 KiB per tensor per tile
constexpr int KV_DMA_PER = 2 * (KV_TILE_BYTES / 1024) / ATT_WAVES;  // K+V DMAs per wave and tile = 8
constexpr float LAZY_LOG2 = 8.0f;  // allowed growth of 2^x above the current shift

typedef __attribute__((address_space(3))) void lds_void_t;
typedef const __attribute__((address_space(1))) void glb_void_t;

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

__global__ __launch_bounds__(ATT_THREADS) void attention_flash_kernel(
    float* __restrict__ out, const float* __restrict__ qkv, int T, int NH, int nqt,
    float scale_log2e) {
  // [buffer][K tile | V tile]
  __shared__ f32x4 kv_lds[2][2 * BKV * KV_CH];
  char* const lds_bytes = reinterpret_cast<char*>(&kv_lds[0][0]);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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

  const int q0 = qtile * BQ;          // first query of the workgroup
  const int qgroup = wave >> 1;       // which 32 queries
  const int khalf = wave & 1;         // which 32 keys of every 64-key tile
  const int qw = q0 + qgroup * 32;    // first query of this wave
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

  // ---- K/V LDS-DMA: one instruction moves 4 rows of 256 bytes ------------------
  // DMA j of this wave: group gi = wave*KV_DMA_PER + j of the tile's 32 groups
  // (0..15: K rows 4*gi.., 16..31: V rows).  Lane l lands at LDS slot l of the group:
  // row l/16, chunk position l%16; for K it fetches logical chunk (l%16) ^ (row & 7).
  // An address is a wave-uniform base (the tile's first K row, moved on with scalar
  // adds) plus a fixed 32-bit per-lane offset.  Only a last, partial tile (T % 64 != 0)
  // needs per-lane work: keys at or past T are clamped to T-1 there; they only ever
  // meet queries < key, i.e. they are masked, or queries >= T, which are not stored.
  const char* const kv_base = reinterpret_cast<const char*>(base + C);  // K; V is C floats on
  const unsigned row_bytes = (unsigned)(row_stride * 4);
  int dma_row[KV_DMA_PER];       // row inside the tile
  unsigned dma_col[KV_DMA_PER];  // byte offset inside the (K|V) row, V's includes +C floats
  unsigned dma_off[KV_DMA_PER];  // dma_row * row_bytes + dma_col
#pragma unroll
  for (int j = 0; j < KV_DMA_PER; j++) {
    const int gi = wave * KV_DMA_PER + j;
    const bool is_v = gi >= 16;
    const int row = 4 * (gi & 15) + (lane >> 4);
    const int c = is_v ? (lane & 15) : ((lane & 15) ^ (row & 7));
    dma_row[j] = row;
    dma_col[j] = (unsigned)(c * 16 + (is_v ? C * 4 : 0));
    dma_off[j] = (unsigned)row * row_bytes + dma_col[j];
  }
  auto dma_tile = [&](int tile, int buf) {
    const char* tile_base = kv_base + (size_t)tile * BKV * row_bytes;
    char* const dst = lds_bytes + buf * (2 * KV_TILE_BYTES) + wave * (KV_DMA_PER * 1024);
    if ((tile + 1) * BKV <= T) {
      asm volatile("" : "+s"(tile_base));  // keep "scalar base + lane offset" intact for selection
#pragma unroll
      for (int j = 0; j < KV_DMA_PER; j++)
        __builtin_amdgcn_global_load_lds((glb_void_t*)(tile_base + dma_off[j]),
                                         (lds_void_t*)(dst + j * 1024), 16, 0, 0);
    } else {
#pragma unroll
      for (int j = 0; j < KV_DMA_PER; j++) {
        const int key = min(tile * BKV + dma_row[j], T - 1);
        __builtin_amdgcn_global_load_lds(
            (glb_void_t*)(kv_base + (size_t)key * row_bytes + dma_col[j]),
            (lds_void_t*)(dst + j * 1024), 16, 0, 0);
      }
    }
  };

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

  // LDS read addresses (bytes, inside buffer 0, sub-tile 0); buffer and sub-tile are
  // immediate offsets of the read instructions.
  int k_addr[8];
#pragma unroll
  for (int g = 0; g < 8; g++) k_addr[g] = (l32 * KV_CH + ((2 * g + h32) ^ (lane & 7))) * 16;
  const int v_addr = KV_TILE_BYTES + (4 * h32) * (HS * 4) + l32 * 8;

  // Operand registers of one sub-tile: K as eight 16-byte chunks (A operand of the
  // score MFMAs), V as sixteen 8-byte pairs (A operand of the output MFMAs).
  struct Operands {
    f32x4 k[8];
    f32x2 v[16];
  };
  // All LDS reads of a sub-tile are issued in one batch, well before their first use:
  // V is read before the score MFMAs that precede its use, and the next sub-tile's K
  // before the output MFMAs of the current one.
  auto read_k = [&](Operands& op, int off) {
#pragma unroll
    for (int g = 0; g < 8; g++)
      op.k[g] = *reinterpret_cast<const f32x4*>(lds_bytes + k_addr[g] + off);
  };
  auto read_v = [&](Operands& op, int off) {
#pragma unroll
    for (int v = 0; v < 16; v++)
      op.v[v] = *reinterpret_cast<const f32x2*>(lds_bytes + v_addr +
                                                (off + (8 * (v >> 2) + (v & 3)) * (HS * 4)));
  };

  // Scores, lazy online softmax and output update of one sub-tile of 32 keys.
  auto sub_tile = [&](int k0, const Operands& op, auto&& before_output) {
    // S^T = K_sub . Q^T
    f32x16 s;
#pragma unroll
    for (int v = 0; v < 16; v++) s[v] = 0.f;
#pragma unroll
    for (int g = 0; g < 8; g++)
#pragma unroll
      for (int e = 0; e < 4; e++)
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(op.k[g][e], qreg[g][e], s, 0, 0, 0);

    // causal mask on the diagonal sub-tile
    if (k0 + 31 > qw) {
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

    before_output();

    // O^T += V_sub^T . P^T : register v pairs with key 8*(v/4) + 4*h32 + v%4
#pragma unroll
    for (int v = 0; v < 16; v++) {
      o0 = __builtin_amdgcn_mfma_f32_32x32x2f32(op.v[v].x, s[v], o0, 0, 0, 0);
      o1 = __builtin_amdgcn_mfma_f32_32x32x2f32(op.v[v].y, s[v], o1, 0, 0, 0);
    }
  };

  // One tile of 64 keys out of buffer BUF (a compile-time constant, so that every LDS
  // address is register + immediate).
  auto tile_body = [&](int tile, auto buf_tag) {
    constexpr int BUF = decltype(buf_tag)::value;
    constexpr int kbuf = BUF * (2 * KV_TILE_BYTES);
    constexpr int sub1 = 32 * (HS * 4);
    // the other buffer was last read before the barrier that ended the previous tile
    if (tile + 1 < ntile) dma_tile(tile + 1, BUF ^ 1);

    // this wave's 32 keys of the tile; wave-uniform: do they reach down to the diagonal?
    const int k0 = tile * BKV + khalf * 32;
    if (k0 <= qw + 31 && k0 < T) {
      Operands a;
      read_k(a, kbuf + khalf * sub1);
      read_v(a, kbuf + khalf * sub1);
      sub_tile(k0, a, []() {});
    }

    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): my DMAs of the next tile have landed
    __syncthreads();
  };

  dma_tile(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  __syncthreads();
  int tile = 0;
  for (; tile + 1 < ntile; tile += 2) {
    tile_body(tile, std::integral_constant<int, 0>{});
    tile_body(tile + 1, std::integral_constant<int, 1>{});
  }
  if (tile < ntile) tile_body(tile, std::integral_constant<int, 0>{});

  // ---- merge the two key halves of each query group --------------------------
  // The K/V buffers are idle after the loop's last barrier; the second wave of each
  // pair parks its partial state there, one float per (register, lane).
  float* const park = reinterpret_cast<float*>(lds_bytes) + qgroup * (35 * kWave) + lane;
  if (khalf == 1) {
#pragma unroll
    for (int v = 0; v < 16; v++) {
      park[v * kWave] = o0[v];
      park[(16 + v) * kWave] = o1[v];
    }
    park[32 * kWave] = m_used;
    park[33 * kWave] = l_run;
  }
  __syncthreads();
  if (khalf == 0) {
    const float m1 = park[32 * kWave], l1 = park[33 * kWave];
    const float m = fmaxf(m_used, m1);  // m_used is finite: key 0 is visible to every query
    const float a0 = __builtin_amdgcn_exp2f((m_used - m) * scale_log2e);
    const float a1 = __builtin_amdgcn_exp2f((m1 - m) * scale_log2e);  // 0 if that half saw no key
#pragma unroll
    for (int v = 0; v < 16; v++) {
      o0[v] = o0[v] * a0 + park[v * kWave] * a1;
      o1[v] = o1[v] * a0 + park[(16 + v) * kWave] * a1;
    }
    const float inv = 1.0f / pair_sum(l_run * a0 + l1 * a1);
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

__global__ __launch_bounds__(DEC_WAVES* kWave) void attention_decode64_kernel(
    float* __restrict__ out, const float* __restrict__ qkv, float* __restrict__ kc,
    float* __restrict__ vc, int pos, int maxT, int NH, float scale) {
  extern __shared__ float dec_lds[];  // scores [pos+1 rounded up to 64] | partial outputs [16][64]
  __shared__ float red[2 * DEC_WAVES];
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
  for (int g0 = wave; 4 * g0 <= pos; g0 += DEC_UNROLL * DEC_WAVES) {
    f32x4 kf[DEC_UNROLL];
#pragma unroll
    for (int u = 0; u < DEC_UNROLL; u++) {
      const int t = min(4 * (g0 + u * DEC_WAVES) + p4, pos);
      kf[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(kb + (size_t)t * 64));
    }
#pragma unroll
    for (int u = 0; u < DEC_UNROLL; u++) {
      const int t = 4 * (g0 + u * DEC_WAVES) + p4;
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
  for (int w = 1; w < DEC_WAVES; w++) m = fmaxf(m, red[w]);  // finite: position 0 always exists

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

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int g0 = wave; 4 * g0 <= pos; g0 += DEC_UNROLL * DEC_WAVES) {
    f32x4 vf[DEC_UNROLL];
    float pw[DEC_UNROLL];
#pragma unroll
    for (int u = 0; u < DEC_UNROLL; u++) {
      const int t = 4 * (g0 + u * DEC_WAVES) + p4;
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
    for (int w = 0; w < DEC_WAVES; w++) o += part[w * 64 + tid];
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
    hipLaunchKernelGGL(attention_decode64_kernel, dim3((unsigned)(B * NH)), dim3(DEC_WAVES * kWave), lds,
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
  if (hs == HS && aligned16(inp) && aligned16(out)) {
    const int nqt = (T + BQ - 1) / BQ;
    const long long blocks = (long long)nqt * B * NH;
    if (blocks > 0x7fffffffLL) return fail(GPT2HIP_EINVAL, "attention_forward: grid too large");
    const float scale_log2e = (1.0f / sqrtf((float)hs)) * 1.4426950408889634f;
    hipLaunchKernelGGL(attention_flash_kernel, dim3((unsigned)blocks), dim3(ATT_THREADS), 0, stream(), out,
                       inp, T, NH, nqt, scale_log2e);
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
