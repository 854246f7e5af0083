// One decode step (one new position for each of B <= 16 sequences) as ONE persistent
// kernel: 5 phases per transformer block + the lm-head, separated by grid-wide barriers.
//
// Why one kernel.  A decode step streams every weight once (498 MB for GPT-2 124M: 62 us
// at HBM speed) through 62 dependent matrix-vector-shaped operations.  As separate launches
// each of them costs 6-12 us however little it does (dispatch, ramp, drain), 0.61 ms per
// step.  Inside one kernel the hand-over between two operations is a barrier across the
// workgroups (~2 us, see below), and the next operation's weights are already on their
// way into registers while the current one computes.
//
// Work split.  The grid is exactly 256 workgroups of 4 waves (one wave per SIMD), one per
// compute unit, all resident at once.  Every workgroup takes N / 256 consecutive weight rows
// (= output columns) of each GEMM for the whole K: no output is shared between workgroups
// and nothing is reduced through memory.  The layernorms run inside the GEMMs that consume
// them (every workgroup recomputes the statistics of the <= 16 rows from the activations it
// loads anyway: llm.c's two passes, mean then variance), the residual adds inside the GEMMs
// that produce the update, GELU in the fc epilogue:
//   qkv = LN1(x) Wqkv | attention over the cache | x += y Wproj | h = gelu(LN2(x) Wfc) |
//   x += h Wfcproj
// (Four waves, not sixteen: a phase is a few hundred instructions of bookkeeping per wave
// around a few dozen loads and MFMAs, and every wave repeats the bookkeeping.)
// Attention takes one workgroup per (sequence, head) -- at long contexts one per range of
// positions of a (sequence, head) -- which appends the new key and value to the cache and
// runs the softmax over its positions, 16 lanes per cache row.
// The lm-head gives every wave 16-row groups of wte for the whole K (no cross-wave sum),
// with the normalised activations staged in LDS.
//
// Hand-over between workgroups.  Activations written in one phase are read by every
// workgroup in the next, across the eight XCDs, whose L2 caches are not coherent with
// each other.  Acquire/release fences at device scope (write back and invalidate the
// whole L2) made a grid barrier cost 12 us on this chip; instead the few KB of activations
// are written and read with cache-bypassing accesses (sc0 sc1) and the barrier is an array
// of per-workgroup epoch flags accessed the same way: a workgroup waits for its own
// stores to be acknowledged, publishes the phase number, and polls everybody's flag.
// Weights and the cache rows of earlier steps are read-only for the kernel and go through
// the caches normally.  Every wait is bounded: a workgroup that spins too long writes the
// step's position into an error word that makes every workgroup leave the kernel -- each
// filling the logits it owns with NaN -- and the host reports it when it next looks.
#include "common.hpp"

namespace g2 {

constexpr int DS_WAVES = 4;
constexpr int DS_THREADS = DS_WAVES * kWave;
constexpr int TRACE_SLOTS = 2;
constexpr int DS_GRID = 256;  // workgroups: the shapes below are compiled for exactly this many
constexpr int FLAG_STRIDE = 16;  // one 64-byte line per workgroup's flag

// LDS carve-up, in floats
constexpr int LDS_STAT = 0;                               // [2][16 sequences][4 waves x 4 lane rows]
constexpr int LDS_SMALL = LDS_STAT + 2 * 16 * 16;         // attention: max per (wave, lane row) [16] | sum per wave [4]
constexpr int LDS_BAD = LDS_SMALL + 32;                   // one int: a wait timed out
// GEMM phases: partial tiles [waves][NQ][64] | gamma, beta [2C]; attention: scores | partial
// outputs; lm-head: normalised rows | gamma, beta
constexpr int LDS_FREE = LDS_BAD + 32;


// Layout of the activations that one phase writes and every workgroup reads in the next (the
// residual stream x, the attention output, the MLP's hidden row): granules of 4 sequences x 4
// channels, [sequence / 4][channel / 4][sequence % 4][channel % 4], always 4 * JG sequences
// tall.  Lane (block b, r) of a wave feeds the MFMA sequence 4*jg + r at k = 4*b..4*b+3, so
// with this layout the 64 lanes of a load read 1 KB of consecutive memory.  With one row per
// sequence the same load touched 4 rows x 256 bytes, neighbouring lanes in different rows,
// and took the compute unit's load path four times as long (measured: 96 KB per workgroup
// in 2.9 us instead of 1.3 us).
__device__ __forceinline__ int granule_index(int seq, int channel, int channels) {
  return (seq >> 2) * 4 * channels + (channel >> 2) * 16 + (seq & 3) * 4 + (channel & 3);
}
// (maximum, sum) of range `split` of (sequence, head): the four sequences of a group side by side
__device__ __forceinline__ int split_stat_index(int split, int seq, int head, int heads) {
  return (((split * (kDecodeMaxBatch / 4) + (seq >> 2)) * heads + head) * 4 + (seq & 3)) * 2;
}
// Workgroup barrier that orders LDS traffic only (no wait for global loads in flight).
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory");
}

// The thread index as a value the compiler cannot trace back to threadIdx: address arithmetic
// built on it stays inside the phase that uses it instead of being computed once for all
// phases and kept in (spilled) registers across the whole kernel.
__device__ __forceinline__ int opaque_tid() {
  int t = threadIdx.x;
  asm volatile("" : "+v"(t));
  return t;
}

// ---- grid barrier ---------------------------------------------------------------------------
// arrive(): this workgroup's stores of the phase are acknowledged, its flag shows `epoch`.
__device__ __forceinline__ void trace_mark(const DecodeStep& a, unsigned phase, int k) {
  if (a.trace != nullptr && threadIdx.x == 0)
    a.trace[(size_t)(TRACE_SLOTS * phase + k) * gridDim.x + blockIdx.x] = wall_clock64();
}
__device__ __forceinline__ void grid_arrive(const DecodeStep& a, unsigned epoch) {
  trace_mark(a, epoch - a.epoch0 - 1, 0);
  wait_vm();
  __syncthreads();
  if (threadIdx.x == 0)
    __hip_atomic_store(&a.flags[(size_t)blockIdx.x * FLAG_STRIDE], epoch, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}
// wait(): every workgroup's flag shows `epoch` or later.  False if the wait was given up
// (then every workgroup gives up and the kernel ends).
__device__ __forceinline__ bool grid_wait(const DecodeStep& a, float* lds, unsigned epoch) {
  int* const bad = reinterpret_cast<int*>(lds + LDS_BAD);
  unsigned* const err = a.flags + (size_t)gridDim.x * FLAG_STRIDE;
  // Wave 0 polls, four flags per lane with all four loads in flight; the other waves come
  // straight to the barrier below.  (A poll is a trip to the memory side and back, ~0.9 us, and
  // a flag that lands just after a poll has passed waits a whole trip for the next one; a second
  // poll kept in flight half a trip behind the first was measured and is slower, 0.342-0.356
  // against 0.333 ms per step at 8 sequences: the 256 x 256 flag reads of a poll round are
  // traffic that the flags themselves have to get through.)
  if (threadIdx.x < kWave) {
    constexpr int PER = DS_GRID / kWave;
    unsigned spins = 0;
    auto issue = [&](unsigned (&v)[PER]) {
#pragma unroll
      for (int i = 0; i < PER; i++)
        v[i] = __hip_atomic_load(a.flags + (size_t)(threadIdx.x + kWave * i) * FLAG_STRIDE, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
    };
    auto complete = [&](const unsigned (&v)[PER]) {
      bool all = true;
#pragma unroll
      for (int i = 0; i < PER; i++) all = all && (int)(v[i] - epoch) >= 0;
      return all;
    };
    // after a poll that did not see everybody: whether to give up (and say so)
    auto give_up = [&]() {
      ++spins;
      const bool seen = (spins & 63) == 0 && __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (spins > a.spin_limit || seen) {
        // the error word names the step that failed first: position + 1, written once
        // (whoever writes it also tells the host, in the pinned word the host looks at once the
        // step has ended: the host does not copy the device's word behind every step)
        if (!seen && atomicCAS(err, 0u, (unsigned)a.pos + 1u) == 0u)
          __hip_atomic_store(a.error_host, (unsigned)a.pos + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        *bad = 1;
        return true;
      }
      return false;
    };
    for (;;) {
      unsigned v[PER];
      issue(v);
      if (complete(v)) break;
      __builtin_amdgcn_s_sleep(2);
      if (give_up()) break;
    }
  }
  lds_barrier();
  trace_mark(a, epoch - a.epoch0 - 1, 1);
  return *bad == 0;
}

// What a GEMM phase needs that does not depend on other workgroups: this lane's pieces of
// the workgroup's ROWS weight rows, this thread's piece of gamma and beta, the bias of the
// outputs this thread finishes.  It is loaded into registers one phase AHEAD, while the
// previous phase computes: HBM latency (and the 7-9 MB burst the 256 workgroups make of it)
// then runs under that phase's arithmetic, not in front of this phase and not while a grid
// barrier's flags have to get through the memory system.
template <int ROWS, int KG, int JG, bool LN>
struct PhaseWeights {
  static constexpr int RG = (ROWS + 3) / 4;
  static constexpr int NQ = RG * JG * 4;       // accumulator registers: (rg, jg, v)
  static constexpr int NIT = (NQ + 31) / 32;   // epilogue passes of 32 registers
  static constexpr int K = 256 * KG;
  f32x4 w[KG][RG];
  static constexpr int GN = (K + 1023) / 1024;  // pieces of gamma / beta per thread
  f32x4 g[GN], b[GN];  // gamma / beta [1024 p + 4 tid .. + 3]
  float bias[NIT];  // of output row 4*rg + v, for the thread that finishes register q = (rg, jg, v)
};
template <int ROWS, int KG, int JG, bool LN>
__device__ __forceinline__ void load_phase_weights(PhaseWeights<ROWS, KG, JG, LN>& pw, const float* __restrict__ W,
                                                   const float* __restrict__ bias,
                                                   const float* __restrict__ ln_w,
                                                   const float* __restrict__ ln_b) {
  using PW = PhaseWeights<ROWS, KG, JG, LN>;
  const int tid = opaque_tid(), lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int blk = lane >> 2, r4 = lane & 3;
  const int n0 = (int)blockIdx.x * ROWS;
  const int koff = wave * (KG * 64) + 4 * blk;  // this lane's first float of the wave's quarter of K
  // rows past the workgroup's share repeat the last one (they feed accumulator entries that
  // are never stored)
#pragma unroll
  for (int rg = 0; rg < PW::RG; rg++) {
    const float* wp = W + (size_t)(n0 + min(4 * rg + r4, ROWS - 1)) * PW::K + koff;
#pragma unroll
    for (int c = 0; c < KG; c++) pw.w[c][rg] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(wp + c * 64));
  }
  if (LN) {
#pragma unroll
    for (int p = 0; p < PW::GN; p++) {
      const int i = min(1024 * p + 4 * tid, PW::K - 4);
      pw.g[p] = *reinterpret_cast<const f32x4*>(ln_w + i);
      pw.b[p] = *reinterpret_cast<const f32x4*>(ln_b + i);
    }
  }
  const int eq = tid >> 3;
#pragma unroll
  for (int it = 0; it < PW::NIT; it++) {
    const int q = eq + 32 * it, row = 4 * (q / (4 * JG)) + (q & 3);
    pw.bias[it] = bias[n0 + min(row, ROWS - 1)];
  }
}

// The input of the projection phase when attention ran in S ranges per (sequence, head): the
// ranges' results combined, x = sum_s e_s o_s / sum_s e_s l_s with e_s = exp(m_s - max m).
// K = C, and a wave's group c of 64 k is exactly head wave * KG + c.  All loads are issued
// before anything is combined.
template <int S, int KG, int JG>
__device__ __forceinline__ void merge_splits(const DecodeStep& a, f32x4 (&xv)[KG][JG], int wave, int lane) {
  const int K = a.C, r4 = lane & 3;
  const Bypass part(a.att_part, (size_t)S * kDecodeMaxBatch * K);
  const int xoff = wave * (KG * 256) + 4 * lane;
  unsigned long long ml[JG][KG][S];
  f32x4 os[JG][KG][S];
#pragma unroll
  for (int jg = 0; jg < JG; jg++)
#pragma unroll
    for (int c = 0; c < KG; c++)
#pragma unroll
      for (int sp = 0; sp < S; sp++) {
        const float* p = a.att_ml + split_stat_index(sp, 4 * jg + r4, wave * KG + c, a.NH);
        ml[jg][c][sp] = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
        os[jg][c][sp] = part.load4(sp * kDecodeMaxBatch * K + jg * 4 * K + xoff + c * 256);
      }
#pragma unroll
  for (int jg = 0; jg < JG; jg++)
#pragma unroll
    for (int c = 0; c < KG; c++) {
      float ms[S], ls[S], mmax = -INFINITY;
#pragma unroll
      for (int sp = 0; sp < S; sp++) {
        ms[sp] = __builtin_bit_cast(float, (unsigned)(ml[jg][c][sp] & 0xffffffffu));
        ls[sp] = __builtin_bit_cast(float, (unsigned)(ml[jg][c][sp] >> 32));
        mmax = fmaxf(mmax, ms[sp]);
      }
      f32x4 num = {0.f, 0.f, 0.f, 0.f};
      float den = 0.f;
#pragma unroll
      for (int sp = 0; sp < S; sp++) {
        const float e = expf(ms[sp] - mmax);
        num += e * os[jg][c][sp];
        den += e * ls[sp];
      }
      xv[c][jg] = num / den;  // sequences past B: whatever the buffers hold, never stored
    }
}

// out[j][n0 + i] = resid + act( LN(in)[j] . W[n0 + i] + bias ) for this workgroup's ROWS output
// columns n0 = ROWS * blockIdx.x, on v_mfma_f32_4x4x1_16B_f32: sixteen independent 4x4 outer
// products per instruction, block b of lanes 4b..4b+3.  Lane (b, r) feeds weight row 4*rg + r
// and activation row 4*jg + r at the same k, so a block accumulates a 4x4 tile of
// (rows of group rg) x (sequences of group jg) over the k it is given; the 16 blocks take 16
// different k (element e of the lane's 16 bytes at k = 64*c + 4*b + e), the 4 waves a quarter
// of K each.  Loads are dense -- one instruction brings 256 bytes of each of 4 rows, every
// lane a distinct 16 bytes -- which is what bounds a phase: the compute unit's load path
// moves 64 bytes per cycle whether or not lanes repeat each other's addresses.  (A 16x16x4
// tile with 3 weight rows and 8 sequences in it spent 5 us of a 9 us phase issuing loads that
// were mostly repeats, and 3 us in mostly empty MFMAs.)  The 64 partial tiles (16 blocks x 4
// waves) are summed through LDS in a fixed order.
// KG: groups of 64 k per wave (K = 256 * KG); JG: groups of 4 sequences.
// GATHER: the input rows are wte[ids[j]] + wpe[pos] (the first phase of a step); workgroup 0
// also stores them as the residual stream x.  `in` and `resid` are in the granule layout, and
// so is `out` unless ROWMAJOR_OUT (qkv, which attention reads a head at a time).
// MERGE: the projection phase; with a.att_splits > 1 its input is combined from attention's
// ranges (merge_splits) instead of loaded from `in`.
template <bool LN, bool GELU, bool GATHER, bool ROWMAJOR_OUT, bool MERGE, int ROWS, int KG, int JG,
          typename LoadNext>
__device__ __forceinline__ void gemm_phase(const DecodeStep& a, float* lds,
                                           const PhaseWeights<ROWS, KG, JG, LN>& pw, const float* in, float* out,
                                           const float* resid, LoadNext&& load_next) {
  using PW = PhaseWeights<ROWS, KG, JG, LN>;
  constexpr int RG = PW::RG, NQ = PW::NQ, NIT = PW::NIT;
  constexpr int K = 256 * KG, N = ROWS * DS_GRID;
  const int tid = opaque_tid(), lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int blk = lane >> 2, r4 = lane & 3;
  const int n0 = (int)blockIdx.x * ROWS;
  const int B = a.B;
  float* const red = lds + LDS_FREE;             // [wave][NQ][64]
  float* const gb = red + DS_WAVES * NQ * kWave;  // gamma [K] | beta [K], with LN only

  // Epilogue role: threads 8q..8q+7 sum register q (+32 per pass) over blocks and waves; the
  // first four of them finish one output each (row 4*rg + v, sequence 4*jg + esub).
  const int eq = tid >> 3, esub = tid & 7;
  float rs[NIT];
  bool mine[NIT];
#pragma unroll
  for (int it = 0; it < NIT; it++) {
    const int q = eq + 32 * it, row = 4 * (q / (4 * JG)) + (q & 3), j = 4 * ((q >> 2) % JG) + esub;
    mine[it] = esub < 4 && q < NQ && row < ROWS && j < B;
    rs[it] = 0.f;
    if (resid != nullptr && mine[it]) rs[it] = load_bypass(resid + granule_index(j, n0 + row, N));
  }

  // this lane's first float of the wave's quarter of K
  const int koff = wave * (KG * 64) + 4 * blk;
  // Sequences past B are rows nobody writes (they feed accumulator entries that are never
  // stored).  This lane's granule (k piece wave * 16 KG + 16 c + blk, sequence 4 jg + r4):
  f32x4 xv[KG][JG];
  const Bypass xin(GATHER ? a.x : in, (size_t)4 * JG * K);
  const int xoff = wave * (KG * 256) + 4 * lane;
  // (the combinations the host asks for: up to 4 ranges with at most 4 sequences, 2 with at
  // most 8, none beyond: every combination is code that all phases share the instruction
  // cache with)
  const bool merge = MERGE && JG <= 2 && a.att_splits > 1;
  if (merge) {
    if (JG > 1 || a.att_splits == 2)
      merge_splits<2, KG, JG>(a, xv, wave, lane);
    else if (a.att_splits == 3)
      merge_splits<3, KG, JG>(a, xv, wave, lane);
    else
      merge_splits<4, KG, JG>(a, xv, wave, lane);
  }
#pragma unroll
  for (int jg = 0; jg < JG; jg++) {
    if (merge) break;
    if (GATHER) {
      const int bj = min(4 * jg + r4, B - 1);
      const int id = a.ids[bj];
      const bool ok = (unsigned)id < (unsigned)a.V;
      const float* tp = a.wte + (size_t)(ok ? id : 0) * K + koff;
      const float* pp = a.wpe_row + koff;
      const float qn = __builtin_nanf("");
#pragma unroll
      for (int c = 0; c < KG; c++) {
        xv[c][jg] = *reinterpret_cast<const f32x4*>(tp + c * 64) + *reinterpret_cast<const f32x4*>(pp + c * 64);
        if (!ok) xv[c][jg] = f32x4{qn, qn, qn, qn};
        if (blockIdx.x == 0 && 4 * jg + r4 < B) xin.store4(jg * 4 * K + xoff + c * 256, xv[c][jg]);
      }
    } else {
#pragma unroll
      for (int c = 0; c < KG; c++) xv[c][jg] = xin.load4(jg * 4 * K + xoff + c * 256);
    }
  }

  // The next phase's weights are requested right behind this phase's activations, before
  // anything waits: loads return in order, so the compiler's own waits for the activations
  // (a count of the loads issued after them) leave the weights in flight, and these have the
  // whole phase and its barrier to arrive in.  (Requested only once the activations had arrived,
  // the last of them were still missing when the phase ended: 0.346 -> 0.337 ms per step at 8
  // sequences, 0.432 -> 0.420 at 16.)
  load_next();
  if (LN) {
#pragma unroll
    for (int p = 0; p < PW::GN; p++)
      if (1024 * p + 4 * tid < K) {
        *reinterpret_cast<f32x4*>(gb + 1024 * p + 4 * tid) = pw.g[p];
        *reinterpret_cast<f32x4*>(gb + K + 1024 * p + 4 * tid) = pw.b[p];
      }
  }
  if (LN) {
    // Statistics of sequence 4*jg + r4: its row is spread over the 16 blocks of all 4 waves.
    // Two rotations inside each row of 16 lanes sum the row's 4 blocks; the 16 partial sums
    // (4 waves x 4 lane rows) of a sequence meet in LDS.
    float* const stat = lds + LDS_STAT;
    const int srow = wave * 4 + (lane >> 4);
    float mean[JG], rstd[JG];
#pragma unroll
    for (int jg = 0; jg < JG; jg++) {
      float sum = 0.f;
#pragma unroll
      for (int c = 0; c < KG; c++) sum += (xv[c][jg][0] + xv[c][jg][1]) + (xv[c][jg][2] + xv[c][jg][3]);
      sum += dpp<0x124>(sum);  // row_ror:4
      sum += dpp<0x128>(sum);  // row_ror:8
      if ((lane & 12) == 0) stat[(4 * jg + r4) * 16 + srow] = sum;
    }
    lds_barrier();  // not __syncthreads(): that would wait for the next phase's weights in flight
#pragma unroll
    for (int jg = 0; jg < JG; jg++) {
      const f32x4* const p = reinterpret_cast<const f32x4*>(stat + (4 * jg + r4) * 16);
      const f32x4 s4 = (p[0] + p[1]) + (p[2] + p[3]);
      const float m = (s4[0] + s4[1]) + (s4[2] + s4[3]);
      mean[jg] = m / (float)K;
      float q = 0.f;
#pragma unroll
      for (int c = 0; c < KG; c++) {
        const f32x4 d = xv[c][jg] - mean[jg];
        q += (d[0] * d[0] + d[1] * d[1]) + (d[2] * d[2] + d[3] * d[3]);
      }
      q += dpp<0x124>(q);
      q += dpp<0x128>(q);
      if ((lane & 12) == 0) stat[256 + (4 * jg + r4) * 16 + srow] = q;
    }
    lds_barrier();  // not __syncthreads(): that would wait for the next phase's weights in flight
#pragma unroll
    for (int jg = 0; jg < JG; jg++) {
      const f32x4* const p = reinterpret_cast<const f32x4*>(stat + 256 + (4 * jg + r4) * 16);
      const f32x4 s4 = (p[0] + p[1]) + (p[2] + p[3]);
      const float var = (s4[0] + s4[1]) + (s4[2] + s4[3]);
      rstd[jg] = 1.0f / sqrtf(var / (float)K + 1e-5f);
    }
#pragma unroll
    for (int c = 0; c < KG; c++) {
      const f32x4 g = *reinterpret_cast<const f32x4*>(gb + koff + c * 64);
      const f32x4 be = *reinterpret_cast<const f32x4*>(gb + K + koff + c * 64);
#pragma unroll
      for (int jg = 0; jg < JG; jg++) xv[c][jg] = (xv[c][jg] - mean[jg]) * rstd[jg] * g + be;
    }
  }

  f32x4 acc[RG][JG];
#pragma unroll
  for (int rg = 0; rg < RG; rg++)
#pragma unroll
    for (int jg = 0; jg < JG; jg++) acc[rg][jg] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int c = 0; c < KG; c++)
#pragma unroll
    for (int e = 0; e < 4; e++)
#pragma unroll
      for (int rg = 0; rg < RG; rg++)
#pragma unroll
        for (int jg = 0; jg < JG; jg++)
          acc[rg][jg] = __builtin_amdgcn_mfma_f32_4x4x1f32(pw.w[c][rg][e], xv[c][jg][e], acc[rg][jg], 0, 0, 0);

  // register v of lane (b, r) of acc[rg][jg]: weight row 4*rg + v, sequence 4*jg + r, block b's k
#pragma unroll
  for (int rg = 0; rg < RG; rg++)
#pragma unroll
    for (int jg = 0; jg < JG; jg++)
#pragma unroll
      for (int v = 0; v < 4; v++) red[(wave * NQ + (rg * JG + jg) * 4 + v) * kWave + lane] = acc[rg][jg][v];
  lds_barrier();  // not __syncthreads(): that would wait for the next phase's weights in flight
#pragma unroll
  for (int it = 0; it < NIT; it++) {
    const int q = eq + 32 * it;
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    if (q < NQ) {
#pragma unroll
      for (int w = 0; w < DS_WAVES; w++)
#pragma unroll
        for (int bi = 0; bi < 2; bi++)
          sum += *reinterpret_cast<const f32x4*>(red + (w * NQ + q) * kWave + (2 * esub + bi) * 4);
    }
#pragma unroll
    for (int j = 0; j < 4; j++) {
      sum[j] += dpp<0xB1>(sum[j]);   // quad_perm [1,0,3,2]
      sum[j] += dpp<0x4E>(sum[j]);   // quad_perm [2,3,0,1]
      sum[j] += dpp<0x141>(sum[j]);  // row_half_mirror: the other quad of the 8 lanes
    }
    const int row = 4 * (q / (4 * JG)) + (q & 3), j = 4 * ((q >> 2) % JG) + esub;
    if (mine[it]) {
      float val = (esub == 0 ? sum[0] : esub == 1 ? sum[1] : esub == 2 ? sum[2] : sum[3]) + pw.bias[it];
      if (GELU) val = gelu_tanh(val);
      store_bypass(out + (ROWMAJOR_OUT ? j * N + n0 + row : granule_index(j, n0 + row, N)), val + rs[it]);
    }
  }
}

// Attention of one new position against the cache, head size 64.  A compute unit streams
// cache rows at ~35 GB/s however many loads it keeps in flight, so at long contexts B * NH
// workgroups alone would leave the phase waiting for a third of the chip: from
// kSplitFromPos positions on, a (sequence, head) is cut into S = a.att_splits consecutive
// ranges of positions, one workgroup each.  Every range runs its own softmax -- maximum m,
// sum l, unnormalised weighted values o -- and stores (m, l, o); the projection phase
// combines the ranges when it loads its input (merge_splits).  With S = 1 the normalised
// result is stored as that phase's input directly.
//
// One range [tb, te]: 16 lanes hold one cache row, a wave instruction covers four positions,
// 16 of them in flight; scores go through LDS, weighted values the same way.  The range that
// ends at the new position appends the new key and value (taken from the qkv row other
// workgroups just wrote) to the cache first.
__device__ __forceinline__ void attention_item(const DecodeStep& a, float* lds, float* kc, float* vc,
                                               int b, int head, int split) {
  constexpr int UN = 16;
  const int tid = opaque_tid(), lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int p4 = lane >> 4, sub = lane & 15;
  const int C = a.C, pos = a.pos, S = a.att_splits;
  // ranges are multiples of four positions long; S > 1 only where every range is non-empty
  const int chunk = S == 1 ? pos + 1 : (((pos + S) / S + 3) & ~3);
  const int tb = split * chunk, te = min(pos, tb + chunk - 1), n = te - tb + 1;
  float* const sc = lds + LDS_FREE;
  float* const part = sc + ((n + 63) & ~63);
  float* const small = lds + LDS_SMALL;
  const float scale = 0.125f;
  // the cache is (B, NH, maxT, 64): the rows of this (sequence, head) are consecutive
  float* const kb = kc + ((size_t)(b * a.NH + head) * a.maxT + tb) * 64 + 4 * sub;
  float* const vb = vc + ((size_t)(b * a.NH + head) * a.maxT + tb) * 64 + 4 * sub;

  const Bypass qkv(a.qkv, (size_t)a.B * 3 * C);
  const int qi = b * 3 * C + head * 64 + 4 * sub;
  const f32x4 q4 = qkv.load4(qi);
  if (te == pos && tid < 16) {
    *reinterpret_cast<f32x4*>(kb + (size_t)(n - 1) * 64) = qkv.load4(qi + C);
    *reinterpret_cast<f32x4*>(vb + (size_t)(n - 1) * 64) = qkv.load4(qi + 2 * C);
  }
  __syncthreads();  // the appended row is visible to the whole workgroup

  float mx = -INFINITY;
  for (int g0 = wave; 4 * g0 < n; g0 += UN * DS_WAVES) {
    f32x4 kf[UN];
#pragma unroll
    for (int u = 0; u < UN; u++) {
      const int t = min(4 * (g0 + u * DS_WAVES) + p4, n - 1);
      kf[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(kb + (size_t)t * 64));
    }
#pragma unroll
    for (int u = 0; u < UN; u++) {
      const int t = 4 * (g0 + u * DS_WAVES) + p4;
      const f32x4 pr = q4 * kf[u];
      const float sv = row16_sum((pr[0] + pr[1]) + (pr[2] + pr[3])) * scale;
      if (t < n) {
        if (sub == 0) sc[t] = sv;
        mx = fmaxf(mx, sv);
      }
    }
  }
  // the 16 lanes of a row hold the same maximum; the 16 rows of the workgroup meet in LDS
  if (sub == 0) small[wave * 4 + p4] = mx;
  __syncthreads();
  float m;
  {
    const f32x4* const p = reinterpret_cast<const f32x4*>(small);
    const f32x4 m4 = {fmaxf(fmaxf(p[0][0], p[1][0]), fmaxf(p[2][0], p[3][0])),
                      fmaxf(fmaxf(p[0][1], p[1][1]), fmaxf(p[2][1], p[3][1])),
                      fmaxf(fmaxf(p[0][2], p[1][2]), fmaxf(p[2][2], p[3][2])),
                      fmaxf(fmaxf(p[0][3], p[1][3]), fmaxf(p[2][3], p[3][3]))};
    m = fmaxf(fmaxf(m4[0], m4[1]), fmaxf(m4[2], m4[3]));  // finite: the range is not empty
  }

  float sum = 0.f;
  for (int t = tid; t < n; t += DS_THREADS) {
    const float e = expf(sc[t] - m);
    sc[t] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  if (lane == 0) small[16 + wave] = sum;
  __syncthreads();
  float l = 0.f;
#pragma unroll
  for (int w = 0; w < DS_WAVES; w++) l += small[16 + w];

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int g0 = wave; 4 * g0 < n; g0 += UN * DS_WAVES) {
    f32x4 vf[UN];
    float pw[UN];
#pragma unroll
    for (int u = 0; u < UN; u++) {
      const int t = 4 * (g0 + u * DS_WAVES) + p4;
      pw[u] = (t < n) ? sc[t] : 0.f;
      vf[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(vb + (size_t)min(t, n - 1) * 64));
    }
#pragma unroll
    for (int u = 0; u < UN; u++) acc += pw[u] * vf[u];
  }
  *reinterpret_cast<f32x4*>(part + tid * 4) = acc;  // [wave][lane row][64 channels]
  __syncthreads();
  if (tid < 64) {
    float o = 0.f;
#pragma unroll
    for (int w = 0; w < 4 * DS_WAVES; w++) o += part[w * 64 + tid];
    if (S == 1) {
      store_bypass(a.atty + granule_index(b, head * 64 + tid, C), o / l);
    } else {
      store_bypass(a.att_part + (size_t)split * kDecodeMaxBatch * C + granule_index(b, head * 64 + tid, C), o);
      if (tid < 2) store_bypass(a.att_ml + split_stat_index(split, b, head, a.NH) + tid, tid == 0 ? m : l);
    }
  }
}

// logits = LNf(x) . wte^T.  The normalised rows go to LDS once per workgroup; wave w then
// takes the 16-row groups g + gridDim.x * (w + 4 i) of wte for the whole K, UC units at a
// time.
__device__ __forceinline__ int lm_head_first_group(int wave) {
  return (int)blockIdx.x + (int)gridDim.x * wave;
}
// U1: units of K per wave in the layernorm (K = 64 * U1); UC: units per chunk of a wave's
// sweep over K.
template <int U1, int UC>
__device__ __forceinline__ void lm_head_phase(const DecodeStep& a, float* lds) {
  const int tid = opaque_tid(), lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, kq = lane >> 4;
  const int K = a.C, B = a.B, V = a.V;
  const int ldx = K + 4;  // row stride of the staged activations
  float* const xs = lds + LDS_FREE;
  // Every group is NCH (even) chunks of UC units.  One chunk is always in flight ahead of the
  // MFMAs, across group boundaries too: while the last chunk of a group is multiplied, the
  // first chunk of the wave's next group is already loading -- and the very first chunk loads
  // while the layernorm below runs (its barriers do not wait for loads in flight).
  constexpr int NCH = 4 * U1 / UC;
  static_assert(NCH * UC == 4 * U1 && NCH % 2 == 0, "a group is an even number of chunks");
  const int step = (int)gridDim.x * DS_WAVES;
  int cg = lm_head_first_group(wave);
  f32x4 wa[UC], wb[UC];
  const float* wp = a.wte + (size_t)min(cg * 16 + r16, V - 1) * K + 4 * kq;
  {
    const size_t koff = (size_t)wave * (U1 * 16) + 4 * kq;
    float* const gb = xs + (size_t)B * ldx;  // gamma [K] | beta [K], shared by all rows
    for (int i = tid * 4; i < K; i += DS_THREADS * 4) {
      *reinterpret_cast<f32x4*>(gb + i) = *reinterpret_cast<const f32x4*>(a.lnfw + i);
      *reinterpret_cast<f32x4*>(gb + K + i) = *reinterpret_cast<const f32x4*>(a.lnfb + i);
    }
    f32x4 xv[U1];
    {
      const Bypass xin(a.x, (size_t)16 * K);  // granule layout; rows past B are never stored below
      const int xi = granule_index(r16, (int)koff, K);
#pragma unroll
      for (int c = 0; c < U1; c++) xv[c] = xin.load4(xi + c * 64);
    }
    if (cg * 16 < V) {
#pragma unroll
      for (int c = 0; c < UC; c++)
        wa[c] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(wp + (size_t)c * 16));
    }
    float* const stat = lds + LDS_STAT;
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < U1; c++) sum += (xv[c][0] + xv[c][1]) + (xv[c][2] + xv[c][3]);
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    if (kq == 0) stat[wave * 16 + r16] = sum;
    lds_barrier();
    float mean = 0.f;
#pragma unroll
    for (int w = 0; w < DS_WAVES; w++) mean += stat[w * 16 + r16];
    mean /= (float)K;
    float q = 0.f;
#pragma unroll
    for (int c = 0; c < U1; c++) {
      const f32x4 d = xv[c] - mean;
      q += (d[0] * d[0] + d[1] * d[1]) + (d[2] * d[2] + d[3] * d[3]);
    }
    q += __shfl_xor(q, 16, 64);
    q += __shfl_xor(q, 32, 64);
    if (kq == 0) stat[DS_WAVES * 16 + wave * 16 + r16] = q;
    lds_barrier();
    float var = 0.f;
#pragma unroll
    for (int w = 0; w < DS_WAVES; w++) var += stat[DS_WAVES * 16 + w * 16 + r16];
    const float rstd = 1.0f / sqrtf(var / (float)K + 1e-5f);
    if (r16 < B) {
#pragma unroll
      for (int c = 0; c < U1; c++)
        *reinterpret_cast<f32x4*>(xs + (size_t)r16 * ldx + koff + c * 16) =
            (xv[c] - mean) * rstd * *reinterpret_cast<const f32x4*>(gb + koff + c * 16) +
            *reinterpret_cast<const f32x4*>(gb + K + koff + c * 16);
    }
    lds_barrier();
  }

  const float* const xrow = xs + (size_t)min(r16, B - 1) * ldx + 4 * kq;
  for (; cg * 16 < V; cg += step) {
    const int n0 = cg * 16;
    const float* const wnext = a.wte + (size_t)min(n0 + step * 16 + r16, V - 1) * K + 4 * kq;
    const bool more = (cg + step) * 16 < V;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ch = 0; ch < NCH; ch++) {
      f32x4(&cur)[UC] = (ch & 1) ? wb : wa;
      f32x4(&nxt)[UC] = (ch & 1) ? wa : wb;
      if (ch + 1 < NCH) {
#pragma unroll
        for (int c = 0; c < UC; c++)
          nxt[c] = __builtin_nontemporal_load(
              reinterpret_cast<const f32x4*>(wp + (size_t)((ch + 1) * UC + c) * 16));
      } else if (more) {
        // rows of the next group (clamped: past the end nothing is stored, and the loop ends)
#pragma unroll
        for (int c = 0; c < UC; c++)
          nxt[c] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(wnext + (size_t)c * 16));
      }
#pragma unroll
      for (int c = 0; c < UC; c++) {
        const f32x4 xq = *reinterpret_cast<const f32x4*>(xrow + (ch * UC + c) * 16);
#pragma unroll
        for (int e = 0; e < 4; e++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(cur[c][e], xq[e], acc, 0, 0, 0);
      }
    }
    wp = wnext;
    if (r16 < B) {
      float* op = a.logits + (size_t)r16 * V + n0 + 4 * kq;
#pragma unroll
      for (int v = 0; v < 4; v++)
        if (n0 + 4 * kq + v < V) op[v] = acc[v];
    }
  }
}

// Workgroups without an attention item would only wait at the phase's barrier.  Instead each
// reads cache rows on behalf of one item whose workgroup sits in the same XCD (consecutive
// workgroup ids are dealt round-robin to the 8 XCDs), so that they are in that XCD's L2 when
// the item asks for them: `first` (this layer's values, which the item wants only after its
// pass over the keys) and `second` (the next layer's keys, wanted five phases from now).
// The values are discarded; a wrong guess about the XCD costs nothing but the benefit.
__device__ __forceinline__ void warm_rows(const DecodeStep& a, const float* first, const float* second, int items) {
  const int g = (int)blockIdx.x, x = g & 7;
  const int idle0 = items + ((x - items) & 7);  // the first idle workgroup of this XCD
  const int item = x + 8 * ((g - idle0) >> 3);  // the XCD's items are x, x + 8, ...
  // (only while every item finds a helper: with more items than idle workgroups the extra
  // traffic cost more than the warmed items gained)
  if (2 * items > (int)gridDim.x || item >= items) return;
  const size_t base = (size_t)item * a.maxT * 64;
  const int floats = a.pos * 64;  // rows 0 .. pos-1 of the (sequence, head)
  f32x4 sink = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
  for (int pass = 0; pass < 2; pass++) {
    const float* rows = pass == 0 ? first : second;
    if (rows == nullptr) continue;
    rows += base;
    for (int i = (int)threadIdx.x * 4; i < floats; i += DS_THREADS * 4 * 8) {
      f32x4 t[8];
#pragma unroll
      for (int u = 0; u < 8; u++)
        t[u] = *reinterpret_cast<const f32x4*>(rows + min(i + u * DS_THREADS * 4, floats - 4));
#pragma unroll
      for (int u = 0; u < 8; u++) sink += t[u];
    }
  }
  asm volatile("" : : "v"(sink));
}

// A step that ends early must not leave the previous step's logits behind as if they were its
// own: every workgroup that leaves fills the logits it owns in the lm-head phase (the same
// 16-row groups, for every sequence) with NaN.  Nobody else writes those, so they stay NaN
// whatever the other workgroups still manage to do.
__device__ __forceinline__ void fail_logits(const DecodeStep& a) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int step = (int)gridDim.x * DS_WAVES;
  for (int cg = lm_head_first_group(wave); cg * 16 < a.V; cg += step) {
    const int n = cg * 16 + (lane & 15);
    if (n < a.V)
      for (int b = lane >> 4; b < a.B; b += 4) a.logits[(size_t)b * a.V + n] = __builtin_nanf("");
  }
}

// KG1 = C / 256: groups of 64 k per wave where K = C, and weight rows per workgroup where
// N = C (the grid is exactly DS_GRID = 256 workgroups).  JG: groups of 4 sequences.
// ULM: units of 16 k per chunk of the lm-head's sweep.
template <int KG1, int JG, int ULM>
__global__ __launch_bounds__(DS_THREADS) void decode_step_kernel(const DecodeStep a) {
  extern __shared__ float lds[];
  constexpr int C = 256 * KG1;
  constexpr size_t cs = (size_t)C;
  unsigned* const err = a.flags + (size_t)gridDim.x * FLAG_STRIDE;
  // a launch that follows a failed one computes nothing until the host has cleared the error
  if (threadIdx.x == 0)
    *reinterpret_cast<int*>(lds + LDS_BAD) =
        __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
  __syncthreads();
  if (*reinterpret_cast<int*>(lds + LDS_BAD) != 0) {
    fail_logits(a);
    return;
  }
  unsigned epoch = a.epoch0;

  const int items = a.B * a.NH * a.att_splits;  // (sequence, head, range) triples of the attention phase
  PhaseWeights<3 * KG1, KG1, JG, true> w_qkv;
  PhaseWeights<KG1, KG1, JG, false> w_proj;
  PhaseWeights<4 * KG1, KG1, JG, true> w_fc;
  PhaseWeights<KG1, 4 * KG1, JG, false> w_fcproj;
  load_phase_weights(w_qkv, a.qkvw, a.qkvb, a.ln1w, a.ln1b);
#pragma unroll 1
  for (int l = 0; l < a.L; l++) {
    float* const kc = a.kv + (2 * (size_t)l) * a.plane;
    float* const vc = kc + a.plane;
    // qkv = LN1(x) Wqkv + b
    auto next_proj = [&]() { load_phase_weights(w_proj, a.attprojw + l * cs * cs, a.attprojb + l * cs, nullptr, nullptr); };
    if (l == 0)
      gemm_phase<true, false, true, true, false>(a, lds, w_qkv, nullptr, a.qkv, nullptr, next_proj);
    else
      gemm_phase<true, false, false, true, false>(a, lds, w_qkv, a.x, a.qkv, nullptr, next_proj);
    grid_arrive(a, ++epoch);
    if (!grid_wait(a, lds, epoch)) {
      fail_logits(a);
      return;
    }

    // attention over the cache
    // at most one item per workgroup: B <= 16 sequences of at most 1024 / 64 heads, and the
    // host splits only as far as the grid goes
    if ((int)blockIdx.x < items) {
      const int bh = (int)blockIdx.x / a.att_splits;
      attention_item(a, lds, kc, vc, bh / a.NH, bh % a.NH, (int)blockIdx.x % a.att_splits);
    } else if (a.att_splits == 1) {
      // this layer's values (the item asks for them only after its pass over the keys) and the
      // next layer's keys
      warm_rows(a, vc, l + 1 < a.L ? kc + 2 * a.plane : nullptr, items);
    }
    grid_arrive(a, ++epoch);
    if (!grid_wait(a, lds, epoch)) {
      fail_logits(a);
      return;
    }

    // x += y Wproj + b
    gemm_phase<false, false, false, false, true>(a, lds, w_proj, a.atty, a.x, a.x, [&]() {
      load_phase_weights(w_fc, a.fcw + l * 4 * cs * cs, a.fcb + l * 4 * cs, a.ln2w + l * cs, a.ln2b + l * cs);
    });
    grid_arrive(a, ++epoch);
    if (!grid_wait(a, lds, epoch)) {
      fail_logits(a);
      return;
    }

    // h = gelu(LN2(x) Wfc + b)
    gemm_phase<true, true, false, false, false>(a, lds, w_fc, a.x, a.h, nullptr, [&]() {
      load_phase_weights(w_fcproj, a.fcprojw + l * 4 * cs * cs, a.fcprojb + l * cs, nullptr, nullptr);
    });
    grid_arrive(a, ++epoch);
    if (!grid_wait(a, lds, epoch)) {
      fail_logits(a);
      return;
    }

    // x += h Wfcproj + b
    gemm_phase<false, false, false, false, false>(a, lds, w_fcproj, a.h, a.x, a.x, [&]() {
      if (l + 1 < a.L)
        load_phase_weights(w_qkv, a.qkvw + (l + 1) * 3 * cs * cs, a.qkvb + (l + 1) * 3 * cs,
                           a.ln1w + (l + 1) * cs, a.ln1b + (l + 1) * cs);
    });
    grid_arrive(a, ++epoch);
    if (!grid_wait(a, lds, epoch)) {
      fail_logits(a);
      return;
    }
  }
  lm_head_phase<4 * KG1, ULM>(a, lds);
  trace_mark(a, 5u * (unsigned)a.L, 0);
}

// ---- host ---------------------------------------------------------------------------------
// The kernel runs on exactly DS_GRID workgroups, one per compute unit, all resident at once.
static bool device_has_grid(int device) {
  int cus = 0;  // a cached attribute of the runtime: no state of our own to keep per device or thread
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return false;
  return cus >= DS_GRID;
}

size_t decode_step_flag_bytes(int device) {
  (void)device;
  return ((size_t)DS_GRID * FLAG_STRIDE + FLAG_STRIDE) * sizeof(unsigned);
}

size_t decode_step_probe_slots(int num_layers) {
  return (size_t)DS_GRID * TRACE_SLOTS * (5 * (size_t)num_layers + 1);
}

// Ranges per (sequence, head) of the attention phase at position pos.  Splitting pays from a
// few hundred positions on (the projection phase loads S results instead of one: +1.3 us, and
// with every workgroup holding an item nobody is left to warm cache rows, see warm_rows): from
// 384 positions where up to four ranges are possible, from 640 where only two are (measured
// at 5, 6 and 8 sequences: unsplit is ahead up to 600-700 positions, split beyond).
constexpr int kSplitFromPos = 384, kSplitInTwoFromPos = 640;
int decode_step_attention_splits(const GPT2Config& c, int B, int pos) {
  if (pos < kSplitFromPos) return 1;
  const int s = DS_GRID / (B * c.num_heads);  // as far as the grid goes
  if (s < 2 || B > 8) return 1;  // the kernel combines ranges only for up to 8 sequences,
  if (B > 4) return pos < kSplitInTwoFromPos ? 1 : 2;  // and more than 2 of them only for up to 4
  return s > kDecodeMaxSplits ? kDecodeMaxSplits : s;
}

// Floats of the activation buffer the kernel hands data between workgroups in: x, attention
// output, hidden row (granule layout, 16 sequences tall), the attention ranges' partial
// outputs and their (maximum, sum) pairs.
size_t decode_step_activation_floats(const GPT2Config& c) {
  const size_t C = c.channels;
  return (size_t)kDecodeMaxBatch * (6 + kDecodeMaxSplits) * C +
         (size_t)kDecodeMaxSplits * kDecodeMaxBatch * c.num_heads * 2;
}

static size_t decode_step_lds_bytes(const GPT2Config& c, int B, int pos) {
  const size_t C = c.channels, jg = (B + 3) / 4;
  const size_t gemm = 2 * C + DS_WAVES * ((C / 256) * jg * 4) * kWave;  // gamma, beta | partial tiles
  const size_t att = (size_t)((pos + 64) & ~63) + 4 * DS_WAVES * 64;    // scores | partial outputs
  const size_t lm = (size_t)B * (C + 4) + 2 * C;                        // rows | gamma, beta
  size_t most = gemm > att ? gemm : att;
  if (lm > most) most = lm;
  return (LDS_FREE + most) * sizeof(float);
}

bool decode_step_supported(const GPT2Config& c, int B, int device) {
  const int C = c.channels;
  if (!device_has_grid(device)) return false;
  if (B < 1 || B > kDecodeMaxBatch || c.num_heads * 64 != C) return false;
  if (B * c.num_heads > DS_GRID) return false;  // the attention phase has one workgroup per (sequence, head)
  // the instantiated sizes (1280 channels, GPT-2 large: with 9 to 16 sequences the fcproj phase's 20
  // weight pieces and 20 activation pieces per group of four sequences no longer all fit in
  // registers and 80-420 bytes per lane spill; a step is still a third shorter than one launch per
  // operation: 1.79 / 1.83 against 2.74 / 2.89 ms at 9 / 12 sequences, 36 layers; its 20 heads allow
  // 12 sequences)
  if (C != 256 && C != 512 && C != 768 && C != 1024 && C != 1280) return false;
  return decode_step_lds_bytes(c, B, c.max_seq_len - 1) <= 160 * 1024;
}

template <int KG1, int ULM>
static const void* kernel_for(int jg) {
  switch (jg) {
    case 1: return reinterpret_cast<const void*>(decode_step_kernel<KG1, 1, ULM>);
    case 2: return reinterpret_cast<const void*>(decode_step_kernel<KG1, 2, ULM>);
    case 3: return reinterpret_cast<const void*>(decode_step_kernel<KG1, 3, ULM>);
    default: return reinterpret_cast<const void*>(decode_step_kernel<KG1, 4, ULM>);
  }
}

int decode_step_launch(const DecodeStep& step, const GPT2Config& c, int device) {
  if (!decode_step_supported(c, step.B, device))
    return fail(GPT2HIP_EINVAL, "decode step kernel: model or batch not supported");
  const size_t lds = decode_step_lds_bytes(c, step.B, step.pos);
  const int jg = (step.B + 3) / 4, kg1 = c.channels / 256;
  const void* kernel = kg1 == 1   ? kernel_for<1, 8>(jg)
                       : kg1 == 2 ? kernel_for<2, 16>(jg)
                       : kg1 == 3 ? kernel_for<3, 24>(jg)
                       : kg1 == 4 ? kernel_for<4, 16>(jg)
                                  : kernel_for<5, 10>(jg);
  // the dynamic-LDS limit is a per-device property of the kernel: remembered per thread and
  // device, like the GEMM launchers do
  if (lds > 48 * 1024) {
    static thread_local int raised_on = -1;
    static thread_local bool raised[5][4];
    if (raised_on != device) {
      raised_on = device;
      for (auto& row : raised)
        for (bool& b : row) b = false;
    }
    if (!raised[kg1 - 1][jg - 1]) {
      G2_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
      raised[kg1 - 1][jg - 1] = true;
    }
  }
  // An ordinary launch: with one workgroup per compute unit's worth of resources and nothing
  // else running on the device, all DS_GRID workgroups are resident at once, which the grid
  // barrier needs.  If they ever are not (a device shared with other work), the barrier's
  // bounded wait ends the kernel and the error is reported; it cannot hang.
  DecodeStep copy = step;
  void* args[] = {&copy};
  G2_HIP(hipLaunchKernel(kernel, dim3(DS_GRID), dim3(DS_THREADS), args, lds, stream()));
  return GPT2HIP_OK;
}

}  // namespace g2
