// One decode step (one new position for each of B <= 16 sequences) as ONE persistent
// kernel: 5 phases per transformer block + the lm-head, separated by grid-wide barriers.
//
// Why one kernel.  A decode step streams every weight once (498 MB for GPT-2 124M: 62 us
// at HBM speed) through 62 dependent matrix-vector-shaped operations.  As separate launches
// each of them costs 7-12 us however little it does (dispatch, ramp, drain), 0.73 ms per
// step.  Inside one kernel the hand-over between two operations is a barrier across the
// workgroups (~1.5 us, see below), and the next operation's weights are already on their
// way into the L2 while the barrier is waited for.
//
// Work split.  Every workgroup (one per compute unit, 4 waves: one per SIMD) takes N / gridDim.x
// consecutive weight rows (= output columns) of each GEMM for the whole K, at most 16 of
// them: one 16x16 MFMA tile per workgroup whose K range is split over the 4 waves
// (v_mfma_f32_16x16x4_f32, A = 16 weight rows, B = the <= 16 activation rows; partial
// tiles summed through LDS in wave order, so results are deterministic).  No output is
// shared between workgroups and nothing is reduced through memory.  The layernorms run
// inside the GEMMs that consume them (every workgroup recomputes the statistics of the
// <= 16 rows from the activations it loads anyway: llm.c's two passes, mean then
// variance), the residual adds inside the GEMMs that produce the update, GELU in the fc
// epilogue:
//   qkv = LN1(x) Wqkv | attention over the cache | x += y Wproj | h = gelu(LN2(x) Wfc) |
//   x += h Wfcproj
// (Four waves, not sixteen: a phase is a few hundred instructions of bookkeeping per wave
// around a few dozen loads and MFMAs, every wave repeats the bookkeeping, and with sixteen
// waves that repetition -- not memory -- set the pace: 5.4 us per layernorm+GEMM phase.)
// Attention takes one workgroup per (sequence, head): it appends the new key and value to
// the cache and runs the softmax over positions 0..pos, 16 lanes per cache row.
// The lm-head gives every wave 16-row groups of wte for the whole K (no cross-wave sum),
// with the normalised activations staged in LDS.
//
// Hand-over between workgroups.  Activations written in one phase are read by every
// workgroup in the next, across the eight XCDs, whose L2 caches are not coherent with
// each other.  Acquire/release fences at device scope (write back and invalidate the
// whole L2) made a grid barrier cost 12 us on this chip; instead the few KB of activations
// are written and read with cache-bypassing accesses (sc0 sc1) and the barrier is an array
// of per-workgroup epoch flags accessed the same way: a workgroup waits for its own
// stores to be acknowledged, publishes the phase number, and polls everybody's flag
// (1.5 us for 256 workgroups).  Weights and the cache rows of earlier steps are read-only
// for the kernel and go through the caches normally.  Every wait is bounded: a
// workgroup that spins too long raises an error word that makes every workgroup leave the
// kernel, and the host reports it on the next call.
#include "common.hpp"

namespace g2 {

constexpr int DS_WAVES = 4;
constexpr int DS_THREADS = DS_WAVES * kWave;
constexpr int TRACE_SLOTS = 8;
constexpr int FLAG_STRIDE = 16;  // one 64-byte line per workgroup's flag

// LDS carve-up, in floats
constexpr int LDS_RED = 0;                                // [waves][4][64] partial tiles
constexpr int LDS_STAT = LDS_RED + DS_WAVES * 4 * kWave;  // [2][waves][16 rows]
constexpr int LDS_SMALL = LDS_STAT + 2 * DS_WAVES * 16;   // [2][waves]: attention max / sum per wave
constexpr int LDS_BAD = LDS_SMALL + 2 * DS_WAVES;         // one int: a wait timed out
constexpr int LDS_SINK = LDS_BAD + 32;                    // 1 KiB that prefetches write and nobody reads
constexpr int LDS_FREE = LDS_SINK + 256;                  // attention scores | lm-head activations


// ---- cache-bypassing accesses for data that other workgroups wrote in this launch ---------
__device__ __forceinline__ f32x4 load_bypass4(const float* p) {
  f32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1" : "=v"(v) : "v"(p) : "memory");
  return v;  // not valid before wait_vm() + pin()
}
// The same into a register that already holds a value: lanes that are switched off keep it.
__device__ __forceinline__ void load_bypass4_into(f32x4& v, const float* p) {
  asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1" : "+v"(v) : "v"(p) : "memory");
}
__device__ __forceinline__ void store_bypass4(float* p, f32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" : : "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(0)" : : : "memory"); }
// Makes later uses of v depend on this point of the instruction stream (after wait_vm()).
__device__ __forceinline__ void pin(f32x4& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ float load_bypass(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_bypass(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
  for (int g = threadIdx.x; g < (int)gridDim.x; g += DS_THREADS) {
    const unsigned* f = a.flags + (size_t)g * FLAG_STRIDE;
    unsigned spins = 0;
    while ((int)(__hip_atomic_load(f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - epoch) < 0) {
      __builtin_amdgcn_s_sleep(1);
      ++spins;
      if (spins > a.spin_limit ||
          ((spins & 63) == 0 && __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
        __hip_atomic_store(err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *bad = 1;
        break;
      }
    }
  }
  lds_barrier();
  trace_mark(a, epoch - a.epoch0 - 1, 1);
  return *bad == 0;
}

// A workgroup's share of the N output columns.
struct Rows {
  int n0, nrows;
};
__device__ __forceinline__ Rows wg_rows(int N) {
  const int rp = (N + (int)gridDim.x - 1) / (int)gridDim.x;
  const int n0 = (int)blockIdx.x * rp;
  return {n0, min(rp, N - n0)};
}

// Warming the L2 of this workgroup's XCD with what the workgroup reads in its next phase:
// loads that write to a scrap KiB of LDS (global_load_lds_dwordx4: no destination registers
// that a late-landing load could clobber).  Issued right after the workgroup has arrived at
// a grid barrier, so that HBM latency runs while the barrier is waited for; the phase's own
// loads then hit the L2.
typedef __attribute__((address_space(3))) void lds_void_t;
typedef const __attribute__((address_space(1))) void glb_void_t;
__device__ __forceinline__ void touch(const float* p, float* lds) {
  __builtin_amdgcn_global_load_lds((glb_void_t*)p, (lds_void_t*)(lds + LDS_SINK), 16, 0, 0);
}
// n floats from p, 1 KiB per wave instruction, spread over the waves.
__device__ __forceinline__ void prefetch_span(float* lds, const float* p, int n, int pw, int lane) {
  for (int i = pw * 256 + lane * 4; i < n; i += DS_WAVES * 256) touch(p + i, lds);
}
// The weight rows, bias and layernorm parameters of a GEMM phase.
__device__ __forceinline__ void prefetch_gemm(float* lds, const float* W, const float* bias, int N, int K,
                                              const float* ln_w, const float* ln_b) {
  const int tid = opaque_tid(), lane = tid & 63;
  const int pw = __builtin_amdgcn_readfirstlane(tid >> 6);
  const Rows r = wg_rows(N);
  if (r.nrows <= 0) return;
  const float* wp = W + (size_t)(r.n0 + min(lane & 15, r.nrows - 1)) * K + 4 * (lane >> 4);
  const int units = K >> 4;
  for (int u = pw; u < units; u += DS_WAVES) touch(wp + (size_t)u * 16, lds);
  if (ln_w != nullptr) {
    prefetch_span(lds, ln_w, K, pw, lane);
    prefetch_span(lds, ln_b, K, pw, lane);
  }
  if (bias != nullptr && pw == 0 && lane < 5) {
    // the 16-byte pieces that hold bias[n0 .. n0 + nrows): at most five
    const float* b0 = bias + ((r.n0 & ~3) + 4 * lane);
    if (b0 < bias + r.n0 + r.nrows) touch(b0, lds);
  }
}
// The cache rows attention_item() will read for this workgroup's first (sequence, head): up to
// 24 wave instructions (4 rows of 256 bytes each) of keys and as many of values per wave.
__device__ __forceinline__ void prefetch_cache(const DecodeStep& a, float* lds, const float* kc,
                                               const float* vc) {
  const int tid = opaque_tid(), lane = tid & 63;
  const int pw = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int item = blockIdx.x;
  if (item >= a.B * a.NH || a.pos < 1) return;
  const int b = item / a.NH, head = item % a.NH;
  const size_t off = (size_t)b * a.maxT * a.C + head * 64 + 4 * (lane & 15);
  const int last = a.pos - 1;  // rows 0..pos-1 exist; row pos is written by the phase itself
  for (int i = 0; i < 24; i++) {
    const int t0 = 4 * (pw + DS_WAVES * i);
    if (t0 > last) break;
    const size_t row = (size_t)min(t0 + (lane >> 4), last) * a.C;
    touch(kc + off + row, lds);
    touch(vc + off + row, lds);
  }
}

// out[j][n0 + i] = resid + act( LN(in)[j] . W[n0 + i] + bias ) for this workgroup's columns.
// A wave's share of K is NCH chunks of U units; a chunk's loads are all issued at once.
// (NCH > 1 only without LN, whose statistics need the wave's whole share in registers.)
// GATHER: the input rows are wte[ids[j]] + wpe[pos] (the first phase of a step); workgroup 0
// also stores them as the residual stream x.
template <bool LN, bool GELU, bool GATHER, int U, int NCH>
__device__ __forceinline__ void gemm_phase(const DecodeStep& a, float* lds, const float* __restrict__ W,
                                           const float* __restrict__ bias, int N, int K,
                                           const float* in, const float* __restrict__ ln_w,
                                           const float* __restrict__ ln_b, float* out,
                                           const float* resid, unsigned ph = 0) {
  static_assert(!LN || NCH == 1, "a normalised row is held whole");
  const int tid = opaque_tid(), lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, kq = lane >> 4;
  const Rows r = wg_rows(N);
  if (r.nrows <= 0) return;  // the whole workgroup
  const int B = a.B;
  // epilogue element of this thread: column n0 + oi of row oj
  const int oi = tid & 15, oj = tid >> 4;
  const bool owner = oi < r.nrows && oj < B;
  float rs = 0.f, bs = 0.f;
  if (owner) {
    if (resid != nullptr) rs = load_bypass(resid + (size_t)oj * N + r.n0 + oi);
    if (bias != nullptr) bs = bias[r.n0 + oi];
  }

  // this lane's first float of the wave's share of K
  const size_t koff = (size_t)wave * (U * NCH * 16) + 4 * kq;
  const float* wp = W + (size_t)(r.n0 + r16) * K + koff;
  // Loads cost the compute unit's one load path 64 bytes per cycle whether or not lanes
  // repeat each other's addresses, so lanes beyond the workgroup's weight rows / beyond the
  // B activation rows are switched off (their operands are zero) instead of clamped, and
  // the layernorm's gamma and beta, which every row shares, go through LDS.
  float* const gb = lds + LDS_FREE;  // gamma [K] | beta [K]
  if (LN) {
    for (int i = tid * 4; i < K; i += DS_THREADS * 4) {
      *reinterpret_cast<f32x4*>(gb + i) = *reinterpret_cast<const f32x4*>(ln_w + i);
      *reinterpret_cast<f32x4*>(gb + K + i) = *reinterpret_cast<const f32x4*>(ln_b + i);
    }
  }
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ch = 0; ch < NCH; ch++) {
    f32x4 wv[U], xv[U];
#pragma unroll
    for (int c = 0; c < U; c++) {
      wv[c] = f32x4{0.f, 0.f, 0.f, 0.f};
      xv[c] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    if (r16 < r.nrows) {
#pragma unroll
      for (int c = 0; c < U; c++) wv[c] = *reinterpret_cast<const f32x4*>(wp + (ch * U + c) * 16);
    }
    if (GATHER) {
      if (r16 < B) {
        const int id = a.ids[r16];
        const bool ok = (unsigned)id < (unsigned)a.V;
        const float* tp = a.wte + (size_t)(ok ? id : 0) * K + koff;
        const float* pp = a.wpe_row + koff;
        const float q = __builtin_nanf("");
#pragma unroll
        for (int c = 0; c < U; c++) {
          xv[c] = *reinterpret_cast<const f32x4*>(tp + c * 16) + *reinterpret_cast<const f32x4*>(pp + c * 16);
          if (!ok) xv[c] = f32x4{q, q, q, q};
          if (blockIdx.x == 0) store_bypass4(a.x + (size_t)r16 * K + koff + c * 16, xv[c]);
        }
      }
    } else {
      if (r16 < B) {
        const float* xp = in + (size_t)r16 * K + koff;
#pragma unroll
        for (int c = 0; c < U; c++) load_bypass4_into(xv[c], xp + (ch * U + c) * 16);
      }
      if (ch == 0) trace_mark(a, ph, 2);
      wait_vm();
#pragma unroll
      for (int c = 0; c < U; c++) pin(xv[c]);
      if (ch == 0) trace_mark(a, ph, 3);
    }

    if (LN) {
      // row r16's statistics: lanes r16 + 16*kq of all the waves hold the row between them
      float* const stat = lds + LDS_STAT;
      float sum = 0.f;
#pragma unroll
      for (int c = 0; c < U; c++) sum += (xv[c][0] + xv[c][1]) + (xv[c][2] + xv[c][3]);
      sum += __shfl_xor(sum, 16, 64);
      sum += __shfl_xor(sum, 32, 64);
      if (kq == 0) stat[wave * 16 + r16] = sum;
      __syncthreads();
      float mean = 0.f;
#pragma unroll
      for (int w = 0; w < DS_WAVES; w++) mean += stat[w * 16 + r16];
      mean /= (float)K;
      float q = 0.f;
#pragma unroll
      for (int c = 0; c < U; c++) {
        const f32x4 d = xv[c] - mean;
        q += (d[0] * d[0] + d[1] * d[1]) + (d[2] * d[2] + d[3] * d[3]);
      }
      q += __shfl_xor(q, 16, 64);
      q += __shfl_xor(q, 32, 64);
      if (kq == 0) stat[DS_WAVES * 16 + wave * 16 + r16] = q;
      __syncthreads();
      float var = 0.f;
#pragma unroll
      for (int w = 0; w < DS_WAVES; w++) var += stat[DS_WAVES * 16 + w * 16 + r16];
      const float rstd = 1.0f / sqrtf(var / (float)K + 1e-5f);
#pragma unroll
      for (int c = 0; c < U; c++)
        xv[c] = (xv[c] - mean) * rstd * *reinterpret_cast<const f32x4*>(gb + koff + c * 16) +
                *reinterpret_cast<const f32x4*>(gb + K + koff + c * 16);
      trace_mark(a, ph, 4);
    }

#pragma unroll
    for (int c = 0; c < U; c++) {
#pragma unroll
      for (int e = 0; e < 4; e++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[c][e], xv[c][e], acc, 0, 0, 0);
    }
  }
  trace_mark(a, ph, 5);
  // lane l holds D[4*(l/16) + v][l % 16]: weight row (output column) 4*(l/16)+v, activation row l%16
  float* const red = lds + LDS_RED;
#pragma unroll
  for (int v = 0; v < 4; v++) red[(wave * 4 + v) * kWave + lane] = acc[v];
  __syncthreads();
  if (owner) {
    const int v = oi & 3, l = (oi >> 2) * 16 + oj;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < DS_WAVES; w++) sum += red[(w * 4 + v) * kWave + l];
    sum += bs;
    if (GELU) sum = gelu_tanh(sum);
    sum += rs;
    store_bypass(out + (size_t)oj * N + r.n0 + oi, sum);
  }
}

// One (sequence, head) of attention against the cache, head size 64: appends the new key and
// value (taken from the qkv row other workgroups just wrote), scores positions 0..pos with
// 16 lanes per cache row (a wave instruction covers four positions, 16 of them in flight),
// softmax through LDS, weighted values the same way.
__device__ __forceinline__ void attention_item(const DecodeStep& a, float* lds, float* kc, float* vc,
                                               int b, int head) {
  constexpr int UN = 16;
  const int tid = opaque_tid(), lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int p4 = lane >> 4, sub = lane & 15;
  const int C = a.C, pos = a.pos;
  float* const sc = lds + LDS_FREE;
  float* const part = sc + ((pos + 64) & ~63);
  float* const small = lds + LDS_SMALL;
  const float scale = 0.125f;
  const float* qrow = a.qkv + (size_t)b * 3 * C + head * 64 + 4 * sub;
  float* const kb = kc + (size_t)b * a.maxT * C + head * 64 + 4 * sub;
  float* const vb = vc + (size_t)b * a.maxT * C + head * 64 + 4 * sub;

  f32x4 q4 = load_bypass4(qrow);
  if (tid < 16) {
    f32x4 kn = load_bypass4(qrow + C);
    f32x4 vn = load_bypass4(qrow + 2 * C);
    wait_vm();
    pin(kn);
    pin(vn);
    *reinterpret_cast<f32x4*>(kb + (size_t)pos * C) = kn;
    *reinterpret_cast<f32x4*>(vb + (size_t)pos * C) = vn;
  }
  wait_vm();
  pin(q4);
  __syncthreads();  // the appended row is visible to the whole workgroup

  float mx = -INFINITY;
  for (int g0 = wave; 4 * g0 <= pos; g0 += UN * DS_WAVES) {
    f32x4 kf[UN];
#pragma unroll
    for (int u = 0; u < UN; u++) {
      const int t = min(4 * (g0 + u * DS_WAVES) + p4, pos);
      kf[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(kb + (size_t)t * C));
    }
#pragma unroll
    for (int u = 0; u < UN; u++) {
      const int t = 4 * (g0 + u * DS_WAVES) + p4;
      const f32x4 pr = q4 * kf[u];
      const float sv = row16_sum((pr[0] + pr[1]) + (pr[2] + pr[3])) * scale;
      if (t <= pos) {
        if (sub == 0) sc[t] = sv;
        mx = fmaxf(mx, sv);
      }
    }
  }
  mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
  mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
  if (lane == 0) small[wave] = mx;
  __syncthreads();
  float m = small[0];
#pragma unroll
  for (int w = 1; w < DS_WAVES; w++) m = fmaxf(m, small[w]);  // finite: position 0 always exists

  float sum = 0.f;
  for (int t = tid; t <= pos; t += DS_THREADS) {
    const float e = expf(sc[t] - m);
    sc[t] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  if (lane == 0) small[DS_WAVES + wave] = sum;
  __syncthreads();
  float l = 0.f;
#pragma unroll
  for (int w = 0; w < DS_WAVES; w++) l += small[DS_WAVES + w];

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int g0 = wave; 4 * g0 <= pos; g0 += UN * DS_WAVES) {
    f32x4 vf[UN];
    float pw[UN];
#pragma unroll
    for (int u = 0; u < UN; u++) {
      const int t = 4 * (g0 + u * DS_WAVES) + p4;
      pw[u] = (t <= pos) ? sc[t] : 0.f;
      vf[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(vb + (size_t)min(t, pos) * C));
    }
#pragma unroll
    for (int u = 0; u < UN; u++) acc += pw[u] * vf[u];
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
    for (int w = 0; w < DS_WAVES; w++) o += part[w * 64 + tid];
    store_bypass(a.atty + (size_t)b * C + head * 64 + tid, o / l);
  }
  __syncthreads();  // LDS is reused by the workgroup's next item
}

// logits = LNf(x) . wte^T.  The normalised rows go to LDS once per workgroup; wave w then
// takes the 16-row groups g + gridDim.x * (w + 4 i) of wte for the whole K, UC units at a
// time; the first units of its first group were requested into the L2 before the last barrier.
__device__ __forceinline__ int lm_head_first_group(int wave) {
  return (int)blockIdx.x + (int)gridDim.x * wave;
}
template <int UC>
__device__ __forceinline__ void prefetch_lm_head(const DecodeStep& a, float* lds) {
  const int tid = opaque_tid(), lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int K = a.C;
  prefetch_span(lds, a.lnfw, K, wave, lane);
  prefetch_span(lds, a.lnfb, K, wave, lane);
  const int cg = lm_head_first_group(wave);
  if (cg * 16 >= a.V) return;
  const float* wp = a.wte + (size_t)min(cg * 16 + (lane & 15), a.V - 1) * K + 4 * (lane >> 4);
#pragma unroll
  for (int c = 0; c < UC; c++) touch(wp + c * 16, lds);
}

// U1: units of K per wave in the layernorm (K = 64 * U1); UC: units per chunk of a wave's sweep
// over K (a divisor of 4 * U1).
template <int U1, int UC>
__device__ __forceinline__ void lm_head_phase(const DecodeStep& a, float* lds) {
  const int tid = opaque_tid(), lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, kq = lane >> 4;
  const int K = a.C, B = a.B, V = a.V;
  const int ldx = K + 4;  // row stride of the staged activations
  float* const xs = lds + LDS_FREE;
  {
    const size_t koff = (size_t)wave * (U1 * 16) + 4 * kq;
    float* const gb = xs + (size_t)B * ldx;  // gamma [K] | beta [K], shared by all rows
    for (int i = tid * 4; i < K; i += DS_THREADS * 4) {
      *reinterpret_cast<f32x4*>(gb + i) = *reinterpret_cast<const f32x4*>(a.lnfw + i);
      *reinterpret_cast<f32x4*>(gb + K + i) = *reinterpret_cast<const f32x4*>(a.lnfb + i);
    }
    f32x4 xv[U1];
#pragma unroll
    for (int c = 0; c < U1; c++) xv[c] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (r16 < B) {
      const float* xp = a.x + (size_t)r16 * K + koff;
#pragma unroll
      for (int c = 0; c < U1; c++) load_bypass4_into(xv[c], xp + c * 16);
    }
    wait_vm();
#pragma unroll
    for (int c = 0; c < U1; c++) pin(xv[c]);
    float* const stat = lds + LDS_STAT;
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < U1; c++) sum += (xv[c][0] + xv[c][1]) + (xv[c][2] + xv[c][3]);
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    if (kq == 0) stat[wave * 16 + r16] = sum;
    __syncthreads();
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
    __syncthreads();
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
    __syncthreads();
  }

  constexpr int NCH = 4 * U1 / UC;
  static_assert(NCH * UC == 4 * U1, "UC must divide the units of K");
  const float* const xrow = xs + (size_t)min(r16, B - 1) * ldx + 4 * kq;
  for (int cg = lm_head_first_group(wave); cg * 16 < V; cg += (int)gridDim.x * DS_WAVES) {
    const int n0 = cg * 16;
    const float* wp = a.wte + (size_t)min(n0 + r16, V - 1) * K + 4 * kq;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
    for (int ch = 0; ch < NCH; ch++) {
      f32x4 wv[UC];
#pragma unroll
      for (int c = 0; c < UC; c++)
        wv[c] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(wp + (size_t)(ch * UC + c) * 16));
#pragma unroll
      for (int c = 0; c < UC; c++) {
        const f32x4 xq = *reinterpret_cast<const f32x4*>(xrow + (ch * UC + c) * 16);
#pragma unroll
        for (int e = 0; e < 4; e++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[c][e], xq[e], acc, 0, 0, 0);
      }
    }
    if (r16 < B) {
      float* op = a.logits + (size_t)r16 * V + n0 + 4 * kq;
#pragma unroll
      for (int v = 0; v < 4; v++)
        if (n0 + 4 * kq + v < V) op[v] = acc[v];
    }
  }
}

// U1: units of K (16 floats) per wave where K = C (C = 64 * U1, so every wave has exactly that
// many and the loops carry no guards); where K = 4C a wave takes N4 chunks of U4 units
// (U4 * N4 = 4 * U1).  ULM: units per chunk of the lm-head's sweep.
template <int U1, int U4, int N4, int ULM>
__global__ __launch_bounds__(DS_THREADS) void decode_step_kernel(const DecodeStep a) {
  extern __shared__ float lds[];
  const int C = a.C;
  const size_t cs = (size_t)C;
  unsigned* const err = a.flags + (size_t)gridDim.x * FLAG_STRIDE;
  // a launch that follows a failed one does nothing until the host has cleared the error
  if (threadIdx.x == 0)
    *reinterpret_cast<int*>(lds + LDS_BAD) =
        __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
  __syncthreads();
  if (*reinterpret_cast<int*>(lds + LDS_BAD) != 0) return;
  unsigned epoch = a.epoch0;

#pragma unroll 1
  for (int l = 0; l < a.L; l++) {
    // qkv = LN1(x) Wqkv + b
    if (l == 0)
      gemm_phase<true, false, true, U1, 1>(a, lds, a.qkvw, a.qkvb, 3 * C, C, nullptr, a.ln1w, a.ln1b,
                                               a.qkv, nullptr, epoch - a.epoch0);
    else
      gemm_phase<true, false, false, U1, 1>(a, lds, a.qkvw + l * 3 * cs * cs, a.qkvb + l * 3 * cs, 3 * C,
                                                C, a.x, a.ln1w + l * cs, a.ln1b + l * cs, a.qkv, nullptr, epoch - a.epoch0);
    grid_arrive(a, ++epoch);
    prefetch_cache(a, lds, a.kv + (2 * (size_t)l) * a.plane, a.kv + (2 * (size_t)l + 1) * a.plane);
    if (!grid_wait(a, lds, epoch)) return;

    // attention over the cache
    for (int item = blockIdx.x; item < a.B * a.NH; item += gridDim.x)
      attention_item(a, lds, a.kv + (2 * (size_t)l) * a.plane, a.kv + (2 * (size_t)l + 1) * a.plane,
                     item / a.NH, item % a.NH);
    grid_arrive(a, ++epoch);
    prefetch_gemm(lds, a.attprojw + l * cs * cs, a.attprojb + l * cs, C, C, nullptr, nullptr);
    if (!grid_wait(a, lds, epoch)) return;

    // x += y Wproj + b
    gemm_phase<false, false, false, U1, 1>(a, lds, a.attprojw + l * cs * cs, a.attprojb + l * cs, C, C,
                                               a.atty, nullptr, nullptr, a.x, a.x, epoch - a.epoch0);
    grid_arrive(a, ++epoch);
    prefetch_gemm(lds, a.fcw + l * 4 * cs * cs, a.fcb + l * 4 * cs, 4 * C, C, a.ln2w + l * cs, a.ln2b + l * cs);
    if (!grid_wait(a, lds, epoch)) return;

    // h = gelu(LN2(x) Wfc + b)
    gemm_phase<true, true, false, U1, 1>(a, lds, a.fcw + l * 4 * cs * cs, a.fcb + l * 4 * cs, 4 * C, C,
                                             a.x, a.ln2w + l * cs, a.ln2b + l * cs, a.h, nullptr, epoch - a.epoch0);
    grid_arrive(a, ++epoch);
    prefetch_gemm(lds, a.fcprojw + l * 4 * cs * cs, a.fcprojb + l * cs, C, 4 * C, nullptr, nullptr);
    if (!grid_wait(a, lds, epoch)) return;

    // x += h Wfcproj + b
    gemm_phase<false, false, false, U4, N4>(a, lds, a.fcprojw + l * 4 * cs * cs, a.fcprojb + l * cs, C,
                                               4 * C, a.h, nullptr, nullptr, a.x, a.x, epoch - a.epoch0);
    grid_arrive(a, ++epoch);
    if (l + 1 < a.L)
      prefetch_gemm(lds, a.qkvw + (l + 1) * 3 * cs * cs, a.qkvb + (l + 1) * 3 * cs, 3 * C, C,
                    a.ln1w + (l + 1) * cs, a.ln1b + (l + 1) * cs);
    else
      prefetch_lm_head<ULM>(a, lds);
    if (!grid_wait(a, lds, epoch)) return;
  }
  lm_head_phase<U1, ULM>(a, lds);
  trace_mark(a, 5u * (unsigned)a.L, 0);
}

// ---- host ---------------------------------------------------------------------------------
int decode_step_workgroups(int device) {
  static int cached_device = -1, cached = 0;
  if (device == cached_device) return cached;
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return 0;
  cached_device = device;
  cached = cus;
  return cus;
}

size_t decode_step_flag_bytes(int device) {
  return ((size_t)decode_step_workgroups(device) * FLAG_STRIDE + FLAG_STRIDE) * sizeof(unsigned);
}

static size_t decode_step_lds_bytes(const GPT2Config& c, int B, int pos) {
  const size_t att = (size_t)((pos + 64) & ~63) + DS_WAVES * 64;
  const size_t lm = (size_t)B * (c.channels + 4) + 2 * (size_t)c.channels;  // rows | gamma | beta
  return (LDS_FREE + (att > lm ? att : lm)) * sizeof(float);
}

bool decode_step_supported(const GPT2Config& c, int B, int device) {
  const int C = c.channels, G = decode_step_workgroups(device);
  if (G < 1 || G > DS_THREADS) return false;
  if (B < 1 || B > 16 || c.num_heads * 64 != C) return false;
  // every wave takes exactly C/64 (4C/64) units of 16 floats of K; instantiated sizes only
  if (C != 64 && C != 128 && C != 256 && C != 512 && C != 768 && C != 1024) return false;
  if ((4 * C + G - 1) / G > 16) return false;  // the widest N: at most 16 weight rows per workgroup
  return decode_step_lds_bytes(c, B, c.max_seq_len - 1) <= 160 * 1024;
}

int decode_step_launch(const DecodeStep& step, const GPT2Config& c, int device) {
  const int G = decode_step_workgroups(device);
  const size_t lds = decode_step_lds_bytes(c, step.B, step.pos);
  const void* kernel;
  int slot;
  switch (c.channels) {
    case 64: kernel = reinterpret_cast<const void*>(decode_step_kernel<1, 4, 1, 4>); slot = 0; break;
    case 128: kernel = reinterpret_cast<const void*>(decode_step_kernel<2, 8, 1, 8>); slot = 1; break;
    case 256: kernel = reinterpret_cast<const void*>(decode_step_kernel<4, 16, 1, 16>); slot = 2; break;
    case 512: kernel = reinterpret_cast<const void*>(decode_step_kernel<8, 32, 1, 16>); slot = 3; break;
    case 768: kernel = reinterpret_cast<const void*>(decode_step_kernel<12, 48, 1, 24>); slot = 4; break;
    case 1024: kernel = reinterpret_cast<const void*>(decode_step_kernel<16, 32, 2, 32>); slot = 5; break;
    default: return fail(GPT2HIP_EINVAL, "decode step kernel: channels %d not supported", c.channels);
  }
  static bool lds_raised[6] = {false, false, false, false, false, false};
  if (lds > 48 * 1024 && !lds_raised[slot]) {
    G2_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    lds_raised[slot] = true;
  }
  DecodeStep copy = step;
  void* args[] = {&copy};
  G2_HIP(hipLaunchCooperativeKernel(kernel, dim3((unsigned)G), dim3(DS_THREADS), args, (unsigned)lds,
                                    stream()));
  return GPT2HIP_OK;
}

}  // namespace g2
