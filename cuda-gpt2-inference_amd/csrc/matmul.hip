// matmul_forward for gfx950: out(M,N) = inp(M,K) . weight(N,K)^T + bias(N),
// optional tanh-GELU epilogue.  True fp32 on the matrix cores
// (v_mfma_f32_32x32x2_f32; gfx950 has no xf32 path).
//
// The kernels (matmul_dma_kernel, matmul_ring_kernel and matmul_mfma_kernel share one tiling,
// LDS layout and MFMA mapping):
//   matmul_dma_kernel      K % 32 == 0 (every GPT-2 shape): K slabs go from global
//                          memory straight into LDS (global_load_lds_dwordx4)
//   matmul_ring_kernel     the same for problems of few small tiles (short prompts):
//                          deeper slab ring, optional K split between a tile's waves
//   (both also in a form that splits K between the workgroups of a tile, for callers that
//   lend a workspace: splitk_combine, matmul_forward_splitk_status)
//   matmul_skinny_kernel   at most 16 rows (a decode step): weights streamed through
//                          registers once, 16x16x4 MFMA, K split over 16 waves
//   matmul_mfma_kernel     any K % 4 == 0: slabs staged through registers, K tail
//                          zero-filled
//   matmul_generic_kernel  anything else (K % 4 != 0, unaligned pointers)
//
// Tiling.  A workgroup owns a BM x BN output tile and walks K in slabs of
// BK = 32.  Both operands are K-contiguous in memory ("NT" GEMM), so a slab of
// either is rows of 32 floats = 8 chunks of 16 bytes, held in one of two LDS
// buffers; there is one barrier per slab, placed inside the slab's MFMA work so
// that no wave waits on a fill->barrier->read chain.  In LDS, chunk c of row r sits
// at chunk position c ^ (r & 7): eight lanes that read the same logical chunk of
// eight consecutive rows then hit eight different 16-byte bank groups.
//
// MFMA operand mapping.  v_mfma_f32_32x32x2_f32 takes A[i][k] from lane
// (i = lane%32, k = lane/32) and B[k][j] from lane (j = lane%32, k = lane/32).
// A lane with h = lane/32 reads the 16-byte chunk 2g+h of its row, i.e.
// k = 8g+4h .. 8g+4h+3, and feeds element s of it to the s-th of four MFMAs:
// that MFMA multiplies k = 8g+s (lanes 0..31) and k = 8g+4+s (lanes 32..63).
// A and B use the same k permutation, so the contraction is unchanged and one
// ds_read_b128 per 32 rows feeds four MFMAs.
//
// The accumulator of lane l, register v holds D[8*(v/4) + 4*(l/32) + v%4][l%32]:
// a lane owns one output column, so the bias is folded into the accumulator's
// initial value (as the reference does, 9_matmul_async_cg_tf32_gelu.cuh:56-84)
// and every store instruction writes two 128-byte row segments.
//
// What bounds it.  Measured with the in-kernel clock probe below: a slab of a
// 128x192 tile costs 6363 shader clocks against 6144 cycles of MFMA work (96.6 %
// issue efficiency); the shader clock itself sits at 2.0-2.2 GHz under this kernel
// with N(0,1) operands and at 2.25-2.35 GHz with all-zero operands, i.e. the chip's
// power management, not the instruction stream, sets the distance to the 2.4 GHz peak.
#include <algorithm>
#include <mutex>
#include <type_traits>
#include <unordered_set>

#include "common.hpp"

namespace g2 {

constexpr int BK = 32;           // floats per K slab
constexpr int CHUNKS = BK / 4;   // 16-byte chunks per slab row

// Workgroup -> tile.  Hardware deals consecutive workgroup ids round-robin to
// the 8 XCDs (each with a private L2).  When the number of row tiles divides by
// 8, XCD x is given the band of row tiles [x*band, (x+1)*band) and walks it
// column tile by column tile, so that the band's A rows stay in that XCD's L2
// and each B column tile is fetched once per XCD.  When the product is wider than
// it is tall (short prompts: B*T < OC) and the column tiles divide by 8, the bands
// are bands of column tiles instead: every XCD then reads an eighth of the weights
// and all of the (smaller) activations, not all of the weights.
template <int BM, int BN>
__device__ __forceinline__ void tile_of_block(int pid, int ntm, int ntn, int& tm, int& tn) {
  if ((ntn & 7) == 0 && (long long)ntn * BN > (long long)ntm * BM) {
    const int band = ntn >> 3;
    const int xcd = pid & 7;
    const int q = pid >> 3;
    tn = xcd * band + q % band;
    tm = q / band;
  } else if ((ntm & 7) == 0) {
    const int band = ntm >> 3;
    const int xcd = pid & 7;
    const int q = pid >> 3;
    tm = xcd * band + q % band;
    tn = q / band;
  } else {
    tm = pid % ntm;
    tn = pid / ntm;
  }
}

// Argmax over the 32 lanes of a half-wave for N rows at once: bv[e] / bx[e] are this
// lane's (value, column) candidates for rows e = 0..N-1, the same rows in every lane.
// Butterfly over lane bits 4..0 (OFF = 16..1).  While a lane still holds more rows than
// the exchange distance, partners split the rows between them (each keeps one half of
// the list and hands the other half over), so the work halves at every step and, for
// N = 32, lane l ends up with the finished pair of row l alone; 32 lanes reducing every
// row five times would cost five times the cross-lane traffic.  On return the lane holds
// max(N / 32, 1) rows starting at row `first`; lanes with writer == false hold duplicates.
template <int N, int OFF>
__device__ __forceinline__ void argmax_fold(float* bv, int* bx, int lane, int& first,
                                            bool& writer) {
  if constexpr (OFF >= 1) {
    const bool up = (lane & OFF) != 0;
    if constexpr (N > OFF) {
      constexpr int HN = N / 2;
#pragma unroll
      for (int e = 0; e < HN; e++) {
        float kv = up ? bv[e + HN] : bv[e];
        int ki = up ? bx[e + HN] : bx[e];
        const float sv = up ? bv[e] : bv[e + HN];
        const int si = up ? bx[e] : bx[e + HN];
        argmax_combine(kv, ki, __shfl_xor(sv, OFF, 64), __shfl_xor(si, OFF, 64));
        bv[e] = kv;
        bx[e] = ki;
      }
      first += up ? HN : 0;
      argmax_fold<HN, OFF / 2>(bv, bx, lane, first, writer);
    } else {
#pragma unroll
      for (int e = 0; e < N; e++)
        argmax_combine(bv[e], bx[e], __shfl_xor(bv[e], OFF, 64), __shfl_xor(bx[e], OFF, 64));
      writer = writer && !up;
      argmax_fold<N, OFF / 2>(bv, bx, lane, first, writer);
    }
  }
}

// The epilogue the tiled kernels share: a wave's TM x TN accumulator tiles go to out (through
// GELU if asked), plus resid's entries of the same positions where resid is given (the residual
// add of a transformer block, which then needs no pass of its own over memory: out = resid +
// act(product); out and resid must not overlap).  row0 / col0: this lane's first row and its
// column in the wave's first tile; ldo: floats from one row of out (and of resid) to the next,
// N unless the launch computes a range of the columns of a wider product.  All of a wave's loads
// of resid are issued before its first store.
// (a full tile's entries of resid, in the accumulators' layout)
template <int TM, int TN>
__device__ __forceinline__ void load_resid_tile(f32x16 (&rs)[TM][TN], const float* __restrict__ resid,
                                                int row0, int col0, int ldo) {
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const float* const rp = resid + (size_t)(row0 + i * 32) * ldo + col0 + j * 32;
#pragma unroll
      for (int v = 0; v < 16; v++) rs[i][j][v] = rp[(size_t)(8 * (v >> 2) + (v & 3)) * ldo];
    }
}
// (a full tile: out = act(acc) + rs)
template <int TM, int TN, bool GELU>
__device__ __forceinline__ void store_tile_sum(const f32x16 (&acc)[TM][TN], const f32x16 (&rs)[TM][TN],
                                               float* __restrict__ out, int row0, int col0, int ldo) {
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
      float* const o = out + (size_t)(row0 + i * 32) * ldo + col0 + j * 32;
#pragma unroll
      for (int v = 0; v < 16; v++) {
        float r = acc[i][j][v];
        if (GELU) r = gelu_tanh(r);
        o[(size_t)(8 * (v >> 2) + (v & 3)) * ldo] = r + rs[i][j][v];
      }
    }
}
template <int TM, int TN, bool GELU>
__device__ __forceinline__ void store_tile(const f32x16 (&acc)[TM][TN], float* __restrict__ out,
                                           const float* __restrict__ resid, int row0, int col0, int M,
                                           int N, int ldo, bool full) {
  if (full && resid != nullptr) {
    f32x16 rs[TM][TN];
    load_resid_tile<TM, TN>(rs, resid, row0, col0, ldo);
    store_tile_sum<TM, TN, GELU>(acc, rs, out, row0, col0, ldo);
    return;
  }
#pragma unroll
  for (int i = 0; i < TM; i++) {
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int col = col0 + j * 32;
      const int rbase = row0 + i * 32;
      float* o = out + (size_t)rbase * ldo + col;
      if (full) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
          float r = acc[i][j][v];
          if (GELU) r = gelu_tanh(r);
          o[(size_t)(8 * (v >> 2) + (v & 3)) * ldo] = r;
        }
      } else if (col < N) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int row = rbase + 8 * (v >> 2) + (v & 3);
          if (row < M) {
            float r = acc[i][j][v];
            if (GELU) r = gelu_tanh(r);
            if (resid != nullptr) r += resid[(size_t)row * ldo + col];
            out[(size_t)row * ldo + col] = r;
          }
        }
      }
    }
  }
}

// K split between workgroups.  The `splits` workgroups of a tile each multiply one
// contiguous range of the K slabs and leave their partial tile (the raw accumulators, lane
// by lane: [tile][part][wave][register quad][lane], 1 KB per store instruction) in a
// workspace; whichever of them finishes last -- a per-tile counter tells it, nobody ever
// waits -- reads all the parts back IN PART ORDER into its accumulators and runs the
// ordinary epilogue, so the result does not depend on which workgroup that was.  The
// partial tiles cross XCDs: they are stored and loaded with the cache-bypassing policy,
// each wave waits for its stores to be acknowledged before the workgroup counts itself
// in, and the last one resets the counter for the next launch.
// Returns false in the workgroups that are done (everyone but the tile's last one).
template <int NW, int TM, int TN>
__device__ __forceinline__ bool splitk_combine(f32x16 (&acc)[TM][TN], float* __restrict__ part_ws,
                                               unsigned* __restrict__ part_cnt, int tile_id, int part,
                                               int splits, int slot, bool holds, int lane, int tid,
                                               int* lds_flag) {
  constexpr int ACC4 = TM * TN * 4;             // register quads per lane
  constexpr int PART_FLOATS = NW * ACC4 * 256;  // one partial tile
  const Bypass ws(part_ws + (size_t)tile_id * splits * PART_FLOATS, (size_t)splits * PART_FLOATS);
  if (holds) {
    const int mine = (part * NW + slot) * (ACC4 * 256) + lane * 4;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int u = 0; u < 4; u++) {
          const f32x4 q = {acc[i][j][4 * u], acc[i][j][4 * u + 1], acc[i][j][4 * u + 2],
                           acc[i][j][4 * u + 3]};
          ws.store4(mine + ((i * TN + j) * 4 + u) * 256, q);
        }
  }
  wait_vm();
  __syncthreads();
  if (tid == 0) {
    const unsigned old =
        __hip_atomic_fetch_add(part_cnt + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool last = old + 1u == (unsigned)splits;
    if (last) __hip_atomic_store(part_cnt + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *lds_flag = last ? 1 : 0;
  }
  __syncthreads();
  if (*lds_flag == 0 || !holds) return false;
  // Four parts at a time, all their loads independent of each other so that as many are in
  // flight as the registers allow; a part past the last one lies beyond the end of the
  // buffer descriptor and reads as zeros without touching memory.
  for (int p0 = 0; p0 < splits; p0 += 4) {
    f32x4 t[4][ACC4];
#pragma unroll
    for (int pp = 0; pp < 4; pp++) {
      const int theirs = ((p0 + pp) * NW + slot) * (ACC4 * 256) + lane * 4;
#pragma unroll
      for (int q = 0; q < ACC4; q++) t[pp][q] = ws.load4(theirs + q * 256);
    }
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int q = (i * TN + j) * 4 + (v >> 2);
          float x = p0 == 0 ? t[0][q][v & 3] : acc[i][j][v] + t[0][q][v & 3];
#pragma unroll
          for (int pp = 1; pp < 4; pp++) x += t[pp][q][v & 3];
          acc[i][j][v] = x;
        }
  }
  return true;
}

template <int BM, int BN, int WGM, int WGN, bool GELU, bool KTAIL>
__global__ __launch_bounds__(WGM* WGN* kWave) void matmul_mfma_kernel(
    float* __restrict__ out, const float* __restrict__ inp, const float* __restrict__ weight,
    const float* __restrict__ bias, const float* __restrict__ resid, int M, int K, int N, int ldo, int ntm,
    int ntn) {
  constexpr int NT = WGM * WGN * kWave;
  constexpr int WM = BM / WGM, WN = BN / WGN;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int A_PER = BM * CHUNKS / NT, B_PER = BN * CHUNKS / NT;
  static_assert(BM * CHUNKS % NT == 0 && BN * CHUNKS % NT == 0, "tile/threads mismatch");
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be 32x32 MFMA tiles");
  constexpr int STAGE = (BM + BN) * CHUNKS;  // f32x4 per LDS buffer

  extern __shared__ f32x4 lds[];  // [2][STAGE]: A rows then B rows

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;

  int tm, tn;
  tile_of_block<BM, BN>(blockIdx.x, ntm, ntn, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  // ---- global -> register staging --------------------------------------
  // chunk q = tid + j*NT of the slab: row q/8, chunk q%8.  Rows past the end of the
  // matrix are clamped to its last row: they produce accumulator rows / columns
  // that the epilogue never stores, so M and N edges need no masking.  Only a K
  // tail (K % 32 != 0, KTAIL) must contribute zeros; that fill is applied when
  // the registers are stored to LDS, a slab after the loads were issued.
  const float* a_src[A_PER];
  const float* b_src[B_PER];
  int a_dst[A_PER], b_dst[B_PER];
  const int kc = (tid & 7) * 4;  // this thread's k offset inside a slab (same for all j)
#pragma unroll
  for (int j = 0; j < A_PER; j++) {
    const int q = tid + j * NT;
    const int r = q >> 3, c = q & 7;
    a_src[j] = inp + (size_t)min(m0 + r, M - 1) * K;
    a_dst[j] = r * CHUNKS + (c ^ (r & 7));
  }
#pragma unroll
  for (int j = 0; j < B_PER; j++) {
    const int q = tid + j * NT;
    const int r = q >> 3, c = q & 7;
    b_src[j] = weight + (size_t)min(n0 + r, N - 1) * K;
    b_dst[j] = BM * CHUNKS + r * CHUNKS + (c ^ (r & 7));
  }

  f32x4 a_reg[A_PER], b_reg[B_PER];
  bool reg_kin = true;  // whether the chunk held in the registers lies inside K
  auto fetch = [&](int k0) {
    reg_kin = (k0 + kc) < K;  // K is a multiple of 4: a chunk is all in or all out
    const int ko = reg_kin ? k0 + kc : 0;  // past the end: re-read a valid address
#pragma unroll
    for (int j = 0; j < A_PER; j++) a_reg[j] = *reinterpret_cast<const f32x4*>(a_src[j] + ko);
#pragma unroll
    for (int j = 0; j < B_PER; j++) b_reg[j] = *reinterpret_cast<const f32x4*>(b_src[j] + ko);
  };
  auto stash = [&](f32x4* s) {
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < A_PER; j++) s[a_dst[j]] = (!KTAIL || reg_kin) ? a_reg[j] : zero;
#pragma unroll
    for (int j = 0; j < B_PER; j++) s[b_dst[j]] = (!KTAIL || reg_kin) ? b_reg[j] : zero;
  };

  // ---- accumulators, initialised with the bias of the lane's column ----
  f32x16 acc[TM][TN];
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int col = n0 + wn * WN + j * 32 + (lane & 31);
    const float bv = (bias != nullptr && col < N) ? bias[col] : 0.f;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = bv;
  }

  // ---- operand read offsets (f32x4 units) inside an LDS buffer ----------
  // row & 7 == lane & 7 because every row base is a multiple of 32.
  const int h = lane >> 5;
  const int sw = lane & 7;
  int a_row[TM], b_row[TN];
#pragma unroll
  for (int i = 0; i < TM; i++) a_row[i] = (wm * WM + i * 32 + (lane & 31)) * CHUNKS;
#pragma unroll
  for (int j = 0; j < TN; j++) b_row[j] = BM * CHUNKS + (wn * WN + j * 32 + (lane & 31)) * CHUNKS;

  // Operands of k-group g (k = 8g .. 8g+7 of the slab) into register set p.
  f32x4 af[2][TM], bf[2][TN];
  auto read_ops = [&](const f32x4* buf, int g, int p) {
#pragma unroll
    for (int i = 0; i < TM; i++) af[p][i] = buf[a_row[i] + ((2 * g + h) ^ sw)];
#pragma unroll
    for (int j = 0; j < TN; j++) bf[p][j] = buf[b_row[j] + ((2 * g + h) ^ sw)];
  };
  auto mfma_group = [&](int p) {
#pragma unroll
    for (int e = 0; e < 4; e++)
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
          acc[i][j] =
              __builtin_amdgcn_mfma_f32_32x32x2f32(af[p][i][e], bf[p][j][e], acc[i][j], 0, 0, 0);
  };
  // Scheduling groups: an MFMA occupies the matrix pipe for 64 cycles but issues in a
  // few, so every LDS / global / VALU instruction of the loop is placed in the shadow
  // of an MFMA instead of between two bursts of them.
#define G2_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
#define G2_MFMA 0x008
#define G2_VMEM_RD 0x020
#define G2_DS_RD 0x100
#define G2_DS_WR 0x200

  // Software pipeline over slabs s = 0 .. nslab-1 (two LDS buffers, cur / nxt).  The
  // body is branch-free: past the last slab it stores zeros to the idle buffer and
  // re-reads a valid address, which nobody consumes.
  //   group 0: MFMAs of group 0, reading group 1's operands
  //   group 1: MFMAs of group 1, reading group 2's operands
  //   group 2: MFMAs of group 2, reading group 3's operands and storing the
  //            prefetched slab s+1 into nxt (whose last reads completed before the
  //            previous barrier)
  //            BARRIER (all cur reads complete; all nxt stores visible)
  //   group 3: MFMAs of group 3, reading group 0 of slab s+1 from nxt and issuing
  //            the global loads of slab s+2
  // so the store->barrier->read chain never sits between two MFMAs with nothing to
  // cover it, and global loads have a full slab of MFMA time to land.
  const int nslab = (K + BK - 1) / BK;
  fetch(0);
  stash(lds);
  fetch(BK);
  __syncthreads();
  read_ops(lds, 0, 0);

  for (int s = 0; s < nslab; s++) {
    const f32x4* cur = lds + (s & 1) * STAGE;
    f32x4* nxt = lds + ((s + 1) & 1) * STAGE;

    read_ops(cur, 1, 1);
    mfma_group(0);
    read_ops(cur, 2, 0);
    mfma_group(1);
    read_ops(cur, 3, 1);
    stash(nxt);
    mfma_group(0);
#pragma unroll
    for (int g = 0; g < 2; g++) {
#pragma unroll
      for (int i = 0; i < TM + TN; i++) {
        G2_SGB(G2_MFMA, 1);
        G2_SGB(G2_DS_RD, 1);
      }
      G2_SGB(G2_MFMA, 4 * TM * TN - (TM + TN));
    }
#pragma unroll
    for (int i = 0; i < TM + TN; i++) {
      G2_SGB(G2_MFMA, 1);
      G2_SGB(G2_DS_RD, 1);
    }
#pragma unroll
    for (int i = 0; i < A_PER + B_PER; i++) {
      G2_SGB(G2_MFMA, 1);
      G2_SGB(G2_DS_WR, 1);
    }
    G2_SGB(G2_MFMA, 4 * TM * TN - (TM + TN) - (A_PER + B_PER));

    __syncthreads();

    read_ops(nxt, 0, 0);
    fetch((s + 2) * BK);
    mfma_group(1);
#pragma unroll
    for (int i = 0; i < TM + TN; i++) {
      G2_SGB(G2_MFMA, 1);
      G2_SGB(G2_DS_RD, 1);
    }
#pragma unroll
    for (int i = 0; i < A_PER + B_PER; i++) {
      G2_SGB(G2_MFMA, 1);
      G2_SGB(G2_VMEM_RD, 1);
    }
    G2_SGB(G2_MFMA, 4 * TM * TN - (TM + TN) - (A_PER + B_PER));
  }
#undef G2_SGB

  // ---- epilogue -----------------------------------------------------------
  const bool full = (m0 + BM <= M) && (n0 + BN <= N);
  store_tile<TM, TN, GELU>(acc, out, resid, m0 + wm * WM + 4 * h, n0 + wn * WN + (lane & 31), M, N, ldo, full);
}

// ---------------------------------------------------------------------------
// Main kernel for K % 32 == 0 (every GPT-2 shape): same tiling, LDS layout and
// MFMA mapping as above, but the K slabs go from global memory straight into LDS
// with global_load_lds_dwordx4 (no staging registers, no ds_write, no per-slab
// address arithmetic), and a wave owns a larger register tile so that fewer LDS
// reads are needed per MFMA.  On this chip every non-MFMA instruction a SIMD
// issues takes issue cycles away from the matrix pipe (measured: ~4 cycles per
// VALU or ds_read, more per ds_write / global load), so the loop is built to
// contain almost nothing but MFMAs: per wave and slab 24*TM*TN/... MFMAs,
// 4*(TM+TN) ds_read_b128, (BM+BN)/8/waves LDS-DMA loads and 2*4 address updates.
//
// An LDS-DMA load writes lane l's 16 bytes to LDS address M0 + 16*l, i.e. one
// instruction fills 8 consecutive 128-byte rows of a buffer.  The XOR chunk
// swizzle is therefore applied on the global side: lane l (row l/8 of the group,
// chunk position l%8) fetches logical chunk (l%8) ^ (l/8) of its row.
typedef __attribute__((address_space(3))) void lds_void_t;
typedef const __attribute__((address_space(1))) void glb_void_t;

// PROBE instantiations additionally record, per workgroup, the wall clock (100 MHz) and
// the shader clock at the start and end of the slab loop: {wall0, wall1, clk0, clk1}
// in probe[4*workgroup ..].  They tell MFMA issue efficiency (shader clocks per slab
// against the 64 cycles per MFMA) apart from the clock frequency the chip sustains.
//
// ARGMAX: instead of storing the tile, every wave reduces its part of each output row to
// one (largest value, its column) pair and stores that in out[row][tn * WGN + wn] (the
// value) and arg_idx[row][tn * WGN + wn] (the column): ntn * WGN pairs per row, which
// argmax_pairs_kernel reduces.  The (M, N) product itself never reaches memory.
//
// SPLIT: the grid is `splits` workgroups per tile (workgroup id = part * tiles + tile), each
// taking slabs [part * nslab / splits, (part + 1) * nslab / splits); see splitk_combine.
//
// RESID: out = resid + product for a product whose tiles come in about one round (every compute
// unit reaches its epilogue at the same moment, and B*T x OC floats of resid read there in one
// burst cost 4-5 us that nothing hides).  Each wave fetches its part of the tile of resid into
// registers during the slab loop instead, wave w two slabs earlier than wave w - 1, so that the
// reads are spread over the loop's last slabs and are long there when the epilogue starts.
template <int BM, int BN, int WGM, int WGN, bool GELU, bool PROBE = false, bool ARGMAX = false,
          bool SPLIT = false, bool RESID = false>
__global__ __launch_bounds__(WGM* WGN* kWave) void matmul_dma_kernel(
    float* __restrict__ out, const float* __restrict__ inp, const float* __restrict__ weight,
    const float* __restrict__ bias, const float* __restrict__ resid, int M, int K, int N, int ldo, int ntm,
    int ntn, unsigned long long* __restrict__ probe, int* __restrict__ arg_idx, float* __restrict__ part_ws,
    unsigned* __restrict__ part_cnt, int splits) {
  constexpr int NW = WGM * WGN;
  constexpr int WM = BM / WGM, WN = BN / WGN;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int GROUPS = (BM + BN) / 8;  // 8-row groups per buffer, one DMA each
  constexpr int DMA_PER = GROUPS / NW;   // DMAs per wave and slab
  static_assert(GROUPS % NW == 0 && BM % 8 == 0, "tile/waves mismatch");
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be 32x32 MFMA tiles");
  constexpr int STAGE = (BM + BN) * CHUNKS;  // f32x4 per LDS buffer
  constexpr int STAGE_BYTES = STAGE * 16;
  constexpr int MFMAS = 4 * TM * TN;  // per k-group of 8

  extern __shared__ f32x4 lds[];  // [2][STAGE]: A rows then B rows
  char* const lds_bytes = reinterpret_cast<char*>(lds);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;

  int pid = blockIdx.x, part = 0;
  if (SPLIT) {
    part = pid / (ntm * ntn);
    pid -= part * (ntm * ntn);
  }
  int tm, tn;
  tile_of_block<BM, BN>(pid, ntm, ntn, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  // this workgroup's slabs: all of K, or its part of it
  const int slab_lo = SPLIT ? (int)((long long)part * (K / BK) / splits) : 0;
  const int nslab = SPLIT ? (int)((long long)(part + 1) * (K / BK) / splits) - slab_lo : K / BK;

  // ---- LDS-DMA descriptors -------------------------------------------------
  // One DMA fills a group of 8 rows of a buffer.  Each wave owns A_PER groups of the A
  // rows and B_PER groups of the B rows.  Rows past the end of a matrix are clamped to
  // its last row: they only feed accumulator rows / columns that the epilogue does not
  // store.  An address is a wave-uniform 64-bit base (the tile's first row of A or of
  // B, moved on by one slab per iteration with scalar adds) plus a fixed 32-bit
  // per-lane byte offset, so the loop spends no vector instructions on addressing.
  constexpr int A_PER = BM / 8 / NW, B_PER = BN / 8 / NW;
  static_assert(BM / 8 % NW == 0 && BN / 8 % NW == 0, "tile/waves mismatch");
  const char* const a_tile = reinterpret_cast<const char*>(inp + (size_t)m0 * K + (size_t)slab_lo * BK);
  const char* const b_tile = reinterpret_cast<const char*>(weight + (size_t)n0 * K + (size_t)slab_lo * BK);
  unsigned dma_off[DMA_PER];
  int dma_group[DMA_PER];  // wave-uniform: which 8-row group of the buffer
  {
    const int rr = lane >> 3, c = (lane & 7) ^ rr;
#pragma unroll
    for (int j = 0; j < DMA_PER; j++) {
      if (j < A_PER) {
        dma_group[j] = wave * A_PER + j;
        const int row = 8 * dma_group[j] + rr;
        dma_off[j] = (unsigned)((min(m0 + row, M - 1) - m0) * K + c * 4) * 4u;
      } else {
        dma_group[j] = BM / 8 + wave * B_PER + (j - A_PER);
        const int row = 8 * (dma_group[j] - BM / 8) + rr;
        dma_off[j] = (unsigned)((min(n0 + row, N - 1) - n0) * K + c * 4) * 4u;
      }
    }
  }
  auto dma_slab = [&](int slab, int buf) {
    const size_t kbytes = (size_t)min(slab, nslab - 1) * (BK * 4);  // past the end: reload
    const char* a_k = a_tile + kbytes;
    const char* b_k = b_tile + kbytes;
    // Opaque to the optimiser, so that "scalar base + 32-bit lane offset" reaches the
    // instruction selector intact (it is the scalar-base addressing form of the load)
    // instead of being re-associated into a 64-bit vector add per load.
    asm volatile("" : "+s"(a_k), "+s"(b_k));
#pragma unroll
    for (int j = 0; j < DMA_PER; j++)
      __builtin_amdgcn_global_load_lds(
          (glb_void_t*)((j < A_PER ? a_k : b_k) + dma_off[j]),
          (lds_void_t*)(lds_bytes + buf * STAGE_BYTES + dma_group[j] * 1024), 16, 0, 0);
  };
  // the first two slabs are on their way before anything else is set up
  dma_slab(0, 0);
  dma_slab(1, 1);

  // ---- accumulators, initialised with the bias of the lane's column (in the part that
  // takes the first slabs, when K is split) ----
  f32x16 acc[TM][TN];
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int col = n0 + wn * WN + j * 32 + (lane & 31);
    const float bv = (bias != nullptr && col < N && part == 0) ? bias[col] : 0.f;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = bv;
  }

  // ---- operand read addresses (bytes) inside buffer 0: one per k-group for A and
  // for B.  The other buffer and the wave's further 32-row tiles are immediate
  // offsets of the read instruction. ----
  const int h = lane >> 5;
  const int sw = lane & 7;
  int a_addr[4], b_addr[4];
#pragma unroll
  for (int g = 0; g < 4; g++) {
    a_addr[g] = ((wm * WM + (lane & 31)) * CHUNKS + ((2 * g + h) ^ sw)) * 16;
    b_addr[g] = (BM * CHUNKS + (wn * WN + (lane & 31)) * CHUNKS + ((2 * g + h) ^ sw)) * 16;
  }
  f32x4 af[2][TM], bf[2][TN];
  auto read_ops = [&](int g, int p, int buf) {
#pragma unroll
    for (int i = 0; i < TM; i++)
      af[p][i] = *reinterpret_cast<const f32x4*>(lds_bytes + a_addr[g] +
                                                 (buf * STAGE_BYTES + i * (32 * BK * 4)));
#pragma unroll
    for (int j = 0; j < TN; j++)
      bf[p][j] = *reinterpret_cast<const f32x4*>(lds_bytes + b_addr[g] +
                                                 (buf * STAGE_BYTES + j * (32 * BK * 4)));
  };
  auto mfma_group = [&](int p) {
#pragma unroll
    for (int e = 0; e < 4; e++)
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
          acc[i][j] =
              __builtin_amdgcn_mfma_f32_32x32x2f32(af[p][i][e], bf[p][j][e], acc[i][j], 0, 0, 0);
  };
#define G2_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
#define G2_READS_IN_SHADOW()           \
  _Pragma("unroll") for (int i_ = 0; i_ < TM + TN; i_++) { \
    G2_SGB(0x008, 1);                  \
    G2_SGB(0x100, 1);                  \
  }

  // Pipeline (two buffers; slab s lives in buffer s & 1):
  //   groups 0..2 of slab s: MFMAs, each group reading the next group's operands
  //   wait for this wave's DMAs of slab s+1, BARRIER: every wave's reads of slab s
  //     are complete and every wave's DMAs of slab s+1 have landed
  //   group 3: MFMAs, reading group 0 of slab s+1 and issuing the DMAs of slab s+2
  //     into the buffer slab s just vacated
  // The slab loop is unrolled by two so that the buffer is a compile-time constant.
  auto slab_body = [&](int s, auto buf_tag) {
    constexpr int buf = decltype(buf_tag)::value;
    read_ops(1, 1, buf);
    mfma_group(0);
    read_ops(2, 0, buf);
    mfma_group(1);
    read_ops(3, 1, buf);
    mfma_group(0);
#pragma unroll
    for (int g = 0; g < 3; g++) {
      G2_READS_IN_SHADOW();
      G2_SGB(0x008, MFMAS - (TM + TN));
    }

    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): my DMAs of slab s+1 have landed
    __syncthreads();

    read_ops(0, 0, buf ^ 1);
    dma_slab(s + 2, buf);
    mfma_group(1);
    G2_READS_IN_SHADOW();
#pragma unroll
    for (int i = 0; i < DMA_PER; i++) {
      G2_SGB(0x008, 1);
      G2_SGB(0x020, 1);
    }
    G2_SGB(0x008, MFMAS - (TM + TN) - DMA_PER);
  };
  __builtin_amdgcn_s_waitcnt(0x0F70 | DMA_PER);  // vmcnt(DMA_PER): slab 0 has landed
  __syncthreads();
  read_ops(0, 0, 0);
  unsigned long long wall0 = 0, clk0 = 0;
  if (PROBE) {
    wall0 = wall_clock64();
    clk0 = clock64();
  }
  // RESID: this wave's entries of resid (full tiles; an edge tile reads them in the epilogue)
  const bool full = (m0 + BM <= M) && (n0 + BN <= N);
  const int row0 = m0 + wm * WM + 4 * (lane >> 5), col0 = n0 + wn * WN + (lane & 31);
  f32x16 rs[RESID ? TM : 1][RESID ? TN : 1];
  const int resid_at = RESID && full ? max(0, nslab / 2 - 1 - wave) : -1;  // pair of slabs to fetch in front of
  bool resid_loaded = false;
  int s = 0;
  // (RESID: the last NW pairs of slabs run in a second copy of the loop, which is the one that
  // carries the check for the wave's turn to fetch; the check in the loop itself cost every
  // pair of slabs 70 ns)
  const int s_check = RESID ? max(0, nslab / 2 - NW) * 2 : nslab;
  for (; s + 1 < min(nslab, s_check); s += 2) {
    slab_body(s, std::integral_constant<int, 0>{});
    slab_body(s + 1, std::integral_constant<int, 1>{});
  }
  if constexpr (RESID) {
    for (; s + 1 < nslab; s += 2) {
      if ((s >> 1) == resid_at) {
        load_resid_tile<TM, TN>(rs, resid, row0, col0, ldo);
        resid_loaded = true;
      }
      slab_body(s, std::integral_constant<int, 0>{});
      slab_body(s + 1, std::integral_constant<int, 1>{});
    }
  }
  if (s < nslab) slab_body(s, std::integral_constant<int, 0>{});
  if constexpr (RESID) {
    if (full && !resid_loaded) load_resid_tile<TM, TN>(rs, resid, row0, col0, ldo);
  }
  if (PROBE && tid == 0) {
    probe[4 * blockIdx.x + 0] = wall0;
    probe[4 * blockIdx.x + 1] = wall_clock64();
    probe[4 * blockIdx.x + 2] = clk0;
    probe[4 * blockIdx.x + 3] = clock64();
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // drain the (unused) DMAs before the LDS is released
#undef G2_SGB
#undef G2_READS_IN_SHADOW

  if constexpr (SPLIT) {
    __syncthreads();  // every wave has finished with the LDS buffers: word 0 becomes the flag
    if (!splitk_combine<NW, TM, TN>(acc, part_ws, part_cnt, pid, part, splits, wave, true, lane, tid,
                                    reinterpret_cast<int*>(lds_bytes)))
      return;
  }

  // ---- epilogue -----------------------------------------------------------
  if (ARGMAX) {
    const size_t pairs = (size_t)ntn * WGN;
    const size_t slot = (size_t)tn * WGN + wn;
    // This lane's best over its own columns, for each of its R rows (ascending columns:
    // a strict > keeps the first maximum).
    constexpr int R = TM * 16;
    float bv[R];
    int bx[R];
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int v = 0; v < 16; v++) {
        float best = -INFINITY;
        int bi = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < TN; j++) {
          const int col = n0 + wn * WN + j * 32 + (lane & 31);
          const float a = acc[i][j][v];
          const bool take = (col < N) & (a > best);
          best = take ? a : best;
          bi = take ? col : bi;
        }
        bv[i * 16 + v] = best;
        bx[i * 16 + v] = bi;
      }
    }
    int first = 0;
    bool writer = true;
    argmax_fold<R, 16>(bv, bx, lane, first, writer);
    constexpr int n = R > 32 ? R / 32 : 1;  // rows a lane ends up with
#pragma unroll
    for (int e = 0; e < n; e++) {
      const int r = first + e;  // index i * 16 + v of the row this lane finished
      const int row = m0 + wm * WM + (r >> 4) * 32 + 4 * h + 8 * ((r & 15) >> 2) + (r & 3);
      if (writer && row < M) {
        out[(size_t)row * pairs + slot] = bv[e];
        arg_idx[(size_t)row * pairs + slot] = bx[e];
      }
    }
    return;
  }
  if constexpr (RESID) {
    if (full) {
      store_tile_sum<TM, TN, GELU>(acc, rs, out, row0, col0, ldo);
      return;
    }
  }
  // A product larger than the 256 MiB Infinity Cache (the logits) will not be read back
  // from any cache: its tiles are stored with streaming stores, so that they do not push
  // the operands that other tiles are about to re-read out of L2.
  const bool stream_out = (size_t)M * ldo * sizeof(float) > ((size_t)256 << 20);
  if (full && stream_out && resid == nullptr) {
    // Row by row: the wave's TN segments of 128 bytes of one row go out back to back, as one run
    // of TN * 128 bytes.  Rows of such a product (N = 50257) start at any multiple of 4 bytes, so
    // every segment straddles memory lines; segments of one row that reach the L2 together are
    // merged there, and only the two ends of the run are left as partial lines.
#pragma unroll
    for (int i = 0; i < TM; i++) {
      float* const o = out + (size_t)(m0 + wm * WM + i * 32 + 4 * h) * ldo + n0 + wn * WN + (lane & 31);
#pragma unroll
      for (int v = 0; v < 16; v++) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
          float r = acc[i][j][v];
          if (GELU) r = gelu_tanh(r);
          __builtin_nontemporal_store(r, o + (size_t)(8 * (v >> 2) + (v & 3)) * ldo + j * 32);
        }
      }
    }
    return;
  }
  store_tile<TM, TN, GELU>(acc, out, resid, row0, col0, M, N, ldo, full);
}

// s_waitcnt immediate that waits until at most n vector-memory operations of this wave
// are outstanding and waits for nothing else (vmcnt is split over bits 3:0 and 15:14).
constexpr int vmcnt_only(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }

// Small problems (few output tiles): same LDS layout, DMA fill and MFMA mapping as
// matmul_dma_kernel, organised for latency instead of issue rate.  With one small tile
// per CU there is too little MFMA work per slab to cover a memory round trip, so the
// slabs go through a ring of NBUF buffers with NBUF-1 fills in flight, and the waves of
// a workgroup can also split K (KS): wave set ks takes k-groups ks*4/KS .. of every
// slab, so a 32x32 tile still keeps all four SIMDs of its CU busy.  The partial
// accumulators are summed through LDS in a fixed order (ks = 0, 1, ...), so results do
// not depend on timing.
// SPLIT: K is also split between `splits` workgroups per tile, as in matmul_dma_kernel.
// PIPE: the slab loop is software-pipelined (see below); otherwise a slab is read and
// multiplied after its barrier.  Measured per shape over B*T = 64 .. 8192: the pipelined loop
// is 3-11 % faster for 64x96 tiles (whose waves have two k-groups of 12 MFMAs per slab to
// hide reads under) and up to 35 % SLOWER for 32x32 tiles with few slabs' worth of work per
// wave, where what counts is how far ahead the fills run: waiting for slab s + 1 before
// slab s is multiplied costs a slab of lead.
template <int BM, int BN, int WGM, int WGN, int KS, int NBUF, bool GELU, bool SPLIT = false,
          bool PIPE = false>
__global__ __launch_bounds__(WGM* WGN* KS* kWave) void matmul_ring_kernel(
    float* __restrict__ out, const float* __restrict__ inp, const float* __restrict__ weight,
    const float* __restrict__ bias, const float* __restrict__ resid, int M, int K, int N, int ldo, int ntm,
    int ntn, float* __restrict__ part_ws, unsigned* __restrict__ part_cnt, int splits) {
  constexpr int NMN = WGM * WGN;
  constexpr int NW = NMN * KS;
  constexpr int WM = BM / WGM, WN = BN / WGN;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int A_PER = BM / 8 / NW, B_PER = BN / 8 / NW;
  constexpr int DMA_PER = A_PER + B_PER;
  constexpr int GPW = 4 / KS;  // k-groups of a slab per wave
  static_assert(BM / 8 % NW == 0 && BN / 8 % NW == 0, "tile/waves mismatch");
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be 32x32 MFMA tiles");
  static_assert(KS == 1 || KS == 2 || KS == 4, "K split must divide the 4 k-groups");
  static_assert(NBUF >= 2 && NBUF * DMA_PER < 64, "vmcnt is a 6-bit counter");
  constexpr int STAGE_BYTES = (BM + BN) * CHUNKS * 16;
  static_assert((KS - 1) * NMN * TM * TN * 16 * 64 * 4 <= NBUF * STAGE_BYTES,
                "the K-split reduction reuses the ring's LDS");

  extern __shared__ f32x4 lds[];  // [NBUF][(BM + BN) * CHUNKS]: A rows then B rows
  char* const lds_bytes = reinterpret_cast<char*>(lds);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ks = wave / NMN, wmn = wave % NMN;
  const int wm = wmn / WGN, wn = wmn % WGN;

  int pid = blockIdx.x, part = 0;
  if (SPLIT) {
    part = pid / (ntm * ntn);
    pid -= part * (ntm * ntn);
  }
  int tm, tn;
  tile_of_block<BM, BN>(pid, ntm, ntn, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int slab_lo = SPLIT ? (int)((long long)part * (K / BK) / splits) : 0;
  const int nslab = SPLIT ? (int)((long long)(part + 1) * (K / BK) / splits) - slab_lo : K / BK;

  // LDS-DMA descriptors, as in matmul_dma_kernel
  const char* const a_tile = reinterpret_cast<const char*>(inp + (size_t)m0 * K + (size_t)slab_lo * BK);
  const char* const b_tile = reinterpret_cast<const char*>(weight + (size_t)n0 * K + (size_t)slab_lo * BK);
  unsigned dma_off[DMA_PER];
  int dma_group[DMA_PER];
  {
    const int rr = lane >> 3, c = (lane & 7) ^ rr;
#pragma unroll
    for (int j = 0; j < DMA_PER; j++) {
      if (j < A_PER) {
        dma_group[j] = wave * A_PER + j;
        const int row = 8 * dma_group[j] + rr;
        dma_off[j] = (unsigned)((min(m0 + row, M - 1) - m0) * K + c * 4) * 4u;
      } else {
        dma_group[j] = BM / 8 + wave * B_PER + (j - A_PER);
        const int row = 8 * (dma_group[j] - BM / 8) + rr;
        dma_off[j] = (unsigned)((min(n0 + row, N - 1) - n0) * K + c * 4) * 4u;
      }
    }
  }
  auto dma_slab = [&](int slab, int buf) {
    const size_t kbytes = (size_t)min(slab, nslab - 1) * (BK * 4);  // past the end: reload
    const char* a_k = a_tile + kbytes;
    const char* b_k = b_tile + kbytes;
    asm volatile("" : "+s"(a_k), "+s"(b_k));  // keep the scalar-base addressing form
#pragma unroll
    for (int j = 0; j < DMA_PER; j++)
      __builtin_amdgcn_global_load_lds(
          (glb_void_t*)((j < A_PER ? a_k : b_k) + dma_off[j]),
          (lds_void_t*)(lds_bytes + buf * STAGE_BYTES + dma_group[j] * 1024), 16, 0, 0);
  };
#pragma unroll
  for (int i = 0; i < NBUF - 1; i++) dma_slab(i, i);

  // accumulators: wave set 0 starts from the bias of the lane's column, the others from 0
  f32x16 acc[TM][TN];
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int col = n0 + wn * WN + j * 32 + (lane & 31);
    const float bv = (bias != nullptr && ks == 0 && part == 0 && col < N) ? bias[col] : 0.f;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = bv;
  }

  const int h = lane >> 5;
  const int sw = lane & 7;
  int a_addr[GPW], b_addr[GPW];
#pragma unroll
  for (int i = 0; i < GPW; i++) {
    const int g = ks * GPW + i;
    a_addr[i] = ((wm * WM + (lane & 31)) * CHUNKS + ((2 * g + h) ^ sw)) * 16;
    b_addr[i] = (BM * CHUNKS + (wn * WN + (lane & 31)) * CHUNKS + ((2 * g + h) ^ sw)) * 16;
  }

  if constexpr (PIPE) {
    // Slab s lives in buffer s % NBUF; NBUF - 1 fills are in flight behind the slab that is
    // being multiplied.  Software pipeline, as in matmul_dma_kernel: the operands of a k-group
    // are read while the MFMAs of the group before it run, and the one barrier per slab sits in
    // front of the slab's LAST group -- by then every wave has read all of the slab into
    // registers (its buffer is refilled right away, with slab s + NBUF) and slab s + 1 has
    // landed for every wave, so that its first operands are read under those last MFMAs.
    f32x4 af[2][TM], bf[2][TN];
    auto read_ops = [&](int bufi, int g, int p) {
      const char* const stage = lds_bytes + bufi * STAGE_BYTES;
#pragma unroll
      for (int i = 0; i < TM; i++)
        af[p][i] = *reinterpret_cast<const f32x4*>(stage + a_addr[g] + i * (32 * BK * 4));
#pragma unroll
      for (int j = 0; j < TN; j++)
        bf[p][j] = *reinterpret_cast<const f32x4*>(stage + b_addr[g] + j * (32 * BK * 4));
    };
    auto mfma_group = [&](int p) {
#pragma unroll
      for (int e = 0; e < 4; e++)
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int j = 0; j < TN; j++)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[p][i][e], bf[p][j][e], acc[i][j], 0, 0, 0);
    };
#define G2_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
    // one k-group: its TM + TN operand reads each in the shadow of an MFMA, then the other MFMAs
#define G2_GROUP_SCHEDULE()                                  \
    _Pragma("unroll") for (int i_ = 0; i_ < TM + TN; i_++) {   \
      G2_SGB(0x008, 1);                                        \
      G2_SGB(0x100, 1);                                        \
    }                                                          \
    G2_SGB(0x008, 4 * TM * TN - (TM + TN));
    int buf = 0;
    auto slab_body = [&](int s, auto parity_tag) {
      constexpr int P0 = decltype(parity_tag)::value;  // register set holding the slab's first group
#pragma unroll
      for (int g = 0; g + 1 < GPW; g++) {
        read_ops(buf, g + 1, (P0 + g + 1) & 1);
        mfma_group((P0 + g) & 1);
        G2_GROUP_SCHEDULE();
      }
      __builtin_amdgcn_s_waitcnt(vmcnt_only((NBUF - 2) * DMA_PER));  // my fills of slab s + 1 have landed
      __syncthreads();
      dma_slab(s + NBUF, buf);
      buf = buf + 1 == NBUF ? 0 : buf + 1;
      read_ops(buf, 0, (P0 + GPW) & 1);
      mfma_group((P0 + GPW - 1) & 1);
      G2_GROUP_SCHEDULE();
    };
    dma_slab(NBUF - 1, NBUF - 1);  // the NBUF-th fill: every buffer is busy
    __builtin_amdgcn_s_waitcnt(vmcnt_only((NBUF - 1) * DMA_PER));  // slab 0 has landed
    __syncthreads();
    read_ops(0, 0, 0);
    if constexpr (GPW % 2 == 0) {
      for (int s = 0; s < nslab; s++) slab_body(s, std::integral_constant<int, 0>{});
    } else {
      // an odd number of groups per slab: the register sets swap roles from slab to slab
      int s = 0;
      for (; s + 1 < nslab; s += 2) {
        slab_body(s, std::integral_constant<int, 0>{});
        slab_body(s + 1, std::integral_constant<int, 1>{});
      }
      if (s < nslab) slab_body(s, std::integral_constant<int, 0>{});
    }
#undef G2_GROUP_SCHEDULE
#undef G2_SGB
  } else {
    // Slab s lives in buffer s % NBUF.  Per slab: wait for this wave's fills of slab s,
    // BARRIER (every wave's fills of slab s have landed and every wave has finished with
    // slab s-1), refill slab s-1's buffer with slab s+NBUF-1, multiply slab s.
    int buf = 0;
    for (int s = 0; s < nslab; s++) {
      __builtin_amdgcn_s_waitcnt(vmcnt_only((NBUF - 2) * DMA_PER));
      __syncthreads();
      dma_slab(s + NBUF - 1, buf == 0 ? NBUF - 1 : buf - 1);
      const char* const stage = lds_bytes + buf * STAGE_BYTES;
#pragma unroll
      for (int g = 0; g < GPW; g++) {
        f32x4 af[TM], bf[TN];
#pragma unroll
        for (int i = 0; i < TM; i++)
          af[i] = *reinterpret_cast<const f32x4*>(stage + a_addr[g] + i * (32 * BK * 4));
#pragma unroll
        for (int j = 0; j < TN; j++)
          bf[j] = *reinterpret_cast<const f32x4*>(stage + b_addr[g] + j * (32 * BK * 4));
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
          for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][e], bf[j][e], acc[i][j], 0, 0, 0);
      }
      buf = buf + 1 == NBUF ? 0 : buf + 1;
    }
  }
  __builtin_amdgcn_s_waitcnt(vmcnt_only(0));  // drain the (unused) fills past the last slab

  if (KS > 1) {
    // sum the wave sets' partial tiles: [ks-1][wmn][tile][v][lane], lane-contiguous
    __syncthreads();  // every wave is done with the ring
    float* const red = reinterpret_cast<float*>(lds);
    if (ks > 0) {
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int v = 0; v < 16; v++)
            red[((((ks - 1) * NMN + wmn) * (TM * TN) + i * TN + j) * 16 + v) * 64 + lane] =
                acc[i][j][v];
    }
    __syncthreads();
    if (!SPLIT && ks > 0) return;
    if (ks == 0) {
#pragma unroll
      for (int k2 = 1; k2 < KS; k2++)
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++)
              acc[i][j][v] +=
                  red[((((k2 - 1) * NMN + wmn) * (TM * TN) + i * TN + j) * 16 + v) * 64 + lane];
    }
  }
  if constexpr (SPLIT) {
    __syncthreads();  // the LDS is free: word 0 becomes the flag
    if (!splitk_combine<NMN, TM, TN>(acc, part_ws, part_cnt, pid, part, splits, wmn, ks == 0, lane, tid,
                                     reinterpret_cast<int*>(lds_bytes)))
      return;
  }

  const bool full = (m0 + BM <= M) && (n0 + BN <= N);
  store_tile<TM, TN, GELU>(acc, out, resid, m0 + wm * WM + 4 * h, n0 + wn * WN + (lane & 31), M, N, ldo, full);
}

// M <= 16 rows (one token per sequence: a decode step).  Such a product is bound by
// streaming the weights from HBM once, not by arithmetic, and the problem is small: what
// matters is that all of it is in flight at once.  A workgroup owns 16 weight rows
// (output columns) and its 16 waves split K in units of 16 floats; every lane loads its
// units' 16-byte pieces of the weight row straight into registers (no LDS staging: nothing
// is reused) and the matching pieces of the activation row, which stay cache-resident, and
// feeds them to v_mfma_f32_16x16x4_f32 with the same k permutation as the large kernels
// (element e of a lane's chunk goes to the e-th of four MFMAs).  A = 16 weight rows,
// B = up to 16 activation rows; lane l of the result holds D[4*(l/16) + v][l % 16].
// The 16 partial tiles are summed through LDS in wave order, so results are deterministic.
// LN: the activation rows are layer-normalised on the way in (mean / variance over K by
// llm.c's two passes, then gamma and beta), which needs a wave's whole K share in
// registers at once (K <= 16 * 16 * SK_CHUNK_LN = 1536); every workgroup recomputes the statistics
// of the <= 16 rows from the pieces its waves hold anyway.  resid: added to the result
// (out may alias it).  Together these let a decode step run a transformer block in five
// launches instead of seven.
constexpr int SK_WAVES = 16;
// K units (of 16 floats) a wave has in flight at once; fewer with LN, whose statistics
// and affine terms need registers of their own (16 waves leave 128 per lane)
constexpr int SK_CHUNK_PLAIN = 12, SK_CHUNK_LN = 6;

template <bool GELU, bool LN>
__global__ __launch_bounds__(SK_WAVES* kWave) void matmul_skinny_kernel(
    float* out, const float* __restrict__ inp, const float* __restrict__ weight,
    const float* __restrict__ bias, const float* __restrict__ ln_w, const float* __restrict__ ln_b,
    const float* resid, int M, int K, int N) {
  constexpr int SK_CHUNK = LN ? SK_CHUNK_LN : SK_CHUNK_PLAIN;
  __shared__ float red[SK_WAVES][4][kWave];
  __shared__ float stat[2][SK_WAVES][16];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0 = blockIdx.x * 16;
  const int r16 = lane & 15, kq = lane >> 4;
  // rows past the end are clamped: they feed result rows / columns that are not stored
  const float* wp = weight + (size_t)min(n0 + r16, N - 1) * K + 4 * kq;
  const float* xp = inp + (size_t)min(r16, M - 1) * K + 4 * kq;
  const int units = K / 16;
  const int per = units / SK_WAVES, rem = units % SK_WAVES;
  const int u0 = wave * per + min(wave, rem);
  const int cnt = per + (wave < rem ? 1 : 0);  // wave-uniform; <= SK_CHUNK when LN

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int u = 0; u < cnt || (LN && u == 0); u += SK_CHUNK) {
    f32x4 wv[SK_CHUNK], xv[SK_CHUNK];
#pragma unroll
    for (int c = 0; c < SK_CHUNK; c++)
      if (u + c < cnt)
        wv[c] = __builtin_nontemporal_load(
            reinterpret_cast<const f32x4*>(wp + (size_t)(u0 + u + c) * 16));
#pragma unroll
    for (int c = 0; c < SK_CHUNK; c++)
      if (u + c < cnt) xv[c] = *reinterpret_cast<const f32x4*>(xp + (size_t)(u0 + u + c) * 16);
    if (LN) {
      // row r16's statistics: lanes r16, r16+16, r16+32, r16+48 of all 16 waves hold the row
      float s = 0.f;
#pragma unroll
      for (int c = 0; c < SK_CHUNK; c++)
        if (c < cnt) s += (xv[c][0] + xv[c][1]) + (xv[c][2] + xv[c][3]);
      s += __shfl_xor(s, 16, 64);
      s += __shfl_xor(s, 32, 64);
      if (kq == 0) stat[0][wave][r16] = s;
      __syncthreads();
      float mean = 0.f;
#pragma unroll
      for (int w = 0; w < SK_WAVES; w++) mean += stat[0][w][r16];
      mean /= (float)K;
      float q = 0.f;
#pragma unroll
      for (int c = 0; c < SK_CHUNK; c++)
        if (c < cnt) {
          const f32x4 d = xv[c] - mean;
          q += (d[0] * d[0] + d[1] * d[1]) + (d[2] * d[2] + d[3] * d[3]);
        }
      q += __shfl_xor(q, 16, 64);
      q += __shfl_xor(q, 32, 64);
      if (kq == 0) stat[1][wave][r16] = q;
      __syncthreads();
      float var = 0.f;
#pragma unroll
      for (int w = 0; w < SK_WAVES; w++) var += stat[1][w][r16];
      const float rstd = 1.0f / sqrtf(var / (float)K + 1e-5f);
#pragma unroll
      for (int c = 0; c < SK_CHUNK; c++)
        if (c < cnt) {
          const size_t k = (size_t)(u0 + c) * 16 + 4 * kq;
          const f32x4 g = *reinterpret_cast<const f32x4*>(ln_w + k);
          const f32x4 be = *reinterpret_cast<const f32x4*>(ln_b + k);
          xv[c] = (xv[c] - mean) * rstd * g + be;
        }
    }
#pragma unroll
    for (int c = 0; c < SK_CHUNK; c++) {
      if (u + c < cnt) {
#pragma unroll
        for (int e = 0; e < 4; e++)
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[c][e], xv[c][e], acc, 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int v = 0; v < 4; v++) red[wave][v][lane] = acc[v];
  __syncthreads();
  if (tid < 256) {
    const int i = tid & 15, j = tid >> 4;  // output column n0 + i of row j
    const int v = i & 3, l = (i >> 2) * 16 + j;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < SK_WAVES; w++) sum += red[w][v][l];
    if (j < M && n0 + i < N) {
      if (bias != nullptr) sum += bias[n0 + i];
      if (GELU) sum = gelu_tanh(sum);
      if (resid != nullptr) sum += resid[(size_t)j * N + n0 + i];
      out[(size_t)j * N + n0 + i] = sum;
    }
  }
}

// Whether skinny_launch can take the shape (and, with LN, normalise on the way in).
bool skinny_supported(int M, int K, bool ln, const void* inp, const void* weight) {
  if (M < 1 || M > 16 || K % 16 != 0 || !aligned16(inp) || !aligned16(weight)) return false;
  return !ln || (K / 16 + SK_WAVES - 1) / SK_WAVES <= SK_CHUNK_LN;
}

int skinny_launch(float* out, const float* inp, const float* weight, const float* bias,
                  const float* ln_w, const float* ln_b, const float* resid, int M, int K, int N,
                  bool gelu) {
  const bool ln = ln_w != nullptr;
  if (!skinny_supported(M, K, ln, inp, weight) || (ln && (!ln_b || !aligned16(ln_w) || !aligned16(ln_b))))
    return fail(GPT2HIP_EINVAL, "matmul (<= 16 rows): unsupported shape M=%d K=%d", M, K);
  auto kfn = gelu ? (ln ? matmul_skinny_kernel<true, true> : matmul_skinny_kernel<true, false>)
                  : (ln ? matmul_skinny_kernel<false, true> : matmul_skinny_kernel<false, false>);
  hipLaunchKernelGGL(kfn, dim3((unsigned)((N + 15) / 16)), dim3(SK_WAVES * kWave), 0, stream(), out, inp,
                     weight, bias, ln_w, ln_b, resid, M, K, N);
  G2_LAUNCH_CHECK("matmul_forward");
  return GPT2HIP_OK;
}

// Any shape, any alignment; one thread per output.  Only used when K is not a
// multiple of 4 or an operand is not 16-byte aligned.
__global__ __launch_bounds__(256) void matmul_generic_kernel(float* out, const float* inp,
                                                              const float* weight,
                                                              const float* bias, const float* resid,
                                                              int M, int K, int N, int gelu) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (size_t)M * N) return;
  const int row = (int)(idx / N), col = (int)(idx % N);
  const float* x = inp + (size_t)row * K;
  const float* w = weight + (size_t)col * K;
  float acc = bias ? bias[col] : 0.f;
  for (int k = 0; k < K; k++) acc += x[k] * w[k];
  acc = gelu ? gelu_tanh(acc) : acc;
  out[idx] = resid ? acc + resid[idx] : acc;
}

// Reduces the (value, column) pairs that the ARGMAX form of matmul_dma_kernel leaves
// per row to the row's argmax; one wave per row, four rows per block.
__global__ __launch_bounds__(256) void argmax_pairs_kernel(int* __restrict__ ids,
                                                            const float* __restrict__ val,
                                                            const int* __restrict__ idx, int M,
                                                            int pairs) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const int lane = threadIdx.x & 63;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int p = lane; p < pairs; p += 64)
    argmax_combine(best, bi, val[(size_t)row * pairs + p], idx[(size_t)row * pairs + p]);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float ov = __shfl_xor(best, off, 64);
    const int oi = __shfl_xor(bi, off, 64);
    argmax_combine(best, bi, ov, oi);
  }
  // a row of all -inf / NaN never beats the initial value: report index 0
  if (lane == 0) ids[row] = (bi == 0x7fffffff) ? 0 : bi;
}

// Any shape, any alignment: one block per row computes the row's products one thread per
// column (the arithmetic of matmul_generic_kernel) and keeps only their argmax.
__global__ __launch_bounds__(256) void matmul_argmax_generic_kernel(int* __restrict__ ids,
                                                                     const float* inp,
                                                                     const float* weight,
                                                                     const float* bias, int K,
                                                                     int N) {
  const float* x = inp + (size_t)blockIdx.x * K;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int col = threadIdx.x; col < N; col += 256) {
    const float* w = weight + (size_t)col * K;
    float acc = bias ? bias[col] : 0.f;
    for (int k = 0; k < K; k++) acc += x[k] * w[k];
    if (acc > best) {
      best = acc;
      bi = col;
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float ov = __shfl_xor(best, off, 64);
    const int oi = __shfl_xor(bi, off, 64);
    argmax_combine(best, bi, ov, oi);
  }
  __shared__ float sv[4];
  __shared__ int si[4];
  if ((threadIdx.x & 63) == 0) {
    sv[threadIdx.x >> 6] = best;
    si[threadIdx.x >> 6] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; w++) argmax_combine(best, bi, sv[w], si[w]);
    ids[blockIdx.x] = (bi == 0x7fffffff) ? 0 : bi;
  }
}

// Raises the dynamic-LDS limit of a kernel, once per (thread, device, kernel).
static int allow_lds(const void* kfn, size_t lds_bytes) {
  static thread_local int configured_for = -1;
  static thread_local std::unordered_set<const void*> configured;  // grows with the forms touched
  int dev = 0;
  G2_HIP(hipGetDevice(&dev));
  if (configured_for != dev) {
    configured_for = dev;
    configured.clear();
  }
  if (configured.count(kfn)) return GPT2HIP_OK;
  G2_HIP(hipFuncSetAttribute(kfn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
  configured.insert(kfn);
  return GPT2HIP_OK;
}

// What a launch does beyond out = act(inp . weight^T + bias).  resid (optional): added in the
// epilogue.  ldo (0: N): floats from one row of out (and of resid) to the next, when the launch
// computes a range of the columns of a wider product.
struct Epilogue {
  const float* resid = nullptr;
  int ldo = 0;
};

// Register-staged kernel: any K % 4 == 0.
template <int BM, int BN, int WGM, int WGN>
static int launch_mfma(float* out, const float* inp, const float* weight, const float* bias, int M,
                       int K, int N, bool gelu, Epilogue epi = {}) {
  constexpr int NT = WGM * WGN * kWave;
  constexpr size_t lds_bytes = 2 * (size_t)(BM + BN) * BK * sizeof(float);
  const int ntm = (M + BM - 1) / BM, ntn = (N + BN - 1) / BN;
  const long long tiles = (long long)ntm * ntn;
  if (tiles > 0x7fffffffLL) return fail(GPT2HIP_EINVAL, "matmul_forward: too many tiles");
  const bool ktail = (K % BK) != 0;
  auto kfn = ktail ? (gelu ? matmul_mfma_kernel<BM, BN, WGM, WGN, true, true>
                           : matmul_mfma_kernel<BM, BN, WGM, WGN, false, true>)
                   : (gelu ? matmul_mfma_kernel<BM, BN, WGM, WGN, true, false>
                           : matmul_mfma_kernel<BM, BN, WGM, WGN, false, false>);
  if (int rc = allow_lds(reinterpret_cast<const void*>(kfn), lds_bytes)) return rc;
  hipLaunchKernelGGL(kfn, dim3((unsigned)tiles), dim3(NT), lds_bytes, stream(), out, inp, weight, bias,
                     epi.resid, M, K, N, epi.ldo ? epi.ldo : N, ntm, ntn);
  G2_LAUNCH_CHECK("matmul_forward");
  return GPT2HIP_OK;
}

// K split between the workgroups of a tile (splitk_combine): where the partial tiles and the
// per-tile counters live, and how many parts.  splits == 1: no split.
struct SplitK {
  float* ws = nullptr;
  unsigned* cnt = nullptr;
  int splits = 1;
};

// LDS-DMA kernel: K % 32 == 0.  The clock-probe form exists for PROBED tile shapes only.
template <int BM, int BN, int WGM, int WGN, bool PROBED = false>
static int launch_dma(float* out, const float* inp, const float* weight, const float* bias, int M,
                      int K, int N, bool gelu, unsigned long long* probe = nullptr, SplitK sk = {},
                      Epilogue epi = {}) {
  constexpr int NT = WGM * WGN * kWave;
  constexpr size_t lds_bytes = 2 * (size_t)(BM + BN) * BK * sizeof(float);
  const int ntm = (M + BM - 1) / BM, ntn = (N + BN - 1) / BN;
  const long long tiles = (long long)ntm * ntn * sk.splits;
  if (tiles > 0x7fffffffLL) return fail(GPT2HIP_EINVAL, "matmul_forward: too many tiles");
  auto kfn = gelu ? matmul_dma_kernel<BM, BN, WGM, WGN, true> : matmul_dma_kernel<BM, BN, WGM, WGN, false>;
  if (sk.splits > 1) {
    if (probe) return fail(GPT2HIP_EINVAL, "matmul_forward_probe: no probe form with K split");
    kfn = gelu ? matmul_dma_kernel<BM, BN, WGM, WGN, true, false, false, true>
               : matmul_dma_kernel<BM, BN, WGM, WGN, false, false, false, true>;
  } else if (epi.resid && !gelu && !probe && (BM / WGM / 32) * (BN / WGN / 32) <= 3) {
    // (larger register tiles have no room for the tile of resid beside the accumulators: they read
    // it in the epilogue)
    if constexpr ((BM / WGM / 32) * (BN / WGN / 32) <= 3)
      kfn = matmul_dma_kernel<BM, BN, WGM, WGN, false, false, false, false, true>;
  } else if constexpr (PROBED) {
    if (probe) kfn = matmul_dma_kernel<BM, BN, WGM, WGN, false, true>;
  } else if (probe) {
    return fail(GPT2HIP_EINVAL, "matmul_forward_probe: no probe form of the %dx%d tile", BM, BN);
  }
  if (int rc = allow_lds(reinterpret_cast<const void*>(kfn), lds_bytes)) return rc;
  hipLaunchKernelGGL(kfn, dim3((unsigned)tiles), dim3(NT), lds_bytes, stream(), out, inp, weight, bias,
                     epi.resid, M, K, N, epi.ldo ? epi.ldo : N, ntm, ntn, probe, (int*)nullptr, sk.ws, sk.cnt,
                     sk.splits);
  G2_LAUNCH_CHECK("matmul_forward");
  return GPT2HIP_OK;
}

// The 128x192 LDS-DMA kernel in its ARGMAX form followed by the pair reduction.
constexpr int kArgmaxBN = 192, kArgmaxWGN = 2;
template <int WGM>
static int launch_dma_argmax(int* ids, float* pair_val, int* pair_idx, const float* inp,
                             const float* weight, const float* bias, int M, int K, int N) {
  constexpr int BM = 128, BN = kArgmaxBN, WGN = kArgmaxWGN;
  constexpr int NT = WGM * WGN * kWave;
  constexpr size_t lds_bytes = 2 * (size_t)(BM + BN) * BK * sizeof(float);
  const int ntm = (M + BM - 1) / BM, ntn = (N + BN - 1) / BN;
  auto kfn = matmul_dma_kernel<BM, BN, WGM, WGN, false, false, true>;
  if (int rc = allow_lds(reinterpret_cast<const void*>(kfn), lds_bytes)) return rc;
  hipLaunchKernelGGL(kfn, dim3((unsigned)(ntm * ntn)), dim3(NT), lds_bytes, stream(), pair_val, inp, weight,
                     bias, (const float*)nullptr, M, K, N, N, ntm, ntn, (unsigned long long*)nullptr, pair_idx,
                     (float*)nullptr, (unsigned*)nullptr, 1);
  G2_LAUNCH_CHECK("matmul_forward_argmax");
  hipLaunchKernelGGL(argmax_pairs_kernel, dim3((unsigned)((M + 3) / 4)), dim3(256), 0, stream(), ids,
                     pair_val, pair_idx, M, ntn * WGN);
  G2_LAUNCH_CHECK("matmul_forward_argmax");
  return GPT2HIP_OK;
}

// Ring kernel for small problems: K % 32 == 0.
template <int BM, int BN, int WGM, int WGN, int KS, int NBUF, bool PIPE = false>
static int launch_ring(float* out, const float* inp, const float* weight, const float* bias, int M,
                       int K, int N, bool gelu, SplitK sk = {}, Epilogue epi = {}) {
  constexpr int NT = WGM * WGN * KS * kWave;
  constexpr size_t lds_bytes = (size_t)NBUF * (BM + BN) * BK * sizeof(float);
  const int ntm = (M + BM - 1) / BM, ntn = (N + BN - 1) / BN;
  const long long tiles = (long long)ntm * ntn * sk.splits;
  if (tiles > 0x7fffffffLL) return fail(GPT2HIP_EINVAL, "matmul_forward: too many tiles");
  auto kfn = gelu ? matmul_ring_kernel<BM, BN, WGM, WGN, KS, NBUF, true, false, PIPE>
                  : matmul_ring_kernel<BM, BN, WGM, WGN, KS, NBUF, false, false, PIPE>;
  if (sk.splits > 1)
    kfn = gelu ? matmul_ring_kernel<BM, BN, WGM, WGN, KS, NBUF, true, true, PIPE>
               : matmul_ring_kernel<BM, BN, WGM, WGN, KS, NBUF, false, true, PIPE>;
  if (int rc = allow_lds(reinterpret_cast<const void*>(kfn), lds_bytes)) return rc;
  hipLaunchKernelGGL(kfn, dim3((unsigned)tiles), dim3(NT), lds_bytes, stream(), out, inp, weight, bias,
                     epi.resid, M, K, N, epi.ldo ? epi.ldo : N, ntm, ntn, sk.ws, sk.cnt, sk.splits);
  G2_LAUNCH_CHECK("matmul_forward");
  return GPT2HIP_OK;
}

// Tile choice.  A launch of tiles of one shape takes, to within a few per cent over
// M = 64 .. 8192 at the GPT-2 124M and 350M shapes (fitted per shape to a sweep in which
// every shape was forced on every problem),
//     launch + ceil(tiles / 256 CUs) x (a x tile area x K / per-CU MFMA rate + round)
// where a "round" of one tile per compute unit costs its matrix work (a: the smaller the
// tile, the more bytes go through LDS per MFMA) plus the part of a tile's first loads and
// final stores that nothing hides.  The shape with the least predicted time wins: over
// the sweep its time is within 2.4 % of the best forced shape's (0.13 % on average).  A
// problem whose tile count is just above a multiple of 256 with the largest tile (124M qkv
// at M = 4096: 384 tiles of 128x192, two rounds for one and a half rounds of work, 65 % of
// peak) takes a smaller tile that divides evenly (768 tiles of 128x96, three exact rounds,
// 85 %).  The clock probe exists for the two largest shapes only.
struct TileChoice {
  int index;        // into the candidate list below
  int bm, bn;
  long long tiles;
  int splits;       // workgroups per tile (K split between them), 1 = none
  double cost_us;   // what the model below expects the launch to take
};
// fix_*: what a K split between workgroups adds (fitted per shape to a second forced sweep, over
// 2..8 parts): fix_us + fix_part_us x parts + fix_mb_us x MB of partial tiles.  The partial
// tiles cross memory twice (parts x the size of the product each way), which is what makes a
// split pay at K = 3072 or 4096 (up to 20 %, twice as fast at B*T <= 128) and hardly ever at
// K = 768, where that traffic costs as much as the rounds it fills.
struct TileCand { int bm, bn; double a, round_us, launch_us, fix_us, fix_part_us, fix_mb_us; };
// (64x192 and 128x64 were fitted too -- a = 1.033 and 1.042 -- and never won by more than
// 0.4 % anywhere in the sweep: not built)
static const TileCand kTileCands[] = {
    {128, 192, 0.988, 6.42, -2.15, 4.22, 0.90, 0.068}, {128, 128, 1.006, 3.59, -0.11, 3.76, 0.66, 0.020},
    {128, 96, 1.017, 1.84, 1.93, 2.73, 0.54, 0.066},   {64, 128, 1.042, 2.08, 1.01, 2.30, 0.41, 0.0},
    {64, 64, 1.159, 0.40, 1.88, 1.65, 0.22, 0.115},    {32, 32, 1.398, 0.0, 3.54, 0.81, 0.20, 0.492},
    {64, 96, 1.094, 0.98, 3.06, 1.53, 0.44, 0.161},    {256, 192, 0.970, 7.5, 4.9, 1e9, 0.0, 0.0},
    {256, 128, 1.000, 2.8, 4.0, 1e9, 0.0, 0.0},   {128, 160, 1.000, 4.6, 0.5, 4.0, 0.8, 0.05}};
constexpr int kTile128x160 = 9;  // only for products whose width is a multiple of 160 (see choose_tile)
// (256x192 -- eight waves of 64x96 -- moves 30 % fewer bytes into LDS per MFMA than 128x192 and
// wins 1.5-2.5 points where its tiles come out in whole rounds: fc at M = 4096 / 8192, the
// 350M qkv at 4096 / 8192.  256x128 -- eight waves of 64x64 -- does the same against 128x128 for
// the 4096-wide fc of the 350M model: 86.7 -> 89.9 % at M = 4096.  Their K split is never
// planned: a partial tile is 128-192 KB.)
// a split is taken when the model puts it this far ahead of the best plan without one (over
// the sweep no chosen split is then slower than that plan; 0.8 % behind the best forced plan
// on average, 5.1 % ahead of the choice without splits)
constexpr double kSplitMargin = 1.08;
constexpr int kTileCandCount = (int)(sizeof(kTileCands) / sizeof(kTileCands[0]));
constexpr double kCuFlopsPerUs = 579e3;  // what one compute unit sustains in the 128x192 loop
constexpr size_t kSplitCounters = GPT2HIP_SPLITK_COUNTER_BYTES / sizeof(unsigned);

static long long tiles_of(int i, int M, int OC) {
  return (long long)((M + kTileCands[i].bm - 1) / kTileCands[i].bm) *
         ((OC + kTileCands[i].bn - 1) / kTileCands[i].bn);
}

// Whether `splits` workgroups per tile of candidate i fit the workspace (counters first, then
// tiles x splits partial tiles) and the kernel (every part needs a slab).
static bool split_fits(int i, int M, int C, int OC, int splits, size_t workspace_bytes) {
  if (splits == 1) return true;
  const long long t = tiles_of(i, M, OC);
  if (splits < 1 || splits > C / BK || t > (long long)kSplitCounters) return false;
  if (workspace_bytes < GPT2HIP_SPLITK_COUNTER_BYTES) return false;
  const unsigned long long need =
      (unsigned long long)t * splits * kTileCands[i].bm * kTileCands[i].bn * sizeof(float);
  return need <= workspace_bytes - GPT2HIP_SPLITK_COUNTER_BYTES;
}

// The constants of candidate i as it is launched for `groups` workgroups, and the model's time for
// t tiles of it with K split S ways (without what the split itself adds).
static TileCand cand_form(int i, long long groups) {
  TileCand k = kTileCands[i];
  if (i == 4 && groups <= 2 * 256) {  // the ring form of 64x64
    k.a = 1.190;
    k.round_us = 0.35;
    k.launch_us = 2.98;
  }
  return k;
}
static double tile_cost(int i, long long t, int C, int S) {
  const TileCand k = cand_form(i, t * S);
  const double work_us = 2.0 * k.bm * k.bn * (double)C / kCuFlopsPerUs;
  return k.launch_us + (double)((t * S + 255) / 256) * (k.a * work_us / S + k.round_us);
}

// workspace_bytes == 0: no K split between workgroups.
static TileChoice choose_tile(int M, int C, int OC, bool two_largest_only, size_t workspace_bytes = 0) {
  int best = 0, split_best = -1, split_parts = 1;
  double best_cost = 0, split_cost = 0;
  for (int i = 0; i < (two_largest_only ? 2 : kTileCandCount); i++) {
    // 128x160 exists for the widths that no other shape divides into whole rounds (1280 = 8 x 160:
    // GPT-2 large's projections at B*T = 4096 are 256 such tiles, against 224 ragged ones of
    // 128x192 or 320 of 128x128); the GPT-2 124M / 350M widths are no multiples of 160
    if (i == kTile128x160 && OC % 160 != 0) continue;
    const long long t = tiles_of(i, M, OC);
    // K split S ways: S times the workgroups, each with 1/S of the matrix work, plus the
    // partial tiles' trip through memory (written once, read once by the last arrival)
    for (int S = 1; S <= 8; S++) {
      if (S > 1 && (workspace_bytes == 0 || two_largest_only || t * S > 6 * 256 ||
                    !split_fits(i, M, C, OC, S, workspace_bytes)))
        continue;
      const TileCand k = cand_form(i, t * S);
      double cost = tile_cost(i, t, C, S);
      if (S == 1) {
        if (i == 0 || cost < best_cost) {
          best = i;
          best_cost = cost;
        }
      } else {
        cost += k.fix_us + k.fix_part_us * S + k.fix_mb_us * ((double)t * S * k.bm * k.bn * 4e-6);
        if (split_best < 0 || cost < split_cost) {
          split_best = i;
          split_cost = cost;
          split_parts = S;
        }
      }
    }
    // sixteen or more rounds of the largest tile (the lm-head): rounding up to whole
    // rounds costs at most 3 %, less than any smaller tile loses
    if (i == 0 && t >= 16 * 256) break;
  }
  if (split_best >= 0 && split_cost * kSplitMargin < best_cost)
    return TileChoice{split_best, kTileCands[split_best].bm, kTileCands[split_best].bn,
                      tiles_of(split_best, M, OC), split_parts, split_cost};
  return TileChoice{best, kTileCands[best].bm, kTileCands[best].bn, tiles_of(best, M, OC), 1, best_cost};
}

// A product whose tiles come out just above a whole number of rounds loses most of a round to
// the few tiles left over: the lm-head's 50257 columns are 261.75 tiles of 192, so at 256 rows
// there are 262 tiles of 256x192 for 256 compute units, and at 1024 rows 4 x 262; the 2304 columns
// of a qkv product at 1024 rows are 16 x 18 tiles of 64x128.  Such a product (1536 columns or
// more) is computed by two launches over ranges of its columns instead: a whole number of rounds
// of the tile that suits it, then the columns left -- at most a quarter -- with whatever suits
// those (measured for the 768 -> 50257 lm-head: 216 -> 180 us at 256 rows, 348 -> 324 at
// 512, 619 -> 590 at 1024, 1150 -> 1136 at 2048; within 0.5 % either way from 4096 rows on, where
// the product is left as one launch; 768 -> 2304 at 1024 rows 40.8 -> 36.6 us; GPT-2 XL's
// 1600 -> 6400 at 1024 / 2048 rows 188 -> 155 / 351 -> 299 us, its 1600 -> 1600 at 2048 rows,
// which no tile of the set divides, 96 -> 85 us as one round of 128x96 over 1536 columns + 64).
struct ColumnPlan {
  int main_cols;         // columns of the first launch; == OC: one launch
  TileChoice main, rest;
};
static ColumnPlan plan_columns(int M, int C, int OC, bool two_largest_only, size_t workspace_bytes) {
  ColumnPlan plan{OC, choose_tile(M, C, OC, two_largest_only, workspace_bytes), TileChoice{}};
  if (two_largest_only || OC < 1536) return plan;
  // a second launch has to pay for itself: taken only when the model puts it 3 % ahead (over M =
  // 256 ... 8192 at the layer shapes of the four GPT-2 sizes every plan this changes got faster, by
  // 1-17 %; taken at par or 3 % behind, 19 more plans change, 12 of them for the worse)
  double best = plan.main.cost_us * 0.97;
  // 128x192, 256x192, 128x128, 256x128; for products of fewer than 8192 columns also 64x128,
  // 128x96, 64x96 and 128x160
  static const int kWide[] = {0, 7, 1, 8, 3, 2, 6, kTile128x160};
  for (int i : kWide) {
    if ((i == 3 || i == 2 || i == 6 || i == kTile128x160) && OC >= 8192) continue;
    const long long ntm = (M + kTileCands[i].bm - 1) / kTileCands[i].bm;
    const int ntn_all = OC / kTileCands[i].bn;
    for (int ntn = ntn_all; ntn >= 1 && ntn > ntn_all - 16; ntn--) {
      const long long t = ntm * ntn;
      if (t % 256 != 0) continue;
      if (t > 12 * 256) break;  // the more rounds, the less the last one matters
      const int cols = ntn * kTileCands[i].bn;
      if (cols == OC) break;  // (whole rounds already)
      if ((OC - cols) * 4 > OC) break;  // (a remainder, not a second product)
      const TileChoice rest = choose_tile(M, C, OC - cols, false, workspace_bytes);
      const double cost = tile_cost(i, t, C, 1) + rest.cost_us;
      if (cost < best) {
        best = cost;
        plan.main_cols = cols;
        plan.main = TileChoice{i, kTileCands[i].bm, kTileCands[i].bn, t, 1, tile_cost(i, t, C, 1)};
        plan.rest = rest;
      }
      break;  // the widest whole number of rounds of this tile
    }
  }
  return plan;
}

// Launches candidate `best` with the K split of `sk`.
static int launch_choice(int best, long long best_tiles, float* out, const float* inp, const float* weight,
                         const float* bias, int M, int C, int OC, bool gelu, unsigned long long* probe,
                         SplitK sk, Epilogue epi) {
  switch (best) {
    case kTile128x160:
      // four waves of 32x160, two workgroups per compute unit
      return launch_dma<128, 160, 4, 1>(out, inp, weight, bias, M, C, OC, gelu, nullptr, sk, epi);
    case 8:
      // eight waves of 64x64, one workgroup per compute unit
      return launch_dma<256, 128, 4, 2>(out, inp, weight, bias, M, C, OC, gelu, nullptr, sk, epi);
    case 7:
      // eight waves of 64x96, one workgroup per compute unit
      return launch_dma<256, 192, 4, 2>(out, inp, weight, bias, M, C, OC, gelu, nullptr, sk, epi);
    case 6:
      // 64x96: two waves side by side, K split between two such pairs
      return launch_ring<64, 96, 2, 1, 2, 4, true>(out, inp, weight, bias, M, C, OC, gelu, sk, epi);
    case 5:
      // one 32x32 tile per workgroup, its four waves splitting K
      return launch_ring<32, 32, 1, 1, 4, 4>(out, inp, weight, bias, M, C, OC, gelu, sk, epi);
    case 4:
      // up to two workgroups per CU: latency-bound, ring of four slabs and a 2-way K split
      if (best_tiles * sk.splits <= 2 * 256)
        return launch_ring<64, 64, 2, 2, 2, 4>(out, inp, weight, bias, M, C, OC, gelu, sk, epi);
      return launch_dma<64, 64, 2, 2>(out, inp, weight, bias, M, C, OC, gelu, nullptr, sk, epi);
    case 3:
      return launch_dma<64, 128, 2, 2>(out, inp, weight, bias, M, C, OC, gelu, nullptr, sk, epi);
    case 2:
      // four waves of 32x96: two workgroups per compute unit
      return launch_dma<128, 96, 4, 1>(out, inp, weight, bias, M, C, OC, gelu, nullptr, sk, epi);
    case 1:
      return launch_dma<128, 128, 4, 2, true>(out, inp, weight, bias, M, C, OC, gelu, probe, sk, epi);
    default:
      // Many tiles per CU: 4 waves with 64x96 register tiles, two workgroups per CU.
      // Few tiles per CU: 8 waves with 32x96 tiles, so that a lone workgroup still
      // gives every SIMD two waves to alternate between.
      if (best_tiles >= 16 * 256 && sk.splits == 1)
        return launch_dma<128, 192, 2, 2, true>(out, inp, weight, bias, M, C, OC, gelu, probe, SplitK{}, epi);
      return launch_dma<128, 192, 4, 2, true>(out, inp, weight, bias, M, C, OC, gelu, probe, sk, epi);
  }
}

// workspace (optional): GPT2HIP_SPLITK_COUNTER_BYTES of counters that are zero between calls,
// then room for partial tiles; allows K to be split between workgroups.  forced (optional):
// a tile shape and split count to use instead of the cost model's.
struct ForcedPlan { int bm, bn, splits; };
static int matmul_dispatch(float* out, const float* inp, const float* weight, const float* bias,
                           int B, int T, int C, int OC, bool gelu,
                           unsigned long long* probe = nullptr, int* probe_groups = nullptr,
                           void* workspace = nullptr, size_t workspace_bytes = 0,
                           const ForcedPlan* forced = nullptr, const float* resid = nullptr) {
  if (B < 0 || T < 0 || C < 1 || OC < 1)
    return fail(GPT2HIP_EINVAL, "matmul_forward: bad shape B=%d T=%d C=%d OC=%d", B, T, C, OC);
  const long long M64 = (long long)B * T;
  if (M64 > 0x7fffffffLL) return fail(GPT2HIP_EINVAL, "matmul_forward: B*T too large");
  const int M = (int)M64;
  if (M == 0) return GPT2HIP_OK;
  if (!out || !inp || !weight) return fail(GPT2HIP_EINVAL, "matmul_forward: null pointer");
  if (workspace && ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0))
    return fail(GPT2HIP_EINVAL, "matmul_forward: workspace must be 256-byte aligned");
  if (!workspace) workspace_bytes = 0;
  const bool tiled = C % BK == 0 && (long long)C * 192 * 4 < (1LL << 31) && C % 4 == 0 &&
                     aligned16(inp) && aligned16(weight);
  if (forced && !tiled) return fail(GPT2HIP_EINVAL, "matmul_forward: a forced plan needs C %% 32 == 0 and aligned operands");
  if (C % 4 != 0 || !aligned16(inp) || !aligned16(weight)) {
    if (probe) return fail(GPT2HIP_EINVAL, "matmul_forward_probe: needs the MFMA path");
    const size_t total = (size_t)M * OC;
    hipLaunchKernelGGL(matmul_generic_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream(),
                       out, inp, weight, bias, resid, M, C, OC, gelu ? 1 : 0);
    G2_LAUNCH_CHECK("matmul_forward");
    return GPT2HIP_OK;
  }
  if (M <= 16 && C % 16 == 0 && !probe && !forced)
    return skinny_launch(out, inp, weight, bias, nullptr, nullptr, resid, M, C, OC, gelu);
  // per-lane DMA offsets are 32-bit byte offsets inside one tile's rows
  if (tiled) {
    TileChoice choice;
    if (forced) {
      int idx = -1;
      for (int i = 0; i < kTileCandCount; i++)
        if (kTileCands[i].bm == forced->bm && kTileCands[i].bn == forced->bn) idx = i;
      if (idx < 0) return fail(GPT2HIP_EINVAL, "matmul_forward: no %dx%d tile", forced->bm, forced->bn);
      if (!split_fits(idx, M, C, OC, forced->splits, workspace_bytes))
        return fail(GPT2HIP_EINVAL, "matmul_forward: %d-way K split of %dx%d tiles does not fit (K slabs %d, workspace %zu bytes)",
                    forced->splits, forced->bm, forced->bn, C / BK, workspace_bytes);
      choice = TileChoice{idx, forced->bm, forced->bn, tiles_of(idx, M, OC), forced->splits};
    } else {
      const ColumnPlan cp = plan_columns(M, C, OC, probe != nullptr, workspace_bytes);
      choice = cp.main;
      if (cp.main_cols != OC) {
        // two launches over ranges of the columns; rows of out (and resid) stay OC floats apart
        const size_t n1 = (size_t)cp.main_cols;
        if (int rc = launch_choice(cp.main.index, cp.main.tiles, out, inp, weight, bias, M, C, cp.main_cols, gelu,
                                   nullptr, SplitK{}, Epilogue{resid, OC}))
          return rc;
        SplitK sk;
        if (cp.rest.splits > 1) {
          sk.cnt = static_cast<unsigned*>(workspace);
          sk.ws = reinterpret_cast<float*>(static_cast<char*>(workspace) + GPT2HIP_SPLITK_COUNTER_BYTES);
          sk.splits = cp.rest.splits;
        }
        return launch_choice(cp.rest.index, cp.rest.tiles, out + n1, inp, weight + n1 * C, bias ? bias + n1 : nullptr,
                             M, C, OC - cp.main_cols, gelu, nullptr, sk, Epilogue{resid ? resid + n1 : nullptr, OC});
      }
    }
    if (choice.tiles * choice.splits > 0x7fffffffLL) return fail(GPT2HIP_EINVAL, "matmul_forward: too many tiles");
    if (probe_groups) *probe_groups = (int)choice.tiles;
    SplitK sk;
    if (choice.splits > 1) {
      sk.cnt = static_cast<unsigned*>(workspace);
      sk.ws = reinterpret_cast<float*>(static_cast<char*>(workspace) + GPT2HIP_SPLITK_COUNTER_BYTES);
      sk.splits = choice.splits;
    }
    return launch_choice(choice.index, choice.tiles, out, inp, weight, bias, M, C, OC, gelu, probe, sk,
                         Epilogue{resid, 0});
  }
  if (probe) return fail(GPT2HIP_EINVAL, "matmul_forward_probe: needs C %% 32 == 0");
  return launch_mfma<128, 192, 4, 2>(out, inp, weight, bias, M, C, OC, gelu, Epilogue{resid, 0});
}

// ---- lm-head + argmax -------------------------------------------------------------------
static int argmax_dispatch(int* ids, void* workspace, size_t workspace_bytes, const float* inp,
                           const float* weight, const float* bias, int B, int T, int C, int OC) {
  if (B < 0 || T < 0 || C < 1 || OC < 1)
    return fail(GPT2HIP_EINVAL, "matmul_forward_argmax: bad shape B=%d T=%d C=%d OC=%d", B, T, C, OC);
  const long long M64 = (long long)B * T;
  if (M64 > 0x7fffffffLL) return fail(GPT2HIP_EINVAL, "matmul_forward_argmax: B*T too large");
  const int M = (int)M64;
  if (M == 0) return GPT2HIP_OK;
  if (!ids || !inp || !weight) return fail(GPT2HIP_EINVAL, "matmul_forward_argmax: null pointer");
  if (C % BK != 0 || !aligned16(inp) || !aligned16(weight) ||
      (long long)C * 192 * 4 >= (1LL << 31)) {
    hipLaunchKernelGGL(matmul_argmax_generic_kernel, dim3((unsigned)M), dim3(256), 0, stream(), ids, inp,
                       weight, bias, C, OC);
    G2_LAUNCH_CHECK("matmul_forward_argmax");
    return GPT2HIP_OK;
  }
  const size_t need = matmul_forward_argmax_workspace(B, T, OC);
  if (!workspace || workspace_bytes < need)
    return fail(GPT2HIP_EINVAL, "matmul_forward_argmax: workspace of %zu bytes, need %zu",
                workspace_bytes, need);
  const long long tiles = (long long)((M + 127) / 128) * ((OC + 191) / 192);
  if (tiles > 0x7fffffffLL) return fail(GPT2HIP_EINVAL, "matmul_forward_argmax: too many tiles");
  float* pair_val = static_cast<float*>(workspace);
  int* pair_idx = reinterpret_cast<int*>(pair_val + need / 8);
  if (tiles >= 16 * 256)
    return launch_dma_argmax<2>(ids, pair_val, pair_idx, inp, weight, bias, M, C, OC);
  return launch_dma_argmax<4>(ids, pair_val, pair_idx, inp, weight, bias, M, C, OC);
}

// The (value, column) pairs of matmul_forward_argmax_noalloc: 33 MiB of device memory that
// every GPU the library runs on holds from the moment its code is loaded there until the
// process ends (8192 rows x 524 pairs x 8 bytes, the lm-head of GPT-2 at B*T = 8192).  Every
// pair a launch reads is written by the same launch first, so nothing needs clearing between
// calls; two calls that overlap on one GPU (different streams) share the array and race.
static __device__ __align__(256) unsigned char scratch[GPT2HIP_ARGMAX_NOALLOC_BYTES];

// The array's address on the current device.  `scratch` itself is only a host-side handle:
// each device has its own copy at its own address, looked up once per device.
static int scratch_address(void** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex lock;
  static void* address[kMaxDevices];  // zero-initialised
  int dev = 0;
  G2_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(GPT2HIP_EINVAL, "matmul_forward_argmax_noalloc: device %d out of range", dev);
  std::lock_guard<std::mutex> hold(lock);
  if (!address[dev]) {
    void* p = nullptr;
    G2_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(GPT2HIP_EHIP, "matmul_forward_argmax_noalloc: no address for the scratch array");
    address[dev] = p;
  }
  *out = address[dev];
  return GPT2HIP_OK;
}

}  // namespace g2

extern "C" {

int matmul_forward_status(float* out, const float* inp, const float* weight, const float* bias,
                          int B, int T, int C, int OC) {
  const g2::ThreadWorkspace& w = g2::workspace_slot();  // gpt2hip_set_workspace; none by default
  return g2::matmul_dispatch(out, inp, weight, bias, B, T, C, OC, false, nullptr, nullptr, w.ptr, w.bytes);
}

void matmul_forward(float* out, const float* inp, const float* weight, const float* bias, int B,
                    int T, int C, int OC) {
  if (matmul_forward_status(out, inp, weight, bias, B, T, C, OC)) g2::die("matmul_forward");
}

int matmul_forward_probe_status(float* out, const float* inp, const float* weight,
                                const float* bias, int B, int T, int C, int OC,
                                unsigned long long* probe, int probe_capacity, int* workgroups) {
  using namespace g2;
  if (!probe || !workgroups) return fail(GPT2HIP_EINVAL, "matmul_forward_probe: null pointer");
  // the smallest tile shape bounds the number of workgroups any choice can launch
  const long long most = (((long long)B * T + 31) / 32) * ((OC + 31) / 32);
  if (most > probe_capacity)
    return fail(GPT2HIP_EINVAL, "matmul_forward_probe: probe buffer holds %d workgroups, need %lld",
                probe_capacity, most);
  return matmul_dispatch(out, inp, weight, bias, B, T, C, OC, false, probe, workgroups);
}

int matmul_forward_tile_shape(int B, int T, int C, int OC, int* tile_rows, int* tile_cols) {
  using namespace g2;
  const long long M64 = (long long)B * T;
  if (B < 1 || T < 1 || C < 1 || OC < 1 || M64 > 0x7fffffffLL || !tile_rows || !tile_cols)
    return fail(GPT2HIP_EINVAL, "matmul_forward_tile_shape: bad shape B=%d T=%d C=%d OC=%d", B, T, C, OC);
  if (C % BK != 0 || M64 <= 16 || (long long)C * 192 * 4 >= (1LL << 31)) {
    *tile_rows = *tile_cols = 0;  // not one of the tiled LDS-DMA kernels
    return GPT2HIP_OK;
  }
  const TileChoice c = plan_columns((int)M64, C, OC, false, 0).main;
  *tile_rows = c.bm;
  *tile_cols = c.bn;
  return GPT2HIP_OK;
}

size_t matmul_forward_argmax_workspace(int B, int T, int OC) {
  if (B < 1 || T < 1 || OC < 1) return 0;
  const size_t pairs = (size_t)((OC + g2::kArgmaxBN - 1) / g2::kArgmaxBN) * g2::kArgmaxWGN;
  return (size_t)B * T * pairs * 8;
}

int matmul_forward_argmax_status(int* ids, void* workspace, size_t workspace_bytes, const float* inp,
                                 const float* weight, const float* bias, int B, int T, int C,
                                 int OC) {
  return g2::argmax_dispatch(ids, workspace, workspace_bytes, inp, weight, bias, B, T, C, OC);
}

int matmul_forward_argmax_noalloc_status(int* ids, const float* inp, const float* weight,
                                         const float* bias, int B, int T, int C, int OC) {
  using namespace g2;
  const size_t need = matmul_forward_argmax_workspace(B, T, OC);
  if (need > sizeof(scratch))
    return fail(GPT2HIP_EINVAL,
                "matmul_forward_argmax_noalloc: B*T=%lld, OC=%d needs %zu bytes of pairs, the "
                "library's static scratch array holds %zu",
                (long long)B * T, OC, need, sizeof(scratch));
  void* ptr = nullptr;
  if (int rc = scratch_address(&ptr)) return rc;
  return argmax_dispatch(ids, ptr, sizeof(scratch), inp, weight, bias, B, T, C, OC);
}

size_t matmul_forward_splitk_workspace(void) {
  // counters + 512 partial tiles of the largest shape (two per compute unit)
  return GPT2HIP_SPLITK_COUNTER_BYTES + (size_t)512 * 128 * 192 * sizeof(float);
}

int matmul_forward_splitk_status(float* out, const float* inp, const float* weight, const float* bias,
                                 int B, int T, int C, int OC, int is_gelu, void* workspace,
                                 size_t workspace_bytes) {
  return g2::matmul_dispatch(out, inp, weight, bias, B, T, C, OC, is_gelu != 0, nullptr, nullptr,
                             workspace, workspace_bytes);
}

int matmul_forward_residual_status(float* out, const float* inp, const float* weight, const float* bias,
                                   const float* resid, int B, int T, int C, int OC, void* workspace,
                                   size_t workspace_bytes) {
  using namespace g2;
  if (!resid) return fail(GPT2HIP_EINVAL, "matmul_forward_residual: null residual");
  // the kernels read resid and write out through pointers they are told do not alias
  const unsigned long long bytes =
      (unsigned long long)(B > 0 ? B : 0) * (unsigned long long)(T > 0 ? T : 0) * (OC > 0 ? OC : 0) * sizeof(float);
  const uintptr_t o = reinterpret_cast<uintptr_t>(out), r = reinterpret_cast<uintptr_t>(resid);
  if (out && o < r + bytes && r < o + bytes)
    return fail(GPT2HIP_EINVAL, "matmul_forward_residual: out and resid overlap");
  return matmul_dispatch(out, inp, weight, bias, B, T, C, OC, false, nullptr, nullptr, workspace,
                         workspace_bytes, nullptr, resid);
}

int matmul_forward_splitk_forced_status(float* out, const float* inp, const float* weight,
                                        const float* bias, int B, int T, int C, int OC, int is_gelu,
                                        void* workspace, size_t workspace_bytes, int tile_rows,
                                        int tile_cols, int splits) {
  const g2::ForcedPlan plan{tile_rows, tile_cols, splits};
  return g2::matmul_dispatch(out, inp, weight, bias, B, T, C, OC, is_gelu != 0, nullptr, nullptr,
                             workspace, workspace_bytes, &plan);
}

int matmul_forward_splitk_plan(int B, int T, int C, int OC, size_t workspace_bytes, int* tile_rows,
                               int* tile_cols, int* splits) {
  using namespace g2;
  const long long M64 = (long long)B * T;
  if (B < 1 || T < 1 || C < 1 || OC < 1 || M64 > 0x7fffffffLL || !tile_rows || !tile_cols || !splits)
    return fail(GPT2HIP_EINVAL, "matmul_forward_splitk_plan: bad shape B=%d T=%d C=%d OC=%d", B, T, C, OC);
  if (C % BK != 0 || M64 <= 16 || (long long)C * 192 * 4 >= (1LL << 31)) {
    *tile_rows = *tile_cols = 0;  // not one of the tiled LDS-DMA kernels
    *splits = 1;
    return GPT2HIP_OK;
  }
  const TileChoice c = plan_columns((int)M64, C, OC, false, workspace_bytes).main;
  *tile_rows = c.bm;
  *tile_cols = c.bn;
  *splits = c.splits;
  return GPT2HIP_OK;
}

int matmul_forward_first_columns(int B, int T, int C, int OC, size_t workspace_bytes) {
  using namespace g2;
  const long long M64 = (long long)B * T;
  if (B < 1 || T < 1 || C < 1 || OC < 1 || M64 > 0x7fffffffLL) return 0;
  if (C % BK != 0 || M64 <= 16 || (long long)C * 192 * 4 >= (1LL << 31)) return OC;
  return plan_columns((int)M64, C, OC, false, workspace_bytes).main_cols;
}

int matmul_forward_gelu_status(float* out, const float* inp, const float* weight,
                               const float* bias, int B, int T, int C, int OC, int is_gelu) {
  const g2::ThreadWorkspace& w = g2::workspace_slot();
  return g2::matmul_dispatch(out, inp, weight, bias, B, T, C, OC, is_gelu != 0, nullptr, nullptr, w.ptr,
                             w.bytes);
}

void matmul_forward_gelu(float* out, const float* inp, const float* weight, const float* bias,
                         int B, int T, int C, int OC, int is_gelu) {
  if (matmul_forward_gelu_status(out, inp, weight, bias, B, T, C, OC, is_gelu))
    g2::die("matmul_forward_gelu");
}

}  // extern "C"
