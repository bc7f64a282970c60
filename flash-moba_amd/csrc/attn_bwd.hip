// Sparse attention backward over a CSC pattern, without a single global atomic.
//
//   bwd_prep_kernel      : delta[row] = sum_d dO*O (fp32).
//   attn_bwd_dkdv_kernel : COLUMN-stationary.  One workgroup per (64-key block, head,
//                          sequence) keeps K and V of the block in LDS and in operand
//                          registers and walks the block's ascending row list in gathered
//                          32-row tiles:
//                            S = Q K^T, dP = dO V^T             (A = gathered rows, B = K / V halves in registers)
//                            P = exp2(S*scale*log2e - LSE*log2e), dS = P o (dP - delta)
//                            dV^T += dO^T P, dK^T += Q^T dS     (P, dS feed the MFMA from registers;
//                                                                dO^T, Q^T via transposing LDS reads)
//                          dK/dV live in accumulator registers for the whole list and are written
//                          once.  The dS tiles (bf16) are streamed to a workspace indexed by the
//                          row-list position, i.e. written linearly per column.
//   attn_bwd_dq_kernel   : ROW-stationary.  One workgroup owns 128 consecutive query rows and
//                          their fp32 dQ accumulators in LDS; for every column it reads the
//                          contiguous slice of dS rows its superblock owns and adds dS K:
//                          dQ = scale * sum_columns dS K, one GEMM, no recomputation.
// In both kernels half of the waves compute and the other half only move data (global ->
// registers -> LDS) one to two steps ahead of the compute waves.  The dK/dV kernel runs four
// waves of 512 registers: a compute wave keeps 32 keys x head_dim of dK^T and dV^T plus its K and
// V operands in registers, which does not fit in the 256 registers an eight-wave workgroup gets.
#include "fmoba_common.h"

#include <type_traits>

namespace fmoba {

constexpr int kListCap = 4096;  // rows of a column list held in LDS at a time

template <int HD>
struct BwdSmem {
  static constexpr int LDQ = HD + 16;  // elements, K / V / Q / dO tiles
  static constexpr int LDS_ = 32 + 8;  // elements, per-wave dS^T tile [32 keys][32 rows]
  static constexpr size_t oK = 0;
  static constexpr size_t oV = oK + (size_t)64 * LDQ * 2;
  static constexpr size_t oQ = oV + (size_t)64 * LDQ * 2;          // [2 tile slots][32][LDQ]
  static constexpr size_t odO = oQ + (size_t)2 * 32 * LDQ * 2;
  static constexpr size_t odS = odO + (size_t)2 * 32 * LDQ * 2;    // [2 waves][32][LDS_]
  static constexpr size_t oRow = odS + (size_t)2 * 32 * LDS_ * 2;  // int[2][32]
  static constexpr size_t oLse = oRow + 2 * 32 * 4;
  static constexpr size_t oDelta = oLse + 2 * 32 * 4;
  static constexpr size_t oList = oDelta + 2 * 32 * 4;             // int[kListCap]
  static constexpr size_t mainBytes = oList + (size_t)kListCap * 4;
  static constexpr int LDR = HD + 4;  // floats, output transpose buffer [64 keys][LDR]
  static constexpr size_t redBytes = (size_t)64 * LDR * 4;
  static constexpr size_t bytes = mainBytes > redBytes ? mainBytes : redBytes;
};

__device__ __forceinline__ int lower_bound_i32b(const int32_t *p, int n, int v) {
  int lo = 0, hi = n;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (p[mid] < v)
      lo = mid + 1;
    else
      hi = mid;
  }
  return lo;
}

template <typename T, int HD>
__global__ __launch_bounds__(256) void attn_bwd_dkdv_kernel(fmoba_attn_bwd_args a, uint16_t *ds_ws) {
  typedef BwdSmem<HD> SM;
  constexpr int KS = HD / 16, LDQ = SM::LDQ, LDS_ = SM::LDS_, NDT = HD / 32, VPR = HD / 8, LDR = SM::LDR;
  constexpr int NV = 2 * 32 * VPR / 128;  // 16-byte vectors of the two gathered Q (or dO) tiles of a round per loader thread
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint16_t *sK = reinterpret_cast<uint16_t *>(smem + SM::oK);
  uint16_t *sV = reinterpret_cast<uint16_t *>(smem + SM::oV);
  uint16_t *sQ = reinterpret_cast<uint16_t *>(smem + SM::oQ);
  uint16_t *sdO = reinterpret_cast<uint16_t *>(smem + SM::odO);
  int *sRow = reinterpret_cast<int *>(smem + SM::oRow);
  float *sLse = reinterpret_cast<float *>(smem + SM::oLse);
  float *sDelta = reinterpret_cast<float *>(smem + SM::oDelta);
  int *sList = reinterpret_cast<int *>(smem + SM::oList);

  const int nb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int k0 = a.cu_seqlens_k[b], Lk = a.cu_seqlens_k[b + 1] - k0;
  const int key0 = nb * 64;
  if (key0 >= Lk) return;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int off = Lk - Lq;
  const int D = a.head_dim;
  const int hk = h / (a.heads / a.heads_k);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
  const bool is_loader = tid >= 128;
  const int lt = tid & 127;  // loader thread index
  const int kh = wave & 1;   // compute wave: key half
  const bool causal = a.is_causal != 0;
  const float scale_log2 = a.softmax_scale * 1.4426950408889634f;
  constexpr float kLog2e = 1.4426950408889634f;
  uint16_t *sdS = reinterpret_cast<uint16_t *>(smem + SM::odS) + (size_t)(wave & 1) * 32 * LDS_;

  // ---- the key block stays in LDS ---------------------------------------------------------
  {
    const uint16_t *kp = reinterpret_cast<const uint16_t *>(a.k) + (int64_t)(k0 + key0) * a.k_row_stride + (int64_t)hk * a.k_head_stride;
    const uint16_t *vp = reinterpret_cast<const uint16_t *>(a.v) + (int64_t)(k0 + key0) * a.v_row_stride + (int64_t)hk * a.v_head_stride;
    for (int v = tid; v < 64 * VPR; v += 256) {
      const int key = v / VPR, e = (v - key * VPR) * 8;
      Pack8 xk = zero_pack8(), xv = zero_pack8();
      if (key0 + key < Lk && e < D) {
        xk = ld_global16(kp + (int64_t)key * a.k_row_stride + e);
        xv = ld_global16(vp + (int64_t)key * a.v_row_stride + e);
      }
      *reinterpret_cast<Pack8 *>(sK + key * LDQ + e) = xk;
      *reinterpret_cast<Pack8 *>(sV + key * LDQ + e) = xv;
    }
  }
  __syncthreads();

  // ---- this block's column list --------------------------------------------------------------
  const int Bn = a.lg_block_n;
  const int c = key0 / Bn;
  const int koff = key0 - c * Bn;  // offset of this 64-key block inside its column
  const int64_t bh = (int64_t)b * a.heads + h;
  int nnz = 0;
  int64_t lbase = 0;
  int start = 0;
  if (c < a.max_cols) {
    nnz = a.col_nnz[bh * a.max_cols + c];
    lbase = a.col_offsets[bh * a.max_cols + c];
    // rows r with r + off < key0 see no key of this block
    if (causal && nnz > 0) start = lower_bound_i32b(a.row_indices + lbase, nnz, key0 - off);
  }
  const int32_t *list = a.row_indices + lbase;

  // K and V halves of this wave as MFMA B operands, for the whole list
  Pack8 kfr[KS], vfr[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    kfr[ks] = *reinterpret_cast<const Pack8 *>(sK + (kh * 32 + (lane & 31)) * LDQ + (hh * KS + ks) * 8);
    vfr[ks] = *reinterpret_cast<const Pack8 *>(sV + (kh * 32 + (lane & 31)) * LDQ + (hh * KS + ks) * 8);
  }
  f32x16 dv[NDT], dk[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      dv[dt][i] = 0.f;
      dk[dt][i] = 0.f;
    }

  const uint16_t *qg = reinterpret_cast<const uint16_t *>(a.q) + (int64_t)q0 * a.q_row_stride + (int64_t)h * a.q_head_stride;
  const uint16_t *dog = reinterpret_cast<const uint16_t *>(a.dout) + (int64_t)q0 * a.do_row_stride + (int64_t)h * a.do_head_stride;
  const float *lseg = a.softmax_lse + (int64_t)h * a.total_q + q0;
  const float *delg = a.softmax_d + (int64_t)h * ((int64_t)a.total_q + 128 * (int64_t)a.batch) + q0 + 128 * b;

  // loader state: two-deep rings (compile-time parity) of the gathered rows of two rounds
  Pack8 lq0[NV], lq1[NV], ld0[NV], ld1[NV];
  int lrow0 = -1, lrow1 = -1;
  float llse0 = INFINITY, llse1 = INFINITY, ldel0 = 0.f, ldel1 = 0.f;

  for (int seg0 = start; seg0 < nnz; seg0 += kListCap) {
    const int seg_len = min(kListCap, nnz - seg0);
    __syncthreads();
    for (int i = tid; i < seg_len; i += 256) {
      int r = list[seg0 + i];
      sList[i] = (r >= 0 && r < Lq) ? r : -1;  // rows outside the sequence (malformed pattern) are ignored
    }
    __syncthreads();
    const int ntile = (seg_len + 31) >> 5;
    const int nround = (ntile + 1) >> 1;

    auto load_round = [&](auto par, int r) {
      constexpr int P = decltype(par)::value;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int v = lt + 128 * i;
        const int row = v / VPR, e = (v - row * VPR) * 8;  // row 0..63 over the two tiles of the round
        const int j = r * 64 + row;
        const int rid = j < seg_len ? sList[j] : -1;
        Pack8 xq = zero_pack8(), xo = zero_pack8();
        if (rid >= 0 && e < D) {
          xq = ld_global16(qg + (int64_t)rid * a.q_row_stride + e);
          xo = ld_global16(dog + (int64_t)rid * a.do_row_stride + e);
        }
        if constexpr (P == 0) {
          lq0[i] = xq;
          ld0[i] = xo;
        } else {
          lq1[i] = xq;
          ld1[i] = xo;
        }
      }
      if (lt < 64) {
        const int j = r * 64 + lt;
        const int rid = j < seg_len ? sList[j] : -1;
        float xl = INFINITY, xd = 0.f;
        if (rid >= 0) {
          xl = lseg[rid];
          xd = delg[rid];
        }
        if constexpr (P == 0) {
          lrow0 = rid;
          llse0 = xl;
          ldel0 = xd;
        } else {
          lrow1 = rid;
          llse1 = xl;
          ldel1 = xd;
        }
      }
    };
    auto store_round = [&](auto par) {
      constexpr int P = decltype(par)::value;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int v = lt + 128 * i;
        const int row = v / VPR, e = (v - row * VPR) * 8;
        *reinterpret_cast<Pack8 *>(sQ + row * LDQ + e) = P == 0 ? lq0[i] : lq1[i];
        *reinterpret_cast<Pack8 *>(sdO + row * LDQ + e) = P == 0 ? ld0[i] : ld1[i];
      }
      if (lt < 64) {
        sRow[lt] = P == 0 ? lrow0 : lrow1;
        sLse[lt] = P == 0 ? llse0 : llse1;
        sDelta[lt] = P == 0 ? ldel0 : ldel1;
      }
    };

    auto process_tile = [&](int tile, int ts) {
      const uint16_t *tQ = sQ + ts * 32 * LDQ, *tdO = sdO + ts * 32 * LDQ;
      Pack8 qa[KS], doa[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        qa[ks] = *reinterpret_cast<const Pack8 *>(tQ + (lane & 31) * LDQ + (hh * KS + ks) * 8);
        doa[ks] = *reinterpret_cast<const Pack8 *>(tdO + (lane & 31) * LDQ + (hh * KS + ks) * 8);
      }
      f32x16 s, dp;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        s[i] = 0.f;
        dp[i] = 0.f;
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        s = mfma32<T>(qa[ks], kfr[ks], s);
        dp = mfma32<T>(doa[ks], vfr[ks], dp);
      }
      // this lane's key; register i <-> gathered row acc_row(i, hh)
      const int j = key0 + kh * 32 + (lane & 31);
      // key j is visible to row r iff r >= row_thr (rows that do not exist are stored as -1)
      const int row_thr = j >= Lk ? 0x7fffffff : (causal ? max(0, j - off) : 0);
      // register i holds gathered row acc_row(i, hh) = 8*(i/4) + 4*hh + i%4 of the tile
      float pr[16], ds[16];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int base = ts * 32 + 8 * g + 4 * hh;
        const f32x4 l4 = *reinterpret_cast<const f32x4 *>(sLse + base), d4 = *reinterpret_cast<const f32x4 *>(sDelta + base);
        const int4 r4 = *reinterpret_cast<const int4 *>(sRow + base);
        const int rr[4] = {r4.x, r4.y, r4.z, r4.w};
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int i = 4 * g + jj;
          const float x = rr[jj] >= row_thr ? fmaf(s[i], scale_log2, -l4[jj] * kLog2e) : -INFINITY;
          const float p = __builtin_amdgcn_exp2f(x);
          pr[i] = p;
          ds[i] = p * (dp[i] - d4[jj]);
        }
      }
      Pack8 pf[2], dsf[2];
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          pf[s2].w[w] = pack2<T>(pr[8 * s2 + 2 * w], pr[8 * s2 + 2 * w + 1]);
          dsf[s2].w[w] = pack2<T>(ds[8 * s2 + 2 * w], ds[8 * s2 + 2 * w + 1]);
        }
      // dS^T of this wave's 32 keys to its LDS tile [key][row], 4 rows per 8-byte store
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *reinterpret_cast<uint2 *>(sdS + (lane & 31) * LDS_ + 8 * g + 4 * hh) =
            make_uint2(pack2<T>(ds[4 * g], ds[4 * g + 1]), pack2<T>(ds[4 * g + 2], ds[4 * g + 3]));
      // dV^T[d][key] += dO^T[d][row] P[row][key];  dK^T[d][key] += Q^T[d][row] dS[row][key]
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        Pack8 dot[2], qt[2];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          dot[s2] = tr_frag8(tdO, LDQ, 16 * s2 + 4 * hh, 16 * s2 + 8 + 4 * hh, dt * 32, lane);
          qt[s2] = tr_frag8(tQ, LDQ, 16 * s2 + 4 * hh, 16 * s2 + 8 + 4 * hh, dt * 32, lane);
        }
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          dv[dt] = mfma32<T>(dot[s2], pf[s2], dv[dt]);
          dk[dt] = mfma32<T>(qt[s2], dsf[s2], dk[dt]);
        }
      }
      // dS rows of this tile to the workspace: lane (row, hh) holds 8 consecutive keys per step
      wave_lds_fence();
      const int myrow = sRow[ts * 32 + (lane & 31)];
      {
        // the transposing read exchanges data between lanes: every lane takes part, only the store is predicated
        Pack8 x[2];
#pragma unroll
        for (int s4 = 0; s4 < 2; ++s4) x[s4] = tr_frag8(sdS, LDS_, 16 * s4 + 8 * hh, 16 * s4 + 8 * hh + 4, 0, lane);
        if (myrow >= 0) {
          uint16_t *wp = ds_ws + (lbase + seg0 + tile * 32 + (lane & 31)) * Bn + koff + kh * 32;
#pragma unroll
          for (int s4 = 0; s4 < 2; ++s4) *reinterpret_cast<Pack8 *>(wp + 16 * s4 + 8 * hh) = x[s4];
        }
      }
      wave_lds_fence();
    };

    typedef std::integral_constant<int, 0> P0;
    typedef std::integral_constant<int, 1> P1;
    // The two roles run separate loops with the same barrier sequence, so that the loaders' rings
    // and the compute waves' operands do not add up in the register allocation.
    if (is_loader) {
      load_round(P0{}, 0);
      if (nround > 1) load_round(P1{}, 1);
      auto loader_round = [&](auto par, int r) {
        __syncthreads();  // the previous round's readers are done with the tile buffers
        store_round(par);
        __syncthreads();
        if (r + 2 < nround) load_round(par, r + 2);
      };
      for (int r = 0; r < nround; r += 2) {
        loader_round(P0{}, r);
        if (r + 1 < nround) loader_round(P1{}, r + 1);
      }
    } else {
      for (int r = 0; r < nround; ++r) {
        __syncthreads();
        __syncthreads();  // tiles 2r, 2r+1 are in LDS
        process_tile(2 * r, 0);
        if (2 * r + 1 < ntile) process_tile(2 * r + 1, 1);
      }
    }
  }

  // ---- dK^T / dV^T go through LDS to be written as rows, once ------------------------------------
  float *red = reinterpret_cast<float *>(smem);
  uint16_t *dkg = reinterpret_cast<uint16_t *>(a.dk) + (int64_t)(k0 + key0) * a.dk_row_stride + (int64_t)h * a.dk_head_stride;
  uint16_t *dvg = reinterpret_cast<uint16_t *>(a.dv) + (int64_t)(k0 + key0) * a.dv_row_stride + (int64_t)h * a.dv_head_stride;
#pragma unroll
  for (int which = 0; which < 2; ++which) {
    __syncthreads();
    if (!is_loader) {
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          f32x4 v4;
#pragma unroll
          for (int j = 0; j < 4; ++j) v4[j] = which == 0 ? dv[dt][4 * g + j] : dk[dt][4 * g + j];
          *reinterpret_cast<f32x4 *>(red + (size_t)(kh * 32 + (lane & 31)) * LDR + dt * 32 + 8 * g + 4 * hh) = v4;
        }
    }
    __syncthreads();
    const float mul = which == 0 ? 1.f : a.softmax_scale;
    uint16_t *og = which == 0 ? dvg : dkg;
    const int64_t ors = which == 0 ? a.dv_row_stride : a.dk_row_stride;
    for (int v = tid; v < 64 * VPR; v += 256) {
      const int key = v / VPR, e = (v - key * VPR) * 8;
      if (key0 + key >= Lk || e >= D) continue;
      const float *s0 = red + (size_t)key * LDR + e;
      Pack8 o;
#pragma unroll
      for (int w = 0; w < 4; ++w) o.w[w] = pack2<T>(s0[2 * w] * mul, s0[2 * w + 1] * mul);
      *reinterpret_cast<Pack8 *>(og + (int64_t)key * ors + e) = o;
    }
  }
}

// ------------------------------------------------------------------------------------
// dQ: row-stationary
// ------------------------------------------------------------------------------------
constexpr int kDqRows = 128;
constexpr int kDqColBatch = 256;
constexpr int kDqMaxSteps = 512;

template <int HD>
struct DqSmem {
  static constexpr int LDQ = HD + 16;  // elements, K tile
  static constexpr int LDA = HD + 4;   // floats, dQ accumulators
  static constexpr int LDD = 64 + 8;   // elements, dS rows [128][64 keys]
  static constexpr size_t oA = 0;
  static constexpr size_t oK = oA + (size_t)kDqRows * LDA * 4;     // [2][64][LDQ]
  static constexpr size_t oD = oK + (size_t)2 * 64 * LDQ * 2;      // [2][128][LDD]
  static constexpr size_t oRows = oD + (size_t)2 * kDqRows * LDD * 2;  // int[2][128]
  static constexpr size_t oLo = oRows + 2 * kDqRows * 4;
  static constexpr size_t oCnt = oLo + kDqColBatch * 4;
  static constexpr size_t oStep = oCnt + kDqColBatch * 4;
  static constexpr size_t oOff = oStep + kDqMaxSteps * 4;          // int64[kDqColBatch]
  static constexpr size_t oMisc = oOff + kDqColBatch * 8;
  static constexpr size_t bytes = oMisc + 64;
};

struct DqItem {
  int pair, sb;
};
__device__ __forceinline__ DqItem dq_decode_item(int id, int npairs, int nsb_max) {
  // all superblocks of a (sequence, head) pair on one XCD (pair p on XCD p % 8), late ones first
  const int x = id & 7, s = id >> 3;
  const int pl = s / nsb_max, sbi = s - pl * nsb_max;
  DqItem w;
  w.pair = pl * 8 + x;
  w.sb = nsb_max - 1 - sbi;
  if (w.pair >= npairs) w.pair = -1;
  return w;
}

template <typename T, int HD>
__global__ __launch_bounds__(512) void attn_bwd_dq_kernel(fmoba_attn_bwd_args a, const uint16_t *ds_ws, int nsb_max) {
  typedef DqSmem<HD> SM;
  constexpr int LDQ = SM::LDQ, LDA = SM::LDA, LDD = SM::LDD, NDT = HD / 32, VPR = HD / 8;
  constexpr int KVV = 64 * VPR / 256;  // K-tile vectors per loader thread
  constexpr int DVV = kDqRows * 8 / 256;  // dS-row vectors (64 keys = 8 vectors per row) per loader thread
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  float *sA = reinterpret_cast<float *>(smem + SM::oA);
  uint16_t *sK = reinterpret_cast<uint16_t *>(smem + SM::oK);
  uint16_t *sD = reinterpret_cast<uint16_t *>(smem + SM::oD);
  int *sRows = reinterpret_cast<int *>(smem + SM::oRows);
  int *sLo = reinterpret_cast<int *>(smem + SM::oLo);
  int *sCnt = reinterpret_cast<int *>(smem + SM::oCnt);
  int *sStep = reinterpret_cast<int *>(smem + SM::oStep);
  int64_t *sOff = reinterpret_cast<int64_t *>(smem + SM::oOff);
  int *sMisc = reinterpret_cast<int *>(smem + SM::oMisc);

  const DqItem wi = dq_decode_item(blockIdx.x, a.heads * a.batch, nsb_max);
  if (wi.pair < 0) return;
  const int b = wi.pair / a.heads, h = wi.pair - b * a.heads, sb = wi.sb;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int m0 = sb * kDqRows;
  if (m0 >= Lq) return;
  const int k0 = a.cu_seqlens_k[b], Lk = a.cu_seqlens_k[b + 1] - k0;
  const int rows_sb = min(kDqRows, Lq - m0);
  const int off = Lk - Lq;
  const int D = a.head_dim;
  const int hk = h / (a.heads / a.heads_k);
  const int Bn = a.lg_block_n, nsub = Bn / 64;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
  const bool is_loader = tid >= 256;
  const int ltid = tid & 255;
  const bool causal = a.is_causal != 0;

  for (int v = tid; v < kDqRows * LDA; v += 512) sA[v] = 0.f;

  int ncols = min((Lk + Bn - 1) / Bn, a.max_cols);
  const int last_rowpos = m0 + rows_sb - 1 + off;
  if (causal) ncols = last_rowpos < 0 ? 0 : min(ncols, last_rowpos / Bn + 1);
  const int64_t bh = (int64_t)b * a.heads + h;
  const int64_t *coff = a.col_offsets + bh * a.max_cols;
  const uint16_t *kp = reinterpret_cast<const uint16_t *>(a.k) + (int64_t)k0 * a.k_row_stride + (int64_t)hk * a.k_head_stride;
  const int cols_per_batch = min(kDqColBatch, kDqMaxSteps / nsub);

  Pack8 pk0[KVV], pk1[KVV], pd0[DVV], pd1[DVV];
  int prow0 = 0, prow1 = 0;

  for (int cb = 0; cb < ncols; cb += cols_per_batch) {
    const int cend = min(ncols, cb + cols_per_batch);
    __syncthreads();
    for (int c = cb + tid; c < cend; c += 512) {
      const int nnz = a.col_nnz[bh * a.max_cols + c];
      int lo = 0, cnt = 0;
      int64_t base = 0;
      if (nnz > 0) {
        base = coff[c];
        const int32_t *list = a.row_indices + base;
        lo = lower_bound_i32b(list, nnz, m0);
        const int hi = lo + lower_bound_i32b(list + lo, nnz - lo, m0 + kDqRows);
        cnt = min(hi - lo, kDqRows);
      }
      sLo[c - cb] = lo;
      sCnt[c - cb] = cnt;
      sOff[c - cb] = base + lo;
    }
    __syncthreads();
    if (wave == 0) {
      int nst = 0;
      for (int base = 0; base < (cend - cb) * nsub; base += 64) {
        const int idx = base + lane;
        const int cl = idx / nsub, kb = idx - cl * nsub;
        bool act = false;
        if (cl < cend - cb) {
          const int key0 = (cb + cl) * Bn + kb * 64;
          act = sCnt[cl] > 0 && key0 < Lk && !(causal && key0 > last_rowpos);
        }
        const unsigned long long m = __ballot(act);
        if (act) sStep[nst + __popcll(m & ((lane == 0) ? 0ull : (~0ull >> (64 - lane))))] = (cl << 8) | kb;
        nst += __popcll(m);
      }
      if (lane == 0) sMisc[0] = nst;
    }
    __syncthreads();
    const int nsteps = sMisc[0];
    if (nsteps == 0) continue;

    auto load_step = [&](auto par, int step) {
      constexpr int P = decltype(par)::value;
      const int code = sStep[step];
      const int cl = code >> 8, kb = code & 255;
      const int key0 = (cb + cl) * Bn + kb * 64;
      const int n = sCnt[cl];
      const int64_t pos0 = sOff[cl];
#pragma unroll
      for (int i = 0; i < KVV; ++i) {
        const int v = ltid + i * 256;
        const int key = v / VPR, e = (v - key * VPR) * 8;
        Pack8 x = zero_pack8();
        if (key0 + key < Lk && e < D) x = ld_global16(kp + (int64_t)(key0 + key) * a.k_row_stride + e);
        if constexpr (P == 0)
          pk0[i] = x;
        else
          pk1[i] = x;
      }
#pragma unroll
      for (int i = 0; i < DVV; ++i) {
        const int v = ltid + i * 256;
        const int row = v >> 3, e = (v & 7) * 8;
        Pack8 x = zero_pack8();
        if (row < n) x = ld_global16(ds_ws + (pos0 + row) * Bn + kb * 64 + e);
        if constexpr (P == 0)
          pd0[i] = x;
        else
          pd1[i] = x;
      }
      if (ltid < n) {
        const int rr = a.row_indices[pos0 + ltid];  // raw value: arithmetic here would wait for the load
        if constexpr (P == 0)
          prow0 = rr;
        else
          prow1 = rr;
      }
    };
    auto store_step = [&](auto par, int step) {
      constexpr int P = decltype(par)::value;
      const int buf = step & 1;
      const int code = sStep[step];
      const int n = sCnt[code >> 8];
      const int key0 = (cb + (code >> 8)) * Bn + (code & 255) * 64;
#pragma unroll
      for (int i = 0; i < KVV; ++i) {
        const int v = ltid + i * 256;
        const int key = v / VPR, e = (v - key * VPR) * 8;
        *reinterpret_cast<Pack8 *>(sK + ((size_t)buf * 64 + key) * LDQ + e) = P == 0 ? pk0[i] : pk1[i];
      }
#pragma unroll
      for (int i = 0; i < DVV; ++i) {
        const int v = ltid + i * 256;
        const int row = v >> 3, e = (v & 7) * 8;
        *reinterpret_cast<Pack8 *>(sD + ((size_t)buf * kDqRows + row) * LDD + e) = P == 0 ? pd0[i] : pd1[i];
      }
      if (ltid < kDqRows) {
        // the dK/dV pass wrote dS only for rows of this sequence that can see a key of the block
        const int rr = P == 0 ? prow0 : prow1;
        const bool ok = ltid < n && rr >= m0 && rr < m0 + rows_sb && !(causal && rr + off < key0);
        sRows[buf * kDqRows + ltid] = ok ? rr - m0 : -1;
      }
    };
    auto compute_step = [&](int step) {
      const int buf = step & 1;
      const int n = sCnt[sStep[step] >> 8];
      const uint16_t *tK = sK + (size_t)buf * 64 * LDQ;
      const int dt = wave % NDT;
      for (int tile = wave / NDT; tile * 32 < n; tile += 4 / NDT) {
        const int slot = tile * 32 + (lane & 31);
        const int rid = sRows[buf * kDqRows + slot];
        Pack8 df[4], kf[4];
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) {
          df[s4] = *reinterpret_cast<const Pack8 *>(sD + ((size_t)buf * kDqRows + slot) * LDD + 16 * s4 + 8 * hh);
          kf[s4] = tr_frag8(tK, LDQ, 16 * s4 + 8 * hh, 16 * s4 + 8 * hh + 4, dt * 32, lane);
        }
        f32x16 dq;
#pragma unroll
        for (int i = 0; i < 16; ++i) dq[i] = 0.f;
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) dq = mfma32<T>(kf[s4], df[s4], dq);  // dQ^T[d][row] += K^T[d][key] dS^T[key][row]
        if (rid >= 0 && rid < kDqRows) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            float *ap = sA + rid * LDA + dt * 32 + 8 * g + 4 * hh;
            f32x4 old = *reinterpret_cast<f32x4 *>(ap);
#pragma unroll
            for (int j = 0; j < 4; ++j) old[j] += dq[4 * g + j];
            *reinterpret_cast<f32x4 *>(ap) = old;
          }
        }
      }
    };

    typedef std::integral_constant<int, 0> P0;
    typedef std::integral_constant<int, 1> P1;
    // LDS is double buffered by step parity: while the compute waves work on step s the loaders
    // put step s+1 into the other buffer and then fetch step s+3 into the freed registers
    if (is_loader) {
      load_step(P0{}, 0);
      if (nsteps > 1) load_step(P1{}, 1);
      store_step(P0{}, 0);
      if (nsteps > 2) load_step(P0{}, 2);
    }
    auto run_step = [&](auto par, int step) {
      // par is the parity of step + 1 (the ring entry being stored during this step)
      __syncthreads();
      if (is_loader) {
        if (step + 1 < nsteps) {
          store_step(par, step + 1);
          if (step + 3 < nsteps) load_step(par, step + 3);
        }
      } else {
        compute_step(step);
      }
    };
    for (int step = 0; step < nsteps; step += 2) {
      run_step(P1{}, step);
      if (step + 1 < nsteps) run_step(P0{}, step + 1);
    }
  }
  __syncthreads();

  // dQ = scale * accumulator
  {
    uint16_t *op = reinterpret_cast<uint16_t *>(a.dq) + (int64_t)(q0 + m0) * a.dq_row_stride + (int64_t)h * a.dq_head_stride;
    for (int v = tid; v < rows_sb * VPR; v += 512) {
      const int row = v / VPR, e = (v - row * VPR) * 8;
      if (e >= D) continue;
      const float *src = sA + row * LDA + e;
      Pack8 o;
#pragma unroll
      for (int w = 0; w < 4; ++w) o.w[w] = pack2<T>(src[2 * w] * a.softmax_scale, src[2 * w + 1] * a.softmax_scale);
      *reinterpret_cast<Pack8 *>(op + (int64_t)row * a.dq_row_stride + e) = o;
    }
  }
}

// grid (ceil(max_seqlen_q / rows_per_block), heads, batch), block 256.
// LPR lanes cooperate on one row (LPR = power of two >= head_dim / 8).
template <typename T>
__global__ __launch_bounds__(256) void bwd_prep_kernel(fmoba_attn_bwd_args a, int LPR) {
  const int rows_per_block = 256 / LPR;
  const int h = blockIdx.y, b = blockIdx.z;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int r = blockIdx.x * rows_per_block + threadIdx.x / LPR;
  const int sub = threadIdx.x % LPR;
  const int e = sub * 8;
  const int D = a.head_dim;
  float acc = 0.f;
  if (r < Lq && e < D) {
    const Pack8 o = ld_global16(reinterpret_cast<const uint16_t *>(a.out) + (int64_t)(q0 + r) * a.o_row_stride + (int64_t)h * a.o_head_stride + e);
    const Pack8 g = ld_global16(reinterpret_cast<const uint16_t *>(a.dout) + (int64_t)(q0 + r) * a.do_row_stride + (int64_t)h * a.do_head_stride + e);
    float fo[8], fg[8];
    unpack8<T>(o, fo);
    unpack8<T>(g, fg);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc = fmaf(fo[i], fg[i], acc);
  }
  for (int o = LPR >> 1; o >= 1; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if (r < Lq && sub == 0) a.softmax_d[(int64_t)h * ((int64_t)a.total_q + 128 * (int64_t)a.batch) + q0 + 128 * b + r] = acc;
}

__global__ void zero_rows_kernel(void *p, int64_t rows, int64_t row_stride, int heads, int64_t head_stride, int D) {
  // zero a (rows, heads, D) 16-bit tensor with arbitrary row/head strides
  const int vpr = D / 8;
  const int64_t nvec = rows * heads * vpr;
  for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * blockDim.x) {
    const int64_t rh = v / vpr;
    const int e = (int)(v - rh * vpr) * 8;
    const int64_t row = rh / heads;
    const int h = (int)(rh - row * heads);
    *reinterpret_cast<Pack8 *>(reinterpret_cast<uint16_t *>(p) + row * row_stride + (int64_t)h * head_stride + e) = zero_pack8();
  }
}

__global__ void zero_f32_kernel(float *p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0.f;
}

template <typename T, int HD>
static int launch_dkdv(const fmoba_attn_bwd_args &a, uint16_t *ws, hipStream_t s) {
  auto kern = attn_bwd_dkdv_kernel<T, HD>;
  const size_t smem = BwdSmem<HD>::bytes;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("attn_bwd: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  dim3 grid(ceil_div(a.max_seqlen_k, 64), a.heads, a.batch);
  hipLaunchKernelGGL(kern, grid, dim3(256), smem, s, a, ws);
  return 0;
}

template <typename T, int HD>
static int launch_dq(const fmoba_attn_bwd_args &a, const uint16_t *ws, hipStream_t s) {
  auto kern = attn_bwd_dq_kernel<T, HD>;
  const size_t smem = DqSmem<HD>::bytes;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("attn_bwd: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  const int nsb_max = ceil_div(a.max_seqlen_q, kDqRows);
  const int64_t pairs_per_xcd = ((int64_t)a.heads * a.batch + 7) / 8;
  const int64_t items = 8 * pairs_per_xcd * nsb_max;
  if (items >= ((int64_t)1 << 31)) {
    set_error("attn_bwd: too many (sequence, head, superblock) work items");
    return 1;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)items), dim3(512), smem, s, a, ws, nsb_max);
  return 0;
}

template <typename T>
static int run_bwd(const fmoba_attn_bwd_args &a, uint16_t *ws, int phases, hipStream_t s) {
  if (phases & FMOBA_BWD_PREP) {
    int lpr = 1;
    while (lpr * 8 < a.head_dim) lpr <<= 1;
    const int rows_per_block = 256 / lpr;
    hipLaunchKernelGGL(bwd_prep_kernel<T>, dim3(ceil_div(a.max_seqlen_q, rows_per_block), a.heads, a.batch), dim3(256), 0, s, a, lpr);
  }
  if (phases & FMOBA_BWD_DKDV) {
    int rc = a.head_dim <= 64 ? launch_dkdv<T, 64>(a, ws, s) : launch_dkdv<T, 128>(a, ws, s);
    if (rc) return rc;
  }
  if (phases & FMOBA_BWD_DQ) {
    int rc = a.head_dim <= 64 ? launch_dq<T, 64>(a, ws, s) : launch_dq<T, 128>(a, ws, s);
    if (rc) return rc;
  }
  return 0;
}

}  // namespace fmoba

extern "C" size_t fmoba_attn_bwd_workspace_bytes(int64_t num_row_indices, int32_t lg_block_n) {
  if (num_row_indices <= 0 || lg_block_n <= 0) return 256;
  return (size_t)num_row_indices * lg_block_n * 2 + 256;
}

extern "C" int fmoba_attn_bwd(const fmoba_attn_bwd_args *a, void *stream) { return fmoba_attn_bwd_phases(a, 7, stream); }

extern "C" int fmoba_attn_bwd_phases(const fmoba_attn_bwd_args *a, int32_t phases, void *stream) {
  using namespace fmoba;
  FMOBA_REQUIRE(a != nullptr, "attn_bwd: null args");
  FMOBA_REQUIRE(phases > 0 && phases <= 7, "attn_bwd: phases must be a mask of bits 1, 2, 4");
  FMOBA_REQUIRE(a->dtype == FMOBA_DTYPE_F16 || a->dtype == FMOBA_DTYPE_BF16, "FlashMoBA only support fp16 and bf16 data type");
  FMOBA_REQUIRE(a->batch > 0, "batch size must be positive");
  FMOBA_REQUIRE(a->head_dim > 0 && a->head_dim % 8 == 0, "head_size should be a multiple of 8");
  FMOBA_REQUIRE(a->head_dim <= 256, "FlashMoBA backward only supports head dimension at most 256");
  FMOBA_REQUIRE(a->head_dim <= 128, "attn_bwd: head dimensions above 128 are not built yet (got %d)", a->head_dim);
  FMOBA_REQUIRE(a->heads > 0 && a->heads_k > 0 && a->heads % a->heads_k == 0, "Number of heads in key/value must divide number of heads in query");
  FMOBA_REQUIRE(a->lg_block_m % 64 == 0, "m_lg_block_dim must be a multiple of 64");
  FMOBA_REQUIRE(a->lg_block_n > 0 && a->lg_block_n % 64 == 0, "n_lg_block_dim must be a multiple of 64");
  FMOBA_REQUIRE(a->lg_block_n <= 64 * 256, "attn_bwd: n_lg_block_dim above 16384 is not supported");
  FMOBA_REQUIRE(a->total_q >= 0 && a->total_k >= 0 && a->max_seqlen_q >= 0 && a->max_seqlen_k >= 0 && a->max_cols >= 0 && a->num_row_indices >= 0,
                "negative size");
  FMOBA_REQUIRE(a->cu_seqlens_q && a->cu_seqlens_k, "attn_bwd: null cu_seqlens pointer");
  FMOBA_REQUIRE(a->batch <= 65535 && a->heads <= 65535, "attn_bwd: batch/heads too large for the launch grid");
  hipStream_t s = (hipStream_t)stream;
  const int64_t st[] = {a->q_row_stride,  a->q_head_stride,  a->k_row_stride,  a->k_head_stride,  a->v_row_stride,  a->v_head_stride,
                        a->o_row_stride,  a->o_head_stride,  a->do_row_stride, a->do_head_stride, a->dq_row_stride, a->dq_head_stride,
                        a->dk_row_stride, a->dk_head_stride, a->dv_row_stride, a->dv_head_stride};
  for (int64_t x : st) FMOBA_REQUIRE(x % 8 == 0, "attn_bwd: strides must be multiples of 8 elements");
  const void *ptrs[] = {a->dout, a->q, a->k, a->v, a->out, a->dq, a->dk, a->dv};
  for (const void *p : ptrs) FMOBA_REQUIRE(((uintptr_t)p % 16) == 0, "attn_bwd: tensors must be 16-byte aligned");

  if (a->total_k > 0) {
    FMOBA_REQUIRE(a->dk && a->dv, "attn_bwd: null dk/dv");
    if (a->max_seqlen_q == 0 || a->total_q == 0 || a->max_cols == 0) {
      // no query rows: dk = dv = 0 (csrc/flash_moba/flash_moba_api.cpp:834-839)
      hipLaunchKernelGGL(zero_rows_kernel, dim3(1024), dim3(256), 0, s, a->dk, (int64_t)a->total_k, a->dk_row_stride, a->heads, a->dk_head_stride, a->head_dim);
      hipLaunchKernelGGL(zero_rows_kernel, dim3(1024), dim3(256), 0, s, a->dv, (int64_t)a->total_k, a->dv_row_stride, a->heads, a->dv_head_stride, a->head_dim);
    }
  }
  if (a->total_q == 0 || a->max_seqlen_q == 0) {
    if (a->softmax_d) hipLaunchKernelGGL(zero_f32_kernel, dim3(64), dim3(256), 0, s, a->softmax_d, (int64_t)a->heads * ((int64_t)a->total_q + 128 * (int64_t)a->batch));
    FMOBA_LAUNCH_CHECK("attn_bwd(no rows)");
    return 0;
  }
  FMOBA_REQUIRE(a->dout && a->q && a->out && a->softmax_lse && a->dq && a->softmax_d, "attn_bwd: null pointer");
  if (phases & FMOBA_BWD_PREP)
    hipLaunchKernelGGL(zero_f32_kernel, dim3(256), dim3(256), 0, s, a->softmax_d, (int64_t)a->heads * ((int64_t)a->total_q + 128 * (int64_t)a->batch));
  if (a->total_k == 0 || a->max_seqlen_k == 0 || a->max_cols == 0) {
    // no keys: dq = 0
    hipLaunchKernelGGL(zero_rows_kernel, dim3(1024), dim3(256), 0, s, a->dq, (int64_t)a->total_q, a->dq_row_stride, a->heads, a->dq_head_stride, a->head_dim);
    FMOBA_LAUNCH_CHECK("attn_bwd(no keys)");
    return 0;
  }
  FMOBA_REQUIRE(a->k && a->v && a->col_offsets && a->col_nnz && a->row_indices, "attn_bwd: null k/v/CSC pointer");
  FMOBA_REQUIRE(a->workspace != nullptr && a->workspace_bytes >= fmoba_attn_bwd_workspace_bytes(a->num_row_indices, a->lg_block_n),
                "attn_bwd: workspace too small");
  uint16_t *ws = reinterpret_cast<uint16_t *>(((uintptr_t)a->workspace + 255) & ~(uintptr_t)255);
  int rc = a->dtype == FMOBA_DTYPE_BF16 ? run_bwd<bf16_t>(*a, ws, phases, s) : run_bwd<f16_t>(*a, ws, phases, s);
  if (rc) return rc;
  FMOBA_LAUNCH_CHECK("attn_bwd");
  return 0;
}
