// Sparse (gather-and-densify) flash attention forward over a CSC pattern.
//
// One workgroup owns a SUPERBLOCK of 128 consecutive query rows of one (sequence, head).
// The superblock's Q rows (bf16), its fp32 output accumulators and its running softmax
// statistics stay in LDS for the whole kernel; nothing partial is ever written to HBM.
// For every key chunk the rows of the superblock that selected it are found in the
// chunk's ascending row list, gathered from LDS into dense 32-row MFMA tiles and
// processed with S^T = K Q^T (so that one lane owns one query row: the online-softmax
// reductions are in-register) followed by O^T += V^T P^T, where V^T fragments come from
// transposing LDS reads and P^T goes from the S^T accumulators straight into the MFMA
// operand registers.
#include "fmoba_common.h"

#include <type_traits>

namespace fmoba {

constexpr int kSuperRows = 128;
constexpr int kColBatch = 256;   // columns whose list ranges are resolved per batch
constexpr int kMaxSteps = 512;   // (column, 64-key block) steps per batch

template <int HD>
struct FwdSmem {
  static constexpr int LDQ = HD + 16;  // elements, Q / K / V tiles
  static constexpr int LDO = HD + 4;   // floats, output accumulators
  static constexpr int LDP = 64 + 8;   // elements, probability tile [32 rows][64 keys]
  static constexpr size_t oO = 0;
  static constexpr size_t oQ = oO + (size_t)kSuperRows * LDO * 4;
  static constexpr size_t oK = oQ + (size_t)kSuperRows * LDQ * 2;
  static constexpr size_t oV = oK + (size_t)64 * LDQ * 2;
  static constexpr size_t oP = oV + (size_t)64 * LDQ * 2;          // [2][32][LDP]
  static constexpr size_t oM = oP + (size_t)2 * 32 * LDP * 2;
  static constexpr size_t oL = oM + kSuperRows * 4;
  static constexpr size_t oRows = oL + kSuperRows * 4;             // int[2][kSuperRows]
  static constexpr size_t oAlpha = oRows + 2 * kSuperRows * 4;     // float[2][32]
  static constexpr size_t oRid = oAlpha + 2 * 32 * 4;              // int[2][32]
  static constexpr size_t oLo = oRid + 2 * 32 * 4;                 // int[kColBatch]
  static constexpr size_t oCnt = oLo + kColBatch * 4;              // int[kColBatch]
  static constexpr size_t oStep = oCnt + kColBatch * 4;            // int[kMaxSteps]: (column - batch start) << 8 | key block
  static constexpr size_t oOff = oStep + kMaxSteps * 4;            // int64[kColBatch]: list position of the first entry
  static constexpr size_t oMisc = oOff + kColBatch * 8;            // int[16]
  static constexpr size_t bytes = oMisc + 64;
};

__device__ __forceinline__ int lower_bound_i32(const int32_t *p, int n, int v) {
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

// Work items are (sequence, head, superblock).  Hardware deals consecutive workgroup ids
// round-robin to the 8 XCDs, each with its own L2.  The id is decoded so that all
// superblocks of one (sequence, head) pair run on ONE XCD (pair p lives on XCD p % 8) and
// consecutively, so that their K/V re-reads hit that XCD's L2; inside a pair the late
// superblocks (most key chunks, longest running) are issued first.
struct WorkItem {
  int pair, sb;
};
__device__ __forceinline__ WorkItem decode_item(int id, int npairs, int nsb_max) {
  const int x = id & 7, s = id >> 3;
  const int pl = s / nsb_max, sbi = s - pl * nsb_max;
  WorkItem w;
  w.pair = pl * 8 + x;
  w.sb = nsb_max - 1 - sbi;
  if (w.pair >= npairs) w.pair = -1;
  return w;
}

// The four waves of a workgroup form a two-stage pipeline over gathered 32-row tiles:
//   waves 0,1 ("score" stage, 16 rows each): gather Q rows from LDS, S^T = K Q^T on
//       16x16x32 MFMAs (one lane group of 4 owns one query row), causal/length mask, online
//       softmax statistics (kept in LDS per superblock row), probabilities -> LDS as bf16;
//   waves 2,3 ("value" stage, 64 output columns each): O^T += V^T P^T on 32x32x16 MFMAs
//       (V^T through transposing LDS reads), then read-modify-write of the fp32 output rows.
// In slot k the score stage works on tile k while the value stage works on tile k-1, so the
// four SIMDs are busy even when a key chunk has a single tile.  Row statistics are only
// touched by the score stage and output rows only by the value stage, both in tile order,
// so results do not depend on timing.
template <typename T, int HD>
__global__ __launch_bounds__(512) void attn_fwd_kernel(fmoba_attn_fwd_args a, int nsb_max) {
  typedef FwdSmem<HD> SM;
  constexpr int LDQ = SM::LDQ, LDO = SM::LDO, LDP = SM::LDP, NDT = HD / 32, VPR = HD / 8;
  constexpr int KS4 = HD / 32;         // k-steps of a 16x16x32 MFMA over the head dimension
  constexpr int KVV = 64 * VPR / 256;  // 16-byte vectors of a K (or V) tile per thread
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  float *sO = reinterpret_cast<float *>(smem + SM::oO);
  uint16_t *sQ = reinterpret_cast<uint16_t *>(smem + SM::oQ);
  uint16_t *sK = reinterpret_cast<uint16_t *>(smem + SM::oK);
  uint16_t *sV = reinterpret_cast<uint16_t *>(smem + SM::oV);
  uint16_t *sP = reinterpret_cast<uint16_t *>(smem + SM::oP);
  float *sM = reinterpret_cast<float *>(smem + SM::oM);
  float *sL = reinterpret_cast<float *>(smem + SM::oL);
  int *sRows = reinterpret_cast<int *>(smem + SM::oRows);
  float *sAlpha = reinterpret_cast<float *>(smem + SM::oAlpha);
  int *sRid = reinterpret_cast<int *>(smem + SM::oRid);
  int *sLo = reinterpret_cast<int *>(smem + SM::oLo);
  int *sCnt = reinterpret_cast<int *>(smem + SM::oCnt);
  int *sStep = reinterpret_cast<int *>(smem + SM::oStep);
  int *sMisc = reinterpret_cast<int *>(smem + SM::oMisc);
  int64_t *sOff = reinterpret_cast<int64_t *>(smem + SM::oOff);

  const WorkItem wi = decode_item(blockIdx.x, a.heads * a.batch, nsb_max);
  if (wi.pair < 0) return;
  const int b = wi.pair / a.heads, h = wi.pair - b * a.heads, sb = wi.sb;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int m0 = sb * kSuperRows;
  if (m0 >= Lq) return;
  const int k0 = a.cu_seqlens_k[b], Lk = a.cu_seqlens_k[b + 1] - k0;
  const int rows_sb = min(kSuperRows, Lq - m0);
  const int off = Lk - Lq;
  const int D = a.head_dim;
  const int hk = h / (a.heads / a.heads_k);
  const int Bn = a.lg_block_n;
  const int nsub = Bn / 64;
  // waves 0,1: score stage; waves 2,3: value stage; waves 4..7: loaders (global -> registers -> LDS)
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
  const bool is_loader = tid >= 256;
  const int ltid = tid & 255;
  const float scale_log2 = a.softmax_scale * 1.4426950408889634f;
  const bool causal = a.is_causal != 0;

  // ---- superblock state -------------------------------------------------------------
  {
    const uint16_t *qp = reinterpret_cast<const uint16_t *>(a.q) + (int64_t)(q0 + m0) * a.q_row_stride + (int64_t)h * a.q_head_stride;
    for (int v = tid; v < kSuperRows * VPR; v += 512) {
      const int row = v / VPR, e = (v - row * VPR) * 8;
      Pack8 x = zero_pack8();
      if (row < rows_sb && e < D) x = ld_global16(qp + (int64_t)row * a.q_row_stride + e);
      *reinterpret_cast<Pack8 *>(sQ + row * LDQ + e) = x;
    }
    for (int v = tid; v < kSuperRows * LDO; v += 512) sO[v] = 0.f;
    if (tid < kSuperRows) {
      sM[tid] = -INFINITY;
      sL[tid] = 0.f;
    }
  }

  int ncols = min((Lk + Bn - 1) / Bn, a.max_cols);
  const int last_rowpos = m0 + rows_sb - 1 + off;  // largest visible key index of the superblock (causal)
  if (causal) ncols = last_rowpos < 0 ? 0 : min(ncols, last_rowpos / Bn + 1);
  const int64_t bh = (int64_t)b * a.heads + h;
  const int64_t *coff = a.col_offsets + bh * a.max_cols;
  const uint16_t *kp = reinterpret_cast<const uint16_t *>(a.k) + (int64_t)k0 * a.k_row_stride + (int64_t)hk * a.k_head_stride;
  const uint16_t *vp = reinterpret_cast<const uint16_t *>(a.v) + (int64_t)k0 * a.v_row_stride + (int64_t)hk * a.v_head_stride;
  const int cols_per_batch = min(kColBatch, kMaxSteps / nsub);

  // Two-deep register rings carry the K tiles (+ row lists) and, separately, the V tiles of
  // the next two steps from global memory to LDS, so that a load has two pipeline slots to
  // complete.  Ring entries are picked by compile-time parity (no dynamic register indexing).
  Pack8 pk0[KVV], pk1[KVV], pv0[KVV], pv1[KVV];
  int prow0 = 0, prow1 = 0;
  auto step_key0 = [&](int cb, int step) {
    const int code = sStep[step];
    return (cb + (code >> 8)) * Bn + (code & 255) * 64;
  };
  auto load_tile = [&](Pack8(&dst)[KVV], const uint16_t *base, int64_t row_stride, int key0) {
#pragma unroll
    for (int i = 0; i < KVV; ++i) {
      const int v = ltid + i * 256;
      const int key = v / VPR, e = (v - key * VPR) * 8;
      dst[i] = zero_pack8();
      if (key0 + key < Lk && e < D) dst[i] = ld_global16(base + (int64_t)(key0 + key) * row_stride + e);
    }
  };
  auto store_tile = [&](const Pack8(&src)[KVV], uint16_t *dst) {
#pragma unroll
    for (int i = 0; i < KVV; ++i) {
      const int v = ltid + i * 256;
      const int key = v / VPR, e = (v - key * VPR) * 8;
      *reinterpret_cast<Pack8 *>(dst + key * LDQ + e) = src[i];
    }
  };
  auto load_k = [&](auto par, int cb, int step) {
    const int cl = sStep[step] >> 8;
    if constexpr (decltype(par)::value == 0) {
      load_tile(pk0, kp, a.k_row_stride, step_key0(cb, step));
      if (ltid < sCnt[cl]) prow0 = a.row_indices[sOff[cl] + ltid];  // raw value: any arithmetic here would wait for the load
    } else {
      load_tile(pk1, kp, a.k_row_stride, step_key0(cb, step));
      if (ltid < sCnt[cl]) prow1 = a.row_indices[sOff[cl] + ltid];
    }
  };
  auto load_v = [&](auto par, int cb, int step) {
    if constexpr (decltype(par)::value == 0)
      load_tile(pv0, vp, a.v_row_stride, step_key0(cb, step));
    else
      load_tile(pv1, vp, a.v_row_stride, step_key0(cb, step));
  };
  auto store_k = [&](auto par, int step, int n) {
    if constexpr (decltype(par)::value == 0) {
      store_tile(pk0, sK);
      if (ltid < n) sRows[(step & 1) * kSuperRows + ltid] = prow0 - m0;
    } else {
      store_tile(pk1, sK);
      if (ltid < n) sRows[(step & 1) * kSuperRows + ltid] = prow1 - m0;
    }
  };
  auto store_v = [&](auto par) {
    if constexpr (decltype(par)::value == 0)
      store_tile(pv0, sV);
    else
      store_tile(pv1, sV);
  };

  // ---- score stage: one 16-row half of a tile ----------------------------------------------
  auto score_stage = [&](int step, int key0, int n, int tile, int buf) {
    const int l16 = lane & 15, g = lane >> 4;
    const int slot = 16 * wave + l16;              // row slot inside the 32-row tile
    const int ridx = tile * 32 + slot;
    const bool valid = ridx < n;
    const int rid = valid ? (sRows[(step & 1) * kSuperRows + ridx] & (kSuperRows - 1)) : 0;
    Pack8 qf[KS4];
#pragma unroll
    for (int ks = 0; ks < KS4; ++ks) qf[ks] = *reinterpret_cast<const Pack8 *>(sQ + rid * LDQ + (g * KS4 + ks) * 8);
    // S^T: register i of key tile kt holds key key0 + 16*kt + 4*g + i for this lane's row.
    // All K fragments are fetched from LDS before the first MFMA so that the LDS round trips
    // overlap instead of preceding each MFMA.
    Pack8 kf[KS4][4];
#pragma unroll
    for (int ks = 0; ks < KS4; ++ks)
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
        kf[ks][kt] = *reinterpret_cast<const Pack8 *>(sK + (kt * 16 + l16) * LDQ + (g * KS4 + ks) * 8);
    f32x4 s[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) s[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS4; ++ks) {
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) s[kt] = mfma16<T>(kf[ks][kt], qf[ks], s[kt]);
    }
    const int rowpos = m0 + rid + off;
    float mloc = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = key0 + kt * 16 + 4 * g + i;
        const bool vis = valid && j < Lk && (!causal || j <= rowpos);
        const float x = vis ? s[kt][i] * scale_log2 : -INFINITY;
        s[kt][i] = x;
        mloc = fmaxf(mloc, x);
      }
    mloc = max_rows4_f(mloc);
    const float m_old = sM[rid], l_old = sL[rid];
    const float m_new = fmaxf(m_old, mloc);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_old - m_use);
    float rowsum = 0.f;
    uint16_t *prow_p = sP + ((size_t)buf * 32 + slot) * LDP;
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      float pr[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        pr[i] = __builtin_amdgcn_exp2f(s[kt][i] - m_use);
        rowsum += pr[i];
      }
      *reinterpret_cast<uint2 *>(prow_p + kt * 16 + 4 * g) = make_uint2(pack2<T>(pr[0], pr[1]), pack2<T>(pr[2], pr[3]));
    }
    rowsum = sum_rows4_f(rowsum);
    if (g == 0) {
      if (valid) {
        sM[rid] = m_new;
        sL[rid] = l_old * alpha + rowsum;
      }
      sAlpha[buf * 32 + slot] = alpha;
      sRid[buf * 32 + slot] = valid ? rid : -1;
    }
  };

  // ---- value stage: 64 output columns of a tile ------------------------------------------------
  auto value_stage = [&](int buf) {
    const int slot = lane & 31;
    const int rid = sRid[buf * 32 + slot];
    const float alpha = sAlpha[buf * 32 + slot];
    Pack8 pf[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) pf[ks] = *reinterpret_cast<const Pack8 *>(sP + ((size_t)buf * 32 + slot) * LDP + 16 * ks + 8 * hh);
#pragma unroll
    for (int d2 = 0; d2 < NDT / 2; ++d2) {
      const int dt = (wave - 2) * (NDT / 2) + d2;
      Pack8 vf[4];
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) vf[ks] = tr_frag8(sV, LDQ, 16 * ks + 8 * hh, 16 * ks + 8 * hh + 4, dt * 32, lane);
      f32x16 o;
#pragma unroll
      for (int i = 0; i < 16; ++i) o[i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) o = mfma32<T>(vf[ks], pf[ks], o);
      if (rid >= 0) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          float *op = sO + rid * LDO + dt * 32 + 8 * g + 4 * hh;
          f32x4 old = *reinterpret_cast<f32x4 *>(op);
          f32x4 nw;
#pragma unroll
          for (int j = 0; j < 4; ++j) nw[j] = old[j] * alpha + o[4 * g + j];
          *reinterpret_cast<f32x4 *>(op) = nw;
        }
      }
    }
  };

  for (int cb = 0; cb < ncols; cb += cols_per_batch) {
    const int cend = min(ncols, cb + cols_per_batch);
    __syncthreads();
    // rows of this superblock inside each column's ascending list
    for (int c = cb + tid; c < cend; c += 512) {
      const int nnz = a.col_nnz[bh * a.max_cols + c];
      int lo = 0, cnt = 0;
      int64_t base = 0;
      if (nnz > 0) {
        base = coff[c];
        const int32_t *list = a.row_indices + base;
        lo = lower_bound_i32(list, nnz, m0);
        const int hi = lo + lower_bound_i32(list + lo, nnz - lo, m0 + kSuperRows);
        cnt = min(hi - lo, kSuperRows);
      }
      sLo[c - cb] = lo;
      sCnt[c - cb] = cnt;
      sOff[c - cb] = base + lo;
    }
    __syncthreads();
    // ordered list of the (column, 64-key block) steps that have work
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
    typedef std::integral_constant<int, 0> P0;
    typedef std::integral_constant<int, 1> P1;
    if (is_loader) {
      load_k(P0{}, cb, 0);
      load_v(P0{}, cb, 0);
      if (nsteps > 1) {
        load_k(P1{}, cb, 1);
        load_v(P1{}, cb, 1);
      }
    }

    // slot loop: the value stage lags the score stage by one tile
    int slot_id = 0;
    bool prev_valid = false, prev_first = false;
    auto run_step = [&](auto par, int step) {
      typedef std::integral_constant<int, 1 - decltype(par)::value> Other;
      const int n = sCnt[sStep[step] >> 8];
      const int key0 = step_key0(cb, step);
      const int ntile = (n + 31) >> 5;
      for (int tile = 0; tile < ntile; ++tile) {
        __syncthreads();  // every read of the previous slot is done
        // loader waves: LDS stores of this boundary; after the second barrier they issue the
        // global loads for two steps ahead while the compute waves run their stages
        const bool v_other = tile == 0 && prev_valid && prev_first;  // previous step had one tile: its V goes in now
        if (is_loader) {
          if (tile == 0) store_k(par, step, n);
          if (v_other) store_v(Other{});
          if (tile == 1) store_v(par);                                // V of this step, one slot after its K
        }
        __syncthreads();
        if (is_loader) {
          if (tile == 0 && step + 2 < nsteps) load_k(par, cb, step + 2);
          if (v_other && step + 1 < nsteps) load_v(Other{}, cb, step + 1);
          if (tile == 1 && step + 2 < nsteps) load_v(par, cb, step + 2);
        } else if (wave < 2) {
          score_stage(step, key0, n, tile, slot_id & 1);
        } else if (prev_valid) {
          value_stage((slot_id - 1) & 1);
        }
        prev_valid = true;
        prev_first = tile == 0;
        ++slot_id;
      }
    };
    for (int step = 0; step < nsteps; step += 2) {
      run_step(P0{}, step);
      if (step + 1 < nsteps) run_step(P1{}, step + 1);
    }
    // drain: value stage of the last tile
    __syncthreads();
    if (is_loader && prev_valid && prev_first) {
      if ((nsteps - 1) & 1)
        store_v(P1{});
      else
        store_v(P0{});
    }
    __syncthreads();
    if ((wave == 2 || wave == 3) && prev_valid) value_stage((slot_id - 1) & 1);
  }
  __syncthreads();

  // ---- epilogue: normalise, write out and the log-sum-exp -----------------------------
  {
    uint16_t *op = reinterpret_cast<uint16_t *>(a.out) + (int64_t)(q0 + m0) * a.o_row_stride + (int64_t)h * a.o_head_stride;
    for (int v = tid; v < rows_sb * VPR; v += 512) {
      const int row = v / VPR, e = (v - row * VPR) * 8;
      if (e >= D) continue;
      const float l = sL[row];
      const float inv = (l == 0.f || l != l) ? 1.f : 1.f / l;
      const float *src = sO + row * LDO + e;
      Pack8 o;
#pragma unroll
      for (int w = 0; w < 4; ++w) o.w[w] = pack2<T>(src[2 * w] * inv, src[2 * w + 1] * inv);
      *reinterpret_cast<Pack8 *>(op + (int64_t)row * a.o_row_stride + e) = o;
    }
    if (tid < rows_sb) {
      const float l = sL[tid], m = sM[tid];
      const float lse = (l == 0.f || l != l) ? INFINITY : m * 0.6931471805599453f + logf(l);
      a.softmax_lse[(int64_t)h * a.total_q + q0 + m0 + tid] = lse;
    }
  }
}

__global__ void fwd_empty_kernel(void *out, float *lse, int64_t n_out_words, int64_t n_lse) {
  const int64_t i0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, st = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = i0; i < n_out_words; i += st) reinterpret_cast<uint32_t *>(out)[i] = 0u;
  for (int64_t i = i0; i < n_lse; i += st) lse[i] = INFINITY;
}

template <typename T, int HD>
static int launch_fwd(const fmoba_attn_fwd_args &a, hipStream_t s) {
  auto kern = attn_fwd_kernel<T, HD>;
  const size_t smem = FwdSmem<HD>::bytes;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("attn_fwd: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  const int nsb_max = ceil_div(a.max_seqlen_q, kSuperRows);
  const int64_t pairs_per_xcd = ((int64_t)a.heads * a.batch + 7) / 8;
  const int64_t items = 8 * pairs_per_xcd * nsb_max;
  if (items >= ((int64_t)1 << 31)) {
    set_error("attn_fwd: too many (sequence, head, superblock) work items");
    return 1;
  }
  dim3 grid((unsigned)items);
  hipLaunchKernelGGL(kern, grid, dim3(512), smem, s, a, nsb_max);
  return 0;
}

}  // namespace fmoba

extern "C" int fmoba_attn_fwd(const fmoba_attn_fwd_args *a, void *stream) {
  using namespace fmoba;
  FMOBA_REQUIRE(a != nullptr, "attn_fwd: null args");
  FMOBA_REQUIRE(a->dtype == FMOBA_DTYPE_F16 || a->dtype == FMOBA_DTYPE_BF16, "FlashMoBA only support fp16 and bf16 data type");
  FMOBA_REQUIRE(a->batch > 0, "batch size must be positive");
  FMOBA_REQUIRE(a->head_dim > 0 && a->head_dim <= 256, "FlashMoBA forward only supports head dimension at most 256");
  FMOBA_REQUIRE(a->head_dim % 8 == 0, "query, key, value, and out_ must have a head_size that is a multiple of 8");
  FMOBA_REQUIRE(a->head_dim <= 128, "attn_fwd: head dimensions above 128 are not built yet (got %d)", a->head_dim);
  FMOBA_REQUIRE(a->heads > 0 && a->heads_k > 0 && a->heads % a->heads_k == 0, "Number of heads in key/value must divide number of heads in query");
  FMOBA_REQUIRE(a->lg_block_m >= 128 && a->lg_block_m <= 1024, "m_lg_block_dim must be at least 128 and at most 1024");
  FMOBA_REQUIRE(a->lg_block_m % 64 == 0, "m_lg_block_dim must be a multiple of 64");
  FMOBA_REQUIRE(a->lg_block_n > 0 && a->lg_block_n % 64 == 0, "n_lg_block_dim must be a multiple of 64");
  FMOBA_REQUIRE(a->lg_block_n <= 64 * 256, "attn_fwd: n_lg_block_dim above 16384 is not supported");
  FMOBA_REQUIRE(a->total_q >= 0 && a->total_k >= 0 && a->max_seqlen_q >= 0 && a->max_seqlen_k >= 0 && a->max_cols >= 0, "negative size");
  FMOBA_REQUIRE(a->cu_seqlens_q && a->cu_seqlens_k, "attn_fwd: null cu_seqlens pointer");
  FMOBA_REQUIRE(a->batch <= 65535 && a->heads <= 65535, "attn_fwd: batch/heads too large for the launch grid");
  hipStream_t s = (hipStream_t)stream;
  if (a->total_q == 0 || a->max_seqlen_q == 0) return 0;
  FMOBA_REQUIRE(a->q && a->out && a->softmax_lse, "attn_fwd: null q/out/lse pointer");
  if (a->max_seqlen_k == 0 || a->total_k == 0 || a->max_cols == 0) {
    // no keys: out = 0, lse = +inf (csrc/flash_moba/flash_moba_api.cpp:589-593); needs a dense out
    FMOBA_REQUIRE(a->o_head_stride == a->head_dim && a->o_row_stride == (int64_t)a->heads * a->head_dim,
                  "attn_fwd: out must be contiguous when there are no keys");
    hipLaunchKernelGGL(fwd_empty_kernel, dim3(512), dim3(256), 0, s, a->out, a->softmax_lse,
                       (int64_t)a->total_q * a->heads * a->head_dim / 2, (int64_t)a->total_q * a->heads);
    FMOBA_LAUNCH_CHECK("attn_fwd(empty)");
    return 0;
  }
  FMOBA_REQUIRE(a->k && a->v && a->col_offsets && a->col_nnz && a->row_indices, "attn_fwd: null k/v/CSC pointer");
  const int64_t st[] = {a->q_row_stride, a->q_head_stride, a->k_row_stride, a->k_head_stride,
                        a->v_row_stride, a->v_head_stride, a->o_row_stride, a->o_head_stride};
  for (int64_t x : st) FMOBA_REQUIRE(x % 8 == 0, "attn_fwd: strides must be multiples of 8 elements");
  FMOBA_REQUIRE(((uintptr_t)a->q % 16) == 0 && ((uintptr_t)a->k % 16) == 0 && ((uintptr_t)a->v % 16) == 0 && ((uintptr_t)a->out % 16) == 0,
                "attn_fwd: q, k, v and out must be 16-byte aligned");
  int rc;
  if (a->dtype == FMOBA_DTYPE_BF16)
    rc = a->head_dim <= 64 ? launch_fwd<bf16_t, 64>(*a, s) : launch_fwd<bf16_t, 128>(*a, s);
  else
    rc = a->head_dim <= 64 ? launch_fwd<f16_t, 64>(*a, s) : launch_fwd<f16_t, 128>(*a, s);
  if (rc) return rc;
  FMOBA_LAUNCH_CHECK("attn_fwd_kernel");
  return 0;
}
