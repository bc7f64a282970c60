// Sparse attention forward, row-block form, for patterns dense enough that most row blocks
// touch most of the chunks they may see (flash_fwd_kernel.h:325-700 of the reference walks the
// same (row block, key block) grid through its CSC lists).
//
// One workgroup owns a block of consecutive query rows of one (sequence, head) and walks, in ascending
// key order, the 64-key blocks of every chunk that at least one of its rows selected; all rows take
// part in the matrix products of a step, and the rows that did not select the chunk are masked out
// of the softmax (their probabilities are exact zeros).  The running maximum, the running sum and
// the output accumulators stay in registers for the whole walk, so nothing but Q, K, V and the
// output moves.  Two kernels: attn_fwd_rows_kernel (256 rows, eight compute waves that fetch the
// K/V tiles straight into LDS themselves; head dimensions up to 128 and up to 512 chunks per
// sequence) and attn_fwd_rows_loader_kernel (128 rows, four compute and four loader waves; every
// other shape, head dimension 256 included).
//
// The selection of a row is one bit per chunk (a bitmap built from the CSC lists by
// csc_bitmap_kernel); the chunks a workgroup walks are the OR of its rows' bitmaps.
#include "fmoba_common.h"

#include <type_traits>
#include <utility>

namespace fmoba {

constexpr int kRowsStepCap = 4096;  // 64-key steps of one row block (its step list lives in LDS)
constexpr int kRowsWordCap = 128;   // bitmap words per row (32 chunks each)

template <int HD>
struct FwdRowsSmem {
  static constexpr int LDQ = HD + 16;  // elements, K / V tiles (conflict-free for row reads and transposing reads)
  static constexpr int LDO = HD + 8;   // elements, per-wave output tile [32 rows][LDO]
  static constexpr size_t stage = (size_t)2 * 64 * LDQ * 2;  // K then V of one step
  static constexpr size_t oKV = 0;                            // [2 stages]; the output tiles reuse it at the end
  static constexpr size_t oStep = oKV + 2 * stage;            // int[kRowsStepCap]: key block | chunk << 16
  static constexpr size_t oUnion = oStep + (size_t)kRowsStepCap * 4;
  static constexpr size_t oOff = oUnion + (size_t)kRowsWordCap * 4;  // int[kRowsWordCap + 1]
  static constexpr size_t bytes = oOff + (size_t)(kRowsWordCap + 1) * 4 + 12;
  static_assert((size_t)4 * 32 * LDO * 2 <= 2 * stage, "output tiles must fit the K/V stages");
};

// one bit per (row, head, chunk): bm[(h * nw + c / 32) * total_q + q0 + r] bit c % 32 (the layout the gating
// leaves its selection in)
__global__ __launch_bounds__(256) void csc_bitmap_kernel(fmoba_attn_fwd_args a, uint32_t *bm, int nw) {
  const int c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int64_t bh = (int64_t)b * a.heads + h;
  const int nnz = a.col_nnz[bh * a.max_cols + c];
  const int32_t *list = a.row_indices + a.col_offsets[bh * a.max_cols + c];
  const uint32_t bit = 1u << (c & 31);
  for (int i = threadIdx.x; i < nnz; i += 256) {
    const int r = list[i];
    if (r >= 0 && r < Lq) atomicOr(&bm[((int64_t)h * nw + (c >> 5)) * a.total_q + q0 + r], bit);
  }
}

__global__ void fwd_zero_u32_kernel(uint32_t *p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0u;
}

template <typename T, int HD>
__global__ __launch_bounds__(512) void attn_fwd_rows_loader_kernel(fmoba_attn_fwd_args a, const uint32_t *bm, int nw) {
  typedef FwdRowsSmem<HD> SM;
  constexpr int KS = HD / 16, LDQ = SM::LDQ, LDO = SM::LDO, NDT = HD / 32, VPR = HD / 8;
  constexpr int NTHR = 512;
  constexpr int NV = 64 * VPR / 256;    // 16-byte vectors of one 64-key tile per loader thread
  constexpr int KSTEP = 256 / VPR;      // keys between two consecutive vectors of a loader thread
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  int *sStep = reinterpret_cast<int *>(smem + SM::oStep);
  uint32_t *sUnion = reinterpret_cast<uint32_t *>(smem + SM::oUnion);
  int *sOff = reinterpret_cast<int *>(smem + SM::oOff);

  const int nrb = (a.max_seqlen_q + 127) / 128;
  const PairItem item = xcd_pair_item(blockIdx.x, a.batch * a.heads, nrb);
  const int b = item.pair / a.heads, h = item.pair - b * a.heads;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int rb = nrb - 1 - item.idx;  // the longest walks (last rows of a causal sequence) start first
  const int r0 = rb * 128;
  if (r0 >= Lq) return;
  const int k0 = a.cu_seqlens_k[b], Lk = a.cu_seqlens_k[b + 1] - k0;
  const int off = Lk - Lq;
  const int D = a.head_dim;
  const int hk = h / (a.heads / a.heads_k);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
  const bool is_loader = wave >= 4;
  const bool causal = a.is_causal != 0;
  const int Bn = a.lg_block_n, sub = Bn >> 6;
  const float scale_log2 = a.softmax_scale * 1.4426950408889634f;

  // ---- the steps of this row block -------------------------------------------------------------
  const int rlast = min(r0 + 127, Lq - 1);
  const int kend = min(Lk, causal ? rlast + off + 1 : Lk);  // keys [0, kend) are visible to some row
  const int nchunk = kend > 0 ? (kend + Bn - 1) / Bn : 0;
  const int nwu = min((nchunk + 31) >> 5, nw);
  for (int w = tid; w < nwu; w += NTHR) sUnion[w] = 0u;
  __syncthreads();
  {
    const int nrow = rlast - r0 + 1;
    const uint32_t *bp = bm + (int64_t)h * nw * a.total_q + q0 + r0;
    for (int i = tid; i < nrow * nwu; i += NTHR) {
      const int w = i / nrow, row = i - w * nrow;
      const uint32_t x = bp[(int64_t)w * a.total_q + row];
      if (x) atomicOr(&sUnion[w], x);
    }
  }
  __syncthreads();
  // One thread per chunk: a chunk of the union contributes its 64-key blocks that hold a visible key; a scan over the
  // workgroup gives every chunk the place of its first step (a thread per selection word walking its bits one after
  // the other took 6 of the 11 us that a workgroup spends outside its step loop).
  int nstep_all = 0;
  const int nchunk_u = min(nchunk, nwu * 32);
  for (int c0 = 0; c0 < nchunk_u; c0 += NTHR) {
    const int c = c0 + tid;
    int cnt = 0;
    if (c < nchunk_u && ((sUnion[c >> 5] >> (c & 31)) & 1u)) cnt = min(sub, (kend - c * Bn + 63) >> 6);
    int incl = cnt;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o, 64);
      incl += lane >= o ? up : 0;
    }
    if (lane == 63) sOff[wave] = incl;
    __syncthreads();
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < NTHR / 64; ++w) {
      const int v = sOff[w];
      before += w < wave ? v : 0;
      total += v;
    }
    int pos = nstep_all + before + incl - cnt;
    for (int jb = 0; jb < cnt; ++jb, ++pos)
      if (pos < kRowsStepCap) sStep[pos] = (c * sub + jb) | (c << 16);
    nstep_all += total;
    __syncthreads();
  }
  const int nstep = min(nstep_all, kRowsStepCap);

  typedef std::integral_constant<int, 0> C0;
  typedef std::integral_constant<int, 1> C1;
  const int nstep_pad = (nstep + 1) & ~1;
  if (nstep == 0) {  // no visible selected key: out = 0, lse = +inf for the rows of this block
    if (!is_loader) {
      const int row = r0 + wave * 32 + (lane & 31);
      if (row < Lq) {
        uint16_t *op = reinterpret_cast<uint16_t *>(a.out) + (int64_t)(q0 + row) * a.o_row_stride + (int64_t)h * a.o_head_stride;
        for (int e = hh * 8; e < D; e += 16) *reinterpret_cast<Pack8 *>(op + e) = zero_pack8();
        if (hh == 0) a.softmax_lse[(int64_t)h * a.total_q + q0 + row] = INFINITY;
      }
    }
    return;
  }

  // K runs one step ahead of V: while the softmax of step t is evaluated the matrix cores already form
  // S of step t + 1.  Stage (t & 1) of each ring holds K(t) resp. V(t).
  uint16_t *const sKst = reinterpret_cast<uint16_t *>(smem + SM::oKV);
  uint16_t *const sVst = sKst + 2 * 64 * LDQ;

  if (is_loader) {
    const int lt = tid - 256;
    const int kb = lt / VPR, e = (lt - kb * VPR) * 8;
    const int ec = min(e, D - 8);
    const uint16_t *kp = reinterpret_cast<const uint16_t *>(a.k) + (int64_t)k0 * a.k_row_stride + (int64_t)hk * a.k_head_stride + ec;
    const uint16_t *vp = reinterpret_cast<const uint16_t *>(a.v) + (int64_t)k0 * a.v_row_stride + (int64_t)hk * a.v_head_stride + ec;
    Pack8 rk[2][NV], rv[2][NV];
    // loads are unconditional (steps and keys clamped, the surplus zeroed when stored) so that the
    // outstanding loads are counted exactly
    const int64_t kstep_k = (int64_t)KSTEP * a.k_row_stride, kstep_v = (int64_t)KSTEP * a.v_row_stride;
    const bool whole_rows = D == HD;
    auto load_tile = [&](Pack8(&r)[NV], const uint16_t *base, int64_t row_stride, int64_t step_stride, int t) {
      const int key0 = (sStep[min(t, nstep - 1)] & 0xffff) << 6;
      if (key0 + 64 <= Lk) {  // every key of the tile exists: one multiplication, then additions
        const uint16_t *p0 = base + (int64_t)(key0 + kb) * row_stride;
#pragma unroll
        for (int i = 0; i < NV; ++i) r[i] = ld_global16(p0 + i * step_stride);
      } else {
#pragma unroll
        for (int i = 0; i < NV; ++i) r[i] = ld_global16(base + (int64_t)min(key0 + kb + i * KSTEP, Lk - 1) * row_stride);
      }
    };
    auto load_k = [&](auto par, int t) { load_tile(rk[decltype(par)::value], kp, a.k_row_stride, kstep_k, t); };
    auto load_v = [&](auto par, int t) { load_tile(rv[decltype(par)::value], vp, a.v_row_stride, kstep_v, t); };
    auto store_tile = [&](uint16_t *dst, const Pack8(&r)[NV], int t) {
      const int key0 = (sStep[t] & 0xffff) << 6;
      if (whole_rows && key0 + 64 <= Lk) {
#pragma unroll
        for (int i = 0; i < NV; ++i) *reinterpret_cast<Pack8 *>(dst + (kb + i * KSTEP) * LDQ + e) = r[i];
      } else {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
          const int kl = kb + i * KSTEP;
          const bool ok = e < D && key0 + kl < Lk;
          Pack8 x = r[i];
#pragma unroll
          for (int w = 0; w < 4; ++w) x.w[w] = ok ? x.w[w] : 0u;
          *reinterpret_cast<Pack8 *>(dst + kl * LDQ + e) = x;
        }
      }
    };
    load_k(C0{}, 0);
    load_k(C1{}, 1);
    load_v(C0{}, 0);
    store_tile(sKst, rk[0], 0);
    load_k(C0{}, 2);
    load_v(C1{}, 1);
    __syncthreads();  // K(0) is in LDS
    if (1 < nstep) store_tile(sKst + 64 * LDQ, rk[1], 1);
    store_tile(sVst, rv[0], 0);
    load_k(C1{}, 3);
    load_v(C0{}, 2);
    auto loader_step = [&](auto par, int t) {  // par: parity of step t
      constexpr int P = decltype(par)::value;
      __syncthreads();  // K(t + 1) and V(t) are in LDS; the readers of K(t) and V(t - 1) are done
      if (t + 2 < nstep) store_tile(sKst + P * 64 * LDQ, rk[P], t + 2);
      if (t + 1 < nstep) store_tile(sVst + (P ^ 1) * 64 * LDQ, rv[P ^ 1], t + 1);
      load_k(par, t + 4);
      load_v(std::integral_constant<int, (P ^ 1)>{}, t + 3);
    };
    for (int t = 0; t < nstep_pad; t += 2) {
      loader_step(C0{}, t);
      loader_step(C1{}, t + 1);
    }
    __syncthreads();  // the compute waves are done with the stages
  } else {
    const int row = r0 + wave * 32 + (lane & 31);
    const bool valid = row < Lq;
    const int lim = valid ? min(causal ? row + off : 0x7fffffff, Lk - 1) : -1;  // last visible key
    const uint32_t *bmrow = bm + (int64_t)h * nw * a.total_q + q0 + min(row, Lq - 1);
    // this lane's query row as the B operand of S^T = K Q^T
    Pack8 qb[KS];
    {
      const uint16_t *qg = reinterpret_cast<const uint16_t *>(a.q) + (int64_t)(q0 + min(row, Lq - 1)) * a.q_row_stride + (int64_t)h * a.q_head_stride;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int e = (hh * KS + ks) * 8;
        qb[ks] = (valid && e < D) ? ld_global16(qg + e) : zero_pack8();
      }
    }
    f32x16 o[NDT];  // O^T: register i of feature tile dt <-> feature dt*32 + acc_row(i, hh), this lane's row
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
    f32x16 st[2][2];  // S^T of step t in st[t & 1]: register i of tile kt <-> key kt*32 + acc_row(i, hh), this lane's row
    float m_run = -INFINITY, l_run = 0.f;  // running maximum of the raw scores, running sum (this half of the wave)
    int cur_w = -1;
    uint32_t myword = 0u;
    const int kro = (lane & 31) * LDQ + hh * KS * 8;  // this lane's K row / feature slice within a 32-key tile

    auto k_frag = [&](const uint16_t *sK, int kt, int ks) { return *reinterpret_cast<const Pack8 *>(sK + kt * 32 * LDQ + kro + ks * 8); };
    // S of one step, not overlapped with anything (first step, and steps whose softmax the wave skips)
    auto s_plain = [&](const uint16_t *sK, f32x16(&sn)[2]) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        Pack8 kf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) kf[ks] = k_frag(sK, kt, ks);
#pragma unroll
        for (int i = 0; i < 16; ++i) sn[kt][i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) sn[kt] = mfma32<T>(kf[ks], qb[ks], sn[kt]);
      }
      __builtin_amdgcn_sched_barrier(0);
    };

    auto body = [&](auto par, int t) {
      constexpr int P = decltype(par)::value;
      const uint16_t *sKn = sKst + (P ^ 1) * 64 * LDQ;  // K(t + 1)
      const uint16_t *sV = sVst + P * 64 * LDQ;         // V(t)
      f32x16(&sc)[2] = st[P];
      f32x16(&sn)[2] = st[P ^ 1];
      const int s = sStep[t];
      const int key0 = (s & 0xffff) << 6, c = s >> 16;
      if ((c >> 5) != cur_w) {
        cur_w = c >> 5;
        myword = valid ? bmrow[(int64_t)cur_w * a.total_q] : 0u;
      }
      const bool active = ((myword >> (c & 31)) & 1u) != 0u && lim >= key0;
      // ---- part 0: operands of the first half of S(t + 1); row maximum of step t ----
      Pack8 kf[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) kf[ks] = k_frag(sKn, 0, ks);
      const int lim_rel = active ? lim - key0 : -1;
      if (!__all(lim_rel >= 63 || lim_rel < 0)) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int jrel = kt * 32 + 8 * (i >> 2) + (i & 3) + 4 * hh;
            sc[kt][i] = jrel <= lim_rel ? sc[kt][i] : -INFINITY;
          }
      }
      float mloc = -INFINITY;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, sc[kt][i]);
      mloc = max_xor32_f(mloc);
      // The reference point of the row's exponentials only moves when the block's maximum exceeds it by more than
      // 2^8 after scaling (always on the row's first block): p stays below 256, which the 16-bit P and the fp32 sums
      // hold easily, out and lse do not depend on the reference point, and O is rescaled a few times per row
      // instead of whenever one of the wave's 32 rows meets a new maximum.
      const bool grow = active & ((mloc - m_run) * scale_log2 > 8.f);
      const float m_new = grow ? mloc : m_run;
      const float alpha = m_new == m_run ? 1.f : __builtin_amdgcn_exp2f((m_run - m_new) * scale_log2);  // first visit: factor 0 on zeros
      const float neg_mc = active ? -m_new * scale_log2 : -INFINITY;  // rows that did not select the chunk: p = 0
      m_run = m_new;
      l_run *= alpha;
      if (!__all(alpha == 1.f)) {
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
      }
      __builtin_amdgcn_sched_barrier(0);
      // ---- part 1: S(t + 1) on the matrix cores under the exponentials of step t ----
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) sn[kt][i] = 0.f;
      Pack8 pf[2][2];  // P^T as the B operand of O^T += V^T P^T, straight from the accumulators
      Pack8 vt[2][2];  // V^T operands of one feature tile
      lds_cu16 *trV = tr_lane_base(sV, LDQ, lane) + 4 * hh * LDQ;
      float lsum = 0.f;
      static_for<16>([&](auto gi) {
        constexpr int g = decltype(gi)::value;
        constexpr int M0 = g * (2 * KS) / 16, M1 = (g + 1) * (2 * KS) / 16;
#pragma unroll
        for (int mi = M0; mi < M1; ++mi) {
          const int kt = mi / KS, ks = mi % KS;
          sn[kt] = mfma32<T>(kf[ks], qb[ks], sn[kt]);
          if (kt == 0) kf[ks] = k_frag(sKn, 1, ks);  // the operand of the second key tile takes the register over
        }
        constexpr int kte = g / 8, j = g % 8;
        const float p0 = __builtin_amdgcn_exp2f(fmaf(sc[kte][2 * j], scale_log2, neg_mc));
        const float p1 = __builtin_amdgcn_exp2f(fmaf(sc[kte][2 * j + 1], scale_log2, neg_mc));
        lsum += p0 + p1;
        pf[kte][j / 4].w[j % 4] = pack2<T>(p0, p1);
        if (g == 14) {  // V^T operands of the first feature tile
#pragma unroll
          for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
              const int lo = (kt * 32 + 16 * s2) * LDQ;
              vt[kt][s2] = tr_frag8_at(trV, lo, lo + 8 * LDQ);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      l_run += lsum;
      // ---- part 2: O^T += V^T P^T ----
      static_for<NDT>([&](auto di) {
        constexpr int dt = decltype(di)::value;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            o[dt] = mfma32<T>(vt[kt][s2], pf[kt][s2], o[dt]);
            if (dt + 1 < NDT) {  // the operand of the next feature tile takes the register over
              const int lo = (kt * 32 + 16 * s2) * LDQ + (dt + 1) * 32;
              vt[kt][s2] = tr_frag8_at(trV, lo, lo + 8 * LDQ);
            }
          }
        __builtin_amdgcn_sched_barrier(0);
      });
    };

    __syncthreads();  // K(0) is in LDS
    s_plain(sKst, st[0]);
    for (int t = 0; t < nstep_pad; t += 2) {
      __syncthreads();  // K(t + 1) and V(t) are in LDS
      body(C0{}, t);
      __syncthreads();
      if (t + 1 < nstep) body(C1{}, t + 1);
    }
    __syncthreads();  // every wave is done with the stages: they now hold the output tiles

    const float l_tot = sum_xor32_f(l_run);
    const bool empty = !(l_tot > 0.f);
    const float inv = empty ? 0.f : 1.f / l_tot;
    uint16_t *sOut = reinterpret_cast<uint16_t *>(smem + SM::oKV) + (size_t)wave * 32 * LDO;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *reinterpret_cast<uint2 *>(sOut + (lane & 31) * LDO + dt * 32 + 8 * g + 4 * hh) =
            make_uint2(pack2<T>(o[dt][4 * g] * inv, o[dt][4 * g + 1] * inv), pack2<T>(o[dt][4 * g + 2] * inv, o[dt][4 * g + 3] * inv));
    if (valid && hh == 0)
      a.softmax_lse[(int64_t)h * a.total_q + q0 + row] = empty ? INFINITY : (m_run * scale_log2 + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f;
    wave_lds_fence();
    // rows leave as 16-byte pieces, VPR of them per row, consecutive lanes taking consecutive pieces
#pragma unroll
    for (int v0 = 0; v0 < 32 * VPR; v0 += 64) {
      const int v = v0 + lane, rl = v / VPR, e = (v - rl * VPR) * 8;
      const int r2 = r0 + wave * 32 + rl;
      if (r2 < Lq && e < D) {
        const Pack8 x = *reinterpret_cast<const Pack8 *>(sOut + rl * LDO + e);
        *reinterpret_cast<Pack8 *>(reinterpret_cast<uint16_t *>(a.out) + (int64_t)(q0 + r2) * a.o_row_stride + (int64_t)h * a.o_head_stride + e) = x;
      }
    }
  }
}

// ------------------------------------------------------------------------------------
// The same walk with EIGHT compute waves (256 query rows per workgroup, two waves per SIMD) and no loader waves, for
// head dimensions up to 128: the matrix products of one wave run under the softmax arithmetic of the other wave of
// its SIMD.  K and V tiles go from global memory straight into LDS (every wave issues an eighth of a tile's loads,
// three steps ahead for K and two for V, rings of three stages) in rows of exactly HD elements, swizzled instead of
// padded (piece c of row r lies at piece c ^ tile_swz(r)): the 16-byte row reads of the K operands and the transposing
// reads of the V^T operands both spread over all banks.  Keys past the sequence and features past head_dim are fetched
// from a key and a piece that exist: the scores of such keys are masked, Q is zero in such features and the
// corresponding output features are never stored.
// ------------------------------------------------------------------------------------
constexpr int kRows8 = 256;  // rows of a workgroup
constexpr int kRows8Words = 16;  // selection words per row that the workgroup keeps in LDS (512 chunks)

template <int HD>
struct FwdRows8Smem {
  static constexpr int LDO = HD + 8;   // elements, per-wave output tile [32 rows][LDO]
  static constexpr size_t tile = (size_t)64 * HD * 2;       // one 64-key tile of K or V
  static constexpr size_t oK = 0;                             // [3 stages]
  static constexpr size_t oV = oK + 3 * tile;                 // [4 stages]; the output tiles reuse both rings at the end
  static constexpr size_t oStep = oV + 4 * tile;              // int[kRowsStepCap]: key block | chunk << 16
  static constexpr size_t oUnion = oStep + (size_t)kRowsStepCap * 4;
  static constexpr size_t oOff = oUnion + (size_t)kRowsWordCap * 4;  // int[8]
  static constexpr size_t oBits = oOff + (size_t)(kRowsWordCap + 1) * 4 + 12;  // uint32[kRows8Words][256]: the rows' selection words
  static constexpr size_t bytes = oBits + (size_t)kRows8Words * kRows8 * 4;
  static_assert((size_t)8 * 32 * LDO * 2 <= 7 * tile, "output tiles must fit the K/V rings");
  static_assert(bytes <= 160 * 1024, "LDS of one compute unit");
};

template <typename T, int HD>
__global__ __launch_bounds__(512) void attn_fwd_rows_kernel(fmoba_attn_fwd_args a, const uint32_t *bm, int nw) {
  typedef FwdRows8Smem<HD> SM;
  constexpr int KS = HD / 16, LDO = SM::LDO, NDT = HD / 32, VPR = HD / 8;
  constexpr int NTHR = 512;
  constexpr int RB = HD * 2;            // bytes of a tile row
  constexpr int RPI = 64 / VPR;         // tile rows per direct-to-LDS instruction (64 lanes x 16 bytes)
  constexpr int NI = 64 / RPI / 4;      // such instructions per tile and feeding wave
  static_assert(NI >= 1, "four waves share the loads of a tile");
  extern __shared__ __attribute__((aligned(256))) uint8_t smem[];
  int *sStep = reinterpret_cast<int *>(smem + SM::oStep);
  uint32_t *sUnion = reinterpret_cast<uint32_t *>(smem + SM::oUnion);
  int *sOff = reinterpret_cast<int *>(smem + SM::oOff);
  uint32_t *sBits = reinterpret_cast<uint32_t *>(smem + SM::oBits);

  const int nrb = (a.max_seqlen_q + kRows8 - 1) / kRows8;
  const PairItem item = xcd_pair_item(blockIdx.x, a.batch * a.heads, nrb);
  const int b = item.pair / a.heads, h = item.pair - b * a.heads;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int rb = nrb - 1 - item.idx;  // the longest walks (last rows of a causal sequence) start first
  const int r0 = rb * kRows8;
  if (r0 >= Lq) return;
  const int k0 = a.cu_seqlens_k[b], Lk = a.cu_seqlens_k[b + 1] - k0;
  const int off = Lk - Lq;
  const int D = a.head_dim;
  const int hk = h / (a.heads / a.heads_k);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
  const bool causal = a.is_causal != 0;
  const int Bn = a.lg_block_n, sub = Bn >> 6;
  const float scale_log2 = a.softmax_scale * 1.4426950408889634f;

  // ---- the steps of this row block -------------------------------------------------------------
  const int rlast = min(r0 + kRows8 - 1, Lq - 1);
  const int kend = min(Lk, causal ? rlast + off + 1 : Lk);  // keys [0, kend) are visible to some row
  const int nchunk = kend > 0 ? (kend + Bn - 1) / Bn : 0;
  const int nwu = min((nchunk + 31) >> 5, nw);
  for (int w = tid; w < nwu; w += NTHR) sUnion[w] = 0u;
  __syncthreads();
  {
    const int nrow = rlast - r0 + 1;
    const uint32_t *bp = bm + (int64_t)h * nw * a.total_q + q0 + r0;
    // (the words stay in LDS for the walk: a load from global memory inside the step loop would make the compiler
    // wait for every outstanding load of the wave, the tile loads included, at every step)
    for (int i = tid; i < nrow * nwu; i += NTHR) {
      const int w = i / nrow, row = i - w * nrow;
      const uint32_t x = bp[(int64_t)w * a.total_q + row];
      sBits[w * kRows8 + row] = x;
      if (x) atomicOr(&sUnion[w], x);
    }
  }
  __syncthreads();
  // one thread per chunk: a chunk of the union contributes its 64-key blocks that hold a visible key; a scan over the
  // workgroup gives every chunk the place of its first step
  int nstep_all = 0;
  const int nchunk_u = min(nchunk, nwu * 32);
  for (int c0 = 0; c0 < nchunk_u; c0 += NTHR) {
    const int c = c0 + tid;
    int cnt = 0;
    if (c < nchunk_u && ((sUnion[c >> 5] >> (c & 31)) & 1u)) cnt = min(sub, (kend - c * Bn + 63) >> 6);
    int incl = cnt;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o, 64);
      incl += lane >= o ? up : 0;
    }
    if (lane == 63) sOff[wave] = incl;
    __syncthreads();
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < NTHR / 64; ++w) {
      const int v = sOff[w];
      before += w < wave ? v : 0;
      total += v;
    }
    int pos = nstep_all + before + incl - cnt;
    for (int jb = 0; jb < cnt; ++jb, ++pos)
      if (pos < kRowsStepCap) sStep[pos] = (c * sub + jb) | (c << 16);
    nstep_all += total;
    __syncthreads();
  }
  const int nstep = min(nstep_all, kRowsStepCap);

  typedef std::integral_constant<int, 0> C0;
  typedef std::integral_constant<int, 1> C1;
  const int row = r0 + wave * 32 + (lane & 31);
  const bool valid = row < Lq;
  if (nstep == 0) {  // no visible selected key: out = 0, lse = +inf for the rows of this block
    if (valid) {
      uint16_t *op = reinterpret_cast<uint16_t *>(a.out) + (int64_t)(q0 + row) * a.o_row_stride + (int64_t)h * a.o_head_stride;
      for (int e = hh * 8; e < D; e += 16) *reinterpret_cast<Pack8 *>(op + e) = zero_pack8();
      if (hh == 0) a.softmax_lse[(int64_t)h * a.total_q + q0 + row] = INFINITY;
    }
    return;
  }

  // ---- feeding the rings: the waves 0..3 fetch the tiles, rows wave * 16 .. wave * 16 + 15 each.  They reach the
  // barrier of a step well before the waves 4..7 (which run a step's last part one step late and meet them on the
  // matrix cores at the end of the step), so the loads are theirs ---------------------------------------------------
  const uint32_t ldsK = (uint32_t)(uintptr_t)(smem + SM::oK), ldsV = (uint32_t)(uintptr_t)(smem + SM::oV);
  const uint16_t *kg = reinterpret_cast<const uint16_t *>(a.k) + (int64_t)k0 * a.k_row_stride + (int64_t)hk * a.k_head_stride;
  const uint16_t *vg = reinterpret_cast<const uint16_t *>(a.v) + (int64_t)k0 * a.v_row_stride + (int64_t)hk * a.v_head_stride;
  // A lane's piece of row tr = wave * 16 + i * RPI + lane / VPR of a tile: its byte offset from the tile's first key, for K
  // and for V.  A tile whose 64 keys all exist is fetched from a wave-uniform base plus these offsets (no vector
  // instruction per load); the last tile of a sequence clamps the keys per lane.
  uint32_t lofK[NI], lofV[NI];
  {
    const int rl = lane / VPR, p = lane - rl * VPR;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int tr = (wave & 3) * (64 / 4) + i * RPI + rl;
      const uint32_t e = (uint32_t)min((p ^ tile_swz<HD>(tr)) * 8, D - 8);
      lofK[i] = ((uint32_t)tr * (uint32_t)a.k_row_stride + e) * 2u;
      lofV[i] = ((uint32_t)tr * (uint32_t)a.v_row_stride + e) * 2u;
    }
  }
  auto feed = [&](const uint16_t *g, uint32_t row_stride, const uint32_t(&lof)[NI], uint32_t lds_ring, int stage, int t) {
    if (wave >= 4) return;
    const int key0 = __builtin_amdgcn_readfirstlane((sStep[min(t, nstep - 1)] & 0xffff) << 6);
    const uint32_t dst = lds_ring + (uint32_t)__builtin_amdgcn_readfirstlane(stage * (int)SM::tile + wave * (64 / 4) * RB);
    if (key0 + 64 <= Lk) {
      const uint16_t *base = g + (uint64_t)(uint32_t)key0 * row_stride;
#pragma unroll
      for (int i = 0; i < NI; ++i) global_to_lds16_sbase(lof[i], base, dst + (uint32_t)(i * RPI * RB));
    } else {
      const int rl = lane / VPR, p = lane - rl * VPR;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int tr = wave * (64 / 4) + i * RPI + rl;  // row of the tile
        const uint32_t e = (uint32_t)min((p ^ tile_swz<HD>(tr)) * 8, D - 8);
        const uint32_t key = (uint32_t)min(key0 + tr, Lk - 1);
        global_to_lds16(g + ((uint64_t)key * row_stride + e), dst + (uint32_t)(i * RPI * RB));
      }
    }
  };
  auto feed_k = [&](int t) { feed(kg, (uint32_t)a.k_row_stride, lofK, ldsK, t % 3, t); };
  auto feed_v = [&](int t) { feed(vg, (uint32_t)a.v_row_stride, lofV, ldsV, t & 3, t); };
  // the loads of a step, once per feeding wave: the wait before the next barrier lets exactly these stay in flight
  constexpr int kLoadsPerStep = 2 * NI;

  const int lim = valid ? min(causal ? row + off : 0x7fffffff, Lk - 1) : -1;  // last visible key
  // this lane's query row as the B operand of S^T = K Q^T
  Pack8 qb[KS];
  {
    const uint16_t *qg = reinterpret_cast<const uint16_t *>(a.q) + (int64_t)(q0 + min(row, Lq - 1)) * a.q_row_stride + (int64_t)h * a.q_head_stride;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int e = (hh * KS + ks) * 8;
      qb[ks] = (valid && e < D) ? ld_global16(qg + e) : zero_pack8();
    }
  }
  // (Q is in registers before the first tile loads are issued: from here on the wave counts its outstanding loads)
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(qb[ks].w[0]), "+v"(qb[ks].w[1]), "+v"(qb[ks].w[2]), "+v"(qb[ks].w[3]));
#endif
  wait_all_loads();
  feed_k(0);
  feed_k(1);
  feed_v(0);
  feed_k(2);
  feed_v(1);

  f32x16 o[NDT];  // O^T: register i of feature tile dt <-> feature dt*32 + acc_row(i, hh), this lane's row
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
  f32x16 st[2][2];  // S^T of step t in st[t & 1]: register i of tile kt <-> key kt*32 + acc_row(i, hh), this lane's row
  float m_run = -INFINITY, l_run = 0.f;  // running maximum of the raw scores, running sum (this half of the wave)
  // byte offsets of this lane's pieces inside a tile: row reads (key lane % 32 of a 32-key half, pieces hh * KS ..) and
  // transposing reads (key (lane % 16) / 4 + 4 hh, feature tile 0); every other operand is an exclusive-or on the piece
  // bits plus a constant
  const uint32_t rowoff = (uint32_t)((lane & 31) * RB + (((hh * KS) ^ tile_swz<HD>(lane & 31)) * 16));
  const int li = lane & 15, r0t = (li >> 2) + 4 * hh;
  const uint32_t troff = (uint32_t)(r0t * RB + ((((((lane >> 4) & 1) * 2 + ((li & 3) >> 1))) ^ tile_swz<HD>(r0t)) * 16) + (li & 1) * 8);
  auto opaque = [](uint32_t &x) {
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("" : "+v"(x));
#else
    (void)x;
#endif
  };
  auto k_frag = [&](uint32_t ak, int kt, int ks) { return lds_read16((ak ^ (uint32_t)(ks * 16)) + (uint32_t)(kt * 32 * RB)); };
  auto v_frag = [&](uint32_t tv, int dt, int kt, int s2) {
    const uint32_t xlo = (uint32_t)(dt * 4 * 16), xhi = (uint32_t)(((dt * 4) ^ TileSwz<HD>::kRow8) * 16);
    const uint32_t olo = (uint32_t)((kt * 32 + 16 * s2) * RB), ohi = olo + (uint32_t)(8 * RB);
    return lds_tr8((tv ^ xlo) + olo, (tv ^ xhi) + ohi);
  };
  // S of the first step, not overlapped with anything
  auto s_plain = [&](uint32_t ak, f32x16(&sn)[2]) {
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      Pack8 kf[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) kf[ks] = k_frag(ak, kt, ks);
#pragma unroll
      for (int i = 0; i < 16; ++i) sn[kt][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) sn[kt] = mfma32<T>(kf[ks], qb[ks], sn[kt]);
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // A step in three parts.  part0: masks, row maximum and the reference point of step t (vector arithmetic); part1:
  // S(t + 1) on the matrix cores under the exponentials of step t; part2: O^T += V^T P^T of step t (matrix cores).
  // The waves 4..7 share their SIMDs with the waves 0..3 and run part2 one step late, before part0 and part1 of the
  // next step: every step begins at a workgroup barrier, and two waves that walk the parts in the same order want the
  // matrix cores, then the vector unit, at the same moments.
  Pack8 pf[2][2];      // P^T as the B operand of O^T += V^T P^T, straight from the accumulators
  Pack8 kf[KS];        // K operands of S(t + 1): read at the start of part0, their latency runs under its arithmetic
  Pack8 vt[2][2];      // V^T operands of the first feature tile of step t: read at the end of part1
  float neg_mc = 0.f;  // minus the reference point of the row's exponentials, scaled; -inf for a row that skips the step
  int s_nx = sStep[0];  // entry of the next step and this row's word of selection bits for its chunk
  uint32_t word_nx = sBits[((s_nx >> 16) >> 5) * kRows8 + wave * 32 + (lane & 31)];
  auto part0 = [&](auto par, int t) {
    constexpr int P = decltype(par)::value;
    f32x16(&sc)[2] = st[P];
    {
      uint32_t akn = ldsK + (uint32_t)(((t + 1) % 3) * (int)SM::tile) + rowoff;  // K(t + 1)
      opaque(akn);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) kf[ks] = k_frag(akn, 0, ks);
    }
    // (the step's entry and this row's selection word were read during the step before: two dependent LDS reads at
    // this place would be waited for with nothing to do, by every wave at the start of every step)
    const int s = s_nx;
    const int key0 = (s & 0xffff) << 6, c = s >> 16;
    const uint32_t myword = word_nx;
    const bool active = valid && ((myword >> (c & 31)) & 1u) != 0u && lim >= key0;
    const int lim_rel = active ? lim - key0 : -1;
    if (!__all(lim_rel >= 63 || lim_rel < 0)) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int jrel = kt * 32 + 8 * (i >> 2) + (i & 3) + 4 * hh;
          sc[kt][i] = jrel <= lim_rel ? sc[kt][i] : -INFINITY;
        }
    }
    float mloc = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, sc[kt][i]);
    mloc = max_xor32_f(mloc);
    // The reference point of the row's exponentials only moves when the block's maximum exceeds it by more than 2^8
    // after scaling (always on the row's first block): p stays below 256, out and lse do not depend on the reference
    // point, and O is rescaled a few times per row instead of whenever one of the wave's 32 rows meets a new maximum.
    const bool grow = active & ((mloc - m_run) * scale_log2 > 8.f);
    const float m_new = grow ? mloc : m_run;
    const float alpha = m_new == m_run ? 1.f : __builtin_amdgcn_exp2f((m_run - m_new) * scale_log2);  // first visit: factor 0 on zeros
    neg_mc = active ? -m_new * scale_log2 : -INFINITY;  // rows that did not select the chunk: p = 0
    m_run = m_new;
    l_run *= alpha;
    if (!__all(alpha == 1.f)) {
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto part1 = [&](auto par, int t) {
    constexpr int P = decltype(par)::value;
    uint32_t akn = ldsK + (uint32_t)(((t + 1) % 3) * (int)SM::tile) + rowoff;  // K(t + 1)
    opaque(akn);
    f32x16(&sc)[2] = st[P];
    f32x16(&sn)[2] = st[P ^ 1];
    uint32_t tv = ldsV + (uint32_t)((t & 3) * (int)SM::tile) + troff;  // V(t)
    opaque(tv);
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) sn[kt][i] = 0.f;
    float lsum = 0.f;
    static_for<16>([&](auto gi) {
      constexpr int g = decltype(gi)::value;
      constexpr int M0 = g * (2 * KS) / 16, M1 = (g + 1) * (2 * KS) / 16;
#pragma unroll
      for (int mi = M0; mi < M1; ++mi) {
        const int kt = mi / KS, ks = mi % KS;
        sn[kt] = mfma32<T>(kf[ks], qb[ks], sn[kt]);
        if (kt == 0) kf[ks] = k_frag(akn, 1, ks);  // the operand of the second key tile takes the register over
      }
      constexpr int kte = g / 8, j = g % 8;
      const float p0 = __builtin_amdgcn_exp2f(fmaf(sc[kte][2 * j], scale_log2, neg_mc));
      const float p1 = __builtin_amdgcn_exp2f(fmaf(sc[kte][2 * j + 1], scale_log2, neg_mc));
      lsum += p0 + p1;
      pf[kte][j / 4].w[j % 4] = pack2<T>(p0, p1);
      if (g == 2) s_nx = sStep[min(t + 1, nstep - 1)];
      if (g == 8) word_nx = sBits[((s_nx >> 16) >> 5) * kRows8 + wave * 32 + (lane & 31)];
      if (g == 14) {  // V^T operands of the first feature tile
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) vt[kt][s2] = v_frag(tv, 0, kt, s2);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    l_run += lsum;
  };
  auto part2 = [&](int t) {
    uint32_t tv = ldsV + (uint32_t)((t & 3) * (int)SM::tile) + troff;  // V(t)
    opaque(tv);
    static_for<NDT>([&](auto di) {
      constexpr int dt = decltype(di)::value;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          o[dt] = mfma32<T>(vt[kt][s2], pf[kt][s2], o[dt]);
          if (dt + 1 < NDT) vt[kt][s2] = v_frag(tv, dt + 1, kt, s2);  // the operand of the next feature tile takes the register over
        }
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  auto wait_older_loads = [&]() {  // all but the loads of the current step
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (kLoadsPerStep == 8)
      asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else
      asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
#endif
  };
  static_assert(kLoadsPerStep == 8 || kLoadsPerStep == 4, "wait_older_loads");

  // K(0), K(1), V(0) have to be there for the first step: the two youngest groups of loads (K(2), V(1)) may stay out
  wait_older_loads();
  __syncthreads();
  {
    uint32_t ak0 = ldsK + rowoff;
    opaque(ak0);
    s_plain(ak0, st[0]);
  }
  const int nstep_pad = (nstep + 1) & ~1;
  const bool late = wave >= 4;
  auto step = [&](auto par, int t) {
    // K(t + 1) and V(t) are in LDS (the wait before the last barrier); the readers of K(t) and V(t - 2) are done
    feed_k(t + 3);
    feed_v(t + 2);
    if (late) {
      if (t >= 1 && t - 1 < nstep) part2(t - 1);
      if (t < nstep) {
        part0(par, t);
        part1(par, t);
      }
    } else if (t < nstep) {
      part0(par, t);
      part1(par, t);
      part2(t);
    }
    wait_older_loads();
    __syncthreads();
  };
  for (int t = 0; t < nstep_pad; t += 2) {
    step(C0{}, t);
    step(C1{}, t + 1);
  }
  if (late && nstep_pad - 1 < nstep) part2(nstep_pad - 1);  // (an even number of steps: the last one's products are still due)
  wait_all_loads();
  __syncthreads();  // every wave is done with the rings and nothing is in flight: they now hold the output tiles

  const float l_tot = sum_xor32_f(l_run);
  const bool empty = !(l_tot > 0.f);
  const float inv = empty ? 0.f : 1.f / l_tot;
  uint16_t *sOut = reinterpret_cast<uint16_t *>(smem + SM::oK) + (size_t)wave * 32 * LDO;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g)
      *reinterpret_cast<uint2 *>(sOut + (lane & 31) * LDO + dt * 32 + 8 * g + 4 * hh) =
          make_uint2(pack2<T>(o[dt][4 * g] * inv, o[dt][4 * g + 1] * inv), pack2<T>(o[dt][4 * g + 2] * inv, o[dt][4 * g + 3] * inv));
  if (valid && hh == 0)
    a.softmax_lse[(int64_t)h * a.total_q + q0 + row] = empty ? INFINITY : (m_run * scale_log2 + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f;
  wave_lds_fence();
  // rows leave as 16-byte pieces, VPR of them per row, consecutive lanes taking consecutive pieces
#pragma unroll
  for (int v0 = 0; v0 < 32 * VPR; v0 += 64) {
    const int v = v0 + lane, rl = v / VPR, e = (v - rl * VPR) * 8;
    const int r2 = r0 + wave * 32 + rl;
    if (r2 < Lq && e < D) {
      const Pack8 x = *reinterpret_cast<const Pack8 *>(sOut + rl * LDO + e);
      *reinterpret_cast<Pack8 *>(reinterpret_cast<uint16_t *>(a.out) + (int64_t)(q0 + r2) * a.o_row_stride + (int64_t)h * a.o_head_stride + e) = x;
    }
  }
}

template <typename T, int HD>
static int launch_rows_eight(const fmoba_attn_fwd_args &a, const uint32_t *bm, int nw, hipStream_t s) {
  auto kern = attn_fwd_rows_kernel<T, HD>;
  const size_t smem = FwdRows8Smem<HD>::bytes;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("attn_fwd: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  const int64_t items = (int64_t)a.batch * a.heads * ceil_div(a.max_seqlen_q, kRows8);
  if (items >= ((int64_t)1 << 31)) {
    set_error("attn_fwd: too many (sequence, head, row block) work items");
    return 1;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)items), dim3(512), smem, s, a, bm, nw);
  return 0;
}

template <typename T, int HD>
static int launch_rows_loader(const fmoba_attn_fwd_args &a, const uint32_t *bm, int nw, hipStream_t s) {
  auto kern = attn_fwd_rows_loader_kernel<T, HD>;
  const size_t smem = FwdRowsSmem<HD>::bytes;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("attn_fwd: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  const int64_t items = (int64_t)a.batch * a.heads * ceil_div(a.max_seqlen_q, 128);
  if (items >= ((int64_t)1 << 31)) {
    set_error("attn_fwd: too many (sequence, head, row block) work items");
    return 1;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)items), dim3(512), smem, s, a, bm, nw);
  return 0;
}

bool fwd_rows_feasible(const fmoba_attn_fwd_args &a) {
  return a.head_dim <= 256 && ceil_div(a.max_cols, 32) <= kRowsWordCap && ceil_div(a.max_seqlen_k, 64) <= kRowsStepCap &&
         a.max_cols < 32768 && a.lg_block_n % 64 == 0;
}

size_t fwd_rows_workspace_bytes(const fmoba_attn_fwd_args &a) {
  if (a.selection_bits != nullptr) return 256;
  const size_t rows = (size_t)a.total_q * a.heads;
  return ((rows * (size_t)ceil_div(a.max_cols, 32) * 4 + 255) & ~(size_t)255) + 256;
}

// bitmap build (phase 1) + the row-block pass (phase 2)
int run_fwd_rows(const fmoba_attn_fwd_args &a, int phases, hipStream_t s) {
  const int nw = ceil_div(a.max_cols, 32);
  const int64_t rows = (int64_t)a.total_q * a.heads;
  const uint32_t *bm = a.selection_bits;
  if (bm == nullptr) {
    uint32_t *own = reinterpret_cast<uint32_t *>(((uintptr_t)a.workspace + 255) & ~(uintptr_t)255);
    bm = own;
    if (phases & 1) {
      hipLaunchKernelGGL(fwd_zero_u32_kernel, dim3(512), dim3(256), 0, s, own, rows * nw);
      hipLaunchKernelGGL(csc_bitmap_kernel, dim3(a.max_cols, a.heads, a.batch), dim3(256), 0, s, a, own, nw);
    }
  }
  if (phases & 2) {
    const bool bf = a.dtype == FMOBA_DTYPE_BF16;
    int rc;
    // eight compute waves when the rows' selection words fit the workgroup's LDS (up to 512 chunks per sequence)
    // (and the rows of a tile lie within 32-bit byte offsets of its first key)
    const bool eight = nw <= kRows8Words && a.k_row_stride < ((int64_t)1 << 24) && a.v_row_stride < ((int64_t)1 << 24);
    if (a.head_dim <= 64)
      rc = eight ? (bf ? launch_rows_eight<bf16_t, 64>(a, bm, nw, s) : launch_rows_eight<f16_t, 64>(a, bm, nw, s))
                 : (bf ? launch_rows_loader<bf16_t, 64>(a, bm, nw, s) : launch_rows_loader<f16_t, 64>(a, bm, nw, s));
    else if (a.head_dim <= 128)
      rc = eight ? (bf ? launch_rows_eight<bf16_t, 128>(a, bm, nw, s) : launch_rows_eight<f16_t, 128>(a, bm, nw, s))
                 : (bf ? launch_rows_loader<bf16_t, 128>(a, bm, nw, s) : launch_rows_loader<f16_t, 128>(a, bm, nw, s));
    else
      rc = bf ? launch_rows_loader<bf16_t, 256>(a, bm, nw, s) : launch_rows_loader<f16_t, 256>(a, bm, nw, s);
    if (rc) return rc;
  }
  return 0;
}

}  // namespace fmoba
