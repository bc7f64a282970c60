// Sparse attention forward over a CSC pattern: the entry points, and the column-stationary form in two
// launches (sparse patterns; the row-block form for dense ones is in attn_fwd_rows.hip).
//
//   attn_fwd_col_kernel     : one workgroup per (key block of KB = 64 or 128 keys, head,
//                             sequence).  K of the block lives in MFMA operand registers, V in
//                             LDS; the block's ascending row list is walked in gathered 32-row
//                             tiles: S^T = K Q^T (one lane owns one query row, so the softmax
//                             reductions over the block's keys stay in registers), P^T goes from
//                             the accumulators straight into the operand registers of
//                             O^T = V^T P^T (V^T through transposing LDS reads).  Every visit of
//                             a (row, key block) pair leaves a PARTIAL result: the block-local
//                             maximum m, the sum l of exp2(s - m) and the unnormalised output row
//                             (16-bit), in a slot that the row hands out from a counter.
//   attn_fwd_combine_kernel : sixteen lanes per (row, head) merge the row's partials in ascending
//                             key-block order (sorted by block id, so the result does not depend
//                             on which slot a visit happened to get): out, log-sum-exp.
//
// Work and traffic are proportional to the number of (row, key block) visits whatever the number of
// chunks per sequence; a row-stationary formulation degenerates when every 128-row block touches
// thousands of chunks with one or two rows each.
// In the first kernel all four waves compute (one tile each per round, one wave per SIMD: K of the block and
// the operands of a tile take most of its registers); the gathered Q rows go from global memory straight to
// LDS (global_load_lds), one round ahead.
#include "fmoba_common.h"

#include <algorithm>
#include <type_traits>
#include <utility>

namespace fmoba {

// row-block form when a row selects at least 10/50 (64-key blocks) resp. 10/27 (128-key blocks) of the chunks it may see:
// measured break-even points (16 heads of 128, 8K and 16K tokens per sequence, top-k 8 to 32)
constexpr int kFwdRowsDensity64 = 50, kFwdRowsDensity128 = 27;

constexpr int kFwdRoundRows = 128;  // rows of a column list per round: one 32-row tile per wave

template <int HD, int KB>
struct FwdColSmem {
  static constexpr int LDQ = HD + 16;  // elements, K / V rows (conflict-free for the 16-byte row reads and the transposing reads)
  static constexpr int LDO = HD + 8;   // elements, per-wave output tile [32 rows][LDO]
  static constexpr size_t tileBytes = (size_t)32 * HD * 2;  // a gathered Q tile: rows of exactly HD elements, swizzled
  static constexpr size_t oV = 0;
  static constexpr size_t oQ = oV + (size_t)KB * LDQ * 2;           // [2 buffers][4 tiles][32][HD]; K passes through it on its way to registers
  static constexpr size_t oOut = oQ + 8 * tileBytes;                 // [4 waves][32][LDO]
  static constexpr size_t oRid = oOut + (size_t)4 * 32 * LDO * 2;    // int[2][128]: row ids, one round before the rest
  static constexpr size_t oRow = oRid + 2 * kFwdRoundRows * 4;       // int[2][128]
  static constexpr size_t oSlot = oRow + 2 * kFwdRoundRows * 4;      // int[2][128]
  static constexpr size_t bytes = oSlot + 2 * kFwdRoundRows * 4;
  static_assert((size_t)KB * LDQ * 2 <= 8 * tileBytes + (size_t)4 * 32 * LDO * 2, "K passes through the Q tiles and the output tiles");
  static_assert(bytes <= 160 * 1024, "LDS of one compute unit");
};

struct FwdWs {
  int32_t *cnt;      // [total_q * heads] visits handed out per (row, head)
  float4 *hdr;       // [total_q * heads * cap] {m (log2 domain), l, key block id, -}
  uint16_t *part;    // [total_q * heads * cap][head_dim] unnormalised partial outputs
  int32_t cap;
};

template <typename T, int HD, int KB>
__global__ __launch_bounds__(256) void attn_fwd_col_kernel(fmoba_attn_fwd_args a, FwdWs ws) {
  typedef FwdColSmem<HD, KB> SM;
  constexpr int NTHR = 256;
  constexpr int KS = HD / 16, LDQ = SM::LDQ, LDO = SM::LDO, NDT = HD / 32, VPR = HD / 8;
  constexpr int KT = KB / 32;                 // 32-key tiles of the block
  constexpr uint32_t TB = (uint32_t)SM::tileBytes;
  constexpr int RB = HD * 2;                  // bytes of a tile row
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint16_t *sV = reinterpret_cast<uint16_t *>(smem + SM::oV);
  int *sRid = reinterpret_cast<int *>(smem + SM::oRid);
  int *sRow = reinterpret_cast<int *>(smem + SM::oRow);
  int *sSlot = reinterpret_cast<int *>(smem + SM::oSlot);

  const PairItem item = xcd_pair_item(blockIdx.x, a.batch * a.heads, (a.max_seqlen_k + KB - 1) / KB, (int64_t)a.max_seqlen_q * HD * 4 >= kOnePairBytes);
  const int nb = item.idx, b = item.pair / a.heads, h = item.pair - b * a.heads;
  const int k0 = a.cu_seqlens_k[b], Lk = a.cu_seqlens_k[b + 1] - k0;
  const int key0 = nb * KB;
  if (key0 >= Lk) return;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int off = Lk - Lq;
  const int D = a.head_dim;
  const int hk = h / (a.heads / a.heads_k);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
  const bool causal = a.is_causal != 0;
  const float scale_log2 = a.softmax_scale * 1.4426950408889634f;

  // ---- K and V of the block: the loads are issued first and stored after the look-up of the column list, so
  // that the two chains of dependent loads wait together (one workgroup per compute unit: nothing else covers them)
  constexpr int NKV = KB * VPR / NTHR;
  Pack8 xk[NKV], xv[NKV];
  {
    const uint16_t *kp = reinterpret_cast<const uint16_t *>(a.k) + (int64_t)(k0 + key0) * a.k_row_stride + (int64_t)hk * a.k_head_stride;
    const uint16_t *vp = reinterpret_cast<const uint16_t *>(a.v) + (int64_t)(k0 + key0) * a.v_row_stride + (int64_t)hk * a.v_head_stride;
#pragma unroll
    for (int i = 0; i < NKV; ++i) {
      const int v = tid + NTHR * i;
      const int key = v / VPR, e = (v - key * VPR) * 8;
      xk[i] = zero_pack8();
      xv[i] = zero_pack8();
      if (key0 + key < Lk && e < D) {
        xk[i] = ld_global16(kp + (int64_t)key * a.k_row_stride + e);
        xv[i] = ld_global16(vp + (int64_t)key * a.v_row_stride + e);
      }
    }
  }

  // ---- the block's column list --------------------------------------------------------------------
  const int Bn = a.lg_block_n;
  const int c = key0 / Bn;
  const int64_t bh = (int64_t)b * a.heads + h;
  int nnz = 0;
  int64_t lbase = 0;
  int start = 0;
  if (c < a.max_cols) {
    nnz = a.col_nnz[bh * a.max_cols + c];
    lbase = a.col_offsets[bh * a.max_cols + c];
    if (causal && nnz > 0) start = lower_bound_wave_i32(a.row_indices + lbase, nnz, key0 - off);  // earlier rows see no key of the block
  }
  const int32_t *list = a.row_indices + lbase + start;
  const int n = nnz - start;  // rows of the list that the block walks
  const int nround = (n + kFwdRoundRows - 1) / kFwdRoundRows;
  const int ntile = (n + 31) >> 5;
  const uint16_t *qg = reinterpret_cast<const uint16_t *>(a.q) + (int64_t)q0 * a.q_row_stride + (int64_t)h * a.q_head_stride;
  int32_t *cntg = ws.cnt + (int64_t)q0 * a.heads + h;       // counter of local row r: cntg[r * heads]
  if (nround == 0) return;
  int rid01[2] = {-1, -1};  // threads 0..127: row ids of rounds 0 and 1
  if (tid < kFwdRoundRows) {
#pragma unroll
    for (int sr = 0; sr < 2; ++sr) {
      const int j = sr * kFwdRoundRows + tid;
      const int r = list[min(j, n - 1)];
      rid01[sr] = tile_row_code(r, j < n, Lq);
    }
  }
  {
    uint16_t *sK = reinterpret_cast<uint16_t *>(smem + SM::oQ);
#pragma unroll
    for (int i = 0; i < NKV; ++i) {
      const int v = tid + NTHR * i;
      const int key = v / VPR, e = (v - key * VPR) * 8;
      *reinterpret_cast<Pack8 *>(sK + key * LDQ + e) = xk[i];
      *reinterpret_cast<Pack8 *>(sV + key * LDQ + e) = xv[i];
    }
  }
  __syncthreads();
  // K of this block as the A operand of S^T = K Q^T: lane -> key (lane % 32) of each 32-key tile
  // (kept in accumulation registers, where the MFMAs read them; S^T and O^T tiles are produced in ordinary registers,
  // where the softmax and the packing read them: no copy between the two register files in the loop)
  u32x4_t kfr[KT][KS];
  {
    const uint16_t *sK = reinterpret_cast<const uint16_t *>(smem + SM::oQ);
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        kfr[kt][ks] = pack8_vec(*reinterpret_cast<const Pack8 *>(sK + (kt * 32 + (lane & 31)) * LDQ + (hh * KS + ks) * 8));
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("" : "+a"(kfr[kt][ks]));
#endif
      }
  }
  if (tid < kFwdRoundRows) {
    sRid[tid] = rid01[0];
    sRid[kFwdRoundRows + tid] = rid01[1];
  }
  __syncthreads();  // K is in registers; the row ids of rounds 0 and 1 are in LDS

  // ---- feeding the tiles: all four waves compute, nothing passes through registers.  Every wave fetches the tile
  // it will work on in the NEXT round with loads that write straight to LDS, issued at the start of a round and
  // awaited at its end.  Threads 0..127 carry the per-row scalars: the row id of round s+2 (it has to be in LDS one
  // round before the tile loads that use it) and the partial slot of round s+1.
  typedef std::integral_constant<int, 0> C0;
  typedef std::integral_constant<int, 1> C1;
  const uint32_t ldsQ = (uint32_t)(uintptr_t)(smem + SM::oQ);
  int n_rid = -1, v_rid = rid01[1], m_rid = -1, m_slot = 0;  // v_rid: the checked row id that was stored last = the one of the next round
  int ft = tid;  // thread index for the feeding code, re-made opaque in every round: what is derived from it must not be kept in registers across rounds
  auto rid_issue = [&](int sr) {
    if (tid < kFwdRoundRows) {
      n_rid = list[min(sr * kFwdRoundRows + ft, n - 1)];  // used (and checked) only when it is stored: no wait for it here
    }
  };
  auto rid_store = [&](int sr) {
    if (tid < kFwdRoundRows) {
      const int j = sr * kFwdRoundRows + ft;
      v_rid = tile_row_code(n_rid, j < n, Lq);
      sRid[(sr & 1) * kFwdRoundRows + ft] = v_rid;
    }
  };
  auto meta_issue = [&](int rid) {  // rid: this thread's row of the round after the current one
    if (tid < kFwdRoundRows) {
      m_rid = rid;
      // every visit of a (row, key block) pair takes one slot of the row (a shared dummy counter for absent
      // rows would serialise the whole grid on one address)
      if (m_rid >= 0) m_slot = atomicAdd(cntg + (int64_t)m_rid * a.heads, 1);
    }
  };
  auto meta_store = [&](int sr) {
    if (tid < kFwdRoundRows) {
      sRow[(sr & 1) * kFwdRoundRows + ft] = m_rid;
      // where the visit's partial goes, as an index of partial rows (it fits 32 bits: 2^31 partial rows would be half a
      // terabyte), or -1 for a row that is absent or has more visits than the caller's bound
      sSlot[(sr & 1) * kFwdRoundRows + ft] = (m_rid >= 0 && m_slot < ws.cap) ? ((q0 + m_rid) * a.heads + h) * ws.cap + m_slot : -1;
    }
  };
  auto tile_issue = [&](int sr) {  // tile `wave` of round sr
    constexpr int RPI = 64 / VPR, NI = 32 / RPI;  // tile rows per instruction, instructions per tile
    const int fl = ft & 63, rl = fl / VPR, p = fl - rl * VPR;
    const uint32_t dst = ldsQ + (uint32_t)__builtin_amdgcn_readfirstlane(((sr & 1) * 4 + wave) * (int)TB);
    const uint32_t qs = (uint32_t)a.q_row_stride;  // (32 x 32 -> 64-bit product: one instruction)
    // Absent rows and features past head_dim are fetched from a row and a piece that exist (tile_row_code): every load
    // is unconditional; the scores of absent rows are masked, and K is zero in the features past head_dim.
    int src[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) src[i] = sRid[(sr & 1) * kFwdRoundRows + wave * 32 + i * RPI + rl] & 0x7fffffff;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const uint32_t e = (uint32_t)min((p ^ tile_swz<HD>(i * RPI + rl)) * 8, D - 8);
      global_to_lds16(qg + ((uint64_t)(uint32_t)src[i] * qs + e), dst + (uint32_t)(i * RPI * RB));
    }
  };
  meta_issue(rid01[0]);
  tile_issue(0);
  meta_store(0);
  wait_all_loads();
  __syncthreads();

  lds_cu16 *trV = tr_lane_base(sV, LDQ, lane) + 4 * hh * LDQ;
  uint16_t *sOut = reinterpret_cast<uint16_t *>(smem + SM::oOut) + (size_t)wave * 32 * LDO;
  // byte address of this lane's row (lane % 32 of the wave's tile, buffer 0), piece hh * KS; the other pieces
  // are an exclusive-or on the piece bits
  const uint32_t qrow = ldsQ + (uint32_t)wave * TB + (uint32_t)((lane & 31) * RB + (((hh * KS) ^ tile_swz<HD>(lane & 31)) * 16));

  // LDS addresses are one register (made opaque to the compiler where it is used) plus an offset in the instruction:
  // left alone, the compiler computes every address of a tile outside the loop and parks them in spare registers
  auto opaque = [](uint32_t &x) {
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("" : "+v"(x));
#else
    (void)x;
#endif
  };
  const uint32_t ldsOut = (uint32_t)(uintptr_t)sOut, ldsRow = (uint32_t)(uintptr_t)(smem + SM::oRow) + (uint32_t)(wave * 32 * 4);
  // A tile in two steps: the products and the softmax (the partial goes to the wave's LDS tile), then the stores.
  // Between them the round waits for the loads of the next tile: one counter covers loads and stores alike, so
  // stores issued before that wait would be waited for as well instead of completing under the next round.
  float t_m = 0.f, t_l = 0.f;
  int t_rid = -1;
  auto compute_tile = [&](auto pc) {
    constexpr int PB = decltype(pc)::value;
    const int sidx = PB * kFwdRoundRows + wave * 32 + (lane & 31);
    const int rid = sRow[sidx];
    // this lane's query row as the B operand
    Pack8 qb[KS];
    uint32_t bq = qrow;
    opaque(bq);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qb[ks] = lds_read16((bq ^ (uint32_t)(ks * 16)) + (uint32_t)(PB * 4) * TB);
    __builtin_amdgcn_sched_barrier(0);
    // block-local softmax of the row, log2 domain; keys beyond lim are masked: in a tile that has such pairs S^T starts
    // from 0 / -inf per pair and the products add to that (the exponential of -inf is 0), in the others it starts from
    // nothing, and the softmax has no comparison in either
    const int lim = rid < 0 ? -1 : min(causal ? rid + off : 0x7fffffff, Lk - 1) - key0;  // last visible key, relative
    f32x16 st[KT];  // S^T: register i of tile kt <-> key kt*32 + acc_row(i, hh), this lane's row
    const bool masked = !__all(lim >= KB - 1);
    if (masked) {
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int jrel = kt * 32 + 8 * (i >> 2) + (i & 3) + 4 * hh;
          st[kt][i] = jrel <= lim ? 0.f : -INFINITY;
        }
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) mfma32_a_acc<T, false>(st[kt], kfr[kt][0], qb[0]);
    } else {
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) mfma32_a_acc<T, true>(st[kt], kfr[kt][0], qb[0]);
    }
#pragma unroll
    for (int ks = 1; ks < KS; ++ks)
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) mfma32_a_acc<T, false>(st[kt], kfr[kt][ks], qb[ks]);
    static_assert(KT == 2 || KT == 4, "key blocks of 64 or 128 keys");
    if constexpr (KT == 2) {
      mfma_results_ready(st[0], st[1]);
    } else {
      mfma_results_ready(st[0], st[1]);
      mfma_results_ready(st[2], st[3]);
    }
    __builtin_amdgcn_sched_barrier(0);
    // V^T operands of the first half of the feature tiles: their LDS latency runs under the softmax arithmetic
    Pack8 vt[NDT][KT][2];
#pragma unroll
    for (int dt = 0; dt < NDT / 2; ++dt)
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const int lo = (kt * 32 + 16 * s2) * LDQ + dt * 32;
          vt[dt][kt][s2] = tr_frag8_at(trV, lo, lo + 8 * LDQ);
        }
    __builtin_amdgcn_sched_barrier(0);
    // (the scores stay raw: the scale, positive, goes into the exponent's multiply-add)
    float m = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) m = fmaxf(m, st[kt][i]);
    m = max_xor32_f(m) * scale_log2;
    const float m_use = m == -INFINITY ? 0.f : m;
    float l = 0.f;
    Pack8 pf[KT][2];  // P^T as the B operand of O^T = V^T P^T, straight from the accumulators
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const float p0 = __builtin_amdgcn_exp2f(fmaf(st[kt][8 * s2 + 2 * w], scale_log2, -m_use));
          const float p1 = __builtin_amdgcn_exp2f(fmaf(st[kt][8 * s2 + 2 * w + 1], scale_log2, -m_use));
          l += p0 + p1;
          pf[kt][s2].w[w] = pack2<T>(p0, p1);
        }
    l = sum_xor32_f(l);
    __builtin_amdgcn_sched_barrier(0);
    // O^T[d][row] = sum_key V^T[d][key] P^T[key][row]; register i of d-tile dt <-> d = dt*32 + acc_row(i, hh)
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      if (dt == 0) {  // second half of the V^T operands, under the first products
#pragma unroll
        for (int d2 = NDT / 2; d2 < NDT; ++d2)
#pragma unroll
          for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
              const int lo = (kt * 32 + 16 * s2) * LDQ + d2 * 32;
              vt[d2][kt][s2] = tr_frag8_at(trV, lo, lo + 8 * LDQ);
            }
        __builtin_amdgcn_sched_barrier(0);
      }
      f32x16 o;
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          if (kt == 0 && s2 == 0)
            mfma32_vv<T, true>(o, vt[dt][kt][s2], pf[kt][s2]);
          else
            mfma32_vv<T, false>(o, vt[dt][kt][s2], pf[kt][s2]);
        }
      mfma_results_ready(o);
      // to the wave's row-major output tile, four features (8 bytes) at a time
      uint32_t bo = ldsOut + (uint32_t)(((lane & 31) * LDO + 4 * hh) * 2);
      opaque(bo);
#pragma unroll
      for (int g = 0; g < 4; ++g)
        lds_write_vec<uint2>(bo + (uint32_t)((dt * 32 + 8 * g) * 2), make_uint2(pack2<T>(o[4 * g], o[4 * g + 1]), pack2<T>(o[4 * g + 2], o[4 * g + 3])));
      __builtin_amdgcn_sched_barrier(0);
    }
    t_m = m;
    t_l = l;
    t_rid = rid;
  };
  auto store_tile = [&](auto pc) {
    constexpr int PB = decltype(pc)::value;
    const int sidx = PB * kFwdRoundRows + wave * 32 + (lane & 31);
    const int rid = t_rid;
    const float m = t_m, l = t_l;
    // header of the partial
    const int pidx = sSlot[sidx];
    if (pidx >= 0 && hh == 0) ws.hdr[pidx] = make_float4(m, l, __int_as_float(nb), 0.f);
    wave_lds_fence();
    // rows leave as 16-byte pieces: lane -> (row 4k + lane / 16, features 8 * (lane % 16))
    if ((lane & 15) * 8 < D) {
      uint32_t br = ldsRow + (uint32_t)((lane >> 4) * 4), bx = ldsOut + (uint32_t)(((lane >> 4) * LDO + (lane & 15) * 8) * 2);
      opaque(br);
      opaque(bx);
      // all indices, then all rows, then the stores: one LDS latency each instead of sixteen in a chain
      int p2[8];
      Pack8 x[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) p2[k] = lds_read_vec<int>(br + (uint32_t)((PB * kFwdRoundRows + 4 * k) * 4) + (uint32_t)(SM::oSlot - SM::oRow));
#pragma unroll
      for (int k = 0; k < 8; ++k) x[k] = lds_read16(bx + (uint32_t)(4 * k * LDO * 2));
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (p2[k] >= 0) st_stream16(ws.part + ((uint64_t)(uint32_t)p2[k] * (uint32_t)D + (uint32_t)((lane & 15) * 8)), x[k]);
    }
    wave_lds_fence();
  };

  auto round = [&](auto pc, int r) {
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("" : "+v"(ft));
#endif
    rid_issue(r + 2);
    meta_issue(v_rid);
    tile_issue(r + 1);
    const bool mine = 4 * r + wave < ntile;
    if (mine) compute_tile(pc);
    wait_all_loads();
    meta_store(r + 1);
    rid_store(r + 2);
    if (mine) store_tile(pc);
    __syncthreads();  // round r + 1 is in LDS; everyone is done with round r
  };
  for (int r = 0; r < nround; r += 2) {
    round(C0{}, r);
    if (r + 1 < nround) round(C1{}, r + 1);
  }
}

// One 16-lane group per (row, head), four per wave, sixteen per block of 256: a row's chain of dependent steps (count,
// headers, order, rows) is mostly waiting, so a wave runs four of them side by side.  Lane li of a group owns the
// 16-byte piece li of the row.
template <typename T>
__global__ __launch_bounds__(256) void attn_fwd_combine_kernel(fmoba_attn_fwd_args a, FwdWs ws, int capl) {
  extern __shared__ __attribute__((aligned(16))) int sOrdAll[];  // [16 groups][capl]: slot of the partial of rank r
  __shared__ float sWgt[16][16], sWl[16][16];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, grp = lane >> 4, li = lane & 15;
  const int sg = wv * 4 + grp;  // group of the block
  int *sOrd = sOrdAll + (size_t)sg * capl;
  const int64_t total = (int64_t)a.total_q * a.heads;
  const int64_t rh_raw = (int64_t)blockIdx.x * 16 + sg;  // (global row) * heads + head
  const bool valid = rh_raw < total;
  const int64_t rh = valid ? rh_raw : total - 1;
  const int64_t row = rh / a.heads;
  const int h = (int)(rh - row * a.heads);
  const int D = a.head_dim;
  const int nall = valid ? ws.cnt[rh] : 0;
  const int n = min(nall, ws.cap);
  if (nall > ws.cap && li == 0 && a.visits_overflow != nullptr) atomicMax(a.visits_overflow, nall);  // visits were dropped
  int nmax = max(n, __shfl_xor(n, 16, 64));
  nmax = max(nmax, __shfl_xor(nmax, 32, 64));  // the wave walks the longest of its four rows
  const int c8 = li * 8;
  const bool mine = c8 < D;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  float L = 0.f, M = -INFINITY;
  const float4 *hdr = ws.hdr + rh * ws.cap;
  const uint16_t *part = ws.part + rh * ws.cap * D;
  // The slot a visit got is arbitrary (a counter handed it out), the sum must not depend on it: every partial gets
  // its rank in ascending key-block order over the WHOLE row (equal ids, a malformed pattern, are ordered by slot),
  // and the partials are merged in rank order, 16 at a time.
  group_rank_order(reinterpret_cast<const int *>(hdr) + 2, 4, n, nmax, sOrd, lane);
  for (int base = 0; base < nmax; base += 16) {
    const int cntb = min(16, max(n - base, 0));
    float mj = -INFINITY, lj = 0.f;
    int slot = 0;
    if (li < cntb) {
      slot = sOrd[base + li];
      const float4 x = hdr[slot];
      mj = x.x;
      lj = x.y;
    }
    float mb = mj;
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) mb = fmaxf(mb, __shfl_xor(mb, o, 64));
    const float Mn = fmaxf(M, mb);
    const float Mu = Mn == -INFINITY ? 0.f : Mn;
    const float resc = __builtin_amdgcn_exp2f(M - Mu);  // M = -inf: nothing accumulated yet, factor 0 on zeros
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] *= resc;
    L *= resc;
    M = Mn;
    const float wj = (li < cntb) ? __builtin_amdgcn_exp2f(mj - Mu) : 0.f;
    wave_lds_fence();
    if (li < cntb) {
      sWgt[sg][li] = wj;
      sWl[sg][li] = wj * lj;
    }
    wave_lds_fence();
    // sums in rank order: every lane of the group adds the same sequence
    for (int t = 0; t < cntb; ++t) L += sWl[sg][t];
    if (mine) {
      auto add = [&](const Pack8 &x, float w) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          acc[2 * k] = fmaf(w, elem_to_float<T>((uint16_t)(x.w[k] & 0xffffu)), acc[2 * k]);
          acc[2 * k + 1] = fmaf(w, elem_to_float<T>((uint16_t)(x.w[k] >> 16)), acc[2 * k + 1]);
        }
      };
      int t = 0;
      for (; t + 4 <= cntb; t += 4) {  // independent loads, four in flight
        Pack8 x[4];
        float w[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          x[u] = ld_stream16(part + (int64_t)sOrd[base + t + u] * D + c8);
          w[u] = sWgt[sg][t + u];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) add(x[u], w[u]);
      }
      for (; t < cntb; ++t) add(ld_stream16(part + (int64_t)sOrd[base + t] * D + c8), sWgt[sg][t]);
    }
  }
  if (!valid) return;
  const bool empty = !(L > 0.f);
  const float inv = empty ? 0.f : 1.f / L;
  if (mine) {
    Pack8 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) o.w[k] = pack2<T>(acc[2 * k] * inv, acc[2 * k + 1] * inv);
    *reinterpret_cast<Pack8 *>(reinterpret_cast<uint16_t *>(a.out) + row * a.o_row_stride + (int64_t)h * a.o_head_stride + c8) = o;
  }
  if (li == 0) a.softmax_lse[(int64_t)h * a.total_q + row] = empty ? INFINITY : (M + __builtin_amdgcn_logf(L)) * 0.6931471805599453f;
}

__global__ void fwd_empty_kernel(void *out, float *lse, int64_t n_out_words, int64_t n_lse) {
  const int64_t i0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, st = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = i0; i < n_out_words; i += st) reinterpret_cast<uint32_t *>(out)[i] = 0u;
  for (int64_t i = i0; i < n_lse; i += st) lse[i] = INFINITY;
}

__global__ void fwd_zero_i32_kernel(int32_t *p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0;
}

// visits per (row, head) of a pattern: grid over list entries is not possible without the segment of each
// entry, so one workgroup walks one column list
__global__ __launch_bounds__(256) void csc_row_visits_kernel(fmoba_attn_fwd_args a, int32_t *cnt, int kb) {
  const int c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int Lk = a.cu_seqlens_k[b + 1] - a.cu_seqlens_k[b];
  const int64_t bh = (int64_t)b * a.heads + h;
  const int nnz = a.col_nnz[bh * a.max_cols + c];
  const int32_t *list = a.row_indices + a.col_offsets[bh * a.max_cols + c];
  // key blocks of this column that exist in the sequence
  const int key_lo = c * a.lg_block_n, key_hi = min(Lk, key_lo + a.lg_block_n);
  const int nblk = key_hi > key_lo ? (key_hi - key_lo + kb - 1) / kb : 0;
  if (nblk == 0) return;
  for (int i = threadIdx.x; i < nnz; i += 256) {
    const int r = list[i];
    if (r >= 0 && r < Lq) atomicAdd(&cnt[(int64_t)(q0 + r) * a.heads + h], nblk);
  }
}
__global__ __launch_bounds__(256) void max_i32_kernel(const int32_t *p, int64_t n, int32_t *out) {
  int m = 0;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) m = max(m, p[i]);
  for (int o = 32; o >= 1; o >>= 1) m = max(m, __shfl_xor(m, o, 64));
  if ((threadIdx.x & 63) == 0 && m > 0) atomicMax(out, m);
}

static inline size_t fwd_align256(size_t x) { return (x + 255) & ~(size_t)255; }
static inline int fwd_key_block(int lg_block_n) { return lg_block_n % 128 == 0 ? 128 : 64; }

// the row-block form (attn_fwd_rows.hip)
bool fwd_rows_feasible(const fmoba_attn_fwd_args &a);
size_t fwd_rows_workspace_bytes(const fmoba_attn_fwd_args &a);
int run_fwd_rows(const fmoba_attn_fwd_args &a, int phases, hipStream_t s);

// Which form runs.  The row-block form multiplies every row of a 128-row block with every chunk that
// any of its rows selected, the column form only the selected pairs but pays a partial result per
// visit: the first wins while a row selects more than about a fifth of the chunks it may see (64-key blocks) or
// more than about three eighths of them (128-key blocks, whose visits cost the column form less per key).
static bool fwd_use_rows(const fmoba_attn_fwd_args &a) {
  if (a.head_dim > 128) return true;  // head dimensions above 128 only have the row-block form
  if (a.fwd_mode == 1) return false;
  if (!fwd_rows_feasible(a)) return false;
  if (a.fwd_mode == 2) return true;
  const int64_t chunks_per_seq = std::max<int64_t>(1, ceil_div64(ceil_div64(std::max(a.total_k, 1), a.batch), a.lg_block_n));
  const int64_t chunks_per_row = std::max<int64_t>(1, (int64_t)a.max_visits_per_row * fwd_key_block(a.lg_block_n) / a.lg_block_n);
  const int64_t seen = a.is_causal ? (chunks_per_seq + 1) / 2 : chunks_per_seq;
  return chunks_per_row * (fwd_key_block(a.lg_block_n) == 128 ? kFwdRowsDensity128 : kFwdRowsDensity64) >= seen * 10;
}

template <typename T, int HD, int KB>
static int launch_fwd_col(const fmoba_attn_fwd_args &a, const FwdWs &ws, hipStream_t s) {
  auto kern = attn_fwd_col_kernel<T, HD, KB>;
  const size_t smem = FwdColSmem<HD, KB>::bytes;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("attn_fwd: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  const int64_t items = (int64_t)a.batch * a.heads * ceil_div(a.max_seqlen_k, KB);
  if (items >= ((int64_t)1 << 31)) {
    set_error("attn_fwd: too many (sequence, head, key block) work items");
    return 1;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)items), dim3(256), smem, s, a, ws);
  return 0;
}
template <typename T>
static int run_fwd(const fmoba_attn_fwd_args &a, const FwdWs &ws, int phases, hipStream_t s) {
  const int64_t rows = (int64_t)a.total_q * a.heads;
  if (phases & FMOBA_FWD_COLUMNS) {
    hipLaunchKernelGGL(fwd_zero_i32_kernel, dim3(512), dim3(256), 0, s, ws.cnt, rows);
    const int kb = fwd_key_block(a.lg_block_n);
    int rc;
    if (a.head_dim <= 64)
      rc = kb == 128 ? launch_fwd_col<T, 64, 128>(a, ws, s) : launch_fwd_col<T, 64, 64>(a, ws, s);
    else
      rc = kb == 128 ? launch_fwd_col<T, 128, 128>(a, ws, s) : launch_fwd_col<T, 128, 64>(a, ws, s);
    if (rc) return rc;
  }
  if (phases & FMOBA_FWD_COMBINE) {
    const int capl = combine_order_entries(ws.cap);
    const size_t smem = (size_t)16 * capl * 4;
    auto kern = attn_fwd_combine_kernel<T>;
    if (smem > 32 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
      set_error("attn_fwd: a row with up to %d visits needs %zu bytes of LDS for the order of its partial results", ws.cap, smem);
      return 2;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)((rows + 15) / 16)), dim3(256), smem, s, a, ws, capl);
  }
  return 0;
}

}  // namespace fmoba

extern "C" int32_t fmoba_attn_fwd_key_block(int32_t lg_block_n) { return fmoba::fwd_key_block(lg_block_n); }

static size_t fwd_cols_workspace_bytes(int32_t total_q, int32_t heads, int32_t head_dim, int32_t max_visits_per_row) {
  using namespace fmoba;
  if (total_q <= 0 || heads <= 0 || head_dim <= 0 || max_visits_per_row <= 0) return 256;
  const size_t rows = (size_t)total_q * heads;
  return fwd_align256((rows + 1) * 4) + fwd_align256(rows * max_visits_per_row * 16) + fwd_align256(rows * max_visits_per_row * head_dim * 2) + 256;
}

extern "C" size_t fmoba_attn_fwd_workspace_bytes(const fmoba_attn_fwd_args *a) {
  using namespace fmoba;
  if (a == nullptr || a->total_q <= 0 || a->heads <= 0 || a->head_dim <= 0 || a->batch <= 0 || a->lg_block_n <= 0) return 256;
  if (fwd_use_rows(*a)) return fwd_rows_workspace_bytes(*a);
  return fwd_cols_workspace_bytes(a->total_q, a->heads, a->head_dim, a->max_visits_per_row);
}

extern "C" int32_t fmoba_attn_fwd_uses_row_blocks(const fmoba_attn_fwd_args *a) {
  using namespace fmoba;
  if (a == nullptr || a->total_q <= 0 || a->heads <= 0 || a->head_dim <= 0 || a->batch <= 0 || a->lg_block_n <= 0) return 0;
  return fwd_use_rows(*a) ? 1 : 0;
}

static int fwd_check_common(const fmoba_attn_fwd_args *a) {
  using namespace fmoba;
  FMOBA_REQUIRE(a != nullptr, "attn_fwd: null args");
  FMOBA_REQUIRE(a->dtype == FMOBA_DTYPE_F16 || a->dtype == FMOBA_DTYPE_BF16, "FlashMoBA only support fp16 and bf16 data type");
  FMOBA_REQUIRE(a->batch > 0, "batch size must be positive");
  FMOBA_REQUIRE(a->head_dim > 0 && a->head_dim <= 256, "FlashMoBA forward only supports head dimension at most 256");
  FMOBA_REQUIRE(a->head_dim % 8 == 0, "query, key, value, and out_ must have a head_size that is a multiple of 8");
  FMOBA_REQUIRE(a->heads > 0 && a->heads_k > 0 && a->heads % a->heads_k == 0, "Number of heads in key/value must divide number of heads in query");
  FMOBA_REQUIRE(a->lg_block_m >= 128 && a->lg_block_m <= 1024, "m_lg_block_dim must be at least 128 and at most 1024");
  FMOBA_REQUIRE(a->lg_block_m % 64 == 0, "m_lg_block_dim must be a multiple of 64");
  FMOBA_REQUIRE(a->lg_block_n > 0 && a->lg_block_n % 64 == 0, "n_lg_block_dim must be a multiple of 64");
  FMOBA_REQUIRE(a->total_q >= 0 && a->total_k >= 0 && a->max_seqlen_q >= 0 && a->max_seqlen_k >= 0 && a->max_cols >= 0, "negative size");
  FMOBA_REQUIRE(a->cu_seqlens_q && a->cu_seqlens_k, "attn_fwd: null cu_seqlens pointer");
  FMOBA_REQUIRE(a->batch <= 65535 && a->heads <= 65535, "attn_fwd: batch/heads too large for the launch grid");
  return 0;
}

extern "C" int fmoba_csc_max_row_visits(const fmoba_attn_fwd_args *a, int32_t *counts, int32_t *max_out, void *stream) {
  using namespace fmoba;
  if (int rc = fwd_check_common(a)) return rc;
  FMOBA_REQUIRE(counts && max_out, "csc_max_row_visits: null output pointer");
  hipStream_t s = (hipStream_t)stream;
  const int64_t rows = (int64_t)a->total_q * a->heads;
  hipLaunchKernelGGL(fwd_zero_i32_kernel, dim3(256), dim3(256), 0, s, counts, rows);
  hipLaunchKernelGGL(fwd_zero_i32_kernel, dim3(1), dim3(64), 0, s, max_out, (int64_t)1);
  if (rows > 0 && a->max_cols > 0 && a->total_k > 0) {
    FMOBA_REQUIRE(a->col_offsets && a->col_nnz && a->row_indices, "csc_max_row_visits: null CSC pointer");
    hipLaunchKernelGGL(csc_row_visits_kernel, dim3(a->max_cols, a->heads, a->batch), dim3(256), 0, s, *a, counts, fwd_key_block(a->lg_block_n));
    hipLaunchKernelGGL(max_i32_kernel, dim3(256), dim3(256), 0, s, counts, rows, max_out);
  }
  FMOBA_LAUNCH_CHECK("csc_max_row_visits");
  return 0;
}

extern "C" int fmoba_attn_fwd(const fmoba_attn_fwd_args *a, void *stream) { return fmoba_attn_fwd_phases(a, 3, stream); }

extern "C" int fmoba_attn_fwd_phases(const fmoba_attn_fwd_args *a, int32_t phases, void *stream) {
  using namespace fmoba;
  if (int rc = fwd_check_common(a)) return rc;
  FMOBA_REQUIRE(phases > 0 && phases <= 3, "attn_fwd: phases must be a mask of bits 1, 2");
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
  FMOBA_REQUIRE(a->q_row_stride < ((int64_t)1 << 31), "attn_fwd: q_row_stride must be below 2^31 elements");
  FMOBA_REQUIRE(((uintptr_t)a->q % 16) == 0 && ((uintptr_t)a->k % 16) == 0 && ((uintptr_t)a->v % 16) == 0 && ((uintptr_t)a->out % 16) == 0,
                "attn_fwd: q, k, v and out must be 16-byte aligned");
  FMOBA_REQUIRE(a->max_visits_per_row > 0, "attn_fwd: max_visits_per_row must be positive");
  FMOBA_REQUIRE(a->fwd_mode >= 0 && a->fwd_mode <= 2, "attn_fwd: fwd_mode must be 0 (automatic), 1 (columns) or 2 (row blocks)");
  FMOBA_REQUIRE(a->fwd_mode != 1 || a->head_dim <= 128, "attn_fwd: head dimensions above 128 only have the row-block form");
  FMOBA_REQUIRE((a->fwd_mode != 2 && a->head_dim <= 128) || fwd_rows_feasible(*a), "attn_fwd: the row-block form does not take this shape (more than %d chunks or %d keys per sequence)",
                32 * 128, 64 * 4096);
  const size_t need = fmoba_attn_fwd_workspace_bytes(a);
  FMOBA_REQUIRE(a->workspace != nullptr && a->workspace_bytes >= need, "attn_fwd: workspace too small (%zu < %zu)", a->workspace_bytes, need);
  if (fwd_use_rows(*a)) {
    if (int rc = run_fwd_rows(*a, phases, s)) return rc;
    FMOBA_LAUNCH_CHECK("attn_fwd");
    return 0;
  }
  const size_t rows = (size_t)a->total_q * a->heads;
  FMOBA_REQUIRE(rows * (size_t)a->max_visits_per_row < ((size_t)1 << 31),
                "attn_fwd: %zu partial rows exceed the 2^31 the column form indexes (their workspace would not fit any device either)",
                rows * (size_t)a->max_visits_per_row);
  uintptr_t p = ((uintptr_t)a->workspace + 255) & ~(uintptr_t)255;
  FwdWs ws;
  ws.cap = a->max_visits_per_row;
  ws.cnt = reinterpret_cast<int32_t *>(p);
  p += fwd_align256((rows + 1) * 4);
  ws.hdr = reinterpret_cast<float4 *>(p);
  p += fwd_align256(rows * ws.cap * 16);
  ws.part = reinterpret_cast<uint16_t *>(p);
  int rc = a->dtype == FMOBA_DTYPE_BF16 ? run_fwd<bf16_t>(*a, ws, phases, s) : run_fwd<f16_t>(*a, ws, phases, s);
  if (rc) return rc;
  FMOBA_LAUNCH_CHECK("attn_fwd");
  return 0;
}
