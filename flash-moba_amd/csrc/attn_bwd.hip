// Sparse attention backward over a CSC pattern, without a single global atomic.
//
//   bwd_prep_kernel      : delta[row] = sum_d dO*O (fp32).
//   attn_bwd_dkdv_kernel : COLUMN-stationary.  One workgroup per (64-key block, head,
//                          sequence) keeps K and V of the block in registers and walks the block's
//                          ascending row list in gathered 32-row tiles:
//                            S = Q K^T, dP = dO V^T             (A = gathered rows, B = K / V halves)
//                            P = exp2(S*scale*log2e - LSE*log2e), dS = P o (dP - delta)
//                            dV^T += dO^T P, dK^T += Q^T dS     (P, dS feed the MFMA from registers;
//                                                                dO^T, Q^T via transposing LDS reads)
//                            dQ^T_partial = K^T dS^T            (per visit of a (row, key block) pair)
//                          dK/dV live in accumulator registers for the whole list and are written
//                          once.  For dQ the kernel leaves either its dS tiles (16-bit, indexed by
//                          row-list position) or, per visit, a dQ partial row (16-bit, unscaled) in a
//                          slot that the row hands out from a counter.
//   attn_bwd_dq_kernel   : dQ from the dS tiles, one workgroup per 128 query rows, dQ in registers
//                          (patterns in which a 128-row block meets a dozen rows or more per step).
//   attn_bwd_dq_combine_kernel : dQ from the partials, sixteen lanes per (row, head) add them in ascending
//                          key-block order and scales.  Work and traffic are proportional to
//                          the number of visits, whatever the number of chunks per sequence.
// The dK/dV kernel runs four waves of 512 registers, one per SIMD, and all four compute: two pairs
// (one wave per 32-key half) that take alternate pairs of tiles and add their sums at the end.  A wave keeps
// 32 keys x head_dim of dK^T and dV^T plus its K and V operands in registers, which leaves no room for a
// second wave on the SIMD, so nothing moves data through registers: the gathered Q / dO rows go from global
// memory straight to LDS (global_load_lds), one round (four tiles) ahead.
#include "fmoba_common.h"

#include <type_traits>
#include <utility>

namespace fmoba {

constexpr int kBwdRoundRows = 128;  // rows of a column list the workgroup takes per round: two 32-row tiles per wave pair

template <int HD>
struct BwdSmem {
  // The gathered Q / dO tiles have rows of exactly HD elements (the loads that fill them write 64 lanes x 16 bytes
  // to consecutive addresses) and are swizzled instead of padded: the 16-byte piece c of tile row r lies at piece
  // c ^ tile_swz<HD>(r).  With that, the 16-byte row reads (lane -> row lane % 32) and the transposing 8-byte
  // reads both spread over all banks.
  static constexpr int LDQ = HD + 16;  // elements, K and V while they are read into registers (plain padded rows)
  static constexpr int LDS_ = 32 + 8;  // elements, dS^T tile rows [key][32 rows]
  static constexpr size_t tileBytes = (size_t)32 * HD * 2;
  static constexpr size_t oQ = 0;                                   // [2 buffers][4 tiles][32][HD]
  static constexpr size_t odO = oQ + 8 * tileBytes;
  static constexpr size_t odS = odO + 8 * tileBytes;               // partials form: [2 pairs][2 tile slots][64 keys][LDS_] or [2 tile slots][128 keys][LDS_]; dS form: [4 waves][32 keys][LDS_]
  static constexpr size_t oRid = odS + (size_t)2 * 2 * 64 * LDS_ * 2;  // int[2 buffers][128]: row ids, one round before the rest
  static constexpr size_t oRow = oRid + 2 * kBwdRoundRows * 4;     // int[2 buffers][128]
  static constexpr size_t oSlot = oRow + 2 * kBwdRoundRows * 4;
  static constexpr size_t oLse = oSlot + 2 * kBwdRoundRows * 4;    // LSE * log2(e)
  static constexpr size_t oDelta = oLse + 2 * kBwdRoundRows * 4;
  static constexpr size_t bytes = oDelta + 2 * kBwdRoundRows * 4;
  static constexpr int LDR = HD + 4;  // floats, output transpose buffer [2][64 or 128 keys][LDR]
  static_assert((size_t)2 * 128 * LDQ * 2 <= 16 * tileBytes, "K and V pass through the tiles");
  static_assert(bytes <= 160 * 1024, "LDS of one compute unit");
};

struct BwdWs {
  int32_t *cnt;    // [total_q * heads] visits handed out per (row, head)
  int32_t *pid;    // [total_q * heads * cap] key block id of each partial
  uint16_t *part;  // [total_q * heads * cap][head_dim] dQ partials (unscaled)
  int32_t cap;
  uint16_t *ds;    // dS tiles (row-stationary dQ form): [row list position / 32][key of the column / 8][position % 32][8 keys]
};

// a * b of two values below 2^24, b the same in every lane: one full-rate instruction (a 32-bit multiply takes four
// times as long)
__device__ __forceinline__ uint32_t mul24_u32(uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
  uint32_t d;
  asm("v_mul_u32_u24 %0, %1, %2" : "=v"(d) : "v"(a), "s"(b));
  return d;
#else
  return a * b;
#endif
}

// DQP = true: dQ partials per visit (for the combine kernel); false: dS^T tiles to ws.ds (for the row-stationary dQ kernel).
// KB = 1: the workgroup owns 64 keys, wave pair px takes tiles 2 px, 2 px + 1 of a round and wave kq of the pair the
// key half kq.  KB = 2 (columns of a multiple of 128 keys, whose two 64-key blocks share one row list): it owns 128
// keys, every wave takes all four tiles for its key quarter kq, so a gathered row serves twice the keys and a visit
// leaves one dQ partial instead of two.
// NEAR: the host has checked that a gathered row's place in q and dout is a 32-bit byte offset from the sequence's first
// row that one 24-bit multiply makes (launch_dkdv); otherwise the loads take 64-bit addresses per lane.
template <typename T, int HD, bool DQP, int KB, bool NEAR>
__global__ __launch_bounds__(256) void attn_bwd_dkdv_kernel(fmoba_attn_bwd_args a, BwdWs ws) {
  typedef BwdSmem<HD> SM;
  constexpr int KS = HD / 16, LDQ = SM::LDQ, LDS_ = SM::LDS_, NDT = HD / 32, VPR = HD / 8, LDR = SM::LDR;
  constexpr int NKEY = 64 * KB;         // keys of the workgroup
  constexpr int NDH = NDT / (2 * KB);   // feature tiles of dQ per wave
  constexpr int LDH = NDH * 32 + 8;     // elements, per-wave dQ part-row tile [32][LDH]
  static_assert(NDH >= 1, "128-key workgroups need head_dim 128");
  static_assert((size_t)KB * 32 * LDH * 2 <= SM::tileBytes, "the dQ part rows of KB waves pass through a tile");
  constexpr uint32_t TB = (uint32_t)SM::tileBytes;
  constexpr int RB = HD * 2;    // bytes of a tile row
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  int *sRid = reinterpret_cast<int *>(smem + SM::oRid);
  int *sRow = reinterpret_cast<int *>(smem + SM::oRow);
  int *sSlot = reinterpret_cast<int *>(smem + SM::oSlot);
  float *sLse = reinterpret_cast<float *>(smem + SM::oLse);
  float *sDelta = reinterpret_cast<float *>(smem + SM::oDelta);

  const PairItem item = xcd_pair_item(blockIdx.x, a.batch * a.heads, (a.max_seqlen_k + NKEY - 1) / NKEY, (int64_t)a.max_seqlen_q * HD * 4 >= kOnePairBytes);
  const int nb = item.idx, b = item.pair / a.heads, h = item.pair - b * a.heads;
  const int key0 = nb * NKEY;
  // One workgroup per compute unit: nothing covers the dependent loads before the first round, so their chain is kept
  // short.  Where the block's column list lies depends on nothing that is loaded: asked for together with the
  // sequence bounds.
  const int Bn = a.lg_block_n;
  const int c = key0 / Bn;
  const int64_t bh = (int64_t)b * a.heads + h;
  int nnz = 0;
  int64_t lbase = 0;
  if (c < a.max_cols) {
    nnz = a.col_nnz[bh * a.max_cols + c];
    lbase = a.col_offsets[bh * a.max_cols + c];
  }
  const int k0 = a.cu_seqlens_k[b], Lk = a.cu_seqlens_k[b + 1] - k0;
  if (key0 >= Lk) return;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int off = Lk - Lq;
  const int D = a.head_dim;
  const int hk = h / (a.heads / a.heads_k);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
  const int kq = KB == 1 ? (wave & 1) : wave;  // this wave's 32 keys of the block, and its share of the dQ features
  const int px = KB == 1 ? (wave >> 1) : 0;    // KB = 1: wave pair, takes tiles 2 px and 2 px + 1 of every round
  const bool causal = a.is_causal != 0;
  const float scale_log2 = a.softmax_scale * 1.4426950408889634f;
  constexpr float kLog2e = 1.4426950408889634f;

  // ---- the key block: through LDS into registers.  The loads are issued first and stored after the look-up of
  // the column list below, so that the two chains of dependent loads wait together (one workgroup per compute
  // unit: nothing else covers them) ----------------------------------------------
  constexpr int NKV = NKEY * VPR / 256;
  Pack8 xk[NKV], xv[NKV];
  {
    const uint16_t *kp = reinterpret_cast<const uint16_t *>(a.k) + (int64_t)(k0 + key0) * a.k_row_stride + (int64_t)hk * a.k_head_stride;
    const uint16_t *vp = reinterpret_cast<const uint16_t *>(a.v) + (int64_t)(k0 + key0) * a.v_row_stride + (int64_t)hk * a.v_head_stride;
#pragma unroll
    for (int i = 0; i < NKV; ++i) {
      const int v = tid + 256 * i;
      const int key = v / VPR, e = (v - key * VPR) * 8;
      xk[i] = zero_pack8();
      xv[i] = zero_pack8();
      if (key0 + key < Lk && e < D) {
        xk[i] = ld_global16(kp + (int64_t)key * a.k_row_stride + e);
        xv[i] = ld_global16(vp + (int64_t)key * a.v_row_stride + e);
      }
    }
  }

  // ---- this block's column list --------------------------------------------------------------
  // The rows of the first two rounds are asked for together with the probes of the search below, as if the walk
  // began at the head of the list (it does unless rows of the list lie before the block); otherwise they are
  // fetched again.
  int spec01[2] = {0, 0};
  if (tid < kBwdRoundRows && nnz > 0) {
#pragma unroll
    for (int sr = 0; sr < 2; ++sr) spec01[sr] = a.row_indices[lbase + min(sr * kBwdRoundRows + tid, nnz - 1)];
  }
  int start = 0;
  // rows r with r + off < key0 see no key of this block
  if (causal && nnz > 0) start = lower_bound_wave_i32(a.row_indices + lbase, nnz, key0 - off);
  const int32_t *list = a.row_indices + lbase + start;
  const int n = nnz - start;               // rows of the list that the block walks
  const int nround = (n + kBwdRoundRows - 1) / kBwdRoundRows;
  const int koff = key0 - c * Bn;  // offset of this 64-key block inside its column
  int rid01[2] = {-1, -1};         // threads 0..127: row ids of rounds 0 and 1
  if (tid < kBwdRoundRows && n > 0) {
#pragma unroll
    for (int sr = 0; sr < 2; ++sr) {
      const int j = sr * kBwdRoundRows + tid;
      const int r = start == 0 ? spec01[sr] : list[min(j, n - 1)];
      rid01[sr] = tile_row_code(r, j < n, Lq);
    }
  }

  {
    uint16_t *sK = reinterpret_cast<uint16_t *>(smem), *sV = sK + NKEY * LDQ;
#pragma unroll
    for (int i = 0; i < NKV; ++i) {
      const int v = tid + 256 * i;
      const int key = v / VPR, e = (v - key * VPR) * 8;
      *reinterpret_cast<Pack8 *>(sK + key * LDQ + e) = xk[i];
      *reinterpret_cast<Pack8 *>(sV + key * LDQ + e) = xv[i];
    }
  }
  __syncthreads();
  // B operands of S and dP: this lane's key, its half of the head dim; K^T of this wave's half of the features for
  // the dQ products.  They never change, so they stay in registers.
  u32x4_t kb[KS], vb[KS];  // (in accumulation registers)
  u32x4_t kt[NDH][4 * KB];  // (in accumulation registers)
  {
    const uint16_t *sK = reinterpret_cast<const uint16_t *>(smem), *sV = sK + NKEY * LDQ;
#pragma unroll
    for (int t = 0; t < KS; ++t) {
      kb[t] = pack8_vec(*reinterpret_cast<const Pack8 *>(sK + (kq * 32 + (lane & 31)) * LDQ + (hh * KS + t) * 8));
      vb[t] = pack8_vec(*reinterpret_cast<const Pack8 *>(sV + (kq * 32 + (lane & 31)) * LDQ + (hh * KS + t) * 8));
#if defined(__HIP_DEVICE_COMPILE__)
      asm volatile("" : "+a"(kb[t]), "+a"(vb[t]));
#endif
    }
    if constexpr (DQP) {
      lds_cu16 *trK = tr_lane_base(sK, LDQ, lane) + 8 * hh * LDQ;
#pragma unroll
      for (int s4 = 0; s4 < 4 * KB; ++s4)
#pragma unroll
        for (int d2 = 0; d2 < NDH; ++d2) {
          const int lo = 16 * s4 * LDQ + (kq * NDH + d2) * 32;
          kt[d2][s4] = pack8_vec(tr_frag8_at(trK, lo, lo + 4 * LDQ));
#if defined(__HIP_DEVICE_COMPILE__)
          asm volatile("" : "+a"(kt[d2][s4]));
#endif
        }
    }
  }

  const uint16_t *qg = reinterpret_cast<const uint16_t *>(a.q) + (int64_t)q0 * a.q_row_stride + (int64_t)h * a.q_head_stride;
  const uint16_t *dog = reinterpret_cast<const uint16_t *>(a.dout) + (int64_t)q0 * a.do_row_stride + (int64_t)h * a.do_head_stride;
  const float *lseg = a.softmax_lse + (int64_t)h * a.total_q + q0;
  const float *delg = a.softmax_d + (int64_t)h * ((int64_t)a.total_q + 128 * (int64_t)a.batch) + q0 + 128 * b;
  int32_t *cntg = ws.cnt + (int64_t)q0 * a.heads + h;  // counter of local row r: cntg[r * heads]
  float *red = reinterpret_cast<float *>(smem);  // [2][NKEY][LDR]: dV^T, dK^T on their way out

  f32x16 dv[NDT], dk[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      dv[dt][i] = 0.f;
      dk[dt][i] = 0.f;
    }

  if (nround > 0) {
    // ---- feeding the tiles --------------------------------------------------------------------------
    // Nothing passes through registers: every wave fetches one of the four tiles of the NEXT round with loads that
    // write straight to LDS, issued in the first half of a round and awaited at its end.  Threads 0..127 carry the
    // per-row scalars: the row id of round s+2 (it has to be in LDS one round before the tile loads that use it),
    // and LSE, delta and the dQ-partial slot of round s+1.
    const uint32_t ldsQ = (uint32_t)(uintptr_t)(smem + SM::oQ), ldsdO = (uint32_t)(uintptr_t)(smem + SM::odO);
    int n_rid = -1, v_rid = rid01[1], m_rid = -1, m_slot = 0;  // v_rid: the checked row id that was stored last = the one of the next round
    float m_lse = 0.f, m_del = 0.f;
    int ft = tid;  // thread index for the feeding code, re-made opaque in every round (see below)
    auto rid_issue = [&](int sr) {
      if (tid < kBwdRoundRows) {
        n_rid = list[min(sr * kBwdRoundRows + ft, n - 1)];  // used (and checked) only when it is stored: no wait for it here
      }
    };
    auto rid_store = [&](int sr) {
      if (tid < kBwdRoundRows) {
        const int j = sr * kBwdRoundRows + ft;
        v_rid = tile_row_code(n_rid, j < n, Lq);
        sRid[(sr & 1) * kBwdRoundRows + ft] = v_rid;
      }
    };
    auto meta_issue = [&](int rid) {  // rid: this thread's row of the round after the current one
      if (tid < kBwdRoundRows) {
        m_rid = rid;
        const int rc = max(m_rid, 0);
        m_lse = lseg[rc];
        m_del = delg[rc];
        // every visit of a (row, key block) pair takes one dQ-partial slot of the row
        if constexpr (DQP) {
          if (m_rid >= 0) m_slot = atomicAdd(cntg + (int64_t)m_rid * a.heads, 1);
        }
      }
    };
    const int64_t trash = (int64_t)a.total_q * a.heads * ws.cap;  // spare row: takes the writes of absent rows, no branch
    auto meta_store = [&](int sr) {
      if (tid < kBwdRoundRows) {
        const int i = (sr & 1) * kBwdRoundRows + ft;
        const bool ok = m_rid >= 0;
        sRow[i] = m_rid;
        // where the visit's dQ partial goes, as an index of partial rows (2^31 of them would be half a terabyte): the
        // row's slot, or the spare row for an absent row and for a visit beyond the caller's bound
        if constexpr (DQP) sSlot[i] = (ok && m_slot < ws.cap) ? (int)((((int64_t)(q0 + m_rid)) * a.heads + h) * ws.cap + m_slot) : (int)trash;
        sLse[i] = ok ? m_lse * kLog2e : INFINITY;  // absent rows: exp2(x - inf) = 0
        sDelta[i] = ok ? m_del : 0.f;
      }
    };
    auto tile_issue = [&](int sr) {  // tile `wave` of round sr
      constexpr int RPI = 64 / VPR, NI = 32 / RPI;  // tile rows per instruction, instructions per tile
      const int fl = ft & 63, rl = fl / VPR, p = fl - rl * VPR;
      const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane(((sr & 1) * 4 + wave) * (int)TB);
      const uint32_t qs = (uint32_t)a.q_row_stride, dos = (uint32_t)a.do_row_stride;  // (32 x 32 -> 64-bit products: one instruction each)
      // Absent rows and features past head_dim are fetched from a row and a piece that exist (tile_row_code): every
      // load is unconditional, and what such data meets is an exact zero (probabilities of absent rows, K / V features
      // past head_dim) or is never written out.
      int src[NI];
#pragma unroll
      for (int i = 0; i < NI; ++i) src[i] = sRid[(sr & 1) * kBwdRoundRows + wave * 32 + i * RPI + rl] & 0x7fffffff;
      if constexpr (NEAR) {
        // the sequence's rows lie within 4 GB of its first one: a 32-bit byte offset per lane from a wave-uniform base,
        // one full-rate multiply (the 64-bit products take four times as long, and an address takes two more additions)
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const uint32_t e2 = (uint32_t)min((p ^ tile_swz<HD>(i * RPI + rl)) * 8, D - 8) * 2u;
          global_to_lds16_sbase(mul24_u32((uint32_t)src[i], qs * 2u) + e2, qg, ldsQ + dst + (uint32_t)(i * RPI * RB));
          global_to_lds16_sbase(mul24_u32((uint32_t)src[i], dos * 2u) + e2, dog, ldsdO + dst + (uint32_t)(i * RPI * RB));
        }
      } else {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const uint32_t e = (uint32_t)min((p ^ tile_swz<HD>(i * RPI + rl)) * 8, D - 8);
          global_to_lds16(qg + ((uint64_t)(uint32_t)src[i] * qs + e), ldsQ + dst + (uint32_t)(i * RPI * RB));
          global_to_lds16(dog + ((uint64_t)(uint32_t)src[i] * dos + e), ldsdO + dst + (uint32_t)(i * RPI * RB));
        }
      }
    };

    // The same loads one at a time, for rows near the base.  A load instruction of a kilobyte holds the wave for about
    // 70 clocks while the unit's four waves issue theirs together (the unit's vector memory path takes 64 bytes per
    // clock: a round's 64 KB are a thousand clocks of it), and a wave that waits there issues no products either.  So
    // the Q loads go between the products of the round's first stage, one per two products, and the dO loads between
    // those of the second, instead of all at the start of the round; the offsets stay in registers until then.  (With
    // a test per load of whether the rows are near, that gain was lost: hence the NEAR instantiations.)
    constexpr bool kSpreadLoads = NEAR;
    constexpr int NTI = 32 / (64 / VPR);  // load instructions per tile and operand
    static_assert(NTI == KS, "one pair of tile loads per k-step of the first stage");
    uint32_t t_q[kSpreadLoads ? NTI : 1], t_do[kSpreadLoads ? NTI : 1], t_dst = 0;  // byte offsets of this lane's pieces
    auto tile_rows = [&](int sr) {
      constexpr int RPI = 64 / VPR;
      const int fl = ft & 63, rl = fl / VPR, p = fl - rl * VPR;
      t_dst = (uint32_t)__builtin_amdgcn_readfirstlane(((sr & 1) * 4 + wave) * (int)TB);
      const uint32_t qs = (uint32_t)a.q_row_stride, dos = (uint32_t)a.do_row_stride;
#pragma unroll
      for (int i = 0; i < (kSpreadLoads ? NTI : 0); ++i) {
        const uint32_t src = (uint32_t)(sRid[(sr & 1) * kBwdRoundRows + wave * 32 + i * RPI + rl] & 0x7fffffff);
        const uint32_t e2 = (uint32_t)min((p ^ tile_swz<HD>(i * RPI + rl)) * 8, D - 8) * 2u;
        t_q[i] = mul24_u32(src, qs * 2u) + e2;
        t_do[i] = mul24_u32(src, dos * 2u) + e2;
      }
    };
    auto tile_issue_q = [&](auto ic) {
      constexpr int I = decltype(ic)::value, RPI = 64 / VPR;
      if constexpr (kSpreadLoads) global_to_lds16_sbase(t_q[I], qg, ldsQ + t_dst + (uint32_t)(I * RPI * RB));
    };
    auto tile_issue_do = [&](auto ic) {
      constexpr int I = decltype(ic)::value, RPI = 64 / VPR;
      if constexpr (kSpreadLoads) global_to_lds16_sbase(t_do[I], dog, ldsdO + t_dst + (uint32_t)(I * RPI * RB));
    };

    if (tid < kBwdRoundRows) {
      sRid[tid] = rid01[0];
      sRid[kBwdRoundRows + tid] = rid01[1];
    }
    __syncthreads();  // K, V are in registers; the row ids of rounds 0 and 1 are in LDS
    meta_issue(rid01[0]);
    tile_issue(0);
    meta_store(0);
    wait_all_loads();
    __syncthreads();

    // ---- compute-wave stages ---------------------------------------------------------------------
    // A wave is alone on its SIMD, so the MFMA pipe only stays busy if the softmax arithmetic
    // of one tile runs between the products of the other tile of the round.  Every stage is cut into
    // four chunks (a quarter of the products + a quarter of the softmax rows); the operands of chunk
    // g+1 are read from LDS while chunk g computes, and the scheduler is fenced between chunks: left
    // alone, the compiler sinks every read next to the MFMA that uses it and waits for it there.
    typedef std::integral_constant<int, 0> C0;
    typedef std::integral_constant<int, 1> C1;
    constexpr int KC = KS / 4;       // k-steps of S / dP per chunk
    constexpr int BC = NDT / 2;      // (d-tile, row-half) operand pairs of dV / dK per chunk
    // byte addresses of this lane's pieces in tile 0 of the pair, buffer 0: row reads (row lane % 32, pieces
    // hh * KS ..) and transposing reads (row (lane % 16) / 4 + 4 hh, feature tile 0); every other operand is an
    // exclusive-or on the piece bits plus a constant
    const uint32_t pairQ = ldsQ + (uint32_t)(px * 2) * TB, pairdO = ldsdO + (uint32_t)(px * 2) * TB;
    const uint32_t rowoff = (uint32_t)((lane & 31) * RB + (((hh * KS) ^ tile_swz<HD>(lane & 31)) * 16));
    const int li = lane & 15, r0t = (li >> 2) + 4 * hh;
    const uint32_t troff = (uint32_t)(r0t * RB + ((((((lane >> 4) & 1) * 2 + ((li & 3) >> 1))) ^ tile_swz<HD>(r0t)) * 16) + (li & 1) * 8);
    // The operand addresses derived from them (an exclusive-or per piece) are formed once and stay in registers: the
    // products leave room for them since their sums live in the accumulation registers.  (Made opaque, or the
    // compiler forms them again at every read.)
    // (The form with dQ partials has no registers to spare: there the bases are re-made opaque wherever they are used,
    // so that nothing derived from them is kept from one use to the next.)
    constexpr bool kKeepAddresses = !DQP;
    uint32_t aQ = pairQ + rowoff, adO = pairdO + rowoff, tQ = pairQ + troff, tdO = pairdO + troff;
    uint32_t aQk[KS], adOk[KS];                              // row reads: piece hh * KS + k of this lane's row
    uint32_t tQlo[NDT], tQhi[NDT], tdOlo[NDT], tdOhi[NDT];  // transposing reads: feature tile dt, rows (0..3) + 4 hh and the same + 8
#pragma unroll
    for (int k = 0; k < (kKeepAddresses ? KS : 0); ++k) {
      aQk[k] = aQ ^ (uint32_t)(k * 16);
      adOk[k] = adO ^ (uint32_t)(k * 16);
#if defined(__HIP_DEVICE_COMPILE__)
      asm volatile("" : "+v"(aQk[k]), "+v"(adOk[k]));
#endif
    }
#pragma unroll
    for (int dt = 0; dt < (kKeepAddresses ? NDT : 0); ++dt) {
      const uint32_t xlo = (uint32_t)(dt * 4 * 16), xhi = (uint32_t)(((dt * 4) ^ TileSwz<HD>::kRow8) * 16);
      tQlo[dt] = tQ ^ xlo;
      tQhi[dt] = tQ ^ xhi;
      tdOlo[dt] = tdO ^ xlo;
      tdOhi[dt] = tdO ^ xhi;
#if defined(__HIP_DEVICE_COMPILE__)
      asm volatile("" : "+v"(tQlo[dt]), "+v"(tQhi[dt]), "+v"(tdOlo[dt]), "+v"(tdOhi[dt]));
#endif
    }
    auto opaque = [](uint32_t &x, uint32_t &y) {
#if defined(__HIP_DEVICE_COMPILE__)
      asm volatile("" : "+v"(x), "+v"(y));
#else
      (void)x, (void)y;
#endif
    };
    auto opaque1 = [](uint32_t &x) {
#if defined(__HIP_DEVICE_COMPILE__)
      asm volatile("" : "+v"(x));
#else
      (void)x;
#endif
    };
    uint16_t *sdS = reinterpret_cast<uint16_t *>(smem + SM::odS) + (DQP ? (size_t)px * 2 * 64 * LDS_ : (size_t)wave * 32 * LDS_);  // (px = 0 with 128 keys)
    lds_cu16 *trdS = tr_lane_base(sdS, LDS_, lane) + 8 * hh * LDS_;  // dS^T tile: 8 consecutive keys per read
    // the dQ part rows of a tile leave through the first tile of the pair, which nobody reads after the barrier in
    // the middle of the round: Q's for even waves, dO's for odd ones, one half of it each with four key quarters
    uint16_t *sdQ0 = reinterpret_cast<uint16_t *>(smem + ((kq & 1) ? SM::odO : SM::oQ) + (size_t)(px * 2) * TB + (size_t)(kq >> 1) * (TB / 2));
    const int *pRow = sRow + px * 64;
    uint32_t smx0 = (uint32_t)(uintptr_t)(smem + SM::oRow) + (uint32_t)(px * 64 * 4 + hh * 16);  // softmax inputs of this lane's rows
    Pack8 qa[2][KC], doa[2][KC];     // A operands of S and dP (this lane's row, its half of the head dim), double-buffered by chunk
    Pack8 dot[2][BC], qt[2][BC];     // dO^T / Q^T operands of the dV / dK products, double-buffered by chunk
    f32x4 lse4[2], del4[2];          // softmax inputs of a chunk's four rows
    Pack8 pf[2][2], dsf[2][2];       // P and dS of both tiles of the round as MFMA operands
    Pack8 dsx[4 * KB];               // dS^T of all keys of the block as the B operand of the dQ products
    f32x16 dqa[NDH];
    f32x16 s[2], dp[2];
    auto fence = [&]() { __builtin_amdgcn_sched_barrier(0); };
    // pc: buffer of the round; pp: tile pair (always 0 with KB = 1, where the pair is part of the addresses); tsc: tile of the pair
    auto ld_a = [&](auto pc, auto pp, auto tsc, auto gc) {
      constexpr uint32_t TO = (uint32_t)(decltype(pc)::value * 4 + decltype(pp)::value * 2 + decltype(tsc)::value) * TB;
      constexpr int G = decltype(gc)::value;
      if constexpr (!kKeepAddresses) opaque(aQ, adO);
#pragma unroll
      for (int t = 0; t < KC; ++t) {
        if constexpr (kKeepAddresses) {
          qa[G & 1][t] = lds_read16(aQk[G * KC + t] + TO);
          doa[G & 1][t] = lds_read16(adOk[G * KC + t] + TO);
        } else {
          qa[G & 1][t] = lds_read16((aQ ^ (uint32_t)((G * KC + t) * 16)) + TO);
          doa[G & 1][t] = lds_read16((adO ^ (uint32_t)((G * KC + t) * 16)) + TO);
        }
      }
    };
    // this lane's key; key j is visible to row r iff r >= row_thr (rows that do not exist are stored as -1)
    const int j = key0 + kq * 32 + (lane & 31);
    const int row_thr = j >= Lk ? 0x7fffffff : (causal ? max(0, j - off) : 0);
    // rows from this one on see every key of the block (no row does if the block reaches past the sequence)
    const int all_visible_from = key0 + NKEY > Lk ? 0x7fffffff : (causal ? max(0, key0 + NKEY - 1 - off) : 0);
    // The causal rule and the end of the sequence enter S as its starting value: 0 where row and key see each other,
    // -inf elsewhere (the products then leave -inf there and the exponential gives 0), and only in rounds that have
    // such pairs at all (`masked`, the same for the whole wave): the rows of a list come in ascending order, so
    // from the first row that sees every key of the block on, S starts from nothing and no comparison is made.
    auto mm_a = [&](auto pc, auto pp, auto tsc, auto gc, bool masked, auto &&after_step) {
      constexpr int TS = decltype(tsc)::value, G = decltype(gc)::value;
      static_for<KC>([&](auto tc) {
        constexpr int t = decltype(tc)::value;
        if (G == 0 && t == 0) {
          if (masked) {
            constexpr int TSG = decltype(pc)::value * 4 + decltype(pp)::value * 2 + TS;
            opaque1(smx0);
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
              const int4 r4 = lds_read_vec<int4>(smx0 + (uint32_t)(TSG * 32 + 8 * g4) * 4);
              s[TS][4 * g4] = r4.x >= row_thr ? 0.f : -INFINITY;
              s[TS][4 * g4 + 1] = r4.y >= row_thr ? 0.f : -INFINITY;
              s[TS][4 * g4 + 2] = r4.z >= row_thr ? 0.f : -INFINITY;
              s[TS][4 * g4 + 3] = r4.w >= row_thr ? 0.f : -INFINITY;
            }
            mfma32_b_acc<T, false>(s[TS], qa[G & 1][t], kb[G * KC + t]);
          } else {
            mfma32_b_acc<T, true>(s[TS], qa[G & 1][t], kb[G * KC + t]);
          }
          mfma32_b_acc<T, true>(dp[TS], doa[G & 1][t], vb[G * KC + t]);
        } else {
          mfma32_b_acc<T, false>(s[TS], qa[G & 1][t], kb[G * KC + t]);
          mfma32_b_acc<T, false>(dp[TS], doa[G & 1][t], vb[G * KC + t]);
        }
        after_step(std::integral_constant<int, G * KC + t>{});
      });
      if constexpr (G == 3) mfma_results_ready(s[TS], dp[TS]);
    };
    auto ld_b = [&](auto pc, auto pp, auto tsc, auto gc) {
      constexpr uint32_t TO = (uint32_t)(decltype(pc)::value * 4 + decltype(pp)::value * 2 + decltype(tsc)::value) * TB;
      constexpr int G = decltype(gc)::value;
      if constexpr (!kKeepAddresses) opaque(tQ, tdO);
#pragma unroll
      for (int t = 0; t < BC; ++t) {
        const int pi = G * BC + t, dt = pi >> 1, s2 = pi & 1;
        // rows 16 s2 + (0..3) + 4 hh and the same + 8, features dt * 32 ..
        const uint32_t olo = TO + (uint32_t)(16 * s2 * RB), ohi = olo + (uint32_t)(8 * RB);
        if constexpr (kKeepAddresses) {
          dot[G & 1][t] = lds_tr8(tdOlo[dt] + olo, tdOhi[dt] + ohi);
          qt[G & 1][t] = lds_tr8(tQlo[dt] + olo, tQhi[dt] + ohi);
        } else {
          const uint32_t xlo = (uint32_t)(dt * 4 * 16), xhi = (uint32_t)(((dt * 4) ^ TileSwz<HD>::kRow8) * 16);
          dot[G & 1][t] = lds_tr8((tdO ^ xlo) + olo, (tdO ^ xhi) + ohi);
          qt[G & 1][t] = lds_tr8((tQ ^ xlo) + olo, (tQ ^ xhi) + ohi);
        }
      }
    };
    auto mm_b = [&](auto tsc, auto gc) {
      constexpr int TS = decltype(tsc)::value, G = decltype(gc)::value;
      // dV^T[d][key] += dO^T[d][row] P[row][key];  dK^T[d][key] += Q^T[d][row] dS[row][key]
#pragma unroll
      for (int t = 0; t < BC; ++t) {
        const int pi = G * BC + t, dt = pi >> 1, s2 = pi & 1;
        static_for<NDT>([&](auto dc) {
          constexpr int DT = decltype(dc)::value;
          if (DT == dt) {
            mfma32_c_acc<T, 2 * DT>(dv[DT], dot[G & 1][t], pf[TS][s2]);
            mfma32_c_acc<T, 2 * DT + 1>(dk[DT], qt[G & 1][t], dsf[TS][s2]);
          }
        });
      }
    };
    auto ld_s = [&](auto pc, auto pp, auto tsc, auto gc) {
      constexpr int TS = decltype(pc)::value * 4 + decltype(pp)::value * 2 + decltype(tsc)::value, G = decltype(gc)::value;
      // accumulator registers 4G..4G+3 hold rows TS * 32 + 8 G + 4 hh + (0..3); one address register, the rest
      // are offsets in the instructions
      constexpr uint32_t O = (uint32_t)(TS * 32 + 8 * G) * 4;
      opaque1(smx0);
      lse4[G & 1] = lds_read_vec<f32x4>(smx0 + O + (uint32_t)(SM::oLse - SM::oRow));
      del4[G & 1] = lds_read_vec<f32x4>(smx0 + O + (uint32_t)(SM::oDelta - SM::oRow));
    };
    auto smx = [&](auto tsc, auto gc) {
      constexpr int TS = decltype(tsc)::value, G = decltype(gc)::value;
      float pr[4], ds[4];
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int i = 4 * G + jj;
        const float x = fmaf(s[TS][i], scale_log2, -lse4[G & 1][jj]);  // (-inf for a masked pair, see mm_a)
        pr[jj] = __builtin_amdgcn_exp2f(x);
        ds[jj] = pr[jj] * (dp[TS][i] - del4[G & 1][jj]);
      }
      // operand register s2 = G/2 holds rows 16*s2 + 8*(w/2) + 4*hh + ..: words 2*(G%2), 2*(G%2)+1
      pf[TS][G >> 1].w[2 * (G & 1)] = pack2<T>(pr[0], pr[1]);
      pf[TS][G >> 1].w[2 * (G & 1) + 1] = pack2<T>(pr[2], pr[3]);
      dsf[TS][G >> 1].w[2 * (G & 1)] = pack2<T>(ds[0], ds[1]);
      dsf[TS][G >> 1].w[2 * (G & 1) + 1] = pack2<T>(ds[2], ds[3]);
    };
    // dQ of the tile: both waves of a pair put dS^T of their 32 keys into one LDS tile [64 keys][32 rows]; after a
    // barrier each wave computes dQ^T = K^T dS^T over all 64 keys for ITS half of the features.  The
    // half rows (16-bit, unscaled) go to the partial slot that the row handed out for this visit.
    auto ds_write = [&](auto tsc) {
      constexpr int TS = decltype(tsc)::value;
      // partials form: tile slot TS of the pair, rows of all keys of the block; else: this wave's private tile
      uint16_t *t = sdS + (size_t)((DQP ? TS * NKEY + kq * 32 : 0) + (lane & 31)) * LDS_;
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        *reinterpret_cast<uint2 *>(t + 16 * s2 + 4 * hh) = make_uint2(dsf[TS][s2].w[0], dsf[TS][s2].w[1]);
        *reinterpret_cast<uint2 *>(t + 16 * s2 + 8 + 4 * hh) = make_uint2(dsf[TS][s2].w[2], dsf[TS][s2].w[3]);
      }
      if constexpr (!DQP) wave_lds_order();  // (the partials form waits for both key halves at a workgroup barrier later)
    };
    // dS form: the wave's 32 keys of every row go to the dS tile of the row's list entry
    int dsrow = -1;
    auto ds_read = [&](auto pc, auto pp, auto tsc) {
      constexpr int TS = decltype(pc)::value * 4 + decltype(pp)::value * 2 + decltype(tsc)::value;
      dsrow = pRow[TS * 32 + (lane & 31)];
#pragma unroll
      for (int s4 = 0; s4 < 2; ++s4) dsx[s4] = tr_frag8_at(trdS, 16 * s4 * LDS_, (16 * s4 + 4) * LDS_);
      wave_lds_order();
    };
    auto ds_store = [&](int tile) {
      if (dsrow >= 0) {
        // key groups koff / 8 + 4 kq + 2 s4 + hh of list position p: consecutive lanes write consecutive 16-byte pieces
        const int64_t p = lbase + start + tile * 32 + (lane & 31);
        uint16_t *wp = ws.ds + ds_piece_offset(p, (koff >> 3) + 4 * kq + hh, Bn >> 3);
#pragma unroll
        for (int s4 = 0; s4 < 2; ++s4) *reinterpret_cast<Pack8 *>(wp + s4 * 512) = dsx[s4];
      }
    };
    auto dq_load = [&](auto tsc) {
      constexpr int TS = decltype(tsc)::value;
#pragma unroll
      for (int s4 = 0; s4 < 4 * KB; ++s4) dsx[s4] = tr_frag8_at(trdS, (TS * NKEY + 16 * s4) * LDS_, (TS * NKEY + 16 * s4 + 4) * LDS_);
    };
    auto dq_mma = [&](auto gc) {  // a quarter of the products per chunk
      constexpr int G = decltype(gc)::value;
#pragma unroll
      for (int d2 = 0; d2 < NDH; ++d2) {
#pragma unroll
        for (int t = 0; t < KB; ++t) {
          if (G == 0 && t == 0)
            mfma32_a_acc<T, true>(dqa[d2], kt[d2][G * KB + t], dsx[G * KB + t]);
          else
            mfma32_a_acc<T, false>(dqa[d2], kt[d2][G * KB + t], dsx[G * KB + t]);
        }
      }
      if constexpr (G == 3) {
        static_assert(NDH <= 2, "one or two feature tiles of dQ per wave");
        if constexpr (NDH == 1)
          mfma_results_ready(dqa[0]);
        else
          mfma_results_ready(dqa[0], dqa[1]);
      }
    };
    auto dq_store = [&](auto pc, auto pp, auto tsc) {
      constexpr int TS = decltype(pc)::value * 4 + decltype(pp)::value * 2 + decltype(tsc)::value;
      constexpr uint32_t SO = (uint32_t)(decltype(pc)::value * 4 + decltype(pp)::value * 2) * TB;  // the tile that serves as staging
      // register i of feature tile d2 <-> feature d2*32 + acc_row(i, hh) of this wave's half, this lane's row
      uint32_t bw = (uint32_t)(uintptr_t)sdQ0 + (uint32_t)(((lane & 31) * LDH + 4 * hh) * 2), unused_w = 0;
      opaque(bw, unused_w);
#pragma unroll
      for (int d2 = 0; d2 < NDH; ++d2)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          lds_write_vec<uint2>(bw + SO + (uint32_t)((d2 * 32 + 8 * g) * 2),
                               make_uint2(pack2<T>(dqa[d2][4 * g], dqa[d2][4 * g + 1]), pack2<T>(dqa[d2][4 * g + 2], dqa[d2][4 * g + 3])));
      wave_lds_fence();
      constexpr int LPR = NDH * 4;        // lanes per part row (16 bytes each)
      constexpr int RPP = 64 / LPR;       // rows per pass
      const int col = (lane % LPR) * 8;
      uint32_t bs = (uint32_t)(uintptr_t)(smem + SM::oRow) + (uint32_t)((px * 64 + lane / LPR) * 4);
      uint32_t bx = (uint32_t)(uintptr_t)sdQ0 + (uint32_t)(((lane / LPR) * LDH + col) * 2);
      opaque(bs, bx);
      // (one test around all rows of the tile rather than one per store: a lane either has features of the head
      // dimension in its piece or it has not)
      uint32_t pidx[32 / RPP];
#pragma unroll
      for (int k = 0; k < 32 / RPP; ++k) pidx[k] = (uint32_t)lds_read_vec<int>(bs + (uint32_t)(TS * 32 + k * RPP) * 4 + (uint32_t)(SM::oSlot - SM::oRow));
      if (kq * (NDH * 32) + col < D) {
#pragma unroll
        for (int k = 0; k < 32 / RPP; ++k) {
          const Pack8 x = lds_read16(bx + SO + (uint32_t)(k * RPP * LDH * 2));
          st_stream16(ws.part + ((uint64_t)pidx[k] * (uint32_t)D + (uint32_t)(kq * (NDH * 32) + col)), x);
        }
      }
      if (kq == 0 && col == 0) {
#pragma unroll
        for (int k = 0; k < 32 / RPP; ++k) ws.pid[pidx[k]] = nb;
      }
      wave_lds_fence();
    };
    // One round of a pair = its tiles 2 px and 2 px + 1, both already in LDS.  Tiles past the end of the list hold
    // absent rows (row id -1, zero data): they run through the same code and add nothing.
    auto process_round = [&](auto pc, auto pp, int r) {  // pc: parity of r = the LDS buffer that holds the round
      const int tile0 = 4 * r + 2 * (KB == 1 ? px : decltype(pp)::value);  // position of the pair's first tile in the list
      // (the first row of the pair's first tile is its earliest; -1 if the pair has no row)
      const bool masked = __builtin_amdgcn_readfirstlane(pRow[(decltype(pc)::value * 4 + decltype(pp)::value * 2) * 32]) < all_visible_from;
      // S, dP of the first tile
      ld_a(pc, pp, C0{}, C0{});
      fence();
      static_for<4>([&](auto gc) {
        constexpr int G = decltype(gc)::value;
        if constexpr (G < 3) {
          ld_a(pc, pp, C0{}, std::integral_constant<int, G + 1>{});
        } else {  // the first operands of the next stage: a stage that began with its own reads began with their latency
          ld_a(pc, pp, C1{}, C0{});
          ld_s(pc, pp, C0{}, C0{});
        }
        mm_a(pc, pp, C0{}, gc, masked, [&](auto ic) {
          if constexpr (kSpreadLoads && decltype(pp)::value == 0) tile_issue_q(ic);
        });
        fence();
      });
      // S, dP of the second tile between the softmax rows of the first
      static_for<4>([&](auto gc) {
        constexpr int G = decltype(gc)::value;
        if constexpr (G < 3) {
          ld_a(pc, pp, C1{}, std::integral_constant<int, G + 1>{});
          ld_s(pc, pp, C0{}, std::integral_constant<int, G + 1>{});
        } else {
          ld_b(pc, pp, C0{}, C0{});
          ld_s(pc, pp, C1{}, C0{});
        }
        mm_a(pc, pp, C1{}, gc, masked, [&](auto ic) {
          if constexpr (kSpreadLoads && decltype(pp)::value == 0) tile_issue_do(ic);
        });
        smx(C0{}, gc);
        fence();
      });
      // dV, dK of the first tile between the softmax rows of the second
      // (a second pair of the same waves reuses the dS^T tiles of the first: its readers have to be done)
      if constexpr (DQP && decltype(pp)::value == 1) __syncthreads();
      ds_write(C0{});
      if constexpr (!DQP) ds_read(pc, pp, C0{});
      fence();
      static_for<4>([&](auto gc) {
        constexpr int G = decltype(gc)::value;
        if constexpr (G < 3) {
          ld_b(pc, pp, C0{}, std::integral_constant<int, G + 1>{});
          ld_s(pc, pp, C1{}, std::integral_constant<int, G + 1>{});
        } else {
          ld_b(pc, pp, C1{}, C0{});
        }
        mm_b(C0{}, gc);
        smx(C1{}, gc);
        if constexpr (!DQP && G == 0) ds_store(tile0);
        fence();
      });
      // dV, dK of the second tile; in the partials form dQ of the first one runs between them: by now all key
      // groups have put dS^T of both tiles into LDS, so the one barrier the exchange needs hardly ever waits
      ds_write(C1{});
      if constexpr (DQP) __syncthreads();
      if constexpr (DQP)
        dq_load(C0{});
      else
        ds_read(pc, pp, C1{});
      fence();
      static_for<4>([&](auto gc) {
        constexpr int G = decltype(gc)::value;
        if constexpr (G < 3) ld_b(pc, pp, C1{}, std::integral_constant<int, G + 1>{});
        mm_b(C1{}, gc);
        if constexpr (DQP) dq_mma(gc);
        if constexpr (!DQP && G == 0) ds_store(tile0 + 1);
        fence();
      });
      if constexpr (DQP) {
        dq_store(pc, pp, C0{});
        // dQ of the second tile
        dq_load(C1{});
        fence();
        static_for<4>([&](auto gc) {
          dq_mma(gc);
          fence();
        });
        // The tiles of the next round must be in LDS before the barrier that ends this one, and one counter covers
        // loads and stores alike: the round's last partial rows are issued after that wait, so that they complete
        // under the next round instead of being waited for.
        if constexpr (KB == 1 || decltype(pp)::value == 1) {
          wait_all_loads();
          meta_store(r + 1);
          rid_store(r + 2);
        }
        dq_store(pc, pp, C1{});
      }
    };
    auto round = [&](auto pc, int r) {
#if defined(__HIP_DEVICE_COMPILE__)
      asm volatile("" : "+v"(ft));
#endif
      rid_issue(r + 2);
      meta_issue(v_rid);
      if constexpr (kSpreadLoads)
        tile_rows(r + 1);
      else
        tile_issue(r + 1);
      process_round(pc, C0{}, r);
      if constexpr (KB == 2) process_round(pc, C1{}, r);
      if constexpr (!DQP) {
        meta_store(r + 1);
        rid_store(r + 2);
        wait_all_loads();
      }
      __syncthreads();  // round r + 1 is in LDS; everyone is done with round r
    };
    for (int r = 0; r < nround; r += 2) {
      round(C0{}, r);
      if (r + 1 < nround) round(C1{}, r + 1);
    }
  }

  // ---- dK^T / dV^T: every wave puts its sums into LDS (one copy per pair); with two pairs the rows add them on their way out
  __syncthreads();  // K and V have left LDS (lists without rows come here directly)
  constexpr int NCOPY = KB == 1 ? 2 : 1;
  constexpr size_t kCopy = (size_t)2 * NKEY * LDR;  // floats of one copy: dV^T then dK^T
  static_assert(NCOPY * kCopy * 4 <= SM::bytes, "the output buffers reuse the tiles");
  {
    float *mine = red + (size_t)px * kCopy;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float *rp = mine + (size_t)(kq * 32 + (lane & 31)) * LDR + dt * 32 + 8 * g + 4 * hh;
        f32x4 v4, k4;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          v4[jj] = dv[dt][4 * g + jj];
          k4[jj] = dk[dt][4 * g + jj];
        }
        *reinterpret_cast<f32x4 *>(rp) = v4;
        *reinterpret_cast<f32x4 *>(rp + NKEY * LDR) = k4;
      }
  }
  __syncthreads();

  // ---- dK^T / dV^T leave as rows, once ----------------------------------------------------------------
  uint16_t *dkg = reinterpret_cast<uint16_t *>(a.dk) + (int64_t)(k0 + key0) * a.dk_row_stride + (int64_t)h * a.dk_head_stride;
  uint16_t *dvg = reinterpret_cast<uint16_t *>(a.dv) + (int64_t)(k0 + key0) * a.dv_row_stride + (int64_t)h * a.dv_head_stride;
  for (int v = tid; v < NKEY * VPR; v += 256) {
    const int key = v / VPR, e = (v - key * VPR) * 8;
    if (key0 + key >= Lk || e >= D) continue;
    const float *s0 = red + (size_t)key * LDR + e, *s1 = s0 + NKEY * LDR;
    float fv[8], fk[8];
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      fv[w] = s0[w];
      fk[w] = s1[w];
      if constexpr (NCOPY == 2) {
        fv[w] += s0[kCopy + w];
        fk[w] += s1[kCopy + w];
      }
    }
    Pack8 ov, ok;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      ov.w[w] = pack2<T>(fv[2 * w], fv[2 * w + 1]);
      ok.w[w] = pack2<T>(fk[2 * w] * a.softmax_scale, fk[2 * w + 1] * a.softmax_scale);
    }
    *reinterpret_cast<Pack8 *>(dvg + (int64_t)key * a.dv_row_stride + e) = ov;
    *reinterpret_cast<Pack8 *>(dkg + (int64_t)key * a.dk_row_stride + e) = ok;
  }
}

// ------------------------------------------------------------------------------------
// dQ, first form: row blocks.  One workgroup owns 256 or 512 consecutive query rows of one (sequence, head) and
// walks the 64-key blocks of every column in which one of its rows appears.  The dS rows of a step (written by the
// dK/dV pass in list order) go from global memory straight into the registers of the lane that owns the query row;
// rows that are absent contribute zeros, so every wave multiplies its own 32-row tiles and keeps dQ in registers
// for the whole walk.  All eight waves compute, two per SIMD, and nothing in the workgroup only moves data.  What a
// step needs from other threads -- its K tile (global memory straight into LDS, global_load_lds, every wave a share
// of the tile, swizzled rows of exactly head_dim elements) and the list positions of its rows (scattered into LDS by
// the thread whose index is the row's place in the step's run) -- is prepared for a whole group of G steps at once,
// one group ahead, so the workgroup meets at a barrier once per group: inside a group every wave runs at its own
// pace, and a wave's chain of dependent steps (where are my rows in this column's list -> fetch them -> multiply)
// is covered by the products of the other wave of its SIMD.
// ------------------------------------------------------------------------------------
constexpr int kDqWaves = 8;
constexpr int kDqColBatch = 256;
constexpr int kDqMaxSteps = 512;

template <int HD, int RT>
struct DqSmem {
  static constexpr int ROWS = kDqWaves * 32 * RT;
  static constexpr int G = HD == 128 ? 4 : 2;  // steps per group (one workgroup barrier per group)
  static constexpr int NS = 2 * G;              // K tiles / position slots in LDS: the group in use and the next one
  static constexpr int LDO = HD + 8;   // elements, per-wave output tile [32 rows][LDO] (reuses the K tiles at the end)
  static constexpr size_t tileBytes = (size_t)64 * HD * 2;
  static constexpr size_t outBytes = (size_t)kDqWaves * 32 * LDO * 2;
  static constexpr size_t prepBytes = (size_t)kDqColBatch * 16 + (size_t)kDqMaxSteps * 4;
  static constexpr size_t oK = 0;                                   // [NS][64 keys][HD], swizzled; later the output tiles
  static constexpr size_t ringBytes = NS * tileBytes > outBytes ? NS * tileBytes : outBytes;
  static_assert(prepBytes <= ringBytes, "the preparation arrays lie over the K tiles");
  static constexpr size_t oTag = oK + ringBytes;                   // int[NS][ROWS]: (step tag << 10) | list position of the row in that step
  static constexpr size_t oInfo = oTag + (size_t)NS * ROWS * 4;    // int4[kDqMaxSteps]: key0, rows, list position (lo, hi)
  static constexpr size_t oMisc = oInfo + (size_t)kDqMaxSteps * 16;
  static constexpr size_t bytes = oMisc + 64;
  // what only the preparation of a batch of columns uses (no tile is in use or on its way then)
  static constexpr size_t oOff = oK;                                // int64[kDqColBatch]
  static constexpr size_t oLo = oOff + kDqColBatch * 8;
  static constexpr size_t oCnt = oLo + kDqColBatch * 4;
  static constexpr size_t oStep = oCnt + kDqColBatch * 4;
  static_assert(bytes <= 160 * 1024, "LDS of one compute unit");
};

struct DqItem {
  int pair, sb;
};
__device__ __forceinline__ DqItem dq_decode_item(int id, int npairs, int nsb_max) {
  // late row blocks (the longest walks) first
  const PairItem item = xcd_pair_item(id, npairs, nsb_max);
  DqItem w;
  w.pair = item.pair < npairs ? item.pair : -1;
  w.sb = nsb_max - 1 - item.idx;
  return w;
}

template <int N>
__device__ __forceinline__ void wait_loads_but() {  // until at most N of the wave's vector memory loads are outstanding
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
#endif
}

// RT: 32-row tiles per wave.  With two, a workgroup owns 512 rows and every K^T operand read from LDS feeds two MFMAs.
template <typename T, int HD, int RT>
__global__ __launch_bounds__(512, (HD > 128 || RT > 1) ? 2 : 4) void attn_bwd_dq_kernel(fmoba_attn_bwd_args a, const uint16_t *ds_ws, int nsb_max) {
  typedef DqSmem<HD, RT> SM;
  constexpr int ROWS = SM::ROWS;  // query rows of the workgroup
  constexpr int LDO = SM::LDO, NDT = HD / 32, VPR = HD / 8;
  constexpr int RB = HD * 2;                       // bytes of a K tile row
  constexpr uint32_t TB = (uint32_t)SM::tileBytes;
  constexpr int RPI = 64 / VPR;                    // K rows per load instruction
  constexpr int NKI = 64 / RPI / kDqWaves;         // K load instructions per wave and tile
  static_assert(NKI >= 1 && NKI * RPI * kDqWaves == 64, "the waves share a K tile evenly");
  constexpr int NS = SM::NS, G = SM::G;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  int *sPos = reinterpret_cast<int *>(smem + SM::oTag);
  int *sLo = reinterpret_cast<int *>(smem + SM::oLo);
  int *sCnt = reinterpret_cast<int *>(smem + SM::oCnt);
  int *sStep = reinterpret_cast<int *>(smem + SM::oStep);
  int64_t *sOff = reinterpret_cast<int64_t *>(smem + SM::oOff);
  int4 *sInfo = reinterpret_cast<int4 *>(smem + SM::oInfo);
  int *sMisc = reinterpret_cast<int *>(smem + SM::oMisc);
  const uint32_t ldsK = (uint32_t)(uintptr_t)(smem + SM::oK);

  const DqItem wi = dq_decode_item(blockIdx.x, a.heads * a.batch, nsb_max);
  if (wi.pair < 0) return;
  const int b = wi.pair / a.heads, h = wi.pair - b * a.heads, sb = wi.sb;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int m0 = sb * ROWS;
  if (m0 >= Lq) return;
  const int k0 = a.cu_seqlens_k[b], Lk = a.cu_seqlens_k[b + 1] - k0;
  const int rows_sb = min(ROWS, Lq - m0);
  const int off = Lk - Lq;
  const int D = a.head_dim;
  const int hk = h / (a.heads / a.heads_k);
  const int Bn = a.lg_block_n, nsub = Bn / 64;
  const int tid = threadIdx.x, lane = tid & 63, hh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool causal = a.is_causal != 0;

  for (int v = tid; v < NS * ROWS; v += 512) sPos[v] = 0;  // step tags start at 1

  int ncols = min((Lk + Bn - 1) / Bn, a.max_cols);
  const int last_rowpos = m0 + rows_sb - 1 + off;
  if (causal) ncols = last_rowpos < 0 ? 0 : min(ncols, last_rowpos / Bn + 1);
  const int64_t bh = (int64_t)b * a.heads + h;
  const int64_t *coff = a.col_offsets + bh * a.max_cols;
  const uint16_t *kp = reinterpret_cast<const uint16_t *>(a.k) + (int64_t)k0 * a.k_row_stride + (int64_t)hk * a.k_head_stride;
  const int cols_per_batch = min(kDqColBatch, kDqMaxSteps / nsub);

  // The steps of one batch of columns: for every column the part of its list that falls into this row block, then
  // one record per (column, 64-key block) that has rows and visible keys.  Its scratch arrays lie over the K tiles:
  // no tile is in use or on its way when the workgroup comes here.
  auto prepare_batch = [&](int cb, int cend) {
    __syncthreads();
    for (int c = cb + tid; c < cend; c += 512) {
      const int nnz = a.col_nnz[bh * a.max_cols + c];
      int lo = 0, cnt = 0;
      int64_t base = 0;
      if (nnz > 0) {
        base = coff[c];
        const int32_t *list = a.row_indices + base;
        lo = lower_bound_i32(list, nnz, m0);
        const int hi = lo + lower_bound_i32(list + lo, nnz - lo, m0 + ROWS);
        cnt = min(hi - lo, ROWS);
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
    const int nsteps = __builtin_amdgcn_readfirstlane(sMisc[0]);
    // one record per step
    for (int st = tid; st < nsteps; st += 512) {
      const int code = sStep[st];
      const int cl = code >> 8, kb = code & 255;
      const int64_t pos0 = sOff[cl];
      // (y: rows of the run, at most 512, and above them the 64-key block's number inside its column)
      sInfo[st] = make_int4((cb + cl) * Bn + kb * 64, sCnt[cl] | (kb << 16), (int)(uint32_t)(pos0 & 0xffffffffll), (int)(pos0 >> 32));
    }
    __syncthreads();  // (also: everyone has read the scratch arrays before the first tile loads overwrite them)
    return nsteps;
  };

  f32x16 acc[RT][NDT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[rt][dt][i] = 0.f;
  // Which rows a wave owns: the waves w and w + 4 share a SIMD, and under the causal rule the later rows of the block
  // take part in more steps (the first wave's rows sit out the block's last seven key blocks, the last wave's none), so
  // a SIMD gets the rows w and 7 - w: the four SIMDs then have the same number of products to do.
  const int wtile = wave < 4 ? wave : 11 - wave;
  int myrow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) myrow[rt] = (wtile * RT + rt) * 32 + (lane & 31);

  // K tile loads of this wave: instruction i brings tile rows (wave * NKI + i) * RPI .. + RPI - 1, lane -> row rl, piece p;
  // piece c of tile row r is stored at piece c ^ tile_swz<HD>(r)
  const int krl = lane / VPR, kpp = lane - krl * VPR;
  uint32_t ksrc[NKI];  // element offset of this lane's piece inside a tile that exists completely
#pragma unroll
  for (int i = 0; i < NKI; ++i) {
    const int r = (wave * NKI + i) * RPI + krl;
    ksrc[i] = (uint32_t)(r * (int)a.k_row_stride + min((kpp ^ tile_swz<HD>(r)) * 8, D - 8));
  }
  // K^T operands (transposing reads): lane l (i = l % 16) supplies the address of key 8 hh + i / 4 (+ 4 for the
  // second read) of a 16-key group, features 16 ((l / 16) % 2) + 4 (i % 4) .. of a 32-feature tile
  const int li = lane & 15;
  const int kk0 = 8 * hh + (li >> 2);
  const int low2 = ((lane >> 4) & 1) * 2 + ((li & 3) >> 1);
  const uint32_t tlo = (uint32_t)(kk0 * RB + ((low2 ^ tile_swz<HD>(kk0)) * 16) + (li & 1) * 8);
  const uint32_t thi = (uint32_t)((kk0 + 4) * RB + ((low2 ^ tile_swz<HD>(kk0 + 4)) * 16) + (li & 1) * 8);

  int tag_base = 0;
  Pack8 df[2][RT][4];  // this lane's dS rows of two consecutive steps (B operands)
  bool dfp[2][RT];
  int rid[G];
  for (int cb = 0; cb < ncols; cb += cols_per_batch) {
    const int nsteps = prepare_batch(cb, min(ncols, cb + cols_per_batch));
    if (nsteps == 0) continue;
    auto row_id = [&](int step) {  // row of list position tid of the step (clamped)
      const int4 info = sInfo[min(step, nsteps - 1)];
      const int n = __builtin_amdgcn_readfirstlane(info.y) & 0xffff;
      const int64_t pos0 = (int64_t)(uint32_t)__builtin_amdgcn_readfirstlane(info.z) | ((int64_t)__builtin_amdgcn_readfirstlane(info.w) << 32);
      return a.row_indices[pos0 + min(tid & (ROWS - 1), n - 1)];
    };
    auto put_pos = [&](int step, int rr) {  // thread t tells row rr, the t-th of the step's run, where it is
      if (step < nsteps && tid < ROWS) {
        const int4 info = sInfo[step];
        const int key0 = info.x, n = info.y & 0xffff;
        const int first_rel = causal ? key0 - off - m0 : -0x40000000;  // rows before it see no key of the block
        const int rel = rr - m0;
        if ((tid < n) & ((uint32_t)rel < (uint32_t)rows_sb) & (rel >= first_rel)) sPos[(step % NS) * ROWS + rel] = ((tag_base + step + 1) << 10) | tid;
      }
    };
    auto k_issue = [&](int step) {  // this wave's share of the K tile of `step`
      const int key0 = __builtin_amdgcn_readfirstlane(sInfo[min(step, nsteps - 1)].x);
      const uint32_t dst = ldsK + (uint32_t)__builtin_amdgcn_readfirstlane(step % NS) * TB + (uint32_t)(wave * NKI) * 1024u;
      if (key0 + 64 <= Lk) {
        const uint16_t *kb0 = kp + (int64_t)key0 * a.k_row_stride;
#pragma unroll
        for (int i = 0; i < NKI; ++i) global_to_lds16_sbase(ksrc[i] * 2u, kb0, dst + (uint32_t)i * 1024u);
      } else {  // keys past the end of the sequence: the last key's data, which meets dS = 0
#pragma unroll
        for (int i = 0; i < NKI; ++i) {
          const int r = (wave * NKI + i) * RPI + krl;
          const int key = min(key0 + r, Lk - 1), e = min((kpp ^ tile_swz<HD>(r)) * 8, D - 8);
          global_to_lds16(kp + (int64_t)key * a.k_row_stride + e, dst + (uint32_t)i * 1024u);
        }
      }
    };
    // fetch this lane's dS rows of `step` into ring entry R (unconditional: an absent row reads a piece near its neighbours')
    auto fetch = [&](auto rc, int step) {
      constexpr int R = decltype(rc)::value;
      const int sc_ = min(step, nsteps - 1);
      // (all LDS reads first: one wait)
      const int4 info = sInfo[sc_];
      int v[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) v[rt] = sPos[(sc_ % NS) * ROWS + myrow[rt]];
      const int ny = __builtin_amdgcn_readfirstlane(info.y);
      const int n = ny & 0xffff, kb = ny >> 16;
      const int64_t pos0 = (int64_t)(uint32_t)__builtin_amdgcn_readfirstlane(info.z) | ((int64_t)__builtin_amdgcn_readfirstlane(info.w) << 32);
      // ds_piece_offset(pos0 + j, 8 kb + hh + 2 s4, Bn / 8) in two parts: what the step's run has in common (the tile of
      // its first position and the block's first piece: scalar arithmetic, 64 bits) and the lane's own part (at most
      // 17 tiles further on: 32 bits, no wide multiply among the vector instructions)
      const uint32_t kgs = (uint32_t)Bn >> 3, r0s = (uint32_t)pos0 & 31u;
      const uint16_t *base = ds_ws + (((pos0 >> 5) * (int64_t)kgs + 8 * kb) << 8);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const bool pres = (step < nsteps) & ((v[rt] >> 10) == tag_base + sc_ + 1);
        const uint32_t j = pres ? (uint32_t)(v[rt] & 1023) : mul24_u32((uint32_t)myrow[rt], (uint32_t)n) / (uint32_t)ROWS;
        const uint32_t t = r0s + j;
        const uint32_t lane_bytes = ((mul24_u32(t >> 5, kgs) + (uint32_t)hh) << 9) + ((t & 31u) << 4);
        const uint16_t *rp = reinterpret_cast<const uint16_t *>(reinterpret_cast<const uint8_t *>(base) + lane_bytes);
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) df[R][rt][s4] = ld_global16(rp + 512 * s4);
        dfp[R][rt] = pres;
      }
    };
    // the products of `step`; `between` runs after the first group of them (the tile loads of a later step: issued
    // there, they are younger than every load this step has waited for)
    auto compute = [&](auto rc, int step, auto &&between) {
      constexpr int R = decltype(rc)::value;
      bool anyp = false;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) anyp |= dfp[R][rt];
      if (!__any(anyp) || step >= nsteps) {
        between();
        return;
      }
      Pack8 dz[RT][4];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
          for (int w = 0; w < 4; ++w) dz[rt][s4].w[w] = dfp[R][rt] ? df[R][rt][s4].w[w] : 0u;
      const uint32_t stage = ldsK + (uint32_t)__builtin_amdgcn_readfirstlane(step % NS) * TB;
      const uint32_t alo = tlo + stage, ahi = thi + stage;
      // K^T operands half a feature tile (two products per row tile) ahead of their use
      Pack8 kf[2][2];
      auto kread = [&](int u, Pack8 (&dst)[2]) {  // unit u: feature tile u / 2, keys 32 (u % 2) .. + 31
        const uint32_t x = (uint32_t)((u >> 1) * 64);
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const uint32_t o = (uint32_t)(16 * (2 * (u & 1) + s2) * RB);
          dst[s2] = lds_tr8((alo ^ x) + o, (ahi ^ x) + o);
        }
      };
      kread(0, kf[0]);
#pragma unroll
      for (int u = 0; u < 2 * NDT; ++u) {
        if (u + 1 < 2 * NDT) kread(u + 1, kf[(u + 1) & 1]);
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) acc[rt][u >> 1] = mfma32<T>(kf[u & 1][s2], dz[rt][2 * (u & 1) + s2], acc[rt][u >> 1]);
        if (u == 0) between();
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // before the loop: positions of steps 0 .. G, row ids of steps G + 1 .. 2 G, K tiles of steps 0 .. G - 1, dS rows of step 0
    {
      int r0[G + 1];
#pragma unroll
      for (int g = 0; g <= G; ++g) r0[g] = row_id(g);
#pragma unroll
      for (int g = 0; g < G; ++g) rid[g] = row_id(G + 1 + g);
#pragma unroll
      for (int g = 0; g <= G; ++g) put_pos(g, r0[g]);
    }
#pragma unroll
    for (int g = 0; g < G; ++g) k_issue(g);
    __syncthreads();
    fetch(std::integral_constant<int, 0>{}, 0);
    wait_all_loads();
    // group of steps s0 .. s0 + G - 1: positions of steps s0 + G + 1 .. s0 + 2 G into LDS, row ids of the G steps after
    // those, then per step the dS rows of the next step and the products of this one; the K tile loads of the next
    // group are issued among the products of the group's first step
    const int nsteps_pad = (nsteps + G - 1) / G * G;
    for (int s0 = 0; s0 < nsteps_pad; s0 += G) {
      __syncthreads();  // the K tiles of this group and the positions up to step s0 + G are in LDS; everyone is done with the group before
#pragma unroll
      for (int g = 0; g < G; ++g) put_pos(s0 + G + 1 + g, rid[g]);
#pragma unroll
      for (int g = 0; g < G; ++g) rid[g] = row_id(s0 + 2 * G + 1 + g);
      static_for<G>([&](auto e) {
        constexpr int E = decltype(e)::value;
        const int s = s0 + E;
        fetch(std::integral_constant<int, (E + 1) & 1>{}, s + 1);
        compute(std::integral_constant<int, E & 1>{}, s, [&]() {
          if constexpr (E == 0) {
#pragma unroll
            for (int g = 0; g < G; ++g) k_issue(s0 + G + g);
          }
        });
      });
      // this wave's share of the next group's K tiles has to be in LDS at the barrier: everything but the dS rows
      // fetched after it was issued
      wait_loads_but<(G - 1) * 4 * RT>();
    }
    tag_base += nsteps;
    wait_all_loads();
  }
  __syncthreads();  // every wave is done with the K tiles: they now hold the output tiles (one 32-row tile per wave)
  uint16_t *sOut = reinterpret_cast<uint16_t *>(smem + SM::oK) + (size_t)wave * 32 * LDO;
  uint16_t *op = reinterpret_cast<uint16_t *>(a.dq) + (int64_t)(q0 + m0) * a.dq_row_stride + (int64_t)h * a.dq_head_stride;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *reinterpret_cast<uint2 *>(sOut + (lane & 31) * LDO + dt * 32 + 8 * g + 4 * hh) =
            make_uint2(pack2<T>(acc[rt][dt][4 * g] * a.softmax_scale, acc[rt][dt][4 * g + 1] * a.softmax_scale),
                       pack2<T>(acc[rt][dt][4 * g + 2] * a.softmax_scale, acc[rt][dt][4 * g + 3] * a.softmax_scale));
    wave_lds_fence();
    // rows leave as 16-byte pieces, VPR of them per row, consecutive lanes taking consecutive pieces
#pragma unroll
    for (int v0 = 0; v0 < 32 * VPR; v0 += 64) {
      const int v = v0 + lane, rl = v / VPR, e = (v - rl * VPR) * 8;
      const int r2 = (wtile * RT + rt) * 32 + rl;
      if (r2 < rows_sb && e < D)
        *reinterpret_cast<Pack8 *>(op + (int64_t)r2 * a.dq_row_stride + e) = *reinterpret_cast<const Pack8 *>(sOut + rl * LDO + e);
    }
    wave_lds_fence();
  }
}

// ------------------------------------------------------------------------------------
// dQ, second form: the row's partials are added in ascending key-block order (sorted by block id: the slot a visit
// got is arbitrary, the sum must not depend on it) and scaled.  One 16-lane group per (row, head), four per wave,
// sixteen per block of 256: a row's chain of dependent steps (count, ids, order, rows) is mostly waiting, so a wave
// runs four of them side by side.  Lane li of a group owns the 16-byte piece li of the row.
// ------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void attn_bwd_dq_combine_kernel(fmoba_attn_bwd_args a, BwdWs ws, int capl) {
  extern __shared__ __attribute__((aligned(16))) int sOrdAll[];  // [16 groups][capl]: slot of the partial of rank r
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
  const int32_t *pid = ws.pid + rh * ws.cap;
  const uint16_t *part = ws.part + rh * ws.cap * D;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  // ranks over the whole row: the order of the sum does not depend on which slot a visit got
  group_rank_order(pid, 1, n, nmax, sOrd, lane);
  if (mine) {
    auto add = [&](const Pack8 &x) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        acc[2 * k] += elem_to_float<T>((uint16_t)(x.w[k] & 0xffffu));
        acc[2 * k + 1] += elem_to_float<T>((uint16_t)(x.w[k] >> 16));
      }
    };
    int t = 0;
    for (; t + 4 <= n; t += 4) {  // independent loads, four in flight
      Pack8 x[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) x[u] = ld_stream16(part + (int64_t)sOrd[t + u] * D + c8);
#pragma unroll
      for (int u = 0; u < 4; ++u) add(x[u]);
    }
    for (; t < n; ++t) add(ld_stream16(part + (int64_t)sOrd[t] * D + c8));
  }
  if (valid && mine) {
    Pack8 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) o.w[k] = pack2<T>(acc[2 * k] * a.softmax_scale, acc[2 * k + 1] * a.softmax_scale);
    *reinterpret_cast<Pack8 *>(reinterpret_cast<uint16_t *>(a.dq) + row * a.dq_row_stride + (int64_t)h * a.dq_head_stride + c8) = o;
  }
}

// grid (ceil(max_seqlen_q / rows_per_block), heads, batch), block 256.
// LPR lanes cooperate on one row (LPR = power of two >= head_dim / 8).
constexpr int kPrepRows = 4;  // rows per thread: eight 16-byte loads in flight (with one row a thread had two, 4.7 TB/s)
template <typename T>
__global__ __launch_bounds__(256) void bwd_prep_kernel(fmoba_attn_bwd_args a, int LPR) {
  const int rows_per_pass = 256 / LPR;
  const int h = blockIdx.y, b = blockIdx.z;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int r0 = blockIdx.x * rows_per_pass * kPrepRows + threadIdx.x / LPR;
  if (blockIdx.x * rows_per_pass * kPrepRows >= Lq) return;
  const int sub = threadIdx.x % LPR;
  const int e = sub * 8;
  const int D = a.head_dim;
  Pack8 o[kPrepRows], g[kPrepRows];
#pragma unroll
  for (int k = 0; k < kPrepRows; ++k) {
    const int r = r0 + k * rows_per_pass;
    o[k] = zero_pack8();
    g[k] = zero_pack8();
    if (r < Lq && e < D) {
      o[k] = ld_global16(reinterpret_cast<const uint16_t *>(a.out) + (int64_t)(q0 + r) * a.o_row_stride + (int64_t)h * a.o_head_stride + e);
      g[k] = ld_global16(reinterpret_cast<const uint16_t *>(a.dout) + (int64_t)(q0 + r) * a.do_row_stride + (int64_t)h * a.do_head_stride + e);
    }
  }
#pragma unroll
  for (int k = 0; k < kPrepRows; ++k) {
    const int r = r0 + k * rows_per_pass;
    float fo[8], fg[8];
    unpack8<T>(o[k], fo);
    unpack8<T>(g[k], fg);
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc = fmaf(fo[i], fg[i], acc);
    for (int w = LPR >> 1; w >= 1; w >>= 1) acc += __shfl_xor(acc, w, 64);
    if (r < Lq && sub == 0) a.softmax_d[(int64_t)h * ((int64_t)a.total_q + 128 * (int64_t)a.batch) + q0 + 128 * b + r] = acc;
  }
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

__global__ void zero_i32_kernel(int32_t *p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0;
}

__global__ void zero_f32_kernel(float *p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0.f;
}

template <typename T, int HD, bool DQP, int KB, bool NEAR>
static int launch_dkdv_form(const fmoba_attn_bwd_args &a, const BwdWs &ws, hipStream_t s) {
  auto kern = attn_bwd_dkdv_kernel<T, HD, DQP, KB, NEAR>;
  const size_t smem = BwdSmem<HD>::bytes;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("attn_bwd: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  const int64_t items = (int64_t)a.batch * a.heads * ceil_div(a.max_seqlen_k, 64 * KB);
  if (items >= ((int64_t)1 << 31)) {
    set_error("attn_bwd: too many (sequence, head, key block) work items");
    return 1;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)items), dim3(256), smem, s, a, ws);
  return 0;
}
// NEAR: every row of a sequence's q and dout lies within 2 GB of the sequence's first row and is less than 2^24 rows
// and 2^22 elements per row away, so a gathered row's place is a 32-bit offset made by one 24-bit multiply.
template <typename T, int HD, bool DQP, int KB>
static int launch_dkdv(const fmoba_attn_bwd_args &a, const BwdWs &ws, hipStream_t s) {
  const bool near_rows = a.max_seqlen_q < (1 << 24) && a.q_row_stride < (1 << 22) && a.do_row_stride < (1 << 22) &&
                         (int64_t)a.max_seqlen_q * a.q_row_stride < (int64_t)0x7fff0000 && (int64_t)a.max_seqlen_q * a.do_row_stride < (int64_t)0x7fff0000;
  return near_rows ? launch_dkdv_form<T, HD, DQP, KB, true>(a, ws, s) : launch_dkdv_form<T, HD, DQP, KB, false>(a, ws, s);
}

template <typename T, int HD, int RT>
static int launch_dq(const fmoba_attn_bwd_args &a, const uint16_t *ws, hipStream_t s) {
  auto kern = attn_bwd_dq_kernel<T, HD, RT>;
  const size_t smem = DqSmem<HD, RT>::bytes;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("attn_bwd: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  const int nsb_max = ceil_div(a.max_seqlen_q, DqSmem<HD, RT>::ROWS);
  const int64_t items = (int64_t)a.heads * a.batch * nsb_max;
  if (items >= ((int64_t)1 << 31)) {
    set_error("attn_bwd: too many (sequence, head, superblock) work items");
    return 1;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)items), dim3(512), smem, s, a, ws, nsb_max);
  return 0;
}

// head dimensions above 128 (attn_bwd_wide.hip)
int run_bwd_dkdv_wide(const fmoba_attn_bwd_args &a, uint16_t *ds_ws, hipStream_t s);

// columns of a multiple of 128 keys: one workgroup (and one dQ partial per visit) per 128 keys
static inline bool bwd_wide_blocks(const fmoba_attn_bwd_args &a) { return a.head_dim > 64 && a.lg_block_n % 128 == 0; }

// Which form of the dQ computation a call uses.  The row-stationary form works on (128-row block, key block) steps
// and is the faster one while a step has enough rows; with many chunks per sequence a step has one or two rows and
// only the per-visit partials scale.  Measured break-even points (16 heads of 128, 8K and 16K tokens per sequence,
// top-k 8 to 32): a row selects a tenth of the chunks it may see (64-key blocks), three eighths with 128-key blocks,
// where a visit leaves one partial per 128 keys.
static int bwd_dq_partials(const fmoba_attn_bwd_args &a) {
  if (a.head_dim > 128) return 0;  // head dimensions above 128: dS tiles and the row-block pass only
  if (a.dq_mode == 1) return 0;
  if (a.dq_mode == 2) return 1;
  const double chunks_per_seq = (double)a.total_k / a.batch / a.lg_block_n;
  const double chunks_per_row = (double)a.max_visits_per_row * 64.0 / a.lg_block_n;
  const double seen = a.is_causal ? 0.5 * chunks_per_seq : chunks_per_seq;
  return chunks_per_row < (bwd_wide_blocks(a) ? 0.37 : 0.10) * seen;
}
// partial slots per (row, head): max_visits_per_row counts 64-key blocks; with 128-key blocks a row has half as many
// visits (only the last column of a sequence can have an odd number of 64-key blocks)
static inline int32_t bwd_partial_cap(const fmoba_attn_bwd_args &a) {
  const int32_t mv = a.max_visits_per_row > 0 ? a.max_visits_per_row : 1;
  return bwd_wide_blocks(a) ? (mv + 1) / 2 : mv;
}

template <typename T>
static int run_bwd(const fmoba_attn_bwd_args &a, const BwdWs &ws, int phases, hipStream_t s) {
  const bool partials = bwd_dq_partials(a);
  if (phases & FMOBA_BWD_PREP) {
    int lpr = 1;
    while (lpr * 8 < a.head_dim) lpr <<= 1;
    const int rows_per_block = 256 / lpr;
    hipLaunchKernelGGL(bwd_prep_kernel<T>, dim3(ceil_div(a.max_seqlen_q, rows_per_block * kPrepRows), a.heads, a.batch), dim3(256), 0, s, a, lpr);
  }
  if (a.head_dim > 128) {
    // the plain feature-split dK/dV kernel (attn_bwd_wide.hip), then the row-block dQ pass over its dS tiles
    if (phases & FMOBA_BWD_DKDV)
      if (int rc = run_bwd_dkdv_wide(a, ws.ds, s)) return rc;
    if (phases & FMOBA_BWD_DQ)
      if (int rc = launch_dq<T, 256, 1>(a, ws.ds, s)) return rc;
    return 0;
  }
  if (phases & FMOBA_BWD_DKDV) {
    int rc;
    // columns of a multiple of 128 keys: one workgroup per 128 keys (the two 64-key blocks share their row list)
    const bool wide = bwd_wide_blocks(a);
    if (partials) {
      hipLaunchKernelGGL(zero_i32_kernel, dim3(512), dim3(256), 0, s, ws.cnt, (int64_t)a.total_q * a.heads);
      rc = a.head_dim <= 64 ? launch_dkdv<T, 64, true, 1>(a, ws, s) : (wide ? launch_dkdv<T, 128, true, 2>(a, ws, s) : launch_dkdv<T, 128, true, 1>(a, ws, s));
    } else {
      rc = a.head_dim <= 64 ? launch_dkdv<T, 64, false, 1>(a, ws, s) : (wide ? launch_dkdv<T, 128, false, 2>(a, ws, s) : launch_dkdv<T, 128, false, 1>(a, ws, s));
    }
    if (rc) return rc;
  }
  if (phases & FMOBA_BWD_DQ) {
    if (partials) {
      const int64_t rows = (int64_t)a.total_q * a.heads;
      const int capl = combine_order_entries(ws.cap);
      const size_t smem = (size_t)16 * capl * 4;
      auto kern = attn_bwd_dq_combine_kernel<T>;
      if (smem > 32 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
        set_error("attn_bwd: a row with up to %d visits needs %zu bytes of LDS for the order of its partial results", ws.cap, smem);
        return 2;
      }
      hipLaunchKernelGGL(kern, dim3((unsigned)((rows + 15) / 16)), dim3(256), smem, s, a, ws, capl);
    } else {
      int rc = a.head_dim <= 64 ? launch_dq<T, 64, 1>(a, ws.ds, s) : launch_dq<T, 128, 2>(a, ws.ds, s);
      if (rc) return rc;
    }
  }
  return 0;
}

static inline size_t bwd_align256(size_t x) { return (x + 255) & ~(size_t)255; }

}  // namespace fmoba

extern "C" int32_t fmoba_attn_bwd_uses_partials(const fmoba_attn_bwd_args *a) {
  if (a == nullptr || a->batch <= 0 || a->lg_block_n <= 0) return 0;
  return fmoba::bwd_dq_partials(*a);
}

extern "C" size_t fmoba_attn_bwd_workspace_bytes(const fmoba_attn_bwd_args *a) {
  using namespace fmoba;
  if (a == nullptr || a->total_q <= 0 || a->heads <= 0 || a->head_dim <= 0 || a->batch <= 0 || a->lg_block_n <= 0) return 256;
  if (!bwd_dq_partials(*a)) return ds_workspace_tiles(a->num_row_indices) * (size_t)a->lg_block_n * 64 + 256;
  const size_t rows = (size_t)a->total_q * a->heads, cap = (size_t)bwd_partial_cap(*a);
  // one spare partial row / block id at the end takes the writes of absent rows
  return bwd_align256(rows * 4) + bwd_align256((rows * cap + 1) * 4) + bwd_align256((rows * cap + 1) * a->head_dim * 2) + 256;
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
  FMOBA_REQUIRE(a->heads > 0 && a->heads_k > 0 && a->heads % a->heads_k == 0, "Number of heads in key/value must divide number of heads in query");
  FMOBA_REQUIRE(a->lg_block_m % 64 == 0, "m_lg_block_dim must be a multiple of 64");
  FMOBA_REQUIRE(a->lg_block_n > 0 && a->lg_block_n % 64 == 0, "n_lg_block_dim must be a multiple of 64");
  FMOBA_REQUIRE(a->lg_block_n <= 64 * 256, "attn_bwd: n_lg_block_dim above 16384 is not supported");
  FMOBA_REQUIRE(a->total_q >= 0 && a->total_k >= 0 && a->max_seqlen_q >= 0 && a->max_seqlen_k >= 0 && a->max_cols >= 0 && a->max_visits_per_row >= 0 && a->num_row_indices >= 0,
                "negative size");
  FMOBA_REQUIRE(a->cu_seqlens_q && a->cu_seqlens_k, "attn_bwd: null cu_seqlens pointer");
  FMOBA_REQUIRE(a->batch <= 65535 && a->heads <= 65535, "attn_bwd: batch/heads too large for the launch grid");
  hipStream_t s = (hipStream_t)stream;
  const int64_t st[] = {a->q_row_stride,  a->q_head_stride,  a->k_row_stride,  a->k_head_stride,  a->v_row_stride,  a->v_head_stride,
                        a->o_row_stride,  a->o_head_stride,  a->do_row_stride, a->do_head_stride, a->dq_row_stride, a->dq_head_stride,
                        a->dk_row_stride, a->dk_head_stride, a->dv_row_stride, a->dv_head_stride};
  for (int64_t x : st) FMOBA_REQUIRE(x % 8 == 0, "attn_bwd: strides must be multiples of 8 elements");
  FMOBA_REQUIRE(a->k_row_stride < ((int64_t)1 << 24), "attn_bwd: k_row_stride must be below 2^24 elements");
  FMOBA_REQUIRE(a->q_row_stride < ((int64_t)1 << 31) && a->do_row_stride < ((int64_t)1 << 31), "attn_bwd: q / dout row strides must be below 2^31 elements");
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
  FMOBA_REQUIRE(a->max_visits_per_row > 0, "attn_bwd: max_visits_per_row must be positive");
  FMOBA_REQUIRE(a->dq_mode >= 0 && a->dq_mode <= 2, "attn_bwd: dq_mode must be 0 (automatic), 1 (row blocks) or 2 (partials)");
  FMOBA_REQUIRE(a->dq_mode != 2 || a->head_dim <= 128, "attn_bwd: head dimensions above 128 only have the row-block form of dQ");
  FMOBA_REQUIRE(a->workspace != nullptr && a->workspace_bytes >= fmoba_attn_bwd_workspace_bytes(a), "attn_bwd: workspace too small");
  const size_t rows = (size_t)a->total_q * a->heads;
  uintptr_t wp = ((uintptr_t)a->workspace + 255) & ~(uintptr_t)255;
  BwdWs ws;
  ws.cap = bwd_partial_cap(*a);
  // (the dK/dV pass keeps the place of a visit's dQ partial as a 32-bit index of partial rows)
  FMOBA_REQUIRE(!fmoba::bwd_dq_partials(*a) || rows * (size_t)ws.cap + 1 < ((size_t)1 << 31),
                "attn_bwd: %zu rows x heads with up to %d dQ partials each are more partial rows than the partials form addresses", rows, ws.cap);
  ws.ds = reinterpret_cast<uint16_t *>(wp);
  ws.cnt = reinterpret_cast<int32_t *>(wp);
  wp += bwd_align256(rows * 4);
  ws.pid = reinterpret_cast<int32_t *>(wp);
  wp += bwd_align256((rows * ws.cap + 1) * 4);
  ws.part = reinterpret_cast<uint16_t *>(wp);
  int rc = a->dtype == FMOBA_DTYPE_BF16 ? run_bwd<bf16_t>(*a, ws, phases, s) : run_bwd<f16_t>(*a, ws, phases, s);
  if (rc) return rc;
  FMOBA_LAUNCH_CHECK("attn_bwd");
  return 0;
}
