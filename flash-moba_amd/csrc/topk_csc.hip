// Fused top-k block gating and deterministic CSC build.
//
//   topk_gate_kernel : scores S^T = KM * Q^T on MFMA, per-row exact top-k by bisection on
//                      order-preserving keys held in registers (no score matrix, no sorted
//                      list and no per-row index list ever reaches HBM); emits one selection
//                      BIT per (row, chunk) and per-(2048-row segment, chunk) counts.
//   csc_scan_kernel  : per (sequence, head) scan of the counts -> col_nnz, col_offsets
//                      (int64) and per-segment start offsets; clears the unused tail of
//                      the row-list buffer.
//   csc_fill_kernel  : walks the bit columns in row order and writes each chunk's row list
//                      ascending, so no sort pass is needed afterwards.
#include "fmoba_common.h"

#include <mutex>

namespace fmoba {

constexpr int kGateRows = 128;   // query rows per workgroup (4 waves x 32)
constexpr int kSegRows = 2048;   // rows per counting segment (fewer for small problems, see csc_seg_rows)

struct TopkParams {
  fmoba_fused_topk_args a;
  uint32_t *sel;      // [heads][W][total_q] selection bits, word w covers chunks 32w..32w+31
  int32_t *segcnt;    // [batch][heads][nseg][max_cols]
  int32_t W, nseg, max_cols, seg_rows;
};

// Rows per counting segment.  A wave of the fill kernel walks one segment of one 32-chunk word column, 64 rows at a
// time, one step after the other, and a step is a chain (load the words, 32 ballots, a store per chunk) that only
// other waves can cover: segments of 2048 rows keep the counts small, but the fill wants many thousands of waves,
// so segments shrink (down to 256 rows, a multiple of the gate's 128-row blocks) until there are 16384 of them.  The
// headline batch (eight sequences, 65536 tokens) gets 512-row segments: fill 116 -> 63 us against 6272 waves of 2048
// rows (256-row segments: 56 us, but twice the counts to clear, scan and keep); a single sequence of 8192 tokens
// 86 -> 15 us against its 128 waves.  Beyond that the fill does not gain (262144 tokens: 131072 waves of 2048 rows
// 1.55 ms, twice as many of 1024 rows 1.62 ms and the scan of the counts four times as long).
static inline int csc_seg_rows(int64_t batch, int64_t heads, int64_t max_seqlen_q, int64_t W) {
  int seg_rows = kSegRows;
  const int64_t lq = max_seqlen_q > 0 ? max_seqlen_q : 1;
  while (seg_rows > 256 && batch * heads * W * ((lq + seg_rows - 1) / seg_rows) < 16384) seg_rows >>= 1;
  return seg_rows;
}

// n + (x0 > y) + (x1 > y) + (x2 > y) + (x3 > y): four compares into four scalar register pairs, then four adds with
// carry, so that no add follows its compare at once (a vector instruction that reads a scalar register written by the
// one before it has to wait; left alone, the compiler pairs every compare with its consumer and pads with idle slots)
__device__ __forceinline__ int count4_gt(int n, float x0, float x1, float x2, float x3, float y) {
#if defined(__HIP_DEVICE_COMPILE__)
  unsigned long long m0, m1, m2, m3;
  asm("v_cmp_gt_f32_e64 %1, %5, %9\n\t"
      "v_cmp_gt_f32_e64 %2, %6, %9\n\t"
      "v_cmp_gt_f32_e64 %3, %7, %9\n\t"
      "v_cmp_gt_f32_e64 %4, %8, %9\n\t"
      "v_addc_co_u32_e64 %0, vcc, 0, %0, %1\n\t"
      "v_addc_co_u32_e64 %0, vcc, 0, %0, %2\n\t"
      "v_addc_co_u32_e64 %0, vcc, 0, %0, %3\n\t"
      "v_addc_co_u32_e64 %0, vcc, 0, %0, %4"
      : "+v"(n), "=&s"(m0), "=&s"(m1), "=&s"(m2), "=&s"(m3)
      : "v"(x0), "v"(x1), "v"(x2), "v"(x3), "v"(y)
      : "vcc");
  return n;
#else
  return n + (x0 > y) + (x1 > y) + (x2 > y) + (x3 > y);
#endif
}

// n + (x >= y) in two halves: four compares into four scalar register pairs first, then an add with carry per flag
// where the count is needed (a vector instruction that reads a scalar register written by the one before it has to
// wait two slots: with the compares of four scores ahead of their adds nothing waits; left alone, the compiler
// materialises every flag as 0 / 1 first).  Volatile, so that the compares stay ahead of the adds.
struct Flags4 {
  unsigned long long m[4];
};
__device__ __forceinline__ Flags4 flags4_ge(float x0, float x1, float x2, float x3, float y) {
  Flags4 f;
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("v_cmp_ge_f32_e64 %0, %4, %8\n\t"
               "v_cmp_ge_f32_e64 %1, %5, %8\n\t"
               "v_cmp_ge_f32_e64 %2, %6, %8\n\t"
               "v_cmp_ge_f32_e64 %3, %7, %8"
               : "=&s"(f.m[0]), "=&s"(f.m[1]), "=&s"(f.m[2]), "=&s"(f.m[3])
               : "v"(x0), "v"(x1), "v"(x2), "v"(x3), "v"(y));
#else
  f.m[0] = x0 >= y;
  f.m[1] = x1 >= y;
  f.m[2] = x2 >= y;
  f.m[3] = x3 >= y;
#endif
  return f;
}
__device__ __forceinline__ int count_flag(int n, unsigned long long flag) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("v_addc_co_u32_e64 %0, vcc, 0, %0, %1" : "+v"(n) : "s"(flag) : "vcc");
  return n;
#else
  return n + (int)(flag & 1);
#endif
}

// the same with x > y
__device__ __forceinline__ Flags4 flags4_gt(float x0, float x1, float x2, float x3, float y) {
  Flags4 f;
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("v_cmp_gt_f32_e64 %0, %4, %8\n\t"
               "v_cmp_gt_f32_e64 %1, %5, %8\n\t"
               "v_cmp_gt_f32_e64 %2, %6, %8\n\t"
               "v_cmp_gt_f32_e64 %3, %7, %8"
               : "=&s"(f.m[0]), "=&s"(f.m[1]), "=&s"(f.m[2]), "=&s"(f.m[3])
               : "v"(x0), "v"(x1), "v"(x2), "v"(x3), "v"(y));
#else
  f.m[0] = x0 > y;
  f.m[1] = x1 > y;
  f.m[2] = x2 > y;
  f.m[3] = x3 > y;
#endif
  return f;
}
// (w << 1) | flag of the lane: one add with carry
__device__ __forceinline__ uint32_t shift_in_flag(uint32_t w, unsigned long long flag) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("v_addc_co_u32_e64 %0, vcc, %0, %0, %1" : "+v"(w) : "s"(flag) : "vcc");
  return w;
#else
  return (w << 1) | (uint32_t)(flag & 1);
#endif
}

template <typename T, int HD, int NT>
__global__ __launch_bounds__(256, (NT == 8 || HD > 128) ? 2 : 4) void topk_gate_kernel(TopkParams p) {
  constexpr int KS = HD / 16;
  constexpr int VPR = HD / 8;    // 16-byte pieces of a row of chunk means
  constexpr int RPI = 64 / VPR;  // tile rows one load instruction brings (64 lanes x 16 bytes)
  constexpr int RB = HD * 2;     // bytes of a tile row: exactly HD elements, swizzled instead of padded
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  int *sHist = reinterpret_cast<int *>(smem + (size_t)NT * 32 * RB);

  const fmoba_fused_topk_args &a = p.a;
  const int mb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int q0 = a.cu_seqlens_q[b];
  const int Lq = a.cu_seqlens_q[b + 1] - q0;
  const int m0 = mb * kGateRows;
  if (m0 >= Lq) return;
  const int Lk = a.cu_seqlens_k[b + 1] - a.cu_seqlens_k[b];
  const int km0 = a.cu_seqlens_km[b];
  const int Cb = a.cu_seqlens_km[b + 1] - km0;
  const int off = Lk - Lq;
  const int B = a.chunk;
  const int D = a.head_dim;
  const int hk = h / (a.heads / a.heads_k);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;

  // chunks [0, nsc) can be candidates of some row of this block
  int nsc;
  if (a.is_causal) {
    const int rmax = min(m0 + kGateRows - 1, Lq - 1) + off;
    nsc = rmax < 0 ? 0 : min(Cb, rmax / B);
  } else {
    nsc = Cb;
  }
  nsc = min(nsc, min(p.max_cols, NT * 32));  // never beyond the LDS tile, whatever max_seqlen_k the caller gave
  const int n_tiles = (nsc + 31) >> 5;

  // The chunk means of this (sequence, kv head) go from global memory straight into LDS (global_load_lds, all loads
  // of a wave in flight at once): piece c of tile row r lies at piece c ^ tile_swz<HD>(r).  Rows past the last chunk
  // that can be a candidate and features past head_dim are fetched from a row / piece that exists: such scores are
  // masked below, such features meet zeros of q.
  const uint32_t ldsTile = (uint32_t)(uintptr_t)smem;
  if (nsc > 0) {
    const uint16_t *kmp = reinterpret_cast<const uint16_t *>(a.km) + (int64_t)hk * a.km_head_stride;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int ninstr = n_tiles * 32 / RPI;
    for (int v = wave_u; v < ninstr; v += 4) {
      const int c = v * RPI + lane / VPR, pc = lane % VPR;
      const int e = min((pc ^ tile_swz<HD>(c)) * 8, D - 8);
      global_to_lds16(kmp + (int64_t)(km0 + min(c, nsc - 1)) * a.km_row_stride + e, ldsTile + (uint32_t)v * 1024u);
    }
  }
  for (int v = tid; v < NT * 32; v += 256) sHist[v] = 0;

  // this lane's query row and its operand slices (contraction index permuted so that each
  // half-wave reads one contiguous half of the row)
  const int r = m0 + wave * 32 + (lane & 31);
  const bool valid = r < Lq;
  Pack8 qf[KS];
  {
    const uint16_t *qp = reinterpret_cast<const uint16_t *>(a.q) + (int64_t)(q0 + (valid ? r : 0)) * a.q_row_stride + (int64_t)h * a.q_head_stride;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int e = (hh * KS + ks) * 8;
      qf[ks] = (valid && e < D) ? ld_global16(qp + e) : zero_pack8();
    }
  }
  wait_all_loads();
  __syncthreads();

  // scores: lane (query l%32) gets chunk t*32 + acc_row(i, hh) in register i of tile t;
  // chunks that are not candidates of the row hold -inf
  float sc[NT][16];
  const int rp = r + off;
  int nc;  // number of candidate chunks of this row: chunks strictly before its own chunk
  if (a.is_causal)
    nc = (valid && rp >= 0) ? min(rp / B, Cb) : 0;
  else
    nc = valid ? Cb : 0;
  nc = min(nc, nsc);
  float vmin = INFINITY, vmax = -INFINITY;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    if (t < n_tiles) {
      f32x16 acc;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const Pack8 af = lds_read16(ldsTile + (uint32_t)((t * 32 + (lane & 31)) * RB) + (uint32_t)(((hh * KS + ks) ^ tile_swz<HD>(lane & 31)) * 16));
        acc = mfma32<T>(af, qf[ks], acc);
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int c = t * 32 + acc_row(i, hh);
        const bool cand = c < nc;
        const float x = acc[i];
        sc[t][i] = cand ? x : -INFINITY;
        vmin = fminf(vmin, cand ? x : INFINITY);
        vmax = fmaxf(vmax, sc[t][i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) sc[t][i] = -INFINITY;
    }
  }
  vmin = min_xor32_f(vmin);
  vmax = max_xor32_f(vmax);

  // K' = number of scored chunks to keep (the own chunk takes one slot in causal mode).
  // A row keeps every candidate x with x > tau, plus, among the candidates equal to tau_eq,
  // those with chunk index >= iota.  tau is found by bisection between the row's smallest
  // and largest score and the search stops as soon as exactly K' scores lie above the probe.
  // The bracket is kept as order-preserving integer keys (lo_k, hi_k]; the first probes
  // bisect the VALUE range (few steps for ordinary score distributions), later ones the key
  // range (at most 32 more steps whatever the values).  If the bracket closes first, the
  // scores inside it are all equal and tie across the cut: the highest chunk indices win.
  const int kp = a.is_causal ? a.topk - 1 : a.topk;
  const bool need = (nc > kp) && (kp > 0);
  float tau = -INFINITY;    // nc <= K': every candidate with a score above -inf
  float tau_eq = INFINITY;  // no tie group by default
  int n_eq = 0;
  uint32_t iota = 0u;
  uint32_t lo_k = float_order_key(vmin) - 1u;  // count(x > lo) = nc > K'
  uint32_t hi_k = float_order_key(vmax);       // count(x > hi) = 0  < K'
  int c_lo = nc, c_hi = 0;
  bool open = need;
  // A row whose bracket holds exactly one score too many, or one too few, needs no more probes: the cut lies right
  // below the largest score of the bracket, or right at its smallest.  When every open row of the wave is in that state
  // (about eight probes in, where the search of the slowest row takes twelve or thirteen), one pass over the scores
  // finds that score for all of them, the largest of -x for the rows that want the smallest.  The cut it gives is
  // exact unless the score occurs twice; such rows are found by their count below and searched to the end.
  bool guessed = false;
  auto bisect = [&](bool may_finish) {
    for (int iter = 0;; ++iter) {
      if (open && hi_k - lo_k <= 1u) {
        // nothing representable strictly inside: every score in (lo, hi] equals hi
        tau = order_key_float(hi_k);
        if (tau != -INFINITY) {
          tau_eq = tau;
          n_eq = kp - c_hi;
        }
        open = false;
      }
      if (!__any(open)) break;
      if (may_finish) {
        const bool up = kp - c_hi == 1, dn = c_lo - kp == 1;
        if (__all(!open || up || dn)) {
          const bool want_min = open && !up;
          const uint32_t flip = want_min ? 0x80000000u : 0u;
          // (x > lo for a score x is x >= the next float above lo, which after -0 is the smallest positive number)
          const uint32_t above_lo = lo_k + (lo_k == 0x7fffffffu ? 2u : 1u);
          const float bound = want_min ? -order_key_float(above_lo) : order_key_float(hi_k);
          float best = -INFINITY;
#pragma unroll
          for (int t = 0; t < NT; ++t)
            if (t < n_tiles) {
#pragma unroll
              for (int i = 0; i < 16; ++i) {
                const float y = __uint_as_float(__float_as_uint(sc[t][i]) ^ flip);
                best = fmaxf(best, y <= bound ? y : -INFINITY);
              }
            }
          best = max_xor32_f(best);
          if (open) {
            const float v = __uint_as_float(__float_as_uint(best) ^ flip);
            uint32_t below = float_order_key(v) - 1u;  // (the float below +0 that compares below it is not -0)
            if (below == 0x7fffffffu) below -= 1u;
            tau = up ? order_key_float(below) : v;
            guessed = true;
            open = false;
          }
          break;
        }
      }
      uint32_t pk = lo_k + ((hi_k - lo_k) >> 1);
      if (iter < 12) {
        const float mf = 0.5f * order_key_float(lo_k + 1u) + 0.5f * order_key_float(hi_k);
        const uint32_t mk = float_order_key(mf);
        if (mk > lo_k && mk < hi_k) pk = mk;
      }
      const float probe = order_key_float(pk);
      int cnt = 0;
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (t < n_tiles) {
#pragma unroll
          for (int i = 0; i < 16; i += 4) cnt = count4_gt(cnt, sc[t][i], sc[t][i + 1], sc[t][i + 2], sc[t][i + 3], probe);
        }
      cnt = sum_xor32_i(cnt);
      if (open) {
        if (cnt == kp) {
          tau = probe;
          open = false;
        } else if (cnt > kp) {
          lo_k = pk;
          c_lo = cnt;
        } else {
          hi_k = pk;
          c_hi = cnt;
        }
      }
    }
  };
  // K' = number of scored chunks to keep (the own chunk takes one slot in causal mode).
  // A row keeps every candidate x with x > tau, plus, among the candidates equal to tau_eq,
  // those with chunk index >= iota.  tau is found by bisection between the row's smallest
  // and largest score and the search stops as soon as exactly K' scores lie above the probe.
  // The bracket is kept as order-preserving integer keys (lo_k, hi_k]; the first probes
  // bisect the VALUE range (few steps for ordinary score distributions), later ones the key
  // range (at most 32 more steps whatever the values).  If the bracket closes first, the
  // scores inside it are all equal and tie across the cut: the highest chunk indices win.
  bisect(true);
  bool any_tie = __any(n_eq > 0);  // some row of the wave has a tie across its cut
  // Without a tie in the wave a score is selected iff it lies above tau: the flags of the lane's 16 scores of a tile,
  // shifted in one by one (w + w + flag: one add with carry each), highest first.
  uint32_t bits[NT];
  auto flags_above_tau = [&]() {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      bits[t] = 0u;
      if (t < n_tiles) {
#pragma unroll
        for (int i4 = 3; i4 >= 0; --i4) {
          const Flags4 f = flags4_gt(sc[t][4 * i4 + 3], sc[t][4 * i4 + 2], sc[t][4 * i4 + 1], sc[t][4 * i4], tau);
#pragma unroll
          for (int j = 0; j < 4; ++j) bits[t] = shift_in_flag(bits[t], f.m[j]);
        }
      }
    }
  };
  if (!any_tie) flags_above_tau();
  if (__any(guessed)) {
    int above = 0;
    if (!any_tie) {
#pragma unroll
      for (int t = 0; t < NT; ++t) above += __popc(bits[t]);
    } else {
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (t < n_tiles) {
#pragma unroll
          for (int i = 0; i < 16; i += 4) above = count4_gt(above, sc[t][i], sc[t][i + 1], sc[t][i + 2], sc[t][i + 3], tau);
        }
    }
    above = sum_xor32_i(above);
    const bool again = guessed && above != kp;
    if (__any(again)) {
      open = again;
      bisect(false);
      any_tie = __any(n_eq > 0);
      if (!any_tie) flags_above_tau();
    }
  }
  // a tie group keeps its n_eq highest chunk indices
  if (any_tie) {
    const bool tie = n_eq > 0;
    int ceq = 0;
#pragma unroll
    for (int t = 0; t < NT; ++t)
      if (t < n_tiles) {
#pragma unroll
        for (int i = 0; i < 16; ++i) ceq += (sc[t][i] == tau_eq) ? 1 : 0;
      }
    ceq = sum_xor32_i(ceq);
    const bool split = tie && ceq > n_eq;
    if (__any(split)) {
      uint32_t i_acc = 0u;
      constexpr int IB = (NT * 32 <= 64) ? 6 : (NT * 32 <= 128 ? 7 : 8);
      for (int bit = IB - 1; bit >= 0; --bit) {
        const uint32_t trial = i_acc | (1u << bit);
        int cnt = 0;
#pragma unroll
        for (int t = 0; t < NT; ++t)
          if (t < n_tiles) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const uint32_t c = (uint32_t)(t * 32 + acc_row(i, hh));
              cnt += ((sc[t][i] == tau_eq) & (c >= trial)) ? 1 : 0;
            }
          }
        cnt = sum_xor32_i(cnt);
        if (cnt >= n_eq) i_acc = trial;
      }
      if (split) iota = i_acc;
    }
  }

  // selection words (32 chunks each), own chunk forced in causal mode
  const bool has_self = a.is_causal && valid && rp >= 0;
  const int pself = has_self ? rp / B : -1;
  const int seg = m0 / p.seg_rows;
  uint32_t *selp = p.sel + (int64_t)h * p.W * a.total_q + q0 + r;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    if (t < p.W) {
      uint32_t w = 0u;
      if (t < n_tiles && kp > 0) {
        if (!any_tie) {
          // the four nibbles of the flags move to the places of the lane's chunks (4 hh + 8 g .. + 3)
          const uint32_t b = bits[t];
          w = ((b & 0xfu) | ((b & 0xf0u) << 4) | ((b & 0xf00u) << 8) | ((b & 0xf000u) << 12)) << (4 * hh);
        } else {
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const uint32_t c = (uint32_t)(t * 32 + acc_row(i, hh));
            const float x = sc[t][i];
            const bool s = (x > tau) | ((x == tau_eq) & (c >= iota));
            w |= s ? (1u << ((8 * (i >> 2) + (i & 3)) + 4 * hh)) : 0u;
          }
        }
      }
      {
        const UPair wp = swap32(w);
        w = wp.a | wp.b;
      }
      if (has_self && (pself >> 5) == t) w |= 1u << (pself & 31);
      if (!valid) w = 0u;
      if (valid && hh == 0) selp[(int64_t)t * a.total_q] = w;
      // per-chunk counts of this wave's 32 rows (both halves of the wave hold the rows' words)
      if (__any(w != 0u)) {
        const int mycnt = bit_column_count32(w, lane);
        if (lane < 32 && mycnt) atomicAdd(&sHist[t * 32 + lane], mycnt);
      }
    }
  }
  __syncthreads();
  for (int c = tid; c < p.W * 32 && c < p.max_cols; c += 256) {
    const int v = sHist[c];
    if (v) atomicAdd(&p.segcnt[(((int64_t)b * a.heads + h) * p.nseg + seg) * p.max_cols + c], v);
  }
}

// ------------------------------------------------------------------------------------
// The same gate for sequences with more key chunks than one register tile set holds
// (NT*32).  Chunks are scored in groups of NT*32; after every group the row keeps the
// K' best (score, chunk) pairs seen so far in LDS, and the next group competes against
// them.  The total order (score descending, chunk index descending) is strict, so the
// running winners after the last group are exactly the global top-K'.  Selection words
// and counts are then assembled in LDS and written out like the small kernel's.
// ------------------------------------------------------------------------------------
constexpr int kBigCap = 32;   // running winners per row (K' = scored chunks kept) of the common variants
constexpr int kBigCapMax = 64;  // ... of the variant for top-k above 33: moba_topk goes up to 64 at any sequence length

// CAP: entries of a row's list of running winners (16, kBigCap or kBigCapMax).  With 16 and groups of 128 chunks the
// kernel needs half the LDS and fewer registers, and two workgroups share a compute unit.  With 64 a row has ONE list
// (two would not fit the LDS): every group then takes the general path, which has read the whole list into registers
// before it writes the winners back; the streaming update of the smaller variants needs the second list for its entrants.
template <typename T, int HD, int NT, int CAP>
__global__ __launch_bounds__(256, CAP < kBigCap ? 2 : 1) void topk_gate_big_kernel(TopkParams p) {
  constexpr bool TWO_LISTS = CAP <= kBigCap;
  constexpr int NLIST = TWO_LISTS ? 2 : 1;
  constexpr int KS = HD / 16;
  constexpr int LD = HD + 16;
  constexpr int GC = NT * 32;        // chunks per group
  constexpr int PL = CAP / 2;    // previous winners held per lane (two lanes per row)
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint16_t *sKm = reinterpret_cast<uint16_t *>(smem);
  uint32_t *sSel = reinterpret_cast<uint32_t *>(smem);  // [word columns of a pass][128], reuses the chunk-mean tile after the last group
  float *sVal = reinterpret_cast<float *>(smem + (size_t)GC * LD * 2);   // [NLIST][128][CAP]
  int *sIdx = reinterpret_cast<int *>(sVal + NLIST * kGateRows * CAP);   // [NLIST][128][CAP]
  int *sCnt = sIdx + NLIST * kGateRows * CAP;                            // [2][128]
  int *sHist = sCnt + 2 * kGateRows;                                     // [32 chunks per word column the tile holds as selection words]
  int *sTrash = sHist + (size_t)GC * LD * 2 / (kGateRows * 4) * 32;      // [256]: takes the stores of lanes that have nothing to store

  const fmoba_fused_topk_args &a = p.a;
  const int mb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int q0 = a.cu_seqlens_q[b];
  const int Lq = a.cu_seqlens_q[b + 1] - q0;
  const int m0 = mb * kGateRows;
  if (m0 >= Lq) return;
  const int Lk = a.cu_seqlens_k[b + 1] - a.cu_seqlens_k[b];
  const int km0 = a.cu_seqlens_km[b];
  const int Cb = min(a.cu_seqlens_km[b + 1] - km0, p.max_cols);
  const int off = Lk - Lq;
  const int B = a.chunk;
  const int D = a.head_dim;
  const int hk = h / (a.heads / a.heads_k);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
  const int rs = wave * 32 + (lane & 31);  // row slot inside the block

  int nsc;  // chunks [0, nsc) can be candidates of some row of this block
  if (a.is_causal) {
    const int rmax = min(m0 + kGateRows - 1, Lq - 1) + off;
    nsc = rmax < 0 ? 0 : min(Cb, rmax / B);
  } else {
    nsc = Cb;
  }
  const int ngroups = (nsc + GC - 1) / GC;

  const int r = m0 + rs;
  const bool valid = r < Lq;
  Pack8 qf[KS];
  {
    const uint16_t *qp = reinterpret_cast<const uint16_t *>(a.q) + (int64_t)(q0 + (valid ? r : 0)) * a.q_row_stride + (int64_t)h * a.q_head_stride;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int e = (hh * KS + ks) * 8;
      qf[ks] = (valid && e < D) ? ld_global16(qp + e) : zero_pack8();
    }
  }
  const int rp = r + off;
  int nc;  // candidate chunks of this row: chunks strictly before its own chunk
  if (a.is_causal)
    nc = (valid && rp >= 0) ? min(rp / B, Cb) : 0;
  else
    nc = valid ? Cb : 0;
  const int kp = a.is_causal ? a.topk - 1 : a.topk;

  if (tid < 2 * kGateRows) sCnt[tid] = 0;
  int cur = 0;
  const uint16_t *kmp = reinterpret_cast<const uint16_t *>(a.km) + (int64_t)hk * a.km_head_stride;
#pragma nounroll
  for (int g = 0; g < ngroups; ++g) {
    const int c0 = g * GC;
    const int gsc = min(GC, nsc - c0);
    const int n_tiles = (gsc + 31) >> 5;
    __syncthreads();  // the previous group's tile and lists are no longer read
    {
      const int vecs = HD / 8;
      for (int v = tid; v < n_tiles * 32 * vecs; v += 256) {
        const int c = v / vecs, e = (v - c * vecs) * 8;
        Pack8 x = zero_pack8();
        if (c < gsc && e < D) x = ld_global16(kmp + (int64_t)(km0 + c0 + c) * a.km_row_stride + e);
        *reinterpret_cast<Pack8 *>(sKm + c * LD + e) = x;
      }
    }
    const int nxt = cur ^ 1;
    if (hh == 0) sCnt[nxt * kGateRows + rs] = 0;
    __syncthreads();

    // this group's scores and the winners so far
    float sc[NT][16];
    float pv[PL];
    int pi[PL];
    const int m_prev = sCnt[cur * kGateRows + rs];
    float vmin = INFINITY, vmax = -INFINITY;
#pragma unroll
    for (int j = 0; j < PL; ++j) {
      const int e = 2 * j + hh;  // the two lanes of a row hold alternate entries of its list
      const bool ok = e < m_prev;
      pv[j] = ok ? sVal[((TWO_LISTS ? cur : 0) * kGateRows + rs) * CAP + e] : -INFINITY;
      pi[j] = ok ? sIdx[((TWO_LISTS ? cur : 0) * kGateRows + rs) * CAP + e] : -1;
      vmin = fminf(vmin, ok ? pv[j] : INFINITY);
      vmax = fmaxf(vmax, pv[j]);
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (t < n_tiles) {
        f32x16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const Pack8 af = *reinterpret_cast<const Pack8 *>(sKm + (t * 32 + (lane & 31)) * LD + (hh * KS + ks) * 8);
          acc = mfma32<T>(af, qf[ks], acc);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int c = c0 + t * 32 + acc_row(i, hh);
          const bool cand = c < nc;
          const float x = acc[i];
          sc[t][i] = cand ? x : -INFINITY;
          vmin = fminf(vmin, cand ? x : INFINITY);
          vmax = fmaxf(vmax, sc[t][i]);
        }
      } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[t][i] = -INFINITY;
      }
    }
    // ---- later groups: streaming update ---------------------------------------------------------
    // A row that still has candidates in this group had at least GC of them in the first one, so it already holds
    // kp winners.  Only the new scores that reach its weakest winner can enter (a new chunk has a higher index than
    // every earlier one, so an equal score wins the tie): they are put into the row's other list, then each takes
    // the place of the weakest winner if it beats it.  That is the top kp of the union, in the same total order
    // (score descending, chunk descending) as the bisection below, which stays for the first group and for rows
    // with more entrants than a list holds.
    if (TWO_LISTS && g > 0 && __all(m_prev == kp || nc <= c0)) {
      float pmin = INFINITY;
#pragma unroll
      for (int j = 0; j < PL; ++j) pmin = fminf(pmin, pi[j] >= 0 ? pv[j] : INFINITY);
      pmin = min_xor32_f(pmin);
      int ne = 0;
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (t < n_tiles) {
#pragma unroll
          for (int i = 0; i < 16; ++i) ne += (sc[t][i] >= pmin) ? 1 : 0;
        }
      int slot = 0;
      if (ne > 0) slot = atomicAdd(&sCnt[nxt * kGateRows + rs], ne);
      wave_lds_fence();
      const int ne_row = sCnt[nxt * kGateRows + rs];
      wave_lds_fence();
      if (__all(ne_row <= CAP)) {
        float *ev = sVal + (size_t)(nxt * kGateRows + rs) * CAP;
        int *ei = sIdx + (size_t)(nxt * kGateRows + rs) * CAP;
        // (no branches: a lane without an entrant at this position stores to its trash word)
#pragma unroll
        for (int t = 0; t < NT; ++t)
          if (t < n_tiles) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const bool w = sc[t][i] >= pmin;
              *(w ? ev + slot : reinterpret_cast<float *>(sTrash + tid)) = sc[t][i];
              *(w ? ei + slot : sTrash + tid) = c0 + t * 32 + acc_row(i, hh);
              slot += w ? 1 : 0;
            }
          }
        wave_lds_fence();
        // (with at most 16 winners a lane holds at most 8 of them: the short variant of the loop)
        auto stream = [&](auto plc) {
          constexpr int PLX = decltype(plc)::value;
#pragma nounroll
          for (int e = 0; __any(e < ne_row); ++e) {
            const bool has = e < ne_row;
            const float x = has ? ev[e] : -INFINITY;
            const int c = has ? ei[e] : -1;
            // the weakest winner of this lane's half of the list, then of the row
            float vw = INFINITY;
            int cw = 0x7fffffff, jw = -1;
#pragma unroll
            for (int j = 0; j < PLX; ++j) {
              const bool better = (pi[j] >= 0) & ((pv[j] < vw) | ((pv[j] == vw) & (pi[j] < cw)));
              vw = better ? pv[j] : vw;
              cw = better ? pi[j] : cw;
              jw = better ? j : jw;
            }
            const float vo = shfl_xor32_f(vw);
            const int co = shfl_xor32_i(cw);
            const bool mine = (jw >= 0) & ((vw < vo) | ((vw == vo) & (cw < co)));
            const float vr = mine ? vw : vo;
            const int cr = mine ? cw : co;
            const bool beats = has & ((x > vr) | ((x == vr) & (c > cr)));
            const int jr = (beats & mine) ? jw : -1;
#pragma unroll
            for (int j = 0; j < PLX; ++j) {
              pv[j] = j == jr ? x : pv[j];
              pi[j] = j == jr ? c : pi[j];
            }
          }
        };
        if (kp <= PL)
          stream(std::integral_constant<int, PL / 2>{});
        else
          stream(std::integral_constant<int, PL>{});
        // the updated winners go back to where they came from; the list keeps its length
#pragma unroll
        for (int j = 0; j < PL; ++j) {
          const int e = 2 * j + hh;  // the two lanes of a row hold alternate entries of its list
          if (e < m_prev) {
            sVal[(cur * kGateRows + rs) * CAP + e] = pv[j];
            sIdx[(cur * kGateRows + rs) * CAP + e] = pi[j];
          }
        }
        continue;
      }
      // more entrants than a list holds: the general path below recounts from scratch
      if (hh == 0) sCnt[nxt * kGateRows + rs] = 0;
      wave_lds_fence();
    }
    vmin = min_xor32_f(vmin);
    vmax = max_xor32_f(vmax);
    const int ntot = m_prev + max(0, min(nc - c0, GC));  // candidates that compete in this group
    const bool need = (ntot > kp) && (kp > 0);

    auto count_gt = [&](float probe) {
      int cnt = 0;
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (t < n_tiles) {
#pragma unroll
          for (int i = 0; i < 16; i += 4) cnt = count4_gt(cnt, sc[t][i], sc[t][i + 1], sc[t][i + 2], sc[t][i + 3], probe);
        }
      static_assert(PL % 4 == 0, "the winners are counted four at a time");
#pragma unroll
      for (int j = 0; j < PL; j += 4) cnt = count4_gt(cnt, pv[j], pv[j + 1], pv[j + 2], pv[j + 3], probe);
      return sum_xor32_i(cnt);
    };
    float tau = -INFINITY, tau_eq = INFINITY;
    int n_eq = 0;
    uint32_t iota = 0u;
    {
      uint32_t lo_k = float_order_key(vmin) - 1u;
      uint32_t hi_k = float_order_key(vmax);
      int c_hi = 0;
      bool open = need;
#pragma nounroll
      for (int iter = 0;; ++iter) {
        if (open && hi_k - lo_k <= 1u) {
          tau = order_key_float(hi_k);
          if (tau != -INFINITY) {
            tau_eq = tau;
            n_eq = kp - c_hi;
          }
          open = false;
        }
        if (!__any(open)) break;
        uint32_t pk = lo_k + ((hi_k - lo_k) >> 1);
        if (iter < 12) {
          const float mf = 0.5f * order_key_float(lo_k + 1u) + 0.5f * order_key_float(hi_k);
          const uint32_t mk = float_order_key(mf);
          if (mk > lo_k && mk < hi_k) pk = mk;
        }
        const float probe = order_key_float(pk);
        const int cnt = count_gt(probe);
        if (open) {
          if (cnt == kp) {
            tau = probe;
            open = false;
          } else if (cnt > kp) {
            lo_k = pk;
          } else {
            hi_k = pk;
            c_hi = cnt;
          }
        }
      }
      const bool tie = n_eq > 0;
      if (__any(tie)) {
        auto count_eq_ge = [&](uint32_t trial) {
          int cnt = 0;
#pragma unroll
          for (int t = 0; t < NT; ++t)
            if (t < n_tiles) {
#pragma unroll
              for (int i = 0; i < 16; ++i) {
                const uint32_t c = (uint32_t)(c0 + t * 32 + acc_row(i, hh));
                cnt += ((sc[t][i] == tau_eq) & (c >= trial)) ? 1 : 0;
              }
            }
#pragma unroll
          for (int j = 0; j < PL; ++j) cnt += ((pv[j] == tau_eq) & ((uint32_t)pi[j] >= trial) & (pi[j] >= 0)) ? 1 : 0;
          return sum_xor32_i(cnt);
        };
        const int ceq = count_eq_ge(0u);
        const bool split = tie && ceq > n_eq;
        if (__any(split)) {
          uint32_t i_acc = 0u;
#pragma nounroll
          for (int bit = 23; bit >= 0; --bit) {
            const uint32_t trial = i_acc | (1u << bit);
            const int cnt = count_eq_ge(trial);
            if (cnt >= n_eq) i_acc = trial;
          }
          if (split) iota = i_acc;
        }
      }
    }

    // winners of this round -> the other list: count per lane, reserve slots once, then store
    int nwin = 0;
    if (kp > 0) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (t < n_tiles) {
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const uint32_t c = (uint32_t)(c0 + t * 32 + acc_row(i, hh));
            const float x = sc[t][i];
            nwin += ((x > tau) | ((x == tau_eq) & (c >= iota))) ? 1 : 0;
          }
        }
#pragma unroll
      for (int j = 0; j < PL; ++j) nwin += ((pi[j] >= 0) & ((pv[j] > tau) | ((pv[j] == tau_eq) & ((uint32_t)pi[j] >= iota)))) ? 1 : 0;
    }
    int slot = 0;
    if (nwin > 0) slot = atomicAdd(&sCnt[nxt * kGateRows + rs], nwin);
    float *ov = sVal + (size_t)((TWO_LISTS ? nxt : 0) * kGateRows + rs) * CAP;
    int *oi = sIdx + (size_t)((TWO_LISTS ? nxt : 0) * kGateRows + rs) * CAP;
    if (!TWO_LISTS) wave_lds_fence();  // (one list: both lanes of the row have read it into registers)
    if (__any(nwin > 0)) {  // (no branches inside: a lane without a winner at a position stores to its trash word)
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (t < n_tiles) {
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const uint32_t c = (uint32_t)(c0 + t * 32 + acc_row(i, hh));
            const float x = sc[t][i];
            const bool w = (kp > 0) & ((x > tau) | ((x == tau_eq) & (c >= iota))) & (slot < CAP);
            *(w ? ov + slot : reinterpret_cast<float *>(sTrash + tid)) = x;
            *(w ? oi + slot : sTrash + tid) = (int)c;
            slot += w ? 1 : 0;
          }
        }
#pragma unroll
      for (int j = 0; j < PL; ++j) {
        const bool w = (kp > 0) & (pi[j] >= 0) & ((pv[j] > tau) | ((pv[j] == tau_eq) & ((uint32_t)pi[j] >= iota))) & (slot < CAP);
        *(w ? ov + slot : reinterpret_cast<float *>(sTrash + tid)) = pv[j];
        *(w ? oi + slot : sTrash + tid) = pi[j];
        slot += w ? 1 : 0;
      }
    }
    cur = nxt;
  }
  __syncthreads();

  // selection words and per-chunk counts of the block, assembled in LDS and written out in passes of WP word columns
  // (what the chunk-mean tile holds), so that a sequence may have any number of chunks
  const int WP = min(p.W, (int)((size_t)GC * LD * 2 / (kGateRows * 4)));
  const int m_fin = valid ? min(sCnt[cur * kGateRows + rs], CAP) : 0;
  const int seg = m0 / p.seg_rows;
  for (int w0 = 0; w0 < p.W; w0 += WP) {
    const int wn = min(WP, p.W - w0);
    __syncthreads();  // the pass before has been written out
    for (int v = tid; v < wn * kGateRows; v += 256) sSel[v] = 0u;
    for (int c = tid; c < wn * 32; c += 256) sHist[c] = 0;
    __syncthreads();
    if (valid) {
#pragma unroll
      for (int j = 0; j < PL; ++j) {
        const int e = 2 * j + hh;  // the two lanes of a row hold alternate entries of its list
        if (e < m_fin) {
          const int c = sIdx[((TWO_LISTS ? cur : 0) * kGateRows + rs) * CAP + e];
          const int cw = (c >> 5) - w0;
          if ((uint32_t)cw < (uint32_t)wn) {
            atomicOr(&sSel[cw * kGateRows + rs], 1u << (c & 31));
            atomicAdd(&sHist[c - 32 * w0], 1);
          }
        }
      }
      if (hh == 0 && a.is_causal && rp >= 0) {
        const int c = rp / B;  // the own chunk is always selected
        const int cw = (c >> 5) - w0;
        if (c < p.max_cols && (uint32_t)cw < (uint32_t)wn) {
          atomicOr(&sSel[cw * kGateRows + rs], 1u << (c & 31));
          atomicAdd(&sHist[c - 32 * w0], 1);
        }
      }
    }
    __syncthreads();
    for (int v = tid; v < wn * kGateRows; v += 256) {
      const int t = v / kGateRows, slot_r = v - t * kGateRows;
      if (m0 + slot_r < Lq) p.sel[((int64_t)h * p.W + w0 + t) * a.total_q + q0 + m0 + slot_r] = sSel[v];
    }
    for (int c = tid; c < wn * 32; c += 256) {
      const int v = sHist[c];
      if (v) atomicAdd(&p.segcnt[(((int64_t)b * a.heads + h) * p.nseg + seg) * p.max_cols + 32 * w0 + c], v);
    }
  }
}

// ------------------------------------------------------------------------------------
// The grouped gate for at most 16 running winners per row (top-k up to 17 causal, 16 otherwise): the common case of
// long sequences.  Same total order and result as topk_gate_big_kernel; what differs is where things live:
//  * a row's winners stay in REGISTERS across the groups: eight doubles per lane of the row's lane pair, each lane's
//    share sorted, so that the weakest is at hand and a new winner goes in with one pass of minimum / maximum;
//  * the chunk means of the next group are fetched into registers while the current group is worked on;
//  * the scores of a later group that reach the row's weakest winner ("entrants") are compacted into one list per
//    row in LDS -- the lane with chunks 0..3 of every eight fills it from the bottom, its partner from the top, so
//    that no counter is shared; every score is stored at the lane's next slot and the slot advances only for an
//    entrant, so there are no branches and no address selects -- and each then replaces the weakest winner if it
//    beats it.  More than 16 entrants in some row of a wave, the first group, and rows whose list is not full yet
//    take the bisection over this group's scores and the winners.
// ------------------------------------------------------------------------------------
// A winner is ONE double: order key of its score * 65536 + chunk (exact: below 2^48), so that the order "score
// descending, chunk descending" is the order of the doubles and minimum / maximum are single instructions.
constexpr double kChunkSpan = 65536.0;  // chunk indices stay below it (checked on the host before the launch)
constexpr double kSlotFiller = INFINITY;  // unused slot of a complete list: above every winner, never the weakest
constexpr double kSlotEmpty = -1.0;       // unused slot of a list that is still filling: below every winner

__device__ __forceinline__ double winner_word(float score, int chunk) {
  // (x + 0 turns -0 into +0: the order keys must agree with the float compares of the bisection)
  return fma((double)float_order_key(score + 0.f), kChunkSpan, (double)chunk);
}
__device__ __forceinline__ bool winner_real(double w) { return w >= 0.0 && w < (double)INFINITY; }
__device__ __forceinline__ uint32_t winner_key(double w) { return (uint32_t)(w * (1.0 / kChunkSpan)); }  // (truncates)
__device__ __forceinline__ int winner_chunk(double w) { return (int)fma(-(double)winner_key(w), kChunkSpan, w); }
// minimum and maximum of two winners as one instruction each (fmin / fmax first bring every operand that comes round a
// loop into canonical form, one more instruction per operand and turn; winners are never NaN)
__device__ __forceinline__ double min_winner(double a, double b) {
#if defined(__HIP_DEVICE_COMPILE__)
  double d;
  asm("v_min_f64 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
  return d;
#else
  return a < b ? a : b;
#endif
}
__device__ __forceinline__ double max_winner(double a, double b) {
#if defined(__HIP_DEVICE_COMPILE__)
  double d;
  asm("v_max_f64 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
  return d;
#else
  return a > b ? a : b;
#endif
}
// score and chunk of a list entry (the chunk lies TO_CHUNK bytes after the score), requested here and awaited there: the
// compiler waits for an LDS read of its own where it issues it when the address comes round a loop.  Nothing else of
// the wave may be on its way from LDS between the two calls, and the values may only be used after the second.
template <int TO_CHUNK>
__device__ __forceinline__ void entrant_request(uint32_t lds_addr, float &score, int &chunk) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("ds_read_b32 %0, %2\n\tds_read_b32 %1, %2 offset:%3" : "=&v"(score), "=&v"(chunk) : "v"(lds_addr), "n"(TO_CHUNK));
#else
  score = 0.f;
  chunk = (int)lds_addr;
#endif
}
__device__ __forceinline__ void entrant_await(float &score, int &chunk) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(score), "+v"(chunk));
#endif
}
__device__ __forceinline__ double shfl_xor32_d(double v) {
  const uint64_t u = (uint64_t)__double_as_longlong(v);
  const uint64_t o = ((uint64_t)(uint32_t)shfl_xor32_i((int)(u >> 32)) << 32) | (uint32_t)shfl_xor32_i((int)(uint32_t)u);
  return __longlong_as_double((long long)o);
}

// a * b + c on 24-bit operands, one instruction (the compiler picks a 64-bit multiply-add for this address pattern)
__device__ __forceinline__ uint32_t mad24_u32(int a, int b, uint32_t c) {
#if defined(__HIP_DEVICE_COMPILE__)
  uint32_t d;
  asm("v_mad_i32_i24 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
  return d;
#else
  return (uint32_t)(a * b) + c;
#endif
}
constexpr int kStreamListMargin = 64;  // words on either side of a wave's lists
constexpr int kStreamListStride = 19;  // words from one row's list (18 slots) to the next
constexpr int kStreamListWords = 4 * (32 * kStreamListStride + 2 * kStreamListMargin) + 256;
template <typename T, int HD, int NT>
__global__ __launch_bounds__(256, NT <= 2 ? 3 : 2) void topk_gate_stream_kernel(TopkParams p) {
  constexpr int CAP = 16, PL = 8;
  constexpr int KS = HD / 16;
  constexpr int GC = NT * 32;             // chunks per group
  constexpr int VPR = HD / 8;             // 16-byte pieces of a row of chunk means
  constexpr int RPI = 64 / VPR;           // tile rows one load instruction brings (64 lanes x 16 bytes)
  constexpr int NV = GC / RPI / 4;        // load instructions per wave and tile
  static_assert(NV >= 1 && NV * RPI * 4 == GC, "the four waves share a tile evenly");
  constexpr int RB = HD * 2;              // bytes of a tile row: exactly HD elements, swizzled instead of padded
  constexpr int LS = CAP + 2;                 // slots of a row's list: 16 entries and the two lanes' next slots
  // words of an entrant array: per wave the lists of its 32 rows between two margins, then a trash word per thread.
  // A lane with more entrants than its row's list holds writes on into the lists of the wave's other rows and, from
  // the first and the last row, into a margin (at most 63 - 17 slots beyond the list): such a wave takes the bisection
  // and rebuilds its lists, and no other wave's list is touched, so the slot needs no clamp.
  constexpr int EW = kStreamListWords;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint32_t *sSel = reinterpret_cast<uint32_t *>(smem);  // [word columns of a pass][128], reuses the tile and the lists after the last group
  float *sEv = reinterpret_cast<float *>(smem + (size_t)GC * RB);  // [EW] scores of the entrants
  constexpr size_t head = (size_t)GC * RB + (size_t)2 * EW * 4;
  int *sHist = reinterpret_cast<int *>(smem + head);                   // [32 chunks per word column of a pass]

  const fmoba_fused_topk_args &a = p.a;
  const int mb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int q0 = a.cu_seqlens_q[b];
  const int Lq = a.cu_seqlens_q[b + 1] - q0;
  const int m0 = mb * kGateRows;
  if (m0 >= Lq) return;
  const int Lk = a.cu_seqlens_k[b + 1] - a.cu_seqlens_k[b];
  const int km0 = a.cu_seqlens_km[b];
  const int Cb = min(a.cu_seqlens_km[b + 1] - km0, p.max_cols);
  const int off = Lk - Lq;
  const int B = a.chunk;
  const int D = a.head_dim;
  const int hk = h / (a.heads / a.heads_k);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
  const int rs = wave * 32 + (lane & 31);  // row slot inside the block

  int nsc;  // chunks [0, nsc) can be candidates of some row of this block
  if (a.is_causal) {
    const int rmax = min(m0 + kGateRows - 1, Lq - 1) + off;
    nsc = rmax < 0 ? 0 : min(Cb, rmax / B);
  } else {
    nsc = Cb;
  }
  const int ngroups = (nsc + GC - 1) / GC;

  const int r = m0 + rs;
  const bool valid = r < Lq;
  Pack8 qf[KS];
  {
    const uint16_t *qp = reinterpret_cast<const uint16_t *>(a.q) + (int64_t)(q0 + (valid ? r : 0)) * a.q_row_stride + (int64_t)h * a.q_head_stride;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int e = (hh * KS + ks) * 8;
      qf[ks] = (valid && e < D) ? ld_global16(qp + e) : zero_pack8();
    }
  }
  const int rp = r + off;
  int nc;  // candidate chunks of this row: chunks strictly before its own chunk
  if (a.is_causal)
    nc = (valid && rp >= 0) ? min(rp / B, Cb) : 0;
  else
    nc = valid ? Cb : 0;
  const int kp = a.is_causal ? a.topk - 1 : a.topk;

  const uint16_t *kmp = reinterpret_cast<const uint16_t *>(a.km) + (int64_t)hk * a.km_head_stride;
  // The chunk means of a group go from global memory straight into the LDS tile (global_load_lds: no registers hold
  // them on the way), every wave a quarter of the rows, issued as soon as the scores of the group before have been
  // formed and awaited at the top of the next group: the rest of a group's work runs under them.  Piece c of tile row
  // r lies at piece c ^ tile_swz<HD>(r).  Rows past the last chunk that can be a candidate and features past head_dim
  // are fetched from a row / piece that exists: such scores are masked, such features meet zeros of q.
  const uint32_t ldsTile = (uint32_t)(uintptr_t)smem;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  auto tile_issue = [&](int g) {
    const int c0 = g * GC, gsc = min(GC, nsc - c0);
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int c = (wave_u * NV + v) * RPI + lane / VPR, pc = lane % VPR;
      const int e = min((pc ^ tile_swz<HD>(c)) * 8, D - 8);
      global_to_lds16(kmp + (int64_t)(km0 + c0 + min(c, gsc - 1)) * a.km_row_stride + e, ldsTile + (uint32_t)((wave_u * NV + v) * 1024));
    }
  };
  // this lane's operand row of a 32-chunk tile: row lane % 32, pieces hh * KS ..
  const uint32_t a_row = ldsTile + (uint32_t)((lane & 31) * RB);
  const int a_swz = tile_swz<HD>(lane & 31);
  double win[PL];  // this lane's share of the row's winners, ascending (win[0] is the weakest the lane holds)
#pragma unroll
  for (int j = 0; j < PL; ++j) win[j] = kSlotEmpty;
  int m_prev = 0;    // winners the row holds
  // (lists kStreamListStride = 19 words apart: with 18, an even number, rows l and l + 16 share a bank and every
  // store of the 32 lanes of a half wave takes two turns)
  float *const my_list_v = sEv + wave * (32 * kStreamListStride + 2 * kStreamListMargin) + kStreamListMargin + (lane & 31) * kStreamListStride;
  float *const my_trash = sEv + 4 * (32 * kStreamListStride + 2 * kStreamListMargin) + tid;
  constexpr int kToIdx = EW;  // from a score of the entrant arrays to its chunk, in words

  if (ngroups > 0) tile_issue(0);
#pragma nounroll
  for (int g = 0; g < ngroups; ++g) {
    const int c0 = g * GC;
    const int gsc = min(GC, nsc - c0);
    const int n_tiles = (gsc + 31) >> 5;
    wait_all_loads();
    __syncthreads();  // this group's tile is in LDS

    // this group's scores; chunks that are no candidates of the row (its own chunk and later ones) count as -inf
    float sc[NT][16];
    const bool all_cand = __all(nc >= c0 + GC);
    {
      // The tiles of the group side by side, and the operands of contraction step ks + 1 on their way from LDS while
      // the products of step ks run: one tile after the other, every read awaited by its product, a wave spent a
      // group's worth of LDS latencies in a single chain.  (A tile past the group's last chunk holds copies of
      // chunks that exist, see tile_issue; its scores are masked like those of every chunk that is no candidate.)
      f32x16 acc[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;
      auto operand = [&](int t, int ks) { return lds_read16(a_row + (uint32_t)(t * 32 * RB) + (uint32_t)(((hh * KS + ks) ^ a_swz) * 16)); };
      Pack8 af[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t) af[t] = operand(t, 0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        Pack8 nx[NT];
        if (ks + 1 < KS) {
#pragma unroll
          for (int t = 0; t < NT; ++t) nx[t] = operand(t, ks + 1);
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = mfma32<T>(af[t], qf[ks], acc[t]);
        if (ks + 1 < KS) {
#pragma unroll
          for (int t = 0; t < NT; ++t) af[t] = nx[t];
        }
      }
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        if (all_cand) {
#pragma unroll
          for (int i = 0; i < 16; ++i) sc[t][i] = acc[t][i];
        } else {
#pragma unroll
          for (int i = 0; i < 16; ++i) sc[t][i] = (c0 + t * 32 + acc_row(i, hh) < nc) ? acc[t][i] : -INFINITY;
        }
      }
    }
    __syncthreads();  // everyone has read the tile: the next group's chunk means may land in it
    if (g + 1 < ngroups) tile_issue(g + 1);

    // ---- later groups: streaming update ---------------------------------------------------------
    // A row that still has candidates in this group had at least GC of them in the first one, so it already holds
    // kp winners.  Only the new scores that reach its weakest winner can enter (a new chunk has a higher index than
    // every earlier one, so an equal score wins the tie).
    // In the groups right after the first a row expects about kp ln((g + 1) / g) entrants (every position of a random
    // stream enters with probability kp / position), which for the second group of a row with sixteen winners is more
    // than a list takes for some row of nearly every wave: such groups are streamed tile by tile.
    bool streamed = false;
    if (g > 0 && __all(m_prev == kp || nc <= c0)) {
      const int part_tiles = (kp > 10 * g) ? 1 : NT;
      streamed = true;
#pragma nounroll
      for (int t0 = 0; t0 < n_tiles; t0 += part_tiles) {
        const int t1 = t0 + part_tiles;
        const double weakest = fmin(win[0], shfl_xor32_d(win[0]));
        // (a row without winners, or one whose list is not full because it has no candidates left, admits nothing)
        const float pmin = winner_real(weakest) ? order_key_float(winner_key(weakest)) : INFINITY;
        // slot c of the lane with chunks 0..3 is entry c, of its partner entry LS - 1 - c; beyond the list both stay
        // on the row's last slot
        const uint32_t slot0 = (uint32_t)(uintptr_t)(my_list_v + (hh ? LS - 1 : 0));
        const int slot_step = hh ? -4 : 4;  // bytes
        int cbase = c0 + 4 * hh;
        asm volatile("" : "+v"(cbase));  // (one register: the compiler would add its scalar and vector parts per position)
        int cnt = 0;
#pragma unroll
        for (int t = 0; t < NT; ++t)
          if (t >= t0 && t < t1 && t < n_tiles) {
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
              const Flags4 ge = flags4_ge(sc[t][4 * i4], sc[t][4 * i4 + 1], sc[t][4 * i4 + 2], sc[t][4 * i4 + 3], pmin);
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                const int i = 4 * i4 + j;
                const uint32_t d = mad24_u32(cnt, slot_step, slot0);
                lds_write_vec<float>(d, sc[t][i]);
                lds_write_vec<int>(d + (uint32_t)kToIdx * 4u, cbase + t * 32 + 8 * (i >> 2) + (i & 3));
                cnt = count_flag(cnt, ge.m[j]);
              }
            }
          }
        const int cnt_o = shfl_xor32_i(cnt);
        const int ne_row = cnt + cnt_o;
        if (!__all(ne_row <= CAP)) {
          // the search below takes over; tiles whose entrants have gone into the winners leave the competition
#pragma unroll
          for (int t = 0; t < NT; ++t)
            if (t < t0) {
#pragma unroll
              for (int i = 0; i < 16; ++i) sc[t][i] = -INFINITY;
            }
          streamed = false;
          break;
        }
        wave_lds_fence();
        const int ne_lo = hh ? cnt_o : cnt;  // entrants that came from the bottom of the list
        auto stream = [&](auto plc) {
          constexpr int PLX = decltype(plc)::value;
          // (entrant e + 1 is on its way from the list while entrant e goes up the entries)
          auto slot_of = [&](int e) { return e < ne_row ? (e < ne_lo ? e : LS - 1 - (e - ne_lo)) : 0; };
          const uint32_t list_b = (uint32_t)(uintptr_t)my_list_v;
          float xv;
          int xc;
          entrant_request<kToIdx * 4>(list_b + 4u * (uint32_t)slot_of(0), xv, xc);
          entrant_await(xv, xc);
#pragma nounroll
          for (int e = 0; __any(e < ne_row); ++e) {
            const bool has = e < ne_row;
            const double x = winner_word(xv, xc);
            float xv_next;
            int xc_next;
            entrant_request<kToIdx * 4>(list_b + 4u * (uint32_t)slot_of(e + 1), xv_next, xc_next);
            // the row's weakest winner is the lower of the two lanes' first entries; the lane that holds it drops it
            // and passes the entrant up its sorted entries (a lane that keeps its entries passes its own first entry)
            const double vo = shfl_xor32_d(win[0]);
            const bool rep = has & (win[0] <= vo) & (x > win[0]);
            const double xs = rep ? x : win[0];
            double nw[PLX];
            nw[0] = min_winner(xs, win[1]);
#pragma unroll
            for (int j = 1; j + 1 < PLX; ++j) nw[j] = min_winner(max_winner(win[j], xs), win[j + 1]);
            nw[PLX - 1] = max_winner(win[PLX - 1], xs);
#pragma unroll
            for (int j = 0; j < PLX; ++j) win[j] = nw[j];
            entrant_await(xv_next, xc_next);
            xv = xv_next;
            xc = xc_next;
          }
        };
        // (a lane holds at most (kp + 1) / 2 winners; the fillers above them never move)
        if (kp <= PL)
          stream(std::integral_constant<int, PL / 2>{});
        else
          stream(std::integral_constant<int, PL>{});
        wave_lds_fence();  // (the list takes the next entrants)
      }
    }
    if (streamed) continue;

    // ---- first group, lists that are filling, too many entrants: bisection over scores and winners ------------
    float pv[PL];
    int pi[PL];
    float vmin = INFINITY, vmax = -INFINITY;
#pragma unroll
    for (int j = 0; j < PL; ++j) {
      const bool ok = winner_real(win[j]);
      pv[j] = ok ? order_key_float(winner_key(win[j])) : -INFINITY;
      pi[j] = ok ? winner_chunk(win[j]) : -1;
      vmin = fminf(vmin, ok ? pv[j] : INFINITY);
      vmax = fmaxf(vmax, pv[j]);
    }
    // A full list bounds the search from below: its kp winners all reach its weakest one, so the new threshold cannot
    // lie below that score (if nothing enters, the search closes on it and the tie rule keeps the list as it is).
    const float floor_v = (m_prev == kp && kp > 0) ? min_xor32_f(vmin) : -INFINITY;
#pragma unroll
    for (int t = 0; t < NT; ++t)
      if (t < n_tiles) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const bool cand = c0 + t * 32 + acc_row(i, hh) < nc;
          vmin = fminf(vmin, cand ? sc[t][i] : INFINITY);
          vmax = fmaxf(vmax, sc[t][i]);
        }
      }
    vmin = min_xor32_f(vmin);
    vmax = max_xor32_f(vmax);
    const int ntot = m_prev + max(0, min(nc - c0, GC));  // candidates that compete in this group
    const bool need = (ntot > kp) && (kp > 0);

    auto count_gt = [&](float probe) {
      int cnt = 0;
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (t < n_tiles) {
#pragma unroll
          for (int i = 0; i < 16; i += 4) cnt = count4_gt(cnt, sc[t][i], sc[t][i + 1], sc[t][i + 2], sc[t][i + 3], probe);
        }
      static_assert(PL % 4 == 0, "the winners are counted four at a time");
#pragma unroll
      for (int j = 0; j < PL; j += 4) cnt = count4_gt(cnt, pv[j], pv[j + 1], pv[j + 2], pv[j + 3], probe);
      return sum_xor32_i(cnt);
    };
    float tau = -INFINITY, tau_eq = INFINITY;
    int n_eq = 0;
    uint32_t iota = 0u;
    {
      uint32_t lo_k = float_order_key(fmaxf(vmin, floor_v)) - 1u;
      uint32_t hi_k = float_order_key(vmax);
      int c_hi = 0;
      bool open = need;
#pragma nounroll
      for (int iter = 0;; ++iter) {
        if (open && hi_k - lo_k <= 1u) {
          tau = order_key_float(hi_k);
          if (tau != -INFINITY) {
            tau_eq = tau;
            n_eq = kp - c_hi;
          }
          open = false;
        }
        if (!__any(open)) break;
        uint32_t pk = lo_k + ((hi_k - lo_k) >> 1);
        if (iter < 12) {
          const float mf = 0.5f * order_key_float(lo_k + 1u) + 0.5f * order_key_float(hi_k);
          const uint32_t mk = float_order_key(mf);
          if (mk > lo_k && mk < hi_k) pk = mk;
        }
        const float probe = order_key_float(pk);
        const int cnt = count_gt(probe);
        if (open) {
          if (cnt == kp) {
            tau = probe;
            open = false;
          } else if (cnt > kp) {
            lo_k = pk;
          } else {
            hi_k = pk;
            c_hi = cnt;
          }
        }
      }
      const bool tie = n_eq > 0;
      if (__any(tie)) {
        auto count_eq_ge = [&](uint32_t trial) {
          int cnt = 0;
#pragma unroll
          for (int t = 0; t < NT; ++t)
            if (t < n_tiles) {
#pragma unroll
              for (int i = 0; i < 16; ++i) {
                const uint32_t c = (uint32_t)(c0 + t * 32 + acc_row(i, hh));
                cnt += ((sc[t][i] == tau_eq) & (c >= trial)) ? 1 : 0;
              }
            }
#pragma unroll
          for (int j = 0; j < PL; ++j) cnt += ((pv[j] == tau_eq) & ((uint32_t)pi[j] >= trial) & (pi[j] >= 0)) ? 1 : 0;
          return sum_xor32_i(cnt);
        };
        const int ceq = count_eq_ge(0u);
        const bool split = tie && ceq > n_eq;
        if (__any(split)) {
          uint32_t i_acc = 0u;
#pragma nounroll
          for (int bit = 23; bit >= 0; --bit) {
            const uint32_t trial = i_acc | (1u << bit);
            const int cnt = count_eq_ge(trial);
            if (cnt >= n_eq) i_acc = trial;
          }
          if (split) iota = i_acc;
        }
      }
    }

    // the winners of this round go through the row's LDS list (densely: the partner lane starts where this one ends)
    // and come back as alternate entries per lane
    int nwin = 0;
    if (kp > 0) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (t < n_tiles) {
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const uint32_t c = (uint32_t)(c0 + t * 32 + acc_row(i, hh));
            const float x = sc[t][i];
            nwin += ((x > tau) | ((x == tau_eq) & (c >= iota))) ? 1 : 0;
          }
        }
#pragma unroll
      for (int j = 0; j < PL; ++j) nwin += ((pi[j] >= 0) & ((pv[j] > tau) | ((pv[j] == tau_eq) & ((uint32_t)pi[j] >= iota)))) ? 1 : 0;
    }
    const int nwin_o = shfl_xor32_i(nwin);
    const int m_new = min(nwin + nwin_o, CAP);
    int slot = hh ? nwin_o : 0;
    if (__any(nwin > 0)) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (t < n_tiles) {
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const uint32_t c = (uint32_t)(c0 + t * 32 + acc_row(i, hh));
            const float x = sc[t][i];
            const bool w = (kp > 0) & ((x > tau) | ((x == tau_eq) & (c >= iota))) & (slot < CAP);
            float *d = w ? my_list_v + slot : my_trash;
            d[0] = x;
            reinterpret_cast<int *>(d)[kToIdx] = (int)c;
            slot += w ? 1 : 0;
          }
        }
#pragma unroll
      for (int j = 0; j < PL; ++j) {
        const bool w = (kp > 0) & (pi[j] >= 0) & ((pv[j] > tau) | ((pv[j] == tau_eq) & ((uint32_t)pi[j] >= iota))) & (slot < CAP);
        float *d = w ? my_list_v + slot : my_trash;
        d[0] = pv[j];
        reinterpret_cast<int *>(d)[kToIdx] = pi[j];
        slot += w ? 1 : 0;
      }
    }
    wave_lds_fence();
#pragma unroll
    for (int j = 0; j < PL; ++j) {
      const int e = 2 * j + hh;
      const bool ok = e < m_new;
      const double x = winner_word(my_list_v[ok ? e : 0], reinterpret_cast<const int *>(my_list_v)[kToIdx + (ok ? e : 0)]);
      win[j] = ok ? x : (m_new == kp ? kSlotFiller : kSlotEmpty);
    }
    wave_lds_fence();  // (the list takes this row's entrants next)
    // each lane's share in ascending order (odd-even transposition: this path runs once or twice per row)
#pragma unroll
    for (int rnd = 0; rnd < PL; ++rnd)
#pragma unroll
      for (int j = rnd & 1; j + 1 < PL; j += 2) {
        const double lo = fmin(win[j], win[j + 1]), hi = fmax(win[j], win[j + 1]);
        win[j] = lo;
        win[j + 1] = hi;
      }
    m_prev = m_new;
  }
  __syncthreads();

  // selection words and per-chunk counts of the block, assembled in LDS and written out in passes of WP word columns
  // (what the tile and the lists hold), so that a sequence may have any number of chunks
  const int WP = min(p.W, (int)(head / (kGateRows * 4)));
  const int seg = m0 / p.seg_rows;
  for (int w0 = 0; w0 < p.W; w0 += WP) {
    const int wn = min(WP, p.W - w0);
    __syncthreads();  // the pass before has been written out
    for (int v = tid; v < wn * kGateRows; v += 256) sSel[v] = 0u;
    for (int c = tid; c < wn * 32; c += 256) sHist[c] = 0;
    __syncthreads();
    if (valid) {
#pragma unroll
      for (int j = 0; j < PL; ++j) {
        if (winner_real(win[j])) {
          const int c = winner_chunk(win[j]);
          const int cw = (c >> 5) - w0;
          if ((uint32_t)cw < (uint32_t)wn) {
            atomicOr(&sSel[cw * kGateRows + rs], 1u << (c & 31));
            atomicAdd(&sHist[c - 32 * w0], 1);
          }
        }
      }
      if (hh == 0 && a.is_causal && rp >= 0) {
        const int c = rp / B;  // the own chunk is always selected
        const int cw = (c >> 5) - w0;
        if (c < p.max_cols && (uint32_t)cw < (uint32_t)wn) {
          atomicOr(&sSel[cw * kGateRows + rs], 1u << (c & 31));
          atomicAdd(&sHist[c - 32 * w0], 1);
        }
      }
    }
    __syncthreads();
    for (int v = tid; v < wn * kGateRows; v += 256) {
      const int t = v / kGateRows, slot_r = v - t * kGateRows;
      if (m0 + slot_r < Lq) p.sel[((int64_t)h * p.W + w0 + t) * a.total_q + q0 + m0 + slot_r] = sSel[v];
    }
    for (int c = tid; c < wn * 32; c += 256) {
      const int v = sHist[c];
      if (v) atomicAdd(&p.segcnt[(((int64_t)b * a.heads + h) * p.nseg + seg) * p.max_cols + 32 * w0 + c], v);
    }
  }
}

// grid (heads, batch), block 256
__global__ __launch_bounds__(256) void csc_scan_kernel(TopkParams p) {
  const fmoba_fused_topk_args &a = p.a;
  const int h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  const int q0 = a.cu_seqlens_q[b];
  const int Lq = a.cu_seqlens_q[b + 1] - q0;
  const int nseg_b = (Lq + p.seg_rows - 1) / p.seg_rows;
  const int64_t bh = (int64_t)b * a.heads + h;
  int32_t *segc = p.segcnt + bh * p.nseg * p.max_cols;
  const int64_t base = ((int64_t)q0 * a.heads + (int64_t)Lq * h) * a.topk;
  __shared__ int sscan[256];
  __shared__ int64_t stotal;
  if (tid == 0) stotal = 0;
  __syncthreads();
  for (int c0 = 0; c0 < p.max_cols; c0 += 256) {
    const int c = c0 + tid;
    int nnz = 0;
    if (c < p.max_cols) {
      // eight counts in flight at a time (a long sequence has over a hundred segments, and a load that waits for
      // the store before it costs a round trip each)
      for (int s0 = 0; s0 < nseg_b; s0 += 8) {
        int v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = s0 + i < nseg_b ? segc[(int64_t)(s0 + i) * p.max_cols + c] : 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (s0 + i < nseg_b) segc[(int64_t)(s0 + i) * p.max_cols + c] = nnz;
          nnz += v[i];
        }
      }
    }
    sscan[tid] = nnz;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {
      const int v = (tid >= d) ? sscan[tid - d] : 0;
      __syncthreads();
      sscan[tid] += v;
      __syncthreads();
    }
    const int64_t run = stotal;
    if (c < p.max_cols) {
      a.col_nnz[bh * p.max_cols + c] = nnz;
      a.col_offsets[bh * p.max_cols + c] = base + run + (int64_t)(sscan[tid] - nnz);
    }
    __syncthreads();
    if (tid == 255) stotal = run + sscan[255];
    __syncthreads();
  }
  // slots of this (sequence, head) region that no list uses stay 0
  const int64_t start = base + stotal, end = base + (int64_t)Lq * a.topk;
  for (int64_t i = start + tid; i < end; i += 256) a.flat_indices[i] = 0;
}

// x with the value of lane `lane` (the same in every lane) replaced by v (the same in every lane)
template <int LANE>
__device__ __forceinline__ uint32_t write_lane(uint32_t x, uint32_t v) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm("v_writelane_b32 %0, %1, %2" : "+v"(x) : "s"(v), "n"(LANE));
#else
  (void)v;
#endif
  return x;
}
// base[byte_offset] = value in the lanes of `lanes`, all others do nothing (base: the same in every lane)
__device__ __forceinline__ void store_i32_in_lanes(int32_t *base, uint32_t byte_offset, int value, unsigned long long lanes) {
#if defined(__HIP_DEVICE_COMPILE__)
  unsigned long long saved;
  asm volatile("s_mov_b64 %0, exec\n\t"
               "s_mov_b64 exec, %1\n\t"
               "global_store_dword %2, %3, %4\n\t"
               "s_mov_b64 exec, %0"
               : "=&s"(saved)
               : "s"(lanes), "v"(byte_offset), "v"(value), "s"(base)
               : "memory");
#else
  (void)base, (void)byte_offset, (void)value, (void)lanes;
#endif
}

// grid (nseg * W, heads, batch), block 64: one wave walks the rows of one segment of one 32-chunk word column
__global__ __launch_bounds__(64) void csc_fill_kernel(TopkParams p) {
  const fmoba_fused_topk_args &a = p.a;
  // consecutive workgroups: consecutive segments of one word column, i.e. consecutive memory.  (With the word column
  // as the fast index the waves that run at the same time read addresses a whole word column apart -- total_q words,
  // a power of two more often than not -- and meet in the same memory channel.)
  const int wc = blockIdx.x / p.nseg, seg = blockIdx.x - wc * p.nseg;
  const int h = blockIdx.y, b = blockIdx.z, lane = threadIdx.x;
  const int q0 = a.cu_seqlens_q[b];
  const int Lq = a.cu_seqlens_q[b + 1] - q0;
  const int r0 = seg * p.seg_rows;
  if (r0 >= Lq) return;
  const int r1 = min(Lq, r0 + p.seg_rows);
  // with the causal rule a row selects no chunk beyond its own: the rows before the word column's first chunk hold zeros
  int rb0 = r0;
  if (a.is_causal) {
    const int64_t off = (int64_t)(a.cu_seqlens_k[b + 1] - a.cu_seqlens_k[b]) - Lq;
    const int64_t first_row = (int64_t)wc * 32 * a.chunk - off;
    if (first_row >= r1) return;
    if (first_row > r0) rb0 = r0 + (int)((first_row - r0) / 64 * 64);
  }
  const int64_t bh = (int64_t)b * a.heads + h;
  // Where the next rows of chunk wc * 32 + j go: lane j keeps the position relative to the start of the word column's
  // first list (the 32 lists follow each other, far less than 2^30 entries), the start itself is a scalar.  A step
  // costs vector instructions and nothing else (the vector pipes are busy 85 % of the kernel's time), so a chunk that
  // some row of the step selects takes five: the lane's rank among the rows (mbcnt), the slot, the store in the lanes
  // of the ballot (the ballot itself is the exec mask), and the new position written back into lane j.
  const int64_t first = a.col_offsets[bh * p.max_cols + wc * 32];
  int32_t *const lists = a.flat_indices + first;
  uint32_t rel = 0u;
  {
    const int c = wc * 32 + lane;
    if (lane < 32 && c < p.max_cols)
      rel = (uint32_t)(a.col_offsets[bh * p.max_cols + c] - first) + (uint32_t)p.segcnt[(bh * p.nseg + seg) * p.max_cols + c];
  }
  const uint32_t *words = p.sel + ((int64_t)h * p.W + wc) * a.total_q + q0;
  for (int rb = rb0; rb < r1; rb += 64) {
    const int r = rb + lane;
    const uint32_t w = (r < r1) ? words[r] : 0u;
    // the chunks that some row of the step selects (a scalar, so that the others cost no vector instruction)
    const uint32_t present = __builtin_amdgcn_readfirstlane(__ockl_wfred_or_u32(w));
    if (present == 0u) continue;
    static_for<32>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      if (present & (1u << j)) {
        const unsigned long long m = __ballot((w & (1u << j)) != 0u);
        const uint32_t at = __builtin_amdgcn_readlane(rel, j);
        const uint32_t rank = __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
        store_i32_in_lanes(lists, (at + rank) << 2, r, m);
        rel = write_lane<j>(rel, at + (uint32_t)__popcll(m));
      }
    });
  }
}

// ------------------------------------------------------------------------------------
// ordered per-row lists (indices / values), only produced on request: one wave per
// (row, head).  The SET of chunks is the gate's own (its selection bits: the lists name
// exactly the chunks whose columns hold the row, also where two scores are so close that
// another summation order would rank them the other way round); the scores that order the
// set are plain FMA sums, then rounds of wave-wide arg-max under the total order (score
// desc, chunk desc).
// ------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(64) void topk_raw_kernel(fmoba_fused_topk_args a, int kr, const uint32_t *sel, int W) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  float *sScore = reinterpret_cast<float *>(smem);  // [Cpad]
  const int row_g = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  // locate the sequence of this row
  int b = 0;
  while (b + 1 < a.batch && a.cu_seqlens_q[b + 1] <= row_g) ++b;
  const int q0 = a.cu_seqlens_q[b];
  const int Lq = a.cu_seqlens_q[b + 1] - q0;
  const int r = row_g - q0;
  int32_t *oi = a.raw_indices + ((int64_t)row_g * a.heads + h) * kr;
  float *ov = a.raw_values + ((int64_t)row_g * a.heads + h) * kr;
  for (int s = lane; s < kr; s += 64) {
    oi[s] = -1;
    ov[s] = -INFINITY;
  }
  if (r < 0 || r >= Lq) return;
  const int Lk = a.cu_seqlens_k[b + 1] - a.cu_seqlens_k[b];
  const int km0 = a.cu_seqlens_km[b];
  const int Cb = a.cu_seqlens_km[b + 1] - km0;
  const int rp = r + Lk - Lq;
  const int hk = h / (a.heads / a.heads_k);
  int nc = a.is_causal ? (rp >= 0 ? min(rp / a.chunk, Cb) : 0) : Cb;
  const uint16_t *qp = reinterpret_cast<const uint16_t *>(a.q) + (int64_t)row_g * a.q_row_stride + (int64_t)h * a.q_head_stride;
  const uint16_t *kmp = reinterpret_cast<const uint16_t *>(a.km) + (int64_t)hk * a.km_head_stride;
  const uint32_t *selrow = sel + (int64_t)h * W * a.total_q + row_g;
  for (int c = lane; c < nc; c += 64) {
    float s = -INFINITY;  // (chunks the gate did not select never enter the lists)
    if ((c >> 5) < W && ((selrow[(int64_t)(c >> 5) * a.total_q] >> (c & 31)) & 1u)) {
      s = 0.f;
      const uint16_t *kr_ = kmp + (int64_t)(km0 + c) * a.km_row_stride;
      for (int d = 0; d < a.head_dim; ++d) s = fmaf(elem_to_float<T>(qp[d]), elem_to_float<T>(kr_[d]), s);
      if (s == -INFINITY) s = -3.4028234663852886e38f;  // a selected chunk keeps its place in the list
    }
    sScore[c] = s;
  }
  __syncthreads();
  int slot = 0;
  if (a.is_causal && rp >= 0) {
    if (lane == 0) {
      oi[0] = rp / a.chunk;
      ov[0] = INFINITY;
    }
    slot = 1;
  }
  // previous winner (score key, chunk) bounds the next search from above
  uint32_t pk = 0xffffffffu;
  int pc = 0x7fffffff;
  for (; slot < a.topk; ++slot) {
    uint32_t bk = 0u;
    int bc = -1;
    for (int c = lane; c < nc; c += 64) {
      const float s = sScore[c];
      if (s == -INFINITY) continue;  // never inserted by a strict '>' against -inf
      const uint32_t k = float_order_key(s);
      const bool below_prev = (k < pk) || (k == pk && c < pc);
      const bool better = (k > bk) || (k == bk && c > bc);
      if (below_prev && better) {
        bk = k;
        bc = c;
      }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      const uint32_t ok = (uint32_t)__shfl_xor((int)bk, o, 64);
      const int oc = __shfl_xor(bc, o, 64);
      if (ok > bk || (ok == bk && oc > bc)) {
        bk = ok;
        bc = oc;
      }
    }
    if (bc < 0) break;
    if (lane == 0) {
      oi[slot] = bc;
      ov[slot] = sScore[bc];
    }
    pk = bk;
    pc = bc;
  }
}

__global__ void fill_i32_kernel(int32_t *p, int64_t n, int32_t v) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = v;
}

static inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

}  // namespace fmoba

extern "C" size_t fmoba_fused_topk_workspace_bytes(int32_t batch, int32_t total_q, int32_t heads, int32_t max_seqlen_q,
                                                   int32_t max_seqlen_k, int32_t chunk) {
  using namespace fmoba;
  if (batch <= 0 || heads <= 0 || chunk <= 0 || total_q < 0) return 0;
  const int64_t max_cols = ceil_div64(max_seqlen_k, chunk);
  const int64_t W = ceil_div64(max_cols, 32);
  const int64_t nseg = ceil_div64(max_seqlen_q > 0 ? max_seqlen_q : 1, csc_seg_rows(batch, heads, max_seqlen_q, W));
  return align256((size_t)heads * W * total_q * 4) + align256((size_t)batch * heads * nseg * max_cols * 4) + 256;
}

namespace fmoba {
template <typename T, int HD, int NT>
static int launch_gate(const TopkParams &p, dim3 grid, hipStream_t s) {
  const size_t smem = (size_t)NT * 32 * HD * 2 + (size_t)NT * 32 * 4;
  auto kern = topk_gate_kernel<T, HD, NT>;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("fused_topk: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  hipLaunchKernelGGL(kern, grid, dim3(256), smem, s, p);
  return 0;
}
template <typename T, int HD>
static int launch_gate_nt(const TopkParams &p, dim3 grid, hipStream_t s) {
  if (p.W <= 2) return launch_gate<T, HD, 2>(p, grid, s);
  if (p.W <= 4) return launch_gate<T, HD, 4>(p, grid, s);
  return launch_gate<T, HD, 8>(p, grid, s);
}
template <int HD, int NT, int CAP>
static constexpr size_t gate_big_smem() {
  const size_t tile = (size_t)NT * 32 * (HD + 16) * 2;  // chunk means of a group; later the selection words of a pass
  const size_t hist = tile / (kGateRows * 4) * 32 * 4;   // counts of the chunks of a pass
  return tile + (size_t)(CAP <= kBigCap ? 2 : 1) * kGateRows * CAP * 8 + (size_t)2 * kGateRows * 4 + hist + 256 * 4;
}
// chunk indices are 16-bit fields of the running winners (topk_gate_stream_kernel) and the forward's step lists
constexpr int kMaxChunksPerSequence = 65535;
template <typename T, int HD, int NT, int CAP>
static int launch_gate_big(const TopkParams &p, dim3 grid, hipStream_t s) {
  const size_t smem = gate_big_smem<HD, NT, CAP>();
  static_assert(gate_big_smem<HD, NT, CAP>() <= 160 * 1024, "LDS of one compute unit");
  auto kern = topk_gate_big_kernel<T, HD, NT, CAP>;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("fused_topk: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  hipLaunchKernelGGL(kern, grid, dim3(256), smem, s, p);
  return 0;
}
template <int HD, int NT>
static constexpr size_t gate_stream_smem() {
  const size_t head = (size_t)NT * 32 * HD * 2 + (size_t)2 * kStreamListWords * 4;  // tile and lists; later the selection words of a pass
  return head + head / (kGateRows * 4) * 32 * 4;
}
template <typename T, int HD, int NT>
static int launch_gate_stream(const TopkParams &p, dim3 grid, hipStream_t s) {
  const size_t smem = gate_stream_smem<HD, NT>();
  auto kern = topk_gate_stream_kernel<T, HD, NT>;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("fused_topk: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  hipLaunchKernelGGL(kern, grid, dim3(256), smem, s, p);
  return 0;
}
template <typename T>
static int launch_gate_big_hd(const TopkParams &p, dim3 grid, hipStream_t s) {
  // up to 16 running winners per row: the kernel that keeps them in registers, in groups of 64 chunks (three workgroups
  // per compute unit; with groups of 128 and two workgroups it took 6.4 ms instead of 5.1 at 262144 tokens)
  const int kp = p.a.is_causal ? p.a.topk - 1 : p.a.topk;
  if (p.a.head_dim <= 64) {
    if (kp > kBigCap) return launch_gate_big<T, 64, 4, kBigCapMax>(p, grid, s);
    if (kp <= 16) return launch_gate_stream<T, 64, 2>(p, grid, s);
    return launch_gate_big<T, 64, 8, kBigCap>(p, grid, s);
  }
  if (p.a.head_dim <= 128) {
    if (kp > kBigCap) return launch_gate_big<T, 128, 4, kBigCapMax>(p, grid, s);
    if (kp <= 16) return launch_gate_stream<T, 128, 2>(p, grid, s);
    return launch_gate_big<T, 128, 8, kBigCap>(p, grid, s);
  }
  if (kp > kBigCap) return launch_gate_big<T, 256, 2, kBigCapMax>(p, grid, s);
  if (kp <= 16) return launch_gate_stream<T, 256, 2>(p, grid, s);
  return launch_gate_big<T, 256, 4, kBigCap>(p, grid, s);
}
template <typename T>
static int launch_gate_hd(const TopkParams &p, dim3 grid, hipStream_t s) {
  if (p.a.head_dim <= 64) return launch_gate_nt<T, 64>(p, grid, s);
  if (p.a.head_dim <= 128) return launch_gate_nt<T, 128>(p, grid, s);
  return launch_gate_nt<T, 256>(p, grid, s);
}
}  // namespace fmoba

// The call behind both entry points: everything of `a` except its workspace fields, which come as arguments.
static int fused_topk_run(const fmoba_fused_topk_args *a, void *workspace, size_t workspace_bytes, void *stream) {
  using namespace fmoba;
  FMOBA_REQUIRE(a != nullptr, "fused_topk: null args");
  FMOBA_REQUIRE(a->dtype == FMOBA_DTYPE_F16 || a->dtype == FMOBA_DTYPE_BF16, "FlashMoBA only supports fp16 and bf16 data types");
  FMOBA_REQUIRE(a->topk >= 1 && a->topk <= 64, "moba_topk must be in [1, 64]");
  FMOBA_REQUIRE(a->batch > 0, "batch size must be positive");
  FMOBA_REQUIRE(a->head_dim > 0 && a->head_dim <= 256, "head_size must be <= 256");
  FMOBA_REQUIRE(a->head_dim % 8 == 0, "head_size must be multiple of 8");
  FMOBA_REQUIRE(a->heads > 0 && a->heads_k > 0 && a->heads % a->heads_k == 0, "#heads in key/value must divide #heads in query");
  FMOBA_REQUIRE(a->chunk > 0, "moba_chunk_size must be positive");
  FMOBA_REQUIRE(a->total_q >= 0 && a->max_seqlen_q >= 0 && a->max_seqlen_k >= 0, "negative size");
  FMOBA_REQUIRE(a->cu_seqlens_q && a->cu_seqlens_k && a->cu_seqlens_km, "fused_topk: null cu_seqlens pointer");
  FMOBA_REQUIRE((a->col_offsets && a->col_nnz) || a->max_seqlen_k == 0, "fused_topk: null col_offsets/col_nnz pointer");
  FMOBA_REQUIRE(a->flat_indices || (int64_t)a->total_q * a->heads * a->topk == 0, "fused_topk: null flat_indices pointer");
  FMOBA_REQUIRE((a->raw_indices == nullptr) == (a->raw_values == nullptr), "fused_topk: raw_indices and raw_values go together");
  hipStream_t s = (hipStream_t)stream;
  const int max_cols = ceil_div(a->max_seqlen_k, a->chunk);
  const int64_t nslots = (int64_t)a->total_q * a->heads * a->topk;
  const int kr = (a->topk + 15) / 16 * 16;

  if (max_cols == 0 || a->max_seqlen_k == 0) {
    // no keys: lists stay empty; the reference fills the row list with -1 here
    // (csrc/flash_topk/flash_topk_api.cpp:250-255)
    if (nslots) hipLaunchKernelGGL(fill_i32_kernel, dim3(1024), dim3(256), 0, s, a->flat_indices, nslots, -1);
    if (a->raw_indices && a->total_q) {
      hipLaunchKernelGGL(fill_i32_kernel, dim3(1024), dim3(256), 0, s, a->raw_indices, (int64_t)a->total_q * a->heads * kr, -1);
      hipLaunchKernelGGL(fill_i32_kernel, dim3(1024), dim3(256), 0, s, reinterpret_cast<int32_t *>(a->raw_values),
                         (int64_t)a->total_q * a->heads * kr, (int32_t)0xff800000);
    }
    FMOBA_LAUNCH_CHECK("fused_topk(empty)");
    return 0;
  }
  const bool big = max_cols > 256;  // more chunks than the register-resident gate holds: grouped gate
  FMOBA_REQUIRE(max_cols <= kMaxChunksPerSequence, "fused_topk: %d key chunks per sequence; at most %d are supported", max_cols, kMaxChunksPerSequence);
  // (the fill keeps list positions as 32-bit byte offsets from the first of the 32 lists of a word column)
  FMOBA_REQUIRE(a->max_seqlen_q < (1 << 24), "fused_topk: max_seqlen_q = %d; sequences of up to %d query rows are supported", a->max_seqlen_q,
                (1 << 24) - 1);
  FMOBA_REQUIRE(a->q && a->km, "fused_topk: null q/km pointer");
  FMOBA_REQUIRE(a->q_row_stride % 8 == 0 && a->q_head_stride % 8 == 0 && a->km_row_stride % 8 == 0 && a->km_head_stride % 8 == 0,
                "fused_topk: strides must be multiples of 8 elements");
  FMOBA_REQUIRE(((uintptr_t)a->q % 16) == 0 && ((uintptr_t)a->km % 16) == 0, "fused_topk: q and km must be 16-byte aligned");
  FMOBA_REQUIRE(a->batch <= 65535 && a->heads <= 65535, "fused_topk: batch/heads too large for the launch grid");

  TopkParams p;
  p.a = *a;
  p.max_cols = max_cols;
  p.W = ceil_div(max_cols, 32);
  p.seg_rows = csc_seg_rows(a->batch, a->heads, a->max_seqlen_q, p.W);
  p.nseg = ceil_div(a->max_seqlen_q > 0 ? a->max_seqlen_q : 1, p.seg_rows);
  const size_t sel_bytes = align256((size_t)a->heads * p.W * a->total_q * 4);
  const size_t seg_bytes = align256((size_t)a->batch * a->heads * p.nseg * max_cols * 4);
  FMOBA_REQUIRE(workspace != nullptr && workspace_bytes >= sel_bytes + seg_bytes, "fused_topk: workspace too small (%zu < %zu)",
                workspace_bytes, sel_bytes + seg_bytes);
  uintptr_t wsp = ((uintptr_t)workspace + 255) & ~(uintptr_t)255;
  FMOBA_REQUIRE(wsp + sel_bytes + seg_bytes <= (uintptr_t)workspace + workspace_bytes, "fused_topk: workspace too small after alignment");
  p.sel = reinterpret_cast<uint32_t *>(wsp);
  p.segcnt = reinterpret_cast<int32_t *>(wsp + sel_bytes);

  if (a->total_q == 0 || a->max_seqlen_q == 0) {
    // no query rows: every column is empty, offsets are the (constant) region bases
    const int64_t n = (int64_t)a->batch * a->heads * max_cols;
    hipLaunchKernelGGL(fill_i32_kernel, dim3(256), dim3(256), 0, s, p.segcnt, (int64_t)(seg_bytes / 4), 0);
    hipLaunchKernelGGL(csc_scan_kernel, dim3(a->heads, a->batch), dim3(256), 0, s, p);
    (void)n;
    FMOBA_LAUNCH_CHECK("fused_topk(no rows)");
    return 0;
  }

  hipLaunchKernelGGL(fill_i32_kernel, dim3(512), dim3(256), 0, s, p.segcnt, (int64_t)(seg_bytes / 4), 0);
  dim3 ggrid(ceil_div(a->max_seqlen_q, kGateRows), a->heads, a->batch);
  int rc;
  if (big)
    rc = (a->dtype == FMOBA_DTYPE_BF16) ? launch_gate_big_hd<bf16_t>(p, ggrid, s) : launch_gate_big_hd<f16_t>(p, ggrid, s);
  else
    rc = (a->dtype == FMOBA_DTYPE_BF16) ? launch_gate_hd<bf16_t>(p, ggrid, s) : launch_gate_hd<f16_t>(p, ggrid, s);
  if (rc) return rc;
  FMOBA_LAUNCH_CHECK("topk_gate_kernel");
  hipLaunchKernelGGL(csc_scan_kernel, dim3(a->heads, a->batch), dim3(256), 0, s, p);
  FMOBA_LAUNCH_CHECK("csc_scan_kernel");
  hipLaunchKernelGGL(csc_fill_kernel, dim3(p.nseg * p.W, a->heads, a->batch), dim3(64), 0, s, p);
  FMOBA_LAUNCH_CHECK("csc_fill_kernel");
  if (a->raw_indices) {
    const size_t smem = (size_t)(max_cols + 64) * 4;
    dim3 rgrid(a->total_q, a->heads);
    if (a->dtype == FMOBA_DTYPE_BF16)
      hipLaunchKernelGGL(topk_raw_kernel<bf16_t>, rgrid, dim3(64), smem, s, *a, kr, p.sel, p.W);
    else
      hipLaunchKernelGGL(topk_raw_kernel<f16_t>, rgrid, dim3(64), smem, s, *a, kr, p.sel, p.W);
    FMOBA_LAUNCH_CHECK("topk_raw_kernel");
  }
  return 0;
}

extern "C" int fmoba_fused_topk(const fmoba_fused_topk_args *a, void *stream) {
  FMOBA_REQUIRE(a != nullptr, "fused_topk: null args");
  return fused_topk_run(a, a->workspace, a->workspace_bytes, stream);
}

// ------------------------------------------------------------------------------------
// The same call for callers that cannot allocate device memory (HIP graph capture, serving loops): selection bits and
// segment counts live in a fixed array of the code object instead of a caller's workspace.  Every device that loads
// the library holds its own copy of the array at its own address, which the runtime tells once per device.
// ------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[FMOBA_STATIC_SCRATCH_BYTES];

namespace fmoba {
constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void *g_scratch_ptr[kMaxDevices];  // device address of `scratch` per device, null until asked for
}  // namespace fmoba

extern "C" int fmoba_fused_topk_static(const fmoba_fused_topk_args *a, void *stream) {
  using namespace fmoba;
  FMOBA_REQUIRE(a != nullptr, "fused_topk_static: null args");
  const size_t need = fmoba_fused_topk_workspace_bytes(a->batch, a->total_q, a->heads, a->max_seqlen_q, a->max_seqlen_k, a->chunk);
  FMOBA_REQUIRE(need <= (size_t)FMOBA_STATIC_SCRATCH_BYTES,
                "fused_topk_static: this call needs %zu bytes of scratch memory, the library's fixed buffer holds %zu; use fmoba_fused_topk with a workspace",
                need, (size_t)FMOBA_STATIC_SCRATCH_BYTES);
  int dev = -1;
  FMOBA_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices, "fused_topk_static: no current HIP device (or its index is above %d)", kMaxDevices - 1);
  void *ptr = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
      void *p = nullptr;
      const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      FMOBA_REQUIRE(e == hipSuccess && p != nullptr, "fused_topk_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
      g_scratch_ptr[dev] = p;
    }
    ptr = g_scratch_ptr[dev];
  }
  return fused_topk_run(a, ptr, (size_t)FMOBA_STATIC_SCRATCH_BYTES, stream);
}
