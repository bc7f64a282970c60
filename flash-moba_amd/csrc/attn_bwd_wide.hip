// dK / dV (and the dS tiles of the row-block dQ pass) for head dimensions above 128, up to 256.
//
// Same column-stationary scheme as attn_bwd_dkdv_kernel -- one workgroup per (64-key block, head, sequence) walks the
// block's ascending row list in gathered 32-row tiles: S = Q K^T, dP = dO V^T, P = exp2(S*scale*log2e - LSE*log2e),
// dS = P o (dP - delta), dV^T += dO^T P, dK^T += Q^T dS -- with the feature axis split, because 32 keys x 256 features
// of dK^T and dV^T no longer fit one wave's registers next to the K / V operands: wave w owns the keys 32 (w % 2) ..
// and the features 128 (w / 2) .. of the accumulators.  S and dP need the whole head dimension, so the two waves of a
// key half both form them (6 instead of 4 units of MFMA work per pair, the price of the split), and K / V stay in LDS
// instead of registers.  One tile at a time, loaded by all threads between two barriers: this is the plain form, kept
// simple; the tuned kernels serve head dimensions up to 128 (the reference gives its head dimensions 192 and 256 their
// own, smaller tilings for the same reason: run_moba_bwd_hdim192 / run_moba_bwd_hdim256, flash_bwd_launch_template.h:237-279).
#include "fmoba_common.h"

namespace fmoba {

constexpr int kWideHD = 256;

struct BwdWideSmem {
  static constexpr int LD = kWideHD + 8;   // elements, K / V / Q / dO rows
  static constexpr int LDX = 64 + 8;       // elements, dS tile rows [32 rows][64 keys]
  static constexpr int LDR = kWideHD + 4;  // floats, output staging [64 keys][LDR]
  static constexpr size_t oK = 0;                                    // [64][LD]
  static constexpr size_t oV = oK + (size_t)64 * LD * 2;
  static constexpr size_t oQ = oV + (size_t)64 * LD * 2;             // [32][LD]
  static constexpr size_t odO = oQ + (size_t)32 * LD * 2;
  static constexpr size_t odS = odO + (size_t)32 * LD * 2;           // [32][LDX]
  static constexpr size_t oRow = odS + (size_t)32 * LDX * 2;         // int[32]
  static constexpr size_t oLse = oRow + 32 * 4;                      // float[32]: LSE * log2(e), +inf for absent rows
  static constexpr size_t oDelta = oLse + 32 * 4;
  static constexpr size_t bytes = oDelta + 32 * 4;
  static_assert((size_t)64 * LDR * 4 <= oQ, "one output staging buffer fits where K and V were");
  static_assert(bytes <= 160 * 1024, "LDS of one compute unit");
};

// grid (key blocks of 64, heads, batch), block 256
template <typename T>
__global__ __launch_bounds__(256) void attn_bwd_dkdv_wide_kernel(fmoba_attn_bwd_args a, uint16_t *ds_ws) {
  typedef BwdWideSmem SM;
  constexpr int HD = kWideHD, KS = HD / 16, LD = SM::LD, LDX = SM::LDX, LDR = SM::LDR, VPR = HD / 8;
  constexpr int NDTW = HD / 64;  // feature tiles of 32 per wave (its half of the head dimension)
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint16_t *sK = reinterpret_cast<uint16_t *>(smem + SM::oK), *sV = reinterpret_cast<uint16_t *>(smem + SM::oV);
  uint16_t *sQ = reinterpret_cast<uint16_t *>(smem + SM::oQ), *sdO = reinterpret_cast<uint16_t *>(smem + SM::odO);
  uint16_t *sdS = reinterpret_cast<uint16_t *>(smem + SM::odS);
  int *sRow = reinterpret_cast<int *>(smem + SM::oRow);
  float *sLse = reinterpret_cast<float *>(smem + SM::oLse), *sDelta = reinterpret_cast<float *>(smem + SM::oDelta);

  const int nb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int k0 = a.cu_seqlens_k[b], Lk = a.cu_seqlens_k[b + 1] - k0;
  const int key0 = nb * 64;
  if (key0 >= Lk) return;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int off = Lk - Lq;
  const int D = a.head_dim;
  const int hk = h / (a.heads / a.heads_k);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
  const int kq = wave & 1, fh = wave >> 1;  // key half, feature half
  const bool causal = a.is_causal != 0;
  const float scale_log2 = a.softmax_scale * 1.4426950408889634f;
  constexpr float kLog2e = 1.4426950408889634f;

  // ---- K and V of the block into LDS (keys past the sequence and features past head_dim: zeros) ----
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
      *reinterpret_cast<Pack8 *>(sK + key * LD + e) = xk;
      *reinterpret_cast<Pack8 *>(sV + key * LD + e) = xv;
    }
  }
  // ---- this block's column list ----
  const int Bn = a.lg_block_n;
  const int c = key0 / Bn;
  const int64_t bh = (int64_t)b * a.heads + h;
  int nnz = 0, start = 0;
  int64_t lbase = 0;
  if (c < a.max_cols) {
    nnz = a.col_nnz[bh * a.max_cols + c];
    lbase = a.col_offsets[bh * a.max_cols + c];
    if (causal && nnz > 0) start = lower_bound_wave_i32(a.row_indices + lbase, nnz, key0 - off);  // earlier rows see no key of the block
  }
  const int32_t *list = a.row_indices + lbase + start;
  const int n = nnz - start;
  const int ntile = (n + 31) / 32;
  const int koff = key0 - c * Bn;  // offset of this 64-key block inside its column

  const uint16_t *qg = reinterpret_cast<const uint16_t *>(a.q) + (int64_t)q0 * a.q_row_stride + (int64_t)h * a.q_head_stride;
  const uint16_t *dog = reinterpret_cast<const uint16_t *>(a.dout) + (int64_t)q0 * a.do_row_stride + (int64_t)h * a.do_head_stride;
  const float *lseg = a.softmax_lse + (int64_t)h * a.total_q + q0;
  const float *delg = a.softmax_d + (int64_t)h * ((int64_t)a.total_q + 128 * (int64_t)a.batch) + q0 + 128 * b;

  f32x16 dv[NDTW], dk[NDTW];  // register i of tile dt <-> feature fh*128 + dt*32 + acc_row(i, hh), key kq*32 + lane % 32
#pragma unroll
  for (int dt = 0; dt < NDTW; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      dv[dt][i] = 0.f;
      dk[dt][i] = 0.f;
    }
  // this lane's key; key j is visible to row r iff r >= row_thr
  const int j = key0 + kq * 32 + (lane & 31);
  const int row_thr = j >= Lk ? 0x7fffffff : (causal ? max(0, j - off) : 0);

  for (int tile = 0; tile < ntile; ++tile) {
    __syncthreads();  // the previous tile is no longer read (first pass: K and V are in LDS)
    // gathered Q / dO rows and the per-row scalars of the tile; absent rows: zeros, LSE = +inf
    for (int v = tid; v < 32 * VPR; v += 256) {
      const int rl = v / VPR, e = (v - rl * VPR) * 8;
      const int jj = tile * 32 + rl;
      const int r = jj < n ? list[jj] : -1;
      Pack8 xq = zero_pack8(), xo = zero_pack8();
      if (r >= 0 && r < Lq && e < D) {
        xq = ld_global16(qg + (int64_t)r * a.q_row_stride + e);
        xo = ld_global16(dog + (int64_t)r * a.do_row_stride + e);
      }
      *reinterpret_cast<Pack8 *>(sQ + rl * LD + e) = xq;
      *reinterpret_cast<Pack8 *>(sdO + rl * LD + e) = xo;
    }
    if (tid < 32) {
      const int jj = tile * 32 + tid;
      const int r = jj < n ? list[jj] : -1;
      const bool ok = r >= 0 && r < Lq;
      sRow[tid] = ok ? r : -1;
      sLse[tid] = ok ? lseg[r] * kLog2e : INFINITY;
      sDelta[tid] = ok ? delg[r] : 0.f;
    }
    __syncthreads();
    // S and dP of this wave's 32 keys over the whole head dimension (contraction index permuted so that each half of
    // the wave reads one contiguous half of a row)
    f32x16 s, dp;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i] = 0.f;
      dp[i] = 0.f;
    }
#pragma unroll
    for (int t = 0; t < KS; ++t) {
      const int e = (hh * KS + t) * 8;
      const Pack8 qa = *reinterpret_cast<const Pack8 *>(sQ + (lane & 31) * LD + e);
      const Pack8 kb = *reinterpret_cast<const Pack8 *>(sK + (kq * 32 + (lane & 31)) * LD + e);
      s = mfma32<T>(qa, kb, s);
      const Pack8 da = *reinterpret_cast<const Pack8 *>(sdO + (lane & 31) * LD + e);
      const Pack8 vb = *reinterpret_cast<const Pack8 *>(sV + (kq * 32 + (lane & 31)) * LD + e);
      dp = mfma32<T>(da, vb, dp);
    }
    // P and dS: register i <-> row acc_row(i, hh) of the tile, this lane's key
    Pack8 pf[2], dsf[2];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float pr[4], dsv[4];
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int i = 4 * g + jj, rl = acc_row(i, hh);
        const float x = sRow[rl] >= row_thr ? fmaf(s[i], scale_log2, -sLse[rl]) : -INFINITY;  // (absent rows: row id -1, LSE +inf)
        pr[jj] = __builtin_amdgcn_exp2f(x);
        dsv[jj] = pr[jj] * (dp[i] - sDelta[rl]);
        if (fh == 0) sdS[rl * LDX + kq * 32 + (lane & 31)] = float_to_elem_bits<T>(dsv[jj]);
      }
      // operand register s2 = g / 2 holds rows 16 s2 + 8 (w / 2) + 4 hh + ..: words 2 (g % 2), 2 (g % 2) + 1
      pf[g >> 1].w[2 * (g & 1)] = pack2<T>(pr[0], pr[1]);
      pf[g >> 1].w[2 * (g & 1) + 1] = pack2<T>(pr[2], pr[3]);
      dsf[g >> 1].w[2 * (g & 1)] = pack2<T>(dsv[0], dsv[1]);
      dsf[g >> 1].w[2 * (g & 1) + 1] = pack2<T>(dsv[2], dsv[3]);
    }
    // dV^T[d][key] += dO^T[d][row] P[row][key];  dK^T[d][key] += Q^T[d][row] dS[row][key], this wave's features
#pragma unroll
    for (int dt = 0; dt < NDTW; ++dt)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const int col0 = fh * (HD / 2) + dt * 32;
        const Pack8 dot = tr_frag8(sdO, LD, 16 * s2 + 4 * hh, 16 * s2 + 8 + 4 * hh, col0, lane);
        const Pack8 qt = tr_frag8(sQ, LD, 16 * s2 + 4 * hh, 16 * s2 + 8 + 4 * hh, col0, lane);
        dv[dt] = mfma32<T>(dot, pf[s2], dv[dt]);
        dk[dt] = mfma32<T>(qt, dsf[s2], dk[dt]);
      }
    // the dS tile leaves in 16-byte pieces (8 keys of one list entry), one per thread
    if (ds_ws != nullptr) {
      __syncthreads();
      const int rl = tid & 31, piece = tid >> 5;  // consecutive threads: consecutive list positions of one key group
      if (sRow[rl] >= 0)
        *reinterpret_cast<Pack8 *>(ds_ws + ds_piece_offset(lbase + start + tile * 32 + rl, (koff >> 3) + piece, Bn >> 3)) = *reinterpret_cast<const Pack8 *>(sdS + rl * LDX + piece * 8);
    }
  }

  // ---- dK^T / dV^T leave as rows: through LDS, dV first, then dK (one staging buffer) ----
  float *red = reinterpret_cast<float *>(smem);  // [64 keys][LDR]
  uint16_t *dkg = reinterpret_cast<uint16_t *>(a.dk) + (int64_t)(k0 + key0) * a.dk_row_stride + (int64_t)h * a.dk_head_stride;
  uint16_t *dvg = reinterpret_cast<uint16_t *>(a.dv) + (int64_t)(k0 + key0) * a.dv_row_stride + (int64_t)h * a.dv_head_stride;
#pragma unroll
  for (int which = 0; which < 2; ++which) {
    __syncthreads();  // the staging buffer (K / V at first) is no longer read
#pragma unroll
    for (int dt = 0; dt < NDTW; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4 x;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) x[jj] = which == 0 ? dv[dt][4 * g + jj] : dk[dt][4 * g + jj];
        *reinterpret_cast<f32x4 *>(red + (size_t)(kq * 32 + (lane & 31)) * LDR + fh * (HD / 2) + dt * 32 + 8 * g + 4 * hh) = x;
      }
    __syncthreads();
    const float mul = which == 0 ? 1.f : a.softmax_scale;
    uint16_t *og = which == 0 ? dvg : dkg;
    const int64_t ostride = which == 0 ? a.dv_row_stride : a.dk_row_stride;
    for (int v = tid; v < 64 * VPR; v += 256) {
      const int key = v / VPR, e = (v - key * VPR) * 8;
      if (key0 + key >= Lk || e >= D) continue;
      const float *sp = red + (size_t)key * LDR + e;
      Pack8 o;
#pragma unroll
      for (int w = 0; w < 4; ++w) o.w[w] = pack2<T>(sp[2 * w] * mul, sp[2 * w + 1] * mul);
      *reinterpret_cast<Pack8 *>(og + (int64_t)key * ostride + e) = o;
    }
  }
}

// dK / dV and the dS tiles for head dimensions above 128 (ds_ws: the dS workspace, laid out by ds_piece_offset)
int run_bwd_dkdv_wide(const fmoba_attn_bwd_args &a, uint16_t *ds_ws, hipStream_t s) {
  const size_t smem = BwdWideSmem::bytes;
  const dim3 grid(ceil_div(a.max_seqlen_k, 64), a.heads, a.batch);
  if (a.dtype == FMOBA_DTYPE_BF16) {
    auto kern = attn_bwd_dkdv_wide_kernel<bf16_t>;
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
      set_error("attn_bwd: cannot reserve %zu bytes of LDS", smem);
      return 2;
    }
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, s, a, ds_ws);
  } else {
    auto kern = attn_bwd_dkdv_wide_kernel<f16_t>;
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
      set_error("attn_bwd: cannot reserve %zu bytes of LDS", smem);
      return 2;
    }
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, s, a, ds_ws);
  }
  return 0;
}

}  // namespace fmoba
