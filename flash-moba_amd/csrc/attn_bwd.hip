// Sparse attention backward over a CSC pattern: column-stationary.
//
//   bwd_prep_kernel   : delta[row] = sum_d dO*O (fp32) and clears the fp32 dQ accumulator.
//   attn_bwd_kernel   : one workgroup per (64-key block, head, sequence).  K and V of the
//                       block stay in LDS; each wave walks its share of the block's
//                       ascending row list in gathered 32-row tiles:
//                         S = Q K^T, dP = dO V^T            (A = gathered rows, B = K / V)
//                         P = exp2(S*scale*log2e - LSE*log2e), dS = P o (dP - delta)
//                         dV^T += dO^T P, dK^T += Q^T dS    (P, dS feed the MFMA from registers;
//                                                            dO^T, Q^T via transposing LDS reads)
//                         dQ = dS K                         (dS through LDS, K^T via transposing reads)
//                       dK/dV live in accumulator registers for the whole list and are written
//                       once, without atomics; dQ tiles are added to the fp32 accumulator with
//                       hardware fp32 atomics, 128 contiguous bytes per row per instruction.
//   bwd_convert_kernel: dQ = cast(accumulator * softmax_scale).
#include "fmoba_common.h"

namespace fmoba {

template <int HD>
struct BwdSmem {
  static constexpr int LDQ = HD + 16;   // elements, K/V/Q/dO tiles
  static constexpr int LDS_ = 32 + 8;   // elements, dS^T tile [64 keys][32 rows]
  static constexpr size_t oK = 0;
  static constexpr size_t oV = oK + (size_t)64 * LDQ * 2;
  static constexpr size_t oWave = oV + (size_t)64 * LDQ * 2;
  // per wave
  static constexpr size_t wQ = 0;
  static constexpr size_t wdO = wQ + (size_t)32 * LDQ * 2;
  static constexpr size_t wdS = wdO + (size_t)32 * LDQ * 2;
  static constexpr size_t wRow = wdS + (size_t)64 * LDS_ * 2;
  static constexpr size_t wLse = wRow + 32 * 4;
  static constexpr size_t wDelta = wLse + 32 * 4;
  static constexpr size_t waveBytes = wDelta + 32 * 4;
  static constexpr size_t mainBytes = oWave + 4 * waveBytes;
  static constexpr int LDR = HD + 4;    // floats, reduction buffer [4][64][LDR]
  static constexpr size_t redBytes = (size_t)4 * 64 * LDR * 4;
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
__global__ __launch_bounds__(256) void attn_bwd_kernel(fmoba_attn_bwd_args a, float *dq_accum) {
  typedef BwdSmem<HD> SM;
  constexpr int KS = HD / 16, LDQ = SM::LDQ, LDS_ = SM::LDS_, NDT = HD / 32, VPR = HD / 8, LDR = SM::LDR;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint16_t *sK = reinterpret_cast<uint16_t *>(smem + SM::oK);
  uint16_t *sV = reinterpret_cast<uint16_t *>(smem + SM::oV);

  const int nb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int k0 = a.cu_seqlens_k[b], Lk = a.cu_seqlens_k[b + 1] - k0;
  const int key0 = nb * 64;
  if (key0 >= Lk) return;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int off = Lk - Lq;
  const int D = a.head_dim;
  const int hk = h / (a.heads / a.heads_k);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
  const bool causal = a.is_causal != 0;
  const float scale_log2 = a.softmax_scale * 1.4426950408889634f;
  constexpr float kLog2e = 1.4426950408889634f;

  uint8_t *wbase = smem + SM::oWave + (size_t)wave * SM::waveBytes;
  uint16_t *sQ = reinterpret_cast<uint16_t *>(wbase + SM::wQ);
  uint16_t *sdO = reinterpret_cast<uint16_t *>(wbase + SM::wdO);
  uint16_t *sdS = reinterpret_cast<uint16_t *>(wbase + SM::wdS);
  int *sRow = reinterpret_cast<int *>(wbase + SM::wRow);
  float *sLse = reinterpret_cast<float *>(wbase + SM::wLse);
  float *sDelta = reinterpret_cast<float *>(wbase + SM::wDelta);

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
  const int c = key0 / a.lg_block_n;
  const int64_t bh = (int64_t)b * a.heads + h;
  int nnz = 0;
  const int32_t *list = a.row_indices;
  int start = 0;
  if (c < a.max_cols) {
    nnz = a.col_nnz[bh * a.max_cols + c];
    list = a.row_indices + a.col_offsets[bh * a.max_cols + c];
    // rows r with r + off < key0 see no key of this block
    if (causal && nnz > 0) start = lower_bound_i32b(list, nnz, key0 - off);
  }
  const int ntiles = (nnz - start + 31) / 32;

  f32x16 dv[NDT][2], dk[NDT][2];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        dv[dt][kt][i] = 0.f;
        dk[dt][kt][i] = 0.f;
      }

  const uint16_t *qg = reinterpret_cast<const uint16_t *>(a.q) + (int64_t)q0 * a.q_row_stride + (int64_t)h * a.q_head_stride;
  const uint16_t *dog = reinterpret_cast<const uint16_t *>(a.dout) + (int64_t)q0 * a.do_row_stride + (int64_t)h * a.do_head_stride;
  const float *lseg = a.softmax_lse + (int64_t)h * a.total_q + q0;
  const float *delg = a.softmax_d + (int64_t)h * ((int64_t)a.total_q + 128 * (int64_t)a.batch) + q0 + 128 * b;
  float *dqg = dq_accum + ((int64_t)q0 * a.heads + h) * D;

  for (int tile = wave; tile < ntiles; tile += 4) {
    const int ridx = start + tile * 32 + (lane & 31);
    int r = ridx < nnz ? list[ridx] : -1;
    if (r >= Lq) r = -1;  // rows outside the sequence (malformed pattern) are ignored
    const bool valid = r >= 0;
    wave_lds_fence();  // the previous tile's readers of this wave's LDS region are done
    if (lane < 32) {
      sRow[lane] = r;
      sLse[lane] = valid ? lseg[r] : INFINITY;
      sDelta[lane] = valid ? delg[r] : 0.f;
    }
    // stage the gathered Q and dO rows (row-major, zero padded)
    {
      constexpr int RPI = 64 / VPR;  // rows per wave-wide 16-byte load
      const int e = (lane % VPR) * 8;
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const int row = it * RPI + lane / VPR;
        const int rr = __shfl(r, row, 64);
        Pack8 xq = zero_pack8(), xo = zero_pack8();
        if (rr >= 0 && e < D) {
          xq = ld_global16(qg + (int64_t)rr * a.q_row_stride + e);
          xo = ld_global16(dog + (int64_t)rr * a.do_row_stride + e);
        }
        *reinterpret_cast<Pack8 *>(sQ + row * LDQ + e) = xq;
        *reinterpret_cast<Pack8 *>(sdO + row * LDQ + e) = xo;
      }
    }
    wave_lds_fence();

    Pack8 qa[KS], doa[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qa[ks] = *reinterpret_cast<const Pack8 *>(sQ + (lane & 31) * LDQ + (hh * KS + ks) * 8);
      doa[ks] = *reinterpret_cast<const Pack8 *>(sdO + (lane & 31) * LDQ + (hh * KS + ks) * 8);
    }
    // per-register row data: register i holds row acc_row(i, hh) = 8*(i/4) + 4*hh + i%4
    int rrow[16];
    float rlse[16], rdel[16];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int base = 8 * g + 4 * hh;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        rrow[4 * g + j] = sRow[base + j];
        rlse[4 * g + j] = sLse[base + j] * kLog2e;
        rdel[4 * g + j] = sDelta[base + j];
      }
    }

#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      f32x16 s, dp;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        s[i] = 0.f;
        dp[i] = 0.f;
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const Pack8 kf = *reinterpret_cast<const Pack8 *>(sK + (kt * 32 + (lane & 31)) * LDQ + (hh * KS + ks) * 8);
        const Pack8 vf = *reinterpret_cast<const Pack8 *>(sV + (kt * 32 + (lane & 31)) * LDQ + (hh * KS + ks) * 8);
        s = mfma32<T>(qa[ks], kf, s);
        dp = mfma32<T>(doa[ks], vf, dp);
      }
      // this lane's key; register i <-> gathered row acc_row(i, hh)
      const int j = key0 + kt * 32 + (lane & 31);
      float pr[16], ds[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const bool vis = rrow[i] >= 0 && j < Lk && (!causal || j <= rrow[i] + off);
        const float p = vis ? exp2f(s[i] * scale_log2 - rlse[i]) : 0.f;
        pr[i] = p;
        ds[i] = p * (dp[i] - rdel[i]);
      }
      Pack8 pf[2], dsf[2];
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          pf[s2].w[w] = pack2<T>(pr[8 * s2 + 2 * w], pr[8 * s2 + 2 * w + 1]);
          dsf[s2].w[w] = pack2<T>(ds[8 * s2 + 2 * w], ds[8 * s2 + 2 * w + 1]);
        }
      // dV^T[d][key] += dO^T[d][row] P[row][key];  dK^T[d][key] += Q^T[d][row] dS[row][key]
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const Pack8 dot = tr_frag8(sdO, LDQ, 16 * s2 + 4 * hh, 16 * s2 + 8 + 4 * hh, dt * 32, lane);
          const Pack8 qt = tr_frag8(sQ, LDQ, 16 * s2 + 4 * hh, 16 * s2 + 8 + 4 * hh, dt * 32, lane);
          dv[dt][kt] = mfma32<T>(dot, pf[s2], dv[dt][kt]);
          dk[dt][kt] = mfma32<T>(qt, dsf[s2], dk[dt][kt]);
        }
      // dS^T to LDS: row (kt*32 + lane%32) of the [64 keys][32 rows] tile, 4 rows per 8-byte store
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint32_t w0 = pack2<T>(ds[4 * g], ds[4 * g + 1]), w1 = pack2<T>(ds[4 * g + 2], ds[4 * g + 3]);
        uint2 v2 = make_uint2(w0, w1);
        *reinterpret_cast<uint2 *>(sdS + (kt * 32 + (lane & 31)) * LDS_ + 8 * g + 4 * hh) = v2;
      }
    }
    wave_lds_fence();

    // dQ[row][d] = sum_key dS[row][key] K[key][d]
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      f32x16 dq;
#pragma unroll
      for (int i = 0; i < 16; ++i) dq[i] = 0.f;
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) {
        const Pack8 af = tr_frag8(sdS, LDS_, 16 * s4 + 8 * hh, 16 * s4 + 8 * hh + 4, 0, lane);
        const Pack8 bf = tr_frag8(sK, LDQ, 16 * s4 + 8 * hh, 16 * s4 + 8 * hh + 4, dt * 32, lane);
        dq = mfma32<T>(af, bf, dq);
      }
      const int d = dt * 32 + (lane & 31);
      if (d < D) {
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (rrow[i] >= 0) atomicAdd(dqg + (int64_t)rrow[i] * a.heads * D + d, dq[i]);
      }
    }
  }

  // ---- reduce the four waves' partial dK / dV through LDS and write once -----------------------
  float *red = reinterpret_cast<float *>(smem);
  uint16_t *dkg = reinterpret_cast<uint16_t *>(a.dk) + (int64_t)(k0 + key0) * a.dk_row_stride + (int64_t)h * a.dk_head_stride;
  uint16_t *dvg = reinterpret_cast<uint16_t *>(a.dv) + (int64_t)(k0 + key0) * a.dv_row_stride + (int64_t)h * a.dv_head_stride;
#pragma unroll
  for (int which = 0; which < 2; ++which) {
    __syncthreads();
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          f32x4 v4;
#pragma unroll
          for (int j = 0; j < 4; ++j) v4[j] = which == 0 ? dv[dt][kt][4 * g + j] : dk[dt][kt][4 * g + j];
          *reinterpret_cast<f32x4 *>(red + ((size_t)wave * 64 + kt * 32 + (lane & 31)) * LDR + dt * 32 + 8 * g + 4 * hh) = v4;
        }
    __syncthreads();
    const float mul = which == 0 ? 1.f : a.softmax_scale;
    uint16_t *og = which == 0 ? dvg : dkg;
    const int64_t ors = which == 0 ? a.dv_row_stride : a.dk_row_stride;
    for (int v = tid; v < 64 * VPR; v += 256) {
      const int key = v / VPR, e = (v - key * VPR) * 8;
      if (key0 + key >= Lk || e >= D) continue;
      float acc[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float *src = red + ((size_t)w * 64 + key) * LDR + e;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] += src[i];
      }
      Pack8 o;
#pragma unroll
      for (int w = 0; w < 4; ++w) o.w[w] = pack2<T>(acc[2 * w] * mul, acc[2 * w + 1] * mul);
      *reinterpret_cast<Pack8 *>(og + (int64_t)key * ors + e) = o;
    }
  }
}

// grid (ceil(max_seqlen_q / rows_per_block), heads, batch), block 256.
// LPR lanes cooperate on one row (LPR = power of two >= head_dim / 8).
template <typename T>
__global__ __launch_bounds__(256) void bwd_prep_kernel(fmoba_attn_bwd_args a, float *dq_accum, int LPR) {
  const int rows_per_block = 256 / LPR;
  const int h = blockIdx.y, b = blockIdx.z;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int r = blockIdx.x * rows_per_block + threadIdx.x / LPR;
  const int sub = threadIdx.x % LPR;
  const int e = sub * 8;
  const int D = a.head_dim;
  float acc = 0.f;
  const bool act = r < Lq && e < D;
  if (act) {
    const Pack8 o = ld_global16(reinterpret_cast<const uint16_t *>(a.out) + (int64_t)(q0 + r) * a.o_row_stride + (int64_t)h * a.o_head_stride + e);
    const Pack8 g = ld_global16(reinterpret_cast<const uint16_t *>(a.dout) + (int64_t)(q0 + r) * a.do_row_stride + (int64_t)h * a.do_head_stride + e);
    float fo[8], fg[8];
    unpack8<T>(o, fo);
    unpack8<T>(g, fg);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc = fmaf(fo[i], fg[i], acc);
    float *dq = dq_accum + ((int64_t)(q0 + r) * a.heads + h) * D + e;
    *reinterpret_cast<f32x4 *>(dq) = f32x4{0.f, 0.f, 0.f, 0.f};
    *reinterpret_cast<f32x4 *>(dq + 4) = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  for (int o = LPR >> 1; o >= 1; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if (r < Lq && sub == 0) a.softmax_d[(int64_t)h * ((int64_t)a.total_q + 128 * (int64_t)a.batch) + q0 + 128 * b + r] = acc;
}

template <typename T>
__global__ __launch_bounds__(256) void bwd_convert_kernel(fmoba_attn_bwd_args a, const float *dq_accum) {
  const int D = a.head_dim, vpr = D / 8;
  const int64_t nvec = (int64_t)a.total_q * a.heads * vpr;
  for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * blockDim.x) {
    const int64_t rh = v / vpr;
    const int e = (int)(v - rh * vpr) * 8;
    const int64_t row = rh / a.heads;
    const int h = (int)(rh - row * a.heads);
    const float *src = dq_accum + rh * D + e;
    const f32x4 x0 = *reinterpret_cast<const f32x4 *>(src), x1 = *reinterpret_cast<const f32x4 *>(src + 4);
    Pack8 o;
    o.w[0] = pack2<T>(x0[0] * a.softmax_scale, x0[1] * a.softmax_scale);
    o.w[1] = pack2<T>(x0[2] * a.softmax_scale, x0[3] * a.softmax_scale);
    o.w[2] = pack2<T>(x1[0] * a.softmax_scale, x1[1] * a.softmax_scale);
    o.w[3] = pack2<T>(x1[2] * a.softmax_scale, x1[3] * a.softmax_scale);
    *reinterpret_cast<Pack8 *>(reinterpret_cast<uint16_t *>(a.dq) + row * a.dq_row_stride + (int64_t)h * a.dq_head_stride + e) = o;
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

__global__ void zero_f32_kernel(float *p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0.f;
}

template <typename T, int HD>
static int launch_bwd(const fmoba_attn_bwd_args &a, float *dq_accum, hipStream_t s) {
  auto kern = attn_bwd_kernel<T, HD>;
  const size_t smem = BwdSmem<HD>::bytes;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("attn_bwd: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  dim3 grid(ceil_div(a.max_seqlen_k, 64), a.heads, a.batch);
  hipLaunchKernelGGL(kern, grid, dim3(256), smem, s, a, dq_accum);
  return 0;
}

template <typename T>
static int run_bwd(const fmoba_attn_bwd_args &a, float *dq_accum, int phases, hipStream_t s) {
  if (phases & FMOBA_BWD_PREP) {
    int lpr = 1;
    while (lpr * 8 < a.head_dim) lpr <<= 1;
    const int rows_per_block = 256 / lpr;
    hipLaunchKernelGGL(bwd_prep_kernel<T>, dim3(ceil_div(a.max_seqlen_q, rows_per_block), a.heads, a.batch), dim3(256), 0, s, a, dq_accum, lpr);
  }
  if (phases & FMOBA_BWD_MAIN) {
    int rc = a.head_dim <= 64 ? launch_bwd<T, 64>(a, dq_accum, s) : launch_bwd<T, 128>(a, dq_accum, s);
    if (rc) return rc;
  }
  if (phases & FMOBA_BWD_CONVERT) hipLaunchKernelGGL(bwd_convert_kernel<T>, dim3(2048), dim3(256), 0, s, a, (const float *)dq_accum);
  return 0;
}

}  // namespace fmoba

extern "C" size_t fmoba_attn_bwd_workspace_bytes(int32_t total_q, int32_t heads, int32_t head_dim) {
  if (total_q <= 0 || heads <= 0 || head_dim <= 0) return 0;
  return (size_t)total_q * heads * head_dim * 4 + 256;
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
  FMOBA_REQUIRE(a->total_q >= 0 && a->total_k >= 0 && a->max_seqlen_q >= 0 && a->max_seqlen_k >= 0 && a->max_cols >= 0, "negative size");
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
  FMOBA_REQUIRE(a->workspace != nullptr && a->workspace_bytes >= fmoba_attn_bwd_workspace_bytes(a->total_q, a->heads, a->head_dim),
                "attn_bwd: workspace too small");
  float *dq_accum = reinterpret_cast<float *>(((uintptr_t)a->workspace + 255) & ~(uintptr_t)255);
  if (phases & FMOBA_BWD_PREP)
    hipLaunchKernelGGL(zero_f32_kernel, dim3(256), dim3(256), 0, s, a->softmax_d, (int64_t)a->heads * ((int64_t)a->total_q + 128 * (int64_t)a->batch));
  if (a->total_k == 0 || a->max_seqlen_k == 0 || a->max_cols == 0) {
    // no keys: dq = 0
    hipLaunchKernelGGL(zero_rows_kernel, dim3(1024), dim3(256), 0, s, a->dq, (int64_t)a->total_q, a->dq_row_stride, a->heads, a->dq_head_stride, a->head_dim);
    FMOBA_LAUNCH_CHECK("attn_bwd(no keys)");
    return 0;
  }
  FMOBA_REQUIRE(a->k && a->v && a->col_offsets && a->col_nnz && a->row_indices, "attn_bwd: null k/v/CSC pointer");
  int rc = a->dtype == FMOBA_DTYPE_BF16 ? run_bwd<bf16_t>(*a, dq_accum, phases, s) : run_bwd<f16_t>(*a, dq_accum, phases, s);
  if (rc) return rc;
  FMOBA_LAUNCH_CHECK("attn_bwd");
  return 0;
}
