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

namespace fmoba {

constexpr int kSuperRows = 128;
constexpr int kColBatch = 512;

template <int HD>
struct FwdSmem {
  static constexpr int LDQ = HD + 16;  // elements
  static constexpr int LDO = HD + 4;   // floats
  static constexpr size_t oO = 0;
  static constexpr size_t oQ = oO + (size_t)kSuperRows * LDO * 4;
  static constexpr size_t oK = oQ + (size_t)kSuperRows * LDQ * 2;
  static constexpr size_t oV = oK + (size_t)64 * LDQ * 2;
  static constexpr size_t oM = oV + (size_t)64 * LDQ * 2;
  static constexpr size_t oL = oM + kSuperRows * 4;
  static constexpr size_t oRows = oL + kSuperRows * 4;
  static constexpr size_t oLo = oRows + kSuperRows * 4;
  static constexpr size_t oCnt = oLo + kColBatch * 4;
  static constexpr size_t bytes = oCnt + kColBatch * 4;
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

template <typename T, int HD>
__global__ __launch_bounds__(256) void attn_fwd_kernel(fmoba_attn_fwd_args a) {
  typedef FwdSmem<HD> SM;
  constexpr int KS = HD / 16, LDQ = SM::LDQ, LDO = SM::LDO, NDT = HD / 32, VPR = HD / 8;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  float *sO = reinterpret_cast<float *>(smem + SM::oO);
  uint16_t *sQ = reinterpret_cast<uint16_t *>(smem + SM::oQ);
  uint16_t *sK = reinterpret_cast<uint16_t *>(smem + SM::oK);
  uint16_t *sV = reinterpret_cast<uint16_t *>(smem + SM::oV);
  float *sM = reinterpret_cast<float *>(smem + SM::oM);
  float *sL = reinterpret_cast<float *>(smem + SM::oL);
  int *sRows = reinterpret_cast<int *>(smem + SM::oRows);
  int *sLo = reinterpret_cast<int *>(smem + SM::oLo);
  int *sCnt = reinterpret_cast<int *>(smem + SM::oCnt);

  const int sb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int q0 = a.cu_seqlens_q[b], Lq = a.cu_seqlens_q[b + 1] - q0;
  const int m0 = sb * kSuperRows;
  if (m0 >= Lq) return;
  const int k0 = a.cu_seqlens_k[b], Lk = a.cu_seqlens_k[b + 1] - k0;
  const int rows_sb = min(kSuperRows, Lq - m0);
  const int off = Lk - Lq;
  const int D = a.head_dim;
  const int hk = h / (a.heads / a.heads_k);
  const int Bn = a.lg_block_n;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
  const float scale_log2 = a.softmax_scale * 1.4426950408889634f;
  const bool causal = a.is_causal != 0;

  // ---- superblock state -------------------------------------------------------------
  {
    const uint16_t *qp = reinterpret_cast<const uint16_t *>(a.q) + (int64_t)(q0 + m0) * a.q_row_stride + (int64_t)h * a.q_head_stride;
    for (int v = tid; v < kSuperRows * VPR; v += 256) {
      const int row = v / VPR, e = (v - row * VPR) * 8;
      Pack8 x = zero_pack8();
      if (row < rows_sb && e < D) x = ld_global16(qp + (int64_t)row * a.q_row_stride + e);
      *reinterpret_cast<Pack8 *>(sQ + row * LDQ + e) = x;
    }
    for (int v = tid; v < kSuperRows * LDO; v += 256) sO[v] = 0.f;
    if (tid < kSuperRows) {
      sM[tid] = -INFINITY;
      sL[tid] = 0.f;
    }
  }

  int ncols = min((Lk + Bn - 1) / Bn, a.max_cols);
  const int last_rowpos = m0 + rows_sb - 1 + off;  // largest visible key index of the superblock (causal)
  if (causal) ncols = last_rowpos < 0 ? 0 : min(ncols, last_rowpos / Bn + 1);
  const int64_t bh = (int64_t)b * a.heads + h;
  const uint16_t *kp = reinterpret_cast<const uint16_t *>(a.k) + (int64_t)k0 * a.k_row_stride + (int64_t)hk * a.k_head_stride;
  const uint16_t *vp = reinterpret_cast<const uint16_t *>(a.v) + (int64_t)k0 * a.v_row_stride + (int64_t)hk * a.v_head_stride;

  for (int cb = 0; cb < ncols; cb += kColBatch) {
    const int cend = min(ncols, cb + kColBatch);
    __syncthreads();
    // rows of this superblock inside each column's ascending list
    for (int c = cb + tid; c < cend; c += 256) {
      const int nnz = a.col_nnz[bh * a.max_cols + c];
      int lo = 0, cnt = 0;
      if (nnz > 0) {
        const int32_t *list = a.row_indices + a.col_offsets[bh * a.max_cols + c];
        lo = lower_bound_i32(list, nnz, m0);
        const int hi = lo + lower_bound_i32(list + lo, nnz - lo, m0 + kSuperRows);
        cnt = min(hi - lo, kSuperRows);
      }
      sLo[c - cb] = lo;
      sCnt[c - cb] = cnt;
    }
    __syncthreads();

    for (int c = cb; c < cend; ++c) {
      const int n = sCnt[c - cb];
      if (n == 0) continue;
      const int32_t *list = a.row_indices + a.col_offsets[bh * a.max_cols + c] + sLo[c - cb];
      for (int key0 = c * Bn; key0 < min((c + 1) * Bn, Lk); key0 += 64) {
        if (causal && key0 > last_rowpos) break;
        __syncthreads();  // previous tile's readers are done with sK / sV / sRows
        for (int v = tid; v < 64 * VPR; v += 256) {
          const int key = v / VPR, e = (v - key * VPR) * 8;
          Pack8 xk = zero_pack8(), xv = zero_pack8();
          if (key0 + key < Lk && e < D) {
            xk = ld_global16(kp + (int64_t)(key0 + key) * a.k_row_stride + e);
            xv = ld_global16(vp + (int64_t)(key0 + key) * a.v_row_stride + e);
          }
          *reinterpret_cast<Pack8 *>(sK + key * LDQ + e) = xk;
          *reinterpret_cast<Pack8 *>(sV + key * LDQ + e) = xv;
        }
        if (key0 == c * Bn)
          for (int i = tid; i < n; i += 256) sRows[i] = list[i] - m0;
        __syncthreads();

        for (int tile = wave; tile * 32 < n; tile += 4) {
          const int ridx = tile * 32 + (lane & 31);
          const bool valid = ridx < n;
          const int rid = valid ? (sRows[ridx] & (kSuperRows - 1)) : 0;
          Pack8 qf[KS];
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const Pack8 *>(sQ + rid * LDQ + (hh * KS + ks) * 8);
          // S^T tile: register i of key tile kt holds key key0 + 32*kt + acc_row(i, hh) for query rid
          f32x16 s[2];
#pragma unroll
          for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
            for (int i = 0; i < 16; ++i) s[kt][i] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
              const Pack8 af = *reinterpret_cast<const Pack8 *>(sK + (kt * 32 + (lane & 31)) * LDQ + (hh * KS + ks) * 8);
              s[kt] = mfma32<T>(af, qf[ks], s[kt]);
            }
          }
          const int rowpos = m0 + rid + off;
          float mloc = -INFINITY;
#pragma unroll
          for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const int j = key0 + kt * 32 + acc_row(i, hh);
              const bool vis = valid && j < Lk && (!causal || j <= rowpos);
              const float x = vis ? s[kt][i] * scale_log2 : -INFINITY;
              s[kt][i] = x;
              mloc = fmaxf(mloc, x);
            }
          mloc = fmaxf(mloc, shfl_xor32_f(mloc));
          const float m_old = sM[rid], l_old = sL[rid];
          const float m_new = fmaxf(m_old, mloc);
          const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
          const float alpha = exp2f(m_old - m_use);
          float rowsum = 0.f;
#pragma unroll
          for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const float pr = exp2f(s[kt][i] - m_use);
              s[kt][i] = pr;
              rowsum += pr;
            }
          rowsum += shfl_xor32_f(rowsum);
          if (valid && hh == 0) {
            sM[rid] = m_new;
            sL[rid] = l_old * alpha + rowsum;
          }
          // P^T operand: accumulator registers 8s..8s+7 of key tile kt are k-step (kt, s)
          Pack8 pf[2][2];
#pragma unroll
          for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
              for (int w = 0; w < 4; ++w) pf[kt][s2].w[w] = pack2<T>(s[kt][8 * s2 + 2 * w], s[kt][8 * s2 + 2 * w + 1]);
          // O^T += V^T P^T, then read-modify-write the fp32 rows in LDS
#pragma unroll
          for (int dt = 0; dt < NDT; ++dt) {
            f32x16 o;
#pragma unroll
            for (int i = 0; i < 16; ++i) o[i] = 0.f;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
              for (int s2 = 0; s2 < 2; ++s2) {
                const Pack8 vf = tr_frag8(sV, LDQ, kt * 32 + 16 * s2 + 4 * hh, kt * 32 + 16 * s2 + 8 + 4 * hh, dt * 32, lane);
                o = mfma32<T>(vf, pf[kt][s2], o);
              }
            if (valid) {
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
        }
      }
    }
  }
  __syncthreads();

  // ---- epilogue: normalise, write out and the log-sum-exp -----------------------------
  {
    uint16_t *op = reinterpret_cast<uint16_t *>(a.out) + (int64_t)(q0 + m0) * a.o_row_stride + (int64_t)h * a.o_head_stride;
    for (int v = tid; v < rows_sb * VPR; v += 256) {
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
  dim3 grid(ceil_div(a.max_seqlen_q, kSuperRows), a.heads, a.batch);
  hipLaunchKernelGGL(kern, grid, dim3(256), smem, s, a);
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
