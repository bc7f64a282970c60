// Per-chunk key mean-pool: km[c] = mean(K[c*B : (c+1)*B]) per (sequence, kv head).
// Pure streaming kernel: every 16-byte vector of K is read exactly once, coalesced along
// the (head, dim) axis, accumulated in fp32 and written once.
#include "fmoba_common.h"

namespace fmoba {

// grid (max_chunks, batch, ceil(vecs / 64)), block 256 = 4 waves.
// A wave owns 64 consecutive 16-byte vectors of the (heads_k*head_dim) axis; the four
// waves of the block split the rows of the chunk and reduce through LDS.
template <typename T>
__global__ __launch_bounds__(256) void mean_pool_kernel(fmoba_mean_pool_args a) {
  const int c = blockIdx.x, b = blockIdx.y;
  const int seq_start = a.cu_seqlens_k[b], seq_end = a.cu_seqlens_k[b + 1];
  const int row0 = seq_start + c * a.chunk;
  if (row0 >= seq_end) return;
  const int n = min(a.chunk, seq_end - row0);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int vecs_per_head = a.head_dim >> 3;
  const int nvec = a.heads_k * vecs_per_head;
  const int vec = blockIdx.z * 64 + lane;
  const bool active = vec < nvec;
  const int head = active ? vec / vecs_per_head : 0;
  const int d0 = active ? (vec - head * vecs_per_head) * 8 : 0;

  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  if (active) {
    const uint16_t *base = reinterpret_cast<const uint16_t *>(a.k) + (int64_t)head * a.k_head_stride + d0;
    int r = wave;
    // four independent 16-byte loads in flight per lane
    for (; r + 12 < n; r += 16) {
      Pack8 p0 = ld_global16(base + (int64_t)(row0 + r) * a.k_row_stride);
      Pack8 p1 = ld_global16(base + (int64_t)(row0 + r + 4) * a.k_row_stride);
      Pack8 p2 = ld_global16(base + (int64_t)(row0 + r + 8) * a.k_row_stride);
      Pack8 p3 = ld_global16(base + (int64_t)(row0 + r + 12) * a.k_row_stride);
      float f0[8], f1[8], f2[8], f3[8];
      unpack8<T>(p0, f0);
      unpack8<T>(p1, f1);
      unpack8<T>(p2, f2);
      unpack8<T>(p3, f3);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] += (f0[i] + f1[i]) + (f2[i] + f3[i]);
    }
    for (; r < n; r += 4) {
      Pack8 p0 = ld_global16(base + (int64_t)(row0 + r) * a.k_row_stride);
      float f0[8];
      unpack8<T>(p0, f0);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] += f0[i];
    }
  }
  __shared__ float red[4][64][9];
#pragma unroll
  for (int i = 0; i < 8; ++i) red[wave][lane][i] = acc[i];
  __syncthreads();
  if (wave == 0 && active) {
    const float nf = (float)n;
    float s[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) s[i] = ((red[0][lane][i] + red[1][lane][i]) + (red[2][lane][i] + red[3][lane][i])) / nf;
    Pack8 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o.w[i] = pack2<T>(s[2 * i], s[2 * i + 1]);
    const int out_row = a.cu_seqlens_km[b] + c;
    uint16_t *dst = reinterpret_cast<uint16_t *>(a.km) + (int64_t)out_row * a.km_row_stride + (int64_t)head * a.km_head_stride + d0;
    *reinterpret_cast<Pack8 *>(dst) = o;
  }
}

// cu_km[b] = sum over b' < b of ceil(len_b' / chunk): one block, every thread a contiguous run of sequences.
__global__ __launch_bounds__(256) void chunk_offsets_kernel(const int32_t *cu, int32_t *cu_km, int batch, int chunk) {
  __shared__ int part[256];
  const int tid = threadIdx.x;
  const int per = (batch + 255) / 256;
  const int lo = min(batch, tid * per), hi = min(batch, lo + per);
  int s = 0;
  for (int b = lo; b < hi; ++b) s += (cu[b + 1] - cu[b] + chunk - 1) / chunk;
  part[tid] = s;
  __syncthreads();
  // inclusive scan over the 256 partial sums
  for (int d = 1; d < 256; d <<= 1) {
    const int v = tid >= d ? part[tid - d] : 0;
    __syncthreads();
    part[tid] += v;
    __syncthreads();
  }
  int run = part[tid] - s;
  for (int b = lo; b < hi; ++b) {
    cu_km[b] = run;
    run += (cu[b + 1] - cu[b] + chunk - 1) / chunk;
  }
  if (tid == 255) cu_km[batch] = part[255];
}

}  // namespace fmoba

extern "C" int fmoba_chunk_offsets(const int32_t *cu_seqlens, int32_t *cu_seqlens_km, int32_t batch, int32_t chunk, void *stream) {
  using namespace fmoba;
  FMOBA_REQUIRE(batch > 0, "chunk_offsets: batch size must be positive");
  FMOBA_REQUIRE(chunk > 0, "chunk_offsets: chunk size must be positive");
  FMOBA_REQUIRE(cu_seqlens && cu_seqlens_km, "chunk_offsets: null pointer");
  hipLaunchKernelGGL(chunk_offsets_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, cu_seqlens, cu_seqlens_km, batch, chunk);
  FMOBA_LAUNCH_CHECK("chunk_offsets");
  return 0;
}

extern "C" int fmoba_mean_pool(const fmoba_mean_pool_args *a, void *stream) {
  using namespace fmoba;
  FMOBA_REQUIRE(a != nullptr, "mean_pool: null args");
  FMOBA_REQUIRE(a->dtype == FMOBA_DTYPE_F16 || a->dtype == FMOBA_DTYPE_BF16, "mean_pool: only fp16 and bf16 are supported");
  FMOBA_REQUIRE(a->batch > 0, "mean_pool: batch size must be positive");
  FMOBA_REQUIRE(a->chunk > 0, "mean_pool: chunk size must be positive");
  FMOBA_REQUIRE(a->head_dim > 0 && a->head_dim % 8 == 0, "mean_pool: head_dim must be a multiple of 8");
  FMOBA_REQUIRE(a->heads_k > 0, "mean_pool: heads_k must be positive");
  if (a->max_chunks <= 0) return 0;
  FMOBA_REQUIRE(a->k && a->km && a->cu_seqlens_k && a->cu_seqlens_km, "mean_pool: null pointer");
  FMOBA_REQUIRE(a->k_row_stride % 8 == 0 && a->k_head_stride % 8 == 0 && a->km_row_stride % 8 == 0 && a->km_head_stride % 8 == 0,
                "mean_pool: strides must be multiples of 8 elements (16-byte vectors)");
  FMOBA_REQUIRE(((uintptr_t)a->k % 16) == 0 && ((uintptr_t)a->km % 16) == 0, "mean_pool: k and km must be 16-byte aligned");
  const int nvec = a->heads_k * (a->head_dim / 8);
  dim3 grid(a->max_chunks, a->batch, ceil_div(nvec, 64));
  FMOBA_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "mean_pool: batch or heads*dim too large for the launch grid");
  hipStream_t s = (hipStream_t)stream;
  if (a->dtype == FMOBA_DTYPE_BF16)
    hipLaunchKernelGGL(mean_pool_kernel<bf16_t>, grid, dim3(256), 0, s, *a);
  else
    hipLaunchKernelGGL(mean_pool_kernel<f16_t>, grid, dim3(256), 0, s, *a);
  FMOBA_LAUNCH_CHECK("mean_pool");
  return 0;
}
