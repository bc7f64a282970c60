// Segmented ascending sort of signed int32 keys with 64-bit segment offsets.
//
// Two ways to sort a segment, tried in this order:
//
//  * Bitmap (varlen_sort_bitmap_kernel, the first launch): what row lists are -- keys that do not repeat, in a range
//    of less than 131072 -- is marked in a bitmap in LDS and enumerated in order.  The keys are read once or twice
//    and written once, nothing is staged.  One workgroup of four waves per segment of up to 16384 keys.  A segment
//    the launch cannot finish (a repeated key, a wider range) is marked in the first word of its part of the
//    workspace.
//  * LSD radix sort with 8-bit digits (varlen_sort_kernel), for the marked segments and the longer ones.  The byte
//    positions on which all keys of a segment agree are skipped (row indices of a 8K-token sequence need two passes,
//    not four).  A segment of up to kLdsCapMax keys is read into LDS once (the same pass finds the range of its
//    keys), ping-pongs between two LDS buffers and is written once; longer segments ping-pong between the output
//    and the workspace.  Before its passes a segment tries the bitmap shortcut with the bitmap its LDS buffers can
//    hold (bitmap_sort: up to 32, through HBM 64, times the buffer size), which is what long row lists and
//    the lists of very long sequences take.
//
//    A counting pass is stable without any order between the waves: every wave owns a contiguous block of the keys
//    and a histogram of its own; after the scan, bin d of wave w starts where the keys of smaller digits and the
//    digit-d keys of waves before w end.  A wave then walks its block 64 keys at a time (lanes with equal digits find
//    each other with eight ballots) and advances only its own counters, so the scatter needs no workgroup barrier.
//
//    The LDS a workgroup reserves decides how many of them share a compute unit, so segments are sorted by size
//    class, one launch per class (2048, 8192, 16384 keys per buffer: seven workgroups of four waves, two of eight, one
//    of sixteen per compute unit; the last class also takes the segments that go through HBM).  Every launch looks at
//    the segments 64 at a time with one coalesced load and takes those of its class.
//
// A small launch before the others (sort_cover_kernel) leaves notes behind the keys of the workspace: whether the
// segments tile the buffer (then the output is not cleared first), how many segments are long, and, filled in by the
// bitmap launch, how many segments each radix class has left -- a class without any returns at once.
// Offsets are 64-bit throughout.
#include "fmoba_common.h"

namespace fmoba {

constexpr int kLdsCapMax = 16384;  // keys per LDS buffer of the largest class (2 x 64 KiB)
// the bitmap launch (varlen_sort_bitmap_kernel)
constexpr int kBitmapWords = 4096;       // segments of up to kBitmapMaxKeys keys; the longer ones take the radix passes through HBM
constexpr int kBitmapMaxKeys = 16384;
constexpr uint32_t kSortRetry = 0x52545259u;       // workspace mark of a segment left to the radix launches
constexpr uint32_t kSortDone = 0u;
// What a workspace of the full size holds behind its `total` int32, on a 256-byte boundary.
constexpr int kCoverParts = 16;
struct SortNotes {
  int64_t covered[kCoverParts];     // sums of the lengths of the valid segments, one per workgroup of sort_cover_kernel
  uint32_t n_long[kCoverParts];     // segments of more than kBitmapMaxKeys keys, likewise
  uint32_t left[4];                 // segments the bitmap launch left to radix class 0, 1, 2
};
__host__ __device__ inline int sort_class_of(int64_t n) { return n <= 2048 ? 0 : (n <= 8192 ? 1 : 2); }


// One stable counting pass over keys [0, n): `load(i)` returns the biased key at position i of the
// input, `store(pos, key)` puts a biased key at its position of the output.  hist: [WAVES][256], wsum: [4].
template <int WAVES, typename Load, typename Store>
__device__ __forceinline__ void radix_pass(Load load, Store store, int64_t n, int shift, int *hist, int *wsum) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t per = ((n + WAVES * 64 - 1) / (WAVES * 64)) * 64;  // keys per wave, a multiple of 64
  const int64_t b0 = min(n, wave * per), b1 = min(n, b0 + per);
  int *myh = hist + wave * 256;
  const unsigned long long lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int i = tid; i < WAVES * 256; i += WAVES * 64) hist[i] = 0;
  __syncthreads();
  for (int64_t i = b0 + lane; i < b1; i += 64) atomicAdd(&myh[(load(i) >> shift) & 255u], 1);
  __syncthreads();
  {
    // the first 256 threads, one per bin: exclusive scan of the bin totals, then the waves' shares of the bin in wave order
    int c[WAVES];
    int v = 0, incl = 0;
    if (tid < 256) {
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        c[w] = hist[w * 256 + tid];
        v += c[w];
      }
      incl = v;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int t = __shfl_up(incl, o, 64);
        if (lane >= o) incl += t;
      }
      if (lane == 63) wsum[wave] = incl;
    }
    __syncthreads();
    if (tid < 256) {
      int base = incl - v;
      for (int w = 0; w < wave; ++w) base += wsum[w];
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        hist[w * 256 + tid] = base;
        base += c[w];
      }
    }
  }
  __syncthreads();
  for (int64_t t0 = b0; t0 < b1; t0 += 64) {
    const int64_t i = t0 + lane;
    const bool valid = i < b1;
    const uint32_t k = valid ? load(i) : 0u;
    const uint32_t d = (k >> shift) & 255u;
    unsigned long long peers = __ballot(valid);
#pragma unroll
    for (int bit = 0; bit < 8; ++bit) {
      const bool s = (d >> bit) & 1u;
      const unsigned long long bm = __ballot(valid && s);
      peers &= s ? bm : ~bm;
    }
    const int rank = __popcll(peers & lt);
    int off = 0;
    if (valid && rank == 0) {  // the first lane of each digit advances this wave's counter of the digit
      off = myh[d];
      myh[d] = off + __popcll(peers);
    }
    const int leader = valid ? (__ffsll((long long)peers) - 1) : lane;
    off = __shfl(off, leader, 64);
    if (valid) store(off + rank, k);
  }
  __syncthreads();
}

// The bitmap shortcut inside the radix kernel, for what the bitmap launch (varlen_sort_bitmap_kernel) does not take:
// segments of more than kBitmapMaxKeys keys and ranges wider than its bitmap.  Keys that do not repeat and whose range
// fits a bitmap in the LDS buffers need no radix pass.  Every key sets bit `key - mn`, the set bits are counted per thread (a contiguous block of words each),
// scanned, and enumerated in order.  Returns false, with nothing stored, when a key repeats (the caller then runs
// the radix passes).  `bits` holds nw words, red WAVES.
template <int WAVES, typename Load, typename Store>
__device__ __forceinline__ bool bitmap_sort(Load load, Store store, int64_t n, uint32_t mn, int nw, uint32_t *bits, uint32_t *red) {
  constexpr int kThreads = WAVES * 64;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < nw; i += kThreads) bits[i] = 0u;
  __syncthreads();
  int dup = 0;
  for (int64_t i = tid; i < n; i += kThreads) {
    const uint32_t b = load(i) - mn;
    const uint32_t m = 1u << (b & 31u);
    dup |= (atomicOr(&bits[b >> 5], m) & m) != 0u;
  }
  if (__syncthreads_or(dup)) return false;
  const int per = (nw + kThreads - 1) / kThreads;
  const int w0 = min(nw, tid * per), w1 = min(nw, w0 + per);
  int cnt = 0;
  for (int w = w0; w < w1; ++w) cnt += __popc(bits[w]);
  int incl = cnt;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int t = __shfl_up(incl, o, 64);
    if (lane >= o) incl += t;
  }
  if (lane == 63) red[wave] = (uint32_t)incl;
  __syncthreads();
  int pos = incl - cnt;
  for (int w = 0; w < wave; ++w) pos += (int)red[w];
  for (int w = w0; w < w1; ++w) {
    uint32_t x = bits[w];
    const uint32_t k0 = mn + 32u * (uint32_t)w;
    while (x) {
      store(pos++, k0 + (uint32_t)(__ffs((int)x) - 1));
      x &= x - 1u;
    }
  }
  __syncthreads();
  return true;
}

// range of the biased keys of the workgroup's segment -> number of byte passes (0: all keys equal); mn, mx: the range
template <int WAVES>
__device__ __forceinline__ int radix_passes(uint32_t &mn, uint32_t &mx, uint32_t *red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    mn = min(mn, (uint32_t)__shfl_xor((int)mn, o, 64));
    mx = max(mx, (uint32_t)__shfl_xor((int)mx, o, 64));
  }
  if (lane == 0) {
    red[wave] = mn;
    red[WAVES + wave] = mx;
  }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    mn = min(mn, red[w]);
    mx = max(mx, red[WAVES + w]);
  }
  __syncthreads();  // red is free again
  const uint32_t diff = mn ^ mx;
  return diff == 0u ? 0 : (32 - __clz(diff) + 7) / 8;
}

// Segments of n_lo < n <= n_hi keys: through LDS those of up to CAP keys, through HBM the longer ones (which only the
// last class takes).
// grid: batches of 64 segments x `split` workgroups that share a batch (8 for the smallest class ... 64, i.e. a segment each)
template <int CAP, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void varlen_sort_kernel(const int64_t *starts, const int64_t *ends, int64_t nseg,
                                                                   const int32_t *src, int32_t *dst, int32_t *tmp, int64_t total,
                                                                   int64_t n_lo, int64_t n_hi, int split, const SortNotes *notes) {
  if (notes != nullptr && notes->left[sort_class_of(n_hi)] == 0u) {  // neither a segment the bitmap launch left nor a long one
    uint32_t n_long = 0;
    if (n_hi > kBitmapMaxKeys) {
#pragma unroll
      for (int i = 0; i < kCoverParts; ++i) n_long += notes->n_long[i];
    }
    if (n_long == 0u) return;
  }
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint32_t *bufA = reinterpret_cast<uint32_t *>(smem);
  uint32_t *bufB = bufA + CAP;
  constexpr int kThreads = WAVES * 64;
  int *hist = reinterpret_cast<int *>(bufB + CAP);      // [WAVES][256]
  int *wsum = hist + WAVES * 256;                       // [4]
  uint32_t *red = reinterpret_cast<uint32_t *>(wsum + 4);  // [2 * WAVES]
  const int tid = threadIdx.x, lane = tid & 63;
  const int64_t nbatch = (nseg + 63) / 64;
  if (notes != nullptr) {
    // few segments are left to this launch: a quarter of the workgroups share a batch (every one of them reads the
    // batch's offsets and marks); not fewer, because what is left comes in runs (the long first columns of every head)
    uint32_t mine = notes->left[sort_class_of(n_hi)];
    if (n_hi > kBitmapMaxKeys) {
#pragma unroll
      for (int i = 0; i < kCoverParts; ++i) mine += notes->n_long[i];
    }
    if ((int64_t)mine * 8 < nseg && split >= 4) split /= 4;
  }

  // consecutive workgroups share a batch: the segments of one size class come in runs (the first columns of every
  // head are the long ones), and workgroups are dealt to the eight XCDs in turn
  for (int64_t item = blockIdx.x; item < nbatch * split; item += gridDim.x) {
    const int64_t batch = item / split;
    const int part = (int)(item - batch * split);
    // every wave looks at the same 64 segments, so the set of segments to sort is uniform in the workgroup
    const int64_t sg = batch * 64 + lane;
    int64_t s_l = 0, e_l = 0;
    if (sg < nseg) {
      s_l = starts[sg];
      e_l = ends[sg];
    }
    const int64_t n_l = e_l - s_l;
    bool mine = sg < nseg && n_l > n_lo && n_l <= n_hi && s_l >= 0 && e_l <= total && (lane % split) == part;
    // of the segments the bitmap launch looked at (it marked every one of them), only those it left
    if (mine && n_l <= kBitmapMaxKeys) mine = reinterpret_cast<const uint32_t *>(tmp)[s_l] == kSortRetry;
    unsigned long long todo = __ballot(mine);
    while (todo) {
      const int j = __ffsll((long long)todo) - 1;
      todo &= todo - 1;
      const int64_t s = __shfl(s_l, j, 64);
      const int64_t n = __shfl(n_l, j, 64);
      const uint32_t *in0 = reinterpret_cast<const uint32_t *>(src + s);
      uint32_t *out0 = reinterpret_cast<uint32_t *>(dst + s);
      uint32_t mn = 0xffffffffu, mx = 0u;
      if (n <= CAP) {
        for (int i = tid; i < (int)n; i += kThreads) {
          const uint32_t k = in0[i] ^ 0x80000000u;
          bufA[i] = k;
          mn = min(mn, k);
          mx = max(mx, k);
        }
        const int passes = radix_passes<WAVES>(mn, mx, red);
        if (passes == 0) {
          for (int i = tid; i < (int)n; i += kThreads) out0[i] = bufA[i] ^ 0x80000000u;
          __syncthreads();
          continue;
        }
        if ((uint64_t)(mx - mn) < (uint64_t)CAP * 32u) {  // the bitmap fits bufB (a range too wide for the bitmap launch)
          const uint32_t *c = bufA;
          if (bitmap_sort<WAVES>([&](int64_t i) { return c[i]; }, [&](int pos, uint32_t k) { bufA[pos] = k; }, n, mn,
                                 (int)((mx - mn) / 32u) + 1, bufB, red)) {
            for (int i = tid; i < (int)n; i += kThreads) out0[i] = bufA[i] ^ 0x80000000u;
            __syncthreads();
            continue;
          }
        }
        uint32_t *cur = bufA, *oth = bufB;
        for (int pi = 0; pi < passes; ++pi) {
          const uint32_t *c = cur;
          if (pi == passes - 1) {
            radix_pass<WAVES>([&](int64_t i) { return c[i]; }, [&](int pos, uint32_t k) { out0[pos] = k ^ 0x80000000u; }, n, 8 * pi, hist, wsum);
          } else {
            uint32_t *o = oth;
            radix_pass<WAVES>([&](int64_t i) { return c[i]; }, [&](int pos, uint32_t k) { o[pos] = k; }, n, 8 * pi, hist, wsum);
          }
          uint32_t *t = cur;
          cur = oth;
          oth = t;
        }
      } else {
        for (int64_t i = tid; i < n; i += kThreads) {
          const uint32_t k = in0[i] ^ 0x80000000u;
          mn = min(mn, k);
          mx = max(mx, k);
        }
        const int passes = radix_passes<WAVES>(mn, mx, red);
        if (passes == 0) {
          for (int64_t i = tid; i < n; i += kThreads) out0[i] = in0[i];
          __syncthreads();
          continue;
        }
        if ((uint64_t)(mx - mn) < (uint64_t)CAP * 64u) {  // the bitmap fits the two buffers together
          if (bitmap_sort<WAVES>([&](int64_t i) { return in0[i] ^ 0x80000000u; },
                                 [&](int pos, uint32_t k) { out0[pos] = k ^ 0x80000000u; }, n, mn, (int)((mx - mn) / 32u) + 1, bufA, red))
            continue;
        }
        uint32_t *t1 = reinterpret_cast<uint32_t *>(tmp + s);
        const uint32_t *cur = in0;
        for (int pi = 0; pi < passes; ++pi) {
          const bool first = pi == 0, last = pi == passes - 1;
          uint32_t *o = ((passes - 1 - pi) & 1) ? t1 : out0;  // alternate so that the last pass lands in dst
          const uint32_t *c = cur;
          const uint32_t in_bias = first ? 0x80000000u : 0u, out_bias = last ? 0x80000000u : 0u;
          radix_pass<WAVES>([&](int64_t i) { return c[i] ^ in_bias; }, [&](int64_t pos, uint32_t k) { o[pos] = k ^ out_bias; }, n, 8 * pi, hist,
                     wsum);
          cur = o;
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------
// The first launch of a sort: the bitmap shortcut alone, in a kernel that reserves little LDS (the bitmap of 131072
// bits and a staging area, 24 KiB: six workgroups per compute unit against the one or two of the radix classes' big
// buffers) and never stages the keys.  One workgroup per segment of up to kBitmapMaxKeys keys; longer segments are
// left alone (the last radix class takes them).  A segment the launch cannot finish (a repeated key, a range that
// does not fit) is marked in the first word of its part of the workspace, every other one it looked at is marked
// done, and the radix launches that follow take the marked segments only.
//
// Keys travel in aligned 16-byte loads, sixteen keys per thread in flight at a time; the first batch of the next
// segment is requested before the current one is enumerated.  Keys of one load that fall into the same bitmap word
// are marked together.  A repeated key shows afterwards: fewer bits than keys.
//
// The set bits are enumerated wave by wave: a wave owns a contiguous run of bitmap words, takes 32 of them at a time
// (half a word per lane), puts the positions of their set bits -- below 1024, so 16 bits each -- into its staging
// area at the places an exclusive scan of the bit counts gives, and writes them out with coalesced stores.
// ------------------------------------------------------------------------------------
template <int WAVES, int WORDS>
__global__ __launch_bounds__(WAVES * 64) void varlen_sort_bitmap_kernel(const int64_t *starts, const int64_t *ends, int64_t nseg,
                                                                        const int32_t *src, int32_t *dst, int32_t *tmp, int64_t total,
                                                                        SortNotes *notes) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint32_t *bits = reinterpret_cast<uint32_t *>(smem);                              // [WORDS]
  uint16_t *stage = reinterpret_cast<uint16_t *>(bits + WORDS);                     // [WAVES][1024]
  uint32_t *red = reinterpret_cast<uint32_t *>(stage + WAVES * 1024);               // [2 * WAVES]
  constexpr int kThreads = WAVES * 64;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr int kVec = 4;                       // 16-byte loads per thread and batch
  constexpr int kBatchVecs = kThreads * kVec;   // a batch: 16 keys per thread

  // start and length of segment sg; length 0: nothing to do here (an empty segment, one that leaves the buffer, or a
  // long one, which the radix launch for the segments that go through HBM takes unmarked)
  auto segment = [&](int64_t sg, int64_t &s, int64_t &n) {
    s = 0;
    n = 0;
    if (sg < nseg) {
      const int64_t e = ends[sg];
      s = starts[sg];
      n = (s >= 0 && e <= total && e > s && e - s <= kBitmapMaxKeys) ? e - s : 0;
    }
  };
  // A segment's keys are read with aligned 16-byte loads: `a0` keys come before the first aligned one, `nv` full
  // vectors follow, and the up to six keys before and after them ("edge keys") go one each to threads 0..2 and 4..6.
  auto geometry = [&](int64_t s, int n, int &a0, int &nv, int &edge) {
    a0 = min(n, (int)(((16 - (reinterpret_cast<uintptr_t>(src + s) & 15)) & 15) >> 2));
    nv = (n - a0) >> 2;
    const int tail0 = a0 + 4 * nv;
    edge = -1;
    if (tid < 4) {
      if (tid < a0) edge = tid;
    } else if (tid < 8) {
      if (tail0 + tid - 4 < n) edge = tail0 + tid - 4;
    }
  };
  auto load_vectors = [&](const uint32_t *in0, int a0, int nv, int v0, uint4 (&kv)[kVec]) {
#pragma unroll
    for (int j = 0; j < kVec; ++j) {
      const int v = v0 + tid + kThreads * j;
      kv[j] = v < nv ? *reinterpret_cast<const uint4 *>(in0 + a0 + 4 * v) : make_uint4(0u, 0u, 0u, 0u);
    }
  };
  // the first batch and the edge key of a segment this kernel will try
  auto prefetch = [&](int64_t s, int64_t n64, uint4 (&kv)[kVec], uint32_t &ke) {
    if (n64 <= 0) return;
    int a0, nv, edge;
    geometry(s, (int)n64, a0, nv, edge);
    const uint32_t *in0 = reinterpret_cast<const uint32_t *>(src + s);
    load_vectors(in0, a0, nv, 0, kv);
    ke = edge >= 0 ? in0[edge] : 0u;
  };

  // a workgroup takes every gridDim.x-th segment (the host picks a stride that mixes the long first columns of a head
  // and the short last ones)
  int64_t sg = blockIdx.x, s, n64;
  segment(sg, s, n64);
  uint4 kv[kVec];
  uint32_t ke = 0u;
  prefetch(s, n64, kv, ke);
  while (sg < nseg) {
    const int64_t sg2 = sg + gridDim.x;
    int64_t s2, n2;
    segment(sg2, s2, n2);  // (in flight while this segment is worked on)
    uint32_t *mark = reinterpret_cast<uint32_t *>(tmp + s);
    uint32_t *out0 = reinterpret_cast<uint32_t *>(dst + s);
    bool enumerate = false, retry = false;
    int n = 0, nw = 0;
    uint32_t mn = 0xffffffffu, mx = 0u;
    if (n64 > 0) {
      n = (int)n64;
      const uint32_t *in0 = reinterpret_cast<const uint32_t *>(src + s);
      int a0, nv, edge;
      geometry(s, n, a0, nv, edge);
      const bool in_regs = nv <= kBatchVecs;
      if (edge >= 0) mn = mx = ke ^ 0x80000000u;
      uint4 kw[kVec];
#pragma unroll
      for (int j = 0; j < kVec; ++j) kw[j] = kv[j];
      for (int v0 = 0; v0 < nv; v0 += kBatchVecs) {
        if (v0 > 0) load_vectors(in0, a0, nv, v0, kw);
#pragma unroll
        for (int j = 0; j < kVec; ++j)
          if (v0 + tid + kThreads * j < nv) {
            const uint32_t x = kw[j].x ^ 0x80000000u, y = kw[j].y ^ 0x80000000u, z = kw[j].z ^ 0x80000000u, w = kw[j].w ^ 0x80000000u;
            mn = min(mn, min(min(x, y), min(z, w)));
            mx = max(mx, max(max(x, y), max(z, w)));
          }
      }
#pragma unroll
      for (int o = 32; o >= 1; o >>= 1) {
        mn = min(mn, (uint32_t)__shfl_xor((int)mn, o, 64));
        mx = max(mx, (uint32_t)__shfl_xor((int)mx, o, 64));
      }
      if (lane == 0) {
        red[wave] = mn;
        red[WAVES + wave] = mx;
      }
      __syncthreads();
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        mn = min(mn, red[w]);
        mx = max(mx, red[WAVES + w]);
      }
      if (mx - mn >= (uint32_t)WORDS * 32u) {
        retry = true;
      } else {
        nw = (int)((mx - mn) >> 5) + 1;
        for (int i = tid; i < nw; i += kThreads) bits[i] = 0u;
        __syncthreads();
        // Keys of one vector that fall into the same bitmap word go there together (sorted input: all four), which
        // also spreads the lanes of one instruction over more words.  A repeated key shows afterwards: fewer bits than keys.
        if (edge >= 0) {
          const uint32_t bb = (ke ^ 0x80000000u) - mn;
          atomicOr(&bits[bb >> 5], 1u << (bb & 31u));
        }
        for (int v0 = 0; v0 < nv; v0 += kBatchVecs) {
          if (!in_regs) load_vectors(in0, a0, nv, v0, kw);
#pragma unroll
          for (int j = 0; j < kVec; ++j)
            if (v0 + tid + kThreads * j < nv) {
              const uint32_t b0 = (kw[j].x ^ 0x80000000u) - mn, b1 = (kw[j].y ^ 0x80000000u) - mn, b2 = (kw[j].z ^ 0x80000000u) - mn,
                             b3 = (kw[j].w ^ 0x80000000u) - mn;
              const uint32_t w0 = b0 >> 5, w1 = b1 >> 5, w2 = b2 >> 5, w3 = b3 >> 5;
              uint32_t m0 = 1u << (b0 & 31u), m1 = 1u << (b1 & 31u), m2 = 1u << (b2 & 31u), m3 = 1u << (b3 & 31u);
              if (w1 == w0) {
                m1 |= m0;
                m0 = 0u;
              }
              if (w2 == w1) {
                m2 |= m1;
                m1 = 0u;
              }
              if (w3 == w2) {
                m3 |= m2;
                m2 = 0u;
              }
              if (m0) atomicOr(&bits[w0], m0);
              if (m1) atomicOr(&bits[w1], m1);
              if (m2) atomicOr(&bits[w2], m2);
              atomicOr(&bits[w3], m3);
            }
        }
        enumerate = true;
      }
    }
    prefetch(s2, n2, kv, ke);  // the next segment's keys travel while this one is enumerated
    if (enumerate) {
      __syncthreads();
      // the wave's words: [wb, we), a multiple of 32 of them; a lane takes half a word at a time
      const int per_wave = ((nw + WAVES - 1) / WAVES + 31) & ~31;
      const int wb = wave * per_wave, we = min(nw, wb + per_wave);
      int mine = 0;
      for (int w = wb + lane; w < we; w += 64) mine += __popc(bits[w]);
#pragma unroll
      for (int o = 32; o >= 1; o >>= 1) mine += __shfl_xor(mine, o, 64);
      if (lane == 0) red[wave] = (uint32_t)mine;
      __syncthreads();
      int base = 0, all = 0;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        base += w < wave ? (int)red[w] : 0;
        all += (int)red[w];
      }
      if (all != n) {
        retry = true;  // a key repeats
      } else {
        uint16_t *stg = stage + wave * 1024;
        for (int w0 = wb; w0 < we; w0 += 32) {
          const int w = w0 + (lane >> 1);
          uint32_t x = w < we ? ((bits[w] >> (16 * (lane & 1))) & 0xffffu) : 0u;
          const int c = __popc(x);
          int incl = c;
#pragma unroll
          for (int o = 1; o < 64; o <<= 1) {
            const int t = __shfl_up(incl, o, 64);
            if (lane >= o) incl += t;
          }
          const int round_total = __shfl(incl, 63, 64);
          int at = incl - c;
          while (x) {
            stg[at++] = (uint16_t)(lane * 16 + __ffs((int)x) - 1);
            x &= x - 1u;
          }
          wave_lds_fence();
          const uint32_t k0 = mn + 32u * (uint32_t)w0;
          for (int j = lane; j < round_total; j += 64) out0[base + j] = (k0 + stg[j]) ^ 0x80000000u;
          wave_lds_fence();
          base += round_total;
        }
      }
    }
    if (n64 > 0 && tid == 0) {
      *mark = retry ? kSortRetry : kSortDone;
      if (retry && notes != nullptr) atomicAdd(&notes->left[sort_class_of(n64)], 1u);
    }
    __syncthreads();  // the bitmap and red are free for the next segment
    sg = sg2;
    s = s2;
    n64 = n2;
  }
}

// What the launches of a sort want to know about the segments as a whole (kCoverParts workgroups, a partial result
// each): the sum of the lengths of the valid ones -- segments do not overlap, so a sum that equals the size of the
// buffer means that they tile it and nothing of the output needs to be cleared -- and how many are long; it also
// clears the counts of the segments left to the radix classes.
__global__ __launch_bounds__(256) void sort_cover_kernel(const int64_t *starts, const int64_t *ends, int64_t nseg, int64_t total,
                                                         SortNotes *notes) {
  __shared__ int64_t part[4];
  __shared__ int part_long[4];
  int64_t sum = 0;
  int n_long = 0;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nseg; i += (int64_t)kCoverParts * 256) {
    const int64_t s = starts[i], e = ends[i];
    if (s >= 0 && e <= total && e > s) {
      sum += e - s;
      n_long += (e - s > kBitmapMaxKeys) ? 1 : 0;
    }
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    sum += __shfl_xor(sum, o, 64);
    n_long += __shfl_xor(n_long, o, 64);
  }
  if ((threadIdx.x & 63) == 0) {
    part[threadIdx.x >> 6] = sum;
    part_long[threadIdx.x >> 6] = n_long;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    notes->covered[blockIdx.x] = part[0] + part[1] + part[2] + part[3];
    notes->n_long[blockIdx.x] = (uint32_t)(part_long[0] + part_long[1] + part_long[2] + part_long[3]);
  }
  if (blockIdx.x == 0 && threadIdx.x < 4) notes->left[threadIdx.x] = 0u;
}

// zeros, unless the segments cover all n positions (notes: null, or what sort_cover_kernel found)
__global__ void fill_zero_i32_kernel(int32_t *p, int64_t n, const SortNotes *notes) {
  if (notes != nullptr) {
    int64_t covered = 0;
#pragma unroll
    for (int i = 0; i < kCoverParts; ++i) covered += notes->covered[i];
    if (covered == n) return;
  }
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0;
}

template <int WAVES, int WORDS>
static int launch_sort_bitmap(const int64_t *seg_starts, const int64_t *seg_ends, int64_t num_segments, const int32_t *src, int32_t *dst,
                              int32_t *tmp, int64_t total, SortNotes *notes, hipStream_t s) {
  const size_t smem = (size_t)WORDS * 4 + (size_t)WAVES * 1024 * 2 + 2 * WAVES * 4;
  auto kern = varlen_sort_bitmap_kernel<WAVES, WORDS>;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("varlen_sort: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  // About as many workgroups as the chip holds at a time (LDS: six per compute unit), every one of them a share of the
  // segments.  Row lists come head by head, the long first columns of a head before the short last ones, and a
  // workgroup takes every grid-th segment: with a stride that is a multiple of the columns per head (a power of two,
  // often) a few workgroups would get all the long lists.  1511 is prime and shifts the column by 25 to 57 places per
  // step for 64 ... 2048 columns per head.
  const int64_t resident = 256 * (int64_t)(160 * 1024 / smem);
  const int64_t grid = num_segments < resident ? num_segments : (resident >= 1536 ? 1511 : resident);
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(WAVES * 64), smem, s, seg_starts, seg_ends, num_segments, src, dst, tmp, total, notes);
  FMOBA_LAUNCH_CHECK("varlen_sort(bitmap)");
  return 0;
}

template <int CAP, int WAVES>
static int launch_sort_class(const int64_t *seg_starts, const int64_t *seg_ends, int64_t num_segments, const int32_t *src, int32_t *dst,
                             int32_t *tmp, int64_t total, int64_t n_lo, int64_t n_hi, int split, const SortNotes *notes, hipStream_t s) {
  const size_t smem = (size_t)2 * CAP * 4 + (size_t)WAVES * 256 * 4 + 4 * 4 + 2 * WAVES * 4;
  auto kern = varlen_sort_kernel<CAP, WAVES>;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("varlen_sort: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  const int64_t nbatch = (num_segments + 63) / 64;
  const int64_t items = nbatch * split;
  const int64_t grid = items < 4096 ? items : 4096;  // a workgroup takes every 4096th item: few dispatches, and runs of long segments spread out
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(WAVES * 64), smem, s, seg_starts, seg_ends, num_segments, src, dst, tmp, total, n_lo,
                     n_hi, split, notes);
  FMOBA_LAUNCH_CHECK("varlen_sort");
  return 0;
}

}  // namespace fmoba

// `total` int32 (marks of the bitmap launch, second buffer of the segments sorted through HBM), then, on a 256-byte
// boundary, the notes of the launches (SortNotes)
static inline size_t sort_cover_offset(int64_t total) { return ((size_t)total * 4 + 255) & ~(size_t)255; }
extern "C" size_t fmoba_varlen_sort_workspace_bytes(int64_t total) { return total > 0 ? sort_cover_offset(total) + 256 : 0; }
static_assert(sizeof(fmoba::SortNotes) <= 256, "the notes fit behind the keys");

extern "C" int fmoba_varlen_sort(const int64_t *seg_starts, const int64_t *seg_ends, int64_t num_segments, const int32_t *src,
                                 int32_t *dst, int64_t total, void *workspace, size_t workspace_bytes, void *stream) {
  using namespace fmoba;
  FMOBA_REQUIRE(num_segments >= 0 && total >= 0, "varlen_sort: negative size");
  if (total == 0) return 0;
  FMOBA_REQUIRE(src && dst, "varlen_sort: null src/dst");
  FMOBA_REQUIRE(src != dst, "varlen_sort: the sort is out of place (src == dst)");
  FMOBA_REQUIRE(num_segments == 0 || (seg_starts && seg_ends), "varlen_sort: null segment offsets");
  FMOBA_REQUIRE(workspace != nullptr && workspace_bytes >= (size_t)total * 4, "varlen_sort: workspace must hold %lld int32",
                (long long)total);
  hipStream_t s = (hipStream_t)stream;
  // a workspace of the size fmoba_varlen_sort_workspace_bytes() gives has room for the notes the launches leave each
  // other (an output that the segments tile is not cleared, a radix class without segments returns at once); with
  // `total` int32 only, the output is always cleared and every class looks at every segment
  SortNotes *notes = nullptr;
  if (num_segments > 0 && workspace_bytes >= sort_cover_offset(total) + sizeof(SortNotes)) {
    notes = reinterpret_cast<SortNotes *>(reinterpret_cast<uint8_t *>(workspace) + sort_cover_offset(total));
    hipLaunchKernelGGL(sort_cover_kernel, dim3(kCoverParts), dim3(256), 0, s, seg_starts, seg_ends, num_segments, total, notes);
    FMOBA_LAUNCH_CHECK("varlen_sort(cover)");
  }
  hipLaunchKernelGGL(fill_zero_i32_kernel, dim3(1024), dim3(256), 0, s, dst, total, notes);
  FMOBA_LAUNCH_CHECK("varlen_sort(zero)");
  if (num_segments == 0) return 0;
  int32_t *tmp = reinterpret_cast<int32_t *>(workspace);
  if (int rc = launch_sort_bitmap<4, kBitmapWords>(seg_starts, seg_ends, num_segments, src, dst, tmp, total, notes, s)) return rc;
  if (int rc = launch_sort_class<2048, 4>(seg_starts, seg_ends, num_segments, src, dst, tmp, total, 0, 2048, 8, notes, s)) return rc;
  if (total > 2048)
    if (int rc = launch_sort_class<8192, 8>(seg_starts, seg_ends, num_segments, src, dst, tmp, total, 2048, 8192, 32, notes, s)) return rc;
  if (total > 8192)
    if (int rc = launch_sort_class<kLdsCapMax, 16>(seg_starts, seg_ends, num_segments, src, dst, tmp, total, 8192, INT64_MAX, 64, notes, s))
      return rc;
  return 0;
}
