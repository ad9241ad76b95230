// XFC layer step kernels for gfx950 and their C-ABI entry points.
//
//   fwd   : G = fp16( sigmoid(X . W^T) - Y )      Y from per-label-tile positive buckets
//   dx    : dX = scale * G . W                    split over labels, fp32 partials + reduce
//   dw    : dW = G^T . X, consumed in the tile by  M = mu*M + dW + wd*W ; W -= lr*M
// plus the plain six-argument GEMM the reference extension exposes.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <atomic>

#include <type_traits>

#include "../../include/xfc_mi355x.h"
#include "pipe_core.hpp"

namespace xfc {

// ---------------------------------------------------------------------------------------------
// helpers
// ---------------------------------------------------------------------------------------------
// 1 / (1 + 2^(-z log2 e)) with the bare v_exp_f32 / v_rcp_f32: the exponential may flush to zero or
// overflow to infinity at the ends, where the quotient is 1 or 0 either way, so the range fix-up that
// __expf carries (a compare and a select per element) buys nothing here.
__device__ __forceinline__ float sigmoidf_fast(float z) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(z * -1.44269504088896341f));
}

// Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.  Tiles that
// share an operand slice are given ids that land on one XCD next to each other:
// id -> (inner, outer) with `inner` (size n_inner) varying fastest among ids of one XCD.
__device__ __forceinline__ void xcd_map(int id, int n_inner, int& inner, int& outer) {
  const int xcd = id & 7, local = id >> 3;
  inner = local % n_inner;
  outer = (local / n_inner) * 8 + xcd;
}

// ---------------------------------------------------------------------------------------------
// positives: bucket a sparse label list by label tile
// ---------------------------------------------------------------------------------------------
// One workgroup.  Input is CSR (rowptr/colidx, pos_x == nullptr) or COO (pos_x/pos_y int64).
// Output: bucket_ptr[n_tiles+1] and (ent_row, ent_col)[nnz] grouped by col / tile_w.
// Pairs whose row or column is out of range are dropped.  The per-tile counters live in LDS when
// they fit (IN_LDS, n_tiles <= BUCKET_LDS_TILES) and in the global scratch array `cursor` otherwise.
// Both inputs are walked by entry, one coalesced load per thread and pass: a CSR entry finds its row by a
// binary search of the row pointers, which are staged in LDS when they fit (ROWS_IN_LDS) and searched where they
// are otherwise.  (One row per thread, each thread reading its row's labels one after the other, costs as many
// dependent round trips as the longest row has labels: 17 us instead of 11 at 512 rows.)
constexpr int BUCKET_LDS_TILES = 12288;
constexpr int BUCKET_DYN_LDS_MAX = 56 * 1024;  // next to the 4 KB of scan scratch, within the default 64 KB

template <bool IN_LDS, bool ROWS_IN_LDS>
__global__ void __launch_bounds__(1024) bucket_positives_kernel(
    const int32_t* __restrict__ rowptr, const int32_t* __restrict__ colidx, const int64_t* __restrict__ pos_x,
    const int64_t* __restrict__ pos_y, int64_t nnz, int B, int64_t L, int tile_w, int n_tiles,
    int32_t* __restrict__ bucket_ptr, int32_t* __restrict__ cursor_g, int32_t* __restrict__ ent_row,
    int32_t* __restrict__ ent_col) {
  __shared__ int32_t wave_tot[16];
  extern __shared__ int32_t dyn_l[];
  int32_t* cursor = IN_LDS ? dyn_l : cursor_g;
  int32_t* rows_l = dyn_l + (IN_LDS ? n_tiles : 0);  // ROWS_IN_LDS: rowptr[0..B]
  const int32_t* rows = ROWS_IN_LDS ? rows_l : rowptr;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  for (int i = t; i < n_tiles; i += 1024) cursor[i] = 0;
  if constexpr (ROWS_IN_LDS)
    for (int i = t; i <= B; i += 1024) rows_l[i] = rowptr[i];
  __syncthreads();
  // pass 0 counts, pass 1 places
  auto walk = [&](auto visit) {
    if (pos_x) {
      for (int64_t p = t; p < nnz; p += 1024) {
        const int64_t r = pos_x[p], c = pos_y[p];
        if (r >= 0 && r < B && c >= 0 && c < L) visit((int)r, (int)c);
      }
    } else {
      // whatever the row pointers hold, only colidx[0 .. nnz) is read and every entry is visited at most once
      const int64_t p0 = rows[0] > 0 ? rows[0] : 0;
      const int64_t p1 = rows[B] < nnz ? rows[B] : nnz;
      for (int64_t p = p0 + t; p < p1; p += 1024) {
        const int64_t c = colidx[p];
        int lo = 0, hi = B;  // the row b with rowptr[b] <= p < rowptr[b + 1]: first b whose rowptr[b + 1] > p
        while (lo < hi) {
          const int mid = (lo + hi) >> 1;
          if (rows[mid + 1] > p) hi = mid; else lo = mid + 1;
        }
        if (lo < B && c >= 0 && c < L) visit(lo, (int)c);
      }
    }
  };
  walk([&](int, int c) { atomicAdd(&cursor[c / tile_w], 1); });
  __syncthreads();
  // exclusive scan of the per-tile counts: each thread owns `per` consecutive tiles; lanes scan by shuffles,
  // the sixteen waves' totals go through LDS
  const int per = (n_tiles + 1023) / 1024;
  const int lo = t * per, hi = min(n_tiles, lo + per);
  int s = 0;
  for (int i = lo; i < hi; ++i) s += cursor[i];
  int inc = s;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int v = __shfl_up(inc, off, 64);
    if (lane >= off) inc += v;
  }
  if (lane == 63) wave_tot[wave] = inc;
  __syncthreads();
  int before = 0, total = 0;
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    const int v = wave_tot[w];
    if (w < wave) before += v;
    total += v;
  }
  int run = before + inc - s;
  for (int i = lo; i < hi; ++i) {
    const int c = cursor[i];
    bucket_ptr[i] = run;
    cursor[i] = run;
    run += c;
  }
  if (t == 1023) bucket_ptr[n_tiles] = total;
  __syncthreads();
  walk([&](int r, int c) {
    const int at = atomicAdd(&cursor[c / tile_w], 1);
    ent_row[at] = r;
    ent_col[at] = c;
  });
}

// ---------------------------------------------------------------------------------------------
// forward: out = epilogue(alpha * X . W^T + beta * out)
// ---------------------------------------------------------------------------------------------
enum FwdMode { FWD_LINEAR = 0, FWD_SIGMOID = 1, FWD_GRAD = 2, FWD_SIGMOID_PLAIN = 3 };  // PLAIN: alpha 1, beta 0

// Three row-tile heights: 256 rows for training batches, 128 and 64 for small batches (the reference's
// B = 32 plumbing case, --accum micro-batches, the last partial batch of an epoch), where a 256-row tile
// would spend most of its MFMAs on padding.  The label tile is 256 wide in all of them (it is also the
// width of the positives' buckets).  The smaller tiles leave room for a third ring slot.
using FwdCore = PipeCore<256, 256, 64, 2, 4, 2, true, true, false, false, false, 4>;  // one wave per SIMD fetches
using FwdCore128 = PipeCore<128, 256, 64, 2, 4, 3, true, true, false, false, false, 4>;
using FwdCore64 = PipeCore<64, 256, 64, 2, 4, 3, true, true, false, false, false, 4>;
// beside the ring: the tile's positives bitmap, later reused as store staging (8 rows x TN labels per wave)
template <class C>
struct FwdLds {
  static constexpr int STG_HALVES = 8 * C::TN;
  static constexpr int BITMAP_BYTES = C::BN * (C::BM / 32) * 4;
  static constexpr int AUX_BYTES = BITMAP_BYTES > C::NW * STG_HALVES * 2 ? BITMAP_BYTES : C::NW * STG_HALVES * 2;
  static constexpr int BYTES = C::LDS_BYTES + AUX_BYTES;
  static_assert(C::FN % 2 == 0, "staging read-back walks 64-label pieces");
  static_assert(C::BN == 256 && C::NT == 512, "bucket width and workgroup size are shared by all row-tile heights");
  static_assert(BYTES <= 160 * 1024, "LDS budget");
};

struct FwdArgs {
  const half_t* X; int64_t ldx;     // M x K, K-contiguous
  const half_t* W; int64_t ldw;     // N x K, K-contiguous
  half_t* out; int64_t ldo;         // M x n_store, row-major
  int M, N, K, n_store;             // columns N <= c < n_store are written as zero
  float alpha, beta;
  const int32_t* bucket_ptr; const int32_t* ent_row; const int32_t* ent_col;
  float* loss_part;                 // FWD_GRAD with LOSS: one partial sum per workgroup
  int tiles_m, tiles_n, n_ids;      // n_ids = tiles_m * round_up(tiles_n, 8)
};

// Persistent: workgroup w takes tile ids w, w + gridDim.x, ... (gridDim.x a multiple of 8, so an
// id keeps its XCD and the row tiles of one label tile run side by side on one L2).
template <class C, int MODE, bool BETA, bool LOSS = false>
__global__ void __launch_bounds__(C::NT) fwd_kernel(FwdArgs a) {
  constexpr int FWD_STG_HALVES = FwdLds<C>::STG_HALVES;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  half_t* lds = reinterpret_cast<half_t*>(smem_raw);
  // beside the ring: first the tile's positives bitmap, then per-wave store staging
  uint32_t* bm = reinterpret_cast<uint32_t*>(smem_raw + C::LDS_BYTES);
  const int G = gridDim.x, w = blockIdx.x;
  const int n_items = (a.n_ids - w + G - 1) / G;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform, and known to be
  const int wm = wave / C::WN, wn = wave % C::WN;
  half_t* stg = reinterpret_cast<half_t*>(bm) + wave * FWD_STG_HALVES;  // 8 rows x TN labels
  float loss_acc = 0.f;  // LOSS: this lane's share of sum softplus(z) - sum z[positives]

  auto get = [&](int item, typename C::Operand& oa, typename C::Operand& ob, int& kb, int& ke) {
    int mt, nt;
    xcd_map(item * G + w, a.tiles_m, mt, nt);
    oa = typename C::Operand{a.X, a.ldx, mt * C::BM, a.M, a.K};
    ob = typename C::Operand{a.W, a.ldw, nt < a.tiles_n ? nt * C::BN : 0, a.N, a.K};
    kb = 0;
    ke = a.K;
  };
  auto epilogue = [&](int item, float16v (&acc)[C::FM][C::FN]) {
    int mt, nt;
    xcd_map(item * G + w, a.tiles_m, mt, nt);
    if (nt >= a.tiles_n) return;
    const int m0 = mt * C::BM, n0 = nt * C::BN;
    // positives of this tile -> bitmap [label][row word] -> one word per 32x32 block and lane
    uint32_t words[C::FM][C::FN];
#pragma unroll
    for (int fm = 0; fm < C::FM; ++fm)
#pragma unroll
      for (int fn = 0; fn < C::FN; ++fn) words[fm][fn] = 0u;
    bool has_pos = false;
    if constexpr (MODE == FWD_GRAD) {
      // read through the scalar path (the tile id is uniform and the table is read-only here): a vector
      // load would make the compiler wait for every outstanding vector-memory operation before the first
      // use, which includes the next tile's operand fetches that the main loop has just issued
      typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
      const const_i32_ptr bp = (const_i32_ptr)(uintptr_t)a.bucket_ptr;
      const int s = bp[nt], e = bp[nt + 1];
      has_pos = e > s;
      if (has_pos) {
        __syncthreads();  // every wave is done staging the previous tile
        for (int i = threadIdx.x; i < C::BN * (C::BM / 32); i += C::NT) bm[i] = 0u;
        __syncthreads();
        for (int p = s + threadIdx.x; p < e; p += C::NT) {
          const int r = a.ent_row[p] - m0, c = a.ent_col[p] - n0;
          if (r >= 0 && r < C::BM) atomicOr(&bm[c * (C::BM / 32) + (r >> 5)], 1u << (r & 31));
        }
        __syncthreads();
#pragma unroll
        for (int fm = 0; fm < C::FM; ++fm)
#pragma unroll
          for (int fn = 0; fn < C::FN; ++fn)
            words[fm][fn] = bm[(wn * C::TN + fn * 32 + (lane & 31)) * (C::BM / 32) + ((wm * C::TM + fm * 32) >> 5)];
        __syncthreads();  // bitmap consumed: the area is staging again
      }
    }
    const int h = lane >> 5;
    constexpr int CHS = C::TN / 8;  // 16-byte chunks per staged row
    // The per-element work below is the vector ALU cost of the whole tile (the SIMD cannot overlap it
    // with MFMAs), so the rare cases -- a tile holding positives, a tile crossing the label count -- are
    // compiled as separate paths and the common one carries neither.
    int64_t lane_off[C::FN / 2];  // where this lane's 16 bytes of a staged strip go, relative to the strip
#pragma unroll
    for (int p = 0; p < C::FN / 2; ++p) lane_off[p] = (int64_t)((lane + 64 * p) / CHS) * a.ldo + ((lane + 64 * p) % CHS) * 8;
    auto body = [&](auto pos_tag, auto edge_tag) {
      constexpr bool POS = decltype(pos_tag)::value, EDGE = decltype(edge_tag)::value;
      float tile_loss = 0.f;
      if constexpr (LOSS) {
        static_assert(MODE == FWD_GRAD && !BETA, "the loss is that of the plain logits");
        // The loss terms in a pass of their own over the accumulators, one block at a time: interleaved
        // with the sigmoid and the staging below, the scheduler keeps dozens of elements in flight to
        // hide the transcendentals' latency and spills hundreds of registers.
        // softplus(z) = max(z,0) + log(1 + e^-|z|), minus z where the label is positive (dl_base.py:578-583)
#pragma unroll
        for (int fm = 0; fm < C::FM; ++fm)
#pragma unroll
          for (int fn = 0; fn < C::FN; ++fn) {
            const int ecol = n0 + wn * C::TN + fn * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const float v = acc[fm][fn][r];
              float t = fmaxf(v, 0.f) + 0.69314718f * __log2f(1.0f + __expf(-fabsf(v)));
              if constexpr (POS) t -= v * (float)((words[fm][fn] >> c_row(r, lane)) & 1u);
              if constexpr (EDGE) {
                const int erow = m0 + wm * C::TM + fm * 32 + c_row(r, lane);
                t = (erow < a.M && ecol < a.N) ? t : 0.f;
              }
              tile_loss += t;
            }
            __builtin_amdgcn_sched_barrier(0);
          }
      }
#pragma unroll
      for (int fm = 0; fm < C::FM; ++fm) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
#pragma unroll
          for (int fn = 0; fn < C::FN; ++fn) {
            const int ecol = n0 + wn * C::TN + fn * 32 + (lane & 31);
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
              const int r = 4 * q + rr;
              float v = acc[fm][fn][r];
              if constexpr (BETA) {
                v *= a.alpha;
                const int erow = m0 + wm * C::TM + fm * 32 + c_row(r, lane);
                if (erow < a.M && ecol < a.N) v += a.beta * (float)a.out[(int64_t)erow * a.ldo + ecol];
              } else if constexpr (MODE == FWD_SIGMOID) {
                v *= a.alpha;
              }
              if constexpr (MODE != FWD_LINEAR) v = sigmoidf_fast(v);
              if constexpr (POS) v -= (float)((words[fm][fn] >> c_row(r, lane)) & 1u);
              if constexpr (EDGE) { if (ecol >= a.N) v = 0.f; }
              stg[(4 * h + rr) * C::TN + fn * 32 + (lane & 31)] = (half_t)v;
            }
          }
          // the wave's LDS traffic is ordered: its own writes above are visible to the reads below
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
#pragma unroll
          for (int p = 0; p < C::FN / 2; ++p) {
            const int cid = lane + 64 * p;
            const int srow = cid / CHS, sch = cid % CHS;
            const half8 v8 = *reinterpret_cast<const half8*>(stg + srow * C::TN + sch * 8);
            const int row = m0 + wm * C::TM + fm * 32 + 8 * q + srow;
            const int col = n0 + wn * C::TN + sch * 8;
            if (row < a.M) {
              // uniform part + per-lane part computed once per tile: no per-strip vector multiply
              half_t* dst = a.out + ((int64_t)(m0 + wm * C::TM + fm * 32 + 8 * q) * a.ldo + n0 + wn * C::TN) + lane_off[p];
              if (!EDGE || col + 8 <= a.n_store) {
                __builtin_nontemporal_store(v8, reinterpret_cast<half8*>(dst));  // G is not re-read before it leaves the L2
              } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                  if (col + e < a.n_store) dst[e] = v8[e];
              }
            }
          }
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
      }
      if constexpr (LOSS) loss_acc += tile_loss;
    };
    using T = std::true_type;
    using F = std::false_type;
    const bool edge = n0 + C::BN > a.N || (LOSS && m0 + C::BM > a.M);
    if (edge) { if (has_pos) body(T{}, T{}); else body(F{}, T{}); }
    else { if (has_pos) body(T{}, F{}); else body(F{}, F{}); }
  };
  C::run(0, n_items, lds, get, epilogue);
  if constexpr (LOSS) {
    // deterministic: lanes -> wave (butterfly), waves -> workgroup (LDS, fixed order), one partial per workgroup
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) loss_acc += __shfl_xor(loss_acc, off, 64);
    float* red = reinterpret_cast<float*>(bm);
    __syncthreads();
    if (lane == 0) red[wave] = loss_acc;
    __syncthreads();
    if (threadIdx.x == 0) {
      float t = 0.f;
      for (int i = 0; i < C::NW; ++i) t += red[i];
      a.loss_part[w] = t;
    }
  }
}

// Sum of the per-workgroup loss partials, in double, in index order.
__global__ void __launch_bounds__(64) loss_reduce_kernel(const float* __restrict__ part, int n, float* __restrict__ out) {
  double t = 0.0;
  for (int i = threadIdx.x; i < n; i += 64) t += (double)part[i];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) t += __shfl_xor(t, off, 64);
  if (threadIdx.x == 0) *out = (float)t;
}

// ---------------------------------------------------------------------------------------------
// top-K labels per row of X . W^T, never writing the logits (K <= 8)
// ---------------------------------------------------------------------------------------------
// Each workgroup owns 256 query rows and walks every n_groups-th label tile with the forward main loop.
// Per row it keeps the K best (score, label) pairs seen so far, ordered by score descending and label
// ascending (the order iterated torch.max produces: first maximum wins ties).  A finished tile is first
// filtered against each row's current K-th score; survivors (few once the lists have warmed up) go to
// a small per-row buffer that the row's owner thread merges.  If any row overflows its buffer, the tile
// is rescanned exactly, eight columns at a time.  A second kernel merges the groups' lists.
// The workgroups that share a row tile also share what they have learnt: each publishes its rows' K-th
// scores to `bound` (atomic max) and filters against the largest published one as well.  Any published
// value is the K-th score of K real labels, so nothing below it can be in the row's final list; ties with
// it pass (a tying label of lower id may still rank above).  This only makes the filter tighter sooner:
// the lists, and so the results, do not depend on when a bound becomes visible.
constexpr int TOPK_MAX = 8;
constexpr int TOPK_CAP = 6;  // filtered candidates a row can take per tile on the fast path (what LDS leaves room for)
template <class C>
struct TopkLds {
  float list_v[C::BM][TOPK_MAX];
  int32_t list_i[C::BM][TOPK_MAX];
  float tau[C::BM];
  int32_t cnt[C::BM];
  float buf_v[C::BM][TOPK_CAP];  // fast path: candidates; slow path: 8 staged columns (with buf_i)
  int32_t buf_i[C::BM][TOPK_CAP];
  int32_t overflow;
  static constexpr int BYTES = C::LDS_BYTES + (int)(sizeof(float) * C::BM * (2 * TOPK_MAX + 2 + 2 * TOPK_CAP) + 16);
};
static_assert(TopkLds<FwdCore>::BYTES <= 160 * 1024 && TopkLds<FwdCore128>::BYTES <= 160 * 1024 &&
              TopkLds<FwdCore64>::BYTES <= 160 * 1024, "top-K LDS budget");
static_assert(2 * TOPK_CAP >= 8, "the exact rescan stages 8 columns in the candidate buffers");

struct TopkArgs {
  const half_t* X; int64_t ldx;
  const half_t* W; int64_t ldw;
  int M, N, K;          // rows, labels, feature dims
  int topk;
  float* cand_v; int32_t* cand_i;  // [n_groups][M][topk]
  uint32_t* bound;                 // [M] shared lower bounds of the rows' final K-th scores (ordered keys, 0 = none yet)
  int tiles_m, tiles_n, n_groups;
};

// Floats as unsigned keys in the same order (for atomicMax), and back.
__device__ __forceinline__ uint32_t topk_key(float f) {
  const uint32_t b = __float_as_uint(f);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float topk_unkey(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}
// A value strictly below x (x finite or +inf) and as close to it as a normal number allows: "v > below(x)"
// admits every v >= x.  Tiny magnitudes step to a fixed small negative so that no denormal is ever compared.
__device__ __forceinline__ float topk_below(float x) {
  if (fabsf(x) < 1e-30f) return -1e-30f;
  const uint32_t b = __float_as_uint(x);
  return __uint_as_float(x > 0.f ? b - 1u : b + 1u);
}

__device__ __forceinline__ bool topk_better(float av, int ai, float bv, int bi) {
  return av > bv || (av == bv && ai < bi);
}
__device__ __forceinline__ void topk_insert(float* lv, int32_t* li, int K, float v, int i) {
  if (!topk_better(v, i, lv[K - 1], li[K - 1])) return;
  int p = K - 1;
  while (p > 0 && topk_better(v, i, lv[p - 1], li[p - 1])) {
    lv[p] = lv[p - 1];
    li[p] = li[p - 1];
    --p;
  }
  lv[p] = v;
  li[p] = i;
}

// Inlined on purpose: a function that is called waits for every outstanding memory operation on entry
// (the calling convention cannot know what is in flight), which here is the next tile's prefetch.
template <class S_t>
__device__ __forceinline__ void topk_push(S_t& S, int row, float v, int col) {
  const int slot = atomicAdd(&S.cnt[row], 1);
  if (slot < TOPK_CAP) { S.buf_v[row][slot] = v; S.buf_i[row][slot] = col; }
  else S.overflow = 1;
}

template <class C>
__global__ void __launch_bounds__(C::NT) topk_kernel(TopkArgs a) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  half_t* lds = reinterpret_cast<half_t*>(smem_raw);
  TopkLds<C>& S = *reinterpret_cast<TopkLds<C>*>(smem_raw + C::LDS_BYTES);
  // ids are dealt round-robin to XCDs: the row tiles of one label group sit side by side on one XCD
  int mt, grp;
  xcd_map(blockIdx.x, a.tiles_m, mt, grp);
  const int n_items = grp < a.tiles_n ? (a.tiles_n - grp + a.n_groups - 1) / a.n_groups : 0;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform, and known to be
  const int wm = wave / C::WN, wn = wave % C::WN;
  const int m0 = mt * C::BM;
  const int K = a.topk;
  const float NEG_INF = -__builtin_huge_valf();
  for (int t = threadIdx.x; t < C::BM; t += C::NT) {
    for (int j = 0; j < TOPK_MAX; ++j) { S.list_v[t][j] = NEG_INF; S.list_i[t][j] = 0x7fffffff; }
    S.tau[t] = NEG_INF;
    S.cnt[t] = 0;
  }
  if (threadIdx.x == 0) S.overflow = 0;
  __syncthreads();

  auto get = [&](int item, typename C::Operand& oa, typename C::Operand& ob, int& kb, int& ke) {
    const int nt = grp + item * a.n_groups;
    oa = typename C::Operand{a.X, a.ldx, m0, a.M, a.K};
    ob = typename C::Operand{a.W, a.ldw, nt * C::BN, a.N, a.K};
    kb = 0;
    ke = a.K;
  };
  auto epilogue = [&](int item, float16v (&acc)[C::FM][C::FN]) {
    const int nt = grp + item * a.n_groups;
    const int n0 = nt * C::BN;
    const bool ragged = n0 + C::BN > a.N;
    const int h = lane >> 5;
    // the row owners ask for the shared bound now and use it after the filter
    const bool owner = threadIdx.x < C::BM && m0 + (int)threadIdx.x < a.M;
    uint32_t shared_key = 0u;
    if (owner) shared_key = __hip_atomic_load(a.bound + m0 + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // what the filter compares with from the next tile on: the list's K-th score, or just below the shared bound
    auto settle = [&](int t, bool changed) {
      const float mine = S.list_v[t][K - 1];
      if (changed && owner && mine > NEG_INF)
        __hip_atomic_fetch_max(a.bound + m0 + t, topk_key(mine), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const float theirs = shared_key > topk_key(NEG_INF) ? topk_below(topk_unkey(shared_key)) : NEG_INF;
      S.tau[t] = fmaxf(mine, theirs);
      S.cnt[t] = 0;
    };
    // filter against each row's K-th best so far
#pragma unroll
    for (int fm = 0; fm < C::FM; ++fm) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row0 = wm * C::TM + fm * 32 + 8 * q + 4 * h;
        const float4v tau4 = *reinterpret_cast<const float4v*>(&S.tau[row0]);
        // one branch per strip of 4 rows x TN labels: the compares are combined as lane masks, and only a
        // strip in which some lane holds a survivor walks its elements (rare once the lists have warmed up)
        bool any = false;
#pragma unroll
        for (int fn = 0; fn < C::FN; ++fn)
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) any |= acc[fm][fn][4 * q + rr] > tau4[rr];
        if (__builtin_amdgcn_ballot_w64(any) != 0) {
          // opaque on purpose: the compiler otherwise computes the list addresses of all 128 elements when
          // the kernel starts, spills them, and reloads them here behind a wait for every outstanding fetch
          int r0 = row0;
          asm volatile("" : "+v"(r0));
#pragma unroll
          for (int fn = 0; fn < C::FN; ++fn) {
            const int col = n0 + wn * C::TN + fn * 32 + (lane & 31);
            const bool col_ok = !ragged || col < a.N;
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
              const float v = acc[fm][fn][4 * q + rr];
              if (v > tau4[rr] && col_ok) topk_push(S, r0 + rr, v, col);
            }
          }
        }
        asm volatile("" ::: "memory");  // keep the threshold reads of later strips from being hoisted up here
      }
    }
    __syncthreads();
    const bool overflow = S.overflow != 0;
    if (!overflow) {
      if (threadIdx.x < C::BM) {
        const int t = threadIdx.x;
        const int n = S.cnt[t];
        for (int i = 0; i < n; ++i) topk_insert(S.list_v[t], S.list_i[t], K, S.buf_v[t][i], S.buf_i[t][i]);
        settle(t, n != 0);
      }
    } else {
      // exact rescan: stage 8 columns of all 256 rows at a time, each row's owner inserts them
      float* stage = &S.buf_v[0][0];  // 256 x 8 floats: buf_v and buf_i are adjacent
      __syncthreads();
#pragma unroll
      for (int swn = 0; swn < C::WN; ++swn) {
#pragma unroll
        for (int sfn = 0; sfn < C::FN; ++sfn) {
          for (int sg = 0; sg < 4; ++sg) {
            if (wn == swn && ((lane & 31) >> 3) == sg) {
#pragma unroll
              for (int fm = 0; fm < C::FM; ++fm)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                  stage[(wm * C::TM + fm * 32 + c_row(r, lane)) * 8 + (lane & 7)] = acc[fm][sfn][r];
            }
            __syncthreads();
            if (threadIdx.x < C::BM) {
              const int t = threadIdx.x;
              const int cbase = n0 + swn * C::TN + sfn * 32 + sg * 8;
              for (int e = 0; e < 8; ++e)
                if (cbase + e < a.N) topk_insert(S.list_v[t], S.list_i[t], K, stage[t * 8 + e], cbase + e);
            }
            __syncthreads();
          }
        }
      }
      if (threadIdx.x < C::BM) settle(threadIdx.x, true);
      if (threadIdx.x == 0) S.overflow = 0;
    }
    __syncthreads();
  };
  C::run(0, n_items, lds, get, epilogue);
  __syncthreads();
  if (threadIdx.x < C::BM && m0 + threadIdx.x < a.M && grp < a.n_groups) {
    const int64_t o = ((int64_t)grp * a.M + m0 + threadIdx.x) * K;
    for (int j = 0; j < K; ++j) { a.cand_v[o + j] = S.list_v[threadIdx.x][j]; a.cand_i[o + j] = S.list_i[threadIdx.x][j]; }
  }
}

// One wave per row: K rounds of "best pair strictly after the previous pick" over n_groups*K candidates.
__global__ void __launch_bounds__(64) topk_merge_kernel(const float* __restrict__ cand_v, const int32_t* __restrict__ cand_i,
                                                        int M, int n_groups, int K, int64_t numy,
                                                        float* __restrict__ out_v, int64_t* __restrict__ out_i) {
  const int row = blockIdx.x, lane = threadIdx.x;
  const int n = n_groups * K;
  float pv = __builtin_huge_valf();
  int pi = -1;
  for (int r = 0; r < K; ++r) {
    float bv = -__builtin_huge_valf();
    int bi = 0x7fffffff;
    for (int c = lane; c < n; c += 64) {
      const int g = c / K, j = c % K;
      const int64_t o = ((int64_t)g * M + row) * K + j;
      const float v = cand_v[o];
      const int i = cand_i[o];
      const bool after_prev = v < pv || (v == pv && i > pi);
      if (after_prev && topk_better(v, i, bv, bi)) { bv = v; bi = i; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      if (topk_better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    pv = bv;
    pi = bi;
    if (lane == 0) {
      out_v[(int64_t)row * K + r] = bv;
      int64_t idx = bi;
      if (idx >= numy) idx = numy - 1;  // padded labels are clamped, as the reference does
      out_i[(int64_t)row * K + r] = idx;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// top-K for 8 < K <= 8192: exact selection over rows of fp16 logits (one workgroup per row)
// ---------------------------------------------------------------------------------------------
constexpr int SEL_MAX_K = 8192;  // at most half the capacity of the larger sort buffer
constexpr int SEL_THREADS = 1024;
constexpr int SEL_BINS = 2048;  // histogram over the top 11 bits of the 16-bit key
// candidates that are sorted in LDS: 2048 for K <= 1024 (the reference's K = 100 lives here), 16384 (128 KB of
// LDS, one row per CU at a time) for K up to SEL_MAX_K
constexpr int SEL_CAP_SMALL = 2048, SEL_CAP_LARGE = 16384;
constexpr int SEL_SMALL_MAX_K = SEL_CAP_SMALL / 2;
static_assert(2 * SEL_MAX_K <= SEL_CAP_LARGE, "ranks per row");

// fp16 bit pattern -> 16-bit key that orders like the value (-0 counts as +0).
__device__ __forceinline__ uint32_t sel_key(uint32_t h) {
  if (h == 0x8000u) h = 0u;
  return (h & 0x8000u) ? (~h & 0xffffu) : (h | 0x8000u);
}
__device__ __forceinline__ uint32_t sel_unkey(uint32_t k) { return (k & 0x8000u) ? (k & 0x7fffu) : (~k & 0xffffu); }

template <int SEL_CAP>
struct SelLds {
  int hist[SEL_BINS];
  unsigned long long cand[SEL_CAP];
  int wave_tot[SEL_THREADS / 64];
  int n_cand, bin, above;
};

// The K largest of each row of `logits` (rows x L, leading dimension ldl, a multiple of 8), ordered by
// (value descending, label ascending).  Pass 1 histograms the top 11 key bits and finds the bin that
// holds the K-th largest; when at most SEL_CAP elements lie in that bin or above, they are gathered and
// sorted.  Otherwise pass 2 histograms the bin's low 5 bits to get the exact K-th key; elements above it
// are gathered, and the elements equal to it are taken in label order until K are found.
// With sample_stride > 1 the histogram is first taken over every sample_stride-th 16 KB block of the row
// only: the K-th largest of a subset is never above the K-th largest of the row, so every element in that
// bin or above is still a superset of the answer, about K * sample_stride elements; if they fit the sort
// buffer the row has been read 1 + 1/sample_stride times instead of twice, and if not the full passes run.
template <int SEL_CAP>
__global__ void __launch_bounds__(SEL_THREADS) topk_select_kernel(const half_t* __restrict__ logits, int64_t ldl, int L,
                                                                   int64_t numy, int K, int sample_stride,
                                                                   float* __restrict__ out_v,
                                                                   int64_t* __restrict__ out_i) {
  extern __shared__ __attribute__((aligned(16))) unsigned char sel_raw[];
  SelLds<SEL_CAP>& S = *reinterpret_cast<SelLds<SEL_CAP>*>(sel_raw);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint16_t* row = reinterpret_cast<const uint16_t*>(logits) + (int64_t)blockIdx.x * ldl;
  auto for_each_block = [&](int block_stride, auto&& f) {
    for (int64_t i64 = tid * 8; i64 < L; i64 += (int64_t)SEL_THREADS * 8 * block_stride) {
      const int i = (int)i64;
      const uint4v q = *reinterpret_cast<const uint4v*>(row + i);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (i + e < L) f(sel_key((q[e >> 1] >> (16 * (e & 1))) & 0xffffu), i + e);
    }
  };
  auto for_each = [&](auto&& f) { for_each_block(1, f); };
  // f(key, index) for every element of the row whose key is at least kthr.  Almost none is, so two elements at a
  // time are first tested in packed 16-bit arithmetic: flipping the magnitude bits of a negative fp16 pattern gives
  // a signed 16-bit integer x = key - 32768 (except that -0 gives -1 where its key is that of +0, hence the
  // threshold one lower), and min(x, t - 1) != x exactly when x >= t.  Only a 16-byte piece with a hit goes through
  // the exact per-element test.  Two pieces per thread are in flight.
  auto for_each_from = [&](uint32_t kthr, auto&& f) {
    typedef short short2v __attribute__((ext_vector_type(2)));
    const int xq = (int)kthr - 32768 - 1;  // quick test: x >= xq
    const bool all = xq <= -32768;
    const uint32_t t2 = ((uint32_t)(xq - 1) & 0xffffu) * 0x10001u;
    const short2v tv = __builtin_bit_cast(short2v, t2);
    auto piece = [&](const uint4v& q, int i) {
      uint32_t changed = 0u;
#pragma unroll
      for (int e2 = 0; e2 < 4; ++e2) {
        const uint32_t pair = q[e2];  // (a bit cast straight from the element expression reads element 0)
        const short2v h = __builtin_bit_cast(short2v, pair);
        const short2v x = h ^ ((h >> (short2v)(15)) & (short2v)(0x7fff));
        const short2v m = __builtin_elementwise_min(x, tv);
        changed |= __builtin_bit_cast(uint32_t, m) ^ __builtin_bit_cast(uint32_t, x);
      }
      if (all || changed != 0u) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const uint32_t key = sel_key((q[e >> 1] >> (16 * (e & 1))) & 0xffffu);
          if (i + e < L && key >= kthr) f(key, i + e);
        }
      }
    };
    constexpr int64_t STEP = (int64_t)SEL_THREADS * 8;
    for (int64_t i64 = tid * 8; i64 < L; i64 += 2 * STEP) {
      const int i = (int)i64;
      const bool second = i64 + STEP < L;
      const uint4v q0 = *reinterpret_cast<const uint4v*>(row + i);
      uint4v q1 = {0u, 0u, 0u, 0u};
      if (second) q1 = *reinterpret_cast<const uint4v*>(row + i + STEP);
      piece(q0, i);
      if (second) piece(q1, i + (int)STEP);
    }
  };
  auto push = [&](uint32_t key, int idx) {
    const int slot = atomicAdd(&S.n_cand, 1);
    if (slot < SEL_CAP) S.cand[slot] = ((unsigned long long)(0xffffu - key) << 32) | (uint32_t)idx;
  };
  // Finds, over hist[0..nb), the highest bin b with (count in bins above b) + base < K <= that + hist[b];
  // writes S.bin = b and S.above = base + count above b.  nb is a multiple of 64; executed by wave 0.
  auto find_bin = [&](int nb, int base) {
    if (wave == 0) {
      const int per = nb / 64;
      int p = 0;
      for (int j = 0; j < per; ++j) p += S.hist[lane * per + j];
      int suf = p;  // sum over lanes >= this one
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int v = __shfl_down(suf, off, 64);
        if (lane + off < 64) suf += v;
      }
      const unsigned long long m = __ballot(base + suf >= K);
      const int owner = 63 - __builtin_clzll(m | 1ull);  // m != 0 because K <= L
      if (lane == owner) {
        int above = base + suf - p, b = lane * per + per - 1;
        for (; b > lane * per; --b) {
          if (above + S.hist[b] >= K) break;
          above += S.hist[b];
        }
        S.bin = b;
        S.above = above;
      }
    }
  };

  for (int b = tid; b < SEL_BINS; b += SEL_THREADS) S.hist[b] = 0;
  if (tid == 0) S.n_cand = 0;
  __syncthreads();
  bool done = false;
  if (sample_stride > 1) {
    for_each_block(sample_stride, [&](uint32_t key, int) { atomicAdd(&S.hist[key >> 5], 1); });
    __syncthreads();
    find_bin(SEL_BINS, 0);  // the host only asks for a sample that holds at least K elements
    __syncthreads();
    const int sbin = S.bin;
    for_each_from((uint32_t)sbin << 5, [&](uint32_t key, int idx) { push(key, idx); });
    __syncthreads();
    done = S.n_cand <= SEL_CAP;  // counts every push, also those that found the buffer full
    __syncthreads();
    if (!done) {
      for (int b = tid; b < SEL_BINS; b += SEL_THREADS) S.hist[b] = 0;
      if (tid == 0) S.n_cand = 0;
      __syncthreads();
    }
  }
  int bin = 0, above = 0, in_bin = 0;
  if (!done) {
    for_each([&](uint32_t key, int) { atomicAdd(&S.hist[key >> 5], 1); });
    __syncthreads();
    find_bin(SEL_BINS, 0);
    __syncthreads();
    bin = S.bin;
    above = S.above;
    in_bin = S.hist[bin];
    __syncthreads();
  }
  if (done) {
    // the sampled bound already gathered a superset of the answer
  } else if (above + in_bin <= SEL_CAP) {
    for_each_from((uint32_t)bin << 5, [&](uint32_t key, int idx) { push(key, idx); });
  } else {
    if (tid < 64) S.hist[tid] = 0;
    __syncthreads();
    for_each([&](uint32_t key, int) { if ((int)(key >> 5) == bin) atomicAdd(&S.hist[key & 31u], 1); });
    __syncthreads();
    find_bin(64, above);
    __syncthreads();
    const uint32_t thr = ((uint32_t)bin << 5) | (uint32_t)S.bin;
    const int n_gt = S.above, n_eq = S.hist[S.bin];
    __syncthreads();
    if (n_gt + n_eq <= SEL_CAP) {
      for_each_from(thr, [&](uint32_t key, int idx) { push(key, idx); });
    } else {
      // too many copies of the K-th value to sort: those above it first, then its copies in label order
      for_each_from(thr + 1u, [&](uint32_t key, int idx) { push(key, idx); });
      const int need = K - n_gt;
      int taken = 0;
      for (int base = 0; base < L && taken < need; base += SEL_THREADS * 8) {
        const int i = base + tid * 8;
        uint32_t hit = 0;
        if (i < L) {
          const uint4v q = *reinterpret_cast<const uint4v*>(row + i);
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (i + e < L && sel_key((q[e >> 1] >> (16 * (e & 1))) & 0xffffu) == thr) hit |= 1u << e;
        }
        const int c = __builtin_popcount(hit);
        int inc = c;  // inclusive scan over the wave
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
          const int v = __shfl_up(inc, off, 64);
          if (lane >= off) inc += v;
        }
        if (lane == 63) S.wave_tot[wave] = inc;
        __syncthreads();
        int before = 0, total = 0;
        for (int w = 0; w < SEL_THREADS / 64; ++w) {
          const int t = S.wave_tot[w];
          if (w < wave) before += t;
          total += t;
        }
        int rank = taken + before + inc - c;
        for (int e = 0; e < 8; ++e)
          if (hit & (1u << e)) {
            if (rank < need) S.cand[n_gt + rank] = ((unsigned long long)(0xffffu - thr) << 32) | (uint32_t)(i + e);
            ++rank;
          }
        taken += total;
        __syncthreads();
      }
      if (tid == 0) S.n_cand = K;
    }
  }
  __syncthreads();
  const int n = S.n_cand;  // K <= n <= SEL_CAP
  int n2 = 1;
  while (n2 < n) n2 <<= 1;
  for (int i = n + tid; i < n2; i += SEL_THREADS) S.cand[i] = ~0ull;
  __syncthreads();
  for (int k = 2; k <= n2; k <<= 1)
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int i = tid; i < n2; i += SEL_THREADS) {
        const int x = i ^ j;
        if (x > i) {
          const unsigned long long a = S.cand[i], b = S.cand[x];
          const bool up = (i & k) == 0;
          if ((a > b) == up) { S.cand[i] = b; S.cand[x] = a; }
        }
      }
      __syncthreads();
    }
  for (int r = tid; r < K; r += SEL_THREADS) {
    const unsigned long long c = S.cand[r];
    const uint32_t hbits = sel_unkey(0xffffu - (uint32_t)(c >> 32));
    const uint16_t h16 = (uint16_t)hbits;
    half_t h;
    __builtin_memcpy(&h, &h16, 2);
    int64_t idx = (int64_t)(uint32_t)c;
    if (idx >= numy) idx = numy - 1;
    out_v[(int64_t)blockIdx.x * K + r] = (float)h;
    out_i[(int64_t)blockIdx.x * K + r] = idx;
  }
}

// ---------------------------------------------------------------------------------------------
// dX = alpha * G . W (+ beta * dX): split over the label axis, fp32 partials, then a reduce
// ---------------------------------------------------------------------------------------------
using DxCore = PipeCore<256, 256, 64, 2, 4, 2, true, false, true, false, false, 4>;  // accumulators in AGPRs; one wave per SIMD fetches
using DxCore128 = PipeCore<128, 256, 64, 2, 4, 3, true, false, true, false, false, 4>;  // small batches, as in the forward pass
using DxCore64 = PipeCore<64, 256, 64, 2, 4, 3, true, false, true, false, false, 4>;

struct DxArgs {
  const half_t* G; int64_t ldg;   // M x K, K-contiguous (K = labels)
  const half_t* W; int64_t ldw;   // K x N, N-contiguous
  float* part;                    // [splits][M][N]
  int M, N, K;
  int tiles_m, tiles_n, splits, k_per_split;  // k_per_split is a multiple of BK
};

// One workgroup per (output tile, slice of the label axis); the tiles of one slice get ids on one XCD.
template <class C>
__global__ void __launch_bounds__(C::NT) dx_kernel(DxArgs a) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  half_t* lds = reinterpret_cast<half_t*>(smem_raw);
  int tile, split;
  xcd_map(blockIdx.x, a.tiles_m * a.tiles_n, tile, split);
  const int mt = tile % a.tiles_m, nt = tile / a.tiles_m;
  const int m0 = mt * C::BM, n0 = nt * C::BN;
  const int64_t kb64 = (int64_t)split * a.k_per_split;
  const int k_begin = (int)(kb64 < a.K ? kb64 : a.K);
  const int k_end = (int)(kb64 + a.k_per_split < a.K ? kb64 + a.k_per_split : a.K);
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform, and known to be
  const int wm = wave / C::WN, wn = wave % C::WN;
  float* part = a.part + (int64_t)split * a.M * a.N;
  auto store = [&](float16v (&acc)[C::FM][C::FN]) {
#pragma unroll
    for (int fm = 0; fm < C::FM; ++fm)
#pragma unroll
      for (int fn = 0; fn < C::FN; ++fn) {
        const int col = n0 + wn * C::TN + fn * 32 + (lane & 31);
        if (col < a.N) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int row = m0 + wm * C::TM + fm * 32 + c_row(r, lane);
            if (row < a.M) part[(int64_t)row * a.N + col] = acc[fm][fn][r];
          }
        }
      }
  };
  if (k_end <= k_begin) {  // a slice past the end of the label axis contributes zeros
    float16v acc[C::FM][C::FN];
    C::zero(acc);
    store(acc);
    return;
  }
  auto get = [&](int, typename C::Operand& oa, typename C::Operand& ob, int& kb, int& ke) {
    oa = typename C::Operand{a.G, a.ldg, m0, a.M, a.K};
    ob = typename C::Operand{a.W, a.ldw, n0, a.N, a.K};
    kb = k_begin;
    ke = k_end;
  };
  auto epilogue = [&](int, float16v (&acc)[C::FM][C::FN]) { store(acc); };
  C::run(0, 1, lds, get, epilogue);
}

// out[m][n] = alpha * sum_s part[s][m][n] + beta * out[m][n]; one thread per 4 columns.
__global__ void __launch_bounds__(256) dx_reduce_kernel(const float* __restrict__ part, float* __restrict__ out,
                                                        int64_t ldo, int M, int N, int splits, float alpha,
                                                        float beta) {
  const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int nq = N / 4;
  if (q >= (int64_t)M * nq) return;
  const int m = (int)(q / nq), n = (int)(q % nq) * 4;
  float4v s = {0.f, 0.f, 0.f, 0.f};
  const float* p = part + (int64_t)m * N + n;
  for (int i = 0; i < splits; ++i) s += *reinterpret_cast<const float4v*>(p + (int64_t)i * M * N);
  float* o = out + (int64_t)m * ldo + n;
  float4v r = alpha * s;
  if (beta != 0.f) {
    r[0] += beta * o[0]; r[1] += beta * o[1]; r[2] += beta * o[2]; r[3] += beta * o[3];
  }
  o[0] = r[0]; o[1] = r[1]; o[2] = r[2]; o[3] = r[3];
}

// ---------------------------------------------------------------------------------------------
// dW = G^T . X; either written out (fp32, alpha/beta) or consumed by the momentum update
// ---------------------------------------------------------------------------------------------
enum DwMode { DW_OUT = 0, DW_UPDATE = 1, DW_UPDATE_MASTER = 2 };  // MASTER: fp32 master weights and momentum, fp16 copy of W

// 256 labels x 256 dims x 64 batch rows per stage, eight waves of 64 labels x 128 dims, one workgroup per CU.
// (A 128 x 256 x 32 tile with four waves and two workgroups per CU, meant to overlap one workgroup's update with
// the other's GEMM, measured 7-11 % slower at every batch size: its stages move half again as much through LDS
// and the fetch path per flop, and the update's streaming is bound by HBM either way.)
using DwCore = PipeCore<256, 256, 64, 4, 2, 2, false, false, false, false, false, 4>;
constexpr int DW_STAGE_FLOATS = 8 * 64;  // per wave: 8 label rows x 64 dims
constexpr int DW_LDS_BYTES = DwCore::LDS_BYTES + DwCore::NW * DW_STAGE_FLOATS * 4;
static_assert(DW_LDS_BYTES <= 160 * 1024, "LDS budget");
static_assert(DwCore::TM == 64 && DwCore::TN == 128, "the update epilogue walks 64 x 128 wave tiles");
static_assert(DwCore::FN % 2 == 0, "epilogue walks pairs of 32-column blocks");

struct DwArgs {
  const half_t* G; int64_t ldg;   // K x M (batch rows x labels), label-contiguous
  const half_t* X; int64_t ldx;   // K x N, N-contiguous
  int M, N, K;                    // labels, feature dims, batch rows
  int g_cols;                     // readable columns of G per row (>= M, multiple of 8)
  // DW_OUT
  float* out; int64_t ldo; float alpha, beta;
  // DW_UPDATE
  half_t* Wt; int64_t ldw; half_t* Mo; int64_t ldm; float lr, mu, wd;
  // DW_UPDATE_MASTER: fp32 master weights and momentum; Wt above receives the fp16 copy of the new weights
  float* W32; int64_t ldw32; float* M32; int64_t ldm32;
  float* dw_dump; int64_t ld_dump;  // optional copy of dW (may be null)
  int tiles_m, tiles_n, n_ids;      // n_ids = tiles_n * round_up(tiles_m, 8)
};

// Persistent, one workgroup per CU: workgroup w takes tile ids w, w + gridDim.x, ...; the dim tiles of
// one label tile have neighbouring ids on one XCD, so its slice of G is fetched from HBM once.
template <int MODE>
__global__ void __launch_bounds__(DwCore::NT) dw_kernel(DwArgs a) {
  using C = DwCore;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  half_t* lds = reinterpret_cast<half_t*>(smem_raw);
  const int G = gridDim.x, w = blockIdx.x;
  const int n_items = (a.n_ids - w + G - 1) / G;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform, and known to be
  const int wm = wave / C::WN, wn = wave % C::WN;
  float* stage = reinterpret_cast<float*>(smem_raw + C::LDS_BYTES) + wave * DW_STAGE_FLOATS;

  auto get = [&](int item, typename C::Operand& oa, typename C::Operand& ob, int& kb, int& ke) {
    int nt, mt;
    xcd_map(item * G + w, a.tiles_n, nt, mt);
    oa = typename C::Operand{a.G, a.ldg, mt < a.tiles_m ? mt * C::BM : 0, a.g_cols, a.K};
    ob = typename C::Operand{a.X, a.ldx, nt * C::BN, a.N, a.K};
    kb = 0;
    ke = a.K;
  };
  auto epilogue = [&](int item, float16v (&acc)[C::FM][C::FN]) {
    int nt, mt;
    xcd_map(item * G + w, a.tiles_n, nt, mt);
    if (mt >= a.tiles_m) return;
    const int m0 = mt * C::BM, n0 = nt * C::BN;
    const int h = lane >> 5;
    const int srow = lane >> 3, sch = lane & 7;  // staging read: 8 rows x 8 chunks of 8 dims
    // The tile is walked in NS strips of 8 label rows x 64 dims per wave.  In DW_UPDATE mode the strip's
    // W and M pieces are fetched DEPTH strips ahead: one strip in flight per wave leaves HBM latency-bound.
    // They are read once per step, hence non-temporal (measured: 3 % off the kernel).
    constexpr int NS = C::FM * 4 * (C::FN / 2);
    constexpr int DEPTH = MODE == DW_UPDATE_MASTER ? 2 : 4;  // the fp32 pieces take twice the registers per strip (2-6 measure alike)
    auto strip_row = [&](int s) { return m0 + wm * C::TM + (s / (4 * (C::FN / 2))) * 32 + 8 * ((s / (C::FN / 2)) % 4) + srow; };
    auto strip_col = [&](int s) { return n0 + wn * C::TN + (s % (C::FN / 2)) * 64 + sch * 8; };
    // The fp32 arrays (dW out, master W and M) are touched in two 16-byte pieces per lane and strip.  With a lane
    // on 8 consecutive dims each piece's instruction would write every other 16 bytes of a line; there a lane
    // takes dims c .. c+3 and c+32 .. c+35 instead, so that eight lanes cover a whole 128-byte line each time.
    constexpr bool SPLIT = MODE != DW_UPDATE;
    auto split_col = [&](int s) { return n0 + wn * C::TN + (s % (C::FN / 2)) * 64 + sch * 4; };
    half8 wq[DEPTH], mq[DEPTH];
    float4v w32q[DEPTH][2], m32q[DEPTH][2];  // DW_UPDATE_MASTER
    auto fetch32 = [&](int s, float4v (&wv)[2], float4v (&mv)[2]) {
      int row = strip_row(s), c0 = split_col(s), c1 = c0 + 32;
      row = row < a.M ? row : a.M - 1;
      c0 = c0 < a.N ? c0 : a.N - 4;
      c1 = c1 < a.N ? c1 : a.N - 4;
      const float* wp = a.W32 + (int64_t)row * a.ldw32;
      const float* mp = a.M32 + (int64_t)row * a.ldm32;
      wv[0] = __builtin_nontemporal_load(reinterpret_cast<const float4v*>(wp + c0));
      wv[1] = __builtin_nontemporal_load(reinterpret_cast<const float4v*>(wp + c1));
      mv[0] = __builtin_nontemporal_load(reinterpret_cast<const float4v*>(mp + c0));
      mv[1] = __builtin_nontemporal_load(reinterpret_cast<const float4v*>(mp + c1));
    };
    // unconditional (out-of-range strips read the last valid row / column block and are not stored):
    // straight-line loads let the compiler count exactly how many may stay in flight at each use
    auto fetch = [&](int s, half8& wv, half8& mv) {
      int row = strip_row(s), col = strip_col(s);
      row = row < a.M ? row : a.M - 1;
      col = col < a.N ? col : a.N - 8;
      wv = __builtin_nontemporal_load(reinterpret_cast<const half8*>(a.Wt + (int64_t)row * a.ldw + col));
      mv = __builtin_nontemporal_load(reinterpret_cast<const half8*>(a.Mo + (int64_t)row * a.ldm + col));
    };
    if constexpr (MODE == DW_UPDATE) {
#pragma unroll
      for (int s = 0; s < DEPTH && s < NS; ++s) fetch(s, wq[s], mq[s]);
    }
    if constexpr (MODE == DW_UPDATE_MASTER) {
#pragma unroll
      for (int s = 0; s < DEPTH && s < NS; ++s) fetch32(s, w32q[s], m32q[s]);
    }
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const int fm = s / (4 * (C::FN / 2)), q = (s / (C::FN / 2)) % 4, fp = s % (C::FN / 2);
#pragma unroll
      for (int f = 0; f < 2; ++f)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr)
          stage[(4 * h + rr) * 64 + f * 32 + (lane & 31)] = acc[fm][2 * fp + f][4 * q + rr];
      // the wave's own LDS traffic is ordered: the writes above are visible to the reads below
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      const float4v v0 = *reinterpret_cast<const float4v*>(stage + srow * 64 + (SPLIT ? sch * 4 : sch * 8));
      const float4v v1 = *reinterpret_cast<const float4v*>(stage + srow * 64 + (SPLIT ? 32 + sch * 4 : sch * 8 + 4));
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const int row = strip_row(s), col = SPLIT ? split_col(s) : strip_col(s);
      const int col1 = SPLIT ? col + 32 : col + 4;  // first dim of the lane's second piece
      const bool in = row < a.M && col < a.N, in1 = row < a.M && col1 < a.N;
      const float g[8] = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
      if constexpr (MODE == DW_OUT) {
        float* orow = a.out + (int64_t)row * a.ldo;
        float4v o0, o1;
#pragma unroll
        for (int e = 0; e < 4; ++e) { o0[e] = a.alpha * g[e]; o1[e] = a.alpha * g[4 + e]; }
        if (a.beta != 0.f) {  // both pieces' loads before either store
          float4v p0 = {0.f, 0.f, 0.f, 0.f}, p1 = {0.f, 0.f, 0.f, 0.f};
          if (in) p0 = *reinterpret_cast<const float4v*>(orow + col);
          if (in1) p1 = *reinterpret_cast<const float4v*>(orow + col1);
          o0 += a.beta * p0;
          o1 += a.beta * p1;
        }
        if (in) *reinterpret_cast<float4v*>(orow + col) = o0;
        if (in1) *reinterpret_cast<float4v*>(orow + col1) = o1;
      } else if constexpr (MODE == DW_UPDATE_MASTER) {
        // the reference's regime (fp32 parameter and FusedSGD state, dl_base.py:185, main.py:178-179) with the
        // per-step fp16 cast of W (dl_base.py:562) written from the same pass
        float4v wv[2] = {w32q[s % DEPTH][0], w32q[s % DEPTH][1]}, mv[2] = {m32q[s % DEPTH][0], m32q[s % DEPTH][1]};
        if (s + DEPTH < NS) fetch32(s + DEPTH, w32q[s % DEPTH], m32q[s % DEPTH]);
        if (in) {  // the second piece lies 32 dims past the first: when it is inside N, so is the first
          if (a.dw_dump) {
            float* d = a.dw_dump + (int64_t)row * a.ld_dump;
            *reinterpret_cast<float4v*>(d + col) = v0;
            if (in1) *reinterpret_cast<float4v*>(d + col1) = v1;
          }
          half8 w16;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float wf = wv[e >> 2][e & 3];
            const float gg = g[e] + a.wd * wf;
            const float mf = a.mu * mv[e >> 2][e & 3] + gg;
            float wn = wf - a.lr * mf;
            // the copy is the rounding of the stored fp32 weight, as the reference's cast is (dl_base.py:562):
            // the empty statement keeps the compiler from fusing the subtraction and the conversion into one
            // mixed-precision instruction, which would round the exact difference to fp16 in one step
            asm volatile("" : "+v"(wn));
            mv[e >> 2][e & 3] = mf;
            wv[e >> 2][e & 3] = wn;
            w16[e] = (half_t)wn;
          }
          typedef _Float16 half4 __attribute__((ext_vector_type(4)));
          float* wp = a.W32 + (int64_t)row * a.ldw32;
          float* mp = a.M32 + (int64_t)row * a.ldm32;
          half_t* hp = a.Wt + (int64_t)row * a.ldw;
          *reinterpret_cast<float4v*>(mp + col) = mv[0];
          *reinterpret_cast<float4v*>(wp + col) = wv[0];
          *reinterpret_cast<half4*>(hp + col) = half4{w16[0], w16[1], w16[2], w16[3]};
          if (in1) {
            *reinterpret_cast<float4v*>(mp + col1) = mv[1];
            *reinterpret_cast<float4v*>(wp + col1) = wv[1];
            *reinterpret_cast<half4*>(hp + col1) = half4{w16[4], w16[5], w16[6], w16[7]};
          }
        }
      } else {
        half8 wv = wq[s % DEPTH], mv = mq[s % DEPTH];
        if (s + DEPTH < NS) fetch(s + DEPTH, wq[s % DEPTH], mq[s % DEPTH]);
        if (in) {
          if (a.dw_dump) {
            float* d = a.dw_dump + (int64_t)row * a.ld_dump + col;
            *reinterpret_cast<float4v*>(d) = v0;
            *reinterpret_cast<float4v*>(d + 4) = v1;
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float wf = (float)wv[e];
            const float gg = g[e] + a.wd * wf;
            const float mf = a.mu * (float)mv[e] + gg;
            mv[e] = (half_t)mf;
            wv[e] = (half_t)(wf - a.lr * mf);
          }
          *reinterpret_cast<half8*>(a.Mo + (int64_t)row * a.ldm + col) = mv;
          *reinterpret_cast<half8*>(a.Wt + (int64_t)row * a.ldw + col) = wv;
        }
      }
    }
  };
  C::run(0, n_items, lds, get, epilogue);
}

// ---------------------------------------------------------------------------------------------
// any-stride fallback: 64 x 64 output tile per workgroup, 4 x 4 outputs per thread, operands staged through LDS
// as fp32 in 32-deep slabs.  Each output is one fp32 accumulator summed over k in ascending order.  A slab is
// read with consecutive threads along whichever of its two axes has the smaller stride.
// ---------------------------------------------------------------------------------------------
constexpr int GEN_T = 64, GEN_K = 32, GEN_PAD = 4;
__global__ void __launch_bounds__(256) generic_gemm_kernel(const half_t* __restrict__ A, int64_t as0, int64_t as1,
                                                           const half_t* __restrict__ Bm, int64_t bs0, int64_t bs1,
                                                           void* out, int64_t os0, int64_t os1, int M, int N, int K,
                                                           float alpha, float beta, int sigmoid, int out_half) {
  __shared__ __align__(16) float As[GEN_K][GEN_T + GEN_PAD];
  __shared__ __align__(16) float Bs[GEN_K][GEN_T + GEN_PAD];
  const int tiles_n = (N + GEN_T - 1) / GEN_T;
  const int m0 = (int)(blockIdx.x / tiles_n) * GEN_T, n0 = (int)(blockIdx.x % tiles_n) * GEN_T;
  const int t = threadIdx.x, ty = t >> 4, tx = t & 15;
  const bool a_k_fast = (as1 < 0 ? -as1 : as1) <= (as0 < 0 ? -as0 : as0);
  const bool b_k_fast = (bs0 < 0 ? -bs0 : bs0) <= (bs1 < 0 ? -bs1 : bs1);
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += GEN_K) {
#pragma unroll
    for (int j = 0; j < GEN_T * GEN_K / 256; ++j) {
      const int i = t + j * 256;
      int kk = a_k_fast ? i % GEN_K : i / GEN_T, mm = a_k_fast ? i / GEN_K : i % GEN_T;
      As[kk][mm] = (m0 + mm < M && k0 + kk < K) ? (float)A[(int64_t)(m0 + mm) * as0 + (int64_t)(k0 + kk) * as1] : 0.f;
      kk = b_k_fast ? i % GEN_K : i / GEN_T;
      const int nn = b_k_fast ? i / GEN_K : i % GEN_T;
      Bs[kk][nn] = (n0 + nn < N && k0 + kk < K) ? (float)Bm[(int64_t)(k0 + kk) * bs0 + (int64_t)(n0 + nn) * bs1] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GEN_K; ++kk) {
      const float4 av = *reinterpret_cast<const float4*>(&As[kk][ty * 4]);
      const float4 bv = *reinterpret_cast<const float4*>(&Bs[kk][tx * 4]);
      const float a4[4] = {av.x, av.y, av.z, av.w}, b4[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += a4[i] * b4[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
      if (m >= M || n >= N) continue;
      float v = acc[i][j] * alpha;
      const int64_t o = (int64_t)m * os0 + (int64_t)n * os1;
      if (out_half) {
        half_t* p = reinterpret_cast<half_t*>(out) + o;
        if (beta != 0.f) v += beta * (float)*p;
        if (sigmoid) v = sigmoidf_fast(v);
        *p = (half_t)v;
      } else {
        float* p = reinterpret_cast<float*>(out) + o;
        if (beta != 0.f) v += beta * *p;
        if (sigmoid) v = sigmoidf_fast(v);
        *p = v;
      }
    }
}

// Plain copy, 16 bytes per thread step: the known-size kernel that HBM traffic counters are scaled by.
__global__ void __launch_bounds__(256) fill_u32_kernel(uint32_t* __restrict__ dst, uint32_t value, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = value;
}

// bound[r] = key of a value safely below the K-th largest of row r's sample scores.  The sample scores
// are fp16 roundings (half an ulp from the fp32 score at most), so one part in 1024 plus the smallest fp16
// step below the K-th rounded score is below the K-th fp32 score of the sample, hence of the whole row.
__global__ void __launch_bounds__(256) topk_seed_kernel(const float* __restrict__ sample_v, int K, uint32_t* __restrict__ bound,
                                                        int64_t n) {
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= n) return;
  const float x = sample_v[r * K + K - 1];
  const float lo = x - (fabsf(x) * 0.0009765625f + 1.2e-7f);
  bound[r] = (lo == lo && lo > -__builtin_huge_valf()) ? topk_key(lo) : 0u;  // NaN or -inf: no bound
}

__global__ void __launch_bounds__(256) copy_kernel(const uint4v* __restrict__ src, uint4v* __restrict__ dst, int64_t n16) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

// SGD-momentum on an fp32 gradient (used when dW was accumulated over micro-batches).
__global__ void __launch_bounds__(256) sgd_momentum_kernel(half_t* __restrict__ W, half_t* __restrict__ Mo,
                                                           const float* __restrict__ grad, int64_t n8, float lr,
                                                           float mu, float wd) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  half8 w = reinterpret_cast<half8*>(W)[i];
  half8 m = reinterpret_cast<half8*>(Mo)[i];
  const float4v g0 = reinterpret_cast<const float4v*>(grad)[2 * i];
  const float4v g1 = reinterpret_cast<const float4v*>(grad)[2 * i + 1];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float wf = (float)w[e];
    const float gg = (e < 4 ? g0[e] : g1[e - 4]) + wd * wf;
    const float mf = mu * (float)m[e] + gg;
    m[e] = (half_t)mf;
    w[e] = (half_t)(wf - lr * mf);
  }
  reinterpret_cast<half8*>(W)[i] = w;
  reinterpret_cast<half8*>(Mo)[i] = m;
}

// The same on fp32 master weights and momentum, writing the fp16 copy of the new weights as well.
__global__ void __launch_bounds__(256) sgd_momentum_master_kernel(float* __restrict__ W32, float* __restrict__ M32,
                                                                  half_t* __restrict__ W16, const float* __restrict__ grad,
                                                                  int64_t n8, float lr, float mu, float wd) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  float4v w[2] = {reinterpret_cast<float4v*>(W32)[2 * i], reinterpret_cast<float4v*>(W32)[2 * i + 1]};
  float4v m[2] = {reinterpret_cast<float4v*>(M32)[2 * i], reinterpret_cast<float4v*>(M32)[2 * i + 1]};
  const float4v g[2] = {reinterpret_cast<const float4v*>(grad)[2 * i], reinterpret_cast<const float4v*>(grad)[2 * i + 1]};
  half8 h;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float wf = w[e >> 2][e & 3];
    const float mf = mu * m[e >> 2][e & 3] + g[e >> 2][e & 3] + wd * wf;
    float wn = wf - lr * mf;
    asm volatile("" : "+v"(wn));  // the copy is the rounding of the stored fp32 value (see dw_kernel)
    m[e >> 2][e & 3] = mf;
    w[e >> 2][e & 3] = wn;
    h[e] = (half_t)wn;
  }
  reinterpret_cast<float4v*>(W32)[2 * i] = w[0];
  reinterpret_cast<float4v*>(W32)[2 * i + 1] = w[1];
  reinterpret_cast<float4v*>(M32)[2 * i] = m[0];
  reinterpret_cast<float4v*>(M32)[2 * i + 1] = m[1];
  reinterpret_cast<half8*>(W16)[i] = h;
}

}  // namespace xfc

// Scratch of xfc_fwd_grad_csr_static: one copy per GPU, held until the process ends.  In host code the
// name is only a handle for hipGetSymbolAddress; kernels get the per-device address it returns.
static __device__ __align__(256) unsigned char g_static_scratch[XFC_STATIC_SCRATCH_BYTES];

// =============================================================================================
// C ABI
// =============================================================================================
using namespace xfc;

namespace {

inline int ceil_div(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }
inline int64_t round_up(int64_t a, int64_t b) { return (a + b - 1) / b * b; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_launch() {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    fprintf(stderr, "xfc: kernel launch failed: %s\n", hipGetErrorString(e));
    return XFC_ERR_HIP;
  }
  return XFC_OK;
}

constexpr int MAX_DEVICES = 64;
int current_device() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) dev = 0;
  return dev;
}

// Dynamic LDS above the default limit needs the attribute once per kernel and device.
template <auto Kernel>
hipError_t raise_lds_limit(int lds) {
  static std::atomic<bool> raised[MAX_DEVICES];
  const int dev = current_device();
  if (lds <= 48 * 1024 || raised[dev].load(std::memory_order_acquire)) return hipSuccess;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(Kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  if (e == hipSuccess) raised[dev].store(true, std::memory_order_release);
  return e;
}

// Launches Kernel and returns XFC_OK or XFC_ERR_HIP; nothing is launched when the LDS limit cannot be raised.
template <auto Kernel, class A>
int launch_k(dim3 g, dim3 b, int lds, hipStream_t st, const A& args) {
  const hipError_t e = raise_lds_limit<Kernel>(lds);
  if (e != hipSuccess) {
    fprintf(stderr, "xfc: cannot raise the dynamic LDS limit to %d bytes: %s\n", lds, hipGetErrorString(e));
    return XFC_ERR_HIP;
  }
  hipLaunchKernelGGL(Kernel, g, b, lds, st, args);
  return check_launch();
}

int num_cus() {
  static std::atomic<int> n[MAX_DEVICES];
  const int dev = current_device();
  int v = n[dev].load(std::memory_order_relaxed);
  if (v == 0) {
    int cnt = 0;
    if (hipDeviceGetAttribute(&cnt, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cnt <= 0) cnt = 256;
    v = cnt;
    n[dev].store(v, std::memory_order_relaxed);
  }
  return v;
}

// Device address of g_static_scratch on the current device (each GPU holds its own copy at its own
// address), looked up once per device; nullptr with the error printed if the lookup fails.
void* static_scratch_ptr() {
  static std::atomic<void*> ptr[MAX_DEVICES];
  const int dev = current_device();
  void* p = ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_static_scratch));
    if (e != hipSuccess || p == nullptr) {
      fprintf(stderr, "xfc: hipGetSymbolAddress(static scratch) failed: %s\n", hipGetErrorString(e));
      return nullptr;
    }
    ptr[dev].store(p, std::memory_order_release);
  }
  return p;
}

constexpr size_t LOSS_PART_BYTES = 4096;  // one float per forward workgroup (at most 1024)
struct BucketWs {
  int32_t *bucket_ptr, *cursor, *ent_row, *ent_col;
  float* loss_part;
};

size_t bucket_ws_bytes(int64_t L, int64_t nnz) {
  const int64_t n_tiles = round_up(ceil_div(L, FwdCore::BN), 8);
  return (size_t)round_up((n_tiles + 1) * 4, 256) + (size_t)round_up(n_tiles * 4, 256) +
         2 * (size_t)round_up((nnz > 0 ? nnz : 1) * 4, 256) + LOSS_PART_BYTES;
}

BucketWs carve_bucket_ws(void* ws, int64_t L, int64_t nnz) {
  const int64_t n_tiles = round_up(ceil_div(L, FwdCore::BN), 8);
  unsigned char* p = reinterpret_cast<unsigned char*>(ws);
  BucketWs b;
  b.bucket_ptr = reinterpret_cast<int32_t*>(p); p += round_up((n_tiles + 1) * 4, 256);
  b.cursor = reinterpret_cast<int32_t*>(p); p += round_up(n_tiles * 4, 256);
  b.ent_row = reinterpret_cast<int32_t*>(p); p += round_up((nnz > 0 ? nnz : 1) * 4, 256);
  b.ent_col = reinterpret_cast<int32_t*>(p); p += round_up((nnz > 0 ? nnz : 1) * 4, 256);
  b.loss_part = reinterpret_cast<float*>(p);
  return b;
}

// Row-tile height for a batch of M rows (see FwdCore / FwdCore128 / FwdCore64).
inline int row_tile(int64_t M) { return M <= 64 ? 64 : M <= 128 ? 128 : 256; }

template <class C>
int launch_fwd_c(int mode, FwdArgs a, hipStream_t st, float* loss_part, float* loss_out) {
  constexpr int LDS = FwdLds<C>::BYTES;
  a.tiles_m = ceil_div(a.M, C::BM);
  a.tiles_n = ceil_div(a.n_store, C::BN);
  const int64_t ids = (int64_t)a.tiles_m * round_up(a.tiles_n, 8);
  if (ids <= 0) return XFC_OK;
  if (ids > 0x7fffffff) return XFC_ERR_INVALID;
  a.n_ids = (int)ids;
  int64_t grid = (int64_t)round_up(num_cus(), 8);  // one resident workgroup per CU
  if (grid > ids) grid = ids;                    // ids is a multiple of 8
  dim3 g((unsigned)grid), b(C::NT);
  if (mode == FWD_GRAD && loss_part) {
    int rc = launch_k<fwd_kernel<C, FWD_GRAD, false, true>>(g, b, LDS, st, a);
    if (rc) return rc;
    hipLaunchKernelGGL(loss_reduce_kernel, dim3(1), dim3(64), 0, st, loss_part, (int)grid, loss_out);
    return check_launch();
  }
  if (mode == FWD_GRAD) return launch_k<fwd_kernel<C, FWD_GRAD, false>>(g, b, LDS, st, a);
  if (mode == FWD_SIGMOID && a.beta != 0.f) return launch_k<fwd_kernel<C, FWD_SIGMOID, true>>(g, b, LDS, st, a);
  if (mode == FWD_SIGMOID && a.alpha == 1.0f) return launch_k<fwd_kernel<C, FWD_SIGMOID_PLAIN, false>>(g, b, LDS, st, a);
  if (mode == FWD_SIGMOID) return launch_k<fwd_kernel<C, FWD_SIGMOID, false>>(g, b, LDS, st, a);
  return launch_k<fwd_kernel<C, FWD_LINEAR, false>>(g, b, LDS, st, a);
}

int launch_fwd(int mode, const half_t* X, int64_t ldx, const half_t* W, int64_t ldw, half_t* out, int64_t ldo, int M,
               int N, int K, int n_store, float alpha, float beta, const BucketWs* bk, hipStream_t st,
               float* loss_part = nullptr, float* loss_out = nullptr) {
  FwdArgs a;
  a.X = X; a.ldx = ldx; a.W = W; a.ldw = ldw; a.out = out; a.ldo = ldo;
  a.M = M; a.N = N; a.K = K; a.n_store = n_store; a.alpha = alpha; a.beta = beta;
  a.bucket_ptr = bk ? bk->bucket_ptr : nullptr;
  a.ent_row = bk ? bk->ent_row : nullptr;
  a.ent_col = bk ? bk->ent_col : nullptr;
  a.loss_part = loss_part;
  a.tiles_m = a.tiles_n = a.n_ids = 0;
  switch (row_tile(M)) {
    case 64: return launch_fwd_c<FwdCore64>(mode, a, st, loss_part, loss_out);
    case 128: return launch_fwd_c<FwdCore128>(mode, a, st, loss_part, loss_out);
    default: return launch_fwd_c<FwdCore>(mode, a, st, loss_part, loss_out);
  }
}

// Split count for dX: a multiple of 8 slices of the label axis (workgroup ids are dealt round-robin over
// the 8 XCDs, so the tiles of one slice then meet in one L2), each slice a multiple of the k-step.  The
// count minimises a cost model fitted to measurements: workgroups run in rounds of one per CU, every
// workgroup pays a fixed prologue + partial-tile store, and the partial sums are written and read once.
// A stage of a smaller row tile takes proportionally less time.
// With ws_limit the choice is restricted to slice counts whose partial sums fit that many bytes (8 slices, the
// minimum, is always a candidate: the caller checks the final need).  The unrestricted need is not monotone in M
// (a smaller batch may pick more slices), so a workspace sized for one batch serves smaller ones through this limit.
void dx_plan(int M, int N, int K, int& tiles_m, int& tiles_n, int& splits, int& k_per_split,
             size_t ws_limit = ~(size_t)0) {
  const int bm = row_tile(M);
  tiles_m = ceil_div(M, bm);
  tiles_n = ceil_div(N, DxCore::BN);
  const int64_t tiles = (int64_t)tiles_m * tiles_n > 0 ? (int64_t)tiles_m * tiles_n : 1;
  const int cus = num_cus();
  const double nk = (double)ceil_div(K, DxCore::BK);
  const int max_s = (int)round_up(ceil_div(K, DxCore::BK), 8);
  const double STAGE_US = 2.4 * (bm + 256) / 512.0;
  constexpr double FIXED_STAGES = 6.0, PART_BYTES_PER_US = 3.0e6;
  int best = 8;
  double best_cost = 0.0;
  for (int s = 8; s <= 256 && s <= max_s; s += 8) {
    if (s > 8 && (size_t)s * (size_t)M * (size_t)N * 4 > ws_limit) break;
    const double rounds = (double)ceil_div(tiles * s, cus);
    const double cost = rounds * (nk / s + FIXED_STAGES) * STAGE_US + 2.0 * s * (double)M * N * 4.0 / PART_BYTES_PER_US;
    if (s == 8 || cost < best_cost) { best = s; best_cost = cost; }
  }
  k_per_split = (int)round_up(ceil_div(K, best), DxCore::BK);
  splits = best;
}

int launch_dx(const half_t* G, int64_t ldg, const half_t* W, int64_t ldw, float* out, int64_t ldo, int M, int N, int K,
              float alpha, float beta, void* ws, size_t ws_bytes, hipStream_t st) {
  DxArgs a;
  dx_plan(M, N, K, a.tiles_m, a.tiles_n, a.splits, a.k_per_split, ws ? ws_bytes : 0);
  const size_t need = (size_t)a.splits * M * N * 4;
  if (ws == nullptr || ws_bytes < need) return XFC_ERR_WORKSPACE;
  a.G = G; a.ldg = ldg; a.W = W; a.ldw = ldw; a.part = reinterpret_cast<float*>(ws);
  a.M = M; a.N = N; a.K = K;
  const int64_t grid = (int64_t)a.tiles_m * a.tiles_n * a.splits;
  if (grid <= 0 || M <= 0 || N <= 0) return XFC_OK;
  const dim3 g((unsigned)grid), b(DxCore::NT);
  int rc;
  switch (row_tile(M)) {
    case 64: rc = launch_k<dx_kernel<DxCore64>>(g, b, DxCore64::LDS_BYTES, st, a); break;
    case 128: rc = launch_k<dx_kernel<DxCore128>>(g, b, DxCore128::LDS_BYTES, st, a); break;
    default: rc = launch_k<dx_kernel<DxCore>>(g, b, DxCore::LDS_BYTES, st, a); break;
  }
  if (rc) return rc;
  const int64_t nq = (int64_t)M * (N / 4);
  hipLaunchKernelGGL(dx_reduce_kernel, dim3((unsigned)ceil_div(nq, 256)), dim3(256), 0, st, a.part, out, ldo, M, N,
                     a.splits, alpha, beta);
  return check_launch();
}

int launch_dw(int mode, DwArgs a, hipStream_t st) {
  a.tiles_m = ceil_div(a.M, DwCore::BM);
  a.tiles_n = ceil_div(a.N, DwCore::BN);
  const int64_t ids = (int64_t)a.tiles_n * round_up(a.tiles_m, 8);
  if (ids <= 0) return XFC_OK;
  if (ids > 0x7fffffff) return XFC_ERR_INVALID;
  a.n_ids = (int)ids;
  int64_t grid = (int64_t)round_up(num_cus(), 8);  // one resident workgroup per CU
  if (grid > ids) grid = ids / 8 * 8 > 0 ? ids / 8 * 8 : ids;
  const dim3 g((unsigned)grid), b(DwCore::NT);
  if (mode == DW_UPDATE) return launch_k<dw_kernel<DW_UPDATE>>(g, b, DW_LDS_BYTES, st, a);
  if (mode == DW_UPDATE_MASTER) return launch_k<dw_kernel<DW_UPDATE_MASTER>>(g, b, DW_LDS_BYTES, st, a);
  return launch_k<dw_kernel<DW_OUT>>(g, b, DW_LDS_BYTES, st, a);
}

int launch_generic(const void* in1, int64_t as0, int64_t as1, const void* in2, int64_t bs0, int64_t bs1, void* out,
                   int64_t os0, int64_t os1, int M, int N, int K, float alpha, float beta, int sigmoid, int out_half,
                   hipStream_t st) {
  if (M <= 0 || N <= 0) return XFC_OK;
  const int64_t tiles = (int64_t)ceil_div(M, GEN_T) * ceil_div(N, GEN_T);
  if (tiles > 0x7fffffff) return XFC_ERR_INVALID;
  hipLaunchKernelGGL(generic_gemm_kernel, dim3((unsigned)tiles), dim3(256), 0, st,
                     reinterpret_cast<const half_t*>(in1), as0, as1, reinterpret_cast<const half_t*>(in2), bs0, bs1,
                     out, os0, os1, M, N, K, alpha, beta, sigmoid, out_half);
  return check_launch();
}

struct SelArgs {
  const half_t* logits; int64_t ldl; int L; int64_t numy; int K; int stride; float* out_v; int64_t* out_i;
};
template <int CAP>
int launch_select(int rows, const SelArgs& a, hipStream_t st) {
  constexpr int LDS = (int)sizeof(SelLds<CAP>);
  static_assert(LDS <= 160 * 1024, "LDS budget");
  const hipError_t e = raise_lds_limit<topk_select_kernel<CAP>>(LDS);
  if (e != hipSuccess) {
    fprintf(stderr, "xfc: cannot raise the dynamic LDS limit to %d bytes: %s\n", LDS, hipGetErrorString(e));
    return XFC_ERR_HIP;
  }
  hipLaunchKernelGGL(topk_select_kernel<CAP>, dim3((unsigned)rows), dim3(SEL_THREADS), LDS, st, a.logits, a.ldl, a.L, a.numy,
                     a.K, a.stride, a.out_v, a.out_i);
  return check_launch();
}

bool dims_ok(int64_t v) { return v >= 0 && v <= 0x7fffffff; }

}  // namespace

extern "C" {

const char* xfc_strerror(int code) {
  switch (code) {
    case XFC_OK: return "ok";
    case XFC_ERR_INVALID: return "invalid argument (null pointer, negative or oversized dimension)";
    case XFC_ERR_LAYOUT: return "unsupported operand layout: expected row x column (sigmoid), column x row, or row x row";
    case XFC_ERR_ALIGN: return "operand pointer or leading dimension not aligned to 16 bytes";
    case XFC_ERR_WORKSPACE: return "workspace missing or too small";
    case XFC_ERR_HIP: return "HIP runtime error";
    case XFC_ERR_SHAPE: return "operand shapes do not agree";
    case XFC_ERR_LIMIT: return "problem larger than the fixed capacity of this entry point";
    default: return "unknown error";
  }
}

int xfc_abi_version(void) { return XFC_ABI_VERSION; }

int xfc_init(void) {
  hipError_t e = hipSuccess;
  auto keep = [&](hipError_t r) { if (e == hipSuccess) e = r; };
  auto fwd_limits = [&](auto core_tag, auto dx_tag) {
    using C = typename decltype(core_tag)::type;
    using D = typename decltype(dx_tag)::type;
    constexpr int LDS = FwdLds<C>::BYTES;
    keep(raise_lds_limit<fwd_kernel<C, FWD_GRAD, false, true>>(LDS));
    keep(raise_lds_limit<fwd_kernel<C, FWD_GRAD, false>>(LDS));
    keep(raise_lds_limit<fwd_kernel<C, FWD_SIGMOID, true>>(LDS));
    keep(raise_lds_limit<fwd_kernel<C, FWD_SIGMOID, false>>(LDS));
    keep(raise_lds_limit<fwd_kernel<C, FWD_SIGMOID_PLAIN, false>>(LDS));
    keep(raise_lds_limit<fwd_kernel<C, FWD_LINEAR, false>>(LDS));
    keep(raise_lds_limit<topk_kernel<C>>(TopkLds<C>::BYTES));
    keep(raise_lds_limit<dx_kernel<D>>(D::LDS_BYTES));
  };
  fwd_limits(std::type_identity<FwdCore>{}, std::type_identity<DxCore>{});
  fwd_limits(std::type_identity<FwdCore128>{}, std::type_identity<DxCore128>{});
  fwd_limits(std::type_identity<FwdCore64>{}, std::type_identity<DxCore64>{});
  keep(raise_lds_limit<topk_select_kernel<SEL_CAP_SMALL>>((int)sizeof(SelLds<SEL_CAP_SMALL>)));
  keep(raise_lds_limit<topk_select_kernel<SEL_CAP_LARGE>>((int)sizeof(SelLds<SEL_CAP_LARGE>)));
  keep(raise_lds_limit<dw_kernel<DW_UPDATE>>(DW_LDS_BYTES));
  keep(raise_lds_limit<dw_kernel<DW_OUT>>(DW_LDS_BYTES));
  keep(raise_lds_limit<dw_kernel<DW_UPDATE_MASTER>>(DW_LDS_BYTES));
  (void)num_cus();
  if (static_scratch_ptr() == nullptr) return XFC_ERR_HIP;
  if (e != hipSuccess) {
    fprintf(stderr, "xfc: xfc_init failed: %s\n", hipGetErrorString(e));
    return XFC_ERR_HIP;
  }
  return XFC_OK;
}

size_t xfc_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (!dims_ok(M) || !dims_ok(N) || !dims_ok(K)) return 0;
  int tm, tn, s, kps;
  dx_plan((int)M, (int)N, (int)K, tm, tn, s, kps);
  return (size_t)s * M * N * 4;
}

int xfc_gemm(const void* in1, int64_t in1_rows, int64_t in1_cols, int64_t in1_s0, int64_t in1_s1, const void* in2,
             int64_t in2_rows, int64_t in2_cols, int64_t in2_s0, int64_t in2_s1, void* out, int64_t out_rows,
             int64_t out_cols, int64_t out_s0, int64_t out_s1, float alpha, float beta, int apply_sigmoid,
             void* workspace, size_t workspace_bytes, void* stream) {
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int64_t M = out_rows, N = out_cols, K = in2_rows;
  if (!dims_ok(M) || !dims_ok(N) || !dims_ok(K)) return XFC_ERR_INVALID;
  if (in1_rows != M || in1_cols != K || in2_cols != N) return XFC_ERR_SHAPE;
  if (M == 0 || N == 0) return XFC_OK;
  if (!in1 || !in2 || !out) return XFC_ERR_INVALID;
  const bool a_row = in1_s1 == 1, a_col = in1_s0 == 1, b_row = in2_s1 == 1, b_col = in2_s0 == 1;
  if (apply_sigmoid) {
    // out(fp16) = sigmoid(alpha * in1 . in2 + beta * out), in1 row-major, in2 column-major
    if (!(a_row && b_col)) return XFC_ERR_LAYOUT;
    const bool fast = out_s1 == 1 && out_s0 % 8 == 0 && aligned16(out) && in1_s0 % 8 == 0 && in2_s1 % 8 == 0 &&
                      K % 8 == 0 && aligned16(in1) && aligned16(in2) && K > 0;
    if (fast)
      return launch_fwd(FWD_SIGMOID, (const half_t*)in1, in1_s0, (const half_t*)in2, in2_s1, (half_t*)out, out_s0,
                        (int)M, (int)N, (int)K, (int)N, alpha, beta, nullptr, st);
    return launch_generic(in1, in1_s0, in1_s1, in2, in2_s0, in2_s1, out, out_s0, out_s1, (int)M, (int)N, (int)K, alpha,
                          beta, 1, 1, st);
  }
  if (a_col && b_row) {
    // out(fp32) = alpha * in1 . in2 + beta * out, in1 column-major (G^T view), in2 row-major (X)
    const bool fast = out_s1 == 1 && out_s0 % 4 == 0 && aligned16(out) && in1_s1 % 8 == 0 && in2_s0 % 8 == 0 &&
                      N % 8 == 0 && M % 8 == 0 && aligned16(in1) && aligned16(in2) && K > 0;
    if (fast) {
      DwArgs a = {};
      a.G = (const half_t*)in1; a.ldg = in1_s1; a.X = (const half_t*)in2; a.ldx = in2_s0;
      a.M = (int)M; a.N = (int)N; a.K = (int)K; a.g_cols = (int)round_up(M, 8);
      a.out = (float*)out; a.ldo = out_s0; a.alpha = alpha; a.beta = beta;
      return launch_dw(DW_OUT, a, st);
    }
    return launch_generic(in1, in1_s0, in1_s1, in2, in2_s0, in2_s1, out, out_s0, out_s1, (int)M, (int)N, (int)K, alpha,
                          beta, 0, 0, st);
  }
  if (a_row && b_row) {
    // out(fp32) = alpha * in1 . in2 + beta * out, both row-major: contraction over in1's columns
    const bool fast = out_s1 == 1 && in1_s0 % 8 == 0 && in2_s0 % 8 == 0 && N % 8 == 0 && K % 8 == 0 &&
                      aligned16(in1) && aligned16(in2) && K > 0;
    if (fast) {
      return launch_dx((const half_t*)in1, in1_s0, (const half_t*)in2, in2_s0, (float*)out, out_s0, (int)M, (int)N,
                       (int)K, alpha, beta, workspace, workspace_bytes, st);
    }
    return launch_generic(in1, in1_s0, in1_s1, in2, in2_s0, in2_s1, out, out_s0, out_s1, (int)M, (int)N, (int)K, alpha,
                          beta, 0, 0, st);
  }
  return XFC_ERR_LAYOUT;
}

int xfc_logits(const void* X, int64_t ldx, const void* W, int64_t ldw, void* out, int64_t ldo, int64_t B, int64_t L,
               int64_t d, void* stream) {
  if (!dims_ok(B) || !dims_ok(L) || !dims_ok(d)) return XFC_ERR_INVALID;
  if (B == 0 || L == 0) return XFC_OK;
  if (!X || !W || !out || d <= 0) return XFC_ERR_INVALID;
  if (ldx % 8 || ldw % 8 || ldo % 8 || d % 8 || !aligned16(X) || !aligned16(W) || !aligned16(out))
    return XFC_ERR_ALIGN;
  if (ldo < L) return XFC_ERR_SHAPE;
  return launch_fwd(FWD_LINEAR, (const half_t*)X, ldx, (const half_t*)W, ldw, (half_t*)out, ldo, (int)B, (int)L, (int)d,
                    (int)L, 1.0f, 0.0f, nullptr, reinterpret_cast<hipStream_t>(stream));
}

size_t xfc_fwd_grad_workspace_bytes(int64_t L, int64_t nnz) {
  if (!dims_ok(L) || nnz < 0) return 0;
  return bucket_ws_bytes(L, nnz);
}

static int fwd_grad_impl(const void* X, int64_t ldx, const void* W, int64_t ldw, const int32_t* rowptr,
                         const int32_t* colidx, const int64_t* pos_x, const int64_t* pos_y, int64_t nnz, void* G,
                         int64_t ldg, int64_t B, int64_t L, int64_t d, float* loss, void* ws, size_t ws_bytes,
                         hipStream_t st) {
  if (!dims_ok(B) || !dims_ok(L) || !dims_ok(d) || nnz < 0 || nnz > 0x7fffffff) return XFC_ERR_INVALID;
  if (B == 0 || L == 0) return XFC_OK;
  if (!X || !W || !G || d <= 0) return XFC_ERR_INVALID;
  if (nnz > 0 && !((rowptr && colidx) || (pos_x && pos_y))) return XFC_ERR_INVALID;
  if (ldx % 8 || ldw % 8 || ldg % 8 || d % 8 || !aligned16(X) || !aligned16(W) || !aligned16(G))
    return XFC_ERR_ALIGN;
  if (ldg < L) return XFC_ERR_SHAPE;
  if (!ws || ws_bytes < bucket_ws_bytes(L, nnz)) return XFC_ERR_WORKSPACE;
  BucketWs bk = carve_bucket_ws(ws, L, nnz);
  const int n_tiles = (int)round_up(ceil_div(L, FwdCore::BN), 8);
  const bool coo = pos_x != nullptr;
  const bool in_lds = n_tiles <= BUCKET_LDS_TILES;
  const size_t dyn_tiles = in_lds ? (size_t)n_tiles * 4 : 0;
  const bool rows_in_lds = !coo && dyn_tiles + ((size_t)B + 1) * 4 <= (size_t)BUCKET_DYN_LDS_MAX;
  const size_t dyn = dyn_tiles + (rows_in_lds ? ((size_t)B + 1) * 4 : 0);
  auto launch_bucket = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(1), dim3(1024), dyn, st, coo ? nullptr : rowptr, coo ? nullptr : colidx,
                       coo ? pos_x : nullptr, coo ? pos_y : nullptr, nnz, (int)B, L, FwdCore::BN, n_tiles, bk.bucket_ptr,
                       bk.cursor, bk.ent_row, bk.ent_col);
  };
  if (in_lds && rows_in_lds) launch_bucket(bucket_positives_kernel<true, true>);
  else if (in_lds) launch_bucket(bucket_positives_kernel<true, false>);
  else if (rows_in_lds) launch_bucket(bucket_positives_kernel<false, true>);
  else launch_bucket(bucket_positives_kernel<false, false>);
  int rc = check_launch();
  if (rc) return rc;
  // label columns L .. round_up(L, 8) are written as zero so that G can be read in 16-byte
  // pieces along the label axis by the dX and dW kernels (ldg is a multiple of 8, so they exist)
  const int64_t n_store = round_up(L, 8);
  return launch_fwd(FWD_GRAD, (const half_t*)X, ldx, (const half_t*)W, ldw, (half_t*)G, ldg, (int)B, (int)L, (int)d,
                    (int)n_store, 1.0f, 0.0f, &bk, st, loss ? bk.loss_part : nullptr, loss);
}

int xfc_fwd_grad_csr(const void* X, int64_t ldx, const void* W, int64_t ldw, const int32_t* rowptr,
                     const int32_t* colidx, void* G, int64_t ldg, int64_t B, int64_t L, int64_t d, int64_t nnz,
                     float* loss, void* workspace, size_t workspace_bytes, void* stream) {
  if (B > 0 && !rowptr) return XFC_ERR_INVALID;
  return fwd_grad_impl(X, ldx, W, ldw, rowptr, colidx, nullptr, nullptr, nnz, G, ldg, B, L, d, loss, workspace,
                       workspace_bytes, reinterpret_cast<hipStream_t>(stream));
}

int xfc_fwd_grad_csr_static(const void* X, int64_t ldx, const void* W, int64_t ldw, const int32_t* rowptr,
                            const int32_t* colidx, void* G, int64_t ldg, int64_t B, int64_t L, int64_t d, int64_t nnz,
                            float* loss, void* stream) {
  if (B > 0 && !rowptr) return XFC_ERR_INVALID;
  if (!dims_ok(L) || nnz < 0) return XFC_ERR_INVALID;
  if (bucket_ws_bytes(L, nnz) > (size_t)XFC_STATIC_SCRATCH_BYTES) {
    fprintf(stderr, "xfc_fwd_grad_csr_static: L = %lld labels with %lld positives need %zu bytes of scratch, the static "
                    "buffer holds %d; use xfc_fwd_grad_csr with a caller workspace\n",
            (long long)L, (long long)nnz, bucket_ws_bytes(L, nnz), XFC_STATIC_SCRATCH_BYTES);
    return XFC_ERR_LIMIT;
  }
  void* scratch = static_scratch_ptr();
  if (scratch == nullptr) return XFC_ERR_HIP;
  // every table in the scratch is rebuilt from its first entry by the bucket pass, so nothing of the
  // previous call's contents survives into this one
  return fwd_grad_impl(X, ldx, W, ldw, rowptr, colidx, nullptr, nullptr, nnz, G, ldg, B, L, d, loss, scratch,
                       (size_t)XFC_STATIC_SCRATCH_BYTES, reinterpret_cast<hipStream_t>(stream));
}

int xfc_fwd_grad_coo(const void* X, int64_t ldx, const void* W, int64_t ldw, const int64_t* pos_x, const int64_t* pos_y,
                     int64_t nnz, void* G, int64_t ldg, int64_t B, int64_t L, int64_t d, float* loss, void* workspace,
                     size_t workspace_bytes, void* stream) {
  if (nnz > 0 && !(pos_x && pos_y)) return XFC_ERR_INVALID;
  // an empty list still goes through the bucket pass (it zeroes the bucket table)
  static const int64_t dummy = 0;
  return fwd_grad_impl(X, ldx, W, ldw, nullptr, nullptr, pos_x ? pos_x : &dummy, pos_y ? pos_y : &dummy, nnz, G, ldg, B,
                       L, d, loss, workspace, workspace_bytes, reinterpret_cast<hipStream_t>(stream));
}

size_t xfc_dx_workspace_bytes(int64_t B, int64_t L, int64_t d) { return xfc_gemm_workspace_bytes(B, d, L); }

int xfc_dx(const void* G, int64_t ldg, const void* W, int64_t ldw, float* dX, int64_t lddx, int64_t B, int64_t L,
           int64_t d, float scale, void* workspace, size_t workspace_bytes, void* stream) {
  if (!dims_ok(B) || !dims_ok(L) || !dims_ok(d)) return XFC_ERR_INVALID;
  if (B == 0 || d == 0) return XFC_OK;
  if (!G || !W || !dX) return XFC_ERR_INVALID;
  if (ldg % 8 || ldw % 8 || d % 8 || !aligned16(G) || !aligned16(W)) return XFC_ERR_ALIGN;
  if (ldg < round_up(L, 8)) return XFC_ERR_SHAPE;
  return launch_dx((const half_t*)G, ldg, (const half_t*)W, ldw, dX, lddx, (int)B, (int)d, (int)L, scale, 0.0f,
                   workspace, workspace_bytes, reinterpret_cast<hipStream_t>(stream));
}

int xfc_dw_update(const void* G, int64_t ldg, const void* X, int64_t ldx, void* W, int64_t ldw, void* Mo, int64_t ldm,
                  int64_t B, int64_t L, int64_t d, float lr, float momentum, float weight_decay, float* dW_out,
                  int64_t ld_dw, void* stream) {
  if (!dims_ok(B) || !dims_ok(L) || !dims_ok(d)) return XFC_ERR_INVALID;
  if (L == 0 || d == 0 || B == 0) return XFC_OK;  // an empty batch is not a step: W and M stay as they are
  if (!G || !X || !W || !Mo) return XFC_ERR_INVALID;
  if (ldg % 8 || ldx % 8 || ldw % 8 || ldm % 8 || d % 8 || !aligned16(G) || !aligned16(X) || !aligned16(W) ||
      !aligned16(Mo))
    return XFC_ERR_ALIGN;
  if (dW_out && (ld_dw % 4 || !aligned16(dW_out))) return XFC_ERR_ALIGN;
  if (ldg < round_up(L, 8)) return XFC_ERR_SHAPE;
  DwArgs a = {};
  a.G = (const half_t*)G; a.ldg = ldg; a.X = (const half_t*)X; a.ldx = ldx;
  a.M = (int)L; a.N = (int)d; a.K = (int)B; a.g_cols = (int)round_up(L, 8);
  a.Wt = (half_t*)W; a.ldw = ldw; a.Mo = (half_t*)Mo; a.ldm = ldm;
  a.lr = lr; a.mu = momentum; a.wd = weight_decay; a.dw_dump = dW_out; a.ld_dump = ld_dw;
  return launch_dw(DW_UPDATE, a, reinterpret_cast<hipStream_t>(stream));
}

int xfc_dw_update_master(const void* G, int64_t ldg, const void* X, int64_t ldx, float* W32, int64_t ldw32, float* M32,
                         int64_t ldm32, void* W16, int64_t ldw16, int64_t B, int64_t L, int64_t d, float lr,
                         float momentum, float weight_decay, float* dW_out, int64_t ld_dw, void* stream) {
  if (!dims_ok(B) || !dims_ok(L) || !dims_ok(d)) return XFC_ERR_INVALID;
  if (L == 0 || d == 0 || B == 0) return XFC_OK;  // an empty batch is not a step
  if (!G || !X || !W32 || !M32 || !W16) return XFC_ERR_INVALID;
  if (ldg % 8 || ldx % 8 || ldw16 % 8 || ldw32 % 4 || ldm32 % 4 || d % 8 || !aligned16(G) || !aligned16(X) ||
      !aligned16(W32) || !aligned16(M32) || !aligned16(W16))
    return XFC_ERR_ALIGN;
  if (dW_out && (ld_dw % 4 || !aligned16(dW_out))) return XFC_ERR_ALIGN;
  if (ldg < round_up(L, 8)) return XFC_ERR_SHAPE;
  DwArgs a = {};
  a.G = (const half_t*)G; a.ldg = ldg; a.X = (const half_t*)X; a.ldx = ldx;
  a.M = (int)L; a.N = (int)d; a.K = (int)B; a.g_cols = (int)round_up(L, 8);
  a.Wt = (half_t*)W16; a.ldw = ldw16; a.W32 = W32; a.ldw32 = ldw32; a.M32 = M32; a.ldm32 = ldm32;
  a.lr = lr; a.mu = momentum; a.wd = weight_decay; a.dw_dump = dW_out; a.ld_dump = ld_dw;
  return launch_dw(DW_UPDATE_MASTER, a, reinterpret_cast<hipStream_t>(stream));
}

int xfc_sgd_momentum_master(float* W32, float* M32, void* W16, const float* grad, int64_t count, float lr, float momentum,
                            float weight_decay, void* stream) {
  if (count < 0) return XFC_ERR_INVALID;
  if (count == 0) return XFC_OK;
  if (!W32 || !M32 || !W16 || !grad) return XFC_ERR_INVALID;
  if (count % 8 || !aligned16(W32) || !aligned16(M32) || !aligned16(W16) || !aligned16(grad)) return XFC_ERR_ALIGN;
  const int64_t n8 = count / 8;
  hipLaunchKernelGGL(sgd_momentum_master_kernel, dim3((unsigned)ceil_div(n8, 256)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), W32, M32, (half_t*)W16, grad, n8, lr, momentum, weight_decay);
  return check_launch();
}

int xfc_dw(const void* G, int64_t ldg, const void* X, int64_t ldx, float* grad, int64_t ld_grad, int64_t B, int64_t L,
           int64_t d, float beta, void* stream) {
  if (!dims_ok(B) || !dims_ok(L) || !dims_ok(d)) return XFC_ERR_INVALID;
  if (L == 0 || d == 0) return XFC_OK;
  if (B == 0 && beta == 1.0f) return XFC_OK;  // an empty micro-batch adds nothing
  if (B == 0) return XFC_ERR_INVALID;          // beta != 1 with no rows would only rescale grad: not a dW call
  if (!G || !X || !grad) return XFC_ERR_INVALID;
  if (ldg % 8 || ldx % 8 || d % 8 || ld_grad % 4 || !aligned16(G) || !aligned16(X) || !aligned16(grad))
    return XFC_ERR_ALIGN;
  if (ldg < round_up(L, 8)) return XFC_ERR_SHAPE;
  DwArgs a = {};
  a.G = (const half_t*)G; a.ldg = ldg; a.X = (const half_t*)X; a.ldx = ldx;
  a.M = (int)L; a.N = (int)d; a.K = (int)B; a.g_cols = (int)round_up(L, 8);
  a.out = grad; a.ldo = ld_grad; a.alpha = 1.0f; a.beta = beta;
  return launch_dw(DW_OUT, a, reinterpret_cast<hipStream_t>(stream));
}

int xfc_sgd_momentum(void* W, void* Mo, const float* grad, int64_t count, float lr, float momentum, float weight_decay,
                     void* stream) {
  if (count < 0) return XFC_ERR_INVALID;
  if (count == 0) return XFC_OK;
  if (!W || !Mo || !grad) return XFC_ERR_INVALID;
  if (count % 8 || !aligned16(W) || !aligned16(Mo) || !aligned16(grad)) return XFC_ERR_ALIGN;
  const int64_t n8 = count / 8;
  hipLaunchKernelGGL(sgd_momentum_kernel, dim3((unsigned)ceil_div(n8, 256)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), (half_t*)W, (half_t*)Mo, grad, n8, lr, momentum,
                     weight_decay);
  return check_launch();
}

size_t xfc_step_workspace_bytes(int64_t B, int64_t L, int64_t d, int64_t nnz) {
  return (size_t)round_up(xfc_fwd_grad_workspace_bytes(L, nnz), 256) + xfc_dx_workspace_bytes(B, L, d);
}

int xfc_step_csr(const void* X, int64_t ldx, void* W, int64_t ldw, void* Mo, int64_t ldm, const int32_t* rowptr,
                 const int32_t* colidx, int64_t nnz, void* G, int64_t ldg, float* dX, int64_t lddx, int64_t B,
                 int64_t L, int64_t d, float lr, float momentum, float weight_decay, float scale, void* workspace,
                 size_t workspace_bytes, void* stream) {
  const size_t off = (size_t)round_up(xfc_fwd_grad_workspace_bytes(L, nnz), 256);
  if (!workspace || workspace_bytes < off) return XFC_ERR_WORKSPACE;  // xfc_dx checks its own share
  if (ldg < round_up(L, 8)) return XFC_ERR_SHAPE;
  unsigned char* ws = reinterpret_cast<unsigned char*>(workspace);
  int rc = xfc_fwd_grad_csr(X, ldx, W, ldw, rowptr, colidx, G, ldg, B, L, d, nnz, nullptr, ws, off, stream);
  if (rc) return rc;
  rc = xfc_dx(G, ldg, W, ldw, dX, lddx, B, L, d, scale, ws + off, workspace_bytes - off, stream);
  if (rc) return rc;
  return xfc_dw_update(G, ldg, X, ldx, W, ldw, Mo, ldm, B, L, d, lr, momentum, weight_decay, nullptr, 0, stream);
}

constexpr int TOPK_SAMPLE = 2048;
// K <= 8: the rows' bounds start from the K-th score over a sample of the first TOPK_SAMPLE labels (a small
// logits pass and an exact selection) when every label group has enough tiles for that to pay; otherwise
// from nothing.  Without it every workgroup's first tiles overflow the candidate buffers and are rescanned.
static bool topk_seeded(int64_t L, int tiles_n, int n_groups) {
  return L >= 8 * (int64_t)TOPK_SAMPLE && tiles_n >= 8 * n_groups;
}
// bytes of the K <= 8 pass with n_groups label groups: the groups' candidate lists, the rows' shared bounds,
// and (seeded) the sample logits and their top K
static size_t topk_need(int64_t B, int64_t K, int n_groups, bool seeded) {
  size_t need = (size_t)n_groups * B * K * 8 + (size_t)round_up(B, 4) * 4;
  if (seeded) need += (size_t)B * TOPK_SAMPLE * 2 + (size_t)B * K * 12;
  return need;
}
// Label groups of the K <= 8 pass: enough to give every CU a workgroup, fewer when the workspace holds no more
// (8 at least; the seeding is dropped before the last groups are).  A smaller batch has fewer row tiles and so
// more groups: the need is not monotone in B.
static void topk_plan(int64_t B, int64_t L, int64_t K, size_t ws_limit, int& tiles_m, int& tiles_n, int& n_groups,
                      int& grid, bool& seeded) {
  tiles_m = ceil_div(B, row_tile(B));
  tiles_n = ceil_div(L, FwdCore::BN);
  int per = num_cus() / (8 * tiles_m);  // groups per XCD
  if (per < 1) per = 1;
  n_groups = 8 * per;
  const int cap = (int)round_up(tiles_n, 8);
  if (n_groups > cap) n_groups = cap;
  for (;; n_groups -= 8) {
    seeded = topk_seeded(L, tiles_n, n_groups);
    if (topk_need(B, K, n_groups, seeded) <= ws_limit) break;
    if (seeded && topk_need(B, K, n_groups, false) <= ws_limit) { seeded = false; break; }
    if (n_groups <= 8) break;  // the caller compares the need of this plan with what it was given
  }
  grid = tiles_m * n_groups;
}

size_t xfc_topk_workspace_bytes(int64_t B, int64_t L, int64_t K) {
  if (!dims_ok(B) || !dims_ok(L) || K < 1 || K > SEL_MAX_K || B == 0 || L == 0) return 0;
  if (K > TOPK_MAX) return (size_t)B * (size_t)round_up(L, 8) * 2;  // the logits of every row
  int tm, tn, ng, grid;
  bool seeded;
  topk_plan(B, L, K, ~(size_t)0, tm, tn, ng, grid, seeded);
  return topk_need(B, K, ng, seeded);
}

size_t xfc_layer_workspace_bytes(int64_t max_batch, int64_t L, int64_t d, int64_t max_nnz) {
  if (!dims_ok(max_batch) || !dims_ok(L) || !dims_ok(d) || max_nnz < 0) return 0;
  size_t dx = 0, topk = 0;
  const int64_t k8 = L < TOPK_MAX ? L : TOPK_MAX;
  for (int64_t b = 1; b <= max_batch; ++b) {
    const size_t a = xfc_dx_workspace_bytes(b, L, d);
    if (a > dx) dx = a;
    const size_t t = k8 > 0 ? xfc_topk_workspace_bytes(b, L, k8) : 0;
    if (t > topk) topk = t;
  }
  const size_t step = (size_t)round_up(xfc_fwd_grad_workspace_bytes(L, max_nnz), 256) + dx;
  return step > topk ? step : topk;
}

int xfc_topk(const void* X, int64_t ldx, const void* W, int64_t ldw, int64_t B, int64_t L, int64_t d, int64_t numy,
             int K, float* values, int64_t* indices, void* workspace, size_t workspace_bytes, void* stream) {
  if (!dims_ok(B) || !dims_ok(L) || !dims_ok(d)) return XFC_ERR_INVALID;
  if (B == 0) return XFC_OK;
  if (K < 1 || K > SEL_MAX_K || L < K || numy < 1 || d <= 0) return XFC_ERR_INVALID;
  if (!X || !W || !values || !indices) return XFC_ERR_INVALID;
  if (ldx % 8 || ldw % 8 || d % 8 || !aligned16(X) || !aligned16(W)) return XFC_ERR_ALIGN;
  if (K > TOPK_MAX) {
    // logits of a block of rows into the workspace, then an exact selection per row
    const int64_t ldl = round_up(L, 8);
    const int64_t fit = workspace ? (int64_t)(workspace_bytes / (size_t)(ldl * 2)) : 0;
    if (fit < (B < 256 ? B : 256)) return XFC_ERR_WORKSPACE;
    if (!aligned16(workspace)) return XFC_ERR_ALIGN;
    const int64_t block = fit >= B ? B : fit / 256 * 256;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    for (int64_t r0 = 0; r0 < B; r0 += block) {
      const int64_t rows = B - r0 < block ? B - r0 : block;
      int rc = launch_fwd(FWD_LINEAR, (const half_t*)X + r0 * ldx, ldx, (const half_t*)W, ldw, (half_t*)workspace, ldl,
                          (int)rows, (int)L, (int)d, (int)L, 1.0f, 0.0f, nullptr, st);
      if (rc) return rc;
      // sample every stride-th 16 KB block first when that still holds 16 K elements and points at about a
      // thousand candidates at most (half the sort buffer)
      const int cap = K <= SEL_SMALL_MAX_K ? SEL_CAP_SMALL : SEL_CAP_LARGE;
      int stride = 1;
      while (stride < 16 && (int64_t)K * stride * 2 <= cap / 2 && L / (stride * 2) >= 16 * (int64_t)K &&
             L / (stride * 2) >= (int64_t)SEL_THREADS * 8 * 4)
        stride *= 2;
      const SelArgs sa = {(const half_t*)workspace, ldl, (int)L, numy, K, stride, values + r0 * K, indices + r0 * K};
      rc = K <= SEL_SMALL_MAX_K ? launch_select<SEL_CAP_SMALL>((int)rows, sa, st) : launch_select<SEL_CAP_LARGE>((int)rows, sa, st);
      if (rc) return rc;
    }
    return XFC_OK;
  }
  TopkArgs a;
  int grid;
  bool seeded;
  topk_plan(B, L, K, workspace ? workspace_bytes : 0, a.tiles_m, a.tiles_n, a.n_groups, grid, seeded);
  const size_t need = topk_need(B, K, a.n_groups, seeded);
  if (!workspace || workspace_bytes < need) return XFC_ERR_WORKSPACE;
  if (!aligned16(workspace)) return XFC_ERR_ALIGN;
  a.X = (const half_t*)X; a.ldx = ldx; a.W = (const half_t*)W; a.ldw = ldw;
  a.M = (int)B; a.N = (int)L; a.K = (int)d; a.topk = K;
  a.cand_v = reinterpret_cast<float*>(workspace);
  a.cand_i = reinterpret_cast<int32_t*>(a.cand_v + (size_t)a.n_groups * B * K);
  a.bound = reinterpret_cast<uint32_t*>(a.cand_i + (size_t)a.n_groups * B * K);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (seeded) {
    // 16-byte aligned: the lists above are B * K * 8 * n_groups bytes (n_groups a multiple of 8), the bounds 16-byte padded
    half_t* sample = reinterpret_cast<half_t*>(a.bound + round_up(B, 4));
    int64_t* sample_i = reinterpret_cast<int64_t*>(sample + (size_t)B * TOPK_SAMPLE);
    float* sample_v = reinterpret_cast<float*>(sample_i + (size_t)B * K);
    int rc0 = launch_fwd(FWD_LINEAR, (const half_t*)X, ldx, (const half_t*)W, ldw, sample, TOPK_SAMPLE, (int)B, TOPK_SAMPLE,
                         (int)d, TOPK_SAMPLE, 1.0f, 0.0f, nullptr, st);
    if (rc0) return rc0;
    const SelArgs sa = {(const half_t*)sample, (int64_t)TOPK_SAMPLE, TOPK_SAMPLE, (int64_t)TOPK_SAMPLE, K, 1, sample_v, sample_i};
    if ((rc0 = launch_select<SEL_CAP_SMALL>((int)B, sa, st))) return rc0;
    hipLaunchKernelGGL(topk_seed_kernel, dim3((unsigned)ceil_div(B, 256)), dim3(256), 0, st, (const float*)sample_v, K,
                       a.bound, B);
    if ((rc0 = check_launch())) return rc0;
  } else {
    // a kernel, not a memset: the call may be recorded into a graph
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)ceil_div(B, 256)), dim3(256), 0, st, a.bound, 0u, B);
    if (int rc0 = check_launch()) return rc0;
  }
  const dim3 tg((unsigned)grid), tb(FwdCore::NT);
  int rc;
  switch (row_tile(B)) {
    case 64: rc = launch_k<topk_kernel<FwdCore64>>(tg, tb, TopkLds<FwdCore64>::BYTES, st, a); break;
    case 128: rc = launch_k<topk_kernel<FwdCore128>>(tg, tb, TopkLds<FwdCore128>::BYTES, st, a); break;
    default: rc = launch_k<topk_kernel<FwdCore>>(tg, tb, TopkLds<FwdCore>::BYTES, st, a); break;
  }
  if (rc) return rc;
  hipLaunchKernelGGL(topk_merge_kernel, dim3((unsigned)B), dim3(64), 0, st, a.cand_v, a.cand_i, (int)B, a.n_groups, K,
                     numy, values, indices);
  return check_launch();
}

int xfc_copy(const void* src, void* dst, int64_t bytes, void* stream) {
  if (bytes < 0) return XFC_ERR_INVALID;
  if (bytes == 0) return XFC_OK;
  if (!src || !dst) return XFC_ERR_INVALID;
  if (bytes % 16 || !aligned16(src) || !aligned16(dst)) return XFC_ERR_ALIGN;
  const int64_t n16 = bytes / 16;
  int64_t grid = ceil_div(n16, 256);
  if (grid > 16384) grid = 16384;
  hipLaunchKernelGGL(copy_kernel, dim3((unsigned)grid), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     reinterpret_cast<const uint4v*>(src), reinterpret_cast<uint4v*>(dst), n16);
  return check_launch();
}

}  // extern "C"
