// Tiled fp16 MFMA main loop for gfx950 (CDNA4), shared by the XFC kernels.
//
// One workgroup of WM x WN wavefronts (64 lanes each) computes a BM x BN tile of
// C = A . B with fp32 accumulation, stepping BK along the contraction index.
// Both operands are staged through LDS; the MFMA is v_mfma_f32_32x32x16_f16.
//
// Operand storage in global memory is one of
//   KC ("K-contiguous"):  elem(r, k) at  P[r * ld + k]   (r = row of A / column of B)
//   MC ("M/N-contiguous"): elem(r, k) at  P[k * ld + r]
// KC tiles are kept in LDS as [r][BK] with the 16-byte chunks of each row XOR-
// swizzled, and read with one ds_read_b128 per fragment.  MC tiles are kept as
// [k][R + pad] and read with ds_read_b64_tr_b16, which hands each lane four
// consecutive k for one r, i.e. the MFMA operand layout, without a transpose pass.
//
// MFMA 32x32x16 register layout (checked on hardware):
//   A: lane l holds A[i = l%32][k = 8*(l/32) .. +7]
//   B: lane l holds B[k = 8*(l/32) .. +7][j = l%32]
//   C: lane l, register r holds C[i = 8*(r/4) + 4*(l/32) + r%4][j = l%32]
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace xfc {

typedef _Float16 half_t;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef __fp16 fp16x4_t __attribute__((__vector_size__(4 * sizeof(__fp16))));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

#define XFC_LDS __attribute__((address_space(3)))

// Row of C held by accumulator register r of a 32x32 block, for this lane.
__device__ __forceinline__ int c_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

template <int BK>
__device__ __forceinline__ int kc_swz(int row) {
  if constexpr (BK == 64) return (row ^ (row >> 3)) & 7;
  else return ((row >> 1) ^ (row >> 3)) & 3;
}

// Extra halves per LDS row of an MC tile: makes the row pitch 16 banks (mod 64)
// so the four k-rows one transposing read touches fall in different banks.
constexpr int MC_PAD = 32;

template <int BM_, int BN_, int BK_, int WM_, int WN_, bool A_KC_, bool B_KC_>
struct GemmCore {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
  static constexpr bool A_KC = A_KC_, B_KC = B_KC_;
  static constexpr int NT = 64 * WM * WN;
  static constexpr int TM = BM / WM, TN = BN / WN;
  static constexpr int FM = TM / 32, FN = TN / 32;
  static constexpr int CPR = BK / 8;  // 16-byte chunks per KC row
  static constexpr int A_PITCH = A_KC ? BK : BM + MC_PAD;  // halves
  static constexpr int B_PITCH = B_KC ? BK : BN + MC_PAD;
  static constexpr int A_HALVES = A_KC ? BM * BK : BK * A_PITCH;
  static constexpr int B_HALVES = B_KC ? BN * BK : BK * B_PITCH;
  static constexpr int STAGE_HALVES = A_HALVES + B_HALVES;
  static constexpr int A_CHUNKS = BM * BK / 8 / NT;  // 16-byte chunks per thread per k-tile
  static constexpr int B_CHUNKS = BN * BK / 8 / NT;
  static_assert(BM % (32 * WM) == 0 && BN % (32 * WN) == 0, "wave tile must be 32-multiples");
  static_assert((BM * BK / 8) % NT == 0 && (BN * BK / 8) % NT == 0, "chunk split");
  static_assert(BK == 32 || BK == 64, "BK");

  // One operand's slice of the problem: base pointer, leading dimension (halves),
  // first r of the tile, r limit, k limit.  Chunks wholly past a limit read as 0;
  // the caller guarantees a chunk never straddles one (limits padded to 8 or the
  // buffer zero-padded to a multiple of 8 along the contiguous index).
  struct Operand {
    const half_t* p;
    int64_t ld;
    int r0;
    int rmax;
    int kmax;
  };

  template <bool KC, int R, int CH>
  __device__ __forceinline__ static void gload(const Operand& o, int k0, uint4v (&reg)[CH]) {
    const int t = threadIdx.x;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int q = t + NT * i;
      int r, k;
      if constexpr (KC) { r = q / CPR; k = (q % CPR) * 8; }
      else { k = q / (R / 8); r = (q % (R / 8)) * 8; }
      const int gr = o.r0 + r, gk = k0 + k;
      uint4v v = {0u, 0u, 0u, 0u};
      if (gr < o.rmax && gk < o.kmax) {
        const half_t* src = KC ? o.p + (int64_t)gr * o.ld + gk : o.p + (int64_t)gk * o.ld + gr;
        v = *reinterpret_cast<const uint4v*>(src);
      }
      reg[i] = v;
    }
  }

  template <bool KC, int R, int CH, int PITCH>
  __device__ __forceinline__ static void lstore(half_t* lds, const uint4v (&reg)[CH]) {
    const int t = threadIdx.x;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int q = t + NT * i;
      int off;
      if constexpr (KC) { const int r = q / CPR, c = q % CPR; off = r * BK + ((c ^ kc_swz<BK>(r)) * 8); }
      else { const int k = q / (R / 8), r = (q % (R / 8)) * 8; off = k * PITCH + r; }
      *reinterpret_cast<uint4v*>(lds + off) = reg[i];
    }
  }

  // Fragment of a KC tile for the 32 rows starting at `row0`, k16-step kk.
  __device__ __forceinline__ static half8 frag_kc(const half_t* lds, int row0, int kk, int lane) {
    const int r = row0 + (lane & 31);
    const int c = kk * 2 + (lane >> 5);
    return *reinterpret_cast<const half8*>(lds + r * BK + ((c ^ kc_swz<BK>(r)) * 8));
  }

  // Fragment of an MC tile ([k][pitch]) for the 32 columns starting at `col0`.
  // Within each 16-lane group, lane t supplies the address of row k0 + t/4,
  // columns c0 + 4*(t%4)..+3 and receives column c0 + t, rows k0..k0+3.
  template <int PITCH>
  __device__ __forceinline__ static half8 frag_mc(const half_t* lds, int col0, int kk, int lane) {
    const int g = lane >> 4, t = lane & 15;
    const int k = kk * 16 + 8 * (g >> 1) + (t >> 2);
    const int c = col0 + 16 * (g & 1) + 4 * (t & 3);
    const half_t* p0 = lds + k * PITCH + c;
    fp16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4f16((XFC_LDS fp16x4_t*)(p0));
    fp16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4f16((XFC_LDS fp16x4_t*)(p0 + 4 * PITCH));
    half8 out;
    out[0] = (half_t)lo[0]; out[1] = (half_t)lo[1]; out[2] = (half_t)lo[2]; out[3] = (half_t)lo[3];
    out[4] = (half_t)hi[0]; out[5] = (half_t)hi[1]; out[6] = (half_t)hi[2]; out[7] = (half_t)hi[3];
    return out;
  }

  __device__ __forceinline__ static void compute(const half_t* sa, const half_t* sb, int wm, int wn, int lane,
                                                 float16v (&acc)[FM][FN]) {
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      half8 af[FM], bf[FN];
#pragma unroll
      for (int fm = 0; fm < FM; ++fm) {
        if constexpr (A_KC) af[fm] = frag_kc(sa, wm * TM + fm * 32, kk, lane);
        else af[fm] = frag_mc<A_PITCH>(sa, wm * TM + fm * 32, kk, lane);
      }
#pragma unroll
      for (int fn = 0; fn < FN; ++fn) {
        if constexpr (B_KC) bf[fn] = frag_kc(sb, wn * TN + fn * 32, kk, lane);
        else bf[fn] = frag_mc<B_PITCH>(sb, wn * TN + fn * 32, kk, lane);
      }
#pragma unroll
      for (int fm = 0; fm < FM; ++fm)
#pragma unroll
        for (int fn = 0; fn < FN; ++fn)
          acc[fm][fn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[fm], bf[fn], acc[fm][fn], 0, 0, 0);
    }
  }

  // acc += A[tile rows, k_begin:k_end) . B[k_begin:k_end), tile cols].
  // `lds` must hold STAGES * STAGE_HALVES halves.  All threads of the workgroup
  // must call this together; it ends with every wave past its last LDS read.
  template <int STAGES>
  __device__ __forceinline__ static void run(const Operand& oa, const Operand& ob, int k_begin, int k_end,
                                             half_t* lds, float16v (&acc)[FM][FN]) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave / WN, wn = wave % WN;
    uint4v ra[A_CHUNKS], rb[B_CHUNKS];
    const int nk = (k_end - k_begin + BK - 1) / BK;
    if (nk <= 0) return;
    gload<A_KC, BM, A_CHUNKS>(oa, k_begin, ra);
    gload<B_KC, BN, B_CHUNKS>(ob, k_begin, rb);
    lstore<A_KC, BM, A_CHUNKS, A_PITCH>(lds, ra);
    lstore<B_KC, BN, B_CHUNKS, B_PITCH>(lds + A_HALVES, rb);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
      const bool more = kt + 1 < nk;
      half_t* cur = lds + (STAGES == 2 ? (kt & 1) * STAGE_HALVES : 0);
      half_t* nxt = lds + (STAGES == 2 ? ((kt + 1) & 1) * STAGE_HALVES : 0);
      if (more) {
        gload<A_KC, BM, A_CHUNKS>(oa, k_begin + (kt + 1) * BK, ra);
        gload<B_KC, BN, B_CHUNKS>(ob, k_begin + (kt + 1) * BK, rb);
      }
      compute(cur, cur + A_HALVES, wm, wn, lane, acc);
      if constexpr (STAGES == 1) __syncthreads();
      if (more) {
        lstore<A_KC, BM, A_CHUNKS, A_PITCH>(nxt, ra);
        lstore<B_KC, BN, B_CHUNKS, B_PITCH>(nxt + A_HALVES, rb);
      }
      __syncthreads();
    }
  }
};

}  // namespace xfc
