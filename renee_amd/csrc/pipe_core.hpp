// Multi-stage fp16 MFMA main loop for gfx950 (CDNA4) with direct global->LDS loads.
//
// One workgroup of WM x WN wavefronts owns a BM x BN accumulator tile and walks the
// contraction index in steps of BK.  Operand tiles travel HBM/L2 -> LDS without passing
// through registers (global_load_lds_dwordx4: every lane fetches 16 bytes from its own
// address and the wave's 64 pieces land in 1 KB of consecutive LDS).  STAGES tile pairs
// are resident; STAGES-1 are in flight ahead of the one being multiplied, and the ring keeps
// turning across the tiles a workgroup processes, so a tile's epilogue runs with the next
// tile's operands already on their way.
//
// Operand storage in global memory:
//   KC ("K-contiguous"):  elem(r, k) at P[r*ld + k]     LDS: [r][BK], 16-byte chunks XOR-swizzled by row
//   MC ("M/N-contiguous"): elem(r, k) at P[k*ld + r]    LDS: [k][R],  16-byte chunks XOR-swizzled by k
// KC fragments are read with ds_read_b128, MC fragments with ds_read_b64_tr_b16.
// Pieces outside the operand (row, column or k past its limit) are fetched from a 16-byte
// block of zeros instead, so every LDS slot is always written.
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
typedef __fp16 fp16x4_t __attribute__((__vector_size__(4 * sizeof(__fp16))));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

#define XFC_LDS __attribute__((address_space(3)))
#define XFC_GLB __attribute__((address_space(1)))

__device__ __attribute__((aligned(16))) const uint32_t g_zero16[4] = {0u, 0u, 0u, 0u};

// Row of C held by accumulator register r of a 32x32 block, for this lane.
__device__ __forceinline__ int c_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

// Waits until at most N of this wave's vector-memory operations are outstanding, then joins the
// workgroup barrier.  Written as one asm block: a plain __syncthreads() carries a fence that makes
// the compiler drain every outstanding global->LDS fetch first, which would serialise the ring.
// The "memory" clobber keeps the compiler from moving LDS or global accesses across it.
template <int N>
__device__ __forceinline__ void wait_vmcnt_barrier() {
  static_assert(N >= 0 && N < 64, "vmcnt range");
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_lds_vmcnt_barrier() {
  static_assert(N >= 0 && N < 64, "vmcnt range");
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt range");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// 16 bytes per lane from global memory to LDS at lds_base + lane*16 (lds_base wave-uniform), as
// global_load_lds_dwordx4 with the LDS address in M0.  Written as inline asm on purpose: the compiler
// treats the builtin form as a store to LDS that any later LDS read it cannot disambiguate may alias, and
// puts an s_waitcnt vmcnt(0) in front of such reads (every ds_read_b64_tr_b16 and every epilogue access to
// LDS), which makes each wave wait for the stage it has just requested.  The waits for these fetches are
// the explicit ones in run(); the compiler's own vmcnt bookkeeping for other loads and stores stays
// correct without knowing about them (operations return in order, so it can only wait longer than
// needed).  M0 is a reserved register: the compiler never keeps a value of its own there, it only loads
// it in front of an instruction that reads it.  The asm statements still list it as clobbered, so that the
// pass which hoists and merges M0 initialisations sees a definition here and never moves one of the
// compiler's own M0 loads across a fetch (hipcc warns that the register is reserved; the build silences
// that one warning).  NT marks the fetch non-temporal: for data read once, so that it does not displace
// reused lines from the L2.
// Marks a value the caller knows to be wave-uniform as such (scalar registers, scalar arithmetic).
__device__ __forceinline__ int64_t uniform64(int64_t v) {
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)v >> 32));
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uint64_t)v);
  return (int64_t)(((uint64_t)hi << 32) | (uint64_t)lo);
}
__device__ __forceinline__ uint32_t lds_addr(void* p) { return (uint32_t)(uintptr_t)(XFC_LDS void*)p; }
// address = uniform 64-bit base + per-lane 32-bit offset
template <bool NT = false>
__device__ __forceinline__ void load16_to_lds(const void* ubase, uint32_t voff, void* lds_base) {
  const uint32_t m = lds_addr(lds_base);
  // an integer operand whose halves are marked uniform: the "s" constraint alone is not always honoured
  const uint64_t b0 = reinterpret_cast<uint64_t>(ubase);
  // (readfirstlane returns a signed int: widen through uint32_t, or the low half sign-extends into the high one)
  const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b0 >> 32));
  const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b0);
  const uint64_t b = ((uint64_t)b_hi << 32) | (uint64_t)b_lo;
  if constexpr (NT)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(m), "v"(voff), "s"(b) : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m), "v"(voff), "s"(b) : "memory", "m0");
}
// address = per-lane 64-bit pointer
template <bool NT = false>
__device__ __forceinline__ void load16_to_lds(const void* g, void* lds_base) {
  const uint32_t m = lds_addr(lds_base);
  if constexpr (NT)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(m), "v"(g) : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(m), "v"(g) : "memory", "m0");
}

template <int BK>
__device__ __forceinline__ int kc_swz(int row) {
  // ds_read_b128 is served 16 lanes at a time over 64 banks: the 16 rows one group reads must spread
  // over all 256 bytes.  Measured: 212 B/clk/CU (BK 64) and 220 (BK 32), against 63-122 for other choices.
  if constexpr (BK == 64) return (row >> 1) & 7;
  else return (row >> 2) & 3;
}
// MC tiles: chunk index within a k-row is XORed with 4*(k%4): the four k-rows one
// transposing read touches then sit in four different 64-byte bank groups.
__device__ __forceinline__ int mc_swz(int k) { return (k & 3) << 2; }

// FETCH_WAVES_: how many of the workgroup's waves issue the global->LDS fetches (the first FETCH_WAVES_ wave
// ids; 0 = all).  The fetch path of a CU accepts about 1 KB per 9 ns, so the fetches of one 64 KB stage keep the
// waves that issue them waiting for 700-1200 cycles (shader-clock marks around the burst); a wave waiting there
// issues no MFMA.  A fetch in the scalar-base form does not slow the MFMAs of another wave on the same SIMD
// (3 ns per fetch in a microbenchmark), so with only the first half of the waves fetching -- a workgroup's
// waves are dealt round-robin over the four SIMDs, which makes that one wave per SIMD -- the other wave of each
// SIMD multiplies through the burst: 3-5 % on the forward and dX kernels.
template <int BM_, int BN_, int BK_, int WM_, int WN_, int STAGES_, bool A_KC_, bool B_KC_, bool ACC_AGPR_ = false,
          bool A_NT_ = false, bool B_NT_ = false, int FETCH_WAVES_ = 0>
struct PipeCore {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, STAGES = STAGES_;
  static constexpr bool A_KC = A_KC_, B_KC = B_KC_;
  static constexpr int NW = WM * WN, NT = 64 * NW;
  static constexpr int NWF = FETCH_WAVES_ > 0 ? FETCH_WAVES_ : NW;  // waves that fetch
  static constexpr int TM = BM / WM, TN = BN / WN;
  static constexpr int FM = TM / 32, FN = TN / 32;
  static constexpr int CPR = BK / 8;
  static constexpr int A_HALVES = BM * BK, B_HALVES = BN * BK;
  static constexpr int STAGE_HALVES = A_HALVES + B_HALVES;
  static constexpr int LDS_BYTES = STAGES * STAGE_HALVES * 2;
  static constexpr int A_CH = BM * BK / 8 / (64 * NWF), B_CH = BN * BK / 8 / (64 * NWF);
  static constexpr int LOADS_PER_STAGE = A_CH + B_CH;  // per fetching wave
  static_assert(BM % (32 * WM) == 0 && BN % (32 * WN) == 0, "wave tile must be 32-multiples");
  static_assert((BM * BK / 8) % (64 * NWF) == 0 && (BN * BK / 8) % (64 * NWF) == 0, "chunk split");
  static_assert(NWF <= NW && NWF % 2 == 0, "fetching waves");
  static_assert(BK == 32 || BK == 64, "BK");
  static_assert(A_KC || BM >= 128, "MC swizzle needs 16 chunks per k-row");
  static_assert(B_KC || BN >= 128, "MC swizzle needs 16 chunks per k-row");
  static_assert(STAGES >= 2 && (STAGES - 1) * LOADS_PER_STAGE < 64, "stages");
  static_assert(NW % 2 == 0, "the LDS swizzles assume an even number of waves");

  // One operand's tile: base pointer, leading dimension (halves), first row (KC) or column (MC) of the
  // tile, the limit of that index and the limit of the contraction index.  Requirements: r0 < rmax;
  // for MC operands rmax is a multiple of 8; ld * 2 * 16 < 2^32.  Rows (columns) at or past rmax are
  // fetched from the last valid row (column chunk) instead: they only ever feed outputs the caller
  // discards.  Contraction indices at or past kmax are fetched as zeros.
  struct Operand {
    const half_t* p;
    int64_t ld;
    int r0, rmax, kmax;
  };

  // Addresses of the CH 16-byte pieces a thread fetches for one operand each stage.  Every fetch is
  // "uniform 64-bit base + per-thread 32-bit offset": the bases advance along k with scalar adds, so a
  // steady-state stage costs no vector ALU work, which matters because the SIMD that issues the MFMAs
  // cannot overlap them with other vector instructions.
  template <bool KC, int R, int CH, bool NT>
  struct Loader {
    static constexpr int CPI = KC ? CPR : R / 8;  // 16-byte chunks per tile row (KC) or per k-row (MC)
    static constexpr int RPI = 64 / CPI;          // tile rows (KC) or k-rows (MC) one wave instruction covers
    const char* base;    // uniform
    int64_t grp[CH];     // uniform byte offset of each instruction's first row
    uint32_t voff[CH];   // per-thread byte offset inside the group
    int64_t kbytes;      // uniform byte offset of the current stage along k
    int64_t kstep;       // uniform
    int kmax, kin;       // limit of k; per-thread k offset inside the stage (KC: chunk*8, MC: k-row in group)
    int kgrp[CH];        // uniform: first k-row of each instruction (MC), 0 (KC)
    __device__ __forceinline__ void init(const Operand& o, int k_begin, int wave, int lane) {
      base = reinterpret_cast<const char*>(uniform64(reinterpret_cast<int64_t>(o.p)));
      kmax = o.kmax;
      const int sub = lane / CPI, pc = lane % CPI;
      if constexpr (KC) {
        kstep = (int64_t)BK * 2;
        kbytes = uniform64((int64_t)k_begin * 2);
        const int c = pc ^ kc_swz<BK>(wave * RPI + sub);  // the swizzle does not depend on i (NWF is even)
        kin = c * 8;
#pragma unroll
        for (int i = 0; i < CH; ++i) {
          const int row0 = o.r0 + (i * NWF + wave) * RPI;
          const int g = row0 < o.rmax ? row0 : o.rmax - 1;
          const int row = row0 + sub < o.rmax ? row0 + sub : o.rmax - 1;
          grp[i] = uniform64((int64_t)g * o.ld * 2);
          voff[i] = (uint32_t)(row - g) * (uint32_t)(o.ld * 2) + (uint32_t)c * 16u;
          kgrp[i] = 0;
        }
      } else {
        kstep = uniform64((int64_t)BK * o.ld * 2);
        kbytes = uniform64((int64_t)k_begin * o.ld * 2);
        const int c = pc ^ mc_swz(wave * RPI + sub);
        const int col = o.r0 + c * 8 < o.rmax ? o.r0 + c * 8 : o.rmax - 8;
        kin = sub;
#pragma unroll
        for (int i = 0; i < CH; ++i) {
          kgrp[i] = (i * NWF + wave) * RPI;
          grp[i] = uniform64((int64_t)kgrp[i] * o.ld * 2);
          voff[i] = (uint32_t)sub * (uint32_t)(o.ld * 2) + (uint32_t)col * 2u;
        }
      }
    }
    // k0: absolute k of the stage being fetched
    __device__ __forceinline__ void issue(half_t* region, int k0, int wave) {
      if (k0 + BK <= kmax) {
#pragma unroll
        for (int i = 0; i < CH; ++i)
          load16_to_lds<NT>(base + grp[i] + kbytes, voff[i], region + (i * NWF + wave) * 512);
      } else {  // the stage that crosses kmax: pieces past it come from the block of zeros
#pragma unroll
        for (int i = 0; i < CH; ++i) {
          const bool valid = k0 + kgrp[i] + kin < kmax;
          const void* src = valid ? (const void*)(base + grp[i] + kbytes + voff[i]) : (const void*)g_zero16;
          load16_to_lds<NT>(src, region + (i * NWF + wave) * 512);
        }
      }
      kbytes += kstep;
    }
  };
  using LoaderA = Loader<A_KC, BM, A_CH, A_NT_>;
  using LoaderB = Loader<B_KC, BN, B_CH, B_NT_>;

  __device__ __forceinline__ static half8 frag_kc(const half_t* lds, int row0, int kk, int lane) {
    const int r = row0 + (lane & 31);
    const int c = kk * 2 + (lane >> 5);
    return *reinterpret_cast<const half8*>(lds + r * BK + ((c ^ kc_swz<BK>(r)) * 8));
  }

  // 32 columns starting at col0 of an MC tile [k][R]: within each 16-lane group, lane t
  // supplies the address of row k + t/4, columns c0 + 4*(t%4)..+3 and receives column
  // c0 + t for four consecutive k.
  template <int R>
  __device__ __forceinline__ static half8 frag_mc(const half_t* lds, int col0, int kk, int lane) {
    const int g = lane >> 4, t = lane & 15;
    const int k = kk * 16 + 8 * (g >> 1) + (t >> 2);
    const int c = col0 + 16 * (g & 1) + 4 * (t & 3);
    const int off = k * R + ((((c >> 3) ^ mc_swz(k)) << 3) | (c & 7));
    fp16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4f16((XFC_LDS fp16x4_t*)(lds + off));
    fp16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4f16((XFC_LDS fp16x4_t*)(lds + off + 4 * R));
    half8 out;
    out[0] = (half_t)lo[0]; out[1] = (half_t)lo[1]; out[2] = (half_t)lo[2]; out[3] = (half_t)lo[3];
    out[4] = (half_t)hi[0]; out[5] = (half_t)hi[1]; out[6] = (half_t)hi[2]; out[7] = (half_t)hi[3];
    return out;
  }

  struct Frags {
    half8 a[FM], b[FN];
  };
  __device__ __forceinline__ static void load_frags(const half_t* st, int kk, int wm, int wn, int lane, Frags& f) {
    const half_t* sa = st;
    const half_t* sb = st + A_HALVES;
#pragma unroll
    for (int fm = 0; fm < FM; ++fm) {
      if constexpr (A_KC) f.a[fm] = frag_kc(sa, wm * TM + fm * 32, kk, lane);
      else f.a[fm] = frag_mc<BM>(sa, wm * TM + fm * 32, kk, lane);
    }
#pragma unroll
    for (int fn = 0; fn < FN; ++fn) {
      if constexpr (B_KC) f.b[fn] = frag_kc(sb, wn * TN + fn * 32, kk, lane);
      else f.b[fn] = frag_mc<BN>(sb, wn * TN + fn * 32, kk, lane);
    }
  }
  // ACC_AGPR pins the accumulators to the accumulation register file ("a" constraint; the compiler only
  // picks that form by itself above 256 registers).  With the accumulators in ordinary vector registers
  // a SIMD's MFMAs and its global->LDS fetches serialise more (microbenchmark: one stage of fetches plus
  // 32 MFMAs per wave, 1.19 ms-equivalents against 0.83 with AGPR accumulators; 0.69 / 0.61 for either
  // alone), but the AGPR form leaves only 128 ordinary registers and costs a copy per accumulator read,
  // so it pays only where the epilogue is trivial (dX).  Being inline asm, the instruction is invisible
  // to the compiler's MFMA hazard bookkeeping: settle() supplies the wait states an MFMA result needs
  // before ordinary code may read it, zero() those between an accumulator write and its use as source C.
  __device__ __forceinline__ static void mfma_all(const Frags& f, float16v (&acc)[FM][FN]) {
#pragma unroll
    for (int fm = 0; fm < FM; ++fm)
#pragma unroll
      for (int fn = 0; fn < FN; ++fn) {
        if constexpr (ACC_AGPR_)
          asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc[fm][fn]) : "v"(f.a[fm]), "v"(f.b[fn]));
        else
          acc[fm][fn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.a[fm], f.b[fn], acc[fm][fn], 0, 0, 0);
      }
  }
  // At least 18 idle issue slots must separate an MFMA from a non-MFMA read or write of its destination.
  __device__ __forceinline__ static void settle(float16v (&acc)[FM][FN]) {
    if constexpr (ACC_AGPR_) {
#pragma unroll
      for (int fm = 0; fm < FM; ++fm)
#pragma unroll
        for (int fn = 0; fn < FN; ++fn)
          asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 3" : "+a"(acc[fm][fn]));
    }
  }
  __device__ __forceinline__ static void zero(float16v (&acc)[FM][FN]) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j) {
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
        if constexpr (ACC_AGPR_) asm volatile("s_nop 3" : "+a"(acc[i][j]));  // accumulator write -> MFMA source C
      }
  }

  // Walks the work items [item_begin, item_end) of this workgroup.
  //   get(item, oa, ob, k_begin, k_end)  fills the operands and the k range of an item (k_end > k_begin,
  //                                      k_begin a multiple of BK)
  //   epilogue(item, acc)                consumes the finished accumulators; it may use global memory and LDS
  //                                      outside the ring's LDS_BYTES
  // All threads of the workgroup call this together.
  //
  // Schedule per stage c (BK/16 sub-steps): the operand fragments of sub-step kk+1 are read from LDS
  // while the MFMAs of sub-step kk run.  Before the MFMAs of the last sub-step the wave waits for its
  // part of stage c+1 to have landed and joins the barrier; past it, every wave has finished reading
  // stage c, so its slot is refilled with stage c+STAGES, and the first fragments of stage c+1 are
  // read under the last MFMAs of stage c.
  template <class GetItem, class Epilogue>
  __device__ __forceinline__ static void run(int item_begin, int item_end, half_t* lds, GetItem get, Epilogue epilogue) {
    if (item_begin >= item_end) return;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / WN, wn = wave % WN;
    constexpr int KK = BK / 16;
    float16v acc[FM][FN];
    zero(acc);

    // fill cursor
    LoaderA la;
    LoaderB lb;
    int i_item = item_begin, i_k = 0, i_kend = 0, i_slot = 0;
    bool i_live = true;
    {
      Operand oa, ob;
      get(i_item, oa, ob, i_k, i_kend);
      la.init(oa, i_k, wave, lane);
      lb.init(ob, i_k, wave, lane);
    }
    const bool fetcher = wave < NWF;  // wave-uniform
    auto issue_one = [&]() {
      half_t* st = lds + i_slot * STAGE_HALVES;
      if (i_live) {
        if (fetcher) {
          la.issue(st, i_k, wave);
          lb.issue(st + A_HALVES, i_k, wave);
        }
        i_k += BK;
        if (i_k >= i_kend) {
          ++i_item;
          if (i_item < item_end) {
            Operand oa, ob;
            get(i_item, oa, ob, i_k, i_kend);
            la.init(oa, i_k, wave, lane);
            lb.init(ob, i_k, wave, lane);
          } else {
            i_live = false;
          }
        }
      } else if (fetcher) {
        // past the last stage: keep the count of outstanding fetches per iteration constant
#pragma unroll
        for (int i = 0; i < LOADS_PER_STAGE; ++i) load16_to_lds((const void*)g_zero16, 0u, st + (i * NWF + wave) * 512);
      }
      i_slot = i_slot + 1 == STAGES ? 0 : i_slot + 1;
    };
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) issue_one();
    wait_vmcnt_barrier<(STAGES - 2) * LOADS_PER_STAGE>();
    issue_one();

    Frags cur, nxt;
    load_frags(lds, 0, wm, wn, lane, cur);
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    int c_slot = 0;
    bool drain_all = false;
    for (int item = item_begin; item < item_end; ++item) {
      int kb, ke;
      {
        Operand oa, ob;
        get(item, oa, ob, kb, ke);
      }
      const int nk = (ke - kb + BK - 1) / BK;
      for (int kt = 0; kt < nk; ++kt) {
        const half_t* st = lds + c_slot * STAGE_HALVES;
#pragma unroll
        for (int kk = 0; kk + 1 < KK; ++kk) {
          load_frags(st, kk + 1, wm, wn, lane, nxt);
          __builtin_amdgcn_sched_barrier(0);
          mfma_all(cur, acc);
          __builtin_amdgcn_sched_barrier(0);
          cur = nxt;
        }
        const int n_slot = c_slot + 1 == STAGES ? 0 : c_slot + 1;
        // this wave's LDS reads of stage c are complete (lgkmcnt) and its share of stage c+1 has landed.
        // After an epilogue the wave's stores share the counter with the fetches and may retire out of
        // order with them, so the first wait after one drains everything.
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0), in a form the compiler's own wait bookkeeping sees
        if (drain_all) { wait_lds_vmcnt_barrier<0>(); drain_all = false; }
        else wait_lds_vmcnt_barrier<(STAGES - 2) * LOADS_PER_STAGE>();
        issue_one();  // stage c + STAGES into the slot of stage c
        load_frags(lds + n_slot * STAGE_HALVES, 0, wm, wn, lane, nxt);
        __builtin_amdgcn_sched_barrier(0);
        mfma_all(cur, acc);
        __builtin_amdgcn_sched_barrier(0);
        // No LDS read stays pending across the loop edge (the reads above finished long before the
        // MFMAs were all issued): the compiler then knows the next stage's first MFMAs need no wait.
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
        cur = nxt;
        c_slot = n_slot;
      }
      settle(acc);
      epilogue(item, acc);
      zero(acc);
      drain_all = true;
    }
    wait_vmcnt<0>();
  }
};

}  // namespace xfc
