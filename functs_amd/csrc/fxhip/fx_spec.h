// Specialised regions: the region kernels of fx_device.h compiled once more with the
// bytecode of ONE lowered region as a compile-time constant.
//
// A generated translation unit (spec/fx_spec_<hash>.hip, written by
// fx_plan_spec_source) holds the program as a constexpr table and instantiates the
// kernels with FxSpec<Program> as their run policy.  fx_step / fx_pure_step are then
// called with constant instruction words: the opcode switch folds away, A / B / the
// temporaries live in registers, and the compiler schedules the loads of a whole
// straight-line stretch together.  Control flow is rebuilt from the structured jumps of
// the bytecode (a predicated region becomes an `if any lane is live`, a reduction loop
// a counted loop).  Everything that depends on a call (shapes, strides, pointers,
// scalars, the affine maps) is still read from the region descriptor, so a
// specialised kernel takes exactly the arguments of the generic one; the host picks it
// when the hash of a plan's programs matches (fx_spec_find) and falls back to the
// interpreter otherwise.
//
// This is the ahead-of-time counterpart of the reference's run-time code generator
// (fait/tensorexpr/cuda_codegen_tssa.cpp:881-1121, CompileToNVRTC :1319-1414).
#pragma once
#ifndef FX_SPEC_WAVES
#define FX_SPEC_WAVES 4
#endif
#ifndef FX_SPEC_ROWS
#define FX_SPEC_ROWS (3 * FX_K)
#endif
#ifndef FX_SPEC_OCC
#define FX_SPEC_OCC 4
#endif
#include "fx_device.h"

// ---- host side: the table of specialised kernels linked into the library ----
struct FxSpecKernels {
  const void* dense = nullptr;    // fx_region_dense<R, FxSpec<P>>
  const void* count = nullptr;    // fx_compact_count<FxSpec<P>>
  const void* scatter = nullptr;  // fx_compact_scatter<R, FxSpec<P>>
  uint32_t scatter_threads = 0;   // workgroup size that kernel is compiled for
  const void* stream = nullptr;   // fx_compact_stream<R, FxSpec<P>>
  const void* lean = nullptr;     // fx_dense_lean<R, P>: dense regions that fit FxLeanArgs
  bool lean_stages = false;       // ... and whether it stages the descriptor into LDS (a program reads it)
};
void fx_spec_register(uint64_t hash, const FxSpecKernels& k);
const FxSpecKernels* fx_spec_find(uint64_t hash);

namespace {

struct FxSpecEntry {
  int begin, end;  // instruction range; an output program is entered behind its leading load
  int kind;        // 0: output program, 1: mask program of a row compaction
  int pure;        // output program that the batched path may run
};

// Temporaries of a compiled program, and the values its loads fetched (one slot per
// instruction, indexed by compile-time constants only: what is never read is never kept).
template <int N, int NI = 1>
struct FxRegTemps {
  uint32_t v[N > 0 ? N : 1][FX_V] = {};
  uint32_t ld[NI][FX_V];
  __device__ __forceinline__ uint32_t& at(int32_t slot, int j) { return v[slot][j]; }
};

// ---- loads that repeat an earlier load --------------------------------------
// An instruction reads memory through (buffer a, affine record b, dtype): LDA into A,
// anything with FX_F_MEMB into B.  Inside one straight-line stretch of a program (no
// change of the lane mask, no loop edge) two such reads with the same operands fetch
// the same values, so the later one takes them from the register copy of the earlier.
constexpr bool fx_spec_loads(const FxInsn& I) { return I.op == FX_LDA || (I.flags & FX_F_MEMB) != 0; }
constexpr bool fx_spec_barrier(uint32_t op) {
  return op == FX_MIF || op == FX_MELSE || op == FX_MMERGE || op == FX_MEND || op == FX_MIFR || op == FX_RBEGIN ||
         op == FX_RNEXT;
}
template <class P>
constexpr int fx_spec_n_insn() { return (int)(sizeof(P::code) / sizeof(P::code[0])); }

// Loads that do not repeat an earlier one are issued together where their stretch starts (the
// first FX_SPEC_HOIST of them): their addresses depend on the coordinates, the loop counters
// and the lane mask only, and those are fixed over a stretch.  A wave then pays one memory
// round trip per stretch instead of one per load.  Dense regions only: in a row compaction
// the loads of a narrow output are gathers over the kept rows, which gain nothing from being
// in flight together (measured), and the registers they hold cost a wave per SIMD.
#ifndef FX_SPEC_HOIST_COMPACT
#define FX_SPEC_HOIST_COMPACT 0
#endif
#ifndef FX_SPEC_HOIST
#define FX_SPEC_HOIST 8
#endif
template <class P>
constexpr int fx_spec_hoist_cap() {
  for (int e = 0; e < P::n_entries; ++e)
    if (P::entries[e].kind == 1) return FX_SPEC_HOIST_COMPACT;   // a mask program: this is a row compaction
  return FX_SPEC_HOIST;
}

// A stretch is a run of instructions that execute together, in order, under one lane mask
// and one setting of the loop counters: it starts at a program entry, behind an instruction
// that changes the mask or a loop counter, and wherever a structured jump lands.
template <int N>
struct FxSpecTables {
  int begin[N];      // first instruction of the stretch of instruction k
  int end[N];        // first instruction behind it
  int reuse[N];      // earlier instruction of the stretch whose loaded values k takes over, or -1
  bool hoisted[N];   // k's load is issued at the start of its stretch
  bool reused[N];    // a later instruction takes over the values k loads
};
template <class P>
constexpr FxSpecTables<fx_spec_n_insn<P>()> fx_spec_tables() {
  constexpr int N = fx_spec_n_insn<P>();
  FxSpecTables<N> t{};
  bool start[N + 1] = {};
  for (int e = 0; e < P::n_entries; ++e) {
    start[P::entries[e].begin] = true;
    start[P::entries[e].end] = true;
  }
  for (int k = 0; k < N; ++k) {
    const FxInsn J = P::code[k];
    if (fx_spec_barrier(J.op)) start[k + 1] = true;
    if ((J.op == FX_MIF || J.op == FX_MIFR || J.op == FX_MELSE || J.op == FX_RNEXT) && J.a >= 0 && J.a <= N) start[J.a] = true;
    if (J.op == FX_RBEGIN && J.b >= 0 && J.b <= N) start[J.b] = true;
  }
  int b = 0;
  for (int k = 0; k < N; ++k) {
    if (start[k]) b = k;
    t.begin[k] = b;
  }
  int next = N;
  for (int k = N - 1; k >= 0; --k) {
    t.end[k] = next;
    if (start[k] || fx_spec_barrier(P::code[k].op)) next = k;
  }
  for (int k = 0; k < N; ++k) {
    const FxInsn I = P::code[k];
    t.reuse[k] = -1;
    t.hoisted[k] = false;
    t.reused[k] = false;
    if (fx_spec_barrier(I.op) || !fx_spec_loads(I)) continue;
    int rank = 0;
    for (int m = t.begin[k]; m < k; ++m) {
      const FxInsn J = P::code[m];
      if (fx_spec_barrier(J.op) || !fx_spec_loads(J)) continue;
      if (J.a == I.a && J.b == I.b && J.dt == I.dt && ((J.flags ^ I.flags) & FX_F_I2F) == 0) t.reuse[k] = m;
      if (t.reuse[m] < 0) ++rank;
    }
    if (t.reuse[k] >= 0) {
      // chains end at the first of the equal loads, the one that really loads
      while (t.reuse[t.reuse[k]] >= 0) t.reuse[k] = t.reuse[t.reuse[k]];
      t.reused[t.reuse[k]] = true;
    } else {
      t.hoisted[k] = rank < fx_spec_hoist_cap<P>();
    }
  }
  return t;
}
template <class P>
struct FxSpecPlan {
  static constexpr FxSpecTables<fx_spec_n_insn<P>()> T = fx_spec_tables<P>();
};
template <class P> constexpr bool fx_spec_stretch_start(int pc) { return FxSpecPlan<P>::T.begin[pc] == pc; }
template <class P> constexpr int fx_spec_stretch_end(int pc) { return FxSpecPlan<P>::T.end[pc]; }
template <class P> constexpr int fx_spec_reuse(int pc) { return FxSpecPlan<P>::T.reuse[pc]; }
template <class P> constexpr bool fx_spec_hoisted(int pc) { return FxSpecPlan<P>::T.hoisted[pc]; }
template <class P> constexpr bool fx_spec_reused(int pc) { return FxSpecPlan<P>::T.reused[pc]; }

// number of hoisted loads in [K, END), and whether all of them read 32-bit elements as they are
template <class P>
constexpr int fx_spec_hoist_count(int k, int end) {
  int n = 0;
  for (; k < end; ++k) if (fx_spec_hoisted<P>(k)) ++n;
  return n;
}
template <class P>
constexpr bool fx_spec_hoist_plain(int k, int end) {
  for (; k < end; ++k)
    if (fx_spec_hoisted<P>(k) &&
        !((P::code[k].dt == FX_F32 || P::code[k].dt == FX_I32) && (P::code[k].flags & FX_F_I2F) == 0))
      return false;
  return true;
}

// the hoisted loads of the stretch [K, END), one after the other (general form)
template <class P, int R, int K, int END, class TS>
__device__ __forceinline__ void fx_spec_prefetch(const FxCtx& cx, const FxCoord<R>& q, TS& ts, uint32_t M, const FxRegs& rg) {
  if constexpr (K < END) {
    if constexpr (fx_spec_hoisted<P>(K)) {
      constexpr FxInsn J = P::code[K];
      int32_t off[FX_V];
      const bool consecutive = fx_affine<R>(cx, q, J.b, rg.lc0, rg.lc1, off);
      fx_load(cx, J.a, off, M, J.dt, (J.flags & FX_F_I2F) != 0, consecutive, ts.ld[K]);
    }
    fx_spec_prefetch<P, R, K + 1, END, TS>(cx, q, ts, M, rg);
  }
}
// addresses of the hoisted loads of [K, END): element offsets (dead elements: 0), buffers, and
// how many of the loads are runs of FX_V consecutive elements
template <class P, int R, int K, int END, int RANK, int H>
__device__ __forceinline__ void fx_spec_pf_addr(const FxCtx& cx, const FxCoord<R>& q, uint32_t M, const FxRegs& rg,
                                                uint32_t (&off)[H][FX_V], uint64_t (&ptr)[H], int& n_consecutive) {
  if constexpr (K < END) {
    if constexpr (fx_spec_hoisted<P>(K)) {
      constexpr FxInsn J = P::code[K];
      int32_t o[FX_V];
      if (fx_affine<R>(cx, q, J.b, rg.lc0, rg.lc1, o)) ++n_consecutive;
#pragma unroll
      for (int j = 0; j < FX_V; ++j) off[RANK][j] = ((M >> j) & 1u) ? (uint32_t)o[j] : 0u;
      ptr[RANK] = fx_ptr(cx, J.a);
      fx_spec_pf_addr<P, R, K + 1, END, RANK + 1, H>(cx, q, M, rg, off, ptr, n_consecutive);
    } else {
      fx_spec_pf_addr<P, R, K + 1, END, RANK, H>(cx, q, M, rg, off, ptr, n_consecutive);
    }
  }
}
// the loads themselves, back to back with no branch between them: WIDE = one 128-bit load
// per lane, else FX_V single-element loads
template <class P, int K, int END, int RANK, int H, bool WIDE, class TS>
__device__ __forceinline__ void fx_spec_pf_load(TS& ts, const uint32_t (&off)[H][FX_V], const uint64_t (&ptr)[H]) {
  if constexpr (K < END) {
    if constexpr (fx_spec_hoisted<P>(K)) {
      const FX_AS1 uint8_t* base = (const FX_AS1 uint8_t*)ptr[RANK];
      if constexpr (WIDE) {
        const fx_u32x4_a4 v = *(const FX_AS1 fx_u32x4_a4*)(base + (off[RANK][0] << 2));
        ts.ld[K][0] = v.x; ts.ld[K][1] = v.y; ts.ld[K][2] = v.z; ts.ld[K][3] = v.w;
      } else {
#pragma unroll
        for (int j = 0; j < FX_V; ++j) ts.ld[K][j] = *(const FX_AS1 uint32_t*)(base + (off[RANK][j] << 2));
      }
      fx_spec_pf_load<P, K + 1, END, RANK + 1, H, WIDE, TS>(ts, off, ptr);
    } else {
      fx_spec_pf_load<P, K + 1, END, RANK, H, WIDE, TS>(ts, off, ptr);
    }
  }
}
// Entry of a stretch.  When all its hoisted loads read plain 32-bit elements and all of them
// (or none) are 128-bit runs, every address is computed first and the loads follow without a
// branch between them, so that they are in flight together; otherwise one after the other.
template <class P, int R, int K, int END, class TS>
__device__ __forceinline__ void fx_spec_stretch_entry(const FxCtx& cx, const FxCoord<R>& q, TS& ts, uint32_t M,
                                                      const FxRegs& rg) {
  constexpr int H = fx_spec_hoist_count<P>(K, END);
  if constexpr (H >= 2 && fx_spec_hoist_plain<P>(K, END)) {
    uint32_t off[H][FX_V];
    uint64_t ptr[H];
    int n_consecutive = 0;
    fx_spec_pf_addr<P, R, K, END, 0, H>(cx, q, M, rg, off, ptr, n_consecutive);
    const uint32_t VM = (1u << FX_V) - 1u;
    const bool whole = !wave_any(M != 0u && M != VM) && wave_any(M == VM);   // as in fx_load_vec
    if (n_consecutive == 0 || !whole) fx_spec_pf_load<P, K, END, 0, H, false, TS>(ts, off, ptr);
    else if (n_consecutive == H) fx_spec_pf_load<P, K, END, 0, H, true, TS>(ts, off, ptr);
    else fx_spec_prefetch<P, R, K, END, TS>(cx, q, ts, M, rg);
  } else if constexpr (H >= 1) {
    fx_spec_prefetch<P, R, K, END, TS>(cx, q, ts, M, rg);
  }
}

// instructions [PC, END) of program table P
template <class P, int R, int PC, int END, class TS>
__device__ __forceinline__ void fx_spec_range(const FxCtx& cx, const FxCoord<R>& q, TS& ts, uint32_t& M,
                                              uint32_t (&A)[FX_V], FxRegs& rg) {
  if constexpr (PC < END) {
    constexpr FxInsn I = P::code[PC];
    constexpr uint32_t w0 = (uint32_t)I.op | ((uint32_t)I.flags << 16) | ((uint32_t)I.dt << 24);
    if constexpr (I.op == FX_MIF || I.op == FX_MIFR || I.op == FX_MELSE) {
      // [PC + 1, I.a) runs under the new mask, and only if a lane of the wave is live
      static_assert(I.a > PC && I.a <= END, "predicated region leaves its program");
      bool skip = false;
      fx_step<R>(cx, q, ts, w0, I.a, I.b, I.imm, M, A, rg, [&](int32_t) { skip = true; });
      if (!skip) fx_spec_range<P, R, PC + 1, I.a, TS>(cx, q, ts, M, A, rg);
      fx_spec_range<P, R, I.a, END, TS>(cx, q, ts, M, A, rg);
    } else if constexpr (I.op == FX_RBEGIN) {
      // body [PC + 1, I.b - 1), closed by the RNEXT at I.b - 1
      constexpr int32_t ext = (int32_t)I.imm;
      static_assert(I.b > PC + 1 && I.b <= END && P::code[I.b - 1].op == FX_RNEXT, "malformed reduction loop");
      if constexpr ((I.a & 1) == 0) { rg.lc0 = 0; rg.le0 = ext; } else { rg.lc1 = 0; rg.le1 = ext; }
      for (int32_t it = 0; it < ext; ++it) {
        if constexpr ((I.a & 1) == 0) rg.lc0 = it; else rg.lc1 = it;
        fx_spec_range<P, R, PC + 1, I.b - 1, TS>(cx, q, ts, M, A, rg);
      }
      fx_spec_range<P, R, I.b, END, TS>(cx, q, ts, M, A, rg);
    } else {
      static_assert(I.op != FX_RNEXT, "loop edge outside a loop");
      if constexpr (fx_spec_stretch_start<P>(PC))
        fx_spec_stretch_entry<P, R, PC, fx_spec_stretch_end<P>(PC), TS>(cx, q, ts, M, rg);
      constexpr int src = fx_spec_reuse<P>(PC) >= 0 ? fx_spec_reuse<P>(PC) : (fx_spec_hoisted<P>(PC) ? PC : -1);
      if constexpr (src >= 0) {
        if constexpr (I.op == FX_LDA) {
#pragma unroll
          for (int j = 0; j < FX_V; ++j) A[j] = ts.ld[src][j];
        } else {
#pragma unroll
          for (int j = 0; j < FX_V; ++j) rg.B[j] = ts.ld[src][j];
          // the rest of the instruction, with its second operand in place (LDB is done)
          if constexpr (I.op != FX_LDB)
            fx_step<R>(cx, q, ts, w0 & ~((uint32_t)FX_F_MEMB << 16), I.a, I.b, I.imm, M, A, rg, [](int32_t) {});
        }
      } else {
        fx_step<R>(cx, q, ts, w0, I.a, I.b, I.imm, M, A, rg, [](int32_t) {});
        if constexpr (fx_spec_reused<P>(PC)) {
#pragma unroll
          for (int j = 0; j < FX_V; ++j) ts.ld[PC][j] = I.op == FX_LDA ? A[j] : rg.B[j];
        }
      }
      fx_spec_range<P, R, PC + 1, END, TS>(cx, q, ts, M, A, rg);
    }
  }
}

template <class P, int PC, int END, int N>
__device__ __forceinline__ void fx_spec_pure(uint32_t (&X)[N]) {
  if constexpr (PC < END) {
    constexpr FxInsn I = P::code[PC];
    fx_pure_step(I.op, I.imm, X);
    fx_spec_pure<P, PC + 1, END, N>(X);
  }
}

// Run policy of the kernels.  The kernels name a program by its first instruction; the
// entry table of P says which ranges can be asked for.
template <class P>
struct FxSpec {
  template <int R, int KIND, int E>
  static __device__ __forceinline__ void dispatch(const FxCtx& cx, int pc, const FxCoord<R>& q, uint32_t M,
                                                  uint32_t (&A)[FX_V]) {
    if constexpr (E < P::n_entries) {
      constexpr FxSpecEntry en = P::entries[E];
      if constexpr (en.kind == KIND) {
        if (pc == en.begin) {
          FxRegs rg;
          fx_regs_init(rg);
          FxRegTemps<P::n_temps, fx_spec_n_insn<P>()> ts;
          fx_spec_range<P, R, en.begin, en.end>(cx, q, ts, M, A, rg);
          return;
        }
      }
      dispatch<R, KIND, E + 1>(cx, pc, q, M, A);
    }
  }
  template <int R>
  static __device__ __forceinline__ void run(const FxCtx& cx, int pc, int, const FxCoord<R>& q, uint32_t M,
                                             uint32_t (&A)[FX_V]) {
    dispatch<R, 0, 0>(cx, pc, q, M, A);
  }
  static __device__ __forceinline__ void run_mask(const FxCtx& cx, int pc, int, const FxCoord<1>& q, uint32_t M,
                                                  uint32_t (&A)[FX_V]) {
    dispatch<1, 1, 0>(cx, pc, q, M, A);
  }
  template <int E, int N>
  static __device__ __forceinline__ void dispatch_pure(int pc, uint32_t (&X)[N]) {
    if constexpr (E < P::n_entries) {
      constexpr FxSpecEntry en = P::entries[E];
      if constexpr (en.kind == 0 && en.pure != 0) {
        if (pc == en.begin) {
          fx_spec_pure<P, en.begin, en.end, N>(X);
          return;
        }
      }
      dispatch_pure<E + 1, N>(pc, X);
    }
  }
  // compiled code is short: registers are spent on more loads in flight instead
  static constexpr uint32_t kPure = 2 * FX_K;
  // the lean batches of whole-group outputs need few registers per item: twelve in flight
  // (sixteen spill)
  static constexpr uint32_t kRows = FX_SPEC_ROWS;
  // all waves take the narrow outputs first: those share their 128-byte lines, and compiled
  // their programs are too short to be worth overlapping with the wide outputs
  static constexpr int kWalk = 1;
  // Waves per workgroup of the compaction kernel (a power of two, 4 or 8) and the waves per
  // SIMD its register budget is set for.  Eight waves sharing a row tile halve a wave's chain of
  // items for the same set-up, but all tiles of a large launch stay resident only with at most
  // 80 registers (three such workgroups per CU), which these kernels do not reach without
  // spilling: measured slower, so four it is.
  static constexpr uint32_t kWaves = FX_SPEC_WAVES;
  static constexpr uint32_t kOcc = FX_SPEC_OCC;
  template <int N>
  static __device__ __forceinline__ void run_pure(const FxCtx&, int pc, int, uint32_t (&X)[N]) {
    dispatch_pure<0, N>(pc, X);
  }
};

// ---- the lean dense kernel -------------------------------------------------
// fx_region_dense serves every dense region and every element type, and compiled for one
// program it is still tens of kilobytes of code that a workgroup jumps through: on a small
// region the kernel's time is the start of its workgroups (argument segment, descriptor
// staging, instruction fetch), not the data.  Regions of one task class with one or two
// outputs of 32-bit elements (FxLeanArgs, decided at plan time) run this
// kernel instead: unit, output record, leading load and pointers come from a short argument
// block through scalar loads, the leading loads of the unit are issued first, and the
// descriptor is staged into LDS behind them, and only if a program of the region reads it
// (affine maps of further loads, scalars).  Results are those of fx_region_dense bit for bit:
// the same item geometry, the same fx_step / fx_pure_step.
#define FX_AS4 __attribute__((address_space(4)))

template <class P>
constexpr bool fx_spec_reads_descriptor() {
  for (int e = 0; e < P::n_entries; ++e)
    if (P::entries[e].kind == 0 && P::entries[e].pure == 0) return true;
  return false;
}

template <class P, int R, int E, class GETCX>
__device__ __forceinline__ void fx_lean_out(const FX_AS4 uint32_t* od, const uint32_t task, const uint32_t local_block,
                                            const FX_AS4 uint64_t* gp, const uint32_t tp_off, const uint64_t err,
                                            GETCX&& get_cx, const uint32_t lane, const uint32_t wave) {
  constexpr FxSpecEntry en = P::entries[E];
  static_assert(en.kind == 0, "dense regions have output programs only");
  constexpr FxInsn LI = P::code[en.begin > 0 ? en.begin - 1 : 0];   // the leading load, if the output has one
  const bool lead = en.begin > 0 && LI.op == FX_LDA && od[FX_W(FxLeanOut, lead)] != 0;
  // a buffer that does not change with the task was resolved by the host; else its slot is looked up
  auto arg_ptr = [&](uint32_t word, uint32_t slot) -> uint64_t {
    if (slot & FX_SLOT_TASK) return gp[tp_off + (slot & 0xffffu)];
    return ((uint64_t)od[word + 1] << 32) | od[word];
  };
  const uint64_t op = arg_ptr(FX_W(FxLeanOut, out_ptr), od[FX_W(FxLeanOut, ptr_slot)]);
  FxLead ld;
#pragma unroll
  for (int k = 0; k < FX_MAXR; ++k) ld.cf[k] = k < (R > 4 ? FX_MAXR : 4) ? (int32_t)od[FX_W(FxLeanOut, lead_cf) + k] : 0;
  ld.base = (int32_t)od[FX_W(FxLeanOut, lead_base)] + (int32_t)od[FX_W(FxLeanOut, lead_tcoef)] * (int32_t)task;
  ld.p = arg_ptr(FX_W(FxLeanOut, lead_ptr), od[FX_W(FxLeanOut, lead_slot)]);
  ld.err = err;
  ld.dt = LI.dt;
  ld.cvt = (LI.flags & FX_F_I2F) != 0;
  ld.lds = false;
  ld.win = nullptr;
  ld.win_base = 0;

  const uint32_t ublock = local_block - od[FX_W(FxLeanOut, block_begin)];
  const uint32_t obase = od[FX_W(FxLeanOut, task_stride)] * task;
  uint32_t dk[R], mk[R], sk[R];
  dk[0] = mk[0] = sk[0] = 0;
#pragma unroll
  for (int k = 1; k < R; ++k) {
    dk[k] = od[FX_W(FxLeanOut, dms) + 3 * (k - 1)];
    mk[k] = od[FX_W(FxLeanOut, dms) + 3 * (k - 1) + 1];
    sk[k] = od[FX_W(FxLeanOut, dms) + 3 * (k - 1) + 2];
  }
  const uint32_t kmax = od[FX_W(FxLeanOut, unit_items)];   // 1 or FX_K items per wave and unit
  const uint32_t inner = od[FX_W(FxLeanOut, inner)];
  const uint32_t vd = od[FX_W(FxLeanOut, vd)];
  const uint32_t gpr = od[FX_W(FxLeanOut, gpr)];
  const uint32_t gp_magic = od[FX_W(FxLeanOut, gp_magic)], gp_shift = od[FX_W(FxLeanOut, gp_shift)];
  const uint32_t n_groups = od[FX_W(FxLeanOut, n_groups)];   // (rows, for an output whose items are whole rows)
  const uint32_t item0 = ublock * (4u * kmax) + wave * kmax;
  // An output that is reduced over its rows (FX_WMAX / FX_WSUM) takes one row per segment of
  // rowseg lanes, so that the wave-wide reductions see exactly the elements of that row.
  const uint32_t rowseg = od[FX_W(FxLeanOut, rowseg)];
  const uint32_t segsh = 31u - (uint32_t)__builtin_clz(rowseg | 1u);
  const uint32_t rows_per_item = 64u >> segsh;
  const uint32_t n_items = rowseg ? (n_groups + rows_per_item - 1u) / rows_per_item : (n_groups + 63u) / 64u;
  const bool have = item0 < n_items;

  // item k of this wave: 64 lane groups of FX_V consecutive elements along the last dimension
  auto make_item = [&](uint32_t k, uint32_t (&e)[FX_V], uint32_t& M, FxCoord<R>& q) {
    uint32_t row, col0;
    bool live;
    if (rowseg) {
      const uint32_t seg = lane >> segsh;
      row = (item0 + k) * rows_per_item + seg;
      col0 = (lane - seg * rowseg) * FX_V;
      live = row < n_groups;
      if (!live) row = 0;
    } else {
      const uint32_t g = (item0 + k) * 64u + lane;
      live = g < n_groups;
      const uint32_t gg = live ? g : 0u;
      row = fx_fastdiv(gg, gp_magic, gp_shift);
      col0 = (gg - row * gpr) * FX_V;
    }
    M = 0;
#pragma unroll
    for (int j = 0; j < FX_V; ++j) {
      if (live && col0 + j < inner) M |= 1u << j;
      q.cv[j] = (int32_t)(col0 + j);
      e[j] = row * inner + col0 + j;
    }
    q.vd = vd;
    q.step = 1;
    const uint32_t rem = fx_unflatten<R>(row, vd, dk, mk, sk, q.c0);
    q.c0[0] = vd == 0 ? 0 : (int32_t)rem;
  };

  uint32_t A[FX_K][FX_V];
  if (have && lead) {
#pragma unroll
    for (uint32_t k = 0; k < FX_K; ++k) {
      if (k < kmax && item0 + k < n_items) {
        uint32_t e[FX_V], M;
        FxCoord<R> q;
        make_item(k, e, M, q);
        fx_lead_load<R>(ld, q, M, A[k]);
      }
    }
  }
  // every wave of the workgroup comes by here, with or without items: the staging has a barrier
  FxCtx cx = get_cx();
  if (!have) return;
  cx.wseg = rowseg ? rowseg : 64u;
  if constexpr (en.pure != 0) {
#pragma unroll
    for (uint32_t k = 0; k < FX_K; ++k) {
      if (k < kmax && item0 + k < n_items) {
        uint32_t e[FX_V], M;
        FxCoord<R> q;
        make_item(k, e, M, q);
        fx_spec_pure<P, en.begin, en.end, FX_V>(A[k]);
        fx_store_vec(op, obase, e, M, true, FX_F32, FX_VT_F, A[k]);
      }
    }
  } else {
    // one copy of the program: the loop stays rolled, the preloaded values are picked by selects
#pragma unroll 1
    for (uint32_t k = 0; k < FX_K; ++k) {
      if (k < kmax && item0 + k < n_items) {
        uint32_t e[FX_V], M;
        FxCoord<R> q;
        make_item(k, e, M, q);
        uint32_t B[FX_V];
#pragma unroll
        for (int j = 0; j < FX_V; ++j) {
          uint32_t v = A[0][j];
#pragma unroll
          for (uint32_t kk = 1; kk < FX_K; ++kk) v = (k == kk) ? A[kk][j] : v;
          B[j] = lead ? v : 0u;
        }
        FxRegs rg;
        fx_regs_init(rg);
        FxRegTemps<P::n_temps, fx_spec_n_insn<P>()> ts;
        fx_spec_range<P, R, en.begin, en.end>(cx, q, ts, M, B, rg);
        fx_store_vec(op, obase, e, M, true, FX_F32, FX_VT_F, B);
      }
    }
  }
}

template <int R, class P>
__global__ __launch_bounds__(FX_BLOCK, 4) void fx_dense_lean(const uint32_t* __restrict__ sb, const FxLeanArgs) {
  extern __shared__ __attribute__((aligned(16))) uint32_t L[];
  const uint32_t lane = threadIdx.x & 63u, wave = uni(threadIdx.x >> 6);
  // the argument block is read through the argument segment pointer, never by naming the
  // parameter: indexing a by-value aggregate dynamically would copy it to per-lane scratch
  const FX_AS4 uint8_t* ka = (const FX_AS4 uint8_t*)__builtin_amdgcn_kernarg_segment_ptr() + 8;
  const FX_AS4 uint32_t* aw = (const FX_AS4 uint32_t*)ka;
  const FX_AS4 uint64_t* gp = (const FX_AS4 uint64_t*)(ka + offsetof(FxLeanArgs, p));
  const uint32_t total_units = aw[FX_W(FxLeanArgs, total_units)];
  {
    // A word of every line of the block that the prologue will read, asked for together with the
    // first one: the lines then arrive in one trip instead of one trip per level of the reads.
    constexpr uint32_t LW = 16, N_LINES = (56 + (P::n_entries > 1 ? 2 : 1) * (R > 3 ? 160 : 128)) / 64;
    uint32_t t[N_LINES];
#pragma unroll
    for (uint32_t k = 0; k < N_LINES; ++k) t[k] = aw[(k + 1) * LW - 2];
#pragma unroll
    for (uint32_t k = 0; k < N_LINES; ++k) asm volatile("" : : "s"(t[k]));
  }
  const uint32_t bpt = aw[FX_W(FxLeanArgs, bpt)];
  const uint32_t n_sptr = aw[FX_W(FxLeanArgs, n_sptr)], n_tptr = aw[FX_W(FxLeanArgs, n_tptr)];
  const uint64_t err = ((uint64_t)aw[FX_W(FxLeanArgs, err_ptr) + 1] << 32) | aw[FX_W(FxLeanArgs, err_ptr)];
  constexpr uint32_t OUT0 = FX_W(FxLeanArgs, out), OUTW = sizeof(FxLeanOut) / 4;
  bool staged = false;
  for (uint32_t unit = blockIdx.x; unit < total_units; unit += gridDim.x) {
    const uint32_t task = fx_fastdiv(unit, aw[FX_W(FxLeanArgs, bpt_magic)], aw[FX_W(FxLeanArgs, bpt_shift)]);
    const uint32_t local_block = unit - task * bpt;
    auto get_cx = [&]() -> FxCtx {
      FxCtx cx{};
      if constexpr (fx_spec_reads_descriptor<P>()) {
        const uint32_t blob_words = aw[FX_W(FxLeanArgs, blob_words)];
        const uint32_t n_p = aw[FX_W(FxLeanArgs, n_p)], n_s = aw[FX_W(FxLeanArgs, n_s)];
        if (!staged) {
          // LDS layout of fx_stage: [descriptor][pointers: 2 words each][scalars]
          const FX_AS1 fx_u32x4* g4 = (const FX_AS1 fx_u32x4*)sb;
          fx_u32x4* l4 = (fx_u32x4*)L;
          for (uint32_t i = threadIdx.x; i < blob_words / 4; i += FX_BLOCK) l4[i] = g4[i];
          const FX_AS4 uint32_t* gs = (const FX_AS4 uint32_t*)(ka + offsetof(FxLeanArgs, s));
          uint64_t* lp = (uint64_t*)(L + blob_words);
          uint32_t* ls = L + blob_words + 2 * n_p;
          for (uint32_t i = threadIdx.x; i < n_p; i += FX_BLOCK) lp[i] = gp[i];
          for (uint32_t i = threadIdx.x; i < n_s; i += FX_BLOCK) ls[i] = gs[i];
          __syncthreads();
          staged = true;
        }
        FxLaunch la;
        la.blob_words = blob_words;
        la.n_p = n_p;
        la.temps_off = (blob_words + 2 * n_p + n_s + 3u) & ~3u;
        FxWork w;
        w.cls = L + aw[FX_W(FxLeanArgs, cls_off)];
        w.task = (int)task;
        w.local_block = local_block;
        cx = fx_make_ctx(L, la, w);
      }
      return cx;
    };
    const uint32_t tp_off = n_sptr + task * n_tptr;
    if constexpr (P::n_entries > 1) {
      if (local_block >= aw[FX_W(FxLeanArgs, second_begin)]) {
        fx_lean_out<P, R, 1>(aw + OUT0 + OUTW, task, local_block, gp, tp_off, err, get_cx, lane, wave);
        continue;
      }
    }
    fx_lean_out<P, R, 0>(aw + OUT0, task, local_block, gp, tp_off, err, get_cx, lane, wave);
  }
}

template <int R, class P>
const void* fx_spec_lean_kernel() {
  if constexpr (P::n_entries <= FX_FAST_OUTS) return (const void*)&fx_dense_lean<R, P>;
  else return nullptr;
}

struct FxSpecRegistrar {
  FxSpecRegistrar(uint64_t hash, const void* dense, const void* count, const void* scatter, uint32_t scatter_threads,
                  const void* stream = nullptr, const void* lean = nullptr, bool lean_stages = false) {
    FxSpecKernels k;
    k.lean = lean;
    k.lean_stages = lean_stages;
    k.dense = dense;
    k.count = count;
    k.scatter = scatter;
    k.scatter_threads = scatter_threads;
    k.stream = stream;
    fx_spec_register(hash, k);
  }
};

}  // namespace

// (the lean kernel has compile-time code for at most FX_FAST_OUTS outputs)
#define FX_SPEC_DENSE(P, R)                                                                                         \
  static FxSpecRegistrar fx_registrar_##P(P::hash, (const void*)&fx_region_dense<R, FxSpec<P>>, nullptr, nullptr, 0, \
                                          nullptr, fx_spec_lean_kernel<R, P>(), fx_spec_reads_descriptor<P>());
#define FX_SPEC_COMPACT(P, R)                                                                    \
  static FxSpecRegistrar fx_registrar_##P(P::hash, nullptr, (const void*)&fx_compact_count<FxSpec<P>>, \
                                          (const void*)&fx_compact_scatter<R, FxSpec<P>>, 64u * FxSpec<P>::kWaves, \
                                          (const void*)&fx_compact_stream<R, FxSpec<P>>);
