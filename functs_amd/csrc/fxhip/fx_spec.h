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
};
void fx_spec_register(uint64_t hash, const FxSpecKernels& k);
const FxSpecKernels* fx_spec_find(uint64_t hash);

namespace {

struct FxSpecEntry {
  int begin, end;  // instruction range; an output program is entered behind its leading load
  int kind;        // 0: output program, 1: mask program of a row compaction
  int pure;        // output program that the batched path may run
};

template <int N>
struct FxRegTemps {
  uint32_t v[N > 0 ? N : 1][FX_V];
  __device__ __forceinline__ uint32_t& at(int32_t slot, int j) { return v[slot][j]; }
};

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
      fx_step<R>(cx, q, ts, w0, I.a, I.b, I.imm, M, A, rg, [](int32_t) {});
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
          FxRegTemps<P::n_temps> ts = {};
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
  // all waves take the narrow outputs first: those share their 128-byte lines, and compiled
  // their programs are too short to be worth overlapping with the wide outputs
  static constexpr int kWalk = 1;
  // Eight waves share a row tile of the compaction kernel: the set-up of a tile (descriptor
  // copy, offset, row map) is paid once, a wave's chain of items is half as long, and with
  // 80 registers three such workgroups fit a CU, so a launch of up to 768 tiles is resident at once.
  static constexpr uint32_t kWaves = FX_SPEC_WAVES;
  static constexpr uint32_t kOcc = FX_SPEC_OCC;
  template <int N>
  static __device__ __forceinline__ void run_pure(const FxCtx&, int pc, int, uint32_t (&X)[N]) {
    dispatch_pure<0, N>(pc, X);
  }
};

struct FxSpecRegistrar {
  FxSpecRegistrar(uint64_t hash, const void* dense, const void* count, const void* scatter, uint32_t scatter_threads) {
    FxSpecKernels k;
    k.dense = dense;
    k.count = count;
    k.scatter = scatter;
    k.scatter_threads = scatter_threads;
    fx_spec_register(hash, k);
  }
};

}  // namespace

#define FX_SPEC_DENSE(P, R) \
  static FxSpecRegistrar fx_registrar_##P(P::hash, (const void*)&fx_region_dense<R, FxSpec<P>>, nullptr, nullptr, 0);
#define FX_SPEC_COMPACT(P, R)                                                                    \
  static FxSpecRegistrar fx_registrar_##P(P::hash, nullptr, (const void*)&fx_compact_count<FxSpec<P>>, \
                                          (const void*)&fx_compact_scatter<R, FxSpec<P>>, 64u * FxSpec<P>::kWaves);
