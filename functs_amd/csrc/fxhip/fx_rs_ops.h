// Scalar forms of the region instruction set, one function per operation, for code that the
// row-stream generator (fx_rs_gen.cpp) writes: a generated translation unit is straight-line
// calls of these on 32-bit values.  Each body repeats the expression of fx_step
// (fx_device.h) for one element, with the same device functions, so generated code and the
// generic kernels agree bit for bit.
//
// The includer provides FX_RS_FN (function qualifiers), u2f / f2u, floordiv_i / pymod_i,
// fx_fmin / fx_fmax and the three transcendental routines rs_sigmoid / rs_exp / rs_tanh:
// fx_rowstream.h maps them to the device routines, the CPU test harness
// (tests/support/fx_rs_host.cpp) to the ones of the bytecode emulator.
//
// Stands where the reference prints one CUDA expression per NNC node
// (fait/tensorexpr/cuda_codegen_tssa.cpp:641-847, CudaPrinterTssa).
#pragma once
#include <math.h>
#include <stdint.h>

#include "fx_bytecode.h"

#define RS_UN_F(name, expr) \
  FX_RS_FN uint32_t rs_##name(uint32_t x) { const float a = u2f(x); return f2u(expr); }
#define RS_UN_I(name, expr) \
  FX_RS_FN uint32_t rs_##name(uint32_t x) { const int32_t a = (int32_t)x; return (uint32_t)(expr); }
#define RS_BIN_F(name, expr) \
  FX_RS_FN uint32_t rs_##name(uint32_t x, uint32_t y) { const float a = u2f(x), b = u2f(y); return f2u(expr); }
#define RS_CMP_F(name, expr) \
  FX_RS_FN uint32_t rs_##name(uint32_t x, uint32_t y) { const float a = u2f(x), b = u2f(y); return (expr) ? 1u : 0u; }
#define RS_BIN_I(name, expr) \
  FX_RS_FN uint32_t rs_##name(uint32_t x, uint32_t y) { const int32_t a = (int32_t)x, b = (int32_t)y; return (uint32_t)(expr); }

RS_UN_F(FNEG, -a)
RS_UN_F(FABS, fabsf(a))
RS_UN_F(EXP, rs_exp(a))
RS_UN_F(LOG, logf(a))
RS_UN_F(SQRT, sqrtf(a))
RS_UN_F(RSQRT, 1.0f / sqrtf(a))
RS_UN_F(RCP, 1.0f / a)
RS_UN_F(SIGMOID, rs_sigmoid(a))
RS_UN_F(TANH, rs_tanh(a))
RS_UN_F(RELU, (a <= 0.0f) ? 0.0f : a)
RS_UN_F(FLOOR, floorf(a))
RS_UN_F(CEIL, ceilf(a))
RS_UN_F(ROUND, rintf(a))
RS_UN_F(TRUNC, truncf(a))
RS_UN_F(SIN, sinf(a))
RS_UN_F(COS, cosf(a))
RS_UN_F(ERF, erff(a))
RS_UN_F(LOG2, log2f(a))
RS_UN_F(EXP2, exp2f(a))
RS_UN_F(EXPM1, expm1f(a))
RS_UN_F(LOG1P, log1pf(a))

RS_UN_I(INEG, -a)
RS_UN_I(IABS, a < 0 ? -a : a)
RS_UN_I(LNOT, a == 0 ? 1 : 0)
RS_UN_I(INZ, a != 0 ? 1 : 0)
FX_RS_FN uint32_t rs_FNZ(uint32_t x) { return (u2f(x) != 0.0f) ? 1u : 0u; }
FX_RS_FN uint32_t rs_F2I(uint32_t x) { return (uint32_t)(int32_t)u2f(x); }
FX_RS_FN uint32_t rs_I2F(uint32_t x) { return f2u((float)(int32_t)x); }

RS_BIN_F(FADD, a + b)
RS_BIN_F(FSUB, a - b)
RS_BIN_F(FRSUB, b - a)
RS_BIN_F(FMUL, a * b)
RS_BIN_F(FDIV, a / b)
RS_BIN_F(FRDIV, b / a)
RS_BIN_F(FMIN, fx_fmin(a, b))
RS_BIN_F(FMAX, fx_fmax(a, b))
RS_BIN_F(FPOW, powf(a, b))
RS_BIN_F(FMOD, fmodf(a, b))
RS_BIN_F(ATAN2, atan2f(a, b))

RS_BIN_I(IADD, a + b)
RS_BIN_I(ISUB, a - b)
RS_BIN_I(IRSUB, b - a)
RS_BIN_I(IMUL, a * b)
RS_BIN_I(IFDIV, floordiv_i(a, b))
RS_BIN_I(ITDIV, b == 0 ? 0 : a / b)
RS_BIN_I(IPMOD, pymod_i(a, b))
RS_BIN_I(ITMOD, b == 0 ? 0 : a % b)
RS_BIN_I(IMIN, a < b ? a : b)
RS_BIN_I(IMAX, a > b ? a : b)
RS_BIN_I(IAND, a & b)
RS_BIN_I(IOR, a | b)
RS_BIN_I(IXOR, a ^ b)

RS_CMP_F(FLT, a < b)
RS_CMP_F(FLE, a <= b)
RS_CMP_F(FGT, a > b)
RS_CMP_F(FGE, a >= b)
RS_CMP_F(FEQ, a == b)
RS_CMP_F(FNE, a != b)
RS_BIN_I(ILT, a < b ? 1 : 0)
RS_BIN_I(ILE, a <= b ? 1 : 0)
RS_BIN_I(IGT, a > b ? 1 : 0)
RS_BIN_I(IGE, a >= b ? 1 : 0)
RS_BIN_I(IEQ, a == b ? 1 : 0)
RS_BIN_I(INE, a != b ? 1 : 0)

// FX_IRANGE: lo <= a < hi and (a - lo) a multiple of st
FX_RS_FN uint32_t rs_IRANGE(uint32_t x, int32_t lo, int32_t hi, int32_t st) {
  const int32_t a = (int32_t)x;
  bool in = (a >= lo) && (a < hi);
  if (st > 1) in = in && (((a - lo) % st) == 0);
  return in ? 1u : 0u;
}
// FX_MIFR's predicate on the value of its affine record: 0 <= x < hi and x a multiple of st
FX_RS_FN bool rs_INR(uint32_t x, uint32_t hi, int32_t st) {
  bool in = x < hi;
  if (st > 1) in = in && (((int32_t)x % st) == 0);
  return in;
}
FX_RS_FN uint32_t rs_SEL(bool c, uint32_t a, uint32_t b) { return c ? a : b; }

// ---- vector segments: four columns per lane -------------------------------------------
// Thread `tid` of `nt` works on groups tid, tid + nt, ... of the n_kept x ceil(len / 4) groups of
// segment V of the kept rows of a sub-tile: rowmap[r] is the row's place in the window Wb (rows
// of P::S elements), rs0 the index of the window's first row in the task, orow the compacted
// index of the sub-tile's first kept row.  RT: the run-time accessors of the includer.
template <class... T>
struct FxRsList {};

template <class V, class P, class RT>
FX_RS_FN void fx_rs_segment(const RT& rt, const uint32_t* Wb, const uint32_t* rowmap, uint32_t n_kept, uint32_t rs0,
                            uint32_t orow, uint32_t tid, uint32_t nt) {
  constexpr uint32_t G = (V::len + 3u) / 4u;
  constexpr bool raw = (V::dtype == FX_F32 && V::vt == FX_VT_F) || (V::dtype == FX_I32 && V::vt == FX_VT_I);
  const uint32_t ng = n_kept * G;
#pragma unroll 2
  for (uint32_t g = tid; g < ng; g += nt) {
    const uint32_t r = g / G, t0 = (g - r * G) * 4u;
    const uint32_t src = rowmap[r];
    const uint32_t* W = Wb + src * P::S;
    const uint32_t row = rs0 + src;
    uint32_t v[4];
#pragma unroll
    for (uint32_t j = 0; j < 4u; ++j) {
      // the last group of a row may hold fewer than four columns: the others repeat the last one
      const uint32_t t = (V::len % 4u == 0u || t0 + j < V::len) ? t0 + j : V::len - 1u;
      v[j] = V::template elem<RT>(rt, W, row, t);
    }
    if constexpr (V::staged) {
      // the output is put together in LDS (fx_rs_copy_out writes it): row r of the sub-tile's kept rows
#pragma unroll
      for (uint32_t j = 0; j < 4u; ++j)
        if (V::len % 4u == 0u || t0 + j < V::len) rs_stl(rt, V::out, r * V::rowlen + V::col0 + t0 + j, v[j]);
      continue;
    }
    const uint32_t o0 = (orow + r) * V::rowlen + V::col0 + t0;
    if (raw && (V::len % 4u == 0u || t0 + 4u <= V::len)) {
      rs_st4(rt, V::out, o0, v[0], v[1], v[2], v[3]);
    } else {
#pragma unroll
      for (uint32_t j = 0; j < 4u; ++j)
        if (t0 + j < V::len) rs_st<V::dtype, V::vt>(rt, V::out, o0 + j, v[j]);
    }
  }
}
// phase in memory of the run of staged output K that starts at kept row orow
template <class P, uint32_t K, class RT>
FX_RS_FN void fx_rs_phases(RT& rt, uint32_t orow) {
  if constexpr (K < P::n_out) {
    if constexpr (P::stage_rowlen[K] != 0u) rt.ph[K] = (rt.ooff(K) + orow * P::stage_rowlen[K]) & 3u;
    fx_rs_phases<P, K + 1u, RT>(rt, orow);
  }
}
// The kept rows of a sub-tile of staged output K leave LDS as one run of n_kept * rowlen
// consecutive elements from element e0 of the output: whole 16-byte groups where memory has them,
// single elements at the two ends.  rt.staged(K) holds the run at the same phase as memory
// (element i of the run at index (e0 & 3) + i), so the groups are aligned on both sides.
template <class P, uint32_t K, class RT>
FX_RS_FN void fx_rs_copy_out(const RT& rt, uint32_t n_kept, uint32_t orow, uint32_t tid, uint32_t nt) {
  if constexpr (K < P::n_out) {
    constexpr uint32_t RL = P::stage_rowlen[K];
    if constexpr (RL != 0u) {
      const uint32_t n = n_kept * RL;
      const uint32_t e0 = rt.ooff(K) + orow * RL, ph = rt.ph[K];   // = e0 & 3 (fx_rs_phases)
      const uint32_t* src = rt.staged(K);   // element i of the run at src[ph + i]
      const uint32_t head = n < ((4u - ph) & 3u) ? n : ((4u - ph) & 3u);
      const uint32_t groups = (n - head) >> 2, tail = (n - head) & 3u;
      for (uint32_t g = tid; g < groups; g += nt) {
        const uint32_t i = ph + head + 4u * g;   // a multiple of four
        rs_st4_at(rt, K, e0 - ph + i, src[i], src[i + 1u], src[i + 2u], src[i + 3u]);
      }
      for (uint32_t i = tid; i < head; i += nt) rs_st_at(rt, K, e0 + i, src[ph + i]);
      for (uint32_t i = tid; i < tail; i += nt) rs_st_at(rt, K, e0 + head + 4u * groups + i, src[ph + head + 4u * groups + i]);
    }
    fx_rs_copy_out<P, K + 1u, RT>(rt, n_kept, orow, tid, nt);
  }
}

template <class P, class RT>
FX_RS_FN void fx_rs_segments(FxRsList<>, const RT&, const uint32_t*, const uint32_t*, uint32_t, uint32_t, uint32_t, uint32_t,
                             uint32_t) {}
template <class P, class RT, class V, class... Vs>
FX_RS_FN void fx_rs_segments(FxRsList<V, Vs...>, const RT& rt, const uint32_t* Wb, const uint32_t* rowmap, uint32_t n_kept,
                             uint32_t rs0, uint32_t orow, uint32_t tid, uint32_t nt) {
  fx_rs_segment<V, P, RT>(rt, Wb, rowmap, n_kept, rs0, orow, tid, nt);
  fx_rs_segments<P, RT>(FxRsList<Vs...>{}, rt, Wb, rowmap, n_kept, rs0, orow, tid, nt);
}

#undef RS_UN_F
#undef RS_UN_I
#undef RS_BIN_F
#undef RS_CMP_F
#undef RS_BIN_I
