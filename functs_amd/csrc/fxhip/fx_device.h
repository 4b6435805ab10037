// Device side of the fused-region backend: the bytecode interpreter and the three region
// kernels, as templates.  fx_kernels.hip instantiates them for the interpreter; a specialised
// region (fx_spec.h) instantiates them again with its program resolved at compile time.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stddef.h>
#include <stdint.h>

#include "fx_bytecode.h"

namespace {

#define FX_AS1 __attribute__((address_space(1)))
#define FX_AS4 __attribute__((address_space(4)))
typedef uint32_t fx_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t fx_u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));  // 128 bits, 4-byte aligned

// word offset of a field inside a blob structure
#define FX_W(Type, field) (offsetof(Type, field) / 4)

__device__ __forceinline__ uint32_t uni(uint32_t x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ bool wave_any(bool p) { return __builtin_amdgcn_ballot_w64(p) != 0ull; }
__device__ __forceinline__ float u2f(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __float_as_uint(f); }

#define FX_SIDE_WIN 2
struct FxCtx {
  const fx_u32x4* insn;   // LDS: class instruction base
  const uint32_t* aff;    // LDS: class affine base (FX_AFF_WORDS words each)
  const uint64_t* ptrs;   // LDS: [shared ptrs][task 0 ptrs][task 1 ptrs]...
  const uint32_t* scal;   // LDS: [shared scalars][task 0 scalars]...
  uint32_t tp_off;        // index of this task's first pointer
  uint32_t ts_off;        // index of this task's first scalar
  uint32_t* temps;        // LDS, this lane's column: temps[(slot * FX_V + j) * FX_BLOCK]
  uint32_t wseg;          // lanes per segment of the wave reductions (rows per wave = 64 / wseg)
  int task;
  uint64_t err;           // error word that guarded int64 loads report to (0: the region has none)
  // Streaming row compaction: the rows of the tile of the region's widest row-major input sit in
  // LDS; affine loads of that buffer read them there.  win[off - win_base] is element `off` of
  // the buffer (nullptr: no window, every load goes to memory).
  // all_win is a compile-time fact wherever a context is used (set from a constant next to
  // where the context is made; everything is inlined): with it, EVERY affine load of the
  // region's programs reads a window (the host only plans such regions for the streaming
  // kernel), so the code holds no load from memory at all and a wave never waits for the
  // memory pipeline (which would also mean waiting for every store it has issued).
  bool all_win;
  const uint32_t* win;
  int32_t win_slot;
  int32_t win_base;
  // the same for up to FX_SIDE_WIN narrow inputs that are read row by row (anchor tables ...)
  const uint32_t* side[FX_SIDE_WIN];
  int32_t side_slot[FX_SIDE_WIN];
  int32_t side_base[FX_SIDE_WIN];
};

// Data buffers are plain device allocations: address them through the global
// address space (global_load / global_store instead of flat accesses).
// `base_` is wave-uniform (kept in SGPRs by the callers) and `off` is an
// element index below 2^31 / element size: the access is base + 32-bit byte
// offset, which needs no 64-bit vector arithmetic.
// FX_V loads of one instruction.  All of them are issued before anything looks
// at loaded data (no conversion, no select between a loaded and an older value),
// so a wave pays the memory latency once per instruction and the loads of a
// following instruction overlap as well.  Elements that are not live read
// element 0 of the buffer and end up with an unspecified value, like after any
// arithmetic instruction; the host never passes a buffer without an element 0.
__device__ __forceinline__ void fx_load_vec(uint64_t base_, const int32_t (&off)[FX_V], uint32_t M, uint32_t dt,
                                            bool cvt, bool consecutive, uint32_t (&out)[FX_V], uint64_t err = 0) {
  const FX_AS1 uint8_t* base = (const FX_AS1 uint8_t*)base_;
  const uint32_t VM = (1u << FX_V) - 1u;
  // FX_V consecutive 32-bit elements in every lane that is live at all, and at least
  // one such lane (so the buffer holds FX_V elements): one 128-bit load per lane.
  // It needs 4-byte alignment only.
  if (consecutive && (dt == FX_F32 || dt == FX_I32) && !wave_any(M != 0u && M != VM) && wave_any(M == VM)) {
    const uint32_t o0 = M ? (uint32_t)off[0] : 0u;
    const fx_u32x4_a4 v = *(const FX_AS1 fx_u32x4_a4*)(base + (o0 << 2));
    out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
    if (cvt) {
      asm volatile("" ::: "memory");
#pragma unroll
      for (int j = 0; j < FX_V; ++j) out[j] = f2u((float)(int32_t)out[j]);
    }
    return;
  }
  uint32_t o[FX_V];
#pragma unroll
  for (int j = 0; j < FX_V; ++j) o[j] = ((M >> j) & 1u) ? (uint32_t)off[j] : 0u;
  if (dt == FX_F32 || dt == FX_I32) {
#pragma unroll
    for (int j = 0; j < FX_V; ++j) out[j] = *(const FX_AS1 uint32_t*)(base + (o[j] << 2));
  } else if (dt == FX_I64) {
    // int64 data in 32-bit arithmetic: the whole element is read.  Converted to float it is
    // exact; as an integer the low word is the value, and an element that does not fit 32 bits
    // is reported through the error word (the result of this launch is then not to be used).
    uint64_t w[FX_V];
#pragma unroll
    for (int j = 0; j < FX_V; ++j) w[j] = *(const FX_AS1 uint64_t*)(base + (o[j] << 3));
    if (cvt) {
#pragma unroll
      for (int j = 0; j < FX_V; ++j) out[j] = f2u((float)(int64_t)w[j]);
      return;
    }
    bool bad = false;
#pragma unroll
    for (int j = 0; j < FX_V; ++j) {
      out[j] = (uint32_t)w[j];
      bad = bad || (((M >> j) & 1u) && (int64_t)w[j] != (int64_t)(int32_t)(uint32_t)w[j]);
    }
    if (bad && err) __hip_atomic_store((uint32_t*)err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  } else if (dt == FX_I64LO || dt == FX_I64HI) {
    const uint32_t hi = dt == FX_I64HI ? 4u : 0u;
#pragma unroll
    for (int j = 0; j < FX_V; ++j) out[j] = *(const FX_AS1 uint32_t*)(base + (o[j] << 3) + hi);
  } else if (dt == FX_U8) {
#pragma unroll
    for (int j = 0; j < FX_V; ++j) out[j] = base[o[j]];
  } else {
    uint32_t h[FX_V];
#pragma unroll
    for (int j = 0; j < FX_V; ++j) h[j] = *(const FX_AS1 uint16_t*)(base + (o[j] << 1));
    if (dt == FX_F16) {
#pragma unroll
      for (int j = 0; j < FX_V; ++j) out[j] = f2u(__half2float(__ushort_as_half((uint16_t)h[j])));
    } else {
#pragma unroll
      for (int j = 0; j < FX_V; ++j) out[j] = h[j] << 16;
    }
  }
  if (cvt) {
    // a real branch: folded into selects, the conversion would need the data at once
    asm volatile("" ::: "memory");
#pragma unroll
    for (int j = 0; j < FX_V; ++j) out[j] = f2u((float)(int32_t)out[j]);
  }
}

__device__ __forceinline__ void fx_store(uint64_t base_, uint32_t o, uint32_t dt, uint32_t vt, uint32_t v) {
  FX_AS1 uint8_t* base = (FX_AS1 uint8_t*)base_;
  switch (dt) {
    case FX_F32: *(FX_AS1 uint32_t*)(base + (o << 2)) = (vt == FX_VT_F) ? v : f2u((float)(int32_t)v); break;
    case FX_I32: *(FX_AS1 int32_t*)(base + (o << 2)) = (vt == FX_VT_I) ? (int32_t)v : (int32_t)u2f(v); break;
    case FX_I64:
      *(FX_AS1 int64_t*)(base + (o << 3)) = (vt == FX_VT_I) ? (int64_t)(int32_t)v : (int64_t)u2f(v);
      break;
    case FX_I64LO: *(FX_AS1 uint32_t*)(base + (o << 3)) = v; break;
    case FX_I64HI: *(FX_AS1 uint32_t*)(base + (o << 3) + 4u) = v; break;
    case FX_U8: base[o] = (vt == FX_VT_I) ? (uint8_t)v : (uint8_t)(u2f(v) != 0.0f); break;
    case FX_F16: {
      __half hv = __float2half(vt == FX_VT_F ? u2f(v) : (float)(int32_t)v);
      *(FX_AS1 uint16_t*)(base + (o << 1)) = __half_as_ushort(hv);
    } break;
    case FX_BF16: {
      float f = vt == FX_VT_F ? u2f(v) : (float)(int32_t)v;
      uint32_t u = f2u(f);
      uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
      if (f != f) r = 0x7fc0u;
      *(FX_AS1 uint16_t*)(base + (o << 1)) = (uint16_t)r;
    } break;
    default: break;
  }
}

// wave-uniform buffer pointer, returned in scalar registers
__device__ __forceinline__ uint64_t fx_ptr(const FxCtx& cx, int32_t slot) {
  const uint32_t i = (slot & FX_SLOT_TASK) ? cx.tp_off + (uint32_t)(slot & 0xffff) : (uint32_t)(slot & 0xffff);
  const uint64_t p = cx.ptrs[i];
  return ((uint64_t)uni((uint32_t)(p >> 32)) << 32) | (uint64_t)uni((uint32_t)p);
}

// Affine load of an instruction: from the staged window when the buffer is the window's, from
// memory otherwise.  The window holds 32-bit elements (float or int32).
// the staged window that holds buffer `slot` (wave-uniform); selects, no branch
__device__ __forceinline__ const uint32_t* fx_window_of(const FxCtx& cx, uint32_t slot, int32_t& base) {
  const uint32_t* w = cx.win;
  base = cx.win_base;
#pragma unroll
  for (int i = 0; i < FX_SIDE_WIN; ++i) {
    const bool hit = slot == (uint32_t)cx.side_slot[i];
    w = hit ? cx.side[i] : w;
    base = hit ? cx.side_base[i] : base;
  }
  return w;
}

__device__ __forceinline__ void fx_load(const FxCtx& cx, int32_t slot, const int32_t (&off)[FX_V], uint32_t M,
                                        uint32_t dt, bool cvt, bool consecutive, uint32_t (&out)[FX_V]) {
  if (cx.all_win) {
    int32_t wbase;
    const uint32_t* wnd = fx_window_of(cx, uni((uint32_t)slot), wbase);
#pragma unroll
    for (int j = 0; j < FX_V; ++j) out[j] = wnd[((M >> j) & 1u) ? off[j] - wbase : 0];
    if (cvt) {
#pragma unroll
      for (int j = 0; j < FX_V; ++j) out[j] = f2u((float)(int32_t)out[j]);
    }
    return;
  }
  fx_load_vec(fx_ptr(cx, slot), off, M, dt, cvt, consecutive, out, cx.err);
}

__device__ __forceinline__ uint32_t fx_scalar(const FxCtx& cx, int32_t slot) {
  const uint32_t i = (slot & FX_SLOT_TASK) ? cx.ts_off + (uint32_t)(slot & 0xffff) : (uint32_t)(slot & 0xffff);
  return cx.scal[i];
}

__device__ __forceinline__ int32_t floordiv_i(int32_t a, int32_t b) {
  if (b == 0) return 0;
  int32_t q = a / b;
  if ((a % b != 0) && ((a < 0) != (b < 0))) --q;
  return q;
}
__device__ __forceinline__ int32_t pymod_i(int32_t a, int32_t b) {
  if (b == 0) return 0;
  int32_t r = a % b;
  if (r != 0 && ((r < 0) != (b < 0))) r += b;
  return r;
}

// sigmoid(x) = 1 / (1 + 2^(-x * log2 e)).  The product is split into a rounded
// part and its rounding error (hi/lo of log2 e), the error is applied to the
// result as a first-order factor, and the reciprocal is the hardware
// approximation: about 3 ulp in total (3e-7 relative), against a 1e-5 bound,
// for a quarter of the instructions of expf + IEEE division.
__device__ __forceinline__ float fx_sigmoid(float x) {
  const float l2e_hi = 1.44269502e+00f, l2e_lo = 1.92596299e-08f, ln2 = 6.93147182e-01f;
  const float nx = -x;
  const float th = nx * l2e_hi;
  const float tl = __builtin_fmaf(nx, l2e_hi, -th) + nx * l2e_lo;
  float e = __builtin_amdgcn_exp2f(th);
  e = __builtin_fmaf(e, tl * ln2, e);
  float r = __builtin_amdgcn_rcpf(1.0f + e);
  // below about -88.7 (and at -inf) exp2 overflows and the correction term makes inf - inf; at +inf
  // the low word is inf - inf.  NaN inputs fail both comparisons and stay NaN.
  r = (th > 128.0f) ? 0.0f : r;
  r = (th < -150.0f) ? 1.0f : r;
  return r;
}

// exp through the hardware exp2 with a two-word log2(e): about 1.2e-7 relative error
// over the whole range (checked against float64 on 2 M points), a fraction of
// the instructions of the library routine.
__device__ __forceinline__ float fx_exp(float x) {
  const float l2e_hi = 1.44269502e+00f, l2e_lo = 1.92596299e-08f, ln2 = 6.93147182e-01f;
  const float th = x * l2e_hi;
  const float tl = __builtin_fmaf(x, l2e_hi, -th) + x * l2e_lo;
  const float e = __builtin_amdgcn_exp2f(th);
  float r = __builtin_fmaf(e, tl * ln2, e);
  r = (th > 128.0f) ? __builtin_inff() : r;   // also +inf input (tl would be NaN)
  r = (th < -150.0f) ? 0.0f : r;              // also -inf input
  return r;
}

// tanh: odd polynomial below 0.625 (no cancellation), 1 - 2 / (exp(2|x|) + 1) above;
// about 1.5e-7 relative error (checked against float64 on 2 M points).
__device__ __forceinline__ float fx_tanh(float x) {
  const float ax = fabsf(x);
  const float z = x * x;
  float p = -5.70498872745e-3f;
  p = __builtin_fmaf(p, z, 2.06390887954e-2f);
  p = __builtin_fmaf(p, z, -5.37397155531e-2f);
  p = __builtin_fmaf(p, z, 1.33314422036e-1f);
  p = __builtin_fmaf(p, z, -3.33332819422e-1f);
  const float small = __builtin_fmaf(p * z, x, x);
  const float e = fx_exp(2.0f * ax);
  const float big = copysignf(1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f), x);
  return ax < 0.625f ? small : big;
}

// the value of lane (own lane ^ J), inside the vector unit
template <uint32_t J>
__device__ __forceinline__ uint32_t fx_lane_xor(uint32_t v, uint32_t lane) {
  typedef unsigned u32x2v __attribute__((ext_vector_type(2)));
  if constexpr (J == 1u) return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xf, 0xf, false);        // quad_perm [1, 0, 3, 2]
  else if constexpr (J == 2u) return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xf, 0xf, false);   // quad_perm [2, 3, 0, 1]
  else if constexpr (J == 4u) {
    // a rotation of the row of 16 by 4 one way and the other; which of the two is lane ^ 4 depends on bit 2
    const uint32_t from_below = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x124, 0xf, 0xf, false);   // row_ror:4: from lane - 4
    const uint32_t from_above = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x12C, 0xf, 0xf, false);   // row_ror:12: from lane + 4
    return (lane & 4u) ? from_below : from_above;
  } else if constexpr (J == 8u) return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x128, 0xf, 0xf, false);   // row_ror:8
  else if constexpr (J == 16u) {
    const u32x2v t = __builtin_amdgcn_permlane16_swap(v, v, false, false);   // x: rows 0, 0, 2, 2; y: rows 1, 1, 3, 3
    return (lane & 16u) ? t.x : t.y;
  } else {
    const u32x2v t = __builtin_amdgcn_permlane32_swap(v, v, false, false);   // x: lower half twice; y: upper half twice
    return (lane & 32u) ? t.x : t.y;
  }
}
template <uint32_t J>
__device__ __forceinline__ float fx_lane_xor_f(float v, uint32_t lane) {
  return __uint_as_float(fx_lane_xor<J>(__float_as_uint(v), lane));
}

// the sum over the wave, in every lane (integer: the order of the additions does not matter)
__device__ __forceinline__ uint32_t fx_wave_sum(uint32_t v, uint32_t lane) {
  v += fx_lane_xor<32u>(v, lane);
  v += fx_lane_xor<16u>(v, lane);
  v += fx_lane_xor<8u>(v, lane);
  v += fx_lane_xor<4u>(v, lane);
  v += fx_lane_xor<2u>(v, lane);
  v += fx_lane_xor<1u>(v, lane);
  return v;
}

// NaN-propagating min / max (ATen semantics for maximum/minimum/clamp)
__device__ __forceinline__ float fx_fmax(float a, float b) { return (a > b || a != a) ? a : b; }
__device__ __forceinline__ float fx_fmin(float a, float b) { return (a < b || a != a) ? a : b; }


// Coordinates of the FX_V elements a lane works on.  They differ in ONE
// coordinate (vd, wave-uniform): element j has coordinates c0 with c0[vd]
// replaced by cv[j].  `step` (wave-uniform) says cv[j] == cv[0] + j, i.e. the
// lane holds FX_V consecutive elements along dimension vd.
template <int R>
struct FxCoord {
  int32_t c0[R];     // entry vd is 0
  int32_t cv[FX_V];
  uint32_t vd;
  uint32_t step;
};

// off[j] = base + sum_k cf[k] * coordinate_k(element j)
// Returns true (wave-uniform) when off[j] == off[0] + j for every lane.
template <int R>
__device__ __forceinline__ bool fx_offsets(const FxCoord<R>& q, const int32_t (&cf)[FX_MAXR], int32_t base,
                                           int32_t (&off)[FX_V]) {
  int32_t s = base;
#pragma unroll
  for (int k = 0; k < R; ++k) s += cf[k] * q.c0[k];
  int32_t cfv = cf[0];
#pragma unroll
  for (int k = 1; k < R; ++k) cfv = (q.vd == (uint32_t)k) ? cf[k] : cfv;
  if (q.step) {
    const int32_t o0 = s + cfv * q.cv[0];
#pragma unroll
    for (int j = 0; j < FX_V; ++j) off[j] = o0 + j * cfv;
    return uni((uint32_t)cfv) == 1u;
  } else {
#pragma unroll
    for (int j = 0; j < FX_V; ++j) off[j] = s + cfv * q.cv[j];
    return false;
  }
}

// row index (all dimensions but vd, flattened) -> c0[1..R-1]; returns what is
// left for dimension 0.  dk / mk / sk: extent and fast-division constants per dimension.
template <int R>
__device__ __forceinline__ uint32_t fx_unflatten(uint32_t rem, uint32_t vd, const uint32_t (&dk)[R],
                                                 const uint32_t (&mk)[R], const uint32_t (&sk)[R], int32_t (&c0)[R]) {
#pragma unroll
  for (int k = R - 1; k >= 1; --k) {
    if (vd == (uint32_t)k) {
      c0[k] = 0;
    } else {
      const uint32_t d = (__umulhi(rem, mk[k]) + rem) >> sk[k];
      c0[k] = (int32_t)(rem - d * dk[k]);
      rem = d;
    }
  }
  return rem;
}

// Results of one item.  contig (wave-uniform): e[j] == e[0] + j, so a lane whose
// FX_V elements are all live writes them with one 128-bit store.
__device__ __forceinline__ void fx_store_vec(uint64_t base_, uint32_t obase, const uint32_t (&e)[FX_V], uint32_t M,
                                             bool contig, uint32_t dt, uint32_t vt, const uint32_t (&A)[FX_V]) {
  const bool raw32 = (dt == FX_F32 && vt == FX_VT_F) || (dt == FX_I32 && vt == FX_VT_I);
  if (raw32 && contig) {
    FX_AS1 uint8_t* base = (FX_AS1 uint8_t*)base_;
    if (M == (1u << FX_V) - 1u) {
      // The four results pass through an opaque copy: seen as one vector value, the
      // optimiser would turn the interpreter's accumulators into vector registers.
      uint32_t t0 = A[0], t1 = A[1], t2 = A[2], t3 = A[3];
      asm("" : "+v"(t0), "+v"(t1), "+v"(t2), "+v"(t3));
      fx_u32x4 v;
      v.x = t0; v.y = t1; v.z = t2; v.w = t3;
      *(FX_AS1 fx_u32x4_a4*)(base + ((obase + e[0]) << 2)) = v;
    } else {
#pragma unroll
      for (int j = 0; j < FX_V; ++j)
        if ((M >> j) & 1u) *(FX_AS1 uint32_t*)(base + ((obase + e[0] + j) << 2)) = A[j];
    }
  } else {
#pragma unroll
    for (int j = 0; j < FX_V; ++j)
      if ((M >> j) & 1u) fx_store(base_, obase + e[j], dt, vt, A[j]);
  }
}

// Element offsets of affine record `idx` at the FX_V elements of a lane group.
template <int R>
__device__ __forceinline__ bool fx_affine(const FxCtx& cx, const FxCoord<R>& q, int32_t idx, int32_t lc0, int32_t lc1,
                                          int32_t (&off)[FX_V]) {
  const fx_u32x4* ap = (const fx_u32x4*)(cx.aff + idx * FX_AFF_WORDS);
  const fx_u32x4 a0 = ap[0], a1 = ap[1];
  int32_t cf[FX_MAXR];
  cf[0] = (int32_t)a0.x; cf[1] = (int32_t)a0.y; cf[2] = (int32_t)a0.z; cf[3] = (int32_t)a0.w;
  if (R > 4) {
    const fx_u32x4 a2 = ap[2];
    cf[4] = (int32_t)a2.x; cf[5] = (int32_t)a2.y;
  } else {
    cf[4] = 0; cf[5] = 0;
  }
  const int32_t base = (int32_t)a1.y + (int32_t)a1.x * cx.task + (int32_t)a1.z * lc0 + (int32_t)a1.w * lc1;
  return fx_offsets<R>(q, cf, base, off);
}

// Register state of a program besides A: the second operand, the mask stack and the
// counters of the (at most two) nested reduction loops.
struct FxRegs {
  uint32_t B[FX_V];
  uint64_t MS;                  // mask stack, FX_V bits per level
  int32_t lc0, lc1, le0, le1;   // loop counters / extents (wave-uniform)
};
__device__ __forceinline__ void fx_regs_init(FxRegs& r) {
#pragma unroll
  for (int j = 0; j < FX_V; ++j) r.B[j] = 0;
  r.MS = 0;
  r.lc0 = r.lc1 = r.le0 = r.le1 = 0;
}

// Temporaries of the interpreter: one LDS column per lane.
struct FxLdsTemps {
  uint32_t* p;
  __device__ __forceinline__ uint32_t& at(int32_t slot, int j) { return p[(slot * FX_V + j) * FX_BLOCK]; }
};

// One instruction.  `jump(target)` is called when control leaves the straight line (a
// predicated region without a live lane, a loop edge).  With w0 / ia / ib / imm known at
// compile time the switch folds away: specialised regions are built from this function too.
template <int R, class TS, class JF>
__device__ __forceinline__ void fx_step(const FxCtx& cx, const FxCoord<R>& q, TS& ts, const uint32_t w0,
                                        const int32_t ia, const int32_t ib, const uint32_t imm, uint32_t& M,
                                        uint32_t (&A)[FX_V], FxRegs& rg, JF&& jump) {
  uint32_t (&B)[FX_V] = rg.B;
  uint64_t& MS = rg.MS;
  int32_t &lc0 = rg.lc0, &lc1 = rg.lc1, &le0 = rg.le0, &le1 = rg.le1;
  const uint32_t VM = (1u << FX_V) - 1u;
  const uint32_t op = w0 & 0xffffu;
  const bool useimm = (w0 & (FX_F_IMM << 16)) != 0;
  const bool cvt = (w0 & (FX_F_I2F << 16)) != 0;
  const uint32_t dt = w0 >> 24;
#define FX_UNARY_F(expr)                                   \
  {                                                        \
    _Pragma("unroll") for (int j = 0; j < FX_V; ++j) {     \
      float a = u2f(A[j]);                                 \
      A[j] = f2u(expr);                                    \
    }                                                      \
  } break
#define FX_UNARY_I(expr)                                   \
  {                                                        \
    _Pragma("unroll") for (int j = 0; j < FX_V; ++j) {     \
      int32_t a = (int32_t)A[j];                           \
      A[j] = (uint32_t)(expr);                             \
    }                                                      \
  } break
#define FX_BIN_F(expr)                                     \
  {                                                        \
    _Pragma("unroll") for (int j = 0; j < FX_V; ++j) {     \
      float a = u2f(A[j]);                                 \
      float b = u2f(useimm ? imm : B[j]);                  \
      A[j] = f2u(expr);                                    \
    }                                                      \
  } break
#define FX_CMP_F(expr)                                     \
  {                                                        \
    _Pragma("unroll") for (int j = 0; j < FX_V; ++j) {     \
      float a = u2f(A[j]);                                 \
      float b = u2f(useimm ? imm : B[j]);                  \
      A[j] = (expr) ? 1u : 0u;                             \
    }                                                      \
  } break
#define FX_BIN_I(expr)                                     \
  {                                                        \
    _Pragma("unroll") for (int j = 0; j < FX_V; ++j) {     \
      int32_t a = (int32_t)A[j];                           \
      int32_t b = (int32_t)(useimm ? imm : B[j]);          \
      A[j] = (uint32_t)(expr);                             \
    }                                                      \
  } break

    // second operand fetched as part of the instruction (LDB, LDTB and binary operations that
    // took such a load over)
    if (w0 & ((FX_F_MEMB | FX_F_TMPB) << 16)) {
      if (w0 & (FX_F_TMPB << 16)) {
#pragma unroll
        for (int j = 0; j < FX_V; ++j) B[j] = ts.at(ia, j);
      } else {
        int32_t off[FX_V];
        const bool consecutive = fx_affine<R>(cx, q, ib, lc0, lc1, off);
        fx_load(cx, ia, off, M, dt, cvt, consecutive, B);
      }
    }

    switch (op) {
      case FX_NOP: break;
      case FX_LDA:
      case FX_AFFA:
      case FX_AFFB: {
        int32_t off[FX_V];
        const bool consecutive = fx_affine<R>(cx, q, ib, lc0, lc1, off);
        if (op == FX_LDA) {
          fx_load(cx, ia, off, M, dt, cvt, consecutive, A);
        } else {
#pragma unroll
          for (int j = 0; j < FX_V; ++j) {
            const uint32_t v = cvt ? f2u((float)off[j]) : (uint32_t)off[j];
            if (op == FX_AFFA) A[j] = v; else B[j] = v;
          }
        }
      } break;
      case FX_LDB:   // done above: FX_F_MEMB / FX_F_TMPB are always set on these two
      case FX_LDTB:
        break;
      case FX_LDXA: {
        int32_t off[FX_V];
#pragma unroll
        for (int j = 0; j < FX_V; ++j) off[j] = (int32_t)A[j] + (int32_t)imm;
        fx_load_vec(fx_ptr(cx, ia), off, M, dt, false, false, A, cx.err);
      } break;
      case FX_IMMA:
#pragma unroll
        for (int j = 0; j < FX_V; ++j) if ((M >> j) & 1u) A[j] = imm;
        break;
      case FX_IMMB:
#pragma unroll
        for (int j = 0; j < FX_V; ++j) B[j] = imm;
        break;
      case FX_SCLA: {
        uint32_t s = fx_scalar(cx, ia);
        if (cvt) s = f2u((float)(int32_t)s);
#pragma unroll
        for (int j = 0; j < FX_V; ++j) if ((M >> j) & 1u) A[j] = s;
      } break;
      case FX_SCLB: {
        uint32_t s = fx_scalar(cx, ia);
        if (cvt) s = f2u((float)(int32_t)s);
#pragma unroll
        for (int j = 0; j < FX_V; ++j) B[j] = s;
      } break;
      case FX_STT:
#pragma unroll
        for (int j = 0; j < FX_V; ++j) ts.at(ia, j) = A[j];
        break;
      case FX_LDTA:
#pragma unroll
        for (int j = 0; j < FX_V; ++j) if ((M >> j) & 1u) A[j] = ts.at(ia, j);
        break;
      case FX_MOVBA:
#pragma unroll
        for (int j = 0; j < FX_V; ++j) B[j] = A[j];
        break;
      case FX_SWAP:
#pragma unroll
        for (int j = 0; j < FX_V; ++j) { uint32_t t = A[j]; A[j] = B[j]; B[j] = t; }
        break;

      case FX_MIF: {
        MS = (MS << FX_V) | (uint64_t)M;
        uint32_t cnd = 0;
#pragma unroll
        for (int j = 0; j < FX_V; ++j) cnd |= (A[j] != 0u ? 1u : 0u) << j;
        M &= cnd;
        if (!wave_any(M != 0u)) jump(ia);
      } break;
      case FX_MIFR: {
        int32_t off[FX_V];
        fx_affine<R>(cx, q, ib, lc0, lc1, off);
        const uint32_t hi = uni(imm) >> 8;
        const int32_t st = (int32_t)(uni(imm) & 255u);
        MS = (MS << FX_V) | (uint64_t)M;
        uint32_t cnd = 0;
#pragma unroll
        for (int j = 0; j < FX_V; ++j) {
          bool in = (uint32_t)off[j] < hi;
          if (st > 1) in = in && ((off[j] % st) == 0);
          A[j] = in ? 1u : 0u;
          cnd |= (in ? 1u : 0u) << j;
        }
        M &= cnd;
        if (!wave_any(M != 0u)) jump(ia);
      } break;
      case FX_MELSE: {
        uint32_t top = (uint32_t)MS & VM;
        M = top & ~M;
        if (!wave_any(M != 0u)) jump(ia);
      } break;
      case FX_MMERGE: {
#pragma unroll
        for (int j = 0; j < FX_V; ++j) {
          uint32_t t = ts.at(ia, j);
          A[j] = ((M >> j) & 1u) ? A[j] : t;
        }
        M = (uint32_t)MS & VM;
        MS >>= FX_V;
      } break;
      case FX_MEND:
        M = (uint32_t)MS & VM;
        MS >>= FX_V;
        break;

      case FX_FNEG: FX_UNARY_F(-a);
      case FX_FABS: FX_UNARY_F(fabsf(a));
      case FX_EXP: FX_UNARY_F(fx_exp(a));
      case FX_LOG: FX_UNARY_F(logf(a));
      case FX_SQRT: FX_UNARY_F(sqrtf(a));
      case FX_RSQRT: FX_UNARY_F(1.0f / sqrtf(a));
      case FX_RCP: FX_UNARY_F(1.0f / a);
      case FX_SIGMOID: FX_UNARY_F(fx_sigmoid(a));
      case FX_TANH: FX_UNARY_F(fx_tanh(a));
      case FX_RELU: FX_UNARY_F((a <= 0.0f) ? 0.0f : a);
      case FX_FLOOR: FX_UNARY_F(floorf(a));
      case FX_CEIL: FX_UNARY_F(ceilf(a));
      case FX_ROUND: FX_UNARY_F(rintf(a));
      case FX_TRUNC: FX_UNARY_F(truncf(a));
      case FX_SIN: FX_UNARY_F(sinf(a));
      case FX_COS: FX_UNARY_F(cosf(a));
      case FX_ERF: FX_UNARY_F(erff(a));
      case FX_LOG2: FX_UNARY_F(log2f(a));
      case FX_EXP2: FX_UNARY_F(exp2f(a));
      case FX_EXPM1: FX_UNARY_F(expm1f(a));
      case FX_LOG1P: FX_UNARY_F(log1pf(a));

      case FX_INEG: FX_UNARY_I(-a);
      case FX_IABS: FX_UNARY_I(a < 0 ? -a : a);
      case FX_LNOT: FX_UNARY_I(a == 0 ? 1 : 0);
      case FX_INZ: FX_UNARY_I(a != 0 ? 1 : 0);
      case FX_FNZ:
#pragma unroll
        for (int j = 0; j < FX_V; ++j) A[j] = (u2f(A[j]) != 0.0f) ? 1u : 0u;
        break;
      case FX_F2I:
#pragma unroll
        for (int j = 0; j < FX_V; ++j) A[j] = (uint32_t)(int32_t)u2f(A[j]);
        break;
      case FX_I2F:
#pragma unroll
        for (int j = 0; j < FX_V; ++j) A[j] = f2u((float)(int32_t)A[j]);
        break;

      case FX_FADD: FX_BIN_F(a + b);
      case FX_FSUB: FX_BIN_F(a - b);
      case FX_FRSUB: FX_BIN_F(b - a);
      case FX_FMUL: FX_BIN_F(a * b);
      case FX_FDIV: FX_BIN_F(a / b);
      case FX_FRDIV: FX_BIN_F(b / a);
      case FX_FMIN: FX_BIN_F(fx_fmin(a, b));
      case FX_FMAX: FX_BIN_F(fx_fmax(a, b));
      case FX_FPOW: FX_BIN_F(powf(a, b));
      case FX_FMOD: FX_BIN_F(fmodf(a, b));
      case FX_ATAN2: FX_BIN_F(atan2f(a, b));

      case FX_IADD: FX_BIN_I(a + b);
      case FX_ISUB: FX_BIN_I(a - b);
      case FX_IRSUB: FX_BIN_I(b - a);
      case FX_IMUL: FX_BIN_I(a * b);
      case FX_IFDIV: FX_BIN_I(floordiv_i(a, b));
      case FX_ITDIV: FX_BIN_I(b == 0 ? 0 : a / b);
      case FX_IPMOD: FX_BIN_I(pymod_i(a, b));
      case FX_ITMOD: FX_BIN_I(b == 0 ? 0 : a % b);
      case FX_IMIN: FX_BIN_I(a < b ? a : b);
      case FX_IMAX: FX_BIN_I(a > b ? a : b);
      case FX_IAND: FX_BIN_I(a & b);
      case FX_IOR: FX_BIN_I(a | b);
      case FX_IXOR: FX_BIN_I(a ^ b);

      case FX_FLT: FX_CMP_F(a < b);
      case FX_FLE: FX_CMP_F(a <= b);
      case FX_FGT: FX_CMP_F(a > b);
      case FX_FGE: FX_CMP_F(a >= b);
      case FX_FEQ: FX_CMP_F(a == b);
      case FX_FNE: FX_CMP_F(a != b);
      case FX_ILT: FX_BIN_I(a < b ? 1 : 0);
      case FX_ILE: FX_BIN_I(a <= b ? 1 : 0);
      case FX_IGT: FX_BIN_I(a > b ? 1 : 0);
      case FX_IGE: FX_BIN_I(a >= b ? 1 : 0);
      case FX_IEQ: FX_BIN_I(a == b ? 1 : 0);
      case FX_INE: FX_BIN_I(a != b ? 1 : 0);

      case FX_IRANGE: {
        const int32_t lo = ia, hi = ib, st = (int32_t)uni(imm);
#pragma unroll
        for (int j = 0; j < FX_V; ++j) {
          int32_t a = (int32_t)A[j];
          bool in = (a >= lo) && (a < hi);
          if (st > 1) in = in && (((a - lo) % st) == 0);
          A[j] = in ? 1u : 0u;
        }
      } break;
      case FX_WHERE:
#pragma unroll
        for (int j = 0; j < FX_V; ++j) {
          uint32_t cnd = ts.at(ia, j);
          A[j] = cnd != 0u ? A[j] : B[j];
        }
        break;

      case FX_WMAX:
      case FX_WSUM: {
        const bool is_max = op == FX_WMAX;
        float v = is_max ? -__builtin_inff() : 0.0f;
#pragma unroll
        for (int j = 0; j < FX_V; ++j) {
          if ((M >> j) & 1u) v = is_max ? fx_fmax(v, u2f(A[j])) : v + u2f(A[j]);
        }
        // the butterfly stays inside a segment (wave-uniform); the exchanges stay inside the vector unit
        const uint32_t ln = threadIdx.x & 63u;
#define FX_WSTEP(O)                                   \
  if ((uint32_t)(O) < cx.wseg) {                      \
    const float t = fx_lane_xor_f<(O)>(v, ln);        \
    v = is_max ? fx_fmax(v, t) : v + t;               \
  }
        FX_WSTEP(32u) FX_WSTEP(16u) FX_WSTEP(8u) FX_WSTEP(4u) FX_WSTEP(2u) FX_WSTEP(1u)
#undef FX_WSTEP
#pragma unroll
        for (int j = 0; j < FX_V; ++j) A[j] = f2u(v);
      } break;
      case FX_RBEGIN: {
        const uint32_t d = uni((uint32_t)ia) & 1u;
        const int32_t ext = (int32_t)uni(imm);
        if (d == 0) { lc0 = 0; le0 = ext; } else { lc1 = 0; le1 = ext; }
        if (ext <= 0) jump(ib);
      } break;
      case FX_RNEXT: {
        const uint32_t d = uni((uint32_t)ib) & 1u;
        bool again;
        if (d == 0) { lc0 += 1; again = lc0 < le0; } else { lc1 += 1; again = lc1 < le1; }
        if (again) jump(ia);
      } break;
      case FX_RIDX: {
        const int32_t v = (uni((uint32_t)ia) & 1u) ? lc1 : lc0;
#pragma unroll
        for (int j = 0; j < FX_V; ++j) if ((M >> j) & 1u) A[j] = (uint32_t)v;
      } break;
      default: break;
    }
#undef FX_UNARY_F
#undef FX_UNARY_I
#undef FX_BIN_F
#undef FX_CMP_F
#undef FX_BIN_I
}

// The interpreter.  R = number of root coordinates that carry information.
// The program lives in LDS; the next instruction word is fetched while the
// current one executes.  The host pads every program area with one trailing
// NOP so that the look-ahead read stays inside the blob.
template <int R>
__device__ __forceinline__ void fx_run(const FxCtx& cx, int pc, const int pc_end, const FxCoord<R>& q,
                                       uint32_t M, uint32_t (&A)[FX_V]) {
  FxRegs rg;
  fx_regs_init(rg);
  FxLdsTemps ts{cx.temps};
  fx_u32x4 nxt = cx.insn[pc];
  while (pc < pc_end) {
    const fx_u32x4 w = nxt;
    int npc = pc + 1;
    nxt = cx.insn[npc];
    fx_step<R>(cx, q, ts, uni(w.x), (int32_t)w.y, (int32_t)w.z, w.w, M, A, rg, [&](int32_t target) {
      npc = (int)uni((uint32_t)target);
      nxt = cx.insn[npc];
    });
    pc = npc;
  }
}

// Programs that start with an unconditional affine load (flagged by the host in
// FxOut::lead) have that load issued for FX_K work items at once, before any of
// them is computed: FX_K * FX_V loads per lane are in flight instead of FX_V.
// The interpreter then starts behind the load with A preset.
#define FX_K 4
// Interpreter for the tail of a "pure" program (FxOut::pure): coordinate-free
// elementwise instructions with immediate operands.  One pass over the program
// serves the FX_K items of a batch, so fetch and dispatch are paid once per
// FX_K * FX_V elements of a lane.
#define FX_NB (FX_K * FX_V)
template <int N>
__device__ __forceinline__ void fx_pure_step(const uint32_t op, const uint32_t imm, uint32_t (&X)[N]) {
#define FX_PU_F(expr)                                      \
  {                                                        \
    _Pragma("unroll") for (int j = 0; j < N; ++j) {    \
      float a = u2f(X[j]);                                 \
      X[j] = f2u(expr);                                    \
    }                                                      \
  } break
#define FX_PB_F(expr)                                      \
  {                                                        \
    const float b = u2f(imm);                              \
    _Pragma("unroll") for (int j = 0; j < N; ++j) {    \
      float a = u2f(X[j]);                                 \
      X[j] = f2u(expr);                                    \
    }                                                      \
  } break
#define FX_PC_F(expr)                                      \
  {                                                        \
    const float b = u2f(imm);                              \
    _Pragma("unroll") for (int j = 0; j < N; ++j) {    \
      float a = u2f(X[j]);                                 \
      X[j] = (expr) ? 1u : 0u;                             \
    }                                                      \
  } break
    switch (op) {
      case FX_FNEG: FX_PU_F(-a);
      case FX_FABS: FX_PU_F(fabsf(a));
      case FX_EXP: FX_PU_F(fx_exp(a));
      case FX_SQRT: FX_PU_F(sqrtf(a));
      case FX_RSQRT: FX_PU_F(1.0f / sqrtf(a));
      case FX_RCP: FX_PU_F(1.0f / a);
      case FX_SIGMOID: FX_PU_F(fx_sigmoid(a));
      case FX_RELU: FX_PU_F((a <= 0.0f) ? 0.0f : a);
      case FX_F2I:
#pragma unroll
        for (int j = 0; j < N; ++j) X[j] = (uint32_t)(int32_t)u2f(X[j]);
        break;
      case FX_I2F:
#pragma unroll
        for (int j = 0; j < N; ++j) X[j] = f2u((float)(int32_t)X[j]);
        break;
      case FX_FADD: FX_PB_F(a + b);
      case FX_FSUB: FX_PB_F(a - b);
      case FX_FRSUB: FX_PB_F(b - a);
      case FX_FMUL: FX_PB_F(a * b);
      case FX_FDIV: FX_PB_F(a / b);
      case FX_FMIN: FX_PB_F(fx_fmin(a, b));
      case FX_FMAX: FX_PB_F(fx_fmax(a, b));
      case FX_IADD:
#pragma unroll
        for (int j = 0; j < N; ++j) X[j] = (uint32_t)((int32_t)X[j] + (int32_t)imm);
        break;
      case FX_IMUL:
#pragma unroll
        for (int j = 0; j < N; ++j) X[j] = (uint32_t)((int32_t)X[j] * (int32_t)imm);
        break;
      case FX_FLT: FX_PC_F(a < b);
      case FX_FLE: FX_PC_F(a <= b);
      case FX_FGT: FX_PC_F(a > b);
      case FX_FGE: FX_PC_F(a >= b);
      case FX_FEQ: FX_PC_F(a == b);
      case FX_FNE: FX_PC_F(a != b);
      default: break;
    }
#undef FX_PU_F
#undef FX_PB_F
#undef FX_PC_F
}
template <int N>
__device__ __forceinline__ void fx_run_pure(const FxCtx& cx, int pc, const int pc_end, uint32_t (&X)[N]) {
  for (; pc < pc_end; ++pc) {
    const fx_u32x4 w = cx.insn[pc];
    fx_pure_step(uni(w.x) & 0xffffu, uni(w.w), X);
  }
}

// How the kernels below run a program: the interpreter, or (fx_spec.h) code generated by the
// compiler from the same fx_step / fx_pure_step with the program as a compile-time constant.
struct FxInterp {
  template <int R>
  static __device__ __forceinline__ void run(const FxCtx& cx, int pc, int pc_end, const FxCoord<R>& q, uint32_t M,
                                             uint32_t (&A)[FX_V]) {
    fx_run<R>(cx, pc, pc_end, q, M, A);
  }
  static __device__ __forceinline__ void run_mask(const FxCtx& cx, int pc, int pc_end, const FxCoord<1>& q, uint32_t M,
                                                  uint32_t (&A)[FX_V]) {
    fx_run<1>(cx, pc, pc_end, q, M, A);
  }
  // items of a pure program that the compaction kernel batches (the dense kernel: FX_K)
  static constexpr uint32_t kPure = FX_K;
  // ... and of the lean batches of whole-group outputs (fx_rows_batch)
  static constexpr uint32_t kRows = FX_K;
  // order in which a wave of the compaction kernel walks the outputs: 0 = alternate waves
  // backwards, 1 = all forwards (narrow outputs first), 2 = all backwards
  static constexpr int kWalk = 0;
  // waves per workgroup of the compaction kernel (its row tile stays FX_BLOCK rows) and the
  // waves per SIMD that its register budget is set for
  static constexpr uint32_t kWaves = FX_BLOCK / 64;
  static constexpr uint32_t kOcc = 4;
  template <int N>
  static __device__ __forceinline__ void run_pure(const FxCtx& cx, int pc, int pc_end, uint32_t (&X)[N]) {
    fx_run_pure(cx, pc, pc_end, X);
  }
};

// The leading load of a program, decoded once per output: everything about it is
// wave-uniform and the same for every item.
struct FxLead {
  int32_t cf[FX_MAXR];
  int32_t base;
  uint64_t p;
  uint64_t err;
  uint32_t dt;
  bool cvt;
  bool lds;              // the load reads a staged window (see FxCtx::all_win)
  const uint32_t* win;
  int32_t win_base;
};

template <int R>
__device__ __forceinline__ FxLead fx_lead_decode(const FxCtx& cx, int pc) {
  FxLead ld;
  const fx_u32x4 w = cx.insn[pc];
  const uint32_t w0 = uni(w.x);
  ld.cvt = (w0 & (FX_F_I2F << 16)) != 0;
  ld.dt = w0 >> 24;
  const fx_u32x4* ap = (const fx_u32x4*)(cx.aff + (int32_t)w.z * FX_AFF_WORDS);
  const fx_u32x4 a0 = ap[0], a1 = ap[1];
  ld.cf[0] = (int32_t)uni(a0.x); ld.cf[1] = (int32_t)uni(a0.y);
  ld.cf[2] = (int32_t)uni(a0.z); ld.cf[3] = (int32_t)uni(a0.w);
  if (R > 4) {
    const fx_u32x4 a2 = ap[2];
    ld.cf[4] = (int32_t)uni(a2.x); ld.cf[5] = (int32_t)uni(a2.y);
  } else {
    ld.cf[4] = 0; ld.cf[5] = 0;
  }
  ld.base = (int32_t)uni(a1.y) + (int32_t)uni(a1.x) * cx.task;
  ld.p = fx_ptr(cx, (int32_t)w.y);
  ld.err = cx.err;
  ld.lds = cx.all_win;
  ld.win = nullptr;
  ld.win_base = 0;
  if (cx.all_win) ld.win = fx_window_of(cx, uni(w.y), ld.win_base);
  return ld;
}

template <int R>
__device__ __forceinline__ void fx_lead_load(const FxLead& ld, const FxCoord<R>& q, uint32_t M, uint32_t (&P)[FX_V]) {
  int32_t off[FX_V];
  const bool consecutive = fx_offsets<R>(q, ld.cf, ld.base, off);
  if (ld.lds) {
#pragma unroll
    for (int j = 0; j < FX_V; ++j) P[j] = ld.win[((M >> j) & 1u) ? off[j] - ld.win_base : 0];
    if (ld.cvt) {
#pragma unroll
      for (int j = 0; j < FX_V; ++j) P[j] = f2u((float)(int32_t)P[j]);
    }
    return;
  }
  fx_load_vec(ld.p, off, M, ld.dt, ld.cvt, consecutive, P, ld.err);
}

// Leading loads of a batch of KP items, all in flight together.  When every item of the
// batch is a run of FX_V consecutive 32-bit elements in each of its live lanes (decided
// for the whole batch, wave-uniform), the loads are KP unconditional 128-bit loads with
// no branch between them; otherwise each item goes through fx_lead_load.
// make_item(k, e, M, q) sets up item k.
template <int R, int KP, class MI>
__device__ __forceinline__ void fx_lead_batch(const FxLead& ld, MI&& make_item, uint32_t (&X)[KP * FX_V],
                                              uint32_t (&e0)[KP], uint32_t (&Mk)[KP]) {
  const uint32_t VM = (1u << FX_V) - 1u;
  uint32_t o0[KP];
  bool fast = ld.dt == FX_F32 || ld.dt == FX_I32;
#pragma unroll
  for (int k = 0; k < KP; ++k) {
    uint32_t e[FX_V], M;
    FxCoord<R> q;
    make_item((uint32_t)k, e, M, q);
    int32_t off[FX_V];
    const bool consecutive = fx_offsets<R>(q, ld.cf, ld.base, off);
    e0[k] = e[0];
    Mk[k] = M;
    o0[k] = M ? (uint32_t)off[0] : 0u;
    fast = fast && consecutive && !wave_any(M != 0u && M != VM) && wave_any(M == VM);
  }
  if (fast && ld.lds) {
#pragma unroll
    for (int k = 0; k < KP; ++k) {
      const uint32_t* wp = ld.win + (Mk[k] ? (int32_t)o0[k] - ld.win_base : 0);
      X[k * FX_V + 0] = wp[0]; X[k * FX_V + 1] = wp[1]; X[k * FX_V + 2] = wp[2]; X[k * FX_V + 3] = wp[3];
    }
    if (ld.cvt) {
#pragma unroll
      for (int j = 0; j < KP * FX_V; ++j) X[j] = f2u((float)(int32_t)X[j]);
    }
  } else if (fast) {
    const FX_AS1 uint8_t* base = (const FX_AS1 uint8_t*)ld.p;
#pragma unroll
    for (int k = 0; k < KP; ++k) {
      const fx_u32x4_a4 v = *(const FX_AS1 fx_u32x4_a4*)(base + (o0[k] << 2));
      X[k * FX_V + 0] = v.x; X[k * FX_V + 1] = v.y; X[k * FX_V + 2] = v.z; X[k * FX_V + 3] = v.w;
    }
    if (ld.cvt) {
      asm volatile("" ::: "memory");
#pragma unroll
      for (int j = 0; j < KP * FX_V; ++j) X[j] = f2u((float)(int32_t)X[j]);
    }
  } else {
#pragma unroll
    for (int k = 0; k < KP; ++k) {
      uint32_t e[FX_V], M, Pk[FX_V];
      FxCoord<R> q;
      make_item((uint32_t)k, e, M, q);
      fx_lead_load<R>(ld, q, M, Pk);
#pragma unroll
      for (int j = 0; j < FX_V; ++j) X[k * FX_V + j] = Pk[j];
    }
  }
}

__device__ __forceinline__ uint32_t fx_fastdiv(uint32_t n, uint32_t magic, uint32_t shift) {
  return (__umulhi(n, magic) + n) >> shift;
}

// A batch of KP items of a pure output whose rows are whole lane groups: rank 2, FX_V
// consecutive 32-bit elements of one kept row per lane, no ragged group at the end of a
// row, a unit-stride leading load.  Group g is row g / gprow of the tile's kept rows and
// elements [FX_V * (g % gprow), +FX_V) of it, and it is element FX_V * g of the tile's
// rows of the output, so an item costs one division by a constant, one row-map lookup and
// one multiply instead of the general coordinate machinery.  Items past the end of the
// tile have no live lane; dead lanes load the first elements of the source and store nothing.
template <class S, uint32_t KP, uint32_t NW>
__device__ __forceinline__ void fx_rows_batch(const FxCtx& cx, const FxLead& ld, const uint32_t* rowmap, uint32_t it0,
                                              uint32_t lane, uint32_t n_groups, uint32_t gprow, uint32_t gr_magic,
                                              uint32_t gr_shift, uint64_t op, uint32_t obase, int pb, int pe) {
  uint32_t X[KP * FX_V], o0[KP], e0[KP];
  bool live[KP];
#pragma unroll
  for (uint32_t k = 0; k < KP; ++k) {
    const uint32_t g = (it0 + NW * k) * 64u + lane;
    live[k] = g < n_groups;
    const uint32_t gg = live[k] ? g : 0u;
    const uint32_t r = fx_fastdiv(gg, gr_magic, gr_shift);   // < FX_BLOCK
    const uint32_t c = gg - __umul24(r, gprow);                // gprow < 2^24 (checked by the caller)
    const uint32_t row = rowmap[r];
    const uint32_t off = (uint32_t)(ld.base + (int32_t)row * ld.cf[0]) + c * FX_V;
    o0[k] = live[k] ? off : 0u;
    e0[k] = gg * FX_V;
  }
  if (ld.lds) {
#pragma unroll
    for (uint32_t k = 0; k < KP; ++k) {
      const uint32_t* wp = ld.win + (live[k] ? (int32_t)o0[k] - ld.win_base : 0);
      X[k * FX_V + 0] = wp[0]; X[k * FX_V + 1] = wp[1]; X[k * FX_V + 2] = wp[2]; X[k * FX_V + 3] = wp[3];
    }
  } else {
    const FX_AS1 uint8_t* src = (const FX_AS1 uint8_t*)ld.p;
#pragma unroll
    for (uint32_t k = 0; k < KP; ++k) {
      const fx_u32x4_a4 v = *(const FX_AS1 fx_u32x4_a4*)(src + (o0[k] << 2));
      X[k * FX_V + 0] = v.x; X[k * FX_V + 1] = v.y; X[k * FX_V + 2] = v.z; X[k * FX_V + 3] = v.w;
    }
  }
  if (ld.cvt) {
    asm volatile("" ::: "memory");
#pragma unroll
    for (uint32_t j = 0; j < KP * FX_V; ++j) X[j] = f2u((float)(int32_t)X[j]);
  }
  S::run_pure(cx, pb + 1, pe, X);
  FX_AS1 uint8_t* dst = (FX_AS1 uint8_t*)op;
#pragma unroll
  for (uint32_t k = 0; k < KP; ++k) {
    if (live[k]) {
      fx_u32x4 v;
      v.x = X[k * FX_V + 0]; v.y = X[k * FX_V + 1]; v.z = X[k * FX_V + 2]; v.w = X[k * FX_V + 3];
      *(FX_AS1 fx_u32x4_a4*)(dst + ((obase + e0[k]) << 2)) = v;
    }
  }
}

// ---- workgroup prologue ----------------------------------------------------
// LDS layout (words): [blob][pointers: 2 words each][scalars][pad][temps]
struct FxLaunch {
  uint64_t wide;        // 0, or the device address of the call's tables (n_p pointers, then n_s scalars) where the argument block is too small for them
  uint32_t blob_words;  // multiple of 4
  uint32_t n_p;         // pointers in use in FxDyn::p
  uint32_t n_s;         // scalars in use in FxDyn::s
  uint32_t temps_off;   // word offset of the temp area in LDS (multiple of 4)
  uint32_t epoch;       // streaming compaction: tag of this call's tile counts (1 .. 2^23 - 1)
  uint32_t total_units; // dense: work units of FX_UNIT elements; the grid strides over them
  // streaming compaction (fx_compact_stream; one task class): everything a workgroup needs to
  // find its rows of the window input comes from the argument segment, so that the loads of the
  // tile are issued before anything else is read
  uint32_t win_off;      // word offset of the window in LDS (multiple of 4)
  uint32_t spin_limit;   // polls of a look-back wait before the workgroup counts the rows itself
  uint32_t s_tiles;      // row tiles per task
  uint32_t s_rows;       // rows per task
  uint32_t s_tile_rows;  // rows per tile (<= FX_BLOCK)
  uint32_t s_win_slot;   // pointer slot of the window input (FX_SLOT_TASK: per-task table)
  uint32_t s_win_stride; // elements per row of the window input
  int32_t s_win_tcoef;   // element offset per task
  int32_t s_win_lo;      // smallest element offset a program reads inside a row
  uint32_t s_win_span;   // elements from there to the largest one, inclusive
  uint32_t n_sptr;       // layout of the pointer table: shared pointers, then n_tptr per task
  uint32_t n_tptr;
  uint32_t win_buf;      // words of the window (multiple of 4)
  uint32_t n_side;       // side windows in use (at most 64 16-byte lines per lane group: 256 lines each)
  uint32_t side_slot[FX_SIDE_WIN];
  uint32_t side_stride[FX_SIDE_WIN];
  int32_t side_tcoef[FX_SIDE_WIN];
  int32_t side_lo[FX_SIDE_WIN];
  uint32_t side_span[FX_SIDE_WIN];
  uint32_t side_off[FX_SIDE_WIN];   // word offsets in LDS (multiples of 4)
};
static_assert(sizeof(FxLaunch) % 8 == 0, "the tables that follow FxLaunch in the argument segment are 8-byte aligned");
#define FX_KERNARG_DYN_OFF (8 + sizeof(FxLaunch))

template <uint32_t NT = FX_BLOCK>
__device__ __forceinline__ void fx_stage(uint32_t* L, const uint32_t* __restrict__ sb, const FxLaunch& la) {
  const FX_AS1 fx_u32x4* g4 = (const FX_AS1 fx_u32x4*)sb;
  fx_u32x4* l4 = (fx_u32x4*)L;
  for (uint32_t i = threadIdx.x; i < la.blob_words / 4; i += NT) l4[i] = g4[i];
  // The by-value FxDyn block is read through the kernarg segment pointer (never
  // by naming the parameter: indexing a by-value aggregate dynamically would
  // make the compiler copy it to per-lane scratch).
  const uint8_t* ka = (const uint8_t*)__builtin_amdgcn_kernarg_segment_ptr();
  const uint64_t* gp = (const uint64_t*)(ka + FX_KERNARG_DYN_OFF);
  const uint32_t* gs = (const uint32_t*)(ka + FX_KERNARG_DYN_OFF + 8 * FX_DYN_P);
  if (la.wide != 0) {   // a map of many tasks: the tables were uploaded ahead of this launch
    gp = (const uint64_t*)la.wide;
    gs = (const uint32_t*)(gp + la.n_p);
  }
  uint64_t* lp = (uint64_t*)(L + la.blob_words);
  uint32_t* ls = L + la.blob_words + 2 * la.n_p;
  for (uint32_t i = threadIdx.x; i < la.n_p; i += NT) lp[i] = gp[i];
  for (uint32_t i = threadIdx.x; i < la.n_s; i += NT) ls[i] = gs[i];
  __syncthreads();
}

struct FxWork {
  const uint32_t* cls;   // LDS: FxClass words
  int task;
  uint32_t local_block;  // block index inside the task
};

template <bool COUNT_PASS>
__device__ __forceinline__ FxWork fx_locate(const uint32_t* L, uint32_t block) {
  const uint32_t n_classes = uni(L[FX_W(FxHeader, n_classes)]);
  const uint32_t* cls = L + uni(L[FX_W(FxHeader, off_class)]);
  const uint32_t cw = sizeof(FxClass) / 4;
  const uint32_t end_w = COUNT_PASS ? FX_W(FxClass, cnt_block_end) : FX_W(FxClass, block_end);
  uint32_t ci = 0;
  while (ci + 1 < n_classes && block >= uni(cls[ci * cw + end_w])) ++ci;
  const uint32_t* cl = cls + ci * cw;
  const uint32_t rel = block - uni(cl[COUNT_PASS ? FX_W(FxClass, cnt_block_begin) : FX_W(FxClass, block_begin)]);
  const uint32_t bpt = uni(cl[COUNT_PASS ? FX_W(FxClass, cnt_blocks_per_task) : FX_W(FxClass, blocks_per_task)]);
  const uint32_t ti = rel / bpt;
  FxWork w;
  w.cls = cl;
  w.local_block = rel - ti * bpt;
  w.task = (int)uni(L[uni(L[FX_W(FxHeader, off_taskmap)]) + uni(cl[FX_W(FxClass, first_task)]) + ti]);
  return w;
}

__device__ __forceinline__ FxCtx fx_make_ctx(uint32_t* L, const FxLaunch& la, const FxWork& w) {
  FxCtx cx;
  cx.insn = (const fx_u32x4*)(L + uni(w.cls[FX_W(FxClass, off_insn)]));
  cx.aff = L + uni(w.cls[FX_W(FxClass, off_aff)]);
  cx.ptrs = (const uint64_t*)(L + la.blob_words);
  cx.scal = L + la.blob_words + 2 * la.n_p;
  const uint32_t n_sptr = uni(L[FX_W(FxHeader, n_sptr)]), n_tptr = uni(L[FX_W(FxHeader, n_tptr)]);
  const uint32_t n_sscal = uni(L[FX_W(FxHeader, n_sscal)]), n_tscal = uni(L[FX_W(FxHeader, n_tscal)]);
  cx.tp_off = n_sptr + (uint32_t)w.task * n_tptr;
  cx.ts_off = n_sscal + (uint32_t)w.task * n_tscal;
  cx.temps = L + la.temps_off + threadIdx.x;
  cx.wseg = 64;
  cx.task = w.task;
  cx.all_win = false;
  cx.win = nullptr;
  cx.win_slot = -1;
  cx.win_base = 0;
#pragma unroll
  for (int i = 0; i < FX_SIDE_WIN; ++i) { cx.side[i] = nullptr; cx.side_slot[i] = -1; cx.side_base[i] = 0; }
  const uint32_t se = uni(L[FX_W(FxHeader, slot_err)]);
  cx.err = 0;
  if (se) {
    const uint64_t p = cx.ptrs[se - 1u];
    cx.err = ((uint64_t)uni((uint32_t)(p >> 32)) << 32) | (uint64_t)uni((uint32_t)p);
  }
  return cx;
}

}  // namespace

// --------------------------------------------------------------------------
// dense region kernel
// --------------------------------------------------------------------------
template <int R, class S = FxInterp>
__global__ __launch_bounds__(FX_BLOCK, 4) void fx_region_dense(const uint32_t* __restrict__ sb, const FxLaunch la,
                                                            const FxDyn) {
  extern __shared__ __attribute__((aligned(16))) uint32_t L[];
  fx_stage(L, sb, la);   // once per workgroup; the loop below has no barrier
  const uint32_t lane = threadIdx.x & 63u, wave = uni(threadIdx.x >> 6);
  const uint32_t ow = sizeof(FxOut) / 4;

  // Persistent workgroups: work units of FX_UNIT elements (one output of one
  // task each) are strided over the grid; inside a unit every wave owns FX_K
  // consecutive items of FX_ITEM elements.
  for (uint32_t unit = blockIdx.x; unit < la.total_units; unit += gridDim.x) {
    const FxWork w = fx_locate<false>(L, unit);
    FxCtx cx = fx_make_ctx(L, la, w);
    const uint32_t n_outs = uni(w.cls[FX_W(FxClass, n_outs)]);
    const uint32_t* outs = L + uni(w.cls[FX_W(FxClass, off_outs)]);
    uint32_t oi = 0;
    while (oi + 1 < n_outs && w.local_block >= uni(outs[oi * ow + FX_W(FxOut, block_begin)]) +
                                                   uni(outs[oi * ow + FX_W(FxOut, n_blocks)]))
      ++oi;
    const uint32_t* od = outs + oi * ow;
    const uint32_t ublock = w.local_block - uni(od[FX_W(FxOut, block_begin)]);
    const uint32_t numel = uni(od[FX_W(FxOut, numel)]);
    const int pb = (int)uni(od[FX_W(FxOut, prog_begin)]), pe = (int)uni(od[FX_W(FxOut, prog_end)]);
    const uint32_t lead = uni(od[FX_W(FxOut, lead)]);
    const uint64_t op = fx_ptr(cx, (int32_t)od[FX_W(FxOut, ptr_slot)]);
    const uint32_t obase = uni(od[FX_W(FxOut, task_stride)]) * (uint32_t)w.task;
    const uint32_t odt = uni(od[FX_W(FxOut, dtype)]), ovt = uni(od[FX_W(FxOut, vt)]);
    uint32_t dk[R], mk[R], sk[R];
    dk[0] = mk[0] = sk[0] = 0;
#pragma unroll
    for (int k = 1; k < R; ++k) {
      dk[k] = od[FX_W(FxOut, dim) + k];
      mk[k] = od[FX_W(FxOut, magic) + k];
      sk[k] = od[FX_W(FxOut, shift) + k];
    }
    // unit = 4 waves x kmax items; kmax is 1 for heavy or small outputs (more, smaller units).
    // An item is 64 lane groups of FX_V consecutive elements along the last dimension,
    // or one whole row (rowwave) so that the wave-wide reductions see exactly the
    // elements of that row.
    const uint32_t kmax = uni(od[FX_W(FxOut, unit_items)]);
    const uint32_t rowwave = uni(od[FX_W(FxOut, rowwave)]);
    const uint32_t inner = uni(od[FX_W(FxOut, inner)]);
    const uint32_t vd = uni(od[FX_W(FxOut, vd)]);
    const uint32_t gpr = uni(od[FX_W(FxOut, gpr)]);
    const uint32_t gp_magic = od[FX_W(FxOut, gp_magic)], gp_shift = od[FX_W(FxOut, gp_shift)];
    const uint32_t n_groups = uni(od[FX_W(FxOut, n_groups)]);
    const uint32_t item0 = ublock * (4u * kmax) + wave * kmax;
    const uint32_t rowseg = rowwave ? uni(od[FX_W(FxOut, rowseg)]) : 64u;
    const uint32_t segsh = 31u - (uint32_t)__builtin_clz(rowseg);
    const uint32_t rows_per_item = 64u >> segsh;
    cx.wseg = rowseg;
    const uint32_t n_rows_w = numel / inner;
    const uint32_t n_items = rowwave ? (n_rows_w + rows_per_item - 1) / rows_per_item : (n_groups + 63u) / 64u;
    if (item0 >= n_items) continue;

    auto make_item = [&](uint32_t k, uint32_t (&e)[FX_V], uint32_t& M, FxCoord<R>& q) {
      uint32_t row, col0;
      bool live;
      if (rowwave) {
        // 64 / rowseg rows per wave, one per segment of rowseg lanes
        const uint32_t seg = lane >> segsh;
        row = (item0 + k) * rows_per_item + seg;
        col0 = (lane - seg * rowseg) * FX_V;
        live = row < n_rows_w;
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

    if (uni(od[FX_W(FxOut, pure)]) && kmax == FX_K && item0 + FX_K <= n_items) {
      // the FX_K items of this wave as one batch; an incomplete batch takes the generic path
      const FxLead ld = fx_lead_decode<R>(cx, pb);
      uint32_t X[FX_NB], e0[FX_K], Mk[FX_K];
      fx_lead_batch<R, FX_K>(ld, make_item, X, e0, Mk);
      S::run_pure(cx, pb + 1, pe, X);
#pragma unroll
      for (uint32_t k = 0; k < FX_K; ++k) {
        uint32_t e[FX_V], Ak[FX_V];
#pragma unroll
        for (int j = 0; j < FX_V; ++j) { e[j] = e0[k] + j; Ak[j] = X[k * FX_V + j]; }
        fx_store_vec(op, obase, e, Mk[k], true, odt, ovt, Ak);
      }
      continue;
    }
    uint32_t P[FX_K][FX_V];
    if (lead) {
      const FxLead ld = fx_lead_decode<R>(cx, pb);
#pragma unroll
      for (uint32_t k = 0; k < FX_K; ++k) {
        if (k < kmax && item0 + k < n_items) {
          uint32_t e[FX_V], M;
          FxCoord<R> q;
          make_item(k, e, M, q);
          fx_lead_load<R>(ld, q, M, P[k]);
        }
      }
    }
    // one copy of the interpreter: the loop stays rolled, the preloaded values are picked by selects
#pragma unroll 1
    for (uint32_t k = 0; k < FX_K; ++k) {
      if (k < kmax && item0 + k < n_items) {
        uint32_t e[FX_V], M;
        FxCoord<R> q;
        make_item(k, e, M, q);
        uint32_t A[FX_V];
#pragma unroll
        for (int j = 0; j < FX_V; ++j) {
          uint32_t v = P[0][j];
#pragma unroll
          for (uint32_t kk = 1; kk < FX_K; ++kk) v = (k == kk) ? P[kk][j] : v;
          A[j] = lead ? v : 0u;
        }
        S::template run<R>(cx, lead ? pb + 1 : pb, pe, q, M, A);
        fx_store_vec(op, obase, e, M, true, odt, ovt, A);
      }
    }
  }
}

// --------------------------------------------------------------------------
// row compaction, pass 1: evaluate the mask program per row, write one flag
// byte per row and one keep count per row tile.
// grid = per task ceil(n_rows / FX_TILE) blocks; tile counts are per
// row_tile rows (row_tile is 64, 128 or 256).
// --------------------------------------------------------------------------
template <class S = FxInterp>
__global__ __launch_bounds__(FX_BLOCK) void fx_compact_count(const uint32_t* __restrict__ sb, const FxLaunch la,
                                                             const FxDyn) {
  extern __shared__ __attribute__((aligned(16))) uint32_t L[];
  __shared__ uint32_t s_wcnt[FX_V][FX_BLOCK / 64];
  fx_stage(L, sb, la);
  const FxWork w = fx_locate<true>(L, blockIdx.x);
  const FxCtx cx = fx_make_ctx(L, la, w);

  const uint32_t n_rows = uni(w.cls[FX_W(FxClass, n_rows)]);
  FxCoord<1> q;
  q.c0[0] = 0;
  q.vd = 0;
  q.step = 0;
  uint32_t M = 0;
  uint32_t row[FX_V];
#pragma unroll
  for (int j = 0; j < FX_V; ++j) {
    row[j] = w.local_block * FX_TILE + j * FX_BLOCK + threadIdx.x;
    q.cv[j] = (int32_t)row[j];
    if (row[j] < n_rows) M |= 1u << j;
  }
  uint32_t A[FX_V];
#pragma unroll
  for (int j = 0; j < FX_V; ++j) A[j] = 0;
  S::run_mask(cx, (int)uni(w.cls[FX_W(FxClass, mask_begin)]), (int)uni(w.cls[FX_W(FxClass, mask_end)]), q, M, A);

  const uint32_t max_rowtiles = uni(L[FX_W(FxHeader, max_rowtiles)]);
  FX_AS1 uint8_t* flags = (FX_AS1 uint8_t*)cx.ptrs[uni(L[FX_W(FxHeader, slot_flags)])] + (size_t)w.task * uni(L[FX_W(FxHeader, max_rows)]);
  FX_AS1 uint32_t* counts =
      (FX_AS1 uint32_t*)cx.ptrs[uni(L[FX_W(FxHeader, slot_counts)])] + (size_t)w.task * max_rowtiles;
  const uint32_t rt = uni(L[FX_W(FxHeader, row_tile)]);
  const uint32_t mask_vt = uni(w.cls[FX_W(FxClass, mask_vt)]);
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
#pragma unroll
  for (int j = 0; j < FX_V; ++j) {
    const bool live = (M >> j) & 1u;
    const bool keep = live && (mask_vt == FX_VT_F ? (u2f(A[j]) != 0.0f) : (A[j] != 0u));
    if (live) flags[row[j]] = keep ? 1 : 0;
    const uint64_t bal = __builtin_amdgcn_ballot_w64(keep);
    if (lane == 0) s_wcnt[j][wave] = (uint32_t)__popcll(bal);
  }
  __syncthreads();
  const uint32_t waves_per_tile = rt / 64u;
  const uint32_t tiles_per_slab = FX_BLOCK / rt;
  if (threadIdx.x < FX_V * tiles_per_slab) {
    const uint32_t j = threadIdx.x / tiles_per_slab, t = threadIdx.x % tiles_per_slab;
    const uint32_t first_row = w.local_block * FX_TILE + j * FX_BLOCK + t * rt;
    if (first_row < n_rows) {
      uint32_t s = 0;
      for (uint32_t k = 0; k < waves_per_tile; ++k) s += s_wcnt[j][t * waves_per_tile + k];
      counts[first_row / rt] = s;
    }
  }
}

// --------------------------------------------------------------------------
// Outputs of one row tile of a compaction: every output's program evaluated on the kept rows
// (rowmap: their row numbers in source order), written to rows [prefix, prefix + n_kept) of the
// compacted output.  Shared by the second pass of the two-pass form and the streaming kernel.
// --------------------------------------------------------------------------
struct FxNoHook {
  __device__ __forceinline__ void operator()() const {}
};
// before_last(): called by every wave in front of the last output of its walk
template <int R, class S, uint32_t NW, class HK = FxNoHook>
__device__ __forceinline__ void fx_scatter_outputs(const FxCtx& cx, const FxWork& w, const uint32_t* L,
                                                   const uint32_t* s_rowmap, const uint32_t n_kept,
                                                   const uint32_t prefix, const uint32_t lane, const uint32_t wave,
                                                   HK&& before_last = FxNoHook()) {
  const uint32_t n_outs = uni(w.cls[FX_W(FxClass, n_outs)]);
  const uint32_t* outs = L + uni(w.cls[FX_W(FxClass, off_outs)]);
  const uint32_t ow = sizeof(FxOut) / 4;
  // Work items of FX_ITEM elements are dealt to the four waves round-robin over
  // ALL outputs of the tile, so that a long program of a narrow output (a few
  // items) overlaps with the short programs of the wide ones instead of
  // serialising the whole workgroup behind it.  No barrier from here on.
  const uint32_t wave_u = uni(wave);
  // Half of the waves walk the outputs backwards: a latency-bound output (a long
  // predicated program on a few items) then overlaps, on the same SIMD, with the
  // arithmetic-bound wide outputs of the other waves.
  const bool backwards = S::kWalk == 0 ? ((blockIdx.x + wave_u) & 1u) != 0 : S::kWalk == 2;
  for (uint32_t oo = 0; oo < n_outs; ++oo) {
    if (oo + 1u == n_outs) before_last();
    const uint32_t oi = backwards ? n_outs - 1u - oo : oo;
    const uint32_t* od = outs + oi * ow;
    const uint32_t rowlen = uni(od[FX_W(FxOut, rowlen)]);
    const uint32_t colmajor = uni(od[FX_W(FxOut, colmajor)]);
    const uint32_t inner = uni(od[FX_W(FxOut, inner)]);
    const uint32_t vd = uni(od[FX_W(FxOut, vd)]);
    const uint32_t gpr = uni(od[FX_W(FxOut, gpr)]);
    const uint32_t gp_magic = od[FX_W(FxOut, gp_magic)], gp_shift = od[FX_W(FxOut, gp_shift)];
    const uint32_t gprow = uni(od[FX_W(FxOut, gprow)]);
    const uint32_t gr_magic = od[FX_W(FxOut, gr_magic)], gr_shift = od[FX_W(FxOut, gr_shift)];
    const uint32_t chunks = (n_kept + FX_ITEM - 1) / FX_ITEM;   // row chunks per column (column-major)
    // lane groups: FX_V consecutive elements of a kept row along the last dimension, or
    // (rank 1) FX_V consecutive kept rows
    const uint32_t n_groups = vd == 0 ? (n_kept + FX_V - 1) / FX_V : n_kept * gprow;
    const uint32_t n_items = colmajor ? rowlen * chunks : (n_groups + 63u) / 64u;
    const uint64_t op = fx_ptr(cx, (int32_t)od[FX_W(FxOut, ptr_slot)]);
    const uint32_t obase = uni(od[FX_W(FxOut, task_stride)]) * (uint32_t)w.task + prefix * rowlen;
    const int pb = (int)uni(od[FX_W(FxOut, prog_begin)]), pe = (int)uni(od[FX_W(FxOut, prog_end)]);
    const uint32_t odt = uni(od[FX_W(FxOut, dtype)]), ovt = uni(od[FX_W(FxOut, vt)]);
    uint32_t dk[R], mk[R], sk[R];
    dk[0] = mk[0] = sk[0] = 0;
#pragma unroll
    for (int k = 1; k < R; ++k) {
      dk[k] = od[FX_W(FxOut, dim) + k];
      mk[k] = od[FX_W(FxOut, magic) + k];
      sk[k] = od[FX_W(FxOut, shift) + k];
    }
    const uint32_t lead = uni(od[FX_W(FxOut, lead)]);
    auto make_item = [&](uint32_t it, uint32_t (&e)[FX_V], uint32_t& M, FxCoord<R>& q) {
      M = 0;
      if (colmajor) {
        // all lanes of the item share one column: predicates on the inner
        // coordinates are wave-uniform and whole branches get skipped
        const uint32_t cc = it / chunks, ch = it - cc * chunks;
#pragma unroll
        for (int j = 0; j < FX_V; ++j) {
          const uint32_t r = ch * FX_ITEM + j * 64u + lane;
          const bool live = r < n_kept;
          if (live) M |= 1u << j;
          e[j] = r * rowlen + cc;
          q.cv[j] = live ? (int32_t)s_rowmap[r] : 0;
        }
        q.vd = 0;
        q.step = 0;
        fx_unflatten<R>(cc, 0u, dk, mk, sk, q.c0);
        q.c0[0] = 0;
      } else if (vd == 0) {
        const uint32_t r0 = (it * 64u + lane) * FX_V;
#pragma unroll
        for (int j = 0; j < FX_V; ++j) {
          const bool live = r0 + j < n_kept;
          if (live) M |= 1u << j;
          e[j] = r0 + j;
          q.cv[j] = live ? (int32_t)s_rowmap[r0 + j] : 0;
        }
        q.vd = 0;
        q.step = 0;
#pragma unroll
        for (int k = 0; k < R; ++k) q.c0[k] = 0;
      } else {
        const uint32_t g = it * 64u + lane;
        const bool live = g < n_groups;
        const uint32_t gg = live ? g : 0u;
        const uint32_t r = fx_fastdiv(gg, gr_magic, gr_shift);
        const uint32_t t = gg - r * gprow;
        const uint32_t mid = fx_fastdiv(t, gp_magic, gp_shift);
        const uint32_t col0 = (t - mid * gpr) * FX_V;
#pragma unroll
        for (int j = 0; j < FX_V; ++j) {
          if (live && col0 + j < inner) M |= 1u << j;
          e[j] = r * rowlen + mid * inner + col0 + j;
          q.cv[j] = (int32_t)(col0 + j);
        }
        q.vd = vd;
        q.step = 1;
        fx_unflatten<R>(mid, vd, dk, mk, sk, q.c0);
        q.c0[0] = (int32_t)s_rowmap[r];
      }
    };
    const bool contig = !colmajor;
    // items of this output that belong to this wave: first, first + NW, ...
    // taken FX_K at a time so that their leading loads overlap
    // (the rotation by the output index spreads single-item outputs over the waves; it
    // must not depend on the order in which a wave walks the outputs)
    uint32_t it0 = (wave_u + NW - (oi & (NW - 1u))) & (NW - 1u);
    FxLead ld;
    if (lead) ld = fx_lead_decode<R>(cx, pb);
    bool rows_fast = false;
    if constexpr (R == 2) {
      rows_fast = uni(od[FX_W(FxOut, pure)]) && lead && !colmajor && vd == 1u && gprow == gpr && gpr * FX_V == inner &&
                  inner == rowlen && gprow < (1u << 24) && (ld.dt == FX_F32 || ld.dt == FX_I32) && ld.cf[1] == 1 &&
                  ((odt == FX_F32 && ovt == FX_VT_F) || (odt == FX_I32 && ovt == FX_VT_I));
    }
    if (rows_fast) {
      constexpr uint32_t KP = S::kRows;
      const uint32_t grm = uni(gr_magic), grs = uni(gr_shift);
      for (; it0 + NW * (KP - 1u) < n_items; it0 += NW * KP)
        fx_rows_batch<S, KP, NW>(cx, ld, s_rowmap, it0, lane, n_groups, gprow, grm, grs, op, obase, pb, pe);
      for (; it0 < n_items; it0 += NW * 2u)
        fx_rows_batch<S, 2, NW>(cx, ld, s_rowmap, it0, lane, n_groups, gprow, grm, grs, op, obase, pb, pe);
    } else if (uni(od[FX_W(FxOut, pure)])) {
      // S::kPure items as one batch; an incomplete batch at the end takes the generic path
      constexpr uint32_t KP = S::kPure;
      for (; it0 + NW * (KP - 1u) < n_items; it0 += NW * KP) {
        uint32_t X[KP * FX_V], e0[KP], Mk[KP];
        fx_lead_batch<R, (int)KP>(
            ld, [&](uint32_t k, uint32_t (&e)[FX_V], uint32_t& M, FxCoord<R>& q) { make_item(it0 + NW * k, e, M, q); }, X,
            e0, Mk);
        S::run_pure(cx, pb + 1, pe, X);
#pragma unroll
        for (uint32_t k = 0; k < KP; ++k) {
          uint32_t e[FX_V], Ak[FX_V];
#pragma unroll
          for (int j = 0; j < FX_V; ++j) { e[j] = e0[k] + j; Ak[j] = X[k * FX_V + j]; }
          fx_store_vec(op, obase, e, Mk[k], true, odt, ovt, Ak);
        }
      }
    }
    for (; it0 < n_items; it0 += NW * FX_K) {
      uint32_t P[FX_K][FX_V];
      if (lead) {
#pragma unroll
        for (uint32_t k = 0; k < FX_K; ++k) {
          const uint32_t it = it0 + NW * k;
          if (it < n_items) {
            uint32_t e[FX_V], M;
            FxCoord<R> q;
            make_item(it, e, M, q);
            fx_lead_load<R>(ld, q, M, P[k]);
          }
        }
      }
#pragma unroll 1
      for (uint32_t k = 0; k < FX_K; ++k) {
        const uint32_t it = it0 + NW * k;
        if (it < n_items) {
          uint32_t e[FX_V], M;
          FxCoord<R> q;
          make_item(it, e, M, q);
          uint32_t A[FX_V];
#pragma unroll
          for (int j = 0; j < FX_V; ++j) {
            uint32_t v = P[0][j];
#pragma unroll
            for (uint32_t kk = 1; kk < FX_K; ++kk) v = (k == kk) ? P[kk][j] : v;
            A[j] = lead ? v : 0u;
          }
          S::template run<R>(cx, lead ? pb + 1 : pb, pe, q, M, A);
          fx_store_vec(op, obase, e, M, contig, odt, ovt, A);
        }
      }
    }
  }
}

// --------------------------------------------------------------------------
// row compaction, pass 2.  One workgroup per (task, row tile):
//   offset  = sum of the keep counts of the earlier tiles of this task
//   row map = kept rows of this tile in source order (ballot + popcount prefix)
//   for every output: evaluate its program on the kept rows only and write
//   rows [offset, offset + kept) of the compacted output.
// The last tile of a task also publishes the task's total.
// --------------------------------------------------------------------------
template <int R, class S = FxInterp>
__global__ __launch_bounds__(64 * S::kWaves, S::kOcc) void fx_compact_scatter(const uint32_t* __restrict__ sb,
                                                                              const FxLaunch la, const FxDyn) {
  constexpr uint32_t NW = S::kWaves, NT = 64u * NW;   // the row tile is at most FX_BLOCK rows, NT >= FX_BLOCK
  extern __shared__ __attribute__((aligned(16))) uint32_t L[];
  __shared__ uint32_t s_rowmap[FX_BLOCK];
  __shared__ uint32_t s_wsum[NW];
  __shared__ uint32_t s_woff[NW + 1];
  __shared__ uint32_t s_prefix;
  fx_stage<NT>(L, sb, la);
  const FxWork w = fx_locate<false>(L, blockIdx.x);
  FxCtx cx = fx_make_ctx(L, la, w);

  const uint32_t n_rows = uni(w.cls[FX_W(FxClass, n_rows)]);
  const uint32_t rt = uni(L[FX_W(FxHeader, row_tile)]);
  const uint32_t max_rowtiles = uni(L[FX_W(FxHeader, max_rowtiles)]);
  const uint32_t tile = w.local_block;
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const FX_AS1 uint8_t* flags =
      (const FX_AS1 uint8_t*)cx.ptrs[uni(L[FX_W(FxHeader, slot_flags)])] + (size_t)w.task * uni(L[FX_W(FxHeader, max_rows)]);
  const FX_AS1 uint32_t* counts =
      (const FX_AS1 uint32_t*)cx.ptrs[uni(L[FX_W(FxHeader, slot_counts)])] + (size_t)w.task * max_rowtiles;

  // this thread's row flag and its share of the counts of the earlier tiles: both loads are
  // issued before either value is used
  const uint32_t row = tile * rt + threadIdx.x;
  const bool in_tile = (threadIdx.x < rt) && (row < n_rows);
  const uint32_t flag = in_tile ? (uint32_t)flags[row] : 0u;
  // exclusive offset of this tile
  uint32_t part = 0;
  for (uint32_t t = threadIdx.x; t < tile; t += NT) part += counts[t];
  part = fx_wave_sum(part, threadIdx.x & 63u);
  if (lane == 0) s_wsum[wave] = part;

  // row map of this tile
  const bool keep = flag != 0u;
  const uint64_t bal = __builtin_amdgcn_ballot_w64(keep);
  const uint32_t before = (uint32_t)__popcll(bal & ((1ull << lane) - 1ull));
  if (lane == 0) s_woff[wave + 1] = (uint32_t)__popcll(bal);
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t p = 0;
    for (uint32_t k = 0; k < NW; ++k) p += s_wsum[k];
    s_prefix = p;
    uint32_t acc = 0;
    s_woff[0] = 0;
    for (uint32_t k = 1; k <= NW; ++k) { acc += s_woff[k]; s_woff[k] = acc; }
  }
  __syncthreads();
  if (keep) s_rowmap[s_woff[wave] + before] = row;
  __syncthreads();
  const uint32_t n_kept = uni(s_woff[NW]);
  const uint32_t prefix = uni(s_prefix);
  if (tile + 1 == uni(w.cls[FX_W(FxClass, n_rowtiles)]) && threadIdx.x == 0) {
    // The host polls this word while the kernel still runs: a system-scope store goes through
    // to host memory instead of waiting in L2 for the end of the kernel.  (Relaxed: the host
    // reads the count only; everything else of the call is consumed in stream order.)
    __hip_atomic_store((uint32_t*)cx.ptrs[uni(L[FX_W(FxHeader, slot_total)])] + w.task, prefix + n_kept, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_SYSTEM);
  }
  if (n_kept == 0) return;

  fx_scatter_outputs<R, S, NW>(cx, w, L, s_rowmap, n_kept, prefix, lane, wave);
}

// --------------------------------------------------------------------------
// Row compaction in ONE pass (opt-in, fx_set_streaming) for regions with one task class whose
// inputs are all row-major matrices that the programs read row by row (the prediction tensor
// of a detection head and its anchor tables).  Persistent workgroups stride over (task, row
// tile) pairs:
//   1. The tile's rows of every input are contiguous runs of memory.  They are fetched with
//      coalesced 128-bit loads whose addresses come from the argument segment alone (issued
//      before anything else for the first tile, and for the next tile while the current one is
//      worked on: the lines travel in registers) and parked in LDS ("windows").  The programs
//      then read nothing but LDS: the code holds no load from memory, so a wave never waits for
//      the memory pipeline, where it would also wait for every store it has issued.
//   2. mask program per row (from the window), ballot + popcount row map, tile count.
//   3. The count is published in a status word tagged with the call's epoch; the tile's write
//      offset is the sum of the counts of the earlier tiles of its task, read from their status
//      words as they appear (earlier tiles never wait for later ones).  Every poll loop is
//      bounded: when a word does not show up within spin_limit polls the workgroup counts the
//      kept rows of the earlier tiles itself, from memory, so the kernel ends whatever the order
//      in which workgroups are started.
//   4. outputs as in the two-pass form (fx_scatter_outputs).
// Status words belong to the library (one per tile, zero when allocated, never reset: a word
// of an earlier call carries an older epoch).
// --------------------------------------------------------------------------
#ifndef FX_STREAM_OCC
#define FX_STREAM_OCC 2   // waves per SIMD the register budget is set for: two workgroups per CU
#endif
#define FX_STATUS_BITS 9u   // a tile holds at most FX_BLOCK = 256 rows

// Where the rows of tile `b` of the window input start, in 16-byte lines, and how many lines
// they span.
struct FxWinAddr {
  const FX_AS1 fx_u32x4* g4;
  uint32_t n_vec, shift, r0, rows, task_i, tile;
  int32_t e0;
};
__device__ __forceinline__ FxWinAddr fx_win_addr_of(const FxLaunch& la, uint32_t b, uint32_t sl, uint32_t stride,
                                                    int32_t tcoef, int32_t lo, uint32_t span) {
  FxWinAddr a;
  a.task_i = b / la.s_tiles;
  a.tile = b - a.task_i * la.s_tiles;
  a.r0 = a.tile * la.s_tile_rows;
  a.rows = min(la.s_tile_rows, la.s_rows - a.r0);
  const uint8_t* ka = (const uint8_t*)__builtin_amdgcn_kernarg_segment_ptr();
  const uint64_t* gp = (const uint64_t*)(ka + FX_KERNARG_DYN_OFF);
  const uint32_t pi = (sl & FX_SLOT_TASK) ? la.n_sptr + a.task_i * la.n_tptr + (sl & 0xffffu) : (sl & 0xffffu);
  const uint64_t wp = gp[pi];
  a.e0 = tcoef * (int32_t)a.task_i + (int32_t)(a.r0 * stride) + lo;   // >= 0 (host)
  const uint32_t n_el = (a.rows - 1u) * stride + span;
  const uint64_t a0 = wp + ((uint64_t)(uint32_t)a.e0 << 2);
  a.shift = ((uint32_t)a0 & 15u) >> 2;            // elements between the 16-byte line and e0
  a.g4 = (const FX_AS1 fx_u32x4*)(a0 & ~(uint64_t)15);
  a.n_vec = (a.shift + n_el + 3u) >> 2;           // <= window words / 4 (host)
  return a;
}
__device__ __forceinline__ FxWinAddr fx_win_addr(const FxLaunch& la, uint32_t b) {
  return fx_win_addr_of(la, b, la.s_win_slot, la.s_win_stride, la.s_win_tcoef, la.s_win_lo, la.s_win_span);
}
__device__ __forceinline__ FxWinAddr fx_side_addr(const FxLaunch& la, uint32_t b, int i) {
  return fx_win_addr_of(la, b, la.side_slot[i], la.side_stride[i], la.side_tcoef[i], la.side_lo[i], la.side_span[i]);
}

#define FX_WK 12   // 128-bit loads per lane that carry the next tile's rows while this tile is worked on
template <int R, class S = FxInterp>
__global__ __launch_bounds__(FX_BLOCK, FX_STREAM_OCC) void fx_compact_stream(const uint32_t* __restrict__ sb,
                                                                            const FxLaunch la, const FxDyn) {
  constexpr uint32_t NT = FX_BLOCK, NW = NT / 64u;
  extern __shared__ __attribute__((aligned(16))) uint32_t L[];
  __shared__ uint32_t s_rowmap[FX_BLOCK];
  __shared__ uint32_t s_wsum[NW];
  __shared__ uint32_t s_woff[NW + 1];
  __shared__ uint32_t s_prefix, s_ok;
  const uint32_t n_tiles = la.total_units;   // tiles of the whole call; the workgroups stride over them
  const uint32_t lane = threadIdx.x & 63u, wave = uni(threadIdx.x >> 6);
  fx_u32x4* const w4 = (fx_u32x4*)(L + la.win_off);

  // the rows of the first tile are on their way before anything else is read
  fx_u32x4 wr[FX_WK];
  {
    const FxWinAddr a = fx_win_addr(la, blockIdx.x);
#pragma unroll
    for (uint32_t k = 0; k < FX_WK; ++k) {
      const uint32_t v = threadIdx.x + k * NT;
      if (v < a.n_vec) wr[k] = a.g4[v];
    }
  }
  fx_u32x4 ws[FX_SIDE_WIN];   // side windows: one line per lane
#pragma unroll
  for (int i = 0; i < FX_SIDE_WIN; ++i) {
    if ((uint32_t)i < la.n_side) {
      const FxWinAddr a = fx_side_addr(la, blockIdx.x, i);
      if (threadIdx.x < a.n_vec) ws[i] = a.g4[threadIdx.x];
    }
  }
  fx_stage(L, sb, la);   // descriptor and tables; ends with a barrier
  const uint32_t* cls0 = L + uni(L[FX_W(FxHeader, off_class)]);
  const int mb = (int)uni(cls0[FX_W(FxClass, mask_begin)]), me = (int)uni(cls0[FX_W(FxClass, mask_end)]);
  const uint32_t mask_vt = uni(cls0[FX_W(FxClass, mask_vt)]);

  for (uint32_t b = blockIdx.x; b < n_tiles; b += gridDim.x) {
    const FxWinAddr wa = fx_win_addr(la, b);
    __syncthreads();   // the previous tile's window and row map are no longer read
#pragma unroll
    for (uint32_t k = 0; k < FX_WK; ++k) {
      const uint32_t v = threadIdx.x + k * NT;
      if (v < wa.n_vec) w4[v] = wr[k];
    }
    for (uint32_t v = threadIdx.x + FX_WK * NT; v < wa.n_vec; v += NT) w4[v] = wa.g4[v];
    FxWinAddr sa[FX_SIDE_WIN];
#pragma unroll
    for (int i = 0; i < FX_SIDE_WIN; ++i) {
      if ((uint32_t)i < la.n_side) {
        sa[i] = fx_side_addr(la, b, i);
        if (threadIdx.x < sa[i].n_vec) ((fx_u32x4*)(L + la.side_off[i]))[threadIdx.x] = ws[i];
      }
    }
    __syncthreads();

    // one task class: tile and task follow from the tile number
    FxWork w;
    w.cls = cls0;
    w.local_block = wa.tile;
    w.task = (int)uni(L[uni(L[FX_W(FxHeader, off_taskmap)]) + wa.task_i]);
    FxCtx cx = fx_make_ctx(L, la, w);
    cx.all_win = true;
    cx.win = L + la.win_off + wa.shift;
    cx.win_slot = (int32_t)la.s_win_slot;
    cx.win_base = wa.e0;
#pragma unroll
    for (int i = 0; i < FX_SIDE_WIN; ++i) {
      if ((uint32_t)i < la.n_side) {
        cx.side[i] = L + la.side_off[i] + sa[i].shift;
        cx.side_slot[i] = (int32_t)la.side_slot[i];
        cx.side_base[i] = sa[i].e0;
      }
    }

    // ---- mask, row map ----------------------------------------------------
    auto mask_of = [&](const FxCtx& c, uint32_t row, bool live) -> bool {
      FxCoord<1> q;
      q.c0[0] = 0;
      q.vd = 0;
      q.step = 0;
#pragma unroll
      for (int j = 0; j < FX_V; ++j) q.cv[j] = 0;
      q.cv[0] = live ? (int32_t)row : 0;
      uint32_t A[FX_V];
#pragma unroll
      for (int j = 0; j < FX_V; ++j) A[j] = 0;
      S::run_mask(c, mb, me, q, live ? 1u : 0u, A);
      return live && (mask_vt == FX_VT_F ? (u2f(A[0]) != 0.0f) : (A[0] != 0u));
    };
    const uint32_t row = wa.r0 + threadIdx.x;
    const bool keep = mask_of(cx, row, threadIdx.x < wa.rows);
    const uint64_t bal = __builtin_amdgcn_ballot_w64(keep);
    const uint32_t before = (uint32_t)__popcll(bal & ((1ull << lane) - 1ull));
    if (lane == 0) s_woff[wave + 1] = (uint32_t)__popcll(bal);
    __syncthreads();
    if (threadIdx.x == 0) {
      uint32_t acc = 0;
      s_woff[0] = 0;
      for (uint32_t k = 1; k <= NW; ++k) { acc += s_woff[k]; s_woff[k] = acc; }
    }
    __syncthreads();
    if (keep) s_rowmap[s_woff[wave] + before] = row;
    const uint32_t n_kept = uni(s_woff[NW]);

    // ---- publish the count, sum the earlier tiles --------------------------
    uint32_t* status = (uint32_t*)cx.ptrs[uni(L[FX_W(FxHeader, slot_status)])];
    if (threadIdx.x == 0)
      __hip_atomic_store(status + b, (la.epoch << FX_STATUS_BITS) | n_kept, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (wave == 0) {
      const uint32_t first = b - wa.tile;
      uint32_t part = 0;
      bool ok = true;
      for (uint32_t i = lane; i < wa.tile; i += 64u) {
        uint32_t wv = 0, polls = 0;
        for (;;) {
          wv = __hip_atomic_load(status + first + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if ((wv >> FX_STATUS_BITS) == la.epoch) break;
          if (polls >= la.spin_limit) { ok = false; break; }
          ++polls;
          __builtin_amdgcn_s_sleep(1);
        }
        part += ok ? (wv & ((1u << FX_STATUS_BITS) - 1u)) : 0u;
      }
      part = fx_wave_sum(part, threadIdx.x & 63u);
      const bool all_ok = __builtin_amdgcn_ballot_w64(!ok) == 0ull;
      if (lane == 0) { s_prefix = part; s_ok = all_ok ? 1u : 0u; }
    }
    __syncthreads();
    if (uni(s_ok) == 0u) {
      // an earlier tile has not reported in time: count its kept rows here, from memory
      FxCtx cg = cx;
      cg.all_win = false;
      uint32_t cnt = 0;
      for (uint32_t p = 0; p < wa.tile; ++p) {
        const bool k2 = mask_of(cg, p * la.s_tile_rows + threadIdx.x, threadIdx.x < la.s_tile_rows);
        cnt += (uint32_t)__popcll(__builtin_amdgcn_ballot_w64(k2));
      }
      __syncthreads();
      if (lane == 0) s_wsum[wave] = cnt;
      __syncthreads();
      if (threadIdx.x == 0) {
        uint32_t p = 0;
        for (uint32_t k = 0; k < NW; ++k) p += s_wsum[k];
        s_prefix = p;
      }
      __syncthreads();
    }
    const uint32_t prefix = uni(s_prefix);
    if (wa.tile + 1u == la.s_tiles && threadIdx.x == 0)
      __hip_atomic_store((uint32_t*)cx.ptrs[uni(L[FX_W(FxHeader, slot_total)])] + w.task, prefix + n_kept, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_SYSTEM);

    // ---- outputs.  The rows of this workgroup's next tile are requested in front of the last,
    // widest output: behind the loads that the narrow outputs wait for, because loads return in
    // order.  They travel in registers until the next turn of the loop parks them in LDS.
    const uint32_t bn = b + gridDim.x;
    auto prefetch = [&]() {
      if (bn < n_tiles) {
        const FxWinAddr na = fx_win_addr(la, bn);
#pragma unroll
        for (uint32_t k = 0; k < FX_WK; ++k) {
          const uint32_t v = threadIdx.x + k * NT;
          if (v < na.n_vec) wr[k] = na.g4[v];
        }
#pragma unroll
        for (int i = 0; i < FX_SIDE_WIN; ++i) {
          if ((uint32_t)i < la.n_side) {
            const FxWinAddr a = fx_side_addr(la, bn, i);
            if (threadIdx.x < a.n_vec) ws[i] = a.g4[threadIdx.x];
          }
        }
      }
    };
    if (n_kept == 0) {
      prefetch();
      continue;
    }
    fx_scatter_outputs<R, S, NW>(cx, w, L, s_rowmap, n_kept, prefix, lane, wave, prefetch);
  }
}
