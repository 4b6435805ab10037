// Test-only: a generated row-stream translation unit (fx_plan_rowstream_source) compiled as plain
// C++ and driven on the CPU the way the device skeleton (fx_rowstream.h) drives it: chunks of a
// task in order, sub-tiles of a chunk copied into a window buffer, row map from the mask, one
// call of P::row per kept row, the vector segments thread by thread.  The transcendental
// routines are those of the bytecode emulator (fx_emul.cpp), so the results must equal the
// emulator's bit for bit: this checks the generator (symbolic execution, folding of column
// predicates, shared sub-expressions, merged loads, segment bounds) without a GPU.
// Build: g++ -DFX_RS_GENERATED='"<file>"' -shared -fPIC fx_rs_host.cpp
#include <math.h>
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <vector>

#define FX_RS_HOST 1
#define FX_RS_FN inline
#include "../../functs_amd/csrc/fxhip/fx_bytecode.h"
#include "../../functs_amd/csrc/fxhip/fx_rs.h"

namespace {
float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
int32_t floordiv_i(int32_t a, int32_t b) {
  if (b == 0) return 0;
  int32_t q = a / b;
  if ((a % b != 0) && ((a < 0) != (b < 0))) --q;
  return q;
}
int32_t pymod_i(int32_t a, int32_t b) {
  if (b == 0) return 0;
  int32_t r = a % b;
  if (r != 0 && ((r < 0) != (b < 0))) r += b;
  return r;
}
float fx_fmax(float a, float b) { return (a > b || a != a) ? a : b; }
float fx_fmin(float a, float b) { return (a < b || a != a) ? a : b; }
// as the emulator computes them
float rs_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
float rs_exp(float x) { return expf(x); }
float rs_tanh(float x) { return tanhf(x); }

uint32_t half_to_f32(uint16_t h) {
  uint32_t s = (h >> 15) & 1, e = (h >> 10) & 31, m = h & 1023;
  if (e == 0) {
    if (m == 0) return s << 31;
    float f = ldexpf((float)m, -24);
    return f2u(s ? -f : f);
  }
  if (e == 31) return (s << 31) | 0x7f800000u | (m << 13);
  return (s << 31) | ((e + 112) << 23) | (m << 13);
}

struct FxRsRt {
  const FxRsLaunch& la;
  uint32_t task;
  const FxDyn* dyn;
  uint32_t* errw;
  uint32_t* stg[FX_RS_MAX_OUT];
  uint32_t ph[FX_RS_MAX_OUT];
  const uint32_t* staged(int k) const { return stg[k]; }
  uint64_t ptr(uint32_t slot) const {
    const uint32_t pi = (slot & FX_SLOT_TASK) ? la.n_sptr + task * la.n_tptr + (slot & 0xffffu) : (slot & 0xffffu);
    return dyn->p[pi];
  }
  uint32_t scal(int32_t slot) const {
    const uint32_t si = ((uint32_t)slot & FX_SLOT_TASK) ? la.n_sscal + task * la.n_tscal + ((uint32_t)slot & 0xffffu) : ((uint32_t)slot & 0xffffu);
    return dyn->s[si];
  }
  uint32_t fimm(int k) const { return la.fimm[k]; }
  uint64_t in(int k) const { return ptr(la.in_slot[k]); }
  uint32_t toff(int k) const { return (uint32_t)(la.in_tcoef[k] * (int32_t)task); }
  uint64_t out(int k) const { return ptr(la.out_slot[k]); }
  uint32_t ooff(int k) const { return la.out_tstride[k] * task; }
};

template <int CVT>
uint32_t rs_scal(const FxRsRt& rt, int32_t slot) {
  const uint32_t s = rt.scal(slot);
  return CVT ? f2u((float)(int32_t)s) : s;
}
template <uint32_t DT, int CVT>
uint32_t rs_ldx_at(const FxRsRt& rt, int k, uint32_t o) {
  const uint8_t* base = (const uint8_t*)(uintptr_t)rt.in(k);
  uint32_t v = 0;
  switch (DT) {
    case FX_F32: case FX_I32: memcpy(&v, base + ((size_t)o << 2), 4); break;
    case FX_I64: {
      int64_t w;
      memcpy(&w, base + ((size_t)o << 3), 8);
      if (CVT) return f2u((float)w);
      if (w != (int64_t)(int32_t)w && rt.errw) *rt.errw = 1u;
      v = (uint32_t)w;
    } break;
    case FX_I64LO: memcpy(&v, base + ((size_t)o << 3), 4); break;
    case FX_I64HI: memcpy(&v, base + ((size_t)o << 3) + 4, 4); break;
    case FX_U8: v = base[o]; break;
    case FX_F16: { uint16_t h; memcpy(&h, base + ((size_t)o << 1), 2); v = half_to_f32(h); } break;
    default: { uint16_t h; memcpy(&h, base + ((size_t)o << 1), 2); v = (uint32_t)h << 16; } break;
  }
  if (CVT) v = f2u((float)(int32_t)v);
  return v;
}
template <uint32_t DT, int CVT>
uint32_t rs_ld(const FxRsRt& rt, int k, uint32_t off) { return rs_ldx_at<DT, CVT>(rt, k, off + rt.toff(k)); }
template <uint32_t DT>
uint32_t rs_ldx(const FxRsRt& rt, int k, uint32_t off) { return rs_ldx_at<DT, 0>(rt, k, off); }
void rs_ld2(const FxRsRt& rt, int k, uint32_t off, uint32_t& a, uint32_t& b) {
  a = rs_ld<FX_F32, 0>(rt, k, off);
  b = rs_ld<FX_F32, 0>(rt, k, off + 1);
}
void rs_ld4(const FxRsRt& rt, int k, uint32_t off, uint32_t& a, uint32_t& b, uint32_t& c, uint32_t& d) {
  a = rs_ld<FX_F32, 0>(rt, k, off);
  b = rs_ld<FX_F32, 0>(rt, k, off + 1);
  c = rs_ld<FX_F32, 0>(rt, k, off + 2);
  d = rs_ld<FX_F32, 0>(rt, k, off + 3);
}
template <uint32_t DT, uint32_t VT>
void rs_st(const FxRsRt& rt, int k, uint32_t off, uint32_t v) {
  uint8_t* base = (uint8_t*)(uintptr_t)rt.out(k);
  const size_t o = (size_t)off + rt.ooff(k);
  switch (DT) {
    case FX_F32: { uint32_t w = VT == FX_VT_F ? v : f2u((float)(int32_t)v); memcpy(base + (o << 2), &w, 4); } break;
    case FX_I32: { int32_t w = VT == FX_VT_I ? (int32_t)v : (int32_t)u2f(v); memcpy(base + (o << 2), &w, 4); } break;
    case FX_I64: { int64_t w = VT == FX_VT_I ? (int64_t)(int32_t)v : (int64_t)u2f(v); memcpy(base + (o << 3), &w, 8); } break;
    case FX_I64LO: memcpy(base + (o << 3), &v, 4); break;
    case FX_I64HI: memcpy(base + (o << 3) + 4, &v, 4); break;
    case FX_U8: base[o] = VT == FX_VT_I ? (uint8_t)v : (uint8_t)(u2f(v) != 0.0f); break;
    case FX_BF16: {
      float f = VT == FX_VT_F ? u2f(v) : (float)(int32_t)v;
      uint32_t u = f2u(f);
      uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
      if (f != f) r = 0x7fc0u;
      uint16_t h = (uint16_t)r;
      memcpy(base + (o << 1), &h, 2);
    } break;
    default: break;
  }
}
void rs_st4(const FxRsRt& rt, int k, uint32_t off, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  rs_st<FX_F32, FX_VT_F>(rt, k, off, a);
  rs_st<FX_F32, FX_VT_F>(rt, k, off + 1, b);
  rs_st<FX_F32, FX_VT_F>(rt, k, off + 2, c);
  rs_st<FX_F32, FX_VT_F>(rt, k, off + 3, d);
}

void rs_stl(const FxRsRt& rt, int k, uint32_t off, uint32_t v) { rt.stg[k][rt.ph[k] + off] = v; }
void rs_st_at(const FxRsRt& rt, int k, uint32_t e, uint32_t v) {
  memcpy((uint8_t*)(uintptr_t)rt.out(k) + ((size_t)e << 2), &v, 4);
}
void rs_st4_at(const FxRsRt& rt, int k, uint32_t e, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  if (e & 3u) __builtin_trap();   // a group that is not aligned in memory
  rs_st_at(rt, k, e, a);
  rs_st_at(rt, k, e + 1, b);
  rs_st_at(rt, k, e + 2, c);
  rs_st_at(rt, k, e + 3, d);
}

}  // namespace
#include "../../functs_amd/csrc/fxhip/fx_rs_ops.h"
namespace {

uint64_t g_key = 0;
uint32_t g_S = 0;
typedef void (*RunFn)(const FxRsLaunch&, const FxDyn*, uint32_t*, uint32_t);
RunFn g_run = nullptr;

template <class P>
void run_policy(const FxRsLaunch& la, const FxDyn* dyn, uint32_t* totals, uint32_t nt) {
  const uint32_t S = P::S;
  uint32_t errw = 0;
  for (uint32_t task = 0; task < la.n_tasks; ++task) {
    FxRsRt rt{la, task, dyn, &errw, {}, {}};
    // staged outputs: sub_rows rows each and a group of slack, poisoned before every sub-tile
    std::vector<std::vector<uint32_t>> stage(FX_RS_MAX_OUT);
    for (uint32_t k = 0; k < FX_RS_MAX_OUT; ++k) {
      stage[k].assign(k < P::n_out && P::stage_rowlen[k] ? (size_t)la.sub_rows * P::stage_rowlen[k] + 8u : 8u, 0u);
      rt.stg[k] = stage[k].data();
      rt.ph[k] = 0;
    }
    const uint32_t* win = (const uint32_t*)(uintptr_t)rt.in(0) + (int64_t)la.in_tcoef[0] * task;
    uint32_t prefix = 0;
    for (uint32_t chunk = 0; chunk < la.chunks; ++chunk) {
      const uint32_t c_r0 = chunk * la.chunk_rows;
      const uint32_t c_rows = la.chunk_rows < la.n_rows - c_r0 ? la.chunk_rows : la.n_rows - c_r0;
      std::vector<uint8_t> keep(c_rows);
      for (uint32_t r = 0; r < c_rows; ++r) keep[r] = P::template mask<FxRsRt>(rt, c_r0 + r) ? 1 : 0;
      const uint32_t n_sub0 = (c_rows + la.sub_rows - 1u) / la.sub_rows;
      const uint32_t sub_rows = (c_rows + n_sub0 - 1u) / n_sub0;
      const uint32_t n_sub = (c_rows + sub_rows - 1u) / sub_rows;
      uint32_t before = 0;
      for (uint32_t s = 0; s < n_sub; ++s) {
        const uint32_t t_r0 = s * sub_rows, t_rows = sub_rows < c_rows - t_r0 ? sub_rows : c_rows - t_r0;
        const uint32_t rs0 = c_r0 + t_r0;
        // the window: a copy of the sub-tile's rows behind a few words of padding (on the device:
        // the elements between the 16-byte line and the first row)
        std::vector<uint32_t> L(3 + (size_t)t_rows * S + 4, 0xdeadbeefu);
        memcpy(L.data() + 3, win + (size_t)rs0 * S, (size_t)t_rows * S * 4);
        const uint32_t* Wb = L.data() + 3;
        std::vector<uint32_t> rowmap;
        for (uint32_t r = 0; r < t_rows; ++r)
          if (keep[t_r0 + r]) rowmap.push_back(r);
        const uint32_t n_kept = (uint32_t)rowmap.size();
        const uint32_t orow = prefix + before;
        for (auto& st : stage) std::fill(st.begin(), st.end(), 0xdeadbeefu);
        fx_rs_phases<P, 0u, FxRsRt>(rt, orow);
        if (P::n_row_cols != 0u)
          for (uint32_t r = 0; r < n_kept; ++r) {
            typename P::Side sd;
            P::template row_side<FxRsRt>(rt, rs0 + rowmap[r], sd);
            P::template row<FxRsRt>(rt, Wb + rowmap[r] * S, sd, rs0 + rowmap[r], orow + r, r);
          }
        for (uint32_t tid = 0; tid < nt; ++tid)
          fx_rs_segments<P, FxRsRt>(typename P::Vecs{}, rt, Wb, rowmap.data(), n_kept, rs0, orow, tid, nt);
        if (P::n_staged != 0u)
          for (uint32_t tid = 0; tid < nt; ++tid) fx_rs_copy_out<P, 0u, FxRsRt>(rt, n_kept, orow, tid, nt);
        before += n_kept;
      }
      prefix += before;
    }
    if (totals) totals[task] = prefix;
  }
}

struct FxRsRegistrar {
  FxRsRegistrar(uint64_t key, uint32_t S, RunFn fn) { g_key = key; g_S = S; g_run = fn; }
};
}  // namespace

#define FX_RS_REGISTER(P) static FxRsRegistrar fx_rs_registrar_host(P::key, P::S, &run_policy<P>);

#include FX_RS_GENERATED

extern "C" uint64_t fx_rs_host_key(void) { return g_key; }
extern "C" size_t fx_rs_host_launch_bytes(void) { return sizeof(FxRsLaunch); }
// la: what fx_plan_rowstream_launch filled in (geometry included); dyn: the marshalled block
extern "C" int fx_rs_host_run(const void* la, const void* dyn, uint32_t* totals, uint32_t threads) {
  if (!g_run || !la || !dyn) return -1;
  const FxRsLaunch* l = (const FxRsLaunch*)la;
  if (l->chunk_rows == 0 || l->sub_rows == 0 || l->chunks * l->chunk_rows < l->n_rows) return -2;
  g_run(*l, (const FxDyn*)dyn, totals, threads ? threads : 1u);
  return 0;
}
