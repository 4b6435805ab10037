// TEST INFRASTRUCTURE ONLY - never linked into or loaded by the product.
//
// Scalar CPU emulator of the region bytecode (functs_amd/csrc/fxhip/fx_bytecode.h).
// It executes a lowered region blob one element at a time with host pointers,
// so that the host lowering (shape functions, index arithmetic, predication,
// slot marshalling) can be checked against the oracle without a GPU.  The GPU
// kernels are checked separately against the same oracle.
#include <math.h>
#include <stdint.h>
#include <string.h>

#include <vector>

#include "../../functs_amd/csrc/fxhip/fx_bytecode.h"

namespace {

float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

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

// int64 data in 32-bit arithmetic: converted to float the whole value counts; as an integer
// the low word is the value and an element that does not fit is reported through *err
uint32_t load_elem(const void* base, int64_t off, uint32_t dt, bool cvt = false, uint32_t* err = nullptr) {
  switch (dt) {
    case FX_F32: case FX_I32: return ((const uint32_t*)base)[off];
    case FX_I64: {
      const int64_t v = ((const int64_t*)base)[off];
      if (cvt) return f2u((float)v);
      if (v != (int64_t)(int32_t)v && err) *err = 1u;
      return (uint32_t)v;
    }
    case FX_I64LO: return ((const uint32_t*)base)[2 * off];
    case FX_I64HI: return ((const uint32_t*)base)[2 * off + 1];
    case FX_U8: return ((const uint8_t*)base)[off];
    case FX_F16: return half_to_f32(((const uint16_t*)base)[off]);
    case FX_BF16: return ((uint32_t)((const uint16_t*)base)[off]) << 16;
  }
  return 0;
}

void store_elem(void* base, int64_t off, uint32_t dt, uint32_t vt, uint32_t v) {
  switch (dt) {
    case FX_F32: ((uint32_t*)base)[off] = vt == FX_VT_F ? v : f2u((float)(int32_t)v); break;
    case FX_I32: ((int32_t*)base)[off] = vt == FX_VT_I ? (int32_t)v : (int32_t)u2f(v); break;
    case FX_I64: ((int64_t*)base)[off] = vt == FX_VT_I ? (int64_t)(int32_t)v : (int64_t)u2f(v); break;
    case FX_I64LO: ((uint32_t*)base)[2 * off] = v; break;
    case FX_I64HI: ((uint32_t*)base)[2 * off + 1] = v; break;
    case FX_U8: ((uint8_t*)base)[off] = vt == FX_VT_I ? (uint8_t)v : (uint8_t)(u2f(v) != 0.0f); break;
    case FX_BF16: {
      float f = vt == FX_VT_F ? u2f(v) : (float)(int32_t)v;
      uint32_t u = f2u(f);
      uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
      if (f != f) r = 0x7fc0u;
      ((uint16_t*)base)[off] = (uint16_t)r;
    } break;
    default: break;  // f16 stores are not emulated
  }
}

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

struct Ctx {
  const FxInsn* insn;
  const FxAffine* aff;
  const uint64_t* sptr;
  const uint64_t* tptr;
  const uint32_t* sscal;
  const uint32_t* tscal;
  int task;
  uint32_t* err;
};

const void* ptr_of(const Ctx& cx, int32_t slot) {
  uint64_t p = (slot & FX_SLOT_TASK) ? cx.tptr[slot & 0xffff] : cx.sptr[slot & 0xffff];
  return (const void*)(uintptr_t)p;
}
uint32_t scalar_of(const Ctx& cx, int32_t slot) {
  return (slot & FX_SLOT_TASK) ? cx.tscal[slot & 0xffff] : cx.sscal[slot & 0xffff];
}

// A batch of elements executed in lockstep, like the lanes of one wave item:
// control flow is uniform, `live` mirrors the lane mask.  Batches of one element
// are used for ordinary outputs; row-per-wave outputs run one row per batch so
// that FX_WMAX / FX_WSUM see exactly the elements the GPU wave sees.
struct Lane {
  uint32_t A = 0, B = 0;
  bool M = true;
  std::vector<bool> stack;
  uint32_t temps[FX_MAX_TEMPS];
  int32_t c[FX_MAXR];
};

void run(const Ctx& cx, int pc, int pc_end, std::vector<Lane>& L) {
  for (auto& l : L) { l.A = 0; l.B = 0; l.M = true; l.stack.clear(); memset(l.temps, 0, sizeof(l.temps)); }
  int32_t lc[FX_MAXLOOP] = {0, 0}, le[FX_MAXLOOP] = {0, 0};
  long guard = 0;
  auto any_live = [&]() { for (auto& l : L) if (l.M) return true; return false; };
  while (pc < pc_end) {
    if (++guard > 50000000) break;
    const FxInsn ins = cx.insn[pc++];
    const bool useimm = ins.flags & FX_F_IMM;
    if (ins.op == FX_MIF) {
      for (auto& l : L) { l.stack.push_back(l.M); l.M = l.M && (l.A != 0); }
      if (!any_live()) pc = ins.a;
      continue;
    }
    auto affine_at = [&](const Lane& l, int idx) {
      const FxAffine& af = cx.aff[idx];
      int32_t off = af.base + af.tcoef * cx.task + af.rcoef[0] * lc[0] + af.rcoef[1] * lc[1];
      for (int k = 0; k < FX_MAXR; ++k) off += fx_aff_coef(&af, k) * l.c[k];
      return off;
    };
    if (ins.op == FX_MIFR) {
      const uint32_t hi = ins.imm >> 8;
      const int32_t st = (int32_t)(ins.imm & 255u);
      for (auto& l : L) {
        const int32_t x = affine_at(l, ins.b);
        const bool in = (uint32_t)x < hi && (st <= 1 || x % st == 0);
        l.A = in ? 1u : 0u;
        l.stack.push_back(l.M);
        l.M = l.M && in;
      }
      if (!any_live()) pc = ins.a;
      continue;
    }
    if (ins.op == FX_MELSE) {
      for (auto& l : L) l.M = l.stack.back() && !l.M;
      if (!any_live()) pc = ins.a;
      continue;
    }
    if (ins.op == FX_RBEGIN) { int d = ins.a & (FX_MAXLOOP - 1); lc[d] = 0; le[d] = (int32_t)ins.imm; if (le[d] <= 0) pc = ins.b; continue; }
    if (ins.op == FX_RNEXT) { int d = ins.b & (FX_MAXLOOP - 1); lc[d] += 1; if (lc[d] < le[d]) pc = ins.a; continue; }
    if (ins.op == FX_WMAX || ins.op == FX_WSUM) {
      float v = ins.op == FX_WMAX ? -INFINITY : 0.0f;
      for (auto& l : L) if (l.M) v = ins.op == FX_WMAX ? fx_fmax(v, u2f(l.A)) : v + u2f(l.A);
      for (auto& l : L) l.A = f2u(v);
      continue;
    }
    for (auto& l : L) {
      uint32_t& A = l.A;
      uint32_t& B = l.B;
      const bool M = l.M;
      uint32_t* temps = l.temps;
      const int32_t* c = l.c;
      if (ins.flags & FX_F_TMPB) B = temps[ins.a];
      else if ((ins.flags & FX_F_MEMB) && M) {
        const bool wide = ins.dt == FX_I64 && (ins.flags & FX_F_I2F);
        B = load_elem(ptr_of(cx, ins.a), affine_at(l, ins.b), ins.dt, wide, l.M ? cx.err : nullptr);
        if ((ins.flags & FX_F_I2F) && !wide) B = f2u((float)(int32_t)B);
      }
      const float fa = u2f(A), fb = u2f(useimm ? ins.imm : B);
      const int32_t ia = (int32_t)A, ib = (int32_t)(useimm ? ins.imm : B);
      switch (ins.op) {
        case FX_NOP: break;
        case FX_LDB: case FX_LDTB: break;  // the operand fetch above did it
        case FX_LDA: case FX_AFFA: case FX_AFFB: {
          if (!M) break;
          const int32_t off = affine_at(l, ins.b);
          const bool is_load = ins.op == FX_LDA;
          const bool wide = is_load && ins.dt == FX_I64 && (ins.flags & FX_F_I2F);
          uint32_t v = is_load ? load_elem(ptr_of(cx, ins.a), off, ins.dt, wide, l.M ? cx.err : nullptr) : (uint32_t)off;
          if ((ins.flags & FX_F_I2F) && !wide) v = f2u((float)(int32_t)v);
          if (ins.op == FX_LDA || ins.op == FX_AFFA) A = v; else B = v;
        } break;
        case FX_LDXA: if (M) A = load_elem(ptr_of(cx, ins.a), (int64_t)((int32_t)A + (int32_t)ins.imm), ins.dt, false, cx.err); break;
        case FX_IMMA: if (M) A = ins.imm; break;
        case FX_IMMB: B = ins.imm; break;
        case FX_SCLA: if (M) { A = scalar_of(cx, ins.a); if (ins.flags & FX_F_I2F) A = f2u((float)(int32_t)A); } break;
        case FX_SCLB: B = scalar_of(cx, ins.a); if (ins.flags & FX_F_I2F) B = f2u((float)(int32_t)B); break;
        case FX_STT: temps[ins.a] = A; break;
        case FX_LDTA: if (M) A = temps[ins.a]; break;
        case FX_MOVBA: B = A; break;
        case FX_SWAP: { uint32_t t = A; A = B; B = t; } break;
        case FX_MMERGE: A = M ? A : temps[ins.a]; l.M = l.stack.back(); l.stack.pop_back(); break;
        case FX_MEND: l.M = l.stack.back(); l.stack.pop_back(); break;
        case FX_FNEG: A = f2u(-fa); break;
        case FX_FABS: A = f2u(fabsf(fa)); break;
        case FX_EXP: A = f2u(expf(fa)); break;
        case FX_LOG: A = f2u(logf(fa)); break;
        case FX_SQRT: A = f2u(sqrtf(fa)); break;
        case FX_RSQRT: A = f2u(1.0f / sqrtf(fa)); break;
        case FX_RCP: A = f2u(1.0f / fa); break;
        case FX_SIGMOID: A = f2u(1.0f / (1.0f + expf(-fa))); break;
        case FX_TANH: A = f2u(tanhf(fa)); break;
        case FX_RELU: A = f2u(fa <= 0.0f ? 0.0f : fa); break;
        case FX_FLOOR: A = f2u(floorf(fa)); break;
        case FX_CEIL: A = f2u(ceilf(fa)); break;
        case FX_ROUND: A = f2u(rintf(fa)); break;
        case FX_TRUNC: A = f2u(truncf(fa)); break;
        case FX_SIN: A = f2u(sinf(fa)); break;
        case FX_COS: A = f2u(cosf(fa)); break;
        case FX_ERF: A = f2u(erff(fa)); break;
        case FX_LOG2: A = f2u(log2f(fa)); break;
        case FX_EXP2: A = f2u(exp2f(fa)); break;
        case FX_EXPM1: A = f2u(expm1f(fa)); break;
        case FX_LOG1P: A = f2u(log1pf(fa)); break;
        case FX_INEG: A = (uint32_t)(-ia); break;
        case FX_IABS: A = (uint32_t)(ia < 0 ? -ia : ia); break;
        case FX_LNOT: A = ia == 0; break;
        case FX_INZ: A = ia != 0; break;
        case FX_FNZ: A = fa != 0.0f; break;
        case FX_F2I: A = (uint32_t)(int32_t)fa; break;
        case FX_I2F: A = f2u((float)ia); break;
        case FX_FADD: A = f2u(fa + fb); break;
        case FX_FSUB: A = f2u(fa - fb); break;
        case FX_FRSUB: A = f2u(fb - fa); break;
        case FX_FMUL: A = f2u(fa * fb); break;
        case FX_FDIV: A = f2u(fa / fb); break;
        case FX_FRDIV: A = f2u(fb / fa); break;
        case FX_FMIN: A = f2u(fx_fmin(fa, fb)); break;
        case FX_FMAX: A = f2u(fx_fmax(fa, fb)); break;
        case FX_FPOW: A = f2u(powf(fa, fb)); break;
        case FX_FMOD: A = f2u(fmodf(fa, fb)); break;
        case FX_ATAN2: A = f2u(atan2f(fa, fb)); break;
        case FX_IADD: A = (uint32_t)(ia + ib); break;
        case FX_ISUB: A = (uint32_t)(ia - ib); break;
        case FX_IRSUB: A = (uint32_t)(ib - ia); break;
        case FX_IMUL: A = (uint32_t)(ia * ib); break;
        case FX_IFDIV: A = (uint32_t)floordiv_i(ia, ib); break;
        case FX_ITDIV: A = (uint32_t)(ib == 0 ? 0 : ia / ib); break;
        case FX_IPMOD: A = (uint32_t)pymod_i(ia, ib); break;
        case FX_ITMOD: A = (uint32_t)(ib == 0 ? 0 : ia % ib); break;
        case FX_IMIN: A = (uint32_t)(ia < ib ? ia : ib); break;
        case FX_IMAX: A = (uint32_t)(ia > ib ? ia : ib); break;
        case FX_IAND: A = (uint32_t)(ia & ib); break;
        case FX_IOR: A = (uint32_t)(ia | ib); break;
        case FX_IXOR: A = (uint32_t)(ia ^ ib); break;
        case FX_FLT: A = fa < fb; break;
        case FX_FLE: A = fa <= fb; break;
        case FX_FGT: A = fa > fb; break;
        case FX_FGE: A = fa >= fb; break;
        case FX_FEQ: A = fa == fb; break;
        case FX_FNE: A = fa != fb; break;
        case FX_ILT: A = ia < ib; break;
        case FX_ILE: A = ia <= ib; break;
        case FX_IGT: A = ia > ib; break;
        case FX_IGE: A = ia >= ib; break;
        case FX_IEQ: A = ia == ib; break;
        case FX_INE: A = ia != ib; break;
        case FX_IRANGE: {
          int32_t lo = ins.a, hi = ins.b, st = (int32_t)ins.imm;
          bool in = ia >= lo && ia < hi;
          if (st > 1) in = in && ((ia - lo) % st == 0);
          A = in;
        } break;
        case FX_WHERE: A = temps[ins.a] != 0 ? A : B; break;
        case FX_RIDX: if (M) A = (uint32_t)lc[ins.a & (FX_MAXLOOP - 1)]; break;
        default: break;
      }
    }
  }
}

uint32_t run1(const Ctx& cx, int pc, int pc_end, const int32_t* c) {
  std::vector<Lane> L(1);
  memcpy(L[0].c, c, sizeof(L[0].c));
  run(cx, pc, pc_end, L);
  return L[0].A;
}

void decompose(const FxOut& od, uint32_t e, int32_t* c) {
  for (int k = FX_MAXR - 1; k >= 1; --k) { c[k] = (int32_t)(e % od.dim[k]); e /= od.dim[k]; }
  c[0] = (int32_t)e;
}

}  // namespace

extern "C" int fx_emul_run_tables(const uint32_t* sb, size_t n_words, const uint64_t* pointers, const uint32_t* scalars, uint32_t* totals);
extern "C" int fx_emul_run(const uint32_t* sb, size_t n_words, const void* dyn_, uint32_t* totals) {
  const FxDyn* dyn = (const FxDyn*)dyn_;
  return fx_emul_run_tables(sb, n_words, dyn->p, dyn->s, totals);
}
// the same with the two tables at any length (a map of more tasks than the by-value block holds)
extern "C" int fx_emul_run_tables(const uint32_t* sb, size_t n_words, const uint64_t* pointers, const uint32_t* scalars, uint32_t* totals) {
  (void)n_words;
  struct { const uint64_t* p; const uint32_t* s; } tables = {pointers, scalars}, *dyn = &tables;
  const FxHeader* h = (const FxHeader*)sb;
  if (h->magic != FX_MAGIC) return -1;
  const FxClass* cls = (const FxClass*)(sb + h->off_class);
  const uint32_t* taskmap = sb + h->off_taskmap;
  for (uint32_t ci = 0; ci < h->n_classes; ++ci) {
    const FxClass& cl = cls[ci];
    const FxOut* outs = (const FxOut*)(sb + cl.off_outs);
    for (uint32_t ti = 0; ti < cl.n_tasks; ++ti) {
      int task = (int)taskmap[cl.first_task + ti];
      Ctx cx;
      cx.insn = (const FxInsn*)(sb + cl.off_insn);
      cx.aff = (const FxAffine*)(sb + cl.off_aff);
      cx.sptr = dyn->p;
      cx.tptr = dyn->p + h->n_sptr + (size_t)task * h->n_tptr;
      cx.sscal = dyn->s;
      cx.tscal = dyn->s + h->n_sscal + (size_t)task * h->n_tscal;
      cx.task = task;
      cx.err = h->slot_err ? (uint32_t*)(uintptr_t)dyn->p[h->slot_err - 1] : nullptr;
      if (h->mode == FX_MODE_DENSE) {
        for (uint32_t oi = 0; oi < cl.n_outs; ++oi) {
          const FxOut& od = outs[oi];
          void* op = (void*)ptr_of(cx, (int32_t)od.ptr_slot);
          if (od.rowwave) {
            const uint32_t rows = od.rowlen ? od.numel / od.rowlen : 0;
            for (uint32_t r = 0; r < rows; ++r) {
              std::vector<Lane> L(od.rowlen);
              for (uint32_t k = 0; k < od.rowlen; ++k) decompose(od, r * od.rowlen + k, L[k].c);
              run(cx, (int)od.prog_begin, (int)od.prog_end, L);
              for (uint32_t k = 0; k < od.rowlen; ++k)
                store_elem(op, (int64_t)od.task_stride * task + r * od.rowlen + k, od.dtype, od.vt, L[k].A);
            }
            continue;
          }
          for (uint32_t e = 0; e < od.numel; ++e) {
            int32_t c[FX_MAXR];
            decompose(od, e, c);
            uint32_t v = run1(cx, (int)od.prog_begin, (int)od.prog_end, c);
            store_elem(op, (int64_t)od.task_stride * task + e, od.dtype, od.vt, v);
          }
        }
      } else {
        std::vector<uint32_t> rowmap;
        for (uint32_t r = 0; r < cl.n_rows; ++r) {
          int32_t c[FX_MAXR] = {(int32_t)r, 0, 0, 0, 0, 0};
          uint32_t v = run1(cx, (int)cl.mask_begin, (int)cl.mask_end, c);
          bool keep = cl.mask_vt == FX_VT_F ? (u2f(v) != 0.0f) : (v != 0);
          if (keep) rowmap.push_back(r);
        }
        if (totals) totals[task] = (uint32_t)rowmap.size();
        for (uint32_t oi = 0; oi < cl.n_outs; ++oi) {
          const FxOut& od = outs[oi];
          void* op = (void*)ptr_of(cx, (int32_t)od.ptr_slot);
          for (size_t k = 0; k < rowmap.size(); ++k) {
            for (uint32_t col = 0; col < od.rowlen; ++col) {
              int32_t c[FX_MAXR];
              uint32_t e = col;
              for (int q = FX_MAXR - 1; q >= 1; --q) { c[q] = (int32_t)(e % od.dim[q]); e /= od.dim[q]; }
              c[0] = (int32_t)rowmap[k];
              uint32_t v = run1(cx, (int)od.prog_begin, (int)od.prog_end, c);
              store_elem(op, (int64_t)od.task_stride * task + (int64_t)k * od.rowlen + col, od.dtype, od.vt, v);
            }
          }
        }
      }
    }
  }
  return 0;
}
