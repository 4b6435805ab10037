// Generator of row-stream kernels (fx_rs.h): analysis of a compacting plan and the source of
// the kernel that serves it.
//
// The lowered programs are executed SYMBOLICALLY: registers A / B, the temporaries and the lane
// mask hold nodes of an expression graph instead of values.  The output column is a constant
// (or, in the vector form, a range over which every decision is known to fall the same way), so
// predicates of the index arithmetic (FX_MIFR and friends: "is this column the one the
// select_rev wrote?") are decided here and the branch not taken is never generated.  Nodes are
// hash-consed: the graph of a row holds every load and every sub-expression once, whichever
// columns use it.  A predicate that depends on data or on the row stays in the graph as a
// select, exactly as the lane mask of the interpreter treats it.
//
// Plays the part of the reference's statement-level code generator
// (fait/tensorexpr/cuda_codegen_tssa.cpp:881-1121 Initialize, :641-847 CudaPrinterTssa) together
// with its common-subexpression pass (fait/tensorexpr/elim_common_subexpr.cpp).
#include <algorithm>
#include <array>
#include <cstdio>
#include <cstring>
#include <map>
#include <set>
#include <mutex>
#include <sstream>
#include <unordered_map>

#include "fx_lower.h"

namespace fx {

namespace {

struct Hasher {
  uint64_t h = 1469598103934665603ull;
  void mix(uint64_t v) {
    for (int i = 0; i < 8; ++i) {
      h ^= (v >> (8 * i)) & 0xffu;
      h *= 1099511628211ull;
    }
  }
};

struct Unsupported {
  std::string why;
};

enum NodeKind : int {
  K_CONST = 1,   // i0: 32 bits
  K_FIMM,        // i0: class of the floating-point constant (value at run time)
  K_SCAL,        // i0: scalar slot, i1: convert int -> float
  K_AFF,         // value of an affine record: i0 + i1 * row + i2 * t
  K_LOAD,        // i0: input, i1: dtype | cvt << 8, element offset i2 + i3 * row + i4 * t
  K_LOADG,       // K_LOAD under a mask (a0): a dead element reads element 0
  K_LOADX,       // a0: element index, i0: input, i1: dtype, i2: constant added to the index
  K_UN,          // op(a0)
  K_BIN,         // op(a0, a1)
  K_SEL,         // a0 (bool) ? a1 : a2
  K_IRANGE,      // a0 in [i0, i1) with step i2 -> 0 / 1
  K_B2I,         // bool a0 -> 0 / 1
  // bool-valued
  K_NZ,          // a0 != 0
  K_INR,         // 0 <= a0 < i0 and a0 % i1 == 0
  K_BAND,        // a0 && a1
  K_BNOT,        // !a0
};
const int M_TRUE = -1, M_FALSE = -2, NONE = -3;

struct Node {
  int kind = 0;
  int op = 0;
  int a[3] = {NONE, NONE, NONE};
  int64_t i[5] = {0, 0, 0, 0, 0};
};

bool isBool(int kind) { return kind >= K_NZ; }

// One expression graph (a row's unrolled columns, a vector segment, or the mask).
struct Graph {
  std::vector<Node> nodes;
  std::map<std::array<int64_t, 10>, int> index;
  int add(const Node& n) {
    std::array<int64_t, 10> k = {n.kind, n.op, n.a[0], n.a[1], n.a[2], n.i[0], n.i[1], n.i[2], n.i[3], n.i[4]};
    auto it = index.find(k);
    if (it != index.end()) return it->second;
    nodes.push_back(n);
    index[k] = (int)nodes.size() - 1;
    return (int)nodes.size() - 1;
  }
  int cst(uint32_t bits) {
    Node n;
    n.kind = K_CONST;
    n.i[0] = bits;
    return add(n);
  }
  bool isConst(int id, uint32_t* v) const {
    if (id < 0 || nodes[id].kind != K_CONST) return false;
    *v = (uint32_t)nodes[id].i[0];
    return true;
  }
};

struct OutDesc {
  uint32_t rank, rowlen, dtype, vt;
  uint32_t dim[FX_MAXR];
  uint32_t prog_begin, prog_end;
};

// A run of columns of one output.  vec: evaluated in the vector form (column col0 + t for t in
// [0, len), which walks the last coordinate); else one column.
struct Segment {
  int out = 0;
  uint32_t col0 = 0, len = 1;
  bool vec = false;
  int32_t c[FX_MAXR] = {0, 0, 0, 0, 0, 0};   // coordinates of the first column (c[0] unused)
  int result = -1;                            // node of the value (in the graph it belongs to)
};

struct Model {
  const FxInsn* ins = nullptr;
  const FxAffine* aff = nullptr;
  uint32_t n_aff = 0;
  FxRsInfo info;
  std::map<int32_t, int> input_of;            // pointer slot -> input index
  std::set<int> tcoef_seen;
  // what the loads that are really executed (for some column) read of each pointer slot
  struct LoadStat { bool bad = false; int64_t S = 0; std::set<int64_t> used; };
  std::map<int32_t, LoadStat> stats;
  bool collecting = false;
  std::map<uint32_t, int> fimm_of;            // float bits -> class
  std::vector<OutDesc> outs;
  uint32_t mask_begin = 0, mask_end = 0, mask_vt = 0;
  int win_slot = -1;
  Graph g_mask, g_row;
  int mask_result = -1;
  std::vector<Segment> row_cols;              // unrolled columns, all in g_row
  std::vector<Segment> vec_segs;              // vector segments, each with its own graph
  std::vector<Graph> g_vec;
  Hasher key;

  int fimmClass(uint32_t bits) {
    auto it = fimm_of.find(bits);
    if (it != fimm_of.end()) return it->second;
    const int k = (int)fimm_of.size();
    if (k >= (int)FX_RS_MAX_FIMM) throw Unsupported{"more than " + std::to_string(FX_RS_MAX_FIMM) + " distinct floating-point constants"};
    fimm_of[bits] = k;
    info.fimm[k] = bits;
    info.n_fimm = (uint32_t)k + 1;
    return k;
  }
  int inputOf(int32_t slot) {
    auto it = input_of.find(slot);
    if (it != input_of.end()) return it->second;
    const int k = (int)input_of.size();
    if (k >= (int)FX_RS_MAX_IN) throw Unsupported{"more than " + std::to_string(FX_RS_MAX_IN) + " input buffers"};
    input_of[slot] = k;
    info.in_slot[k] = (uint32_t)slot;
    info.n_in = (uint32_t)k + 1;
    return k;
  }
};

bool isFloatImmOp(uint32_t op) { return (op >= FX_FADD && op <= FX_ATAN2) || (op >= FX_FLT && op <= FX_FNE); }
bool isAffineLoad(const FxInsn& in) { return in.op == FX_LDA || ((in.flags & FX_F_MEMB) && !(in.flags & FX_F_TMPB)); }

// ---- symbolic execution of one program ------------------------------------------------
struct Exec {
  Model& m;
  Graph& g;
  bool vec = false;        // the last coordinate walks: column = first column + t, t in [0, len)
  int vec_dim = -1;
  uint32_t len = 1;
  int32_t c[FX_MAXR] = {0, 0, 0, 0, 0, 0};   // coordinates of the (first) column
  std::vector<uint32_t>* trace = nullptr;   // decisions of the predicates that are decided here, in order

  int A = 0, B = 0, M = M_TRUE;
  int temps[FX_MAX_TEMPS];
  std::vector<int> stack;

  Exec(Model& m_, Graph& g_) : m(m_), g(g_) {}

  // the parts of an affine record at the current coordinates
  struct Aff { int64_t cst; int32_t c0, cl, tcoef; };
  Aff affOf(int32_t idx) {
    if (idx < 0 || (uint32_t)idx >= m.n_aff) throw Unsupported{"affine record out of range"};
    const FxAffine& a = m.aff[idx];
    if (a.rcoef[0] != 0 || a.rcoef[1] != 0) throw Unsupported{"index arithmetic on a reduction counter"};
    Aff r;
    r.cst = a.base;
    r.cl = 0;
    for (int k = 1; k < FX_MAXR; ++k) {
      r.cst += (int64_t)fx_aff_coef(&a, k) * c[k];
      if (vec && k == vec_dim) r.cl = fx_aff_coef(&a, k);
    }
    r.c0 = fx_aff_coef(&a, 0);
    r.tcoef = a.tcoef;
    return r;
  }
  int affNode(int32_t idx) {
    const Aff a = affOf(idx);
    if (a.tcoef != 0) throw Unsupported{"index arithmetic on the task index outside a load"};
    if (a.c0 == 0 && a.cl == 0) return g.cst((uint32_t)(int32_t)a.cst);
    Node n;
    n.kind = K_AFF;
    n.i[0] = a.cst;
    n.i[1] = a.c0;
    n.i[2] = a.cl;
    return g.add(n);
  }
  int loadNode(const FxInsn& in) {
    const Aff a = affOf(in.b);
    if (m.collecting) {
      // can the rows of this input be staged?  32-bit elements as they are, one row length, every
      // element inside its row
      Model::LoadStat& st = m.stats[in.a];
      const int64_t last = a.cst + (int64_t)a.cl * ((int64_t)len - 1);
      const int64_t lo = std::min(a.cst, last), hi = std::max(a.cst, last);
      if ((in.dt != FX_F32 && in.dt != FX_I32) || (in.flags & FX_F_I2F) || a.c0 <= 0 || lo < 0 || hi >= a.c0) st.bad = true;
      else if (st.S == 0) st.S = a.c0;
      else if (st.S != a.c0) st.bad = true;
      if (!st.bad && a.tcoef != 0 && a.tcoef < a.c0) st.bad = true;   // tasks that walk along the row: each reads a column
      if (!st.bad)
        for (int64_t x = lo; x <= hi; ++x) st.used.insert(x);
    }
    const int k = m.inputOf(in.a);
    // per-task offset: one per input
    if (!m.tcoef_seen.count(k)) {
      m.tcoef_seen.insert(k);
      m.info.in_tcoef[k] = a.tcoef;
    } else if (m.info.in_tcoef[k] != a.tcoef) {
      throw Unsupported{"an input is read at two different per-task offsets"};
    }
    Node n;
    n.kind = K_LOAD;
    n.i[0] = k;
    n.i[1] = (int64_t)in.dt | (((in.flags & FX_F_I2F) ? 1 : 0) << 8);
    n.i[2] = a.cst;
    n.i[3] = a.c0;
    n.i[4] = a.cl;
    if (M >= 0) {   // a mask that is not decided here: the dead element reads element 0
      n.kind = K_LOADG;
      n.a[0] = M;
    }
    return g.add(n);
  }

  int sel(int cond, int x, int y) {
    if (cond == M_TRUE) return x;
    if (cond == M_FALSE) return y;
    if (x == y) return x;
    Node n;
    n.kind = K_SEL;
    n.a[0] = cond;
    n.a[1] = x;
    n.a[2] = y;
    return g.add(n);
  }
  int band(int x, int y) {
    if (x == M_FALSE || y == M_FALSE) return M_FALSE;
    if (x == M_TRUE) return y;
    if (y == M_TRUE) return x;
    if (x == y) return x;
    Node n;
    n.kind = K_BAND;
    n.a[0] = x;
    n.a[1] = y;
    return g.add(n);
  }
  int bnot(int x) {
    if (x == M_TRUE) return M_FALSE;
    if (x == M_FALSE) return M_TRUE;
    Node n;
    n.kind = K_BNOT;
    n.a[0] = x;
    return g.add(n);
  }
  int nz(int x) {
    uint32_t v;
    if (g.isConst(x, &v)) return v != 0 ? M_TRUE : M_FALSE;
    if (g.nodes[x].kind == K_B2I) return g.nodes[x].a[0];
    Node n;
    n.kind = K_NZ;
    n.a[0] = x;
    return g.add(n);
  }
  int b2i(int b) {
    if (b == M_TRUE) return g.cst(1);
    if (b == M_FALSE) return g.cst(0);
    Node n;
    n.kind = K_B2I;
    n.a[0] = b;
    return g.add(n);
  }
  // 0 <= x < hi and x % st == 0 for the value of affine record idx: decided here when it does
  // not depend on the row
  int inRange(int32_t idx, uint32_t hi, int32_t st) {
    const Aff a = affOf(idx);
    if (a.tcoef != 0) throw Unsupported{"a predicate on the task index"};
    if (a.c0 == 0) {
      if (a.cl == 0) {
        const int64_t x = a.cst;
        return (x >= 0 && x < (int64_t)hi && (st <= 1 || x % st == 0)) ? M_TRUE : M_FALSE;
      }
      const int64_t x0 = a.cst, x1 = a.cst + (int64_t)a.cl * ((int64_t)len - 1);
      const int64_t lo = std::min(x0, x1), up = std::max(x0, x1);
      if (up < 0 || lo >= (int64_t)hi) return M_FALSE;
      if (lo >= 0 && up < (int64_t)hi && st <= 1) return M_TRUE;
      throw Unsupported{"a predicate changes inside a vector segment"};
    }
    Node n;
    n.kind = K_INR;
    n.a[0] = affNode(idx);
    n.i[0] = hi;
    n.i[1] = st;
    return g.add(n);
  }
  int un(uint32_t op, int x) {
    Node n;
    n.kind = K_UN;
    n.op = (int)op;
    n.a[0] = x;
    return g.add(n);
  }
  int bin(uint32_t op, int x, int y) {
    uint32_t vx, vy;
    if (op >= FX_IADD && op <= FX_IXOR && g.isConst(x, &vx) && g.isConst(y, &vy)) {
      const int32_t a = (int32_t)vx, b = (int32_t)vy;
      switch (op) {
        case FX_IADD: return g.cst((uint32_t)(a + b));
        case FX_ISUB: return g.cst((uint32_t)(a - b));
        case FX_IRSUB: return g.cst((uint32_t)(b - a));
        case FX_IMUL: return g.cst((uint32_t)(a * b));
        case FX_IAND: return g.cst((uint32_t)(a & b));
        case FX_IOR: return g.cst((uint32_t)(a | b));
        case FX_IXOR: return g.cst((uint32_t)(a ^ b));
        default: break;
      }
    }
    if (op >= FX_ILT && op <= FX_INE && g.isConst(x, &vx) && g.isConst(y, &vy)) {
      const int32_t a = (int32_t)vx, b = (int32_t)vy;
      bool r = false;
      switch (op) {
        case FX_ILT: r = a < b; break;
        case FX_ILE: r = a <= b; break;
        case FX_IGT: r = a > b; break;
        case FX_IGE: r = a >= b; break;
        case FX_IEQ: r = a == b; break;
        default: r = a != b; break;
      }
      return g.cst(r ? 1u : 0u);
    }
    Node n;
    n.kind = K_BIN;
    n.op = (int)op;
    n.a[0] = x;
    n.a[1] = y;
    return g.add(n);
  }

  void decide(uint32_t pc, bool taken) {
    if (trace) trace->push_back((pc << 1) | (taken ? 1u : 0u));
  }
  int temp(int32_t k) const {
    if (k < 0 || k >= FX_MAX_TEMPS) throw Unsupported{"temporary out of range"};
    return temps[k];
  }

  int run(uint32_t pb, uint32_t pe) {
    A = B = g.cst(0);
    for (int& t : temps) t = A;
    M = M_TRUE;
    stack.clear();
    uint32_t pc = pb;
    long guard = 0;
    while (pc < pe) {
      if (++guard > 100000) throw Unsupported{"program does not end"};
      const uint32_t at = pc;
      const FxInsn in = m.ins[pc++];
      const bool useimm = (in.flags & FX_F_IMM) != 0;
      switch (in.op) {
        case FX_MIF: {
          stack.push_back(M);
          M = band(M, nz(A));
          if (M == M_FALSE) { decide(at, false); pc = (uint32_t)in.a; } else if (M == M_TRUE) decide(at, true);
          continue;
        }
        case FX_MIFR: {
          const int p = inRange(in.b, in.imm >> 8, (int32_t)(in.imm & 255u));
          A = b2i(p);
          stack.push_back(M);
          M = band(M, p);
          if (M == M_FALSE) { decide(at, false); pc = (uint32_t)in.a; } else if (M == M_TRUE) decide(at, true);
          continue;
        }
        case FX_MELSE: {
          if (stack.empty()) throw Unsupported{"malformed predicated region"};
          M = band(stack.back(), bnot(M));
          if (M == M_FALSE) { decide(at, false); pc = (uint32_t)in.a; } else if (M == M_TRUE) decide(at, true);
          continue;
        }
        case FX_RBEGIN: case FX_RNEXT: case FX_RIDX:
          throw Unsupported{"a reduction loop"};
        case FX_WMAX: case FX_WSUM:
          throw Unsupported{"a reduction across the wave"};
        default: break;
      }
      // second operand fetched as part of the instruction
      if (in.flags & FX_F_TMPB) B = temp(in.a);
      else if ((in.flags & FX_F_MEMB) && M != M_FALSE) B = loadNode(in);
      int X = B;   // second operand of a binary operation
      if (useimm) {
        if (isFloatImmOp(in.op)) {
          Node n;
          n.kind = K_FIMM;
          n.i[0] = m.fimmClass(in.imm);
          X = g.add(n);
        } else {
          X = g.cst(in.imm);
        }
      }
      switch (in.op) {
        case FX_NOP: case FX_LDB: case FX_LDTB: break;
        case FX_LDA:
          if (M != M_FALSE) A = loadNode(in);
          break;
        case FX_AFFA: case FX_AFFB: {
          if (M == M_FALSE) break;
          int v = affNode(in.b);
          if (in.flags & FX_F_I2F) v = un(FX_I2F, v);
          if (in.op == FX_AFFA) A = sel(M, v, A); else B = sel(M, v, B);
        } break;
        case FX_LDXA: {
          if (M == M_FALSE) break;
          if (m.collecting) m.stats[in.a].bad = true;   // a load through a computed index stays in memory
          Node n;
          n.kind = K_LOADX;
          // a dead element reads element 0
          n.a[0] = M >= 0 ? sel(M, A, g.cst((uint32_t)(-(int32_t)in.imm))) : A;
          n.i[0] = m.inputOf(in.a);
          n.i[1] = in.dt;
          n.i[2] = (int32_t)in.imm;
          A = g.add(n);
        } break;
        case FX_IMMA: A = sel(M, g.cst(in.imm), A); break;
        case FX_IMMB: B = g.cst(in.imm); break;
        case FX_SCLA: case FX_SCLB: {
          Node n;
          n.kind = K_SCAL;
          n.i[0] = in.a;
          n.i[1] = (in.flags & FX_F_I2F) ? 1 : 0;
          const int v = g.add(n);
          if (in.op == FX_SCLA) A = sel(M, v, A); else B = v;
        } break;
        case FX_STT:
          temp(in.a);
          temps[in.a] = A;
          break;
        case FX_LDTA: A = sel(M, temp(in.a), A); break;
        case FX_MOVBA: B = A; break;
        case FX_SWAP: std::swap(A, B); break;
        case FX_MMERGE:
          if (stack.empty()) throw Unsupported{"malformed predicated region"};
          A = sel(M, A, temp(in.a));
          M = stack.back();
          stack.pop_back();
          break;
        case FX_MEND:
          if (stack.empty()) throw Unsupported{"malformed predicated region"};
          M = stack.back();
          stack.pop_back();
          break;
        case FX_IRANGE: {
          uint32_t v;
          if (g.isConst(A, &v)) {
            const int32_t a = (int32_t)v, st = (int32_t)in.imm;
            bool inr = a >= in.a && a < in.b;
            if (st > 1) inr = inr && ((a - in.a) % st == 0);
            A = g.cst(inr ? 1u : 0u);
          } else if (g.nodes[A].kind == K_AFF && g.nodes[A].i[1] == 0) {
            // a value that walks with the column only: decided for the whole segment, or the
            // segment is not one
            const int64_t x0 = g.nodes[A].i[0], x1 = x0 + g.nodes[A].i[2] * ((int64_t)len - 1);
            const int64_t lo = std::min(x0, x1), up = std::max(x0, x1);
            if (up < in.a || lo >= in.b) A = g.cst(0);
            else if (lo >= in.a && up < in.b && (int32_t)in.imm <= 1) A = g.cst(1);
            else throw Unsupported{"a predicate changes inside a vector segment"};
          } else {
            Node n;
            n.kind = K_IRANGE;
            n.a[0] = A;
            n.i[0] = in.a;
            n.i[1] = in.b;
            n.i[2] = (int32_t)in.imm;
            A = g.add(n);
          }
        } break;
        case FX_WHERE: A = sel(nz(temp(in.a)), A, B); break;
        default:
          if ((in.op >= FX_FNEG && in.op <= FX_LOG1P) || (in.op >= FX_INEG && in.op <= FX_IABS)) A = un(in.op, A);
          else if (fx_op_is_binary(in.op)) A = bin(in.op, A, X);
          else throw Unsupported{"instruction " + std::string(opname(in.op)) + " has no row-stream form"};
          break;
      }
    }
    return A;
  }
};

// ---- the key: what the generated code holds as constants -------------------------------
// Everything of the programs but the VALUES of floating-point immediates (their classes enter:
// which of them are equal), the numbering of the pointer slots (order of first use enters) and
// the per-task coefficients of loads.
void keyProgram(Model& m, uint32_t pb, uint32_t pe) {
  m.key.mix(0xC0DEull);
  m.key.mix(pe - pb);
  for (uint32_t pc = pb; pc < pe; ++pc) {
    const FxInsn& x = m.ins[pc];
    m.key.mix(x.op);
    m.key.mix(x.flags);
    m.key.mix(x.dt);
    if (isAffineLoad(x) || x.op == FX_LDXA) {
      m.key.mix((uint64_t)m.inputOf(x.a));
      m.key.mix((uint64_t)(uint32_t)x.b);
    } else if (x.op == FX_MIF || x.op == FX_MIFR || x.op == FX_MELSE) {
      m.key.mix((uint64_t)(uint32_t)(x.a - (int32_t)pb));
      m.key.mix((uint64_t)(uint32_t)x.b);
    } else {
      m.key.mix((uint64_t)(uint32_t)x.a);
      m.key.mix((uint64_t)(uint32_t)x.b);
    }
    if ((x.flags & FX_F_IMM) && isFloatImmOp(x.op)) m.key.mix(0xF1000000ull | (uint64_t)m.fimmClass(x.imm));
    else m.key.mix(x.imm);
  }
}

void coordsOf(const OutDesc& od, uint32_t col, int32_t* c) {
  uint32_t e = col;
  for (int q = FX_MAXR - 1; q >= 1; --q) {
    c[q] = (int32_t)(e % od.dim[q]);
    e /= od.dim[q];
  }
  c[0] = 0;
}

bool buildModel(const Plan& P, Model& m) {
  FxRsInfo& info = m.info;
  try {
    const uint32_t* sb = P.blob.data();
    if (P.blob.size() < sizeof(FxHeader) / 4) throw Unsupported{"no descriptor"};
    const FxHeader* h = (const FxHeader*)sb;
    if (h->mode != FX_MODE_COMPACT) throw Unsupported{"not a row compaction"};
    if (h->n_classes != 1) throw Unsupported{"tasks with different programs"};
    const FxClass& cl = *(const FxClass*)(sb + h->off_class);
    if (cl.n_tasks != h->n_tasks || cl.n_rows == 0) throw Unsupported{"no rows"};
    const uint32_t* taskmap = sb + h->off_taskmap;
    for (uint32_t t = 0; t < cl.n_tasks; ++t)
      if (taskmap[cl.first_task + t] != t) throw Unsupported{"tasks out of order"};
    if (cl.n_outs == 0 || cl.n_outs > FX_RS_MAX_OUT) throw Unsupported{"more than " + std::to_string(FX_RS_MAX_OUT) + " outputs"};
    m.ins = (const FxInsn*)(sb + cl.off_insn);
    m.aff = (const FxAffine*)(sb + cl.off_aff);
    m.n_aff = (cl.off_outs - cl.off_aff) / FX_AFF_WORDS;
    const FxOut* outs = (const FxOut*)(sb + cl.off_outs);
    m.mask_begin = cl.mask_begin;
    m.mask_end = cl.mask_end;
    m.mask_vt = cl.mask_vt;
    info.n_rows = cl.n_rows;
    info.n_tasks = cl.n_tasks;
    info.slot_err = h->slot_err;
    info.n_out = cl.n_outs;
    for (uint32_t k = 0; k < cl.n_outs; ++k) {
      const FxOut& o = outs[k];
      OutDesc od;
      od.rank = std::max<uint32_t>(o.rank, 1u);
      od.rowlen = std::max<uint32_t>(o.rowlen, 1u);
      od.dtype = o.dtype;
      od.vt = o.vt;
      for (int q = 0; q < FX_MAXR; ++q) od.dim[q] = std::max<uint32_t>(o.dim[q], 1u);
      od.prog_begin = o.prog_begin;
      od.prog_end = o.prog_end;
      m.outs.push_back(od);
      info.out_slot[k] = o.ptr_slot;
      info.out_tstride[k] = o.task_stride;
    }

    // ---- the window input: the 32-bit row-major input with the longest rows whose loads all stay
    // inside their row.  What counts are the loads that are executed for some column (a load
    // behind a column predicate is not executed for the other columns): a first run of every
    // program, column by column, collects them.
    {
      m.collecting = true;
      Graph scratch;
      {
        Exec ex(m, scratch);
        ex.run(m.mask_begin, m.mask_end);
      }
      for (const OutDesc& od : m.outs)
        for (uint32_t col = 0; col < od.rowlen; ++col) {
          Exec ex(m, scratch);
          coordsOf(od, col, ex.c);
          ex.run(od.prog_begin, od.prog_end);
        }
      m.collecting = false;
      for (auto& kv : m.stats)
        if (!kv.second.bad && kv.second.S > 0 && (m.win_slot < 0 || kv.second.S > m.stats[m.win_slot].S)) m.win_slot = kv.first;
      if (m.win_slot < 0) throw Unsupported{"no row-major 32-bit input that is read row by row"};
      info.S = (uint32_t)m.stats[m.win_slot].S;
      // streaming whole rows pays when most of a row is used
      if (2 * (int64_t)m.stats[m.win_slot].used.size() < (int64_t)info.S) throw Unsupported{"less than half of every row of the widest input is read"};
      // a sub-tile of at least 8 rows in what FX_RS_KV 128-bit loads per lane carry
      if ((FX_RS_KV * FX_BLOCK * 4u - 6u) / info.S < 8u) throw Unsupported{"rows of the window input too long for a sub-tile"};
      // the numbering of inputs and constants starts over: the key pass below fixes it
      m.input_of.clear();
      m.tcoef_seen.clear();
      m.fimm_of.clear();
      info.n_in = 0;
      info.n_fimm = 0;
      for (uint32_t k = 0; k < FX_RS_MAX_IN; ++k) { info.in_slot[k] = 0; info.in_tcoef[k] = 0; }
    }

    m.key.mix(FX_RS_VERSION);
    m.key.mix(info.S);
    // The affine records are constants of the generated code, all but the per-task coefficient of
    // the records that only loads use (an input's offset per task is a run-time value).
    {
      std::vector<char> in_arith(m.n_aff, 0);
      auto scan = [&](uint32_t pb, uint32_t pe) {
        for (uint32_t pc = pb; pc < pe; ++pc) {
          const FxInsn& x = m.ins[pc];
          if ((x.op == FX_AFFA || x.op == FX_AFFB || x.op == FX_MIFR) && (uint32_t)x.b < m.n_aff) in_arith[x.b] = 1;
        }
      };
      scan(m.mask_begin, m.mask_end);
      for (const OutDesc& od : m.outs) scan(od.prog_begin, od.prog_end);
      for (uint32_t i = 0; i < m.n_aff; ++i) {
        const FxAffine& a = m.aff[i];
        for (int k = 0; k < FX_MAXR; ++k) m.key.mix((uint64_t)(uint32_t)fx_aff_coef(&a, k));
        m.key.mix((uint64_t)(uint32_t)a.base);
        m.key.mix((uint64_t)(uint32_t)a.rcoef[0]);
        m.key.mix((uint64_t)(uint32_t)a.rcoef[1]);
        m.key.mix((in_arith[i] && a.tcoef != 0) ? 1u : 0u);
      }
    }
    m.inputOf(m.win_slot);   // the window is input 0
    keyProgram(m, m.mask_begin, m.mask_end);
    m.key.mix(m.mask_vt);
    for (const OutDesc& od : m.outs) {
      m.key.mix(0xBBull);
      m.key.mix(od.rank);
      m.key.mix(od.rowlen);
      m.key.mix(od.dtype);
      m.key.mix(od.vt);
      for (int q = 1; q < FX_MAXR; ++q) m.key.mix(od.dim[q]);
      keyProgram(m, od.prog_begin, od.prog_end);
      if (od.dtype == FX_F16) throw Unsupported{"a float16 output"};
    }

    // ---- mask
    {
      Exec ex(m, m.g_mask);
      m.mask_result = ex.run(m.mask_begin, m.mask_end);
    }

    // ---- outputs: a trace per column, runs of alike columns, then the graphs
    uint32_t n_unrolled = 0;
    for (size_t oi = 0; oi < m.outs.size(); ++oi) {
      const OutDesc& od = m.outs[oi];
      const int last = (int)od.rank - 1;
      std::vector<std::vector<uint32_t>> traces(od.rowlen);
      {
        Graph scratch;
        for (uint32_t col = 0; col < od.rowlen; ++col) {
          Exec ex(m, scratch);
          coordsOf(od, col, ex.c);
          ex.trace = &traces[col];
          ex.run(od.prog_begin, od.prog_end);
        }
      }
      uint32_t col = 0;
      while (col < od.rowlen) {
        // the run of columns from here with the same decisions, inside one run of the last dimension
        uint32_t end = col + 1;
        if (last >= 1) {
          const uint32_t inner = od.dim[last];
          const uint32_t run_end = (col / inner + 1) * inner;
          while (end < run_end && end < od.rowlen && traces[end] == traces[col]) ++end;
        }
        bool as_vec = end - col >= FX_RS_VEC_MIN;
        if (as_vec) {
          Segment sg;
          sg.out = (int)oi;
          sg.col0 = col;
          sg.len = end - col;
          sg.vec = true;
          coordsOf(od, col, sg.c);
          Graph gv;
          try {
            Exec ex(m, gv);
            memcpy(ex.c, sg.c, sizeof(sg.c));
            ex.vec = true;
            ex.vec_dim = last;
            ex.len = sg.len;
            sg.result = ex.run(od.prog_begin, od.prog_end);
            m.g_vec.push_back(std::move(gv));
            m.vec_segs.push_back(sg);
          } catch (const Unsupported&) {
            as_vec = false;
          }
        }
        if (!as_vec) {
          for (uint32_t cc = col; cc < end; ++cc) {
            Segment s1;
            s1.out = (int)oi;
            s1.col0 = cc;
            coordsOf(od, cc, s1.c);
            Exec ex(m, m.g_row);
            memcpy(ex.c, s1.c, sizeof(s1.c));
            s1.result = ex.run(od.prog_begin, od.prog_end);
            m.row_cols.push_back(s1);
            if (++n_unrolled > FX_RS_MAX_UNROLL) throw Unsupported{"more than " + std::to_string(FX_RS_MAX_UNROLL) + " columns that need code of their own"};
          }
        }
        col = end;
      }
    }
    m.key.mix(info.n_in);
    m.key.mix(info.n_fimm);
    info.key = m.key.h ? m.key.h : 1;
    info.ok = true;
  } catch (const Unsupported& u) {
    info.ok = false;
    info.why = u.why;
  }
  return info.ok;
}

// ---- emission -------------------------------------------------------------------------------
const char* dtName(uint32_t dt) {
  static const char* n[] = {"FX_F32", "FX_I64", "FX_I32", "FX_U8", "FX_F16", "FX_BF16", "FX_I64LO", "FX_I64HI"};
  return dt < 8 ? n[dt] : "FX_F32";
}

struct Emitter {
  const Model& m;
  const Graph& g;
  bool window;            // loads of input 0 read the staged row (W) instead of memory
  std::ostringstream* out;   // where the code goes (emitSide and emitAll of one emitter may write to different places)
  const char* ind;
  std::vector<char> done;
  // Loads from memory whose address depends on the row only, in the order in which emitSide
  // issues them: a row's code in two parts, the loads (which can leave ahead of everything
  // else the wave asks for) and the rest, which finds their values in sd.s[].
  std::vector<int> side;
  Emitter(const Model& m_, const Graph& g_, bool window_, std::ostringstream& o_, const char* ind_)
      : m(m_), g(g_), window(window_), out(&o_), ind(ind_), done(g_.nodes.size(), 0) {}

  std::string ref(int id) const {
    if (id == M_TRUE) return "true";
    if (id == M_FALSE) return "false";
    const Node& n = g.nodes[id];
    char buf[64];
    if (n.kind == K_CONST) { snprintf(buf, sizeof buf, "0x%xu", (uint32_t)n.i[0]); return buf; }
    if (n.kind == K_FIMM) { snprintf(buf, sizeof buf, "rt.fimm(%d)", (int)n.i[0]); return buf; }
    snprintf(buf, sizeof buf, "%c%d", isBool(n.kind) ? 'b' : 'v', id);
    return buf;
  }
  static std::string lin(int64_t cst, int64_t c0, int64_t cl) {
    std::ostringstream s;
    s << "(uint32_t)(" << cst;
    if (c0) s << " + " << c0 << " * (int32_t)row";
    if (cl) s << " + " << cl << " * (int32_t)t";
    s << ")";
    return s.str();
  }
  bool fromWindow(const Node& n) const { return window && (n.kind == K_LOAD || n.kind == K_LOADG) && n.i[0] == 0; }
  std::string loadOff(const Node& n) const {
    // element offset inside the input: the per-task offset of the input is added by rs_ld
    return lin(n.i[2], n.i[3], n.i[4]);
  }
  std::string winOff(const Node& n) const {
    std::ostringstream s;
    s << n.i[2];
    if (n.i[4]) s << " + " << n.i[4] << " * (int32_t)t";
    return s.str();
  }

  void collect(int id, std::vector<char>& seen, std::vector<int>& order) const {
    if (id < 0 || seen[id]) return;
    seen[id] = 1;
    const Node& n = g.nodes[id];
    for (int k = 0; k < 3; ++k) collect(n.a[k], seen, order);
    order.push_back(id);
  }

  void emitNode(int id) {
    if (id < 0 || done[id]) return;
    done[id] = 1;
    const Node& n = g.nodes[id];
    if (n.kind == K_CONST || n.kind == K_FIMM) return;
    const std::string me = ref(id);
    const char* ty = isBool(n.kind) ? "const bool " : "const uint32_t ";
    (*out) << ind << ty << me << " = ";
    switch (n.kind) {
      case K_SCAL: (*out) << "rs_scal<" << n.i[1] << ">(rt, " << n.i[0] << ")"; break;
      case K_AFF: (*out) << lin(n.i[0], n.i[1], n.i[2]); break;
      case K_LOAD:
      case K_LOADG: {
        const uint32_t dt = (uint32_t)(n.i[1] & 0xff);
        const int cvt = (int)(n.i[1] >> 8);
        if (fromWindow(n)) {
          if (n.kind == K_LOADG) (*out) << "W[" << ref(n.a[0]) << " ? (" << winOff(n) << ") : 0]";
          else (*out) << "W[" << winOff(n) << "]";
        } else {
          (*out) << "rs_ld<" << dtName(dt) << ", " << cvt << ">(rt, " << n.i[0] << ", ";
          if (n.kind == K_LOADG) (*out) << ref(n.a[0]) << " ? " << loadOff(n) << " : 0u";
          else (*out) << loadOff(n);
          (*out) << ")";
        }
      } break;
      case K_LOADX:
        (*out) << "rs_ldx<" << dtName((uint32_t)n.i[1]) << ">(rt, " << n.i[0] << ", (uint32_t)((int32_t)" << ref(n.a[0]) << " + " << n.i[2] << "))";
        break;
      case K_UN: (*out) << "rs_" << opname((uint32_t)n.op) << "(" << ref(n.a[0]) << ")"; break;
      case K_BIN: (*out) << "rs_" << opname((uint32_t)n.op) << "(" << ref(n.a[0]) << ", " << ref(n.a[1]) << ")"; break;
      case K_SEL: (*out) << "rs_SEL(" << ref(n.a[0]) << ", " << ref(n.a[1]) << ", " << ref(n.a[2]) << ")"; break;
      case K_IRANGE: (*out) << "rs_IRANGE(" << ref(n.a[0]) << ", " << n.i[0] << ", " << n.i[1] << ", " << n.i[2] << ")"; break;
      case K_B2I: (*out) << "(" << ref(n.a[0]) << " ? 1u : 0u)"; break;
      case K_NZ: (*out) << "(" << ref(n.a[0]) << " != 0u)"; break;
      case K_INR: (*out) << "rs_INR(" << ref(n.a[0]) << ", " << n.i[0] << "u, " << n.i[1] << ")"; break;
      case K_BAND: (*out) << "(" << ref(n.a[0]) << " && " << ref(n.a[1]) << ")"; break;
      case K_BNOT: (*out) << "!" << ref(n.a[0]); break;
      default: (*out) << "0u"; break;
    }
    (*out) << ";\n";
  }

  // The unconditional loads from memory that `roots` need (merged where they are neighbours), each
  // into its slot of sd.s[]; returns the number of slots.  emitAll(roots, ...) of the SAME emitter
  // afterwards takes their values from there.
  size_t emitSide(const std::vector<int>& roots) {
    std::vector<char> seen(g.nodes.size(), 0);
    std::vector<int> order;
    for (int r : roots) collect(r, seen, order);
    emitLoads(order, true, /*to_side=*/true);
    return side.size();
  }

  // Everything the values in `roots` need, loads first.  Plain 32-bit loads of neighbouring
  // elements of one input (same row coefficient, no walk) become one wide load.
  void emitAll(const std::vector<int>& roots, bool merge_loads) {
    std::vector<char> seen(g.nodes.size(), 0);
    std::vector<int> order;
    for (int r : roots) collect(r, seen, order);
    if (!side.empty()) {
      for (size_t k = 0; k < side.size(); ++k) {
        (*out) << ind << "const uint32_t " << ref(side[k]) << " = sd.s[" << k << "];\n";
        done[side[k]] = 1;
      }
    }
    emitLoads(order, merge_loads, false);
    for (int id : order) emitNode(id);
  }

  void emitLoads(const std::vector<int>& order, bool merge_loads, bool to_side) {
    // loads from memory, merged
    std::vector<int> plain;
    for (int id : order) {
      const Node& n = g.nodes[id];
      if (n.kind != K_LOAD || fromWindow(n) || done[id]) continue;
      const uint32_t dt = (uint32_t)(n.i[1] & 0xff);
      if (merge_loads && (dt == FX_F32 || dt == FX_I32) && (n.i[1] >> 8) == 0 && n.i[4] == 0) plain.push_back(id);
    }
    std::sort(plain.begin(), plain.end(), [&](int x, int y) {
      const Node &a = g.nodes[x], &b = g.nodes[y];
      if (a.i[0] != b.i[0]) return a.i[0] < b.i[0];
      if (a.i[3] != b.i[3]) return a.i[3] < b.i[3];
      if (a.i[1] != b.i[1]) return a.i[1] < b.i[1];
      return a.i[2] < b.i[2];
    });
    for (size_t k = 0; k < plain.size();) {
      size_t e = k + 1;
      while (e < plain.size() && e - k < 4) {
        const Node &a = g.nodes[plain[e - 1]], &b = g.nodes[plain[e]];
        if (a.i[0] != b.i[0] || a.i[3] != b.i[3] || a.i[1] != b.i[1] || b.i[2] != a.i[2] + 1) break;
        ++e;
      }
      const size_t w = e - k >= 4 ? 4 : (e - k >= 2 ? 2 : 1);
      if (w > 1) {
        const Node& n0 = g.nodes[plain[k]];
        if (!to_side) {
          (*out) << ind << "uint32_t";
          for (size_t j = 0; j < w; ++j) (*out) << (j ? ", " : " ") << ref(plain[k + j]);
          (*out) << ";\n";
        }
        (*out) << ind << "rs_ld" << w << "(rt, " << n0.i[0] << ", " << loadOff(n0);
        for (size_t j = 0; j < w; ++j) {
          if (to_side) {
            (*out) << ", sd.s[" << side.size() << "]";
            side.push_back(plain[k + j]);
          } else {
            (*out) << ", " << ref(plain[k + j]);
          }
          done[plain[k + j]] = 1;
        }
        (*out) << ");\n";
      }
      k += w;
    }
    // the other loads whose address needs nothing computed
    for (int id : order) {
      const Node& n = g.nodes[id];
      if (n.kind != K_LOAD || done[id] || fromWindow(n)) continue;
      if (to_side) {
        if (n.i[4] != 0) continue;   // (walks along the columns: not a row's load)
        const uint32_t dt = (uint32_t)(n.i[1] & 0xff);
        (*out) << ind << "sd.s[" << side.size() << "] = rs_ld<" << dtName(dt) << ", " << (int)(n.i[1] >> 8) << ">(rt, " << n.i[0] << ", " << loadOff(n) << ");\n";
        side.push_back(id);
        done[id] = 1;
      } else {
        emitNode(id);
      }
    }
    if (to_side)   // (emitAll declares the values again from sd.s[])
      for (int id : side) done[id] = 0;
  }
};

std::string keyHex(uint64_t k) {
  char hx[32];
  snprintf(hx, sizeof hx, "%016llx", (unsigned long long)k);
  return hx;
}

bool raw32(const OutDesc& od) { return (od.dtype == FX_F32 && od.vt == FX_VT_F) || (od.dtype == FX_I32 && od.vt == FX_VT_I); }
// An output whose rows are not whole 16-byte groups is put together in LDS and leaves as one
// aligned run per sub-tile (its kept rows are consecutive in memory): stores that start at any
// 4-byte address, and single columns written with a stride of one row, cost a launch a quarter
// of its time.
bool staged(const OutDesc& od) { return raw32(od) && od.rowlen > 4 && od.rowlen % 4 != 0; }

std::string emitSource(const Model& m, const std::string& label) {
  const std::string hx = keyHex(m.info.key);
  std::ostringstream o;
  o << "// Generated by fx_plan_rowstream_source; do not edit.  Region: " << label << "\n"
    << "// The programs of this row compaction as straight-line code per row: the mask, the columns\n"
    << "// that need code of their own (all of a row in one expression graph) and the vector segments\n"
    << "// (runs of columns that execute the same instructions).  Inputs in order of first use: input 0\n"
    << "// is the window (rows of " << m.info.S << " elements, staged in LDS).\n"
    << "#include \"../fx_rs_policy.h\"\n\nnamespace {\n";
  // vector segments
  for (size_t k = 0; k < m.vec_segs.size(); ++k) {
    const Segment& sg = m.vec_segs[k];
    const OutDesc& od = m.outs[sg.out];
    o << "struct RS_" << hx << "_V" << k << " {\n"
      << "  static constexpr uint32_t out = " << sg.out << ", col0 = " << sg.col0 << ", len = " << sg.len
      << ", rowlen = " << od.rowlen << ", dtype = " << dtName(od.dtype) << ", vt = " << od.vt << ";\n"
      << "  static constexpr bool staged = " << (staged(od) ? "true" : "false") << ";\n"
      << "  template <class RT>\n"
      << "  static FX_RS_FN uint32_t elem(const RT& rt, const uint32_t* W, uint32_t row, uint32_t t) {\n";
    Emitter em(m, m.g_vec[k], true, o, "    ");
    em.emitAll({sg.result}, false);
    o << "    return " << em.ref(sg.result) << ";\n  }\n};\n";
  }
  o << "struct RS_" << hx << " {\n"
    << "  static constexpr uint64_t key = 0x" << hx << "ull;\n"
    << "  static constexpr uint32_t S = " << m.info.S << ", n_in = " << m.info.n_in << ", n_out = " << m.info.n_out
    << ", n_fimm = " << m.info.n_fimm << ";\n"
    << "  // elements per row of the outputs that are put together in LDS (0: written as they are computed)\n"
    << "  static constexpr uint32_t stage_rowlen[" << FX_RS_MAX_OUT << "] = {";
  for (uint32_t k = 0; k < FX_RS_MAX_OUT; ++k) o << (k ? ", " : "") << ((k < m.outs.size() && staged(m.outs[k])) ? m.outs[k].rowlen : 0u);
  {
    uint32_t words = 0, n = 0;
    for (const OutDesc& od : m.outs)
      if (staged(od)) { words += od.rowlen; ++n; }
    o << "};\n  static constexpr uint32_t stage_row_words = " << words << ", n_staged = " << n << ";\n";
  }
  o << "  // is the row kept?  Every load goes to memory: the mask runs ahead of the rows.\n"
    << "  template <class RT>\n"
    << "  static FX_RS_FN bool mask(const RT& rt, uint32_t row) {\n"
    << "    const uint32_t* W = nullptr; (void)W; const uint32_t t = 0; (void)t;\n";
  {
    Emitter em(m, m.g_mask, false, o, "    ");
    em.emitAll({m.mask_result}, true);
    if (m.mask_vt == FX_VT_F) o << "    return u2f(" << em.ref(m.mask_result) << ") != 0.0f;\n";
    else o << "    return " << em.ref(m.mask_result) << " != 0u;\n";
  }
  o << "  }\n"
    << "  // the columns that need code of their own, for one kept row: W is the row in the window,\n"
    << "  // row its index in the task, orow its index among the kept rows of the task, lrow among those\n"
    << "  // of the sub-tile\n"
    << "  static constexpr uint32_t n_row_cols = " << m.row_cols.size() << ";\n";
  {
    // in two parts: what a row reads from memory besides the window (side: its loads can leave
    // ahead of the next sub-tile's requests, which everything later would queue behind), and the rest
    std::ostringstream side_body;
    Emitter em(m, m.g_row, true, side_body, "    ");
    std::vector<int> roots;
    for (const Segment& s : m.row_cols) roots.push_back(s.result);
    const size_t n_side = em.emitSide(roots);
    o << "  struct Side { uint32_t s[" << std::max<size_t>(n_side, 1) << "]; };\n"
      << "  static constexpr uint32_t n_side = " << n_side << ";\n"
      << "  template <class RT>\n"
      << "  static FX_RS_FN void row_side(const RT& rt, uint32_t row, Side& sd) {\n"
      << "    (void)rt; (void)row; (void)sd;\n"
      << side_body.str() << "  }\n"
      << "  template <class RT>\n"
      << "  static FX_RS_FN void row(const RT& rt, const uint32_t* W, const Side& sd, uint32_t row, uint32_t orow, uint32_t lrow) {\n"
      << "    const uint32_t t = 0; (void)t; (void)W; (void)sd; (void)row; (void)orow; (void)lrow;\n";
    em.out = &o;
    em.emitAll(roots, true);
    // stores: four neighbouring columns of a plain 32-bit output as one 128-bit store
    for (size_t k = 0; k < m.row_cols.size();) {
      const Segment& s = m.row_cols[k];
      const OutDesc& od = m.outs[s.out];
      size_t e = k + 1;
      while (e < m.row_cols.size() && e - k < 4 && m.row_cols[e].out == s.out && m.row_cols[e].col0 == m.row_cols[e - 1].col0 + 1) ++e;
      if (staged(od)) {
        o << "    rs_stl(rt, " << s.out << ", lrow * " << od.rowlen << "u + " << s.col0 << "u, " << em.ref(s.result) << ");\n";
        ++k;
      } else if (e - k == 4 && raw32(od)) {
        o << "    rs_st4(rt, " << s.out << ", orow * " << od.rowlen << "u + " << s.col0 << "u";
        for (size_t j = k; j < e; ++j) o << ", " << em.ref(m.row_cols[j].result);
        o << ");\n";
        k = e;
      } else {
        o << "    rs_st<" << dtName(od.dtype) << ", " << od.vt << ">(rt, " << s.out << ", orow * " << od.rowlen << "u + " << s.col0
          << "u, " << em.ref(s.result) << ");\n";
        ++k;
      }
    }
  }
  o << "  }\n  using Vecs = FxRsList<";
  for (size_t k = 0; k < m.vec_segs.size(); ++k) o << (k ? ", " : "") << "RS_" << hx << "_V" << k;
  o << ">;\n};\n}  // namespace\n\nFX_RS_REGISTER(RS_" << hx << ")\n";
  return o.str();
}

}  // namespace

void rs_analyze(Plan* p) {
  Model m;
  buildModel(*p, m);
  p->rs = m.info;
}

std::string rs_source(const Plan& p, const std::string& label) {
  Model m;
  if (!buildModel(p, m)) throw Error(FX_E_UNSUPPORTED, "this plan has no row-stream form: " + m.info.why);
  return emitSource(m, label);
}

}  // namespace fx

// ---- generated kernels linked into the library: they register themselves from static
// initialisers of their translation units (spec/fx_rs_*.hip), before any plan is made ----
static std::unordered_map<uint64_t, FxRsKernel>& rs_table() {
  static std::unordered_map<uint64_t, FxRsKernel> t;
  return t;
}
static std::mutex& rs_mutex() {
  static std::mutex m;
  return m;
}
void fx_rs_register(uint64_t key, const FxRsKernel& k) {
  std::lock_guard<std::mutex> g(rs_mutex());
  rs_table()[key] = k;
}
const FxRsKernel* fx_rs_find(uint64_t key) {
  std::lock_guard<std::mutex> g(rs_mutex());
  auto it = rs_table().find(key);
  return it == rs_table().end() ? nullptr : &it->second;   // entries are never erased
}
int fx_rs_count() {
  std::lock_guard<std::mutex> g(rs_mutex());
  return (int)rs_table().size();
}
