// Region IR -> VM bytecode.  See fx_lower.h.
#include "fx_lower.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <limits>
#include <sstream>

namespace fx {

// thrown by the lowering when it meets a per-task int input in shape or index arithmetic
struct NeedIndexInt { int input; };

#define FX_CHECK(cond, code, msg)                        \
  do {                                                   \
    if (!(cond)) {                                       \
      std::ostringstream oss__;                          \
      oss__ << msg;                                      \
      throw Error(code, oss__.str());                    \
    }                                                    \
  } while (0)

int dtype_size(int dt) {
  switch (dt) {
    case FX_DT_F32: case FX_DT_I32: return 4;
    case FX_DT_I64: return 8;
    case FX_DT_U8: case FX_DT_BOOL: return 1;
    case FX_DT_F16: case FX_DT_BF16: return 2;
  }
  return 0;
}
static bool is_float_dt(int dt) { return dt == FX_DT_F32 || dt == FX_DT_F16 || dt == FX_DT_BF16; }
static uint32_t vt_of(int dt) { return is_float_dt(dt) ? FX_VT_F : FX_VT_I; }
static uint32_t storage_dt(int dt) { return dt == FX_DT_BOOL ? (uint32_t)FX_U8 : (uint32_t)dt; }
static uint32_t fbits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static int int_rank(int dt) {  // ordering for promotion among integral types
  switch (dt) { case FX_DT_BOOL: return 0; case FX_DT_U8: return 1; case FX_DT_I32: return 2; case FX_DT_I64: return 3; }
  return -1;
}
static int promote(int a, int b) {
  if (a < 0) return b;
  if (b < 0) return a;
  bool fa = is_float_dt(a), fb = is_float_dt(b);
  if (fa && fb) return a == b ? a : FX_DT_F32;
  if (fa) return a;
  if (fb) return b;
  return int_rank(a) >= int_rank(b) ? a : b;
}

// ---------------------------------------------------------------------------
// builder-side dtype inference (the role of InferDtypeAndDevice,
// fait/passes/refine_types.cpp:540, for the ops a region may contain)
// ---------------------------------------------------------------------------
int Region::addOp(int opcode, const std::vector<int>& args, int out_dtype) {
  for (int a : args) FX_CHECK(a >= 0 && a < (int)vals.size(), FX_E_INVALID, "bad value id " << a);
  auto tdt = [&](int i) -> int {
    if (i >= (int)args.size()) return -1;
    const Value& v = vals[args[i]];
    if (v.kind == VK_TENSOR) return v.dtype;
    if (v.kind == VK_TENSOR_LIST && !v.args.empty()) return vals[v.args[0]].dtype;
    return -1;
  };
  // dtype contributed by an operand of a binary op: tensors fully, scalars by category
  auto binop_dt = [&]() -> int {
    int dt = -1;
    bool any_float_scalar = false;
    for (int i = 0; i < 2 && i < (int)args.size(); ++i) {
      const Value& v = vals[args[i]];
      if (v.kind == VK_TENSOR) dt = promote(dt, v.dtype);
      else if (v.kind == VK_FLOAT) any_float_scalar = true;
    }
    if (dt < 0) dt = any_float_scalar ? FX_DT_F32 : FX_DT_I64;
    if (any_float_scalar && !is_float_dt(dt)) dt = FX_DT_F32;
    return dt;
  };
  Value v;
  v.prod = P_OP;
  v.op = opcode;
  v.args = args;
  v.kind = VK_TENSOR;
  switch (opcode) {
    case FX_OP_ACCESS: case FX_OP_CLONE: case FX_OP_SELECT: case FX_OP_SLICE: case FX_OP_SQUEEZE:
    case FX_OP_UNSQUEEZE: case FX_OP_VIEW: case FX_OP_PERMUTE: case FX_OP_TRANSPOSE: case FX_OP_EXPAND:
    case FX_OP_EXPAND_AS: case FX_OP_REPEAT: case FX_OP_INDEX: case FX_OP_TRIU: case FX_OP_TRIL: case FX_OP_CAT:
    case FX_OP_STACK: case FX_OP_SELECT_REV: case FX_OP_SLICE_REV: case FX_OP_FORALL_SELECT_REV:
    case FX_OP_NEG: case FX_OP_ABS: case FX_OP_RELU: case FX_OP_CLAMP: case FX_OP_MAX_DIM:
    case FX_OP_FLOOR: case FX_OP_CEIL: case FX_OP_ROUND:
      v.dtype = tdt(0);
      break;
    case FX_OP_ASSIGN: v.dtype = tdt(1); break;
    case FX_OP_SUM_DIM: v.dtype = is_float_dt(tdt(0)) ? tdt(0) : FX_DT_I64; break;
    case FX_OP_FULL: v.dtype = out_dtype >= 0 ? out_dtype : (tdt(0) >= 0 ? tdt(0) : FX_DT_F32); break;
    case FX_OP_ARANGE: v.dtype = out_dtype >= 0 ? out_dtype : FX_DT_I64; break;
    case FX_OP_SCALAR_TENSOR:
      v.dtype = out_dtype >= 0 ? out_dtype : (vals[args[0]].kind == VK_FLOAT ? FX_DT_F32 : FX_DT_I64);
      break;
    case FX_OP_TO:
      FX_CHECK(out_dtype >= 0, FX_E_INVALID, "FX_OP_TO needs an explicit dtype");
      v.dtype = out_dtype;
      break;
    case FX_OP_EXP: case FX_OP_LOG: case FX_OP_SQRT: case FX_OP_RSQRT: case FX_OP_SIGMOID: case FX_OP_TANH:
    case FX_OP_SIN: case FX_OP_COS: case FX_OP_ERF: case FX_OP_RECIPROCAL: case FX_OP_SOFTMAX:
      v.dtype = is_float_dt(tdt(0)) ? tdt(0) : FX_DT_F32;
      break;
    case FX_OP_LOGICAL_NOT: case FX_OP_EQ: case FX_OP_NE: case FX_OP_LT: case FX_OP_LE: case FX_OP_GT:
    case FX_OP_GE:
      v.dtype = FX_DT_BOOL;
      break;
    case FX_OP_ADD: case FX_OP_SUB: case FX_OP_RSUB: case FX_OP_MUL: case FX_OP_MAXIMUM: case FX_OP_MINIMUM:
    case FX_OP_POW: case FX_OP_FMOD: case FX_OP_AND: case FX_OP_OR: case FX_OP_XOR:
      v.dtype = binop_dt();
      break;
    case FX_OP_DIV: {
      int dt = binop_dt();
      v.dtype = is_float_dt(dt) ? dt : FX_DT_F32;
    } break;
    case FX_OP_WHERE: v.dtype = promote(tdt(1), tdt(2)); if (v.dtype < 0) v.dtype = FX_DT_F32; break;
    case FX_OP_INT_ADD: case FX_OP_INT_SUB: case FX_OP_INT_MUL: case FX_OP_INT_NEG: case FX_OP_SIZE:
      v.kind = VK_INT;
      break;
    default:
      FX_CHECK(false, FX_E_UNSUPPORTED, "unknown opcode " << opcode);
  }
  if (v.kind == VK_TENSOR) {
    if (out_dtype >= 0) v.dtype = out_dtype;
    FX_CHECK(v.dtype >= 0, FX_E_INVALID, "cannot infer dtype of op " << opcode);
  }
  return add(v);
}

namespace {

// ---------------------------------------------------------------------------
// symbolic index expressions: affine over root coordinates, the task index,
// reduction loop counters and materialised integer temps
// ---------------------------------------------------------------------------
struct IdxExpr {
  int64_t c[FX_MAXR];
  int64_t ct = 0;
  int64_t rc[FX_MAXLOOP];
  int64_t k = 0;
  std::vector<std::pair<int, int64_t>> tmp;  // (temp slot, coefficient)
  IdxExpr(int64_t k_ = 0) : k(k_) {
    for (auto& x : c) x = 0;
    for (auto& x : rc) x = 0;
  }
  static IdxExpr root(int i) { IdxExpr e; e.c[i] = 1; return e; }
  static IdxExpr task() { IdxExpr e; e.ct = 1; return e; }
  static IdxExpr loop(int d) { IdxExpr e; e.rc[d] = 1; return e; }
  static IdxExpr temp(int slot) { IdxExpr e; e.tmp.push_back({slot, 1}); return e; }
  bool isConst() const {
    for (auto x : c) if (x) return false;
    for (auto x : rc) if (x) return false;
    return ct == 0 && tmp.empty();
  }
  bool affine() const { return tmp.empty(); }
  IdxExpr operator*(int64_t s) const {
    IdxExpr r = *this;
    for (auto& x : r.c) x *= s;
    for (auto& x : r.rc) x *= s;
    r.ct *= s; r.k *= s;
    for (auto& t : r.tmp) t.second *= s;
    if (s == 0) r.tmp.clear();
    return r;
  }
  IdxExpr operator+(const IdxExpr& o) const {
    IdxExpr r = *this;
    for (int i = 0; i < FX_MAXR; ++i) r.c[i] += o.c[i];
    for (int i = 0; i < FX_MAXLOOP; ++i) r.rc[i] += o.rc[i];
    r.ct += o.ct; r.k += o.k;
    for (auto& t : o.tmp) {
      bool found = false;
      for (auto& u : r.tmp) if (u.first == t.first) { u.second += t.second; found = true; }
      if (!found) r.tmp.push_back(t);
    }
    r.tmp.erase(std::remove_if(r.tmp.begin(), r.tmp.end(), [](const std::pair<int, int64_t>& p) { return p.second == 0; }),
                r.tmp.end());
    return r;
  }
  IdxExpr operator-(const IdxExpr& o) const { return *this + o * -1; }
};
typedef std::vector<IdxExpr> Frame;
typedef std::vector<int64_t> Shape;

static int64_t numel_of(const Shape& s) { int64_t n = 1; for (auto d : s) n *= d; return n; }
static Shape contiguous_strides(const Shape& s) {
  Shape st(s.size());
  int64_t b = 1;
  for (int i = (int)s.size() - 1; i >= 0; --i) { st[i] = b; b *= s[i]; }
  return st;
}

struct SlotAlloc;  // plan-global slot tables

// ---------------------------------------------------------------------------
// one lowering context = one task class (identical shapes)
// ---------------------------------------------------------------------------
struct SlotAlloc {
  const Region* R;
  std::vector<PtrSrc> sptr, tptr;
  std::vector<ScalSrc> sscal, tscal;
  std::vector<bool> input_used;
  int ptrSlotOfInput(int input, bool per_task) {
    auto& tab = per_task ? tptr : sptr;
    for (size_t i = 0; i < tab.size(); ++i)
      if (tab[i].kind == PtrSrc::INPUT && tab[i].index == input) return (int)i | (per_task ? FX_SLOT_TASK : 0);
    tab.push_back({PtrSrc::INPUT, input});
    input_used[input] = true;
    return (int)(tab.size() - 1) | (per_task ? FX_SLOT_TASK : 0);
  }
  int scalSlotOfInput(int input, bool per_task, bool as_float) {
    auto& tab = per_task ? tscal : sscal;
    for (size_t i = 0; i < tab.size(); ++i)
      if (tab[i].input == input && tab[i].as_float == as_float) return (int)i | (per_task ? FX_SLOT_TASK : 0);
    tab.push_back({input, as_float});
    return (int)(tab.size() - 1) | (per_task ? FX_SLOT_TASK : 0);
  }
  int ptrSlotOfOutput(int out, bool per_task) {
    auto& tab = per_task ? tptr : sptr;
    tab.push_back({PtrSrc::OUTPUT, out});
    return (int)(tab.size() - 1) | (per_task ? FX_SLOT_TASK : 0);
  }
  int ptrSlotSpecial(PtrSrc::Kind k) {
    sptr.push_back({k, 0});
    return (int)sptr.size() - 1;
  }
};

struct Prog { uint32_t begin, end, vt; bool rowwave; bool wide; };

class Lowerer {
 public:
  Lowerer(const Region& R, const std::vector<const fx_arg*>& in, int n_tasks, SlotAlloc& slots)
      : R_(R), in_(in), nTasks_(n_tasks), slots_(slots), shapeMemo_(R.vals.size()), shapeDone_(R.vals.size(), false) {}

  std::vector<FxInsn> code;
  std::vector<FxAffine> affs;
  int maxTemps = 0;
  bool allowRowWave = false;  // dense outputs only: a reduction over the last dim may use wave-wide ops

  bool usesGuard = false;     // some program loads int64 data into 32-bit arithmetic (checked loads)

  Shape shapeOf(int vid);
  // half: which 32-bit word of an int64 output the program delivers (0 low, 1 high).  Prog::wide
  // says that the low-word program moved int64 data as it is, so that the high words need a
  // program of their own; otherwise the result fits 32 bits and its store sign-extends.
  Prog lower(int vid, const Shape& rootShape, int half = 0);

 private:
  const Region& R_;
  const std::vector<const fx_arg*>& in_;  // representative argument of every region input
  int nTasks_;
  SlotAlloc& slots_;
  std::vector<Shape> shapeMemo_;
  std::vector<bool> shapeDone_;
  // per-program state
  int rootRank_ = 0;
  int64_t rootDim_[FX_MAXR];
  int tempTop_ = 0;
  int maskDepth_ = 0;
  int loopDepth_ = 0;
  int64_t loopExt_[FX_MAXLOOP];
  std::vector<std::pair<int64_t, int64_t>> tempRange_ = std::vector<std::pair<int64_t, int64_t>>(FX_MAX_TEMPS);
  bool loopVarBound_ = false;
  IdxExpr loopVar_;
  bool usedRowWave_ = false;
  // int64 outputs: while only movement operators (views, *_rev merges, cat, index, where ...)
  // lie between a value and the output, the value travels word by word and is exact
  bool moveCtx_ = false;
  int half_ = 0;
  bool sawWide_ = false;
  struct ArithCtx {   // operands of arithmetic: 32-bit values, int64 loads are checked
    Lowerer& l; bool m; int h;
    explicit ArithCtx(Lowerer& l_) : l(l_), m(l_.moveCtx_), h(l_.half_) { l.moveCtx_ = false; l.half_ = 0; }
    ~ArithCtx() { l.moveCtx_ = m; l.half_ = h; }
  };
  void signExtendA() { emitI(FX_ILT, 0, 0, 0, FX_F_IMM); emitI(FX_INEG); }   // A = A < 0 ? -1 : 0
  static uint32_t imm32(int64_t x, const char* what) {
    FX_CHECK(x >= std::numeric_limits<int32_t>::min() && x <= std::numeric_limits<int32_t>::max(), FX_E_UNSUPPORTED,
             what << ": integer constant " << x << " outside 32 bits in integer arithmetic (only moves of int64 data are 64-bit)");
    return (uint32_t)(int32_t)x;
  }
  // true when coordinate `d` of frame f is exactly the innermost root coordinate, nothing else
  // in the frame moves with it, and the whole extent fits one wave item
  bool rowWaveFrame(const Frame& f, int d, int64_t extent) const;

  const Value& V(int id) const { return R_.vals[id]; }

  // ---- scalar evaluation ----
  IdxExpr intOf(int vid);
  int64_t constIntOf(int vid, const char* what);
  bool isNone(int vid) const { return V(vid).kind == VK_NONE; }
  std::vector<int64_t> intListOf(int vid, const char* what);
  std::vector<int> tensorListOf(int vid) const;
  double constScalarOf(int vid, bool* is_float, const char* what);

  // ---- emission helpers ----
  int emitI(uint16_t op, int32_t a = 0, int32_t b = 0, uint32_t imm = 0, uint8_t flags = 0, uint8_t dt = 0) {
    if (op == FX_LDB) flags |= FX_F_MEMB;
    if (op == FX_LDTB) flags |= FX_F_TMPB;
    // A binary operation that follows the load of its B operand takes the load over: one
    // instruction instead of two.  No jump can land between the two: targets are MELSE, MMERGE
    // and loop boundaries, none of which is a binary operation.
    if (fx_op_is_binary(op) && !(flags & FX_F_IMM) && !code.empty() &&
        (code.back().op == FX_LDB || code.back().op == FX_LDTB)) {
      code.back().op = op;
      return (int)code.size() - 1;
    }
    FxInsn i; i.op = op; i.flags = flags; i.dt = dt; i.a = a; i.b = b; i.imm = imm;
    code.push_back(i);
    return (int)code.size() - 1;
  }
  int allocTemp() {
    FX_CHECK(tempTop_ < FX_MAX_TEMPS, FX_E_LIMIT, "region needs more than " << FX_MAX_TEMPS << " temporaries");
    int t = tempTop_++;
    maxTemps = std::max(maxTemps, tempTop_);
    tempRange_[t] = {std::numeric_limits<int32_t>::min(), std::numeric_limits<int32_t>::max()};
    return t;
  }
  void freeTemp(int t) { FX_CHECK(t == tempTop_ - 1, FX_E_INVALID, "temp stack discipline"); --tempTop_; }
  int addAffine(const IdxExpr& e);
  void range(const IdxExpr& e, int64_t* lo, int64_t* hi) const;
  void emitIdx(const IdxExpr& e, bool toB = false, bool i2f = false);  // integer value of e -> A (or B if affine)

  enum RKind { RK_OP, RK_LEAF, RK_IMM, RK_SCALAR, RK_AFFVAL };
  struct Res {
    RKind kind = RK_OP;
    int vid = -1;
    Frame f;
    uint32_t vt = FX_VT_F;   // value class delivered (after post_i2f)
    bool post_i2f = false;   // convert int -> float after producing the value
    // leaf
    int slot = 0; uint32_t dt = 0; IdxExpr addr;
    // imm
    uint32_t imm = 0;
    int64_t imm64 = 0;       // integer constants: the whole value
    // affval
    IdxExpr val;
  };
  Res resolve(int vid, Frame f);
  void emitSimple(const Res& r, bool toB);
  void emit(int vid, const Frame& f);                  // -> A, in the value's own class
  void emitAs(int vid, const Frame& f, uint32_t vt);   // -> A, converted to vt
  void emitOp(const Res& r);
  void emitOpBody(const Res& r);
  void convertA(uint32_t from, uint32_t to) {
    if (from == to) return;
    emitI(from == FX_VT_I ? FX_I2F : FX_F2I);
  }
  // operand of an elementwise op: tensor (broadcast) or scalar
  struct Operand { int vid; Frame f; bool scalar; };
  Operand operandOf(int vid, const Frame& f, const Shape& outShape);
  bool operandSimple(const Operand& o, uint32_t vt, Res* res);
  void emitOperandA(const Operand& o, uint32_t vt);
  void emitBinary(uint16_t op, const Operand& l, const Operand& r, uint32_t vt, double alpha = 1.0);
  void emitCond(const IdxExpr& x, int64_t lo, int64_t hi, int64_t step, const std::function<void()>& thenFn,
                const std::function<void()>& elseFn);
  void emitReduce(uint16_t op, uint32_t identity, int64_t extent, const std::function<void(int depth)>& body, int acc);
  Frame bcastFrame(const Frame& f, const Shape& outShape, const Shape& inShape);
  Frame viewFrame(const Frame& f, const Shape& outShape, const Shape& inShape, std::vector<int>* temps);
  int normDim(int64_t d, int64_t rank, const char* what) {
    if (d < 0) d += rank;
    FX_CHECK(d >= 0 && d < rank, FX_E_INVALID, what << ": dim out of range");
    return (int)d;
  }
  void sliceBounds(int vid_start, int vid_end, int64_t size, int64_t* start, int64_t* end);
  // start as an index expression (may depend on the task index / loop variable) and the
  // number of positions covered before stepping
  bool sliceDynamic(int vid_start, int vid_end, IdxExpr* start, int64_t* extent);
};

// ---------------------------------------------------------------------------
// scalar evaluation
// ---------------------------------------------------------------------------
IdxExpr Lowerer::intOf(int vid) {
  const Value& v = V(vid);
  switch (v.prod) {
    case P_CONST:
      FX_CHECK(v.kind == VK_INT || v.kind == VK_BOOL, FX_E_INVALID, "expected an int value");
      return IdxExpr(v.ival);
    case P_TASK: return IdxExpr::task();
    case P_LOOPVAR:
      FX_CHECK(loopVarBound_, FX_E_INVALID, "loop variable used outside FX_OP_FORALL_SELECT_REV");
      return loopVar_;
    case P_INPUT: {
      FX_CHECK(v.kind == VK_INT || v.kind == VK_BOOL, FX_E_INVALID, "expected an int input");
      // a per-task int that shapes or indices depend on: its values must be part of the plan key
      // and tasks with different values need programs of their own (plan_region starts over)
      if (v.per_task && !(v.input_index < (int)R_.index_ints.size() && R_.index_ints[v.input_index]))
        throw NeedIndexInt{v.input_index};
      return IdxExpr(in_[v.input_index]->ival);
    }
    case P_OP:
      switch (v.op) {
        case FX_OP_INT_ADD: return intOf(v.args[0]) + intOf(v.args[1]);
        case FX_OP_INT_SUB: return intOf(v.args[0]) - intOf(v.args[1]);
        case FX_OP_INT_NEG: return intOf(v.args[0]) * -1;
        case FX_OP_INT_MUL: {
          IdxExpr a = intOf(v.args[0]), b = intOf(v.args[1]);
          if (b.isConst()) return a * b.k;
          if (a.isConst()) return b * a.k;
          FX_CHECK(false, FX_E_UNSUPPORTED, "product of two non-constant ints in index arithmetic");
        }
        case FX_OP_SIZE: {
          Shape s = shapeOf(v.args[0]);
          int d = normDim(constIntOf(v.args[1], "size"), (int64_t)s.size(), "size");
          return IdxExpr(s[d]);
        }
        default: break;
      }
      break;
    default: break;
  }
  FX_CHECK(false, FX_E_UNSUPPORTED, "value " << vid << " is not an integer expression");
  return IdxExpr();
}

int64_t Lowerer::constIntOf(int vid, const char* what) {
  IdxExpr e = intOf(vid);
  FX_CHECK(e.isConst(), FX_E_UNSUPPORTED, what << ": needs a value known when the region is specialised");
  return e.k;
}

std::vector<int64_t> Lowerer::intListOf(int vid, const char* what) {
  const Value& v = V(vid);
  if (v.kind == VK_TENSOR) return shapeOf(vid);  // a tensor where sizes are expected: its sizes (aten::size(t))
  FX_CHECK(v.kind == VK_INT_LIST, FX_E_INVALID, what << ": expected int[]");
  std::vector<int64_t> r;
  for (int a : v.args) r.push_back(constIntOf(a, what));
  return r;
}

std::vector<int> Lowerer::tensorListOf(int vid) const {
  const Value& v = V(vid);
  FX_CHECK(v.kind == VK_TENSOR_LIST, FX_E_INVALID, "expected Tensor[]");
  return v.args;
}

double Lowerer::constScalarOf(int vid, bool* is_float, const char* what) {
  const Value& v = V(vid);
  FX_CHECK(v.prod == P_CONST && (v.kind == VK_FLOAT || v.kind == VK_INT || v.kind == VK_BOOL), FX_E_UNSUPPORTED,
           what << ": expected a constant scalar");
  *is_float = v.kind == VK_FLOAT;
  return v.kind == VK_FLOAT ? v.fval : (double)v.ival;
}

void Lowerer::sliceBounds(int vid_start, int vid_end, int64_t size, int64_t* start, int64_t* end) {
  // ATen slice semantics (clamping) - the functs lowering clamps
  // (nnc_ext.cpp:127-145), the FAIT one does not (custom_lowering_func.cpp:458-470).
  int64_t s = isNone(vid_start) ? 0 : constIntOf(vid_start, "slice start");
  int64_t e = isNone(vid_end) ? size : constIntOf(vid_end, "slice end");
  if (s < 0) s += size;
  if (e < 0) e += size;
  s = std::min(std::max<int64_t>(s, 0), size);
  e = std::min(std::max<int64_t>(e, s), size);
  *start = s;
  *end = e;
}

// A slice whose bounds move with the task index or the collapsed loop variable
// (x[i:i+1] inside a ParallelMap): start stays symbolic, end - start must be a
// constant, and no clamping is applied (the bounds are assumed in range, as the
// FAIT lowering does, custom_lowering_func.cpp:458-470).
bool Lowerer::sliceDynamic(int vid_start, int vid_end, IdxExpr* start, int64_t* extent) {
  if (isNone(vid_start) || isNone(vid_end)) return false;
  IdxExpr s = intOf(vid_start), e = intOf(vid_end);
  if (s.isConst() && e.isConst()) return false;
  IdxExpr d = e - s;
  FX_CHECK(d.isConst(), FX_E_UNSUPPORTED, "slice with task-dependent bounds needs a constant length");
  *start = s;
  *extent = std::max<int64_t>(d.k, 0);
  return true;
}

// ---------------------------------------------------------------------------
// shape functions (fait/fuser/shape_func.cpp:9-374)
// ---------------------------------------------------------------------------
static Shape bcastShape(const Shape& a, const Shape& b) {
  size_t r = std::max(a.size(), b.size());
  Shape o(r);
  for (size_t i = 0; i < r; ++i) {
    int64_t da = i < a.size() ? a[a.size() - 1 - i] : 1;
    int64_t db = i < b.size() ? b[b.size() - 1 - i] : 1;
    FX_CHECK(da == db || da == 1 || db == 1, FX_E_INVALID, "shapes are not broadcastable");
    o[r - 1 - i] = (da == 0 || db == 0) ? 0 : std::max(da, db);
  }
  return o;
}

Shape Lowerer::shapeOf(int vid) {
  if (shapeDone_[vid]) return shapeMemo_[vid];
  const Value& v = V(vid);
  Shape s;
  if (v.kind != VK_TENSOR) {
    s = {};
  } else if (v.prod == P_INPUT) {
    const fx_arg* a = in_[v.input_index];
    s.assign(a->sizes, a->sizes + a->rank);
  } else {
    auto arg = [&](int i) { return v.args.at(i); };
    switch (v.op) {
      case FX_OP_ACCESS: case FX_OP_CLONE: case FX_OP_TRIU: case FX_OP_TRIL: case FX_OP_TO: case FX_OP_EXP:
      case FX_OP_LOG:
      case FX_OP_SQRT: case FX_OP_RSQRT: case FX_OP_SIGMOID: case FX_OP_TANH: case FX_OP_RELU: case FX_OP_NEG:
      case FX_OP_ABS: case FX_OP_FLOOR: case FX_OP_CEIL: case FX_OP_ROUND: case FX_OP_SIN: case FX_OP_COS:
      case FX_OP_ERF: case FX_OP_RECIPROCAL: case FX_OP_LOGICAL_NOT: case FX_OP_CLAMP: case FX_OP_SOFTMAX:
      case FX_OP_SELECT_REV: case FX_OP_SLICE_REV: case FX_OP_FORALL_SELECT_REV:
        s = shapeOf(arg(0));
        break;
      case FX_OP_ASSIGN: s = shapeOf(arg(1)); break;
      case FX_OP_SELECT: {
        s = shapeOf(arg(0));
        int d = normDim(constIntOf(arg(1), "select"), (int64_t)s.size(), "select");
        s.erase(s.begin() + d);
      } break;
      case FX_OP_SLICE: {
        s = shapeOf(arg(0));
        int d = normDim(constIntOf(arg(1), "slice"), (int64_t)s.size(), "slice");
        int64_t st = 0, en = 0;
        IdxExpr dst;
        int64_t ext;
        if (sliceDynamic(arg(2), arg(3), &dst, &ext)) en = ext;
        else sliceBounds(arg(2), arg(3), s[d], &st, &en);
        int64_t step = constIntOf(arg(4), "slice step");
        FX_CHECK(step > 0, FX_E_INVALID, "slice step must be positive");
        s[d] = (en - st + step - 1) / step;
      } break;
      case FX_OP_SQUEEZE: {
        s = shapeOf(arg(0));
        int d = normDim(constIntOf(arg(1), "squeeze"), (int64_t)s.size(), "squeeze");
        if (s[d] == 1) s.erase(s.begin() + d);
      } break;
      case FX_OP_UNSQUEEZE: {
        s = shapeOf(arg(0));
        int d = normDim(constIntOf(arg(1), "unsqueeze"), (int64_t)s.size() + 1, "unsqueeze");
        s.insert(s.begin() + d, 1);
      } break;
      case FX_OP_VIEW: {
        Shape in = shapeOf(arg(0));
        s = intListOf(arg(1), "view");
        int64_t n = numel_of(in), known = 1;
        int neg = -1;
        for (size_t i = 0; i < s.size(); ++i) {
          if (s[i] == -1) { FX_CHECK(neg < 0, FX_E_INVALID, "view: more than one -1"); neg = (int)i; }
          else known *= s[i];
        }
        if (neg >= 0) { FX_CHECK(known != 0 && n % known == 0, FX_E_INVALID, "view: shape mismatch"); s[neg] = n / known; }
        FX_CHECK(numel_of(s) == n, FX_E_INVALID, "view: element count mismatch");
      } break;
      case FX_OP_PERMUTE: {
        Shape in = shapeOf(arg(0));
        auto dims = intListOf(arg(1), "permute");
        FX_CHECK(dims.size() == in.size(), FX_E_INVALID, "permute: rank mismatch");
        s.resize(in.size());
        for (size_t i = 0; i < dims.size(); ++i) s[i] = in[normDim(dims[i], (int64_t)in.size(), "permute")];
      } break;
      case FX_OP_TRANSPOSE: {
        s = shapeOf(arg(0));
        int d0 = normDim(constIntOf(arg(1), "transpose"), (int64_t)s.size(), "transpose");
        int d1 = normDim(constIntOf(arg(2), "transpose"), (int64_t)s.size(), "transpose");
        std::swap(s[d0], s[d1]);
      } break;
      case FX_OP_EXPAND: {
        Shape in = shapeOf(arg(0));
        auto sz = intListOf(arg(1), "expand");
        FX_CHECK(sz.size() >= in.size(), FX_E_INVALID, "expand: rank");
        s.resize(sz.size());
        for (size_t i = 0; i < sz.size(); ++i) {
          int64_t ii = (int64_t)i - (int64_t)(sz.size() - in.size());
          s[i] = sz[i] < 0 ? (ii >= 0 ? in[ii] : 1) : sz[i];
        }
      } break;
      case FX_OP_EXPAND_AS: s = shapeOf(arg(1)); break;
      case FX_OP_REPEAT: {
        Shape in = shapeOf(arg(0));
        auto rep = intListOf(arg(1), "repeat");
        // missing leading repeats count as 1 (computeRepeatShape, shape_func.cpp:206-230)
        while (rep.size() < in.size()) rep.insert(rep.begin(), 1);
        s.resize(rep.size());
        for (size_t i = 0; i < rep.size(); ++i) {
          int64_t ii = (int64_t)i - (int64_t)(rep.size() - in.size());
          s[i] = rep[i] * (ii >= 0 ? in[ii] : 1);
        }
      } break;
      case FX_OP_INDEX: {
        Shape in = shapeOf(arg(0));
        auto idx = tensorListOf(arg(1));
        FX_CHECK(idx.size() == 1, FX_E_UNSUPPORTED, "index: exactly one index tensor (dim 0) is supported");
        s = shapeOf(idx[0]);
        FX_CHECK(!in.empty(), FX_E_INVALID, "index: scalar self");
        s.insert(s.end(), in.begin() + 1, in.end());
      } break;
      case FX_OP_CAT: {
        auto ts = tensorListOf(arg(0));
        FX_CHECK(!ts.empty(), FX_E_INVALID, "cat: empty list");
        s = shapeOf(ts[0]);
        int d = normDim(constIntOf(arg(1), "cat"), (int64_t)s.size(), "cat");
        for (size_t i = 1; i < ts.size(); ++i) s[d] += shapeOf(ts[i])[d];
      } break;
      case FX_OP_STACK: {
        auto ts = tensorListOf(arg(0));
        FX_CHECK(!ts.empty(), FX_E_INVALID, "stack: empty list");
        s = shapeOf(ts[0]);
        int d = normDim(constIntOf(arg(1), "stack"), (int64_t)s.size() + 1, "stack");
        s.insert(s.begin() + d, (int64_t)ts.size());
      } break;
      case FX_OP_FULL: s = V(arg(0)).kind == VK_TENSOR ? shapeOf(arg(0)) : intListOf(arg(0), "full"); break;
      case FX_OP_ARANGE: {
        int64_t a = constIntOf(arg(0), "arange"), b = constIntOf(arg(1), "arange");
        s = {std::max<int64_t>(b - a, 0)};
      } break;
      case FX_OP_SCALAR_TENSOR: s = {}; break;
      case FX_OP_ADD: case FX_OP_SUB: case FX_OP_RSUB: case FX_OP_MUL: case FX_OP_DIV: case FX_OP_MAXIMUM:
      case FX_OP_MINIMUM: case FX_OP_POW: case FX_OP_FMOD: case FX_OP_EQ: case FX_OP_NE: case FX_OP_LT:
      case FX_OP_LE: case FX_OP_GT: case FX_OP_GE: case FX_OP_AND: case FX_OP_OR: case FX_OP_XOR: {
        Shape a = V(arg(0)).kind == VK_TENSOR ? shapeOf(arg(0)) : Shape{};
        Shape b = V(arg(1)).kind == VK_TENSOR ? shapeOf(arg(1)) : Shape{};
        s = bcastShape(a, b);
      } break;
      case FX_OP_WHERE: {
        Shape c = shapeOf(arg(0));
        Shape a = V(arg(1)).kind == VK_TENSOR ? shapeOf(arg(1)) : Shape{};
        Shape b = V(arg(2)).kind == VK_TENSOR ? shapeOf(arg(2)) : Shape{};
        s = bcastShape(c, bcastShape(a, b));
      } break;
      case FX_OP_MAX_DIM: case FX_OP_SUM_DIM: {
        s = shapeOf(arg(0));
        int d = normDim(constIntOf(arg(1), "reduce"), (int64_t)s.size(), "reduce");
        bool keep = v.args.size() > 2 && !isNone(arg(2)) && constIntOf(arg(2), "keepdim") != 0;
        if (keep) s[d] = 1; else s.erase(s.begin() + d);
      } break;
      default:
        FX_CHECK(false, FX_E_UNSUPPORTED, "no shape function for opcode " << v.op);
    }
  }
  shapeMemo_[vid] = s;
  shapeDone_[vid] = true;
  return s;
}

// ---------------------------------------------------------------------------
// index expressions -> code
// ---------------------------------------------------------------------------
int Lowerer::addAffine(const IdxExpr& e) {
  FxAffine a;
  memset(&a, 0, sizeof(a));
  auto fit = [](int64_t x) {
    FX_CHECK(x >= std::numeric_limits<int32_t>::min() && x <= std::numeric_limits<int32_t>::max(), FX_E_LIMIT,
             "index arithmetic exceeds 32 bits");
    return (int32_t)x;
  };
  for (int i = 0; i < FX_MAXR; ++i) fx_aff_set_coef(&a, i, fit(e.c[i]));
  for (int i = 0; i < FX_MAXLOOP; ++i) a.rcoef[i] = fit(e.rc[i]);
  a.tcoef = fit(e.ct);
  a.base = fit(e.k);
  for (size_t i = 0; i < affs.size(); ++i)
    if (memcmp(&affs[i], &a, sizeof(a)) == 0) return (int)i;
  affs.push_back(a);
  return (int)affs.size() - 1;
}

void Lowerer::range(const IdxExpr& e, int64_t* lo, int64_t* hi) const {
  int64_t l = e.k, h = e.k;
  auto term = [&](int64_t coef, int64_t tlo, int64_t thi) {
    if (coef >= 0) { l += coef * tlo; h += coef * thi; } else { l += coef * thi; h += coef * tlo; }
  };
  for (int i = 0; i < FX_MAXR; ++i)
    if (e.c[i]) term(e.c[i], 0, i < rootRank_ ? std::max<int64_t>(rootDim_[i] - 1, 0) : 0);
  if (e.ct) term(e.ct, 0, nTasks_ - 1);
  for (int d = 0; d < FX_MAXLOOP; ++d)
    if (e.rc[d]) term(e.rc[d], 0, d < loopDepth_ ? std::max<int64_t>(loopExt_[d] - 1, 0) : 0);
  for (auto& t : e.tmp) term(t.second, tempRange_[t.first].first, tempRange_[t.first].second);
  *lo = l;
  *hi = h;
}

void Lowerer::emitIdx(const IdxExpr& e, bool toB, bool i2f) {
  if (e.affine()) {
    IdxExpr a = e;
    emitI(toB ? FX_AFFB : FX_AFFA, 0, addAffine(a), 0, i2f ? FX_F_I2F : 0);
    return;
  }
  FX_CHECK(!toB, FX_E_INVALID, "non-affine index into B");
  // A = sum temp_i * coef_i + affine part
  bool first = true;
  for (auto& t : e.tmp) {
    if (first) {
      emitI(FX_LDTA, t.first);
      if (t.second != 1) emitI(FX_IMUL, 0, 0, (uint32_t)(int32_t)t.second, FX_F_IMM);
      first = false;
    } else {
      emitI(FX_LDTB, t.first);
      if (t.second == 1) {
        emitI(FX_IADD);
      } else {
        // A += B * coef : go through a swap to scale B
        emitI(FX_SWAP);
        emitI(FX_IMUL, 0, 0, (uint32_t)(int32_t)t.second, FX_F_IMM);
        emitI(FX_IADD);
      }
    }
  }
  IdxExpr a = e;
  a.tmp.clear();
  bool zero = a.isConst() && a.k == 0;
  if (!zero) {
    if (a.isConst()) {
      emitI(FX_IADD, 0, 0, (uint32_t)(int32_t)a.k, FX_F_IMM);
    } else {
      emitI(FX_AFFB, 0, addAffine(a));
      emitI(FX_IADD);
    }
  }
  if (i2f) emitI(FX_I2F);
}

// ---------------------------------------------------------------------------
// frames
// ---------------------------------------------------------------------------
Frame Lowerer::bcastFrame(const Frame& f, const Shape& outShape, const Shape& inShape) {
  // computeIndicesToBroadcast (nnc_ext.cpp:32-53) / loadBcast (custom_lowering_func.cpp:51-62)
  FX_CHECK(f.size() == outShape.size(), FX_E_INVALID, "frame rank");
  FX_CHECK(inShape.size() <= outShape.size(), FX_E_INVALID, "cannot broadcast to a lower rank");
  size_t off = outShape.size() - inShape.size();
  Frame r(inShape.size());
  for (size_t i = 0; i < inShape.size(); ++i) r[i] = (inShape[i] == 1 && outShape[i + off] != 1) ? IdxExpr(0) : f[i + off];
  return r;
}

// out coordinates of a view/reshape -> coordinates of its input
// (computeImmutView, nnc_ext.cpp:231-295).  Dimensions are matched in groups
// of equal element count; a group with one input dim stays affine, otherwise
// the group's flat index is split with div/mod into integer temps.
Frame Lowerer::viewFrame(const Frame& f, const Shape& outShape, const Shape& inShape, std::vector<int>* temps) {
  Frame r(inShape.size());
  size_t oi = 0, ii = 0;
  while (ii < inShape.size() || oi < outShape.size()) {
    // gather one group
    size_t ob = oi, ib = ii;
    int64_t po = 1, pi = 1;
    if (oi < outShape.size()) po *= outShape[oi++];
    if (ii < inShape.size()) pi *= inShape[ii++];
    while (po != pi) {
      if (po < pi) { FX_CHECK(oi < outShape.size(), FX_E_INVALID, "view: cannot group dims"); po *= outShape[oi++]; }
      else { FX_CHECK(ii < inShape.size(), FX_E_INVALID, "view: cannot group dims"); pi *= inShape[ii++]; }
    }
    // swallow trailing size-1 dims so that groups cover everything
    if (ii == inShape.size()) while (oi < outShape.size() && outShape[oi] == 1) ++oi;
    if (oi == outShape.size()) while (ii < inShape.size() && inShape[ii] == 1) ++ii;
    // flat index of the group over the out dims [ob, oi)
    IdxExpr flat(0);
    int64_t st = 1;
    for (size_t k = oi; k-- > ob;) { flat = flat + f[k] * st; st *= outShape[k]; }
    size_t nin = ii - ib;
    if (nin == 0) continue;
    // input dims of size 1 get 0; if exactly one non-unit dim remains it takes flat
    std::vector<size_t> nonunit;
    for (size_t k = ib; k < ii; ++k) { if (inShape[k] != 1) nonunit.push_back(k); else r[k] = IdxExpr(0); }
    if (nonunit.empty()) continue;
    if (nonunit.size() == 1) { r[nonunit[0]] = flat; continue; }
    if (flat.isConst()) {
      int64_t rem = flat.k;
      for (size_t q = nonunit.size(); q-- > 0;) { size_t k = nonunit[q]; r[k] = IdxExpr(rem % inShape[k]); rem /= inShape[k]; }
      continue;
    }
    // split: dim_k = (flat / stride_k) % size_k
    int64_t stride = 1;
    for (size_t q = nonunit.size(); q-- > 0;) {
      size_t k = nonunit[q];
      emitIdx(flat);
      if (stride != 1) emitI(FX_ITDIV, 0, 0, (uint32_t)(int32_t)stride, FX_F_IMM);
      if (q != 0) emitI(FX_ITMOD, 0, 0, (uint32_t)(int32_t)inShape[k], FX_F_IMM);
      int t = allocTemp();
      emitI(FX_STT, t);
      tempRange_[t] = {0, inShape[k] - 1};
      temps->push_back(t);
      r[k] = IdxExpr::temp(t);
      stride *= inShape[k];
    }
  }
  return r;
}

// ---------------------------------------------------------------------------
// resolve: peel every operator that only transforms coordinates
// ---------------------------------------------------------------------------
Lowerer::Res Lowerer::resolve(int vid, Frame f) {
  Res r;
  bool post_i2f = false;
  for (;;) {
    const Value& v = V(vid);
    FX_CHECK(v.kind == VK_TENSOR, FX_E_INVALID, "value " << vid << " is not a tensor");
    auto arg = [&](int i) { return v.args.at(i); };
    if (v.prod == P_INPUT) {
      const fx_arg* a = in_[v.input_index];
      FX_CHECK((int)f.size() == a->rank, FX_E_INVALID, "frame/rank mismatch at input");
      IdxExpr addr(0);
      for (int d = 0; d < a->rank; ++d) addr = addr + f[d] * a->strides[d];
      r.kind = RK_LEAF;
      r.slot = slots_.ptrSlotOfInput(v.input_index, v.per_task);
      r.dt = storage_dt(v.dtype);
      r.addr = addr;
      r.vt = post_i2f ? FX_VT_F : vt_of(v.dtype);
      r.post_i2f = post_i2f;
      r.vid = vid;
      r.f = f;
      return r;
    }
    FX_CHECK(v.prod == P_OP, FX_E_INVALID, "tensor value without a producer");
    switch (v.op) {
      case FX_OP_ACCESS: case FX_OP_CLONE: vid = arg(0); continue;
      case FX_OP_ASSIGN: vid = arg(1); continue;
      case FX_OP_SELECT: {
        Shape s = shapeOf(arg(0));
        int d = normDim(constIntOf(arg(1), "select"), (int64_t)s.size(), "select");
        IdxExpr idx = intOf(arg(2));
        if (idx.isConst() && idx.k < 0) idx.k += s[d];  // custom_lowering_func.cpp:190-191
        if (idx.isConst()) FX_CHECK(idx.k >= 0 && idx.k < s[d], FX_E_INVALID, "select: index out of range");
        f.insert(f.begin() + d, idx);
        vid = arg(0);
        continue;
      }
      case FX_OP_SLICE: {
        Shape s = shapeOf(arg(0));
        int d = normDim(constIntOf(arg(1), "slice"), (int64_t)s.size(), "slice");
        int64_t st, en;
        int64_t step = constIntOf(arg(4), "slice step");
        IdxExpr dst;
        int64_t ext;
        if (sliceDynamic(arg(2), arg(3), &dst, &ext)) {
          f[d] = f[d] * step + dst;
        } else {
          sliceBounds(arg(2), arg(3), s[d], &st, &en);
          f[d] = f[d] * step + IdxExpr(st);
        }
        vid = arg(0);
        continue;
      }
      case FX_OP_SQUEEZE: {
        Shape s = shapeOf(arg(0));
        int d = normDim(constIntOf(arg(1), "squeeze"), (int64_t)s.size(), "squeeze");
        if (s[d] == 1) f.insert(f.begin() + d, IdxExpr(0));
        vid = arg(0);
        continue;
      }
      case FX_OP_UNSQUEEZE: {
        Shape s = shapeOf(arg(0));
        int d = normDim(constIntOf(arg(1), "unsqueeze"), (int64_t)s.size() + 1, "unsqueeze");
        f.erase(f.begin() + d);
        vid = arg(0);
        continue;
      }
      case FX_OP_PERMUTE: {
        Shape s = shapeOf(arg(0));
        auto dims = intListOf(arg(1), "permute");
        Frame nf(s.size());
        for (size_t i = 0; i < dims.size(); ++i) nf[normDim(dims[i], (int64_t)s.size(), "permute")] = f[i];
        f = nf;
        vid = arg(0);
        continue;
      }
      case FX_OP_TRANSPOSE: {
        Shape s = shapeOf(arg(0));
        int d0 = normDim(constIntOf(arg(1), "transpose"), (int64_t)s.size(), "transpose");
        int d1 = normDim(constIntOf(arg(2), "transpose"), (int64_t)s.size(), "transpose");
        std::swap(f[d0], f[d1]);
        vid = arg(0);
        continue;
      }
      case FX_OP_EXPAND: case FX_OP_EXPAND_AS: {
        f = bcastFrame(f, shapeOf(vid), shapeOf(arg(0)));
        vid = arg(0);
        continue;
      }
      case FX_OP_VIEW: {
        Shape os = shapeOf(vid), is = shapeOf(arg(0));
        // a view is free when it only merges dims or when the frame is constant;
        // otherwise it needs div/mod code -> handled as an operator
        bool needs_code = false;
        {
          size_t oi = 0, ii = 0;
          while (ii < is.size() || oi < os.size()) {
            size_t ib = ii, ob = oi;
            int64_t po = 1, pi = 1;
            if (oi < os.size()) po *= os[oi++];
            if (ii < is.size()) pi *= is[ii++];
            bool bad = false;
            while (po != pi) {
              if (po < pi) { if (oi >= os.size()) { bad = true; break; } po *= os[oi++]; }
              else { if (ii >= is.size()) { bad = true; break; } pi *= is[ii++]; }
            }
            FX_CHECK(!bad, FX_E_INVALID, "view: incompatible shapes");
            if (ii == is.size()) while (oi < os.size() && os[oi] == 1) ++oi;
            if (oi == os.size()) while (ii < is.size() && is[ii] == 1) ++ii;
            int nonunit = 0;
            for (size_t k = ib; k < ii; ++k) if (is[k] != 1) ++nonunit;
            if (nonunit > 1) {
              bool all_const = true;
              for (size_t k = ob; k < oi; ++k) if (!f[k].isConst()) all_const = false;
              if (!all_const) needs_code = true;
            }
          }
        }
        if (needs_code) break;  // RK_OP
        std::vector<int> none;
        f = viewFrame(f, os, is, &none);
        vid = arg(0);
        continue;
      }
      case FX_OP_TO: {
        uint32_t from = vt_of(V(arg(0)).dtype), to = vt_of(v.dtype);
        if (v.dtype == FX_DT_BOOL && V(arg(0)).dtype != FX_DT_BOOL) break;  // needs != 0
        if (from == to) { vid = arg(0); continue; }
        if (from == FX_VT_I && to == FX_VT_F && !post_i2f) { post_i2f = true; vid = arg(0); continue; }
        break;
      }
      case FX_OP_SELECT_REV: {
        Shape s = shapeOf(arg(0));
        int d = normDim(constIntOf(arg(2), "select_rev"), (int64_t)s.size(), "select_rev");
        IdxExpr idx = intOf(arg(3));
        if (idx.isConst() && idx.k < 0) idx.k += s[d];
        IdxExpr diff = f[d] - idx;
        int64_t lo, hi;
        range(diff, &lo, &hi);
        if (lo == 0 && hi == 0) { f.erase(f.begin() + d); vid = arg(1);
          // src may be broadcast against the slab (copy_ semantics)
          { Shape slab = s; slab.erase(slab.begin() + d); f = bcastFrame(f, slab, shapeOf(vid)); }
          continue; }
        if (lo > 0 || hi < 0) { vid = arg(0); continue; }
        break;
      }
      case FX_OP_SLICE_REV: {
        Shape s = shapeOf(arg(0));
        int d = normDim(constIntOf(arg(2), "slice_rev"), (int64_t)s.size(), "slice_rev");
        int64_t st, en;
        sliceBounds(arg(3), arg(4), s[d], &st, &en);
        int64_t step = constIntOf(arg(5), "slice step");
        int64_t lo, hi;
        range(f[d], &lo, &hi);
        if (hi < st || lo >= en || st >= en) { vid = arg(0); continue; }
        if (step == 1 && lo >= st && hi < en) {
          Shape slab = s; slab[d] = en - st;
          f[d] = f[d] - IdxExpr(st);
          vid = arg(1);
          f = bcastFrame(f, slab, shapeOf(vid));
          continue;
        }
        if (f[d].isConst()) {
          // constant coordinate inside [st,en): set iff on the step lattice
          if ((f[d].k - st) % step == 0) {
            Shape slab = s; slab[d] = (en - st + step - 1) / step;
            f[d] = IdxExpr((f[d].k - st) / step);
            vid = arg(1);
            f = bcastFrame(f, slab, shapeOf(vid));
          } else {
            vid = arg(0);
          }
          continue;
        }
        break;
      }
      case FX_OP_FORALL_SELECT_REV: {
        Shape s = shapeOf(arg(0));
        int d = normDim(constIntOf(arg(2), "forall_select_rev"), (int64_t)s.size(), "forall_select_rev");
        int64_t lo_b = constIntOf(arg(3), "loop lower bound"), hi_b = constIntOf(arg(4), "loop upper bound");
        int64_t lo, hi;
        range(f[d], &lo, &hi);
        if (hi < lo_b || lo >= hi_b || lo_b >= hi_b) { vid = arg(0); continue; }
        break;
      }
      case FX_OP_CAT: {
        auto ts = tensorListOf(arg(0));
        Shape s0 = shapeOf(ts[0]);
        int d = normDim(constIntOf(arg(1), "cat"), (int64_t)s0.size(), "cat");
        int64_t lo, hi;
        range(f[d], &lo, &hi);
        int64_t off = 0;
        bool folded = false;
        for (size_t i = 0; i < ts.size(); ++i) {
          int64_t n = shapeOf(ts[i])[d];
          if (lo >= off && hi < off + n) {
            f[d] = f[d] - IdxExpr(off);
            vid = ts[i];
            folded = true;
            break;
          }
          off += n;
        }
        if (folded) continue;
        break;
      }
      case FX_OP_STACK: {
        auto ts = tensorListOf(arg(0));
        Shape s0 = shapeOf(ts[0]);
        int d = normDim(constIntOf(arg(1), "stack"), (int64_t)s0.size() + 1, "stack");
        if (f[d].isConst()) {
          FX_CHECK(f[d].k >= 0 && f[d].k < (int64_t)ts.size(), FX_E_INVALID, "stack index");
          vid = ts[f[d].k];
          f.erase(f.begin() + d);
          continue;
        }
        break;
      }
      case FX_OP_FULL: {
        bool isf;
        const Value& sv = V(arg(1));
        if (sv.prod == P_CONST) {
          double x = constScalarOf(arg(1), &isf, "full");
          r.kind = RK_IMM;
          uint32_t vt = vt_of(v.dtype);
          if (post_i2f) { r.imm = fbits((float)(int64_t)x); r.vt = FX_VT_F; }
          else if (vt == FX_VT_F) { r.imm = fbits((float)x); r.vt = FX_VT_F; }
          else {
            r.imm64 = v.dtype == FX_DT_BOOL ? (int64_t)(x != 0) : (sv.kind == VK_FLOAT ? (int64_t)x : sv.ival);
            r.imm = (uint32_t)r.imm64;
            r.vt = FX_VT_I;
          }
          r.vid = vid;
          return r;
        }
        break;
      }
      case FX_OP_SCALAR_TENSOR: {
        const Value& sv = V(arg(0));
        if (sv.prod == P_CONST) {
          bool isf;
          double x = constScalarOf(arg(0), &isf, "tensor");
          r.kind = RK_IMM;
          uint32_t vt = vt_of(v.dtype);
          if (post_i2f) { r.imm = fbits((float)(int64_t)x); r.vt = FX_VT_F; }
          else if (vt == FX_VT_F) { r.imm = fbits((float)x); r.vt = FX_VT_F; }
          else { r.imm64 = sv.kind == VK_FLOAT ? (int64_t)x : sv.ival; r.imm = (uint32_t)r.imm64; r.vt = FX_VT_I; }
          r.vid = vid;
          return r;
        }
        if (sv.prod == P_INPUT) {
          uint32_t vt = vt_of(v.dtype);
          bool as_float = (vt == FX_VT_F) || post_i2f;
          r.kind = RK_SCALAR;
          r.slot = slots_.scalSlotOfInput(sv.input_index, sv.per_task, as_float);
          r.vt = as_float ? FX_VT_F : FX_VT_I;
          r.vid = vid;
          return r;
        }
        break;
      }
      case FX_OP_ARANGE: {
        IdxExpr start = intOf(arg(0));
        r.kind = RK_AFFVAL;
        r.val = f[0] + start;
        bool to_float = is_float_dt(v.dtype) || post_i2f;
        r.post_i2f = to_float;
        r.vt = to_float ? FX_VT_F : FX_VT_I;
        r.vid = vid;
        if (!r.val.affine()) break;
        return r;
      }
      default: break;
    }
    // needs code
    r.kind = RK_OP;
    r.vid = vid;
    r.f = f;
    r.post_i2f = post_i2f;
    r.vt = post_i2f ? FX_VT_F : vt_of(v.dtype);
    return r;
  }
}

void Lowerer::emitSimple(const Res& r, bool toB) {
  // integer values on their way into an int64 output (move context): int64 data goes word by
  // word, anything narrower is its own low word and its sign is the high word
  const bool mv = moveCtx_ && !toB && r.vt == FX_VT_I && !r.post_i2f;
  switch (r.kind) {
    case RK_LEAF: {
      uint8_t dt = (uint8_t)r.dt;
      bool sext = false;
      if (r.dt == FX_I64 && !r.post_i2f) {
        if (mv) { dt = half_ ? FX_I64HI : FX_I64LO; sawWide_ = true; }
        else usesGuard = true;
      } else if (mv && half_) {
        sext = true;
      }
      if (r.addr.affine()) {
        emitI(toB ? FX_LDB : FX_LDA, r.slot, addAffine(r.addr), 0, r.post_i2f ? FX_F_I2F : 0, dt);
      } else {
        FX_CHECK(!toB, FX_E_INVALID, "indirect load into B");
        { ArithCtx a(*this); emitIdx(r.addr); }
        if (r.post_i2f && r.dt == FX_I64) {
          // the conversion needs the whole element: read both words and combine them as floats
          // is not exact, so the checked 32-bit load stands here
          usesGuard = true;
        }
        emitI(FX_LDXA, r.slot, 0, 0, 0, dt);
        if (r.post_i2f) emitI(FX_I2F);
      }
      if (sext) signExtendA();
    } break;
    case RK_IMM:
      if (mv && r.imm64 != (int64_t)(int32_t)r.imm) sawWide_ = true;
      if (mv && half_) emitI(FX_IMMA, 0, 0, (uint32_t)((uint64_t)r.imm64 >> 32));
      else {
        if (r.vt == FX_VT_I && !mv) (void)imm32(r.imm64, "constant");
        emitI(toB ? FX_IMMB : FX_IMMA, 0, 0, r.imm);
      }
      break;
    case RK_SCALAR: emitI(toB ? FX_SCLB : FX_SCLA, r.slot); if (mv && half_) signExtendA(); break;
    case RK_AFFVAL: emitIdx(r.val, toB, r.post_i2f); if (mv && half_) signExtendA(); break;
    default: FX_CHECK(false, FX_E_INVALID, "emitSimple on an operator");
  }
}

void Lowerer::emit(int vid, const Frame& f) {
  Res r = resolve(vid, f);
  if (r.kind == RK_OP) emitOp(r);
  else emitSimple(r, false);
  // deliver in the value's own class
  uint32_t own = vt_of(V(vid).dtype);
  if (r.vt != own) convertA(r.vt, own);
}

void Lowerer::emitAs(int vid, const Frame& f, uint32_t vt) {
  Res r = resolve(vid, f);
  if (r.kind == RK_OP) emitOp(r);
  else if (r.kind == RK_LEAF && r.vt == FX_VT_I && vt == FX_VT_F && r.addr.affine()) {
    Res q = r; q.post_i2f = true; q.vt = FX_VT_F;
    emitSimple(q, false);
    return;
  } else emitSimple(r, false);
  if (r.vt != vt) convertA(r.vt, vt);
}

Lowerer::Operand Lowerer::operandOf(int vid, const Frame& f, const Shape& outShape) {
  Operand o;
  o.vid = vid;
  const Value& v = V(vid);
  if (v.kind == VK_TENSOR) {
    o.scalar = false;
    o.f = bcastFrame(f, outShape, shapeOf(vid));
  } else {
    FX_CHECK(v.kind == VK_FLOAT || v.kind == VK_INT || v.kind == VK_BOOL, FX_E_INVALID, "operand must be a tensor or scalar");
    o.scalar = true;
  }
  return o;
}

// can this operand be produced straight into B (or as an immediate)?
bool Lowerer::operandSimple(const Operand& o, uint32_t vt, Res* res) {
  if (o.scalar) {
    const Value& v = V(o.vid);
    Res r;
    if (v.prod == P_CONST) {
      r.kind = RK_IMM;
      double x = v.kind == VK_FLOAT ? v.fval : (double)v.ival;
      r.imm = vt == FX_VT_F ? fbits((float)x) : imm32(v.kind == VK_FLOAT ? (int64_t)x : v.ival, "scalar operand");
      r.imm64 = (int64_t)(int32_t)r.imm;
      r.vt = vt;
    } else if (v.prod == P_INPUT) {
      r.kind = RK_SCALAR;
      r.slot = slots_.scalSlotOfInput(v.input_index, v.per_task, vt == FX_VT_F);
      r.vt = vt;
    } else {
      // integer expression (task index, loop var, size ...)
      IdxExpr e = intOf(o.vid);
      if (!e.affine()) return false;
      r.kind = RK_AFFVAL;
      r.val = e;
      r.post_i2f = vt == FX_VT_F;
      r.vt = vt;
    }
    *res = r;
    return true;
  }
  Res r = resolve(o.vid, o.f);
  if (r.kind == RK_OP) return false;
  if (r.kind == RK_LEAF && !r.addr.affine()) return false;
  if (r.vt != vt) {
    if (r.vt == FX_VT_I && vt == FX_VT_F && (r.kind == RK_LEAF || r.kind == RK_AFFVAL)) { r.post_i2f = true; r.vt = FX_VT_F; }
    else if (r.kind == RK_IMM) {
      float fv; memcpy(&fv, &r.imm, 4);
      r.imm = vt == FX_VT_F ? fbits((float)(int32_t)r.imm) : (uint32_t)(int32_t)fv;
      r.vt = vt;
    } else return false;
  }
  *res = r;
  return true;
}

void Lowerer::emitOperandA(const Operand& o, uint32_t vt) {
  if (o.scalar) {
    Res r;
    if (operandSimple(o, vt, &r)) { emitSimple(r, false); return; }
    emitIdx(intOf(o.vid), false, vt == FX_VT_F);
    if (moveCtx_ && half_ && vt == FX_VT_I) signExtendA();
    return;
  }
  emitAs(o.vid, o.f, vt);
}

void Lowerer::emitBinary(uint16_t op, const Operand& l, const Operand& r, uint32_t vt, double alpha) {
  Res rs;
  bool simple = operandSimple(r, vt, &rs);
  if (simple && alpha == 1.0) {
    emitOperandA(l, vt);
    if (rs.kind == RK_IMM) { emitI(op, 0, 0, rs.imm, FX_F_IMM); return; }
    emitSimple(rs, true);
    emitI(op);
    return;
  }
  // general: rhs first, park it in a temp
  emitOperandA(r, vt);
  if (alpha != 1.0) {
    if (vt == FX_VT_F) emitI(FX_FMUL, 0, 0, fbits((float)alpha), FX_F_IMM);
    else emitI(FX_IMUL, 0, 0, (uint32_t)(int32_t)(int64_t)alpha, FX_F_IMM);
  }
  int t = allocTemp();
  emitI(FX_STT, t);
  emitOperandA(l, vt);
  emitI(FX_LDTB, t);
  emitI(op);
  freeTemp(t);
}

// A = (lo <= x < hi && (x-lo) % step == 0) ? then : else, evaluated lazily
void Lowerer::emitCond(const IdxExpr& x, int64_t lo, int64_t hi, int64_t step, const std::function<void()>& thenFn,
                       const std::function<void()>& elseFn) {
  FX_CHECK(maskDepth_ + 1 <= FX_MASK_DEPTH, FX_E_LIMIT, "predicated regions nested deeper than " << FX_MASK_DEPTH);
  const size_t before = code.size();
  emitIdx(x);
  auto fit = [](int64_t v) { return (int32_t)std::min<int64_t>(std::max<int64_t>(v, std::numeric_limits<int32_t>::min()), std::numeric_limits<int32_t>::max()); };
  ++maskDepth_;
  int mif;
  if (code.size() == before + 1 && code.back().op == FX_AFFA && code.back().flags == 0 && lo == 0 && hi > 0 &&
      hi < (1 << 24) && step >= 1 && step < 256) {
    // the index is one affine function of the coordinates: test and predicate in one instruction
    const int32_t aff = code.back().b;
    code.pop_back();
    mif = emitI(FX_MIFR, 0, aff, ((uint32_t)hi << 8) | (uint32_t)step);
  } else {
    emitI(FX_IRANGE, fit(lo), fit(hi), (uint32_t)(int32_t)step);
    mif = emitI(FX_MIF);
  }
  thenFn();
  int t = allocTemp();
  emitI(FX_STT, t);
  int melse = emitI(FX_MELSE);
  code[mif].a = melse;
  elseFn();
  int mm = emitI(FX_MMERGE, t);
  code[melse].a = mm;
  freeTemp(t);
  --maskDepth_;
}

// acc (temp slot) = reduce over loop counter of body()
void Lowerer::emitReduce(uint16_t op, uint32_t identity, int64_t extent, const std::function<void(int)>& body, int acc) {
  FX_CHECK(loopDepth_ < FX_MAXLOOP, FX_E_LIMIT, "reductions nested deeper than " << FX_MAXLOOP);
  int d = loopDepth_++;
  loopExt_[d] = extent;
  emitI(FX_IMMA, 0, 0, identity);
  emitI(FX_STT, acc);
  int rb = emitI(FX_RBEGIN, d, 0, (uint32_t)(int32_t)extent);
  int top = (int)code.size();
  body(d);
  emitI(FX_LDTB, acc);
  emitI(op);
  emitI(FX_STT, acc);
  emitI(FX_RNEXT, top, d);
  code[rb].b = (int)code.size();
  --loopDepth_;
}

static bool isMovementOp(int op) {
  switch (op) {
    case FX_OP_TRIU: case FX_OP_TRIL: case FX_OP_SELECT_REV: case FX_OP_SLICE_REV: case FX_OP_FORALL_SELECT_REV:
    case FX_OP_CAT: case FX_OP_STACK: case FX_OP_VIEW: case FX_OP_REPEAT: case FX_OP_INDEX: case FX_OP_WHERE:
    case FX_OP_FULL: case FX_OP_SCALAR_TENSOR:
      return true;
    default: return false;
  }
}

void Lowerer::emitOp(const Res& r) {
  if (!moveCtx_ || (isMovementOp(V(r.vid).op) && !is_float_dt(V(r.vid).dtype) && !r.post_i2f)) {
    emitOpBody(r);
    return;
  }
  // arithmetic on the way into an int64 output: a 32-bit value whose sign is the high word
  const int half = half_;
  {
    ArithCtx a(*this);
    emitOpBody(r);
  }
  if (half) signExtendA();
}

void Lowerer::emitOpBody(const Res& r) {
  const int vid = r.vid;
  const Value& v = V(vid);
  const Frame& f = r.f;
  auto arg = [&](int i) { return v.args.at(i); };
  const uint32_t own = vt_of(v.dtype);
  auto finish = [&]() { if (r.post_i2f && own == FX_VT_I) emitI(FX_I2F); };
  const Shape outShape = shapeOf(vid);

  struct UOp { int op; uint16_t f; };
  static const UOp unaryF[] = {
      {FX_OP_EXP, FX_EXP}, {FX_OP_LOG, FX_LOG}, {FX_OP_SQRT, FX_SQRT}, {FX_OP_RSQRT, FX_RSQRT},
      {FX_OP_SIGMOID, FX_SIGMOID}, {FX_OP_TANH, FX_TANH}, {FX_OP_SIN, FX_SIN}, {FX_OP_COS, FX_COS},
      {FX_OP_ERF, FX_ERF}, {FX_OP_RECIPROCAL, FX_RCP}, {FX_OP_FLOOR, FX_FLOOR}, {FX_OP_CEIL, FX_CEIL},
      {FX_OP_ROUND, FX_ROUND}};
  for (auto& u : unaryF) {
    if (u.op == v.op) {
      if (own == FX_VT_I) { emitAs(arg(0), f, FX_VT_I); finish(); return; }  // floor/ceil/round of ints
      emitAs(arg(0), f, FX_VT_F);
      emitI(u.f);
      return;
    }
  }
  struct BOp { int op; uint16_t f, i; bool cmp; };
  static const BOp binary[] = {
      {FX_OP_ADD, FX_FADD, FX_IADD, false}, {FX_OP_SUB, FX_FSUB, FX_ISUB, false},
      {FX_OP_RSUB, FX_FRSUB, FX_IRSUB, false}, {FX_OP_MUL, FX_FMUL, FX_IMUL, false},
      {FX_OP_DIV, FX_FDIV, FX_FDIV, false}, {FX_OP_MAXIMUM, FX_FMAX, FX_IMAX, false},
      {FX_OP_MINIMUM, FX_FMIN, FX_IMIN, false}, {FX_OP_POW, FX_FPOW, FX_FPOW, false},
      {FX_OP_FMOD, FX_FMOD, FX_ITMOD, false},
      {FX_OP_EQ, FX_FEQ, FX_IEQ, true}, {FX_OP_NE, FX_FNE, FX_INE, true}, {FX_OP_LT, FX_FLT, FX_ILT, true},
      {FX_OP_LE, FX_FLE, FX_ILE, true}, {FX_OP_GT, FX_FGT, FX_IGT, true}, {FX_OP_GE, FX_FGE, FX_IGE, true},
      {FX_OP_AND, FX_IAND, FX_IAND, false}, {FX_OP_OR, FX_IOR, FX_IOR, false}, {FX_OP_XOR, FX_IXOR, FX_IXOR, false}};
  for (auto& b : binary) {
    if (b.op != v.op) continue;
    Operand l = operandOf(arg(0), f, outShape), rr = operandOf(arg(1), f, outShape);
    // class the arithmetic runs in
    uint32_t cvt;
    if (b.cmp) {
      int dl = V(arg(0)).kind == VK_TENSOR ? V(arg(0)).dtype : (V(arg(0)).kind == VK_FLOAT ? FX_DT_F32 : -1);
      int dr = V(arg(1)).kind == VK_TENSOR ? V(arg(1)).dtype : (V(arg(1)).kind == VK_FLOAT ? FX_DT_F32 : -1);
      int dt = promote(dl, dr);
      cvt = (dt >= 0 && is_float_dt(dt)) ? FX_VT_F : FX_VT_I;
      if (dl < 0 && dr < 0) cvt = FX_VT_I;
    } else if (v.op == FX_OP_AND || v.op == FX_OP_OR || v.op == FX_OP_XOR) {
      cvt = FX_VT_I;
    } else {
      cvt = own;
      if ((v.op == FX_OP_DIV || v.op == FX_OP_POW) ) cvt = FX_VT_F;
    }
    double alpha = 1.0;
    if ((v.op == FX_OP_ADD || v.op == FX_OP_SUB || v.op == FX_OP_RSUB) && v.args.size() > 2 && !isNone(arg(2))) {
      bool isf;
      alpha = constScalarOf(arg(2), &isf, "alpha");
    }
    uint16_t code_op = cvt == FX_VT_F ? b.f : b.i;
    if (v.op == FX_OP_RSUB && alpha != 1.0) {
      // other - alpha * self
      emitBinary(cvt == FX_VT_F ? FX_FSUB : FX_ISUB, rr, l, cvt, alpha);
    } else {
      emitBinary(code_op, l, rr, cvt, alpha);
    }
    uint32_t produced = b.cmp ? (uint32_t)FX_VT_I : cvt;
    if (produced != own) convertA(produced, own);
    finish();
    return;
  }

  switch (v.op) {
    case FX_OP_NEG: emitAs(arg(0), f, own); emitI(own == FX_VT_F ? FX_FNEG : FX_INEG); finish(); return;
    case FX_OP_ABS: emitAs(arg(0), f, own); emitI(own == FX_VT_F ? FX_FABS : FX_IABS); finish(); return;
    case FX_OP_RELU:
      emitAs(arg(0), f, own);
      if (own == FX_VT_F) emitI(FX_RELU); else emitI(FX_IMAX, 0, 0, 0, FX_F_IMM);
      finish();
      return;
    case FX_OP_LOGICAL_NOT: {
      uint32_t src = vt_of(V(arg(0)).dtype);
      emitAs(arg(0), f, src);
      if (src == FX_VT_F) { emitI(FX_FNZ); }
      emitI(FX_LNOT);
      finish();
      return;
    }
    case FX_OP_TO: {
      uint32_t src = vt_of(V(arg(0)).dtype);
      emitAs(arg(0), f, src);
      if (v.dtype == FX_DT_BOOL) emitI(src == FX_VT_F ? FX_FNZ : FX_INZ);
      else convertA(src, own);
      finish();
      return;
    }
    case FX_OP_CLAMP: {
      emitAs(arg(0), f, own);
      for (int k = 1; k <= 2; ++k) {
        if ((int)v.args.size() <= k || isNone(arg(k))) continue;
        Operand o; o.vid = arg(k); o.scalar = true;
        FX_CHECK(V(arg(k)).kind != VK_TENSOR, FX_E_UNSUPPORTED, "clamp with tensor bounds");
        Res rs;
        bool ok = operandSimple(o, own, &rs);
        FX_CHECK(ok, FX_E_UNSUPPORTED, "clamp bound");
        uint16_t op = own == FX_VT_F ? (k == 1 ? FX_FMAX : FX_FMIN) : (k == 1 ? FX_IMAX : FX_IMIN);
        if (rs.kind == RK_IMM) emitI(op, 0, 0, rs.imm, FX_F_IMM);
        else { emitSimple(rs, true); emitI(op); }
      }
      finish();
      return;
    }
    case FX_OP_WHERE: {
      Operand c = operandOf(arg(0), f, outShape), a = operandOf(arg(1), f, outShape), b = operandOf(arg(2), f, outShape);
      uint32_t cv = vt_of(V(arg(0)).dtype);
      { ArithCtx ac(*this); emitOperandA(c, cv); }
      if (cv == FX_VT_F) emitI(FX_FNZ);
      int tc = allocTemp();
      emitI(FX_STT, tc);
      emitOperandA(b, own);
      int tb = allocTemp();
      emitI(FX_STT, tb);
      emitOperandA(a, own);
      emitI(FX_LDTB, tb);
      emitI(FX_WHERE, tc);
      freeTemp(tb);
      freeTemp(tc);
      finish();
      return;
    }
    case FX_OP_TRIU: {
      // computeTriu, custom_lowering_func.cpp:41-49
      FX_CHECK(f.size() >= 2, FX_E_INVALID, "triu needs rank >= 2");
      int64_t diag = constIntOf(arg(1), "triu diagonal");
      IdxExpr x = f[f.size() - 1] - f[f.size() - 2];
      int64_t lo, hi;
      range(x, &lo, &hi);
      if (lo >= diag) { emitAs(arg(0), f, own); finish(); return; }
      uint32_t zero = 0;
      if (hi < diag) { emitI(FX_IMMA, 0, 0, zero); finish(); return; }
      emitCond(x, diag, (int64_t)1 << 40, 1, [&] { emitAs(arg(0), f, own); }, [&] { emitI(FX_IMMA, 0, 0, zero); });
      finish();
      return;
    }
    case FX_OP_TRIL: {
      // the mirror image of triu: element (i, j) survives where j - i <= diagonal
      FX_CHECK(f.size() >= 2, FX_E_INVALID, "tril needs rank >= 2");
      int64_t diag = constIntOf(arg(1), "tril diagonal");
      IdxExpr x = f[f.size() - 1] - f[f.size() - 2];
      int64_t lo, hi;
      range(x, &lo, &hi);
      if (hi <= diag) { emitAs(arg(0), f, own); finish(); return; }
      uint32_t zero = 0;
      if (lo > diag) { emitI(FX_IMMA, 0, 0, zero); finish(); return; }
      emitCond(x, -((int64_t)1 << 40), diag + 1, 1, [&] { emitAs(arg(0), f, own); }, [&] { emitI(FX_IMMA, 0, 0, zero); });
      finish();
      return;
    }
    case FX_OP_SELECT_REV: {
      // computeImmutSelectRev, nnc_ext.cpp:187-212
      Shape s = shapeOf(arg(0));
      int d = normDim(constIntOf(arg(2), "select_rev"), (int64_t)s.size(), "select_rev");
      IdxExpr idx = intOf(arg(3));
      if (idx.isConst() && idx.k < 0) idx.k += s[d];
      Frame fs = f;
      fs.erase(fs.begin() + d);
      Shape slab = s; slab.erase(slab.begin() + d);
      Frame fsrc = bcastFrame(fs, slab, shapeOf(arg(1)));
      emitCond(f[d] - idx, 0, 1, 1, [&] { emitAs(arg(1), fsrc, own); }, [&] { emitAs(arg(0), f, own); });
      finish();
      return;
    }
    case FX_OP_SLICE_REV: {
      // computeImmutSliceRev, nnc_ext.cpp:112-164
      Shape s = shapeOf(arg(0));
      int d = normDim(constIntOf(arg(2), "slice_rev"), (int64_t)s.size(), "slice_rev");
      int64_t st, en;
      sliceBounds(arg(3), arg(4), s[d], &st, &en);
      int64_t step = constIntOf(arg(5), "slice step");
      Shape slab = s; slab[d] = (en - st + step - 1) / step;
      emitCond(f[d], st, en, step,
               [&] {
                 Frame fs = f;
                 int t = -1;
                 if (step == 1) fs[d] = f[d] - IdxExpr(st);
                 else {
                   emitIdx(f[d] - IdxExpr(st));
                   emitI(FX_ITDIV, 0, 0, (uint32_t)(int32_t)step, FX_F_IMM);
                   t = allocTemp();
                   emitI(FX_STT, t);
                   tempRange_[t] = {0, slab[d] - 1};
                   fs[d] = IdxExpr::temp(t);
                 }
                 emitAs(arg(1), bcastFrame(fs, slab, shapeOf(arg(1))), own);
                 if (t >= 0) freeTemp(t);
               },
               [&] { emitAs(arg(0), f, own); });
      finish();
      return;
    }
    case FX_OP_FORALL_SELECT_REV: {
      Shape s = shapeOf(arg(0));
      int d = normDim(constIntOf(arg(2), "forall_select_rev"), (int64_t)s.size(), "forall_select_rev");
      int64_t lo_b = constIntOf(arg(3), "loop lower bound"), hi_b = constIntOf(arg(4), "loop upper bound");
      // eager mode raises IndexError when the loop indexes past the dimension
      FX_CHECK(lo_b >= hi_b || (lo_b >= 0 && hi_b <= s[d]), FX_E_INVALID,
               "collapsed loop over [" << lo_b << ", " << hi_b << ") indexes outside a dimension of size " << s[d]);
      Frame fs = f;
      fs.erase(fs.begin() + d);
      Shape slab = s; slab.erase(slab.begin() + d);
      auto thenFn = [&] {
        bool sb = loopVarBound_; IdxExpr sv = loopVar_;
        loopVarBound_ = true; loopVar_ = f[d];
        emitAs(arg(1), bcastFrame(fs, slab, shapeOf(arg(1))), own);
        loopVarBound_ = sb; loopVar_ = sv;
      };
      int64_t lo, hi;
      range(f[d], &lo, &hi);
      if (lo >= lo_b && hi < hi_b) thenFn();
      else emitCond(f[d], lo_b, hi_b, 1, thenFn, [&] { emitAs(arg(0), f, own); });
      finish();
      return;
    }
    case FX_OP_CAT: {
      // computeCat, custom_lowering_func.cpp:297-330 (nested range tests)
      auto ts = tensorListOf(arg(0));
      Shape s0 = shapeOf(ts[0]);
      int d = normDim(constIntOf(arg(1), "cat"), (int64_t)s0.size(), "cat");
      std::vector<int64_t> offs(ts.size() + 1, 0);
      for (size_t i = 0; i < ts.size(); ++i) offs[i + 1] = offs[i] + shapeOf(ts[i])[d];
      std::function<void(size_t)> rec = [&](size_t i) {
        Frame fi = f;
        fi[d] = f[d] - IdxExpr(offs[i]);
        if (i + 1 == ts.size()) { emitAs(ts[i], fi, own); return; }
        int64_t lo, hi;
        range(f[d], &lo, &hi);
        if (hi < offs[i + 1] && lo >= offs[i]) { emitAs(ts[i], fi, own); return; }
        if (lo >= offs[i + 1] || offs[i + 1] == offs[i]) { rec(i + 1); return; }
        emitCond(f[d], offs[i], offs[i + 1], 1, [&] { emitAs(ts[i], fi, own); }, [&] { rec(i + 1); });
      };
      rec(0);
      finish();
      return;
    }
    case FX_OP_STACK: {
      auto ts = tensorListOf(arg(0));
      Shape s0 = shapeOf(ts[0]);
      int d = normDim(constIntOf(arg(1), "stack"), (int64_t)s0.size() + 1, "stack");
      Frame fi = f;
      fi.erase(fi.begin() + d);
      std::function<void(size_t)> rec = [&](size_t i) {
        if (i + 1 == ts.size()) { emitAs(ts[i], fi, own); return; }
        emitCond(f[d], (int64_t)i, (int64_t)i + 1, 1, [&] { emitAs(ts[i], fi, own); }, [&] { rec(i + 1); });
      };
      rec(0);
      finish();
      return;
    }
    case FX_OP_VIEW: {
      std::vector<int> temps;
      Frame fi = viewFrame(f, outShape, shapeOf(arg(0)), &temps);
      emitAs(arg(0), fi, own);
      for (size_t i = temps.size(); i-- > 0;) freeTemp(temps[i]);
      finish();
      return;
    }
    case FX_OP_REPEAT: {
      // computeImmutRepeat, nnc_ext.cpp:297-318
      Shape in = shapeOf(arg(0));
      size_t off = outShape.size() - in.size();
      Frame fi(in.size());
      std::vector<int> temps;
      for (size_t i = 0; i < in.size(); ++i) {
        const IdxExpr& x = f[i + off];
        int64_t lo, hi;
        range(x, &lo, &hi);
        if (in[i] == 1) fi[i] = IdxExpr(0);
        else if (hi < in[i]) fi[i] = x;
        else if (x.isConst()) fi[i] = IdxExpr(x.k % in[i]);
        else {
          emitIdx(x);
          emitI(FX_ITMOD, 0, 0, (uint32_t)(int32_t)in[i], FX_F_IMM);
          int t = allocTemp();
          emitI(FX_STT, t);
          tempRange_[t] = {0, in[i] - 1};
          temps.push_back(t);
          fi[i] = IdxExpr::temp(t);
        }
      }
      emitAs(arg(0), fi, own);
      for (size_t i = temps.size(); i-- > 0;) freeTemp(temps[i]);
      finish();
      return;
    }
    case FX_OP_INDEX: {
      // computeImmutIndex, nnc_ext.cpp:372-392; negative indices wrap like ATen
      Shape in = shapeOf(arg(0));
      int idx = tensorListOf(arg(1))[0];
      FX_CHECK(!is_float_dt(V(idx).dtype) && V(idx).dtype != FX_DT_BOOL, FX_E_UNSUPPORTED,
               "index: only integer index tensors are fused (bool masks go through fx_region_compact_rows)");
      size_t ir = shapeOf(idx).size();
      Frame fidx(f.begin(), f.begin() + ir);
      { ArithCtx ac(*this); emitAs(idx, fidx, FX_VT_I); }
      emitI(FX_IPMOD, 0, 0, (uint32_t)(int32_t)std::max<int64_t>(in[0], 1), FX_F_IMM);
      int t = allocTemp();
      emitI(FX_STT, t);
      tempRange_[t] = {0, std::max<int64_t>(in[0] - 1, 0)};
      Frame fi;
      fi.push_back(IdxExpr::temp(t));
      fi.insert(fi.end(), f.begin() + ir, f.end());
      emitAs(arg(0), fi, own);
      freeTemp(t);
      finish();
      return;
    }
    case FX_OP_FULL: case FX_OP_SCALAR_TENSOR: {
      int sv = v.op == FX_OP_FULL ? arg(1) : arg(0);
      Operand o; o.vid = sv; o.scalar = true;
      emitOperandA(o, own);
      finish();
      return;
    }
    case FX_OP_ARANGE: {
      emitIdx(f[0] + intOf(arg(0)), false, own == FX_VT_F);
      if (r.post_i2f && own == FX_VT_I) emitI(FX_I2F);
      return;
    }
    case FX_OP_MAX_DIM: case FX_OP_SUM_DIM: {
      // computeMaxDim, custom_lowering_func.cpp:112-132 (serial per output element)
      Shape in = shapeOf(arg(0));
      int d = normDim(constIntOf(arg(1), "reduce"), (int64_t)in.size(), "reduce");
      bool keep = v.args.size() > 2 && !isNone(arg(2)) && constIntOf(arg(2), "keepdim") != 0;
      int acc = allocTemp();
      bool is_max = v.op == FX_OP_MAX_DIM;
      uint32_t ident = own == FX_VT_F ? (is_max ? fbits(-std::numeric_limits<float>::infinity()) : fbits(0.f))
                                      : (is_max ? (uint32_t)std::numeric_limits<int32_t>::min() : 0u);
      uint16_t op = own == FX_VT_F ? (is_max ? FX_FMAX : FX_FADD) : (is_max ? FX_IMAX : FX_IADD);
      emitReduce(op, ident, in[d], [&](int depth) {
        Frame fi = f;
        if (keep) fi[d] = IdxExpr::loop(depth); else fi.insert(fi.begin() + d, IdxExpr::loop(depth));
        emitAs(arg(0), fi, own);
      }, acc);
      emitI(FX_LDTA, acc);
      freeTemp(acc);
      finish();
      return;
    }
    case FX_OP_SOFTMAX: {
      // computeSoftmax, custom_lowering_func.cpp:134-180: max, exp(x-max), sum, div
      Shape in = shapeOf(arg(0));
      int d = normDim(constIntOf(arg(1), "softmax"), (int64_t)in.size(), "softmax");
      if (rowWaveFrame(f, d, in[d])) {
        // the wave holds exactly one row: max / sum are wave reductions instead of a
        // serial loop per element (the reference materialises them as separate
        // kernels, custom_lowering_func.cpp:154-179)
        usedRowWave_ = true;
        emitAs(arg(0), f, FX_VT_F);
        int tx = allocTemp();
        emitI(FX_STT, tx);
        emitI(FX_WMAX);
        emitI(FX_MOVBA);
        emitI(FX_LDTA, tx);
        emitI(FX_FSUB);
        emitI(FX_EXP);
        emitI(FX_STT, tx);
        emitI(FX_WSUM);
        emitI(FX_MOVBA);
        emitI(FX_LDTA, tx);
        emitI(FX_FDIV);
        freeTemp(tx);
        return;
      }
      int tmax = allocTemp();
      emitReduce(FX_FMAX, fbits(-std::numeric_limits<float>::infinity()), in[d], [&](int depth) {
        Frame fi = f; fi[d] = IdxExpr::loop(depth);
        emitAs(arg(0), fi, FX_VT_F);
      }, tmax);
      int tsum = allocTemp();
      emitReduce(FX_FADD, fbits(0.f), in[d], [&](int depth) {
        Frame fi = f; fi[d] = IdxExpr::loop(depth);
        emitAs(arg(0), fi, FX_VT_F);
        emitI(FX_LDTB, tmax);
        emitI(FX_FSUB);
        emitI(FX_EXP);
      }, tsum);
      emitAs(arg(0), f, FX_VT_F);
      emitI(FX_LDTB, tmax);
      emitI(FX_FSUB);
      emitI(FX_EXP);
      emitI(FX_LDTB, tsum);
      emitI(FX_FDIV);
      freeTemp(tsum);
      freeTemp(tmax);
      return;
    }
    default: break;
  }
  FX_CHECK(false, FX_E_UNSUPPORTED, "no lowering for opcode " << v.op);
}

bool Lowerer::rowWaveFrame(const Frame& f, int d, int64_t extent) const {
  if (!allowRowWave || rootRank_ < 1 || maskDepth_ != 0 || loopDepth_ != 0) return false;
  const int r = rootRank_ - 1;
  if (extent != rootDim_[r] || extent > FX_ITEM || extent < 1) return false;
  IdxExpr want = IdxExpr::root(r);
  const IdxExpr& x = f[d];
  if (!x.affine() || x.k != 0 || x.ct != 0) return false;
  for (int i = 0; i < FX_MAXR; ++i) if (x.c[i] != want.c[i]) return false;
  for (int i = 0; i < FX_MAXLOOP; ++i) if (x.rc[i] != 0) return false;
  for (size_t k = 0; k < f.size(); ++k)
    if ((int)k != d && f[k].c[r] != 0) return false;
  return true;
}

Prog Lowerer::lower(int vid, const Shape& rootShape, int half) {
  FX_CHECK(rootShape.size() <= FX_MAXR, FX_E_UNSUPPORTED, "region outputs above rank " << FX_MAXR << " are not supported");
  rootRank_ = (int)rootShape.size();
  for (int i = 0; i < FX_MAXR; ++i) rootDim_[i] = i < rootRank_ ? rootShape[i] : 1;
  tempTop_ = 0;
  maskDepth_ = 0;
  loopDepth_ = 0;
  usedRowWave_ = false;
  moveCtx_ = V(vid).kind == VK_TENSOR && V(vid).dtype == FX_DT_I64;
  half_ = moveCtx_ ? half : 0;
  sawWide_ = false;
  Frame f(rootRank_);
  for (int i = 0; i < rootRank_; ++i) f[i] = IdxExpr::root(i);
  Prog p;
  p.begin = (uint32_t)code.size();
  emit(vid, f);
  p.end = (uint32_t)code.size();
  p.vt = vt_of(V(vid).dtype);
  p.rowwave = usedRowWave_;
  p.wide = sawWide_;
  moveCtx_ = false;
  half_ = 0;
  return p;
}

template <class T>
static uint32_t appendStruct(std::vector<uint32_t>& blob, const T& t) {
  static_assert(sizeof(T) % 4 == 0, "word sized");
  // keep 16-byte alignment for vector scalar loads
  while (blob.size() % 4) blob.push_back(0);
  uint32_t off = (uint32_t)blob.size();
  const uint32_t* w = (const uint32_t*)&t;
  blob.insert(blob.end(), w, w + sizeof(T) / 4);
  return off;
}

struct ClassBuild {
  std::vector<int> tasks;
  std::vector<FxInsn> code;
  std::vector<FxAffine> affs;
  std::vector<FxOut> outs;
  FxClass cls;
};

static void fillDims(FxOut& o, const Shape& s) {
  o.rank = (uint32_t)s.size();
  for (int k = 0; k < FX_MAXR; ++k) {
    uint32_t d = k < (int)s.size() ? (uint32_t)std::max<int64_t>(s[k], 1) : 1u;
    o.dim[k] = d;
    fx_fastdiv_make(d, &o.magic[k], &o.shift[k]);
  }
  // lane groups of FX_V elements along the last dimension
  o.vd = s.empty() ? 0u : (uint32_t)s.size() - 1u;
  o.inner = s.empty() ? 1u : (uint32_t)std::max<int64_t>(s.back(), 1);
  o.gpr = (o.inner + FX_V - 1) / FX_V;
  fx_fastdiv_make(o.gpr, &o.gp_magic, &o.gp_shift);
  int64_t numel = 1;
  for (int64_t d : s) numel *= d;
  o.n_groups = (uint32_t)(numel / o.inner * o.gpr);
  o.gprow = o.gpr;
  fx_fastdiv_make(o.gprow, &o.gr_magic, &o.gr_shift);
}

}  // namespace

// ---------------------------------------------------------------------------
// Window input of a streaming compaction: a tensor input of 32-bit elements that every program
// of the class reads through affine loads of the form  t * task + S * row + (offset inside the
// row)  with one S and one t, so that the rows of a tile are one contiguous run of memory which
// the programs use most of.  Returns false when there is none.
// ---------------------------------------------------------------------------
struct WinCand {
  bool seen = false, bad = false;
  int64_t stride = 0, tcoef = 0, lo = 0, hi = 0;
};
struct WinPick { int slot; int64_t stride, tcoef, lo, span; };
static bool findWindow(const ClassBuild& cb, StreamInfo* si, std::vector<WinPick>* others) {
  std::map<int, WinCand> cand;   // by pointer slot
  bool indirect = false;
  auto scan = [&](uint32_t pb, uint32_t pe, const int64_t* dim, int rank) {
    for (uint32_t pc = pb; pc < pe; ++pc) {
      const FxInsn& in = cb.code[pc];
      const bool affine_load = in.op == FX_LDA || in.op == FX_LDB || (in.flags & FX_F_MEMB);
      if (in.op == FX_LDXA) indirect = true;   // a load through a computed index: stays in memory
      if (in.flags & FX_F_TMPB) continue;
      if (!affine_load) continue;
      WinCand& c = cand[in.a];
      const FxAffine& a = cb.affs[in.b];
      if ((in.dt != FX_F32 && in.dt != FX_I32) || a.rcoef[0] != 0 || a.rcoef[1] != 0) { c.bad = true; continue; }
      const int64_t S = fx_aff_coef(&a, 0);
      int64_t lo = a.base, hi = a.base;
      for (int k = 1; k < FX_MAXR; ++k) {
        const int64_t cf = fx_aff_coef(&a, k);
        if (cf == 0) continue;
        if (k >= rank) { c.bad = true; break; }
        const int64_t ext = cf * (dim[k] - 1);
        lo += std::min<int64_t>(ext, 0);
        hi += std::max<int64_t>(ext, 0);
      }
      if (c.bad) continue;
      if (S <= 0) { c.bad = true; continue; }
      if (!c.seen) { c.seen = true; c.stride = S; c.tcoef = a.tcoef; c.lo = lo; c.hi = hi; }
      else if (c.stride != S || c.tcoef != a.tcoef) c.bad = true;
      else { c.lo = std::min(c.lo, lo); c.hi = std::max(c.hi, hi); }
    }
  };
  const int64_t mdim[FX_MAXR] = {(int64_t)cb.cls.n_rows, 1, 1, 1, 1, 1};
  scan(cb.cls.mask_begin, cb.cls.mask_end, mdim, 1);
  for (const FxOut& od : cb.outs) {
    int64_t dim[FX_MAXR];
    for (int k = 0; k < FX_MAXR; ++k) dim[k] = od.dim[k];
    scan(od.prog_begin, od.prog_end, dim, (int)std::max<uint32_t>(od.rank, 1));
  }
  int best = -1;
  for (auto& kv : cand) {
    const WinCand& c = kv.second;
    if (!c.seen || c.bad || c.lo < 0 || c.tcoef < 0) continue;
    const int64_t span = c.hi - c.lo + 1;
    if (span > c.stride || 2 * span < c.stride) continue;   // rows must be mostly used, and not overlap
    if (best < 0 || c.stride > cand[best].stride) best = kv.first;
  }
  if (best < 0 || indirect) return false;
  // the streaming kernel reads every input from LDS: each of them must be a window
  for (auto& kv : cand) {
    const WinCand& c = kv.second;
    if (kv.first == best) continue;
    if (!c.seen || c.bad || c.lo < 0 || c.tcoef < 0) return false;
    const int64_t span = c.hi - c.lo + 1;
    if (span > c.stride) return false;
    others->push_back({kv.first, c.stride, c.tcoef, c.lo, span});
  }
  if (others->size() > 2) return false;
  const WinCand& c = cand[best];
  si->win_slot = (uint32_t)best;
  si->win_stride = (uint32_t)c.stride;
  si->win_tcoef = (int32_t)c.tcoef;
  si->win_lo = (int32_t)c.lo;
  si->win_span = (uint32_t)(c.hi - c.lo + 1);
  return true;
}

// ---------------------------------------------------------------------------
// plan construction
// ---------------------------------------------------------------------------
static const Plan* plan_region_once(Region& R, const fx_arg* args, int n_args);

const Plan* plan_region(Region& R, const fx_arg* args, int n_args) {
  R.index_ints.resize(R.inputs.size(), 0);
  for (;;) {
    try {
      return plan_region_once(R, args, n_args);
    } catch (const NeedIndexInt& need) {
      FX_CHECK(need.input >= 0 && need.input < (int)R.index_ints.size() && !R.index_ints[need.input], FX_E_INVALID,
               "per-task int input " << need.input << " cannot be resolved");
      R.index_ints[need.input] = 1;
    }
  }
}

static const Plan* plan_region_once(Region& R, const fx_arg* args, int n_args) {
  FX_CHECK(R.finalized, FX_E_INVALID, "region is not finalized");
  const int T = R.degree;
  // argument layout
  std::vector<int> arg_base(R.inputs.size());
  int expect = 0;
  for (size_t i = 0; i < R.inputs.size(); ++i) {
    arg_base[i] = expect;
    expect += R.vals[R.inputs[i]].per_task ? T : 1;
  }
  FX_CHECK(n_args == expect, FX_E_INVALID, "expected " << expect << " arguments, got " << n_args);

  // signature
  std::vector<int64_t> key;
  for (size_t i = 0; i < R.inputs.size(); ++i) {
    const Value& v = R.vals[R.inputs[i]];
    int n = v.per_task ? T : 1;
    for (int t = 0; t < n; ++t) {
      const fx_arg& a = args[arg_base[i] + t];
      if (v.kind == VK_TENSOR) {
        FX_CHECK(a.kind == 0, FX_E_INVALID, "argument " << arg_base[i] + t << " must be a tensor");
        FX_CHECK(a.rank >= 0 && a.rank <= FX_ARG_MAX_RANK, FX_E_INVALID, "bad tensor rank");
        key.push_back(a.dtype); key.push_back(a.rank);
        for (int d = 0; d < a.rank; ++d) { key.push_back(a.sizes[d]); key.push_back(a.strides[d]); }
      } else {
        FX_CHECK(a.kind != 0, FX_E_INVALID, "argument " << arg_base[i] + t << " must be a scalar");
        key.push_back(-7);
        if ((v.kind == VK_INT || v.kind == VK_BOOL) && (!v.per_task || R.index_ints[i])) key.push_back(a.ival);
      }
    }
  }
  auto it = R.plans.find(key);
  if (it != R.plans.end()) return it->second.get();

  std::unique_ptr<Plan> P(new Plan());
  P->region = &R;
  P->arg_base = arg_base;
  P->n_args = n_args;
  P->mode = R.mask >= 0 ? FX_MODE_COMPACT : FX_MODE_DENSE;

  // input dtypes must match the declaration
  for (size_t i = 0; i < R.inputs.size(); ++i) {
    const Value& v = R.vals[R.inputs[i]];
    if (v.kind != VK_TENSOR) continue;
    int n = v.per_task ? T : 1;
    for (int t = 0; t < n; ++t) {
      const fx_arg& a = args[arg_base[i] + t];
      FX_CHECK(a.dtype == v.dtype, FX_E_INVALID, "input " << i << ": dtype differs from the declared one");
      // the kernels address every buffer with a 32-bit byte offset from its base
      int64_t extent = 1;
      for (int d = 0; d < a.rank; ++d) {
        FX_CHECK(a.strides[d] >= 0, FX_E_UNSUPPORTED, "input " << i << ": negative strides are not supported");
        if (a.sizes[d] > 0) extent += (a.sizes[d] - 1) * a.strides[d];
      }
      FX_CHECK(extent * dtype_size(a.dtype) < ((int64_t)1 << 32), FX_E_LIMIT,
               "input " << i << " spans 4 GiB or more; split it before fusing");
      FX_CHECK(a.rank == v.rank || v.rank < 0, FX_E_INVALID, "input " << i << ": rank differs from the declared one");
    }
  }

  // task classes: tasks whose per-task tensors agree in shape and strides
  std::vector<std::vector<int64_t>> tkey(T);
  for (int t = 0; t < T; ++t)
    for (size_t i = 0; i < R.inputs.size(); ++i) {
      const Value& v = R.vals[R.inputs[i]];
      if (!v.per_task) continue;
      const fx_arg& a = args[arg_base[i] + t];
      if (v.kind != VK_TENSOR) {
        if (R.index_ints[i]) tkey[t].push_back(a.ival);
        continue;
      }
      for (int d = 0; d < a.rank; ++d) { tkey[t].push_back(a.sizes[d]); tkey[t].push_back(a.strides[d]); }
    }
  std::vector<ClassBuild> classes;
  {
    std::vector<std::vector<int64_t>> seen;
    for (int t = 0; t < T; ++t) {
      size_t c = 0;
      for (; c < seen.size(); ++c) if (seen[c] == tkey[t]) break;
      if (c == seen.size()) { seen.push_back(tkey[t]); classes.emplace_back(); }
      classes[c].tasks.push_back(t);
    }
  }

  SlotAlloc slots;
  slots.R = &R;
  slots.input_used.assign(R.inputs.size(), false);
  const bool out_per_task = T > 1;
  std::vector<int> out_slot(R.outputs.size());
  for (size_t o = 0; o < R.outputs.size(); ++o) out_slot[o] = slots.ptrSlotOfOutput((int)o, out_per_task);
  int slot_flags = 0, slot_counts = 0, slot_total = 0;
  if (P->mode == FX_MODE_COMPACT) {
    slot_flags = slots.ptrSlotSpecial(PtrSrc::FLAGS);
    slot_counts = slots.ptrSlotSpecial(PtrSrc::COUNTS);
    slot_total = slots.ptrSlotSpecial(PtrSrc::TOTALS);
  }

  P->out_shape.assign(R.outputs.size(), std::vector<Shape>(T));
  P->out_dtype.resize(R.outputs.size());
  for (size_t o = 0; o < R.outputs.size(); ++o) P->out_dtype[o] = R.vals[R.outputs[o]].dtype;

  int max_temps = 0, max_rank = 1;
  int64_t total_rows = 0, max_rows = 0;
  bool uses_guard = false;
  for (auto& cb : classes) {
    std::vector<const fx_arg*> in(R.inputs.size());
    for (size_t i = 0; i < R.inputs.size(); ++i)
      in[i] = &args[arg_base[i] + (R.vals[R.inputs[i]].per_task ? cb.tasks[0] : 0)];
    Lowerer L(R, in, T, slots);
    L.allowRowWave = P->mode == FX_MODE_DENSE;
    memset(&cb.cls, 0, sizeof(cb.cls));
    if (P->mode == FX_MODE_COMPACT) {
      Shape ms = L.shapeOf(R.mask);
      FX_CHECK(ms.size() == 1, FX_E_UNSUPPORTED, "row compaction needs a 1-d mask over dim 0");
      Prog mp = L.lower(R.mask, ms);
      cb.cls.mask_begin = mp.begin;
      cb.cls.mask_end = mp.end;
      cb.cls.mask_vt = mp.vt;
      cb.cls.n_rows = (uint32_t)ms[0];
      total_rows += ms[0] * (int64_t)cb.tasks.size();
      max_rows = std::max<int64_t>(max_rows, ms[0]);
    }
    for (size_t o = 0; o < R.outputs.size(); ++o) {
      Shape s = L.shapeOf(R.outputs[o]);
      FX_CHECK(numel_of(s) * dtype_size(P->out_dtype[o]) < ((int64_t)1 << 32), FX_E_LIMIT,
               "output " << o << " is 4 GiB or larger; split the region");
      for (int t : cb.tasks) P->out_shape[o][t] = s;
      // an int64 output that moves int64 data is two records, one per 32-bit word
      Prog p0 = L.lower(R.outputs[o], s);
      for (int half = 0; half < (p0.wide ? 2 : 1); ++half) {
      Prog p = half == 0 ? p0 : L.lower(R.outputs[o], s, 1);
      FxOut od;
      memset(&od, 0, sizeof(od));
      od.prog_begin = p.begin;
      od.prog_end = p.end;
      od.vt = p.vt;
      fillDims(od, s);
      od.numel = (uint32_t)numel_of(s);
      od.dtype = p0.wide ? (half ? FX_I64HI : FX_I64LO) : storage_dt(P->out_dtype[o]);
      od.ptr_slot = (uint32_t)out_slot[o];
      od.task_stride = 0;
      if (p.rowwave) {
        od.rowwave = 1;
        od.rowlen = (uint32_t)s.back();
        const uint32_t lanes = (od.rowlen + FX_V - 1) / FX_V;
        od.rowseg = lanes <= 16 ? 16u : (lanes <= 32 ? 32u : 64u);
      }
      {
        // leading load: unconditional, affine, not inside a reduction loop
        const FxInsn& i0 = L.code[p.begin];
        od.lead = (p.end > p.begin && i0.op == FX_LDA) ? 1u : 0u;
        bool pure = od.lead != 0 && !p.rowwave;
        for (uint32_t pc = p.begin + 1; pure && pc < p.end; ++pc) {
          const FxInsn& in = L.code[pc];
          pure = fx_op_is_pure_unary(in.op) || (fx_op_is_pure_binary(in.op) && (in.flags & FX_F_IMM));
        }
        od.pure = pure ? 1u : 0u;
      }
      if (P->mode == FX_MODE_COMPACT) {
        FX_CHECK(!s.empty() && s[0] == (int64_t)cb.cls.n_rows, FX_E_INVALID,
                 "compacted output " << o << ": dim 0 must match the mask length");
        od.rowlen = (uint32_t)(s[0] == 0 ? 0 : numel_of(s) / s[0]);
        if (s[0] == 0) { int64_t rl = 1; for (size_t k = 1; k < s.size(); ++k) rl *= s[k]; od.rowlen = (uint32_t)rl; }
        fx_fastdiv_make(std::max<uint32_t>(od.rowlen, 1), &od.rl_magic, &od.rl_shift);
        // narrow rows with a long (predicated) program: walk column by column so that
        // predicates on the inner coordinate are uniform per wave
        od.colmajor = (od.rowlen >= 2 && od.rowlen <= 16 && (p.end - p.begin) >= 24) ? 1u : 0u;
        od.gprow = std::max<uint32_t>(od.rowlen, 1) / od.inner * od.gpr;
        if (s.size() <= 1) od.gprow = 1;  // rank 1: a group is FX_V kept rows
        fx_fastdiv_make(std::max<uint32_t>(od.gprow, 1), &od.gr_magic, &od.gr_shift);
        if (od.colmajor) od.pure = 0;
      }
      max_rank = std::max<int>(max_rank, (int)s.size());
      cb.outs.push_back(od);
      }
    }
    uses_guard = uses_guard || L.usesGuard;
    // The second compaction pass walks the outputs in table order (half of the waves
    // backwards).  Narrow outputs read a few bytes of every kept row, i.e. the same 128-byte
    // lines as each other: next to each other in the walk, the second one finds them in L2.
    if (P->mode == FX_MODE_COMPACT)
      std::stable_sort(cb.outs.begin(), cb.outs.end(), [](const FxOut& a, const FxOut& b) { return a.rowlen < b.rowlen; });
    cb.code = L.code;
    cb.affs = L.affs;
    cb.cls.n_temps = (uint32_t)L.maxTemps;
    max_temps = std::max(max_temps, L.maxTemps);
  }

  // grids.  Row tile of the compaction passes: 256 rows unless that leaves too few
  // tiles to fill 256 CUs.
  uint32_t row_tile = 64;
  if (P->mode == FX_MODE_COMPACT) {
    if (total_rows / 256 >= 512) row_tile = 256;
    else if (total_rows / 128 >= 512) row_tile = 128;
  }
  uint32_t max_rowtiles = (uint32_t)((max_rows + row_tile - 1) / row_tile);
  uint32_t gb = 0, gc = 0, first = 0;
  std::vector<uint32_t> taskmap;
  for (auto& cb : classes) {
    FxClass& c = cb.cls;
    c.first_task = first;
    c.n_tasks = (uint32_t)cb.tasks.size();
    first += c.n_tasks;
    for (int t : cb.tasks) taskmap.push_back((uint32_t)t);
    c.n_outs = (uint32_t)cb.outs.size();
    if (P->mode == FX_MODE_DENSE) {
      uint32_t b = 0;
      for (auto& od : cb.outs) {
        od.block_begin = b;
        // big streaming outputs use large units (per-unit bookkeeping amortised, leading loads of
        // 4 items batched); heavy programs (reduction loops) and small outputs use the smallest
        // unit so that the work spreads over all CUs
        bool heavy = false;
        for (uint32_t pc = od.prog_begin; pc < od.prog_end; ++pc) heavy = heavy || cb.code[pc].op == FX_RBEGIN;
        od.unit_items = (!heavy && od.numel >= (8u << 20)) ? 4u : 1u;
        // a pure tail is evaluated once per four items: worth it as soon as the device still gets
        // four units per CU (a copy of 4 MB takes 2.9 us as 1024 workgroups and 4.4 us as 256)
        if (od.pure && od.numel >= (4u << 20)) od.unit_items = 4u;
        if (od.rowwave) {
          const uint32_t rows = od.rowlen ? od.numel / od.rowlen : 0;
          const uint32_t rows_per_item = 64u / od.rowseg;
          const uint32_t items = (rows + rows_per_item - 1) / rows_per_item;
          od.n_blocks = (items + 4u * od.unit_items - 1) / (4u * od.unit_items);
          od.lead = 0;
        } else {
          const uint32_t unit = 4u * od.unit_items * (FX_ITEM / FX_V);  // groups per work unit
          od.n_blocks = (od.n_groups + unit - 1) / unit;
        }
        b += od.n_blocks;
      }
      c.blocks_per_task = std::max<uint32_t>(b, 1);
      c.block_begin = gb;
      gb += b * c.n_tasks;
      c.block_end = gb;
      if (b == 0) c.blocks_per_task = 1;
    } else {
      c.n_rowtiles = (c.n_rows + row_tile - 1) / row_tile;
      c.blocks_per_task = std::max<uint32_t>(c.n_rowtiles, 1);
      c.block_begin = gb;
      gb += c.n_rowtiles * c.n_tasks;
      c.block_end = gb;
      uint32_t cb_per_task = (c.n_rows + FX_TILE - 1) / FX_TILE;
      c.cnt_blocks_per_task = std::max<uint32_t>(cb_per_task, 1);
      c.cnt_block_begin = gc;
      gc += cb_per_task * c.n_tasks;
      c.cnt_block_end = gc;
    }
  }
  P->grid = gb;
  P->grid_count = gc;
  P->max_rank = max_rank;
  P->n_temps = (uint32_t)max_temps;

  // streaming form of a compaction: one task class with a window input
  int slot_status = 0;
  std::vector<WinPick> side_cand;
  if (P->mode == FX_MODE_COMPACT && classes.size() == 1 && classes[0].cls.n_rows > 0 &&
      findWindow(classes[0], &P->stream, &side_cand)) {
    const ClassBuild& cb = classes[0];
    StreamInfo& si = P->stream;
    // a window must stay inside its buffer for every tile of every task
    auto inside = [&](uint32_t slot, int64_t stride, int64_t tcoef, int64_t lo, int64_t span) {
      const uint32_t idx = slot & 0xffffu;
      const bool per_task = (slot & FX_SLOT_TASK) != 0;
      const PtrSrc& src = per_task ? slots.tptr[idx] : slots.sptr[idx];
      if (src.kind != PtrSrc::INPUT) return false;
      const fx_arg& a = args[arg_base[src.index] + (R.vals[R.inputs[src.index]].per_task ? cb.tasks[0] : 0)];
      int64_t extent = 1;
      for (int d = 0; d < a.rank; ++d) extent += a.sizes[d] > 0 ? (a.sizes[d] - 1) * a.strides[d] : 0;
      for (int d = 0; d < a.rank; ++d) if (a.sizes[d] == 0) extent = 0;
      const int64_t last = tcoef * (T - 1) + (int64_t)(cb.cls.n_rows - 1) * stride + lo + span;
      return last <= extent && last < ((int64_t)1 << 30);
    };
    if (inside(si.win_slot, si.win_stride, si.win_tcoef, si.win_lo, si.win_span)) {
      si.ok = true;
      si.rows = cb.cls.n_rows;
      slot_status = slots.ptrSlotSpecial(PtrSrc::STATUS);
      for (const WinPick& w : side_cand) {
        if (!inside((uint32_t)w.slot, w.stride, w.tcoef, w.lo, w.span)) { si.ok = false; break; }
        const uint32_t i = si.n_side++;
        si.side_slot[i] = (uint32_t)w.slot;
        si.side_stride[i] = (uint32_t)w.stride;
        si.side_tcoef[i] = (int32_t)w.tcoef;
        si.side_lo[i] = (int32_t)w.lo;
        si.side_span[i] = (uint32_t)w.span;
      }
    }
  }

  // checked int64 loads report to an error word of the library
  int slot_err = 0;
  if (uses_guard) slot_err = slots.ptrSlotSpecial(PtrSrc::ERRWORD) + 1;
  P->uses_guard = uses_guard;

  // slot budget
  P->sptr = slots.sptr;
  P->tptr = slots.tptr;
  P->sscal = slots.sscal;
  P->tscal = slots.tscal;
  FX_CHECK(P->tptr.size() <= FX_MAX_TPTR, FX_E_LIMIT, "more than " << FX_MAX_TPTR << " per-task tensors");
  FX_CHECK(P->tscal.size() <= FX_MAX_TSCAL, FX_E_LIMIT, "more than " << FX_MAX_TSCAL << " per-task scalars");
  const size_t n_ptrs = P->sptr.size() + P->tptr.size() * (size_t)T, n_scals = P->sscal.size() + P->tscal.size() * (size_t)T;
  FX_CHECK(n_ptrs <= FX_WIDE_P, FX_E_LIMIT, "tasks x per-task tensors exceeds " << FX_WIDE_P << " pointer slots");
  FX_CHECK(n_scals <= FX_WIDE_S, FX_E_LIMIT, "tasks x per-task scalars exceeds " << FX_WIDE_S << " scalar slots");
  P->wide = n_ptrs > FX_DYN_P || n_scals > FX_DYN_S;
  if (P->wide) P->stream.ok = false;   // (the one-launch forms read their tables from the kernel arguments)

  // scratch: flags [T][max_rows] bytes, counts [T][max_rowtiles] u32
  if (P->mode == FX_MODE_COMPACT) {
    size_t flags = ((size_t)T * (size_t)max_rows + 255) & ~(size_t)255;
    P->flags_off = 0;
    P->counts_off = flags;
    P->scratch_bytes = flags + (((size_t)T * max_rowtiles * 4 + 255) & ~(size_t)255);
    if (P->scratch_bytes == 0) P->scratch_bytes = 256;
    P->launches = 2;
  } else {
    P->launches = gb > 0 ? 1 : 0;
  }
  if (P->wide) {
    P->wide_off = P->scratch_bytes;
    P->wide_bytes = (n_ptrs * 8 + n_scals * 4 + 255) & ~(size_t)255;
    P->scratch_bytes += P->wide_bytes;
  }

  // algorithmic bytes: every referenced input once + dense outputs once
  int64_t bytes = 0;
  for (size_t i = 0; i < R.inputs.size(); ++i) {
    const Value& v = R.vals[R.inputs[i]];
    if (v.kind != VK_TENSOR || !slots.input_used[i]) continue;
    int n = v.per_task ? T : 1;
    for (int t = 0; t < n; ++t) {
      const fx_arg& a = args[arg_base[i] + t];
      int64_t ne = 1;
      for (int d = 0; d < a.rank; ++d) ne *= a.sizes[d];
      bytes += ne * dtype_size(a.dtype);
    }
  }
  if (P->mode == FX_MODE_DENSE)
    for (size_t o = 0; o < R.outputs.size(); ++o)
      for (int t = 0; t < T; ++t) bytes += numel_of(P->out_shape[o][t]) * dtype_size(P->out_dtype[o]);
  P->alg_bytes = bytes;

  // serialise
  std::vector<uint32_t>& blob = P->blob;
  FxHeader h;
  memset(&h, 0, sizeof(h));
  h.magic = FX_MAGIC;
  h.mode = P->mode;
  h.n_classes = (uint32_t)classes.size();
  h.n_tasks = (uint32_t)T;
  h.n_sptr = (uint32_t)P->sptr.size();
  h.n_tptr = (uint32_t)P->tptr.size();
  h.n_sscal = (uint32_t)P->sscal.size();
  h.n_tscal = (uint32_t)P->tscal.size();
  h.row_tile = row_tile;
  h.max_rowtiles = max_rowtiles;
  h.max_rows = (uint32_t)max_rows;
  h.slot_flags = (uint32_t)slot_flags;
  h.slot_counts = (uint32_t)slot_counts;
  h.slot_total = (uint32_t)slot_total;
  h.slot_err = (uint32_t)slot_err;
  h.slot_status = (uint32_t)slot_status;
  appendStruct(blob, h);
  for (auto& cb : classes) {
    while (blob.size() % 4) blob.push_back(0);
    cb.cls.off_insn = (uint32_t)blob.size();
    for (auto& i : cb.code) appendStruct(blob, i);
    { FxInsn nop; memset(&nop, 0, sizeof(nop)); appendStruct(blob, nop); }  // look-ahead pad
    while (blob.size() % 4) blob.push_back(0);
    cb.cls.off_aff = (uint32_t)blob.size();
    for (auto& a : cb.affs) appendStruct(blob, a);
    while (blob.size() % 4) blob.push_back(0);
    cb.cls.off_outs = (uint32_t)blob.size();
    for (auto& o : cb.outs) {
      const uint32_t* w = (const uint32_t*)&o;
      blob.insert(blob.end(), w, w + sizeof(FxOut) / 4);
    }
  }
  while (blob.size() % 4) blob.push_back(0);
  uint32_t off_class = (uint32_t)blob.size();
  for (auto& cb : classes) {
    const uint32_t* w = (const uint32_t*)&cb.cls;
    blob.insert(blob.end(), w, w + sizeof(FxClass) / 4);
  }
  uint32_t off_taskmap = (uint32_t)blob.size();
  blob.insert(blob.end(), taskmap.begin(), taskmap.end());
  while (blob.size() % 4) blob.push_back(0);
  FxHeader* hp = (FxHeader*)blob.data();
  hp->off_class = off_class;
  hp->off_taskmap = off_taskmap;
  hp->total_words = (uint32_t)blob.size();

  // One class of at most FX_FAST_OUTS outputs of 32-bit elements, tasks numbered in order, few
  // enough pointers and scalars: the region fits the lean
  // dense kernel's argument block (the kernel itself exists only for compiled programs).
  memset(&P->lean, 0, sizeof(P->lean));
  if (P->mode == FX_MODE_DENSE && classes.size() == 1 && !classes[0].outs.empty() &&
      classes[0].outs.size() <= FX_FAST_OUTS && P->grid > 0 &&
      P->sptr.size() + P->tptr.size() * (size_t)T <= FX_LEAN_P &&
      P->sscal.size() + P->tscal.size() * (size_t)T <= FX_LEAN_S) {
    const ClassBuild& cb = classes[0];
    bool fits = taskmap.size() == (size_t)T;
    for (size_t i = 0; fits && i < taskmap.size(); ++i) fits = taskmap[i] == (uint32_t)i;
    for (const FxOut& od : cb.outs)
      fits = fits && ((od.dtype == FX_F32 && od.vt == FX_VT_F) || (od.dtype == FX_I32 && od.vt == FX_VT_I));
    if (fits) {
      FxLeanArgs& f = P->lean;
      f.blob_words = (uint32_t)blob.size();
      f.n_p = (uint32_t)(P->sptr.size() + P->tptr.size() * (size_t)T);
      f.n_s = (uint32_t)(P->sscal.size() + P->tscal.size() * (size_t)T);
      f.total_units = P->grid;
      f.n_outs = (uint32_t)cb.outs.size();
      f.bpt = cb.cls.blocks_per_task;
      fx_fastdiv_make(f.bpt, &f.bpt_magic, &f.bpt_shift);
      f.n_sptr = h.n_sptr;
      f.n_tptr = h.n_tptr;
      f.cls_off = off_class;
      f.second_begin = cb.outs.size() > 1 ? cb.outs[1].block_begin : 0xffffffffu;
      P->lean_slot_err = h.slot_err;
      for (size_t o = 0; o < cb.outs.size(); ++o) {
        const FxOut& od = cb.outs[o];
        FxLeanOut& lo = f.out[o];
        lo.ptr_slot = od.ptr_slot;
        lo.lead = od.lead;
        lo.block_begin = od.block_begin;
        lo.task_stride = od.task_stride;
        lo.unit_items = od.unit_items;
        lo.inner = od.inner;
        lo.vd = od.vd;
        lo.gpr = od.gpr;
        lo.gp_magic = od.gp_magic;
        lo.gp_shift = od.gp_shift;
        lo.n_groups = od.rowwave ? (od.inner ? od.numel / od.inner : 0u) : od.n_groups;
        lo.rowseg = od.rowwave ? od.rowseg : 0u;
        for (int k = 1; k < FX_MAXR; ++k) {
          lo.dms[k - 1][0] = od.dim[k];
          lo.dms[k - 1][1] = od.magic[k];
          lo.dms[k - 1][2] = od.shift[k];
        }
        if (!od.lead) continue;
        const FxInsn& li = cb.code[od.prog_begin];
        const FxAffine& af = cb.affs[(size_t)li.b];
        for (int k = 0; k < FX_MAXR; ++k) lo.lead_cf[k] = fx_aff_coef(&af, k);
        lo.lead_base = af.base;
        lo.lead_tcoef = af.tcoef;
        lo.lead_slot = (uint32_t)li.a;
      }
    }
  }

  P->lds_bytes = (uint32_t)((blob.size() + 2 * (P->sptr.size() + P->tptr.size() * (size_t)T) +
                             (P->sscal.size() + P->tscal.size() * (size_t)T) + 4 +
                             (size_t)max_temps * FX_V * FX_BLOCK) * 4);
  // Compiled kernels keep the temporaries in registers: the descriptor alone has to fit.  A
  // region whose interpreter temporaries do not fit as well runs with compiled kernels only.
  const uint32_t lds_descriptor = P->lds_bytes - (uint32_t)((size_t)max_temps * FX_V * FX_BLOCK * 4);
  FX_CHECK(lds_descriptor <= 64 * 1024, FX_E_LIMIT,
           "region descriptor needs " << lds_descriptor << " bytes of LDS (limit 65536)");
  // (a workgroup of the interpreter may take the 160 KB of a CU: 36 temporaries; the launchers
  // ask for what goes beyond the default 64 KB)
  P->needs_compiled = P->lds_bytes > 160 * 1024 - 1024;
  if (P->stream.ok) {
    // Rows per workgroup: the largest of 256 / 128 / 64 whose window fits LDS next to the
    // descriptor (compiled kernels keep temporaries in registers; the interpreter checks its own
    // budget when it launches); smaller while the launch would leave CUs without a workgroup.
    StreamInfo& si = P->stream;
    const int64_t budget = 64000 - (int64_t)lds_descriptor;
    uint32_t rt = 0;
    auto buf_words = [&](uint32_t rows) { return (3 + (int64_t)(rows - 1) * si.win_stride + si.win_span + 3) & ~(int64_t)3; };
    auto side_words_of = [&](uint32_t rows, uint32_t i) {
      return (3 + (int64_t)(rows - 1) * si.side_stride[i] + si.side_span[i] + 3) & ~(int64_t)3;
    };
    // a side window is one 16-byte line per lane: at most FX_BLOCK lines; wider ones stay in memory
    auto side_total = [&](uint32_t rows) {
      int64_t w = 0;
      for (uint32_t i = 0; i < si.n_side; ++i)
        w += side_words_of(rows, i) <= 4 * FX_BLOCK ? side_words_of(rows, i) : ((int64_t)1 << 40);   // must fit
      return w;
    };
    for (uint32_t cand : {256u, 128u, 64u}) {
      if ((buf_words(cand) + side_total(cand)) * 4 > budget) continue;
      rt = cand;
      const int64_t tiles = (int64_t)T * ((si.rows + cand - 1) / cand);
      if (tiles >= 512 || cand == 64u) break;
    }
    if (rt == 0) si.ok = false;
    else {
      si.tile_rows = rt;
      si.tiles_per_task = (si.rows + rt - 1) / rt;
      si.grid = si.tiles_per_task * (uint32_t)T;
      si.win_words = (uint32_t)buf_words(rt);
      for (uint32_t i = 0; i < 2; ++i) si.side_words[i] = i < si.n_side ? (uint32_t)side_words_of(rt, i) : 0u;
    }
  }
  P->spec_key = spec_hash(*P);
  if (!P->wide) {   // (the hand-written kernels read their tables from the kernel arguments)
    match_head(P.get());
    match_classmap(P.get());
  }
  rs_analyze(P.get());
  const Plan* res = P.get();
  R.plans[key] = std::move(P);
  return res;
}

// ---------------------------------------------------------------------------
// disassembler (debugging aid, the analogue of CodeGen::getCodeText)
// ---------------------------------------------------------------------------
const char* opname(uint32_t op) {
  static const char* names[] = {
      "NOP", "LDA", "LDB", "LDXA", "AFFA", "AFFB", "IMMA", "IMMB", "SCLA", "SCLB", "STT", "LDTA", "LDTB", "MOVBA",
      "SWAP", "MIF", "MELSE", "MMERGE", "MEND", "MIFR", "FNEG", "FABS", "EXP", "LOG", "SQRT", "RSQRT", "RCP", "SIGMOID",
      "TANH", "RELU", "FLOOR", "CEIL", "ROUND", "TRUNC", "SIN", "COS", "ERF", "LOG2", "EXP2", "EXPM1", "LOG1P",
      "INEG", "LNOT", "INZ", "FNZ", "F2I", "I2F", "IABS", "FADD", "FSUB", "FRSUB", "FMUL", "FDIV", "FRDIV", "FMIN",
      "FMAX", "FPOW", "FMOD", "ATAN2", "IADD", "ISUB", "IRSUB", "IMUL", "IFDIV", "ITDIV", "IPMOD", "ITMOD", "IMIN",
      "IMAX", "IAND", "IOR", "IXOR", "FLT", "FLE", "FGT", "FGE", "FEQ", "FNE", "ILT", "ILE", "IGT", "IGE", "IEQ",
      "INE", "IRANGE", "WHERE", "RBEGIN", "RNEXT", "RIDX", "WMAX", "WSUM"};
  if (op < sizeof(names) / sizeof(names[0])) return names[op];
  return "?";
}

// ---- specialisation: the compile-time part of a plan, its key and its source ----
int kernel_rank(int rank) { return rank <= 1 ? 1 : rank <= 4 ? rank : FX_MAXR; }

namespace {
struct SpecEntry { int begin, end, kind, pure; };
struct SpecView {
  const FxInsn* ins = nullptr;
  uint32_t n_insn = 0;
  uint32_t n_temps = 0;
  uint32_t mode = 0;
  int rank = 1;
  std::vector<SpecEntry> entries;
};
// Only plans with one task class (all tasks share their programs) are specialised.
bool spec_view(const Plan& p, SpecView* v) {
  const uint32_t* sb = p.blob.data();
  const FxHeader* h = (const FxHeader*)sb;
  if (h->n_classes != 1) return false;
  const FxClass& cl = *(const FxClass*)(sb + h->off_class);
  const FxOut* outs = (const FxOut*)(sb + cl.off_outs);
  v->ins = (const FxInsn*)(sb + cl.off_insn);
  v->n_temps = cl.n_temps;
  v->mode = h->mode;
  v->rank = kernel_rank(p.max_rank);
  uint32_t n = 0;
  if (h->mode == FX_MODE_COMPACT) {
    v->entries.push_back({(int)cl.mask_begin, (int)cl.mask_end, 1, 0});
    n = std::max(n, cl.mask_end);
  }
  for (uint32_t k = 0; k < cl.n_outs; ++k) {
    const FxOut& od = outs[k];
    v->entries.push_back({(int)(od.prog_begin + (od.lead ? 1u : 0u)), (int)od.prog_end, 0, (int)od.pure});
    n = std::max(n, od.prog_end);
  }
  v->n_insn = n;
  return n > 0;
}
}  // namespace

uint64_t spec_hash(const Plan& p) {
  SpecView v;
  if (!spec_view(p, &v)) return 0;
  uint64_t hsh = 1469598103934665603ull;   // FNV-1a, 64 bits
  auto mix = [&](const void* data, size_t n) {
    const uint8_t* b = (const uint8_t*)data;
    for (size_t i = 0; i < n; ++i) { hsh ^= b[i]; hsh *= 1099511628211ull; }
  };
  const uint32_t head[5] = {v.mode, (uint32_t)v.rank, v.n_insn, v.n_temps, (uint32_t)FX_V};
  mix(head, sizeof(head));
  for (uint32_t i = 0; i < v.n_insn; ++i) {
    const FxInsn& x = v.ins[i];
    const uint32_t w[4] = {(uint32_t)x.op | ((uint32_t)x.flags << 16) | ((uint32_t)x.dt << 24), (uint32_t)x.a, (uint32_t)x.b, x.imm};
    mix(w, sizeof(w));
  }
  for (const SpecEntry& e : v.entries) mix(&e, sizeof(e));
  return hsh ? hsh : 1;
}

std::string spec_source(const Plan& p, const std::string& label) {
  SpecView v;
  FX_CHECK(spec_view(p, &v), FX_E_UNSUPPORTED, "only plans whose tasks share one set of programs can be specialised");
  const uint64_t hsh = spec_hash(p);
  char hx[32];
  snprintf(hx, sizeof(hx), "%016llx", (unsigned long long)hsh);
  std::ostringstream o;
  o << "// Generated by fx_plan_spec_source; do not edit.  Region: " << label << "\n"
    << "// The lowered programs of this region as a compile-time table: the region kernels are\n"
    << "// instantiated for it and picked at run time when a plan's programs hash to the same key.\n"
    << "#include \"../fx_spec.h\"\n\nnamespace {\nstruct P_" << hx << " {\n"
    << "  static constexpr uint64_t hash = 0x" << hx << "ull;\n"
    << "  static constexpr int n_temps = " << v.n_temps << ";\n"
    << "  static constexpr FxInsn code[" << v.n_insn << "] = {\n";
  for (uint32_t i = 0; i < v.n_insn; ++i) {
    const FxInsn& x = v.ins[i];
    o << "      {FX_" << opname(x.op) << ", " << (int)x.flags << ", " << (int)x.dt << ", " << x.a << ", " << x.b << ", 0x"
      << std::hex << x.imm << std::dec << "u},  // " << i << "\n";
  }
  o << "  };\n  static constexpr int n_entries = " << v.entries.size() << ";\n"
    << "  static constexpr FxSpecEntry entries[" << v.entries.size() << "] = {";
  for (size_t i = 0; i < v.entries.size(); ++i) {
    const SpecEntry& e = v.entries[i];
    o << (i ? ", " : "") << "{" << e.begin << ", " << e.end << ", " << e.kind << ", " << e.pure << "}";
  }
  o << "};\n};\n}  // namespace\n\n"
    << (v.mode == FX_MODE_COMPACT ? "FX_SPEC_COMPACT" : "FX_SPEC_DENSE") << "(P_" << hx << ", " << v.rank << ")\n";
  return o.str();
}

std::string disasm(const Plan& p) {
  std::ostringstream o;
  const uint32_t* sb = p.blob.data();
  const FxHeader* h = (const FxHeader*)sb;
  o << "mode=" << h->mode << " classes=" << h->n_classes << " tasks=" << h->n_tasks << " sptr=" << h->n_sptr
    << " tptr=" << h->n_tptr << " sscal=" << h->n_sscal << " tscal=" << h->n_tscal << " grid=" << p.grid
    << " grid_count=" << p.grid_count << " lds=" << p.lds_bytes << " row_tile=" << h->row_tile << "\n";
  const FxClass* cls = (const FxClass*)(sb + h->off_class);
  for (uint32_t c = 0; c < h->n_classes; ++c) {
    const FxClass& cl = cls[c];
    o << "class " << c << ": tasks=" << cl.n_tasks << " blocks/task=" << cl.blocks_per_task << " temps=" << cl.n_temps
      << " rows=" << cl.n_rows << "\n";
    const FxInsn* ins = (const FxInsn*)(sb + cl.off_insn);
    const FxAffine* aff = (const FxAffine*)(sb + cl.off_aff);
    const FxOut* outs = (const FxOut*)(sb + cl.off_outs);
    auto dump = [&](uint32_t b, uint32_t e) {
      for (uint32_t i = b; i < e; ++i) {
        const FxInsn& x = ins[i];
        float fv; memcpy(&fv, &x.imm, 4);
        o << "    " << i << ": " << opname(x.op) << " a=" << x.a << " b=" << x.b << " imm=" << (int32_t)x.imm << "/" << fv
          << " fl=" << (int)x.flags << " dt=" << (int)x.dt;
        if (x.op == FX_LDA || x.op == FX_AFFA || x.op == FX_AFFB || x.op == FX_MIFR || (x.flags & FX_F_MEMB)) {
          const FxAffine& a = aff[x.b];
          o << "  [";
          for (int k = 0; k < FX_MAXR; ++k) o << fx_aff_coef(&a, k) << (k + 1 < FX_MAXR ? "," : "");
          o << "] t=" << a.tcoef << " r=" << a.rcoef[0] << "," << a.rcoef[1] << " base=" << a.base;
        }
        o << "\n";
      }
    };
    if (h->mode == FX_MODE_COMPACT) { o << "  mask:\n"; dump(cl.mask_begin, cl.mask_end); }
    for (uint32_t k = 0; k < cl.n_outs; ++k) {
      o << "  out " << k << ": numel=" << outs[k].numel << " rank=" << outs[k].rank << " blocks=" << outs[k].n_blocks
        << " rowlen=" << outs[k].rowlen << " inner=" << outs[k].inner << " lead=" << outs[k].lead
        << " pure=" << outs[k].pure << " unit_items=" << outs[k].unit_items << " colmajor=" << outs[k].colmajor << "\n";
      dump(outs[k].prog_begin, outs[k].prog_end);
    }
  }
  return o.str();
}

}  // namespace fx
