// CanonicalizeOps and HoistLoopInvariants: the two clean-up passes in front of region formation.
//
// CanonicalizeOps (fait/passes/canonicalize.cpp:148-157) brings spellings that mean the same to the
// one spelling the later passes know:
//   arange(end)                    -> arange(0, end)
//   max.other / min.other          -> maximum / minimum
//   new_zeros / new_ones(self, ..) -> zeros / ones with self's dtype and device
//   pow(x, n), n a constant int >= 1 -> products (square and multiply)
//   slice / immut::slice without start and end, step 1 -> the tensor itself
//   t() of a matrix                -> transpose(0, 1)
//   to.dtype / to.other            -> to(device, dtype)
//   view                           -> reshape
// Two rewrites of the reference are narrowed on purpose: its slice rule drops the operator
// whatever the step is (canonicalize.cpp:72-80: x[::2] would become x), and its pow rule yields
// x * x for every odd exponent above one (canonicalize.cpp:51-70: the first set bit is skipped
// while `base` is still unset); here the step must be 1 and pow(x, n) is x multiplied n times.
//
// HoistLoopInvariants (fait/passes/licm.cpp:55-66, called first thing by ParallelizeLoops,
// parallelize_loops.cpp:128-131): scalar-valued pure nodes of a loop or map body whose operands
// are all defined outside move in front of the loop, innermost loops first, so that trip counts
// and sizes stop looking like per-iteration values.
#include <cmath>
#include <ATen/ATen.h>
#include <torch/csrc/jit/ir/constants.h>

#include <sstream>
#include <unordered_set>

#include "passes.h"
#include "symbols.h"

namespace functs {
using namespace torch::jit;

namespace {

bool isTensorValue(const Value* v) { return v->type()->kind() == c10::TypeKind::TensorType; }
bool isNone(Value* v) { return v->mustBeNone(); }
std::optional<int64_t> constInt(Value* v) {
  auto c = toIValue(v);
  if (c && c->isInt()) return c->toInt();
  return std::nullopt;
}

// a node of kind `k` at the insertion point (operands in schema order, keyword-only ones included)
Value* make(Graph* g, Symbol k, at::ArrayRef<Value*> inputs, c10::TypePtr type = c10::TensorType::get()) {
  Node* n = g->create(k, inputs, 1);
  g->insertNode(n);
  n->output()->setType(std::move(type));
  return n->output();
}

// dtype / device of `self` as values: constants when the type says so, prim::dtype / prim::device otherwise
Value* dtypeOf(Graph* g, Value* self) {
  auto tt = self->type()->cast<c10::TensorType>();
  if (tt && tt->scalarType()) return g->insertConstant((int64_t)*tt->scalarType());
  return make(g, c10::prim::dtype, {self}, c10::IntType::get());
}
Value* deviceOf(Graph* g, Value* self) { return make(g, c10::prim::device, {self}, c10::DeviceObjType::get()); }

// returns true when `n` was replaced (and destroyed)
bool rewrite(Node* n) {
  Graph* g = n->owningGraph();
  const Symbol k = n->kind();
  const size_t ni = n->inputs().size();
  WithInsertPoint at(n);
  auto replaceWith = [&](Value* v) {
    v->node()->setSourceRange(n->sourceRange());
    v->setType(n->output(0)->type());   // what was known about the result stays known
    n->output(0)->replaceAllUsesWith(v);
    n->destroy();
    return true;
  };
  if (k == c10::aten::arange && ni == 5 && !isTensorValue(n->input(0))) {   // arange(end, dtype, layout, device, pin_memory)
    Value* zero = g->insertConstant((int64_t)0);
    return replaceWith(make(g, c10::aten::arange, {zero, n->input(0), n->input(1), n->input(2), n->input(3), n->input(4)}));
  }
  if ((k == c10::aten::max || k == c10::aten::min) && ni == 2 && n->outputs().size() == 1 && isTensorValue(n->input(0)) &&
      isTensorValue(n->input(1))) {
    return replaceWith(make(g, k == c10::aten::max ? c10::aten::maximum : c10::aten::minimum, {n->input(0), n->input(1)}));
  }
  if ((k == c10::aten::new_zeros || k == c10::aten::new_ones) && ni == 6) {   // (self, size, dtype, layout, device, pin_memory)
    Value* self = n->input(0);
    Value* dtype = isNone(n->input(2)) ? dtypeOf(g, self) : n->input(2);
    Value* device = isNone(n->input(4)) ? deviceOf(g, self) : n->input(4);
    Value* none = g->insertConstant(c10::IValue());
    return replaceWith(make(g, k == c10::aten::new_zeros ? c10::aten::zeros : c10::aten::ones,
                                 {n->input(1), dtype, none, device, none}));
  }
  if (k == c10::aten::pow && ni == 2 && isTensorValue(n->input(0))) {
    auto e = constInt(n->input(1));
    if (!e || *e < 1 || *e > 64) return false;
    // square and multiply: result = product of the squares that the set bits of e select
    Value* sq = n->input(0);
    Value* acc = nullptr;
    for (int64_t left = *e; left > 0; left >>= 1) {
      if (left & 1) acc = acc ? make(g, c10::aten::mul, {acc, sq}) : sq;
      if (left > 1) sq = make(g, c10::aten::mul, {sq, sq});
    }
    if (acc == n->input(0)) return false;   // e == 1: pow(x, 1) keeps its own node (a copy, not an alias)
    return replaceWith(acc);
  }
  if ((k == c10::aten::slice || k == sym::Slice()) && ni == 5 && isNone(n->input(2)) && isNone(n->input(3)) &&
      constInt(n->input(4)) == std::optional<int64_t>(1)) {
    // the graph is functionalized: nothing writes through the view that aten::slice returns
    n->output(0)->replaceAllUsesWith(n->input(0));
    n->destroy();
    return true;
  }
  if (k == c10::aten::t && ni == 1) {
    auto tt = n->input(0)->type()->cast<c10::TensorType>();
    if (!tt || !tt->dim() || *tt->dim() != 2) return false;   // t() of a vector is the vector
    Value* zero = g->insertConstant((int64_t)0);
    Value* one = g->insertConstant((int64_t)1);
    Value* tr = make(g, c10::aten::transpose, {n->input(0), zero, one});
    tr->node()->setSourceRange(n->sourceRange());
    tr->setType(tt->dimensionedOnly());   // still a matrix of that element type: a t() of it is rewritten as well
    n->output(0)->replaceAllUsesWith(tr);
    n->destroy();
    return true;
  }
  if (k == c10::aten::to && isTensorValue(n->input(0))) {
    Value* self = n->input(0);
    Value* f = g->insertConstant(false);
    Value* none = g->insertConstant(c10::IValue());
    // to.dtype(self, dtype, non_blocking, copy, memory_format)
    if (ni == 5 && n->input(1)->type()->kind() == c10::TypeKind::IntType)
      return replaceWith(make(g, c10::aten::to, {self, deviceOf(g, self), n->input(1), f, f, none}));
    // to.other(self, other, non_blocking, copy, memory_format)
    if (ni == 5 && isTensorValue(n->input(1)))
      return replaceWith(make(g, c10::aten::to, {self, deviceOf(g, n->input(1)), dtypeOf(g, n->input(1)), f, f, none}));
    return false;
  }
  if (k == c10::aten::view && ni == 2 && n->input(1)->type()->cast<c10::ListType>()) {
    return replaceWith(make(g, c10::aten::reshape, {n->input(0), n->input(1)}));
  }
  return false;
}

void canonicalizeIn(Block* b) {
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* n = *it;
    ++it;
    for (Block* inner : n->blocks()) canonicalizeIn(inner);
    rewrite(n);
  }
}

// ---------------------------------------------------------------------------
bool scalarLike(const c10::TypePtr& t) {
  switch (t->kind()) {
    case c10::TypeKind::IntType:
    case c10::TypeKind::FloatType:
    case c10::TypeKind::BoolType:
    case c10::TypeKind::DeviceObjType:
    case c10::TypeKind::NoneType:
      return true;
    case c10::TypeKind::TupleType:
      for (const auto& e : t->containedTypes())
        if (!scalarLike(e)) return false;
      return true;
    default:
      return false;   // tensors stay (licm.cpp:25-27); lists can be appended to
  }
}

bool definedOutside(Value* v, Block* body) {
  for (Block* b = v->node()->owningBlock(); b; b = b->owningNode() ? b->owningNode()->owningBlock() : nullptr)
    if (b == body) return false;
  return true;
}

// operators without side effects that cannot fail for operands that are valid outside the loop
const std::unordered_set<Symbol>& hoistable() {
  using namespace c10;
  static const std::unordered_set<Symbol> s{
      aten::size, aten::dim, aten::add, aten::sub, aten::mul, aten::neg, aten::eq, aten::ne, aten::lt, aten::le,
      aten::gt, aten::ge, aten::__range_length, aten::__derive_index, aten::__not__, aten::__and__, aten::__or__, aten::Int,
      aten::Float, aten::Bool, aten::min, aten::max, prim::device, prim::dtype, prim::TupleConstruct, prim::TupleIndex,
      prim::TupleUnpack, prim::min, prim::max};
  return s;
}

bool invariant(Node* n, Block* body) {
  if (n->outputs().empty() || !n->blocks().empty() || n->hasSideEffects()) return false;
  if (!hoistable().count(n->kind())) return false;
  for (Value* o : n->outputs())
    if (!scalarLike(o->type())) return false;
  for (Value* in : n->inputs())
    if (!definedOutside(in, body)) return false;
  return true;
}

bool hoistIn(Block* b) {
  bool changed = false;
  for (Node* n : b->nodes()) {
    for (Block* inner : n->blocks()) changed = hoistIn(inner) || changed;   // innermost loops first
    if (n->kind() != c10::prim::Loop && n->kind() != sym::ParallelMap()) continue;
    Block* body = n->blocks()[0];
    for (auto it = body->nodes().begin(); it != body->nodes().end();) {
      Node* m = *it;
      ++it;
      if (m->kind() == c10::prim::Constant || !invariant(m, body)) continue;
      m->moveBefore(n);   // what it produced inside an inner loop has already arrived here, so one walk suffices
      changed = true;
    }
  }
  return changed;
}

}  // namespace

namespace {

// ---- static type queries ---------------------------------------------------------------------
// What the static types say about `v`: its own tensor type, or, for an element read from a list
// argument with a refined type, the element's type (the unified one when the index is not a
// constant).
c10::TensorTypePtr staticTensorType(Value* v) {
  if (auto tt = v->type()->cast<c10::TensorType>())
    if (tt->scalarType() || tt->sizes().size() || tt->device()) return tt;
  Node* n = v->node();
  if (n->kind() != c10::aten::__getitem__) return nullptr;
  auto it = refinedTypes().find(n->input(0));
  if (it == refinedTypes().end()) return nullptr;
  const auto& elems = it->second->expectRef<c10::TupleType>().elements();
  if (auto idx = constInt(n->input(1))) {
    int64_t i = *idx < 0 ? *idx + (int64_t)elems.size() : *idx;
    if (i < 0 || i >= (int64_t)elems.size()) return nullptr;
    return elems[i]->cast<c10::TensorType>();
  }
  std::stringstream why_not;
  auto unified = c10::unifyTypeList(elems, why_not);
  return unified ? (*unified)->cast<c10::TensorType>() : nullptr;
}

bool foldQueriesIn(Block* b) {
  static const Symbol kNumel = Symbol::fromQualString("aten::numel");
  bool changed = false;
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* n = *it;
    ++it;
    for (Block* inner : n->blocks()) changed |= foldQueriesIn(inner);
    const auto k = n->kind();
    if (k != c10::aten::size && k != c10::prim::dtype && k != c10::prim::device && k != c10::aten::dim && k != kNumel)
      continue;
    if (n->inputs().empty() || n->outputs().size() != 1) continue;
    auto tt = staticTensorType(n->input(0));
    if (!tt) continue;
    Graph* g = n->owningGraph();
    WithInsertPoint guard(n);
    Value* c = nullptr;
    if (k == c10::aten::size && n->inputs().size() == 2) {
      auto d = constInt(n->input(1));
      auto rank = tt->sizes().size();
      if (d && rank) {
        int64_t dim = *d < 0 ? *d + (int64_t)*rank : *d;
        if (dim >= 0 && dim < (int64_t)*rank && tt->sizes()[dim]) c = g->insertConstant(*tt->sizes()[dim]);
      }
    } else if (k == c10::aten::size && n->inputs().size() == 1) {
      if (auto sizes = tt->sizes().concrete_sizes()) c = g->insertConstant(c10::IValue(c10::List<int64_t>(*sizes)));
    } else if (k == kNumel) {
      if (auto sizes = tt->sizes().concrete_sizes()) {
        int64_t numel = 1;
        for (int64_t v : *sizes) numel *= v;
        c = g->insertConstant(numel);
      }
    } else if (k == c10::aten::dim) {
      if (auto rank = tt->sizes().size()) c = g->insertConstant((int64_t)*rank);
    } else if (k == c10::prim::dtype) {
      if (tt->scalarType()) c = g->insertConstant((int64_t)*tt->scalarType());
    } else if (k == c10::prim::device) {
      // only a GPU: a function built from CPU examples still runs on whatever device its
      // arguments live on, and what it creates there must follow them
      if (tt->device() && tt->device()->is_cuda()) c = g->insertConstant(c10::IValue(*tt->device()));
    }
    if (!c) continue;
    n->output()->replaceAllUsesWith(c);
    n->destroy();
    changed = true;
  }
  return changed;
}

}  // namespace

bool FoldStaticTypeQueries(std::shared_ptr<Graph> graph) { return foldQueriesIn(graph->block()); }

namespace {
// A tensor constant whose elements are all one value (what constant propagation makes of
// zeros_like(c), new_zeros, full over a folded shape) goes back to being a fill: inside a region a
// fill costs nothing, a constant is an argument that is read from memory.
bool fillsIn(Block* b) {
  bool changed = false;
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* n = *it;
    ++it;
    for (Block* inner : n->blocks()) changed |= fillsIn(inner);
    if (n->kind() != c10::prim::Constant || !isTensorValue(n->output())) continue;
    auto iv = toIValue(n->output());
    if (!iv || !iv->isTensor()) continue;
    const at::Tensor t = iv->toTensor();
    if (!t.defined() || t.numel() < 16 || t.is_sparse() || !t.is_contiguous()) continue;
    const auto st = t.scalar_type();
    if (st != c10::kFloat && st != c10::kLong && st != c10::kInt && st != c10::kBool) continue;
    // only where a region can absorb the fill: a reader outside regions would run it on every call
    bool absorbed = !n->output()->uses().empty();
    for (const Use& u : n->output()->uses()) absorbed = absorbed && isFusableNode(u.user);
    if (!absorbed) continue;
    const at::Tensor flat = t.reshape({-1});
    // uniform bit for bit: +0.0 and -0.0 compare equal and are different constants
    const at::Tensor bits = st == c10::kFloat ? flat.view(c10::kInt) : flat;
    if (!at::eq(bits, bits[0]).all().item<bool>()) continue;
    Graph* g = n->owningGraph();
    WithInsertPoint guard(n);
    Value* sizes = g->insertConstant(c10::IValue(c10::List<int64_t>(t.sizes().vec())));
    Value* none = g->insertConstant(c10::IValue());
    Value* dtype = g->insertConstant((int64_t)st);
    Value* device = g->insertConstant(c10::IValue(t.device()));
    const c10::Scalar v = flat[0].item();
    Value* fill = nullptr;
    auto type = c10::TensorType::create(t);
    if (v.to<double>() == 0.0 && !std::signbit(v.to<double>())) {   // aten::zeros makes +0.0
      fill = make(g, c10::aten::zeros, {sizes, dtype, none, device, none}, type);
    } else {
      Value* value = st == c10::kFloat ? g->insertConstant(v.to<double>())
                                       : (st == c10::kBool ? g->insertConstant(v.to<bool>()) : g->insertConstant(v.to<int64_t>()));
      fill = make(g, c10::aten::full, {sizes, value, dtype, none, device, none}, type);
    }
    n->output()->replaceAllUsesWith(fill);
    n->destroy();
    changed = true;
  }
  return changed;
}
}  // namespace

bool UniformConstantsToFills(std::shared_ptr<Graph> graph) { return fillsIn(graph->block()); }

void CanonicalizeOps(std::shared_ptr<Graph> graph) { canonicalizeIn(graph->block()); }

bool HoistLoopInvariants(std::shared_ptr<Graph> graph) { return hoistIn(graph->block()); }

}  // namespace functs
