// CollapseRecurrentLoops: the (time, layer) loop nest of a stacked LSTM, whose loops carry the
// hidden and cell states, becomes ONE node fx::lstm_stack, which ToParallelFunctor wraps into a
// tssa::ParallelFunctor that runs the persistent kernel fx_lstm_stack.
//
// The reference cannot do anything with these loops: a loop with carried values is never
// parallelised (fait/passes/parallelize_loops.cpp:17) and, its trip count not being a constant,
// not unrolled either (fait/passes/unroll_loops.cpp:59-65), so every (t, layer) costs a fused
// kernel and two library GEMMs launched from the host (the reference's worst launch count,
// figures/kernel_launch.py:14).  The program recognised here is the reference's benchmark model
// functs/benchmark/ai_model/lstm/lstm.py:79-133 after functionalization:
//
//   for t in range(T):                       prim::Loop carrying out, state_h, state_c
//     cur = x[t]
//     for j in range(L):                     prim::Loop carrying cur, state_h, state_c
//       h = select(state_h, 0, j); c = select(state_c, 0, j)
//       ih = matmul(cur, wih[j]) + bih[j];  hh = matmul(h, whh[j]) + bhh[j]
//       i, f, g, o = sigmoid(ih[0] + hh[0]), sigmoid(ih[1] + hh[1]), tanh(ih[2] + hh[2]), sigmoid(ih[3] + hh[3])
//       c2 = f * c + i * g;  h2 = o * tanh(c2)
//       state_c = select_rev(state_c, c2, 0, j); state_h = select_rev(state_h, h2, 0, j); cur = h2
//     out = select_rev(out, cur, 0, t)
//
// The match is structural (operand order of the commutative operators free, order of the carried
// values free) and complete: a body with any other node is left alone.
#include <torch/csrc/jit/ir/constants.h>

#include <algorithm>
#include <unordered_set>

#include "../../../include/fxhip.h"
#include "passes.h"
#include "symbols.h"

namespace functs {
using namespace torch::jit;

namespace {

bool isConst(Value* v, int64_t k) {
  auto c = toIValue(v);
  return c && c->isInt() && c->toInt() == k;
}
bool isTrue(Value* v) {
  auto c = toIValue(v);
  return c && c->isBool() && c->toBool();
}
bool isSelectKind(Node* n) { return n->kind() == c10::aten::select || n->kind() == sym::Select(); }

struct Matcher {
  std::unordered_set<Node*> used;

  // select(base, 0, idx) with idx a given value; returns base
  Value* selectAt(Value* v, Value* idx) {
    Node* n = v->node();
    if (!isSelectKind(n) || !isConst(n->input(1), 0) || n->input(2) != idx) return nullptr;
    used.insert(n);
    return n->input(0);
  }
  // select(base, 0, k) with k a constant; returns base
  Value* selectConst(Value* v, int64_t k) {
    Node* n = v->node();
    if (!isSelectKind(n) || !isConst(n->input(1), 0) || !isConst(n->input(2), k)) return nullptr;
    used.insert(n);
    return n->input(0);
  }
  bool binary(Value* v, Symbol kind, Value** a, Value** b) {
    Node* n = v->node();
    if (n->kind() != kind) return false;
    if (kind == c10::aten::add && !(n->inputs().size() == 3 && isConst(n->input(2), 1))) return false;
    used.insert(n);
    *a = n->input(0);
    *b = n->input(1);
    return true;
  }
  Value* unary(Value* v, Symbol kind) {
    Node* n = v->node();
    if (n->kind() != kind) return nullptr;
    used.insert(n);
    return n->input(0);
  }
  // select_rev(self, src, 0, idx)
  bool selectRev(Value* v, Value* idx, Value** self, Value** src) {
    Node* n = v->node();
    if (n->kind() != sym::SelectRev() || !isConst(n->input(2), 0) || n->input(3) != idx) return false;
    used.insert(n);
    *self = n->input(0);
    *src = n->input(1);
    return true;
  }
};

bool definedOutside(Value* v, Node* loop) {
  for (Block* b = v->node()->owningBlock(); b; b = b->owningNode() ? b->owningNode()->owningBlock() : nullptr)
    if (b->owningNode() == loop) return false;
  return true;
}

struct LstmNest {
  Value *x = nullptr, *wih = nullptr, *whh = nullptr, *bih = nullptr, *bhh = nullptr;
  Value *T = nullptr, *L = nullptr;
  size_t out_i = 0, h_i = 0, c_i = 0;   // positions among the outer loop's carried values
  std::vector<Node*> hoist;             // loop-invariant integer arithmetic in the time loop's body
};

// activation(add(select(A, 0, k), select(B, 0, k))); A / B in either order
bool gate(Matcher& m, Value* v, Symbol act, int64_t k, Value** ih, Value** hh) {
  Value* s = m.unary(v, act);
  Value *a, *b;
  if (!s || !m.binary(s, c10::aten::add, &a, &b)) return false;
  Value* pa = m.selectConst(a, k);
  Value* pb = m.selectConst(b, k);
  if (!pa || !pb) return false;
  if (!*ih) { *ih = pa; *hh = pb; return true; }
  if (pa == *ih && pb == *hh) return true;
  if (pa == *hh && pb == *ih) return true;
  return false;
}

bool matchNest(Node* outer, LstmNest* r) {
  if (outer->kind() != c10::prim::Loop || outer->inputs().size() != 5 || !isTrue(outer->input(1))) return false;
  Block* ob = outer->blocks()[0];
  if (!isTrue(ob->outputs()[0])) return false;
  Value* t = ob->inputs()[0];
  // the body: select of x, the layer loop, select_rev into out, constants
  Node *inner = nullptr, *xsel = nullptr, *orev = nullptr;
  for (Node* n : ob->nodes()) {
    if (n->kind() == c10::prim::Constant) continue;
    // integer arithmetic on loop-invariant values, e.g. the layer loop's trip count
    // wih.size(0) - 1 written inside the time loop: moved in front of the loops on a match
    static const std::unordered_set<Symbol> int_ops{c10::aten::size, c10::aten::add, c10::aten::sub, c10::aten::mul,
                                                    c10::aten::neg, c10::aten::floordiv, c10::aten::__range_length};
    if (int_ops.count(n->kind()) && n->outputs().size() == 1 && n->output()->type()->kind() == c10::TypeKind::IntType) {
      bool invariant = true;
      for (Value* v : n->inputs())
        invariant = invariant && (definedOutside(v, outer) ||
                                  std::find(r->hoist.begin(), r->hoist.end(), v->node()) != r->hoist.end());
      if (invariant) {
        r->hoist.push_back(n);
        continue;
      }
    }
    if (n->kind() == c10::prim::Loop && !inner) inner = n;
    else if (isSelectKind(n) && !xsel) xsel = n;
    else if (n->kind() == sym::SelectRev() && !orev) orev = n;
    else return false;
  }
  if (!inner || !xsel || !orev) return false;
  if (inner->inputs().size() != 5 || !isTrue(inner->input(1))) return false;
  Block* ib = inner->blocks()[0];
  if (!isTrue(ib->outputs()[0])) return false;
  Value* j = ib->inputs()[0];
  Matcher m;

  // roles of the inner loop's three carried values, from what the body returns for them
  int ic = -1, ih_ = -1, icur = -1;
  Value *c2 = nullptr, *h2 = nullptr;
  for (int i = 0; i < 3; ++i) {
    Value *self, *src;
    Value* ret = ib->outputs()[1 + i];
    Value* param = ib->inputs()[1 + i];
    if (ret->node()->kind() == sym::SelectRev()) {
      if (!m.selectRev(ret, j, &self, &src) || self != param) return false;
      // which state it is shows below: h2 is also the value returned for `cur`
      if (ic < 0) { ic = i; c2 = src; }
      else { ih_ = i; h2 = src; }
    } else {
      icur = i;
    }
  }
  if (ic < 0 || ih_ < 0 || icur < 0) return false;
  if (ib->outputs()[1 + icur] != h2) {   // the first select_rev seen was the hidden state
    std::swap(ic, ih_);
    std::swap(c2, h2);
    if (ib->outputs()[1 + icur] != h2) return false;
  }
  Value* cur = ib->inputs()[1 + icur];
  Value* Ph = ib->inputs()[1 + ih_];
  Value* Pc = ib->inputs()[1 + ic];

  // h2 = o * tanh(c2)
  Value *a, *b;
  if (!m.binary(h2, c10::aten::mul, &a, &b)) return false;
  Value* og = nullptr;
  if (b->node()->kind() == c10::aten::tanh && m.unary(b, c10::aten::tanh) == c2) og = a;
  else if (a->node()->kind() == c10::aten::tanh && m.unary(a, c10::aten::tanh) == c2) og = b;
  if (!og) return false;
  // c2 = f * c + i * g
  Value *p, *q;
  if (!m.binary(c2, c10::aten::add, &p, &q)) return false;
  Value *p0, *p1, *q0, *q1;
  if (!m.binary(p, c10::aten::mul, &p0, &p1) || !m.binary(q, c10::aten::mul, &q0, &q1)) return false;
  auto isCell = [&](Value* v) { return m.selectAt(v, j) == Pc; };
  Value *fg = nullptr, *ig = nullptr, *gg = nullptr;
  Value *r0 = nullptr, *r1 = nullptr;
  if (isSelectKind(p0->node()) && isCell(p0)) { fg = p1; r0 = q0; r1 = q1; }
  else if (isSelectKind(p1->node()) && isCell(p1)) { fg = p0; r0 = q0; r1 = q1; }
  else if (isSelectKind(q0->node()) && isCell(q0)) { fg = q1; r0 = p0; r1 = p1; }
  else if (isSelectKind(q1->node()) && isCell(q1)) { fg = q0; r0 = p0; r1 = p1; }
  else return false;
  if (r0->node()->kind() == c10::aten::tanh) { gg = r0; ig = r1; } else { gg = r1; ig = r0; }

  Value *IH = nullptr, *HH = nullptr;
  if (!gate(m, ig, c10::aten::sigmoid, 0, &IH, &HH)) return false;
  if (!gate(m, fg, c10::aten::sigmoid, 1, &IH, &HH)) return false;
  if (!gate(m, gg, c10::aten::tanh, 2, &IH, &HH)) return false;
  if (!gate(m, og, c10::aten::sigmoid, 3, &IH, &HH)) return false;

  // IH / HH = matmul(lhs, select(W, 0, j)) + select(b, 0, j); which is which shows at the matmul
  struct Half { Value *lhs, *w, *bias; };
  auto half = [&](Value* v, Half* h) {
    Value *s0, *s1;
    if (!m.binary(v, c10::aten::add, &s0, &s1)) return false;
    Value* mm = s0->node()->kind() == c10::aten::matmul ? s0 : s1;
    Value* bs = mm == s0 ? s1 : s0;
    if (mm->node()->kind() != c10::aten::matmul) return false;
    m.used.insert(mm->node());
    h->lhs = mm->node()->input(0);
    h->w = m.selectAt(mm->node()->input(1), j);
    h->bias = m.selectAt(bs, j);
    return h->w != nullptr && h->bias != nullptr;
  };
  Half h0, h1;
  if (!half(IH, &h0) || !half(HH, &h1)) return false;
  if (h0.lhs != cur) std::swap(h0, h1);
  if (h0.lhs != cur) return false;
  if (!isSelectKind(h1.lhs->node()) || m.selectAt(h1.lhs, j) != Ph) return false;

  // nothing else in the layer loop
  for (Node* n : ib->nodes())
    if (n->kind() != c10::prim::Constant && !m.used.count(n)) return false;

  // the time loop around it
  if (!isConst(xsel->input(1), 0) || xsel->input(2) != t) return false;
  if (inner->input(2 + icur) != xsel->output()) return false;
  Value* Qh = inner->input(2 + ih_);
  Value* Qc = inner->input(2 + ic);
  int oh = -1, oc = -1, oo = -1;
  for (int i = 0; i < 3; ++i) {
    Value* q = ob->inputs()[1 + i];
    if (q == Qh && ob->outputs()[1 + i] == inner->output(ih_)) oh = i;
    // the two states may start from one and the same tensor, but are carried separately
  }
  for (int i = 0; i < 3; ++i) {
    Value* q = ob->inputs()[1 + i];
    if (i != oh && q == Qc && ob->outputs()[1 + i] == inner->output(ic)) oc = i;
  }
  for (int i = 0; i < 3; ++i)
    if (i != oh && i != oc) oo = i;
  if (oh < 0 || oc < 0 || oo < 0) return false;
  Value *oself, *osrc;
  Matcher mo;
  if (ob->outputs()[1 + oo] != orev->output() || !mo.selectRev(orev->output(), t, &oself, &osrc)) return false;
  if (oself != ob->inputs()[1 + oo] || osrc != inner->output(icur)) return false;

  r->x = xsel->input(0);
  r->wih = h0.w; r->bih = h0.bias; r->whh = h1.w; r->bhh = h1.bias;
  r->T = outer->input(0);
  r->L = inner->input(0);
  r->out_i = (size_t)oo; r->h_i = (size_t)oh; r->c_i = (size_t)oc;
  auto hoisted = [&](Value* v) { return std::find(r->hoist.begin(), r->hoist.end(), v->node()) != r->hoist.end(); };
  for (Value* v : {r->x, r->wih, r->whh, r->bih, r->bhh, r->L})
    if (!definedOutside(v, outer) && !hoisted(v)) return false;
  return true;
}

// the kernel's limits (include/fxhip.h fx_lstm_stack), checked on the static types the pipeline
// gave the graph inputs; without static shapes the loops stay as they are
bool shapesFit(const LstmNest& r) {
  auto sizes = [](Value* v) -> std::optional<std::vector<int64_t>> {
    auto tt = v->type()->cast<c10::TensorType>();
    if (!tt || !tt->scalarType() || *tt->scalarType() != c10::kFloat) return std::nullopt;
    return tt->sizes().concrete_sizes();
  };
  auto x = sizes(r.x), wi = sizes(r.wih), wh = sizes(r.whh), bi = sizes(r.bih), bh = sizes(r.bhh);
  if (!x || !wi || !wh || !bi || !bh || x->size() != 3 || wi->size() != 4 || wh->size() != 4) return false;
  const int64_t B = (*x)[1], H = (*x)[2], L = (*wi)[0];
  if (B > INT32_MAX || H > INT32_MAX || L > INT32_MAX || !fx_lstm_stack_fits((int)B, (int)H, (int)L)) return false;
  const std::vector<int64_t> w{L, 4, H, H}, bias{L, 4, 1, H};
  return *wi == w && *wh == w && *bi == bias && *bh == bias;
}

// `v` is a fresh float tensor of zeros [first, x.size(1), x.size(2)]: a buffer that the loop nest
// overwrites completely (out, when `first` is the time loop's trip count) or the zero initial
// state.  The node then takes None in its place and the fill is never launched.
bool isZerosLike(Value* v, Value* first, Value* x) {
  Node* z = v->node();
  if (z->kind() != c10::aten::zeros || z->inputs().size() != 5) return false;
  Node* lc = z->input(0)->node();
  auto xt = x->type()->cast<c10::TensorType>();
  auto xs = xt ? xt->sizes().concrete_sizes() : std::nullopt;
  if (auto whole = toIValue(z->input(0))) {
    // the sizes as one constant list (static shapes folded): [first, x.size(1), x.size(2)] by value
    auto f = constant_as<int64_t>(first);
    if (!whole->isIntList() || !f || !xs || xs->size() != 3) return false;
    const auto v = whole->toIntVector();
    if (v.size() != 3 || v[0] != *f || v[1] != (*xs)[1] || v[2] != (*xs)[2]) return false;
  } else {
    if (lc->kind() != c10::prim::ListConstruct || lc->inputs().size() != 3) return false;
    auto f = constant_as<int64_t>(first);
    if (lc->input(0) != first && !(f && isConst(lc->input(0), *f))) return false;
    for (int64_t d = 1; d <= 2; ++d) {
      Value* e = lc->input((size_t)d);
      Node* en = e->node();
      const bool same_dim = en->kind() == c10::aten::size && en->inputs().size() == 2 && en->input(0) == x && isConst(en->input(1), d);
      if (!same_dim && !(xs && isConst(e, (*xs)[(size_t)d]))) return false;
    }
  }
  auto none = [](Value* a) { return a->mustBeNone(); };
  if (!none(z->input(1)) && !isConst(z->input(1), (int64_t)c10::kFloat)) return false;   // None: the default dtype, checked at run time
  if (!none(z->input(2)) || !none(z->input(4))) return false;
  Node* dn = z->input(3)->node();   // on x's device, or wherever a constant says (the kernel refuses host tensors)
  return (dn->kind() == c10::prim::device && dn->input(0) == x) || dn->kind() == c10::prim::Constant;
}

bool collapseIn(Block* b) {
  bool changed = false;
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* n = *it;
    ++it;
    LstmNest r;
    if (matchNest(n, &r) && shapesFit(r)) {
      Graph* g = b->owningGraph();
      for (Node* h : r.hoist) h->moveBefore(n);
      WithInsertPoint at(n);
      Value* none = g->insertConstant(c10::IValue());
      Value* out0 = n->input(2 + r.out_i);
      Value* h0 = n->input(2 + r.h_i);
      Value* c0 = n->input(2 + r.c_i);
      if (isZerosLike(out0, r.T, r.x)) out0 = none;
      if (isZerosLike(h0, r.L, r.x)) h0 = none;
      if (isZerosLike(c0, r.L, r.x)) c0 = none;
      Node* k = g->create(sym::LstmStack(), {r.x, r.wih, r.whh, r.bih, r.bhh, out0, h0, c0, r.T, r.L}, 3);
      k->setSourceRange(n->sourceRange());
      k->insertBefore(n);
      k->output(0)->copyMetadata(n->output(r.out_i));
      k->output(1)->copyMetadata(n->output(r.h_i));
      k->output(2)->copyMetadata(n->output(r.c_i));
      n->output(r.out_i)->replaceAllUsesWith(k->output(0));
      n->output(r.h_i)->replaceAllUsesWith(k->output(1));
      n->output(r.c_i)->replaceAllUsesWith(k->output(2));
      n->destroy();
      changed = true;
      continue;
    }
    for (Block* inner : n->blocks()) changed = collapseIn(inner) || changed;
  }
  return changed;
}

}  // namespace

bool CollapseRecurrentLoops(std::shared_ptr<Graph> graph) { return collapseIn(graph->block()); }

}  // namespace functs
