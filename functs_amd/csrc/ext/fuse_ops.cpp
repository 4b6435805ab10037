// Region formation: prim::FusionGroup, fx::forall_select_rev, prim::ParallelMap,
// masked-select folding, graph validation, pipeline driver.
//
// Grouping policy follows fait/passes/fuse_ops.cpp:209-527 (reverse greedy walk
// per block, a group needs two "working" operators, non-tensor constants stay
// outside, index-like operators only as group outputs) and
// fait/passes/parallelize_loops.cpp:12-126.
#include <iostream>
#include <torch/csrc/jit/ir/constants.h>
#include <torch/csrc/jit/passes/common_subexpression_elimination.h>
#include <torch/csrc/jit/passes/constant_propagation.h>
#include <torch/csrc/jit/passes/dead_code_elimination.h>
#include <torch/csrc/jit/passes/lower_tuples.h>

#include <functional>
#include <unordered_map>
#include <unordered_set>

#include <torch/csrc/jit/passes/remove_mutation.h>

#include "passes.h"
#include "symbols.h"

namespace functs {
using namespace torch::jit;

namespace {

bool isTensorValue(const Value* v) { return v->type()->kind() == c10::TypeKind::TensorType; }

const std::unordered_set<Symbol>& fusableSymbols() {
  using namespace c10;
  static const std::unordered_set<Symbol> s{
      aten::clone, aten::contiguous, aten::to, aten::zeros, aten::ones, aten::full, aten::full_like, aten::zeros_like,
      aten::ones_like, aten::arange, aten::tensor, aten::exp, aten::sigmoid, aten::tanh, aten::relu, aten::neg,
      aten::abs, aten::sqrt, aten::rsqrt, aten::log, aten::reciprocal, aten::floor, aten::ceil, aten::round,
      aten::sin, aten::cos, aten::erf, aten::triu, aten::tril, aten::clamp, aten::add, aten::sub, aten::rsub, aten::mul,
      aten::div, aten::minimum, aten::maximum, aten::pow, aten::__and__, aten::__or__, aten::__xor__,
      aten::logical_not, aten::eq, aten::ne, aten::lt, aten::le, aten::gt, aten::ge, aten::where, aten::max,
      aten::softmax, aten::select, aten::slice, aten::squeeze, aten::unsqueeze, aten::reshape, aten::view,
      aten::expand, aten::expand_as, aten::permute, aten::transpose, aten::cat, aten::stack, aten::repeat,
      aten::index, aten::size, aten::__derive_index, aten::neg,
      sym::Access(), sym::Assign(), sym::Select(), sym::SelectRev(), sym::Slice(), sym::SliceRev(),
      sym::Squeeze(), sym::Unsqueeze(), sym::View(), sym::Reshape(), sym::Permute(), sym::Expand(),
      sym::ExpandAs(), sym::Repeat(), sym::Index(), sym::ForallSelectRev()};
  return s;
}

// operators that do arithmetic or move data; a group needs two of them
// (fuse_ops.cpp:116-154, 264-273)
const std::unordered_set<Symbol>& workingSymbols() {
  using namespace c10;
  static const std::unordered_set<Symbol> s{
      aten::arange, aten::zeros, aten::to, aten::contiguous, aten::exp, aten::sigmoid, aten::tanh, aten::relu,
      aten::clamp, aten::triu, aten::tril, aten::add, aten::sub, aten::rsub, aten::mul, aten::div, aten::__and__, aten::__or__,
      aten::minimum, aten::maximum, aten::eq, aten::ne, aten::lt, aten::le, aten::gt, aten::ge, aten::where,
      aten::max, aten::softmax, aten::repeat, aten::cat, aten::stack, aten::index, aten::neg, aten::abs,
      aten::sqrt, aten::log, aten::pow, sym::Assign(), sym::Select(), sym::SelectRev(), sym::Slice(),
      sym::SliceRev(), sym::Index(), sym::ForallSelectRev()};
  return s;
}

bool isIndexLike(Node* n) { return n->kind() == c10::aten::index || n->kind() == sym::Index(); }

bool listOfFusableElems(Node* n) {
  if (n->kind() != c10::prim::ListConstruct) return false;
  auto lt = n->output()->type()->cast<c10::ListType>();
  if (!lt) return false;
  auto ek = lt->getElementType()->kind();
  if (ek == c10::TypeKind::OptionalType) {
    auto inner = lt->getElementType()->cast<c10::OptionalType>()->getElementType();
    return inner->kind() == c10::TypeKind::TensorType;
  }
  return ek == c10::TypeKind::IntType || ek == c10::TypeKind::TensorType;
}

}  // namespace

bool isFusableNode(Node* node) {
  if (listOfFusableElems(node)) return true;
  // taking a tuple of scalars apart (e.g. the (h, w) of an image in a List[Tuple[int, int]]):
  // the tuple becomes an argument of the region, its elements scalar inputs
  if (node->kind() == c10::prim::TupleUnpack) {
    for (Value* o : node->outputs()) {
      const auto k = o->type()->kind();
      if (k != c10::TypeKind::IntType && k != c10::TypeKind::FloatType && k != c10::TypeKind::BoolType) return false;
    }
    return true;
  }
  if (!fusableSymbols().count(node->kind())) return false;
  if (node->kind() != sym::ForallSelectRev() && !node->blocks().empty()) return false;
  // a region is compiled for one element type: a dtype operand that is computed at run time
  // (prim::dtype of a tensor whose type is not known) keeps its operator outside
  if (node->maybeSchema())
    for (size_t i = 0; i < node->inputs().size() && i < node->schema().arguments().size(); ++i)
      if (node->schema().arguments()[i].name() == "dtype" && node->input(i)->node()->kind() != c10::prim::Constant) return false;
  // scalar arithmetic that shares a symbol with a tensor operator stays outside
  if (node->kind() == c10::aten::add || node->kind() == c10::aten::sub || node->kind() == c10::aten::mul ||
      node->kind() == c10::aten::neg || node->kind() == c10::aten::eq || node->kind() == c10::aten::ne ||
      node->kind() == c10::aten::lt || node->kind() == c10::aten::le || node->kind() == c10::aten::gt ||
      node->kind() == c10::aten::ge || node->kind() == c10::aten::div || node->kind() == c10::aten::max ||
      node->kind() == c10::aten::pow || node->kind() == c10::aten::abs || node->kind() == c10::aten::floor ||
      node->kind() == c10::aten::ceil || node->kind() == c10::aten::round) {
    bool any_tensor = false;
    for (Value* in : node->inputs()) any_tensor = any_tensor || isTensorValue(in);
    bool int_out = node->output(0)->type()->kind() == c10::TypeKind::IntType;
    if (!any_tensor && !int_out) return false;
    if (!any_tensor && int_out &&
        !(node->kind() == c10::aten::add || node->kind() == c10::aten::sub || node->kind() == c10::aten::mul ||
          node->kind() == c10::aten::neg))
      return false;
  }
  // max: the reduction along a dimension whose indices nobody reads; max(x) over everything and
  // max with used indices stay ATen's
  if (node->kind() == c10::aten::max) {
    bool any_tensor = false;
    for (Value* in : node->inputs()) any_tensor = any_tensor || isTensorValue(in);
    if (any_tensor && !(node->inputs().size() >= 2 && node->outputs().size() == 2 && !node->output(1)->hasUses() &&
                        !isTensorValue(node->input(1))))
      return false;
  }
  // bool-mask indexing is data dependent: never inside a group (it is folded in
  // afterwards by FuseMaskedSelect when possible)
  if (isIndexLike(node)) {
    Node* list = node->input(1)->node();
    if (list->kind() != c10::prim::ListConstruct || list->inputs().size() != 1) return false;
    auto tt = list->input(0)->type()->cast<c10::TensorType>();
    if (!tt || !tt->scalarType() || *tt->scalarType() != c10::kLong) return false;
  }
  return true;
}

namespace {

// ---------------------------------------------------------------------------
// FuseOps
// ---------------------------------------------------------------------------
struct Group {
  std::vector<Node*> nodes;  // program order
};

void groupInOut(const std::vector<Node*>& nodes, std::vector<Value*>& inputs, std::vector<Value*>& outputs) {
  std::unordered_set<Node*> in_group(nodes.begin(), nodes.end());
  std::function<void(Node*)> scanInputs = [&](Node* n) {
    for (Value* v : n->inputs()) {
      Node* def = v->node();
      if (in_group.count(def)) continue;
      // non-tensor constants are re-created inside the group (fuse_ops.cpp:290-294)
      if (def->kind() == c10::prim::Constant && !isTensorValue(v)) continue;
      if (std::find(inputs.begin(), inputs.end(), v) == inputs.end()) inputs.push_back(v);
    }
  };
  for (Node* n : nodes) {
    scanInputs(n);
    for (Value* o : n->outputs()) {
      bool outside = false;
      for (const Use& u : o->uses()) outside = outside || !in_group.count(u.user);
      if (outside) outputs.push_back(o);
    }
  }
}

Node* commitGroup(const std::vector<Node*>& nodes, Node* insertBefore) {
  Graph* g = insertBefore->owningGraph();
  std::vector<Value*> inputs, outputs;
  groupInOut(nodes, inputs, outputs);
  Node* fusion = g->create(c10::prim::FusionGroup, inputs, 0);
  fusion->insertBefore(insertBefore);
  Block* body = fusion->addBlock();
  std::unordered_map<Value*, Value*> map;
  for (Value* in : inputs) map[in] = body->addInput()->setType(in->type());
  auto env = [&](Value* v) -> Value* {
    auto it = map.find(v);
    if (it != map.end()) return it->second;
    if (v->node()->kind() == c10::prim::Constant) {
      Node* c = g->createClone(v->node(), [](Value* x) { return x; });
      body->prependNode(c);
      map[v] = c->output();
      return c->output();
    }
    TORCH_CHECK(false, "FuseOps: value %", v->debugName(), " escapes the group");
  };
  for (Node* n : nodes) {
    Node* c = g->createClone(n, env);
    body->appendNode(c);
    for (size_t i = 0; i < n->outputs().size(); ++i) map[n->output(i)] = c->output(i);
  }
  for (Value* out : outputs) {
    Value* go = fusion->addOutput()->setType(out->type());
    body->registerOutput(map.at(out));
    out->replaceAllUsesAfterNodeWith(fusion, go);
  }
  for (auto it = nodes.rbegin(); it != nodes.rend(); ++it) (*it)->destroy();
  return fusion;
}

bool worthFusing(const std::vector<Node*>& nodes) {
  size_t working = 0;
  static const std::unordered_set<Symbol> comparisons{c10::aten::gt, c10::aten::ge, c10::aten::lt, c10::aten::le, c10::aten::eq, c10::aten::ne};
  for (Node* n : nodes) {
    if (n->kind() == sym::ForallSelectRev()) working += 2;
    else working += workingSymbols().count(n->kind());
    // A comparison whose result is the mask of x[mask] selections behind the group: the group
    // becomes a row compaction (FuseMaskedSelect), which outside a region is a nonzero with its
    // host synchronisation plus a gather per selection.
    if (comparisons.count(n->kind()) && isTensorValue(n->output()))
      for (const Use& u : n->output()->uses())
        if (u.user->kind() == c10::prim::ListConstruct && u.user->inputs().size() == 1)
          for (const Use& lu : u.user->output()->uses())
            if (isIndexLike(lu.user) && lu.offset == 1) working += 1;
  }
  if (working < 2) return false;
  // a region takes its device from its tensor arguments: fills over constant shapes alone stay eager
  std::vector<Value*> inputs, outputs;
  groupInOut(nodes, inputs, outputs);
  for (Value* in : inputs) {
    if (isTensorValue(in)) return true;
    if (auto lt = in->type()->cast<c10::ListType>())
      if (lt->getElementType()->kind() == c10::TypeKind::TensorType) return true;
  }
  return false;
}

// Reverse greedy sweeps (fuse_ops.cpp:364-425): starting at the end of the block,
// fusable nodes are pulled down next to the group being grown as long as nothing
// in between uses their results; a node that cannot join leaves the window where
// it is.  When a sweep ends the group is committed (if worth it) and the next
// sweep starts above it.
Node* liftTo(Block* block, Node* n) {
  while (n && n->owningBlock() != block) n = n->owningBlock() ? n->owningBlock()->owningNode() : nullptr;
  return n;
}

// A pure consumer that sits above the window and feeds nothing in it can step
// aside: it moves below the window, so that the producers above it can still
// join the group (e.g. `x[keep]` between two halves of one decode chain).
bool canSink(Node* n, Node* sink_point, Block* block) {
  if (!n->blocks().empty() || n->hasSideEffects() || n->kind() == c10::prim::Constant) return false;
  const bool container = n->kind() == c10::prim::ListConstruct || n->kind() == c10::prim::TupleConstruct;
  if (!container) {
    const auto* schema = n->maybeSchema();
    if (!schema || schema->is_mutable()) return false;
  }
  for (Value* o : n->outputs())
    for (const Use& u : o->uses()) {
      Node* lifted = liftTo(block, u.user);
      if (!lifted) return false;
      if (lifted != sink_point && !lifted->isAfter(sink_point)) return false;
    }
  return true;
}

void fuseBlock(Block* block, bool force_group) {
  Node* tail = block->return_node();
  for (;;) {
    std::vector<Node*> group;          // collected in reverse program order
    std::unordered_set<Node*> members;
    std::unordered_set<Node*> wanted;  // producers of values a member reads
    Node* head = tail;                 // the group occupies [head, sink_point)
    Node* sink_point = tail;           // nodes that stepped aside occupy [sink_point, tail)
    bool stayed = false;               // a foreign node was left in place above the window
    for (Node* n = tail->prev(); n != block->param_node();) {
      Node* prev = n->prev();
      const bool empty = group.empty();
      bool ok = n->kind() != c10::prim::Constant && isFusableNode(n);
      const bool is_out = !wanted.count(n);
      if (ok) {
        for (Value* o : n->outputs()) {
          bool used_outside = false;
          for (const Use& u : o->uses()) used_outside = used_outside || !members.count(u.user);
          // group outputs must be tensors (fuse_ops.cpp:232-240)
          if (used_outside && !isTensorValue(o)) ok = false;
        }
        if (!is_out && isIndexLike(n)) ok = false;  // only as a group output (fuse_ops.cpp:205-207)
      }
      if (ok) {
        // the node moves down to the group: nothing in between may use its results
        for (Value* o : n->outputs())
          for (const Use& u : o->uses())
            if (!members.count(u.user)) {
              Node* lifted = liftTo(block, u.user);
              if (lifted && lifted->isBefore(head)) ok = false;
            }
      }
      if (!ok) {
        if (empty) {
          tail = n;
          head = n;
          sink_point = n;
        } else if (!stayed && canSink(n, sink_point, block)) {
          n->moveBefore(sink_point);
          sink_point = n;
        } else if (n->kind() != c10::prim::Constant) {
          stayed = true;
        }
        n = prev;
        continue;
      }
      for (Value* in : n->inputs()) wanted.insert(in->node());
      n->moveBefore(head);
      head = n;
      members.insert(n);
      group.push_back(n);
      n = prev;
    }
    if (group.empty()) return;
    std::vector<Node*> ordered(group.rbegin(), group.rend());
    tail = (worthFusing(ordered) || force_group) ? commitGroup(ordered, sink_point) : head;
  }
}

void collectBlocks(Block* b, std::vector<Block*>& out) {
  out.push_back(b);
  for (Node* n : b->nodes()) {
    if (n->kind() == c10::prim::FusionGroup || n->kind() == sym::ForallSelectRev()) continue;
    for (Block* inner : n->blocks()) collectBlocks(inner, out);
  }
}

}  // namespace

void FuseOps(std::shared_ptr<Graph> graph) {
  std::vector<Block*> blocks;
  collectBlocks(graph->block(), blocks);
  for (Block* b : blocks) {
    // a ParallelMap body that is fusable throughout is fused as a whole, whatever its size
    // (one launch instead of a loop); a mixed body follows the ordinary rule, so that a lone
    // view next to an unfusable operator does not become a launch of its own
    bool whole_map = b->owningNode() && b->owningNode()->kind() == sym::ParallelMap();
    if (whole_map)
      for (Node* n : b->nodes())
        whole_map = whole_map && (n->kind() == c10::prim::Constant || isFusableNode(n) || isIndexLike(n));
    fuseBlock(b, whole_map);
  }
}

// ---------------------------------------------------------------------------
// CollapseAssignLoops
// ---------------------------------------------------------------------------
namespace {

bool tryCollapse(Node* loop) {
  // prim::Loop(trip, cond, T0) { block(i, T) ... -> (cond', Tn) }
  if (loop->inputs().size() != 3 || loop->outputs().size() != 1) return false;
  Block* body = loop->blocks()[0];
  auto condc = toIValue(loop->input(1));
  auto nextc = toIValue(body->outputs()[0]);
  if (!condc || !condc->isBool() || !condc->toBool() || !nextc || !nextc->isBool() || !nextc->toBool()) return false;
  Value* i = body->inputs()[0];
  Value* T = body->inputs()[1];
  if (!isTensorValue(T)) return false;
  Node* rev = body->outputs()[1]->node();
  if (rev->kind() != sym::SelectRev() || rev->owningBlock() != body || rev->input(0) != T || rev->input(3) != i)
    return false;
  auto dim = constant_as<int64_t>(rev->input(2));
  if (!dim) return false;
  // every other use of T must be immut::select(T, dim, i)
  for (const Use& u : T->uses()) {
    if (u.user == rev) continue;
    if (u.user->kind() != sym::Select() || u.offset != 0 || u.user->input(2) != i) return false;
    auto d2 = constant_as<int64_t>(u.user->input(1));
    if (!d2 || *d2 != *dim) return false;
  }
  // the body must be straight-line fusable code
  for (Node* n : body->nodes()) {
    if (n->kind() == c10::prim::Constant) continue;
    if (!isFusableNode(n)) return false;
  }
  Graph* g = loop->owningGraph();
  WithInsertPoint guard(loop);
  Value* zero = g->insertConstant((int64_t)0);
  // captured outer values become explicit inputs
  std::vector<Value*> captured;
  for (Node* n : body->nodes())
    for (Value* v : n->inputs())
      if (v->node()->owningBlock() != body && v != i && v != T && v->node()->kind() != c10::prim::Constant &&
          std::find(captured.begin(), captured.end(), v) == captured.end())
        captured.push_back(v);
  std::vector<Value*> inputs{loop->input(2), rev->input(2), zero, loop->input(0)};
  inputs.insert(inputs.end(), captured.begin(), captured.end());
  Node* forall = g->create(sym::ForallSelectRev(), inputs, 1);
  forall->output()->setType(loop->output(0)->type());
  forall->setSourceRange(loop->sourceRange());
  forall->insertBefore(loop);
  Block* fb = forall->addBlock();
  std::unordered_map<Value*, Value*> map;
  map[i] = fb->addInput()->setType(i->type());
  map[T] = fb->addInput()->setType(T->type());
  for (Value* c : captured) map[c] = fb->addInput()->setType(c->type());
  auto env = [&](Value* v) -> Value* {
    auto it = map.find(v);
    if (it != map.end()) return it->second;
    if (v->node()->kind() == c10::prim::Constant) {
      Node* c = g->createClone(v->node(), [](Value* x) { return x; });
      fb->prependNode(c);
      map[v] = c->output();
      return c->output();
    }
    TORCH_CHECK(false, "CollapseAssignLoops: unexpected free value");
  };
  for (Node* n : body->nodes()) {
    if (n == rev) continue;
    Node* c = g->createClone(n, env);
    fb->appendNode(c);
    for (size_t k = 0; k < n->outputs().size(); ++k) map[n->output(k)] = c->output(k);
  }
  fb->registerOutput(env(rev->input(1)));
  loop->output(0)->replaceAllUsesWith(forall->output());
  loop->destroy();
  return true;
}

void collapseIn(Block* b) {
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* n = *it;
    ++it;
    for (Block* inner : n->blocks()) collapseIn(inner);
    if (n->kind() == c10::prim::Loop) tryCollapse(n);
  }
}

}  // namespace

void CollapseAssignLoops(std::shared_ptr<Graph> graph) { collapseIn(graph->block()); }

// ---------------------------------------------------------------------------
// ParallelizeLoops
// ---------------------------------------------------------------------------
namespace {

bool tryParallelize(Node* loop) {
  if (loop->inputs().size() != 2 || !loop->outputs().empty()) return false;  // carried values: parallelize_loops.cpp:17
  Block* body = loop->blocks()[0];
  auto condc = toIValue(loop->input(1));
  auto nextc = toIValue(body->outputs()[0]);
  if (!condc || !condc->isBool() || !condc->toBool() || !nextc || !nextc->isBool() || !nextc->toBool()) return false;
  Value* i = body->inputs()[0];
  std::vector<Node*> reads, appends;
  bool any_fusable = false;
  for (Node* n : body->nodes()) {
    if (n->kind() == c10::prim::Constant) continue;
    if (n->kind() == c10::aten::__getitem__ && n->input(0)->type()->cast<c10::ListType>()) {
      // list reads must be list[i] on a list defined outside (parallelize_loops.cpp:33-41)
      if (n->input(1) != i || n->input(0)->node()->owningBlock() == body) return false;
      reads.push_back(n);
      continue;
    }
    if (n->kind() == c10::aten::append) {
      Node* def = n->input(0)->node();
      if (def->owningBlock() == body || def->kind() != c10::prim::ListConstruct || !def->inputs().empty()) return false;
      // exactly one append per output list, nothing else touches the list in the loop
      for (Node* a : appends) if (a->input(0) == n->input(0)) return false;
      if (!n->output()->uses().empty()) return false;
      appends.push_back(n);
      continue;
    }
    if (!n->blocks().empty()) return false;
    if (isFusableNode(n) || isIndexLike(n)) {
      any_fusable = any_fusable || n->kind() != c10::prim::ListConstruct;
      continue;
    }
    // anything else without effects may stay: SplitParallelMaps gives the fusable stretches
    // maps of their own and the rest returns to a loop (parallelize_loops.cpp:152-362)
    if (n->hasSideEffects()) return false;
    if (const auto* schema = n->maybeSchema())
      if (schema->is_mutable()) return false;
  }
  if (appends.empty() || !any_fusable) return false;
  // output lists: defined right before use, only appended to inside this loop
  for (Node* a : appends)
    for (const Use& u : a->input(0)->uses())
      if (u.user != a && u.user->isBefore(loop)) return false;

  Graph* g = loop->owningGraph();
  std::vector<Value*> args{loop->input(0)};
  for (Node* r : reads)
    if (std::find(args.begin() + 1, args.end(), r->input(0)) == args.end()) args.push_back(r->input(0));
  Node* map = g->create(sym::ParallelMap(), args, appends.size());
  map->setSourceRange(loop->sourceRange());
  map->insertAfter(loop);
  Block* mb = map->addBlock();
  std::unordered_map<Value*, Value*> vm;
  vm[i] = mb->addInput()->setType(i->type());
  std::vector<Value*> elem_params;
  for (size_t k = 1; k < args.size(); ++k) {
    auto lt = args[k]->type()->cast<c10::ListType>();
    elem_params.push_back(mb->addInput()->setType(lt->getElementType()));
  }
  auto env = [&](Value* v) -> Value* {
    auto it = vm.find(v);
    return it != vm.end() ? it->second : v;  // outer values stay visible inside the block
  };
  for (Node* n : body->nodes()) {
    if (n->kind() == c10::aten::__getitem__ && std::find(reads.begin(), reads.end(), n) != reads.end()) {
      size_t k = std::find(args.begin() + 1, args.end(), n->input(0)) - args.begin();
      vm[n->output()] = elem_params[k - 1];
      continue;
    }
    if (n->kind() == c10::aten::append) continue;
    Node* c = g->createClone(n, env);
    mb->appendNode(c);
    for (size_t k = 0; k < n->outputs().size(); ++k) vm[n->output(k)] = c->output(k);
  }
  for (size_t k = 0; k < appends.size(); ++k) {
    mb->registerOutput(env(appends[k]->input(1)));
    Value* out_list = appends[k]->input(0);
    map->output(k)->setType(out_list->type());
    out_list->replaceAllUsesAfterNodeWith(loop, map->output(k));
  }
  std::vector<Node*> list_defs;
  for (Node* a : appends) list_defs.push_back(a->input(0)->node());
  loop->destroy();
  for (Node* d : list_defs)
    if (!d->hasUses()) d->destroy();
  return true;
}

void parallelizeIn(Block* b) {
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* n = *it;
    ++it;
    for (Block* inner : n->blocks()) parallelizeIn(inner);
    if (n->kind() == c10::prim::Loop) tryParallelize(n);
  }
}

}  // namespace

void ParallelizeLoops(std::shared_ptr<Graph> graph) { parallelizeIn(graph->block()); }

// ---------------------------------------------------------------------------
// FuseMaskedSelect
// ---------------------------------------------------------------------------
namespace {

// true when `v` (a value inside a group body) is certainly a bool tensor
bool producesBoolMask(Value* v, int depth = 0) {
  static const std::unordered_set<Symbol> cmp{c10::aten::gt, c10::aten::ge, c10::aten::lt,
                                              c10::aten::le, c10::aten::eq, c10::aten::ne, c10::aten::logical_not};
  auto tt = v->type()->cast<c10::TensorType>();
  if (tt && tt->scalarType()) return *tt->scalarType() == c10::kBool;
  Node* n = v->node();
  if (cmp.count(n->kind())) return true;
  if ((n->kind() == c10::aten::__and__ || n->kind() == c10::aten::__or__) && depth < 8)
    return producesBoolMask(n->input(0), depth + 1) && producesBoolMask(n->input(1), depth + 1);
  return false;
}

// group(...) -> (.., x, .., m);  x[m] for every other output x, and y[m] for values y
// that exist before the group  ==>  group[compact_rows](..., y) -> (.., x', .., y')
// with m as the last block output.
bool foldMaskedSelect(Node* group) {
  if (group->hasAttribute(sym::compact_rows())) return false;
  Block* body = group->blocks()[0];
  for (size_t mi = 0; mi < group->outputs().size(); ++mi) {
    Value* m = group->output(mi);
    if (!isTensorValue(m) || !producesBoolMask(body->outputs()[mi])) continue;
    // the mask is used only as the single entry of index lists
    std::vector<Node*> index_nodes;
    bool ok = !m->uses().empty();
    for (const Use& u : m->uses()) {
      Node* list = u.user;
      if (list->kind() != c10::prim::ListConstruct || list->inputs().size() != 1) { ok = false; break; }
      for (const Use& lu : list->output()->uses()) {
        if (!isIndexLike(lu.user) || lu.offset != 1) { ok = false; break; }
        index_nodes.push_back(lu.user);
      }
      if (!ok) break;
    }
    if (!ok || index_nodes.empty()) continue;
    std::unordered_map<Value*, std::vector<Node*>> selects;  // indexed value -> its index nodes
    std::vector<Value*> order;
    for (Node* ix : index_nodes) {
      Value* x = ix->input(0);
      if (x->node() != group) {
        // a value from outside joins as a pass-through; it has to exist where the group stands
        Node* def = x->node();
        if (!isTensorValue(x)) { ok = false; break; }
        if (def->owningBlock() == group->owningBlock() && !def->isBefore(group)) { ok = false; break; }
        if (def->owningBlock() != group->owningBlock()) {
          Node* lifted = liftTo(def->owningBlock(), group);
          if (!lifted || !def->isBefore(lifted)) { ok = false; break; }
        }
      }
      if (!selects.count(x)) order.push_back(x);
      selects[x].push_back(ix);
    }
    if (!ok) continue;
    // every other output must be consumed only as x[m]
    for (size_t k = 0; k < group->outputs().size() && ok; ++k) {
      Value* o = group->output(k);
      if (o == m) continue;
      if (!selects.count(o)) { ok = false; break; }
      for (const Use& u : o->uses())
        if (std::find(selects[o].begin(), selects[o].end(), u.user) == selects[o].end()) ok = false;
    }
    if (!ok) continue;
    for (Value* x : order) {
      Value* target = x;
      if (x->node() != group) {
        group->addInput(x);
        Value* p = body->addInput()->setType(x->type());
        body->registerOutput(p);
        target = group->addOutput();
      }
      for (Node* ix : selects[x]) {
        target->setType(ix->output()->type());
        ix->output()->replaceAllUsesWith(target);
      }
    }
    for (Node* ix : index_nodes) {
      Node* list = ix->input(1)->node();
      ix->destroy();
      if (!list->hasUses()) list->destroy();
    }
    Value* mask_inner = body->outputs()[mi];
    body->eraseOutput(mi);
    group->eraseOutput(mi);
    body->registerOutput(mask_inner);
    group->i_(sym::compact_rows(), 1);
    return true;
  }
  return false;
}

void collectGroups(Block* b, std::vector<Node*>& out) {
  for (Node* n : b->nodes()) {
    if (n->kind() == c10::prim::FusionGroup) out.push_back(n);
    else for (Block* inner : n->blocks()) collectGroups(inner, out);
  }
}

void foldIn(Block* b) {
  std::vector<Node*> groups;  // folding destroys neighbouring nodes: no live iterators
  collectGroups(b, groups);
  for (Node* g : groups) foldMaskedSelect(g);
}

}  // namespace

void FuseMaskedSelect(std::shared_ptr<Graph> graph) { foldIn(graph->block()); }

// ---------------------------------------------------------------------------
// UnrollLoopsWithDeps (fait/passes/unroll_loops.cpp:11-77) and UnrollSimpleMaps
// (fait/passes/parallelize_loops.cpp:372-456): short loops with carried values whose body did
// not fuse, and maps that only compute from their own parameters and constants, are written
// out; the second FuseOps then fuses across what were iterations.
// ---------------------------------------------------------------------------
namespace {

constexpr int64_t kMaxUnroll = 64;  // the reference has no limit; a long loop stays a loop here

bool bodyIsFlat(Block* body) {
  for (Node* n : body->nodes()) {
    if (!n->blocks().empty() || n->kind() == c10::prim::FusionGroup || n->kind() == sym::ParallelMap() ||
        n->kind() == sym::ForallSelectRev())
      return false;
    if (n->hasSideEffects()) return false;
  }
  return true;
}

void cloneBodyBefore(Block* body, Node* before, std::unordered_map<Value*, Value*>& vm) {
  Graph* g = before->owningGraph();
  auto env = [&](Value* v) -> Value* {
    auto it = vm.find(v);
    return it != vm.end() ? it->second : v;
  };
  for (Node* n : body->nodes()) {
    Node* c = g->createClone(n, env);
    c->insertBefore(before);
    for (size_t k = 0; k < n->outputs().size(); ++k) vm[n->output(k)] = c->output(k);
  }
}

bool tryUnrollLoop(Node* loop) {
  if (loop->inputs().size() <= 2) return false;   // no carried values: ParallelizeLoops' business
  auto trip = constant_as<int64_t>(loop->input(0));
  auto cond = constant_as<bool>(loop->input(1));
  Block* body = loop->blocks()[0];
  auto next = constant_as<bool>(body->outputs()[0]);
  if (!trip || *trip < 0 || *trip > kMaxUnroll || !cond || !*cond || !next || !*next) return false;
  if (!bodyIsFlat(body)) return false;
  Graph* g = loop->owningGraph();
  WithInsertPoint guard(loop);
  std::vector<Value*> carried(loop->inputs().begin() + 2, loop->inputs().end());
  for (int64_t i = 0; i < *trip; ++i) {
    std::unordered_map<Value*, Value*> vm;
    vm[body->inputs()[0]] = g->insertConstant(i);
    for (size_t k = 0; k < carried.size(); ++k) vm[body->inputs()[k + 1]] = carried[k];
    cloneBodyBefore(body, loop, vm);
    for (size_t k = 0; k < carried.size(); ++k) {
      Value* r = body->outputs()[k + 1];
      auto it = vm.find(r);
      carried[k] = it != vm.end() ? it->second : r;
    }
  }
  for (size_t k = 0; k < carried.size(); ++k) loop->output(k)->replaceAllUsesWith(carried[k]);
  loop->destroy();
  return true;
}

bool tryUnrollMap(Node* map) {
  auto trip = constant_as<int64_t>(map->input(0));
  if (!trip || *trip < 0 || *trip > kMaxUnroll) return false;
  Block* body = map->blocks()[0];
  if (!bodyIsFlat(body)) return false;
  for (Node* n : body->nodes())
    for (Value* in : n->inputs())
      if (in->node()->kind() != c10::prim::Constant && in->node()->owningBlock() != body) return false;
  Graph* g = map->owningGraph();
  WithInsertPoint guard(map);
  std::vector<std::vector<Value*>> outs(map->outputs().size());
  for (int64_t i = 0; i < *trip; ++i) {
    std::unordered_map<Value*, Value*> vm;
    Value* idx = g->insertConstant(i);
    vm[body->inputs()[0]] = idx;
    for (size_t k = 1; k < map->inputs().size(); ++k) {
      Node* get = g->create(c10::aten::__getitem__, {map->input(k), idx}, 1);
      get->output()->setType(body->inputs()[k]->type());
      g->insertNode(get);
      vm[body->inputs()[k]] = get->output();
    }
    cloneBodyBefore(body, map, vm);
    for (size_t k = 0; k < outs.size(); ++k) {
      Value* r = body->outputs()[k];
      auto it = vm.find(r);
      outs[k].push_back(it != vm.end() ? it->second : r);
    }
  }
  for (size_t k = 0; k < outs.size(); ++k) {
    auto lt = map->output(k)->type()->cast<c10::ListType>();
    Node* lc = g->createList(lt->getElementType(), outs[k]);
    g->insertNode(lc);
    lc->output()->setType(map->output(k)->type());
    map->output(k)->replaceAllUsesWith(lc->output());
  }
  map->destroy();
  return true;
}

bool unrollIn(Block* b, bool maps) {
  bool changed = false;
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* n = *it;
    ++it;
    for (Block* inner : n->blocks()) changed = unrollIn(inner, maps) || changed;
    if (!maps && n->kind() == c10::prim::Loop) changed = tryUnrollLoop(n) || changed;
    if (maps && n->kind() == sym::ParallelMap()) changed = tryUnrollMap(n) || changed;
  }
  return changed;
}

}  // namespace

// A short loop over the elements of list arguments whose example elements differ in shape (the
// levels of a feature pyramid): inside a loop or a map the elements have no static shape, written
// out every level has its own (fait/passes/refine_types.cpp:57-81 keeps the per-element types for
// exactly this; the reference's detection heads walk their levels with such loops,
// yolov3_bbox.py:209-216).  Appends to lists are kept in order; RemoveListMutation turns them into
// list constructions afterwards.
bool readsRaggedList(Block* body) {
  for (Node* n : body->nodes()) {
    if (n->kind() != c10::aten::__getitem__) continue;
    auto it = refinedTypes().find(n->input(0));
    if (it == refinedTypes().end()) continue;
    const auto& elems = it->second->expectRef<c10::TupleType>().elements();
    for (const auto& e : elems)
      if (*e != *elems[0]) return true;
  }
  return false;
}

bool tryUnrollRagged(Node* loop) {
  auto trip = constant_as<int64_t>(loop->input(0));
  auto cond = constant_as<bool>(loop->input(1));
  Block* body = loop->blocks()[0];
  auto next = constant_as<bool>(body->outputs()[0]);
  if (!trip || *trip < 0 || *trip > 8 || !cond || !*cond || !next || !*next) return false;
  for (Node* n : body->nodes()) {
    if (!n->blocks().empty()) return false;
    if (n->hasSideEffects() && n->kind() != c10::aten::append) return false;
  }
  if (!readsRaggedList(body)) return false;
  // Only where the levels are joined afterwards (every list the body appends to is read by cat /
  // stack alone): what follows then needs the shapes of all levels.  Levels whose results stay
  // apart are independent tasks of different shapes: a map runs them in one launch.
  bool appends = false;
  for (Node* n : body->nodes()) {
    if (n->kind() != c10::aten::append) continue;
    appends = true;
    for (const Use& u : n->input(0)->uses()) {
      if (u.user == n) continue;
      if (u.user->kind() != c10::aten::cat && u.user->kind() != c10::aten::stack) return false;
    }
  }
  if (!appends) return false;
  Graph* g = loop->owningGraph();
  WithInsertPoint guard(loop);
  std::vector<Value*> carried(loop->inputs().begin() + 2, loop->inputs().end());
  for (int64_t i = 0; i < *trip; ++i) {
    std::unordered_map<Value*, Value*> vm;
    vm[body->inputs()[0]] = g->insertConstant(i);
    for (size_t k = 0; k < carried.size(); ++k) vm[body->inputs()[k + 1]] = carried[k];
    cloneBodyBefore(body, loop, vm);
    for (size_t k = 0; k < carried.size(); ++k) {
      Value* r = body->outputs()[k + 1];
      auto it = vm.find(r);
      carried[k] = it != vm.end() ? it->second : r;
    }
  }
  for (size_t k = 0; k < carried.size(); ++k) loop->output(k)->replaceAllUsesWith(carried[k]);
  loop->destroy();
  return true;
}

bool UnrollRaggedListLoops(std::shared_ptr<Graph> graph) {
  bool changed = false;
  Block* b = graph->block();
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* n = *it;
    ++it;
    if (n->kind() == c10::prim::Loop) changed = tryUnrollRagged(n) || changed;
  }
  return changed;
}

bool UnrollLoopsWithDeps(std::shared_ptr<Graph> graph) { return unrollIn(graph->block(), false); }
bool UnrollSimpleMaps(std::shared_ptr<Graph> graph) { return unrollIn(graph->block(), true); }

// ---------------------------------------------------------------------------
// SplitParallelMaps (fait/passes/parallelize_loops.cpp:152-293): a map whose body holds
// fusion groups next to other nodes is cut so that every group is alone in a map (one launch
// for all tasks); what lies between the groups gets maps of its own, which ToParallelFunctor
// turns back into loops.  A value that crosses a cut travels as a list with one element per task.
// ---------------------------------------------------------------------------
namespace {

bool splitMap(Node* map) {
  Graph* g = map->owningGraph();
  Block* mb = map->blocks()[0];
  // constants are free: they move in front of the map and stay visible to every part
  for (auto it = mb->nodes().begin(); it != mb->nodes().end();) {
    Node* n = *it;
    ++it;
    if (n->kind() == c10::prim::Constant) n->moveBefore(map);
  }
  std::vector<std::vector<Node*>> segs;
  bool prev_group = false, any_group = false;
  for (Node* n : mb->nodes()) {
    const bool is_group = n->kind() == c10::prim::FusionGroup;
    any_group = any_group || is_group;
    if (segs.empty() || is_group || prev_group) segs.emplace_back();
    segs.back().push_back(n);
    prev_group = is_group;
  }
  if (!any_group || segs.size() < 2) return false;

  struct Part {
    Node* map = nullptr;
    Block* block = nullptr;
    std::unordered_map<Value*, Value*> vm;       // value of the old body -> value in this part
    std::unordered_map<Value*, Value*> exported; // value of the old body -> list output of this part
  };
  std::vector<Part> parts(segs.size());
  std::unordered_map<Value*, size_t> def_part;   // value of the old body -> part that computes it

  auto exportValue = [&](size_t t, Value* v) -> Value* {
    Part& T = parts[t];
    auto it = T.exported.find(v);
    if (it != T.exported.end()) return it->second;
    T.block->registerOutput(T.vm.at(v));
    Value* list = T.map->addOutput()->setType(c10::ListType::create(v->type()));
    T.exported[v] = list;
    return list;
  };
  std::function<Value*(size_t, Value*)> resolve = [&](size_t s, Value* v) -> Value* {
    Part& P = parts[s];
    auto it = P.vm.find(v);
    if (it != P.vm.end()) return it->second;
    auto pos = std::find(mb->inputs().begin() + 1, mb->inputs().end(), v);
    Value* list = nullptr;
    if (pos != mb->inputs().end()) {
      list = map->input(pos - mb->inputs().begin());      // element of one of the map's own lists
    } else {
      auto d = def_part.find(v);
      if (d == def_part.end()) return v;                  // defined outside the map
      list = exportValue(d->second, v);
    }
    P.map->addInput(list);
    Value* param = P.block->addInput()->copyMetadata(v);
    P.vm[v] = param;
    return param;
  };

  Node* prev = map;
  for (size_t s = 0; s < segs.size(); ++s) {
    Part& P = parts[s];
    P.map = g->create(sym::ParallelMap(), {map->input(0)}, 0);
    P.map->setSourceRange(map->sourceRange());
    P.map->insertAfter(prev);
    prev = P.map;
    P.block = P.map->addBlock();
    P.vm[mb->inputs()[0]] = P.block->addInput()->setType(c10::IntType::get());
    for (Node* n : segs[s]) {
      Node* c = g->createClone(n, [&](Value* v) { return resolve(s, v); });
      P.block->appendNode(c);
      for (size_t k = 0; k < n->outputs().size(); ++k) {
        P.vm[n->output(k)] = c->output(k);
        def_part[n->output(k)] = s;
      }
    }
  }
  for (size_t k = 0; k < map->outputs().size(); ++k) {
    Value* r = mb->outputs()[k];
    auto d = def_part.find(r);
    Value* list;
    if (d != def_part.end()) {
      list = exportValue(d->second, r);
    } else {  // an element of an input list or an outer value handed through: the first part returns it
      Part& P = parts[0];
      P.block->registerOutput(resolve(0, r));
      list = P.map->addOutput();
    }
    list->setType(map->output(k)->type());
    map->output(k)->replaceAllUsesWith(list);
  }
  map->destroy();
  return true;
}

void splitIn(Block* b) {
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* n = *it;
    ++it;
    for (Block* inner : n->blocks()) splitIn(inner);
    if (n->kind() == sym::ParallelMap()) splitMap(n);
  }
}

}  // namespace

void SplitParallelMaps(std::shared_ptr<Graph> graph) { splitIn(graph->block()); }

// ---------------------------------------------------------------------------
// CanonicalizeFusableMaps (fait/passes/parallelize_loops.cpp:458-502): a map whose body is one
// fusion group takes the group's arguments in one order, whatever the order in which the body
// used them: the map index first (added when the body does not use it), then the map's own
// parameters in their order, then what the group takes from outside; the map returns the group's
// results in the group's order.
// ---------------------------------------------------------------------------
namespace {
void canonicalizeMapsIn(Block* b) {
  for (Node* n : b->nodes()) {
    for (Block* inner : n->blocks()) canonicalizeMapsIn(inner);
    if (n->kind() != sym::ParallelMap()) continue;
    Block* mb = n->blocks()[0];
    if (mb->nodes().begin() == mb->nodes().end()) continue;
    Node* group = *mb->nodes().begin();
    if (group->kind() != prim::FusionGroup || group->blocks().empty()) continue;
    Block* gb = group->blocks()[0];
    // every parameter of the map is one argument of the group, and nothing else uses it
    bool plain = true;
    for (Value* p : mb->inputs()) {
      if (p == mb->inputs()[0] && !p->hasUses()) continue;
      plain = plain && p->uses().size() == 1 && p->uses()[0].user == group;
    }
    if (!plain) continue;
    std::vector<size_t> perm;
    Value* index = mb->inputs()[0];
    if (index->hasUses()) {
      perm.push_back(index->uses()[0].offset);
    } else {
      group->insertInput(0, index);
      gb->insertInput(0)->setType(c10::IntType::get());
      perm.push_back(0);
    }
    for (size_t k = 1; k < mb->inputs().size(); ++k) perm.push_back(mb->inputs()[k]->uses()[0].offset);
    for (size_t k = 0; k < group->inputs().size(); ++k)
      if (!std::count(perm.begin(), perm.end(), k)) perm.push_back(k);
    group->permuteInputs(perm);
    gb->permuteInputs(perm);
    // results: only when every result of the group is returned once by the map (a group that
    // compacts rows keeps its row mask to itself)
    std::vector<size_t> ret;
    bool all_returned = group->outputs().size() == mb->outputs().size();
    for (Value* out : group->outputs()) {
      all_returned = all_returned && out->uses().size() == 1 && out->uses()[0].user == mb->return_node();
      if (all_returned) ret.push_back(out->uses()[0].offset);
    }
    if (all_returned) {
      mb->permuteOutputs(ret);
      n->permuteOutputs(ret);
    }
  }
}
}  // namespace

void CanonicalizeFusableMaps(std::shared_ptr<Graph> graph) { canonicalizeMapsIn(graph->block()); }

// ---------------------------------------------------------------------------
// Validate
// ---------------------------------------------------------------------------
namespace {
void validateIn(Block* b, std::unordered_set<const Value*>& defined) {
  for (Value* v : b->inputs()) defined.insert(v);
  for (Node* n : b->nodes()) {
    for (Value* in : n->inputs())
      TORCH_CHECK(defined.count(in), "Validate: %", in->debugName(), " is used by ", n->kind().toQualString(),
                  " before it is defined");
    for (Block* inner : n->blocks()) {
      std::unordered_set<const Value*> scope = defined;
      validateIn(inner, scope);
    }
    for (Value* o : n->outputs()) defined.insert(o);
  }
  for (Value* o : b->outputs()) TORCH_CHECK(defined.count(o), "Validate: block returns an undefined value");
}
}  // namespace

void Validate(std::shared_ptr<Graph> graph) {
  std::unordered_set<const Value*> defined;
  validateIn(graph->block(), defined);
}

// ---------------------------------------------------------------------------
// pipeline
// ---------------------------------------------------------------------------
ValueTypeMap& refinedTypes() {
  thread_local ValueTypeMap map;
  return map;
}

namespace {
// Is the list only read (indexed, measured, iterated by maps and loops)?
bool listIsOnlyRead(const Value* list) {
  for (const Use& u : list->uses()) {
    const auto* schema = u.user->maybeSchema();
    if (!schema) continue;   // prim::Loop, prim::ParallelMap, prim::If ...: lists travel through unchanged
    const auto& args = schema->arguments();
    if (u.offset < args.size() && args[u.offset].alias_info() && args[u.offset].alias_info()->isWrite()) return false;
  }
  return true;
}
struct RefinedTypesScope {
  RefinedTypesScope() { refinedTypes().clear(); }
  ~RefinedTypesScope() { refinedTypes().clear(); }
};
}  // namespace

bool FaitPipeline(std::shared_ptr<Graph> graph, std::vector<c10::TypePtr> input_types) {
  RefinedTypesScope scope;
  bool specialized = false;
  // FUNCTS_PIPELINE_TRACE=1: the graph after the region-forming stages, on stderr
  static const bool tracing = getenv("FUNCTS_PIPELINE_TRACE") && atoi(getenv("FUNCTS_PIPELINE_TRACE")) != 0;
  auto trace = [&](const char* stage) {
    if (tracing) std::cerr << "---- after " << stage << " ----\n" << graph->toString(false) << std::endl;
  };
  // RefineInputTypes (refine_types.cpp:179-195): tensor arguments take the example's type; a list
  // argument whose example is a tuple of tensors keeps the tuple type in the side table
  for (size_t i = 0; i < input_types.size() && i < graph->inputs().size(); ++i) {
    Value* in = graph->inputs()[i];
    if (!input_types[i]) continue;
    if (input_types[i]->kind() == c10::TypeKind::TensorType && isTensorValue(in)) {
      in->setType(input_types[i]);
    } else if (input_types[i]->kind() == c10::TypeKind::TupleType && in->type()->kind() == c10::TypeKind::ListType &&
               in->type()->expectRef<c10::ListType>().getElementType()->kind() == c10::TypeKind::TensorType) {
      const auto& elems = input_types[i]->expectRef<c10::TupleType>().elements();
      bool tensors = !elems.empty();
      for (const auto& e : elems) tensors = tensors && e->kind() == c10::TypeKind::TensorType;
      if (!tensors || !listIsOnlyRead(in)) continue;
      refinedTypes()[in] = input_types[i];
      // the length of the example is the length (the pipeline is specialised to the example's shapes)
      const auto uses = in->uses();
      for (const Use& u : uses) {
        if (u.user->kind() != c10::aten::len) continue;
        WithInsertPoint guard(u.user);
        u.user->output()->replaceAllUsesWith(graph->insertConstant((int64_t)elems.size()));
        u.user->destroy();
        specialized = true;
      }
    }
  }
  ConvertProfilingInstrumentation(graph);   // fait.cpp:137: range markers first, they cut regions
  LowerSimpleTuples(graph);
  if (UnrollRaggedListLoops(graph)) {
    ConstantPropagation(graph);      // list[constant] of a constant list, arithmetic on the level index
    RemoveListMutation(graph);       // the appends of what were iterations become list constructions
    specialized = true;
  }
  // InferShape + constant folding (fait_pipeline.cpp:47-49): sizes of intermediate values that
  // the program asks for (new_zeros(n, x.size(1), 1)) fold like those of the arguments; twice,
  // because a folded size is what lets the next creation operator be typed
  for (int round = 0; round < 3; ++round) {
    const bool typed = InferStaticShapes(graph);
    const bool folded = FoldStaticTypeQueries(graph);
    specialized = specialized || folded;
    ConstantPropagation(graph);
    if (!typed && !folded) break;
  }
  ConstantPropagation(graph);
  UniformConstantsToFills(graph);
  EliminateCommonSubexpression(graph);
  EliminateDeadCode(graph);
  CanonicalizeOps(graph);       // fait_pipeline.cpp:39
  HoistLoopInvariants(graph);   // parallelize_loops.cpp:130
  EliminateCommonSubexpression(graph);
  if (CollapseRecurrentLoops(graph)) EliminateDeadCode(graph);   // buffers the collapsed node no longer reads
  CollapseAssignLoops(graph);
  trace("canonicalisation");
  ParallelizeLoops(graph);
  trace("ParallelizeLoops");
  FuseOps(graph);
  trace("FuseOps");
  // what did not fuse inside short dependent loops and parameter-only maps is written out and
  // gets a second chance across iterations (fait_pipeline.cpp:52-55)
  const bool unrolled_loops = UnrollLoopsWithDeps(graph);
  const bool unrolled_maps = UnrollSimpleMaps(graph);
  if (unrolled_loops || unrolled_maps) {
    ConstantPropagation(graph);
    UniformConstantsToFills(graph);
    EliminateCommonSubexpression(graph);
    EliminateDeadCode(graph);
    FuseOps(graph);
  }
  FuseMaskedSelect(graph);
  trace("FuseMaskedSelect");
  SplitParallelMaps(graph);
  CanonicalizeFusableMaps(graph);   // fait_pipeline.cpp:61
  trace("SplitParallelMaps");
  ToParallelFunctor(graph);
  EliminateDeadCode(graph);
  trace("ToParallelFunctor");
  InferStaticShapes(graph);   // results of the functors, and the argument types of the functors behind them
  if (SinkProducersIntoMaps(graph)) {   // (folds size queries on the producer's results)
    ConstantPropagation(graph);
    UniformConstantsToFills(graph);
    EliminateDeadCode(graph);
    specialized = true;
  }
  FuseDetectionTail(graph);
  Validate(graph);
  return specialized;
}

}  // namespace functs
