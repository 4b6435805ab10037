// TensorSSA functionalization: view + mutation  ->  immut::access / immut::assign
// operators + tssa::update version markers, propagated through prim::Loop /
// prim::If, renamed by dominance, cleaned up.
//
// Behaviour follows functs/csrc/jit/passes/convert_to_tensorssa.cpp:105-481 and
// remove_inplace.cpp:20-73 (pass order, node shapes, mutValues / mutNodes
// bookkeeping; worked example README.md:64-308).  One structural difference:
// the reference reads the view relation out of a vendored copy of AliasDb's
// private element map (convert_to_tensorssa.cpp:28-103); here the view forest
// is rebuilt from the graph itself (definition chains of view operators that
// start at a freshly allocated tensor), and stock AliasDb is only asked, through
// its public interface, whether a root may alias a graph input.
#include "tensorssa.h"

#include <torch/csrc/jit/ir/alias_analysis.h>
#include <torch/csrc/jit/runtime/operator.h>

#include <deque>
#include <functional>
#include <unordered_set>

#include "symbols.h"

namespace functs {
using namespace torch::jit;

void TensorSSAMutateInfo::addMutNodes(Node* updateNode) {
  TORCH_CHECK(updateNode->kind() == sym::Update(), "mutations are recorded through tssa::update nodes");
  Value* mutated = updateNode->input(1);
  if (!mutNodes.count(mutated)) {
    mutValues.push_back(mutated);
    mutNodes.insert({mutated, {}});
  }
  mutNodes[mutated].push_back(updateNode);
}

namespace {

bool isTensor(const Value* v) { return v->type()->kind() == c10::TypeKind::TensorType; }

// does `node` write to its input `i` (a `Tensor(a!)` argument)?
bool writesInput(Node* node, size_t i) {
  auto schema = node->maybeSchema();
  if (!schema || i >= schema->arguments().size()) return false;
  return schema->is_mutable({c10::SchemaArgType::input, i});
}

bool isViewKind(Symbol k) {
  static const std::unordered_set<Symbol> kinds{c10::aten::select, c10::aten::slice,     c10::aten::permute,
                                                c10::aten::squeeze, c10::aten::unsqueeze, c10::aten::view,
                                                c10::aten::reshape, sym::Select(),        sym::Slice(),
                                                sym::Permute(),     sym::Squeeze(),       sym::Unsqueeze(),
                                                sym::View(),        sym::Reshape()};
  return kinds.count(k) != 0;
}

// View operators that have no immut:: twin but whose result is certainly a view of their first
// argument: a later write to the buffer is seen through them, so the rewrite re-derives them from
// the new version of their parent (by cloning the node), as the reference re-derives every value
// AliasDb says aliases the buffer (convert_to_tensorssa.cpp:186-266).  There is no write-back
// operator for them: a write THROUGH such a view leaves its whole tree untouched.
bool isPlainViewKind(Symbol k) {
  static const std::unordered_set<Symbol> kinds{
      c10::aten::t,         c10::aten::transpose, c10::aten::expand,   c10::aten::expand_as, c10::aten::narrow,
      c10::aten::view_as,   c10::aten::movedim,   c10::aten::swapaxes, c10::aten::swapdims,  c10::aten::diagonal,
      c10::aten::numpy_T,   c10::aten::mT,        c10::aten::alias,    c10::aten::detach,    c10::aten::unfold,
      c10::aten::as_strided, c10::aten::unflatten};
  return kinds.count(k) != 0;
}

// does the result of `node` possibly share storage with its input `i` (a `Tensor(a)` argument
// that some return repeats)?  True for the operators above and for those that view or copy
// depending on their arguments (to, contiguous, flatten, reshape_as, chunk, split ...).
bool mayReturnAliasOf(Node* node, size_t i) {
  auto schema = node->maybeSchema();
  if (!schema || i >= schema->arguments().size()) return false;
  const auto* ai = schema->arguments()[i].alias_info();
  if (!ai || ai->isWrite()) return false;
  for (const auto& r : schema->returns())
    if (r.alias_info()) return true;
  return false;
}

// The view forest: every tracked tensor is either a root (owns fresh storage)
// or a view of another tracked tensor (buffer_forest.h:50-65).
class ViewForest {
 public:
  std::unordered_map<Value*, Value*> parent;
  std::unordered_map<Value*, std::vector<Value*>> children;
  std::unordered_set<Node*> mutations;
  std::unordered_set<Value*> plain;   // views made by an operator of isPlainViewKind

  bool has(Value* v) const { return parent.count(v) != 0; }
  Value* parentOf(Value* v) const {
    auto it = parent.find(v);
    return it == parent.end() ? nullptr : it->second;
  }
  Value* rootOf(Value* v) const {
    while (Value* p = parentOf(v)) v = p;
    return v;
  }
  void addRoot(Value* v) { parent[v] = nullptr; }
  void addView(Value* v, Value* of) {
    parent[v] = of;
    children[of].push_back(v);
  }
  void replaceValue(Value* from, Value* to) {
    auto it = parent.find(from);
    if (it == parent.end()) return;
    Value* p = it->second;
    parent.erase(it);
    parent[to] = p;
    if (plain.erase(from)) plain.insert(to);
    if (p)
      for (auto& c : children[p])
        if (c == from) c = to;
    auto ch = children.find(from);
    if (ch != children.end()) {
      auto kids = ch->second;
      children.erase(ch);
      for (auto k : kids) parent[k] = to;
      children[to] = kids;
    }
  }
  void dropTree(Value* root) {
    std::deque<Value*> work{root};
    while (!work.empty()) {
      Value* v = work.front();
      work.pop_front();
      for (auto c : children[v]) work.push_back(c);
      children.erase(v);
      parent.erase(v);
    }
  }
};

bool freshTensorProducer(Node* n, Value* out) {
  switch (n->kind()) {
    case c10::prim::Param: case c10::prim::Loop: case c10::prim::If: case c10::prim::ListUnpack:
    case c10::prim::TupleUnpack: case c10::prim::GetAttr: case c10::aten::__getitem__: case c10::prim::Constant:
      return false;
    default: break;
  }
  if (!n->blocks().empty()) return false;
  auto schema = n->maybeSchema();
  if (!schema) return false;
  for (size_t i = 0; i < n->outputs().size(); ++i)
    if (n->output(i) == out && i < schema->returns().size() && schema->returns()[i].alias_info()) return false;
  return true;
}

void buildForest(Block* b, ViewForest& f) {
  for (Node* n : b->nodes()) {
    for (Block* inner : n->blocks()) buildForest(inner, f);
    if (n->outputs().size() < 1) continue;
    Value* out = n->output(0);
    if (!isTensor(out)) continue;
    if (isViewKind(n->kind()) && f.has(n->input(0))) {
      f.addView(out, n->input(0));
    } else if (isPlainViewKind(n->kind()) && n->outputs().size() == 1 && !n->inputs().empty() && f.has(n->input(0))) {
      f.addView(out, n->input(0));
      f.plain.insert(out);
    } else if ((n->kind() == c10::aten::copy_ || n->kind() == sym::Assign()) && f.has(n->input(0))) {
      f.addView(out, n->input(0));
      f.mutations.insert(n);
    } else if (freshTensorProducer(n, out)) {
      f.addRoot(out);
    }
  }
}

// Trees whose storage may be reached in ways the rewrite cannot see are left
// alone (convert_to_tensorssa.cpp:28-77: wildcards, containers, values defined
// by control flow).
void pruneForest(std::shared_ptr<Graph> g, ViewForest& f) {
  AliasDb db(g);
  std::unordered_set<Value*> bad;
  std::vector<Value*> all;
  for (auto& kv : f.parent) all.push_back(kv.first);
  for (Value* v : all) {
    Value* root = f.rootOf(v);
    for (Value* in : g->inputs())
      if (isTensor(in) && db.mayAlias(v, in)) bad.insert(root);
    for (const Use& u : v->uses()) {
      Node* user = u.user;
      switch (user->kind()) {
        case c10::prim::TupleConstruct: {
          // a tuple that only packs the values the graph returns holds no second name
          bool only_returned = true;
          for (const Use& tu : user->output()->uses())
            only_returned = only_returned && tu.user == g->return_node();
          if (!only_returned) bad.insert(root);
        } break;
        case c10::prim::ListConstruct: case c10::prim::DictConstruct:
        case c10::aten::append: case c10::prim::SetAttr:
          bad.insert(root);
          break;

        default:
          // a write this pass does not understand
          if (user->kind() != c10::aten::copy_ && user->kind() != sym::Assign() && writesInput(user, u.offset))
            bad.insert(root);
          // An operator that may hand back a view of the buffer which the forest does not track
          // (to, contiguous, flatten, chunk ...): a write to the buffer that follows it would have
          // to show through that view or not, depending on run-time facts.  With no such write the
          // operator simply reads the latest version.
          else if (!isViewKind(user->kind()) && !(isPlainViewKind(user->kind()) && u.offset == 0) &&
                   mayReturnAliasOf(user, u.offset)) {
            for (Node* m : f.mutations)
              if (f.has(m->output(0)) && f.rootOf(m->output(0)) == root && !m->isBefore(user)) bad.insert(root);
          }
      }
    }
  }
  // a write through a plain view has no write-back operator
  for (Node* m : f.mutations)
    for (Value* v = m->output(0); v && f.has(v); v = f.parentOf(v))
      if (f.plain.count(v)) bad.insert(f.rootOf(v));
  for (Value* r : bad) {
    std::vector<Node*> drop;
    for (Node* m : f.mutations)
      if (f.has(m->output(0)) && f.rootOf(m->output(0)) == r) drop.push_back(m);
    for (Node* m : drop) f.mutations.erase(m);
    f.dropTree(r);
  }
}

// aten::foo_(x, ...)  ->  t = aten::foo(x, ...); aten::copy_(x, t, False)
// (remove_inplace.cpp:20-73)
void removeInplaceIn(Block* b) {
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* node = *it;
    ++it;
    for (Block* inner : node->blocks()) removeInplaceIn(inner);
    if (node->inputs().empty() || !isTensor(node->input(0)) || !writesInput(node, 0)) continue;
    if (node->kind() == c10::aten::copy_) continue;  // uses of its output are redirected by the rewrite
    std::string name = node->kind().toUnqualString();
    if (name.empty() || name.back() != '_' || node->outputs().size() != 1) continue;
    name.pop_back();
    Symbol fn = Symbol::fromQualString(std::string(node->kind().ns().toUnqualString()) + "::" + name);
    Graph* g = b->owningGraph();
    Node* pure = g->create(fn, node->inputs(), 1)->copyMetadata(node);
    pure->insertBefore(node);
    if (!pure->maybeSchema()) {  // no functional twin with these arguments: keep the in-place op
      pure->destroy();
      continue;
    }
    pure->output()->setType(node->output()->type());
    Value* cfalse;
    {
      WithInsertPoint guard(node);
      cfalse = g->insertConstant(false);
    }
    Node* copy = g->create(c10::aten::copy_, {node->input(0), pure->output(), cfalse}, 1)->copyMetadata(node);
    copy->output()->setType(node->output()->type());
    copy->insertBefore(node);
    node->output()->replaceAllUsesWith(node->input(0));
    node->destroy();
  }
}

// tracked view / copy_ nodes -> immut:: twins (convert_to_tensorssa.cpp:274-306)
void immutablize(Block* b, ViewForest& f) {
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* node = *it;
    ++it;
    for (Block* inner : node->blocks()) immutablize(inner, f);
    auto found = immutableVersion().find(node->kind());
    if (found == immutableVersion().end() || node->outputs().size() != 1 || !f.has(node->output())) continue;
    Graph* g = b->owningGraph();
    std::vector<Value*> inputs(node->inputs().begin(), node->inputs().end());
    Node* imm = g->create(found->second, inputs, 1);
    imm->output()->setType(node->output()->type());
    imm->setSourceRange(node->sourceRange());
    imm->insertAfter(node);
    node->output()->replaceAllUsesWith(imm->output());
    f.replaceValue(node->output(), imm->output());
    if (f.mutations.count(node)) {
      f.mutations.erase(node);
      f.mutations.insert(imm);
    }
    node->destroy();
  }
}

// The write-back operator for `leaf = access(parent, args...)`: the nodes that
// compute the new version of `parent` once the new version `up` of `leaf` is
// known (last node of the result defines it).
std::vector<Node*> makeReverse(Graph* g, Node* leafNode, Value* up) {
  Symbol k = leafNode->kind();
  auto in = leafNode->inputs();
  if (k == sym::Assign()) return {g->create(sym::Assign(), in, 1)};  // the written values themselves
  if (k == sym::Select()) return {g->create(sym::SelectRev(), {in[0], up, in[1], in[2]}, 1)};
  if (k == sym::Slice()) return {g->create(sym::SliceRev(), {in[0], up, in[1], in[2], in[3], in[4]}, 1)};
  if (k == sym::Permute()) return {g->create(sym::PermuteRev(), {in[0], up, in[1]}, 1)};
  if (k == sym::Squeeze()) return {g->create(sym::Unsqueeze(), {up, in[1]}, 1)};
  if (k == sym::Unsqueeze()) return {g->create(sym::Squeeze(), {up, in[1]}, 1)};
  if (k == sym::View() || k == sym::Reshape()) {
    Node* sizes = g->create(c10::aten::size, {in[0]}, 1);
    sizes->output()->setType(c10::ListType::ofInts());
    return {sizes, g->create(sym::View(), {up, sizes->output()}, 1)};
  }
  TORCH_CHECK(false, "no assign operator for access operator ", k.toQualString());
  return {};
}

// convert_to_tensorssa.cpp:105-272: for every mutation, pass the new version up
// to the root of the view tree, then re-derive every view that is still alive.
void aliasRemoval(Block* b, ViewForest& f, TensorSSAMutateInfo& info) {
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* node = *it;
    ++it;
    for (Block* inner : node->blocks()) aliasRemoval(inner, f, info);
    if (!f.mutations.count(node)) continue;
    Graph* g = b->owningGraph();
    Node* resume = node->next();  // everything inserted below goes in front of it

    // pass up
    Value* leaf = node->output(0);
    Value* up = node->input(0);
    Node* at = node;
    while (Value* par = f.parentOf(leaf)) {
      const bool is_assign = leaf->node()->kind() == sym::Assign();
      for (Node* rev : makeReverse(g, leaf->node(), up)) {
        rev->setSourceRange(node->sourceRange());
        rev->insertAfter(at);
        at = rev;
      }
      if (at->kind() != c10::aten::size) at->output(0)->setType(is_assign ? leaf->type() : par->type());
      up = at->output(0);
      leaf = par;
    }
    Value* root = leaf;
    Node* update = g->create(sym::Update(), {up, root}, 0);
    update->insertAfter(at);
    info.addMutNodes(update);

    // pass down, level by level over the views that dominate the mutation; the
    // youngest view of a level first, which reproduces the node order of the
    // reference's printed graphs (README.md:113-140)
    struct Visit { Value* old_value; Value* new_value; Node* update; };
    std::deque<Visit> stack{{root, up, update}};
    while (!stack.empty()) {
      Visit cur = stack.front();
      stack.pop_front();
      auto kids = f.children.find(cur.old_value);
      if (kids == f.children.end()) continue;
      for (auto kit = kids->second.rbegin(); kit != kids->second.rend(); ++kit) {
        Value* from = *kit;
        Node* fromNode = from->node();
        bool alive = (fromNode == node) || (fromNode->isBefore(node) && node->isDominatedBy(fromNode));
        if (!alive) continue;
        Node* down = g->create(fromNode->kind(), fromNode->inputs(), 1);
        down->replaceInput(0, cur.new_value);
        if (fromNode->kind() == sym::Assign()) down->replaceInput(1, cur.new_value);
        down->insertAfter(cur.new_value->node());
        down->output(0)->copyMetadata(from);
        Node* upd = g->create(sym::Update(), {down->output(0), from}, 0);
        upd->insertAfter(cur.update);
        info.addMutNodes(upd);
        stack.push_back({from, down->output(0), upd});
      }
    }
    it = resume->iterator();
  }
}

// convert_to_tensorssa.cpp:322-364
void addMutatedValueToBlock(Value* mutated, Block* block, std::unordered_set<Block*>& visited, bool handleNode = true) {
  if (visited.count(block)) return;
  visited.insert(block);
  block->insertOutput(block->outputs().size(), mutated);
  Node* node = block->owningNode();
  Graph* g = node->owningGraph();
  if (handleNode) {
    Value* ret = node->addOutput();
    ret->setType(mutated->type());
    g->create(sym::Update(), {ret, mutated}, 0)->insertAfter(node);
  }
  switch (node->kind()) {
    case c10::prim::Loop: {
      Value* param = block->addInput();
      param->setType(mutated->type());
      Node* upd = g->create(sym::Update(), {param, mutated}, 0);
      if (block->nodes().begin() == block->nodes().end()) upd->insertBefore(block->return_node());
      else upd->insertBefore(block->nodes().front());
      node->addInput(mutated);
    } break;
    case c10::prim::If: {
      bool second = block == node->blocks()[1];
      addMutatedValueToBlock(mutated, node->blocks()[second ? 0 : 1], visited, false);
    } break;
    default: break;
  }
}

// convert_to_tensorssa.cpp:366-383.  `update(new, old)` renames the uses of `old`
// that follow it inside its own block (nested blocks included); uses further out
// are renamed by the update that value propagation placed behind the owning node.
void renameAfter(Node* update) {
  Value* fresh = update->input(0);
  Value* old = update->input(1);
  Block* scope = update->owningBlock();
  const auto uses = old->uses();  // copy: replaceInput edits the list
  for (const Use& use : uses) {
    Node* user = use.user;
    if (user == update) continue;
    Node* lifted = user;
    while (lifted && lifted->owningBlock() != scope) {
      Block* ob = lifted->owningBlock();
      lifted = ob ? ob->owningNode() : nullptr;
    }
    if (!lifted) continue;
    if (lifted == scope->return_node() || lifted->isAfter(update)) user->replaceInput(use.offset, fresh);
  }
}

void renameIn(Block* b) {
  for (Node* node : b->nodes()) {
    if (node->kind() == sym::Update()) renameAfter(node);
    for (Block* inner : node->blocks()) renameIn(inner);
  }
}

void removeUpdateIn(Block* b) {
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* node = *it;
    ++it;
    for (Block* inner : node->blocks()) removeUpdateIn(inner);
    if (node->kind() == sym::Update()) {
      node->destroy();
    } else if (node->kind() == sym::Assign()) {
      node->output()->replaceAllUsesWith(node->input(1));
      node->destroy();
    }
  }
}

void indexBoolFallbackIn(Block* b) {
  for (Node* node : b->nodes()) {
    for (Block* inner : node->blocks()) indexBoolFallbackIn(inner);
    if (node->kind() != sym::Index()) continue;
    auto indices = node->input(1)->node()->inputs();
    if (indices.empty()) continue;
    auto tt = indices.front()->type()->cast<c10::TensorType>();
    if (!tt || !tt->scalarType() || *tt->scalarType() != c10::kLong) node->replaceWithNewSymbol(c10::aten::index);
  }
}

}  // namespace

void RemoveInplace(std::shared_ptr<Graph> graph) { removeInplaceIn(graph->block()); }

void TensorSSARewriteMutation(std::shared_ptr<Graph> graph, std::shared_ptr<TensorSSAMutateInfo> info) {
  TORCH_CHECK(info, "TensorSSAMutateInfo is required");
  RemoveInplace(graph);
  ViewForest forest;
  buildForest(graph->block(), forest);
  pruneForest(graph, forest);
  immutablize(graph->block(), forest);
  aliasRemoval(graph->block(), forest, *info);
}

void TensorSSAPropagation(std::shared_ptr<Graph> graph, std::shared_ptr<TensorSSAMutateInfo> info) {
  for (Value* mutated : info->mutValues) {
    Block* defBlock = mutated->node()->owningBlock();
    std::unordered_set<Block*> visited;
    for (Node* node : info->mutNodes[mutated])
      for (Block* block = node->owningBlock(); block != defBlock; block = block->owningNode()->owningBlock())
        addMutatedValueToBlock(mutated, block, visited);
  }
}

void TensorSSARename(std::shared_ptr<Graph> graph) { renameIn(graph->block()); }
void TensorSSARemoveUpdate(std::shared_ptr<Graph> graph) { removeUpdateIn(graph->block()); }

void ConvertToTensorSSA(std::shared_ptr<Graph> graph) {
  auto info = std::make_shared<TensorSSAMutateInfo>();
  TensorSSARewriteMutation(graph, info);
  TensorSSAPropagation(graph, info);
  TensorSSARename(graph);
  indexBoolFallbackIn(graph->block());
}

// functs/csrc/jit/passes/convert_to_tensorssa.cpp:308-320: clone every tensor
// argument so that the body owns its buffers
void DumbRemoveInterPrecedureMutation(std::shared_ptr<Graph> graph) {
  for (Value* input : graph->inputs()) {
    if (!isTensor(input)) continue;
    WithInsertPoint guard(graph->block()->nodes().front());
    Value* none = graph->insertConstant(c10::IValue());
    Node* copy = graph->create(c10::aten::clone, {input, none}, 1);
    copy->insertAfter(none->node());
    copy->output()->copyMetadata(input);
    input->replaceAllUsesAfterNodeWith(copy, copy->output());
  }
}

}  // namespace functs
