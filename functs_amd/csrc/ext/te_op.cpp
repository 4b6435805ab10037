// tssa::ParallelFunctor: the operator a fused region runs as, and the pass that
// creates it from prim::FusionGroup / prim::ParallelMap nodes.
//
// Node contract as in the reference (fait/passes/te_op.cpp:34-249, te_op.h:13-23):
//   g(attr::Subgraph)          the region; input 0 is the task index (or a None
//                              placeholder for a plain fused op), then the arguments
//   i(attr::parallel_degree)   number of tasks (-1: taken from the leading int input)
//   i(attr::is_parallel_map)   outputs are List[Tensor] with one entry per task
//   is(attr::is_parallel_args) per argument: 1 = a list holding one value per task
//   tys(attr::input_refine_types)
// plus i(attr::compact_rows): the last subgraph output is a row mask that is
// applied to every other output (see FuseMaskedSelect).
// Stack protocol as GraphBuilder::runKernel (fait/fuser/graph_builder.cpp:901-927):
// pops the arguments, pushes one IValue per output; outputs are freshly
// allocated, inputs are never written.
#include <ATen/ATen.h>
#include <ATen/core/CachingHostAllocator.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/DeviceGuard.h>
#include <torch/csrc/jit/ir/constants.h>
#include <torch/csrc/jit/passes/common_subexpression_elimination.h>
#include <torch/csrc/jit/passes/constant_propagation.h>
#include <torch/csrc/jit/passes/dead_code_elimination.h>
#include <torch/csrc/jit/runtime/custom_operator.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <map>
#include <mutex>
#include <sstream>
#include <tuple>

#include "../../../include/fxhip.h"
#include "passes.h"
#include "symbols.h"

namespace functs {
using namespace torch::jit;

namespace {

bool isTensorValue(const Value* v) { return v->type()->kind() == c10::TypeKind::TensorType; }

// ---------------------------------------------------------------------------
// pass: FusionGroup / ParallelMap -> ParallelFunctor
// ---------------------------------------------------------------------------
void cloneBlockInto(Block* src, Graph* sub, std::unordered_map<Value*, Value*>& map,
                    const std::vector<Value*>* returns = nullptr) {
  auto env = [&](Value* v) -> Value* {
    auto it = map.find(v);
    if (it != map.end()) return it->second;
    if (v->node()->kind() == c10::prim::Constant) {
      Node* c = sub->createClone(v->node(), [](Value* x) { return x; });
      sub->prependNode(c);
      map[v] = c->output();
      return c->output();
    }
    TORCH_CHECK(false, "ParallelFunctor: free value %", v->debugName(), " in a fused region");
  };
  for (Node* n : src->nodes()) {
    Node* c = sub->createClone(n, env);
    sub->appendNode(c);
    for (size_t i = 0; i < n->outputs().size(); ++i) map[n->output(i)] = c->output(i);
  }
  if (returns) {
    for (Value* o : *returns) sub->registerOutput(env(o));
  } else {
    for (Value* o : src->outputs()) sub->registerOutput(env(o));
  }
}

// A region holds pure operators only, so equal expressions can be merged; alias
// analysis has no entry for the collapsed-loop node, regions with one are left as is.
void cseRegion(std::shared_ptr<Graph> sub) {
  for (Node* n : sub->nodes())
    if (n->kind() == sym::ForallSelectRev()) return;
  EliminateCommonSubexpression(sub);
}

Node* functorFromGroup(Node* group) {
  Graph* g = group->owningGraph();
  Node* f = g->createWithSubgraph(sym::ParallelFunctor());
  auto sub = f->g(c10::attr::Subgraph);
  std::vector<c10::TypePtr> types;
  for (Value* in : group->inputs()) {
    f->addInput(in);
    types.push_back(in->type());
  }
  f->tys_(sym::input_refine_types(), types);
  f->i_(sym::parallel_degree(), 1);
  f->i_(sym::is_parallel_map(), 0);
  f->is_(sym::is_parallel_args(), std::vector<int64_t>(group->inputs().size(), 1));  // te_op.cpp:186-187
  f->i_(sym::compact_rows(), group->hasAttribute(sym::compact_rows()) ? group->i(sym::compact_rows()) : 0);
  for (Value* out : group->outputs()) f->addOutput()->copyMetadata(out);
  std::unordered_map<Value*, Value*> map;
  sub->addInput()->setType(c10::NoneType::get());  // placeholder for the task index (te_op.cpp:192)
  Block* body = group->blocks()[0];
  for (Value* p : body->inputs()) map[p] = sub->addInput()->copyMetadata(p);
  cloneBlockInto(body, sub.get(), map);
  cseRegion(sub);
  return f;
}

// ParallelMap(len, lists...) { block(i, elems...): FusionGroup(...) -> rets }
Node* functorFromMap(Node* mapNode, Node* group) {
  Graph* g = mapNode->owningGraph();
  Block* mb = mapNode->blocks()[0];
  Block* body = group->blocks()[0];
  Node* f = g->createWithSubgraph(sym::ParallelFunctor());
  auto sub = f->g(c10::attr::Subgraph);
  auto len = constant_as<int64_t>(mapNode->input(0));
  f->i_(sym::parallel_degree(), len ? *len : -1);
  f->i_(sym::is_parallel_map(), 1);
  f->i_(sym::compact_rows(), group->hasAttribute(sym::compact_rows()) ? group->i(sym::compact_rows()) : 0);
  if (!len) f->addInput(mapNode->input(0));  // trip count travels as the leading argument
  std::vector<int64_t> par;
  std::vector<c10::TypePtr> types;
  std::unordered_map<Value*, Value*> map;
  Value* idx = sub->addInput()->setType(c10::IntType::get());
  // subgraph parameters follow the group's inputs; what they are bound to decides the kind
  std::vector<Value*> params_in_order;
  for (size_t k = 0; k < group->inputs().size(); ++k) {
    Value* in = group->input(k);
    Value* p = body->inputs()[k];
    if (in == mb->inputs()[0]) {  // the loop index
      map[p] = idx;
      continue;
    }
    Value* sp = sub->addInput()->copyMetadata(p);
    map[p] = sp;
    auto pos = std::find(mb->inputs().begin() + 1, mb->inputs().end(), in);
    if (pos != mb->inputs().end()) {
      size_t li = pos - mb->inputs().begin();  // list argument of the map
      f->addInput(mapNode->input(li));
      // a refined list records the unified type of its elements (te_op.cpp:43-59)
      c10::TypePtr recorded = mapNode->input(li)->type();
      auto refined = refinedTypes().find(mapNode->input(li));
      if (refined != refinedTypes().end()) {
        const auto& elems = refined->second->expectRef<c10::TupleType>().elements();
        std::stringstream why_not;
        auto unified = c10::unifyTypeList(elems, why_not);
        if (unified) recorded = *unified;
        TORCH_CHECK(!len || *len <= (int64_t)elems.size(), "ParallelMap: ", *len, " tasks over a list of ", elems.size());
      }
      types.push_back(recorded);
      par.push_back(1);
    } else {
      TORCH_CHECK(in->node()->owningBlock() != mb, "ParallelMap: group input defined inside the map body");
      f->addInput(in);
      types.push_back(in->type());
      par.push_back(0);
    }
  }
  f->is_(sym::is_parallel_args(), par);
  f->tys_(sym::input_refine_types(), types);
  for (Value* out : mapNode->outputs()) f->addOutput()->copyMetadata(out);
  // the map returns group outputs in its own order; the row mask stays last
  std::vector<Value*> returns;
  for (Value* r : mb->outputs()) returns.push_back(body->outputs()[r->offset()]);
  if (f->i(sym::compact_rows())) returns.push_back(body->outputs().back());
  cloneBlockInto(body, sub.get(), map, &returns);
  cseRegion(sub);
  return f;
}

// fx::lstm_stack (the collapsed loop nest of a stacked LSTM, recurrent.cpp) as a region of one
// node: its tensor and int operands are the arguments, its None operands stay constants.
Node* functorFromLstmStack(Node* n) {
  Graph* g = n->owningGraph();
  Node* f = g->createWithSubgraph(sym::ParallelFunctor());
  auto sub = f->g(c10::attr::Subgraph);
  sub->addInput()->setType(c10::NoneType::get());
  std::vector<c10::TypePtr> types;
  std::vector<Value*> operands;
  for (Value* in : n->inputs()) {
    if (in->node()->kind() == c10::prim::Constant) {
      Node* c = sub->createClone(in->node(), [](Value* x) { return x; });
      sub->appendNode(c);
      operands.push_back(c->output());
      continue;
    }
    f->addInput(in);
    types.push_back(in->type());
    operands.push_back(sub->addInput()->copyMetadata(in));
  }
  Node* k = sub->create(sym::LstmStack(), operands, n->outputs().size());
  sub->appendNode(k);
  for (size_t i = 0; i < n->outputs().size(); ++i) {
    k->output(i)->copyMetadata(n->output(i));
    sub->registerOutput(k->output(i));
    f->addOutput()->copyMetadata(n->output(i));
  }
  f->tys_(sym::input_refine_types(), types);
  f->i_(sym::parallel_degree(), 1);
  f->i_(sym::is_parallel_map(), 0);
  f->is_(sym::is_parallel_args(), std::vector<int64_t>(types.size(), 1));
  f->i_(sym::compact_rows(), 0);
  return f;
}

// A map whose body did not end up as exactly one fused group goes back to a
// loop (ConvertInfusibleMapsToLoops, parallelize_loops.cpp:295-362).
Node* mapBackToLoop(Node* mapNode) {
  Graph* g = mapNode->owningGraph();
  Block* mb = mapNode->blocks()[0];
  WithInsertPoint guard(mapNode);
  std::vector<Value*> out_lists;
  for (Value* o : mapNode->outputs()) {
    auto lt = o->type()->cast<c10::ListType>();
    Node* lc = g->createList(lt->getElementType(), {});
    g->insertNode(lc);
    lc->output()->setType(o->type());
    out_lists.push_back(lc->output());
  }
  Value* ctrue = g->insertConstant(true);
  Node* loop = g->create(c10::prim::Loop, {mapNode->input(0), ctrue}, 0);
  g->insertNode(loop);
  Block* lb = loop->addBlock();
  Value* i = lb->addInput()->setType(c10::IntType::get());
  std::unordered_map<Value*, Value*> map;
  map[mb->inputs()[0]] = i;
  for (size_t k = 1; k < mb->inputs().size(); ++k) {
    Node* get = g->create(c10::aten::__getitem__, {mapNode->input(k), i}, 1);
    get->output()->setType(mb->inputs()[k]->type());
    lb->appendNode(get);
    map[mb->inputs()[k]] = get->output();
  }
  auto env = [&](Value* v) -> Value* {
    auto it = map.find(v);
    return it != map.end() ? it->second : v;
  };
  for (Node* n : mb->nodes()) {
    Node* c = g->createClone(n, env);
    lb->appendNode(c);
    for (size_t k = 0; k < n->outputs().size(); ++k) map[n->output(k)] = c->output(k);
  }
  for (size_t k = 0; k < out_lists.size(); ++k) {
    Node* app = g->create(c10::aten::append, {out_lists[k], env(mb->outputs()[k])}, 1);
    app->output()->setType(out_lists[k]->type());
    lb->appendNode(app);
  }
  {
    WithInsertPoint in_body(lb->return_node());
    lb->registerOutput(g->insertConstant(true));
  }
  for (size_t k = 0; k < out_lists.size(); ++k) mapNode->output(k)->replaceAllUsesWith(out_lists[k]);
  mapNode->destroy();
  return loop;
}

void toFunctorIn(Block* b) {
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* n = *it;
    ++it;
    if (n->kind() == c10::prim::FusionGroup || n->kind() == sym::LstmStack()) {
      Node* f = n->kind() == sym::LstmStack() ? functorFromLstmStack(n) : functorFromGroup(n);
      f->insertBefore(n);
      for (size_t k = 0; k < n->outputs().size(); ++k) n->output(k)->replaceAllUsesWith(f->output(k));
      n->destroy();
      continue;
    }
    if (n->kind() == sym::ParallelMap()) {
      Block* mb = n->blocks()[0];
      Node* group = nullptr;
      bool single = true;
      for (Node* m : mb->nodes()) {
        if (m->kind() == c10::prim::Constant) continue;
        if (m->kind() == c10::prim::FusionGroup && !group) group = m;
        else single = false;
      }
      if (group && single)  // every value the map returns comes out of the group
        for (Value* r : mb->outputs()) single = single && r->node() == group;
      if (group && single) {
        Node* f = functorFromMap(n, group);
        f->insertBefore(n);
        for (size_t k = 0; k < n->outputs().size(); ++k) n->output(k)->replaceAllUsesWith(f->output(k));
        n->destroy();
      } else {
        Node* loop = mapBackToLoop(n);
        toFunctorIn(loop->blocks()[0]);
      }
      continue;
    }
    for (Block* inner : n->blocks()) toFunctorIn(inner);
  }
}

// ---------------------------------------------------------------------------
// run time: subgraph -> fx_region (C ABI), argument marshalling, launch
// ---------------------------------------------------------------------------
int fxDtype(c10::ScalarType t) {
  switch (t) {
    case c10::kFloat: return FX_DT_F32;
    case c10::kLong: return FX_DT_I64;
    case c10::kInt: return FX_DT_I32;
    case c10::kByte: return FX_DT_U8;
    case c10::kHalf: return FX_DT_F16;
    case c10::kBFloat16: return FX_DT_BF16;
    case c10::kBool: return FX_DT_BOOL;
    default: TORCH_CHECK(false, "fused regions do not support dtype ", t);
  }
}
c10::ScalarType atDtype(int d) {
  switch (d) {
    case FX_DT_F32: return c10::kFloat;
    case FX_DT_I64: return c10::kLong;
    case FX_DT_I32: return c10::kInt;
    case FX_DT_U8: return c10::kByte;
    case FX_DT_F16: return c10::kHalf;
    case FX_DT_BF16: return c10::kBFloat16;
    case FX_DT_BOOL: return c10::kBool;
  }
  TORCH_CHECK(false, "bad fx dtype");
}

#define FX_OK_OR_THROW(expr)                                            \
  do {                                                                  \
    int rc__ = (expr);                                                  \
    TORCH_CHECK(rc__ >= 0, "fxhip: ", fx_last_error(), " (", #expr, ")"); \
  } while (0)

// What earlier launches reported through the library's error word (include/fxhip.h
// fx_async_error): every report is an error of this call, whichever operator made it - the word
// is cleared by reading it, so a report that is not raised here would be lost.
void resetLstmWorkspaces();
void checkAsyncError() {
  const int e = fx_async_error(1);
  if (e == 0) return;
  if (e & FX_ASYNC_BARRIER) resetLstmWorkspaces();   // a given-up wait leaves its workspace marked: the next call takes a cleared one
  std::string what;
  if (e & FX_ASYNC_INT64)
    what += " a fused region read an int64 element outside 32 bits into integer arithmetic (moves of int64 data are exact, "
            "arithmetic is 32-bit);";
  if (e & FX_ASYNC_BARRIER) what += " fx::lstm_stack gave up a wait between its workgroups (its results were filled with NaN);";
  if (e & FX_ASYNC_NMS_CAPACITY) what += " fx_sort_nms found more candidates in an image than the launch was sized for;";
  if (e & ~(FX_ASYNC_INT64 | FX_ASYNC_BARRIER | FX_ASYNC_NMS_CAPACITY)) what += " unknown report " + std::to_string(e) + ";";
  TORCH_CHECK(false, "functs_amd: an earlier launch reported an error, its results are not valid:", what);
}

// Host time of the operator by section, summed over calls while switched on: where a call's
// time goes between popping the arguments and pushing the results.
enum HostSection { HS_FLATTEN, HS_PLAN, HS_ALLOC, HS_LAUNCH, HS_VIEWS, HS_WAIT, HS_RESIZE, HS_PUSH, HS_COUNT };
const char* const kHostSectionNames[HS_COUNT] = {"flatten", "plan", "alloc", "launch", "views", "wait_counts", "resize", "push"};
std::atomic<bool> g_host_timing{false};
std::atomic<uint64_t> g_host_ns[HS_COUNT];
std::atomic<uint64_t> g_host_calls{0};
struct HostClock {
  const bool on = g_host_timing.load(std::memory_order_relaxed);
  std::chrono::steady_clock::time_point last;
  HostClock() { if (on) last = std::chrono::steady_clock::now(); }
  void tick(HostSection s) {
    if (!on) return;
    const auto now = std::chrono::steady_clock::now();
    g_host_ns[s].fetch_add((uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(now - last).count(),
                           std::memory_order_relaxed);
    last = now;
  }
};

// The key of a call's argument kinds (which variant of the region serves it), put together per
// call: a string with the few appends it needs (a stream costs a locale and an allocation a call).
struct Signature {
  std::string s;
  Signature() { s.reserve(96); }
  Signature& operator<<(const char* t) { s.append(t); return *this; }
  Signature& operator<<(long long v) {
    char buf[24];
    int n = 0;
    unsigned long long u = v < 0 ? 0ull - (unsigned long long)v : (unsigned long long)v;
    do { buf[n++] = (char)('0' + u % 10); u /= 10; } while (u);
    if (v < 0) s.push_back('-');
    while (n) s.push_back(buf[--n]);
    return *this;
  }
  Signature& operator<<(long v) { return *this << (long long)v; }
  Signature& operator<<(int v) { return *this << (long long)v; }
  Signature& operator<<(unsigned v) { return *this << (long long)v; }
  Signature& operator<<(unsigned long v) { return *this << (long long)v; }
  const std::string& str() const { return s; }
};

thread_local EarlyResultsHook* t_early_hook = nullptr;
// between beforeBlocking and afterBlocking of the hook, also when an error leaves the scope
struct BlockingScope {
  EarlyResultsHook* hook;
  explicit BlockingScope(EarlyResultsHook* h) : hook(h) { if (hook) hook->beforeBlocking(); }
  ~BlockingScope() { if (hook) hook->afterBlocking(); }
};

// device scratch and the pinned landing zone of the kept-row counts; a call
// borrows one and hands it back, so concurrent calls never share
struct Workspace {
  at::Tensor scratch, totals;
  void* stream = nullptr;   // stream of the last run that used it (that run may still be in flight)
};

// where the tasks' tensors of every output lie in that output's one allocation: fixed per plan
struct OutSlot { int64_t offset_elems; int32_t rank; int64_t sizes[FX_ARG_MAX_RANK]; };
struct OutLayout {
  std::vector<OutSlot> slots;      // [output][task]
  std::vector<int64_t> total;      // elements to allocate per output
  std::vector<int32_t> dtype;      // FX dtype per output
  std::vector<int64_t> item;       // element size per output
  std::vector<int64_t> base;       // a map's outputs share ONE allocation: byte offset of each output in it
  int64_t block_bytes = 0;
};

struct Variant {
  fx_region* region = nullptr;
  std::mutex mu;
  std::vector<Workspace> pool;
  // the output block of the next call of a map, allocated while the last call's kernels ran
  at::Tensor next_block;
  void* next_stream = nullptr;
  static constexpr int64_t kMaxPrepared = 512ll << 20;
  // likewise the output tensors of the next call of a single task (one per output, at full size)
  std::vector<at::Tensor> next_buffers;
  const fx_plan* next_buffers_plan = nullptr;
  void* next_buffers_stream = nullptr;
  std::vector<at::Tensor> takeBuffers(const fx_plan* plan, void* stream) {
    std::lock_guard<std::mutex> lock(mu);
    if (next_buffers_plan != plan || next_buffers_stream != stream) return {};
    next_buffers_plan = nullptr;
    return std::move(next_buffers);
  }
  void prepareBuffers(const fx_plan* plan, void* stream, std::vector<at::Tensor> buffers) {
    std::lock_guard<std::mutex> lock(mu);
    next_buffers = std::move(buffers);
    next_buffers_plan = plan;
    next_buffers_stream = stream;
  }
  at::Tensor takeBlock(int64_t bytes, c10::Device device, void* stream) {
    {
      std::lock_guard<std::mutex> lock(mu);
      if (next_block.defined() && next_block.numel() == bytes && next_block.device() == device && next_stream == stream)
        return std::move(next_block);
    }
    return at::empty({bytes}, at::TensorOptions().dtype(at::kByte).device(device));
  }
  void prepareBlock(int64_t bytes, c10::Device device, void* stream) {
    if (bytes > kMaxPrepared) return;   // (what is prepared stays allocated between calls)
    at::Tensor b = at::empty({bytes}, at::TensorOptions().dtype(at::kByte).device(device));   // on the current stream
    std::lock_guard<std::mutex> lock(mu);
    next_block = std::move(b);
    next_stream = stream;
  }
  std::unordered_map<const fx_plan*, std::shared_ptr<const OutLayout>> layouts;   // plans live as long as the region
  ~Variant() {
    if (region) fx_region_destroy(region);
  }
  // A workspace goes back to the pool as soon as the kept-row counts are known, while the
  // second pass may still be reading its scratch: on the same stream the next run is ordered
  // behind it; another stream waits for it first.
  Workspace take(size_t scratch_bytes, int64_t degree, c10::Device device, void* stream) {
    {
      std::unique_lock<std::mutex> lock(mu);
      while (!pool.empty()) {
        Workspace ws = std::move(pool.back());
        pool.pop_back();
        if ((size_t)ws.scratch.numel() >= scratch_bytes && ws.totals.numel() >= degree &&
            ws.scratch.device() == device) {
          lock.unlock();
          if (ws.stream != stream) {
            const hipError_t e = hipStreamSynchronize((hipStream_t)ws.stream);
            TORCH_CHECK(e == hipSuccess, "hipStreamSynchronize: ", hipGetErrorString(e));
          }
          return ws;
        }
      }
    }
    Workspace ws;
    ws.scratch = at::empty({(int64_t)std::max<size_t>(scratch_bytes, 1)},
                           at::TensorOptions().dtype(at::kByte).device(device));
    ws.totals = at::empty({degree}, at::TensorOptions().dtype(at::kInt).pinned_memory(true));
    return ws;
  }
  void give(Workspace ws) {
    std::lock_guard<std::mutex> lock(mu);
    if (pool.size() < 4) pool.push_back(std::move(ws));
  }
};

class RegionRunner {
 public:
  explicit RegionRunner(const Node* node)
      : graph_(node->g(c10::attr::Subgraph)),
        is_par_(node->is(sym::is_parallel_args())),
        degree_(node->i(sym::parallel_degree())),
        is_map_(node->i(sym::is_parallel_map()) != 0),
        compact_(node->hasAttribute(sym::compact_rows()) && node->i(sym::compact_rows()) != 0),
        padded_(node->hasAttribute(sym::padded_outputs()) && node->i(sym::padded_outputs()) != 0) {
    TORCH_CHECK(!padded_ || compact_, "ParallelFunctor: padded_outputs is an attribute of compacting functors");
    n_args_ = graph_->inputs().size() - 1;
    TORCH_CHECK(is_par_.size() == n_args_, "ParallelFunctor: is_parallel_args does not match the subgraph");
    n_stack_ = n_args_ + (degree_ < 0 ? 1 : 0);
    n_outs_ = graph_->outputs().size() - (compact_ ? 1 : 0);
  }

  void run(Stack& stack) {
    auto inputs = last(stack, n_stack_);
    int64_t degree = degree_;
    size_t first = 0;
    if (degree_ < 0) {
      degree = inputs[0].toInt();
      first = 1;
    }
    if (!is_map_) degree = 1;
    TORCH_CHECK(degree >= 0, "ParallelFunctor: negative trip count");
    if (degree == 0) {  // an empty map
      TORCH_CHECK(!padded_, "ParallelFunctor: a map with padded outputs needs at least one task");
      drop(stack, n_stack_);
      for (size_t o = 0; o < n_outs_; ++o) push(stack, c10::List<at::Tensor>());
      return;
    }
    HostClock clock;
    // flatten arguments
    std::vector<fx_arg> args;
    {   // one entry per shared argument and per task of a per-task one (more only for list-valued scalars)
      size_t n_par = 0;
      if (is_map_) for (int64_t p : is_par_) n_par += p != 0;
      args.reserve(n_args_ + n_par * (size_t)std::max<int64_t>(degree, 1));
    }
    Signature sig;
    c10::Device device(c10::kCPU);
    bool have_device = false;
    flatten(inputs, first, degree, /*dry=*/false, args, sig, device, have_device);
    TORCH_CHECK(have_device, "ParallelFunctor: a region needs at least one tensor argument");
    c10::DeviceGuard guard(device);
    clock.tick(HS_FLATTEN);

    Variant* var;
    {
      std::lock_guard<std::mutex> lock(mu_);
      auto& slot = variants_[sig.str()];
      if (!slot) {
        slot = std::make_unique<Variant>();
        build(*slot, degree, inputs, first);
      }
      var = slot.get();
    }
    const fx_plan* plan = nullptr;
    FX_OK_OR_THROW(fx_region_plan(var->region, args.data(), (int)args.size(), &plan));
    const int n_out = fx_plan_num_outputs(plan);
    // One allocation per output: the tasks' tensors are views at 256-byte aligned
    // offsets of it.  The views are made after the launch, while the kernels run.
    std::shared_ptr<const OutLayout> layout;
    {
      std::lock_guard<std::mutex> lock(var->mu);
      auto it = var->layouts.find(plan);
      if (it != var->layouts.end()) layout = it->second;
    }
    if (!layout) {
      auto lay = std::make_shared<OutLayout>();
      lay->slots.resize((size_t)n_out * degree);
      lay->total.resize(n_out);
      lay->dtype.resize(n_out);
      lay->item.resize(n_out);
      for (int o = 0; o < n_out; ++o) {
        int32_t dt = 0;
        int64_t total = 0, item = 1;
        for (int64_t t = 0; t < degree; ++t) {
          OutSlot& sl = lay->slots[(size_t)o * degree + t];
          FX_OK_OR_THROW(fx_plan_output(plan, o, (int)t, &dt, &sl.rank, sl.sizes));
          int64_t numel = 1;
          for (int d = 0; d < sl.rank; ++d) numel *= sl.sizes[d];
          item = (int64_t)c10::elementSize(atDtype(dt));
          const int64_t align = 256 / item;
          sl.offset_elems = total;
          total += (numel + align - 1) / align * align;
        }
        lay->total[o] = total;
        lay->dtype[o] = dt;
        lay->item[o] = item;
      }
      lay->base.resize(n_out);
      for (int o = 0; o < n_out; ++o) {
        lay->base[o] = lay->block_bytes;
        lay->block_bytes += (lay->total[o] * lay->item[o] + 255) / 256 * 256;
      }
      std::lock_guard<std::mutex> lock(var->mu);
      layout = var->layouts.emplace(plan, std::move(lay)).first->second;
    }
    clock.tick(HS_PLAN);
    typedef OutSlot Slot;
    const Slot* slot_of = layout->slots.data();   // (full sizes; the kept-row counts replace dimension 0 below)
    // A map: ONE allocation for all outputs of all tasks (an allocation costs about a
    // microsecond of host time); a single task: one tensor per output.
    std::vector<at::Tensor> buffers(n_out);
    at::Tensor block;
    std::vector<void*> ptrs((size_t)n_out * degree);
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(device.index());
    if (degree > 1) block = var->takeBlock(std::max<int64_t>(layout->block_bytes, 1), device, (void*)stream.stream());
    if (degree == 1) {
      std::vector<at::Tensor> prepared = var->takeBuffers(plan, (void*)stream.stream());
      if ((int)prepared.size() == n_out) buffers = std::move(prepared);
    }
    auto newBuffer = [&](int o) {
      const Slot& sl = layout->slots[(size_t)o * degree];   // (at full size: the kept-row counts cut it later)
      return at::empty(at::IntArrayRef(sl.sizes, sl.rank), at::TensorOptions().dtype(atDtype(layout->dtype[o])).device(device));
    };
    for (int o = 0; o < n_out; ++o) {
      const int64_t item = layout->item[o];
      char* base;
      if (degree == 1) {
        if (!buffers[o].defined()) buffers[o] = newBuffer(o);
        base = (char*)buffers[o].data_ptr();
      } else {
        base = (char*)block.data_ptr() + layout->base[o];
      }
      for (int64_t t = 0; t < degree; ++t)
        ptrs[(size_t)o * degree + t] = base + slot_of[(size_t)o * degree + t].offset_elems * item;
    }
    Workspace ws;
    const size_t scratch_bytes = fx_plan_scratch_bytes(plan);   // (a dense map of very many tasks keeps its tables there)
    if (compact_ || scratch_bytes > 0) {
      ws = var->take(scratch_bytes, degree, device, (void*)stream.stream());
      ws.stream = (void*)stream.stream();
    }
    checkAsyncError();
    clock.tick(HS_ALLOC);
    if (padded_) {
      // Every output at its full size, the kept-row counts as a tensor of their own (pinned host
      // memory that the kernels write and the next kernel on the stream reads): nobody waits.
      at::Tensor counts = at::empty({degree}, at::TensorOptions().dtype(at::kInt).pinned_memory(true));
      FX_OK_OR_THROW(fx_region_run(var->region, plan, args.data(), (int)args.size(), ptrs.data(), ws.scratch.data_ptr(),
                                   (uint32_t*)counts.data_ptr(), (void*)stream.stream()));
      // the block is not handed out again before the launch has written it
      at::getHostAllocator(at::kCUDA)->record_event(counts.data_ptr(), counts.storage().data_ptr().get_context(), stream.unwrap());
      clock.tick(HS_LAUNCH);
      var->give(std::move(ws));
      drop(stack, n_stack_);
      for (int o = 0; o < n_out; ++o) {
        if (degree == 1) {
          push(stack, is_map_ ? buffers[o].unsqueeze(0) : std::move(buffers[o]));
          continue;
        }
        const Slot& first_slot = slot_of[(size_t)o * degree];
        const int64_t task_stride = slot_of[(size_t)o * degree + 1].offset_elems - first_slot.offset_elems;
        std::vector<int64_t> sizes{degree}, strides{task_stride};
        int64_t inner = 1;
        for (int d = 0; d < first_slot.rank; ++d) inner *= first_slot.sizes[d];
        for (int d = 0; d < first_slot.rank; ++d) {
          sizes.push_back(first_slot.sizes[d]);
          inner /= std::max<int64_t>(first_slot.sizes[d], 1);
          strides.push_back(first_slot.sizes[d] == 0 ? 1 : inner);
        }
        for (int64_t t = 1; t < degree; ++t) {
          const Slot& sl = slot_of[(size_t)o * degree + t];
          TORCH_CHECK(sl.rank == first_slot.rank && std::equal(sl.sizes, sl.sizes + sl.rank, first_slot.sizes) &&
                          sl.offset_elems == first_slot.offset_elems + t * task_stride,
                      "ParallelFunctor: padded outputs need tasks of one size");
        }
        auto impl = c10::make_intrusive<c10::TensorImpl>(c10::TensorImpl::VIEW, c10::Storage(block.storage()), block.key_set(),
                                                         c10::scalarTypeToTypeMeta(atDtype(layout->dtype[o])));
        impl->set_storage_offset(layout->base[o] / layout->item[o] + first_slot.offset_elems);
        impl->set_sizes_and_strides(sizes, strides);
        push(stack, at::Tensor(std::move(impl)));
      }
      push(stack, std::move(counts));
      clock.tick(HS_PUSH);
      if (clock.on) g_host_calls.fetch_add(1, std::memory_order_relaxed);
      return;
    }
    FX_OK_OR_THROW(fx_region_run(var->region, plan, args.data(), (int)args.size(), ptrs.data(),
                                 ws.scratch.defined() ? ws.scratch.data_ptr() : nullptr,
                                 compact_ ? (uint32_t*)ws.totals.data_ptr() : nullptr, (void*)stream.stream()));
    if (!compact_ && ws.scratch.defined()) var->give(std::move(ws));   // (the next borrower is ordered behind this launch)
    clock.tick(HS_LAUNCH);
    // The tasks' tensors: views of the block, made while the kernels run.
    std::vector<at::Tensor> flat;   // [output][task]
    if (degree > 1) {
      flat.reserve((size_t)n_out * degree);
      for (int o = 0; o < n_out; ++o) {
        const int64_t first_elem = layout->base[o] / layout->item[o];
        for (int64_t t = 0; t < degree; ++t) {
          const Slot& sl = slot_of[(size_t)o * degree + t];
          auto impl = c10::make_intrusive<c10::TensorImpl>(c10::TensorImpl::VIEW, c10::Storage(block.storage()), block.key_set(),
                                                           c10::scalarTypeToTypeMeta(atDtype(layout->dtype[o])));
          impl->set_storage_offset(first_elem + sl.offset_elems);
          impl->set_sizes_contiguous(at::IntArrayRef(sl.sizes, sl.rank));
          flat.emplace_back(std::move(impl));
        }
      }
      // the next call's block is allocated now, while this call's kernels run
      var->prepareBlock(std::max<int64_t>(layout->block_bytes, 1), device, (void*)stream.stream());
    } else {
      int64_t bytes = 0;
      for (int o = 0; o < n_out; ++o) bytes += layout->total[o] * layout->item[o];
      if (bytes <= Variant::kMaxPrepared) {
        std::vector<at::Tensor> next(n_out);
        for (int o = 0; o < n_out; ++o) next[o] = newBuffer(o);
        var->prepareBuffers(plan, (void*)stream.stream(), std::move(next));
      }
    }
    clock.tick(HS_VIEWS);
    EarlyResultsHook* const hook = t_early_hook;
    if (hook && is_map_ && degree > 1 && compact_) hook->tensorsReady((size_t)n_out, degree, flat.data());
    if (compact_) {
      // The kept-row counts decide the output shapes.  ATen's nonzero / masked index
      // synchronise the stream for that; here the counts arrive through pinned memory early
      // in the second pass, and the outputs are valid in stream order.
      // (a caller that holds the interpreter's lock: a short poll first, and word before the long wait)
      int ready = 0;
      if (hook) {
        ready = fx_region_poll_totals(plan, (const uint32_t*)ws.totals.data_ptr(), 200u);
        FX_OK_OR_THROW(ready < 0 ? ready : 0);
      }
      if (!ready) {
        BlockingScope scope(hook);
        FX_OK_OR_THROW(fx_region_wait_totals(plan, (const uint32_t*)ws.totals.data_ptr(), (void*)stream.stream()));
      }
      clock.tick(HS_WAIT);
      const int32_t* tot = ws.totals.data_ptr<int32_t>();
      for (int o = 0; o < n_out; ++o)
        for (int64_t t = 0; t < degree; ++t) {
          const Slot& sl = slot_of[(size_t)o * degree + t];
          int64_t sizes[FX_ARG_MAX_RANK];
          std::copy(sl.sizes, sl.sizes + sl.rank, sizes);
          sizes[0] = tot[t];
          at::Tensor& out = degree == 1 ? buffers[o] : flat[(size_t)o * degree + t];
          out.unsafeGetTensorImpl()->set_sizes_contiguous(at::IntArrayRef(sizes, sl.rank));
        }
      var->give(std::move(ws));
    }
    clock.tick(HS_RESIZE);
    drop(stack, n_stack_);
    for (int o = 0; o < n_out; ++o) {
      if (!is_map_) {
        push(stack, std::move(buffers[o]));
        continue;
      }
      c10::List<at::Tensor> list;
      list.reserve(degree);
      if (degree == 1) list.push_back(std::move(buffers[o]));
      else
        for (int64_t t = 0; t < degree; ++t) list.push_back(std::move(flat[(size_t)o * degree + t]));
      push(stack, std::move(list));
    }
    clock.tick(HS_PUSH);
    if (clock.on) g_host_calls.fetch_add(1, std::memory_order_relaxed);
  }

  // What the library makes of the region for arguments of these types (meta tensors stand for
  // them; nothing runs): `kind` is the first word of fx_plan_head_info when that kernel is in
  // use (0: the generic kernels), `shapes` the shapes of task 0's results.
  void dryRun(const std::vector<c10::IValue>& samples, int64_t* kind, std::vector<std::vector<int64_t>>* shapes,
              int64_t* rowstream = nullptr, std::string* rowstream_why = nullptr, std::vector<c10::ScalarType>* dtypes = nullptr,
              int64_t* kernels = nullptr) {
    TORCH_CHECK(samples.size() == n_stack_, "dryRun: argument count");
    int64_t degree = degree_;
    size_t first = 0;
    if (degree_ < 0) {
      degree = samples[0].toInt();
      first = 1;
    }
    if (!is_map_) degree = 1;
    TORCH_CHECK(degree >= 1, "dryRun: empty map");
    std::vector<fx_arg> args;
    Signature sig;
    c10::Device device(c10::kCPU);
    bool have_device = false;
    flatten(samples, first, degree, /*dry=*/true, args, sig, device, have_device);
    Variant var;
    build(var, degree, samples, first);
    const fx_plan* plan = nullptr;
    FX_OK_OR_THROW(fx_region_plan(var.region, args.data(), (int)args.size(), &plan));
    int64_t info[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    FX_OK_OR_THROW(fx_plan_head_info(plan, info, 8));
    *kind = info[1] ? info[0] : 0;
    if (kernels) {   // [0]: compiled kernels are linked for the region's programs, [1]: a dense region on the lean kernel
      kernels[0] = fx_plan_specialized(plan);
      kernels[1] = fx_plan_dense_lean(plan);
    }
    if (rowstream) {
      FX_OK_OR_THROW(fx_plan_rowstream_info(plan, rowstream, 8));
      if (rowstream_why) {
        char buf[256];
        buf[0] = 0;
        fx_plan_rowstream_why(plan, buf, sizeof buf);
        *rowstream_why = buf;
      }
    }
    shapes->clear();
    for (int o = 0; o < fx_plan_num_outputs(plan); ++o) {
      int32_t dt = 0, rank = 0;
      int64_t sizes[FX_ARG_MAX_RANK];
      FX_OK_OR_THROW(fx_plan_output(plan, o, 0, &dt, &rank, sizes));
      shapes->emplace_back(sizes, sizes + rank);
      if (dtypes) dtypes->push_back(atDtype(dt));
    }
  }

 private:
  std::shared_ptr<Graph> graph_;
  std::vector<int64_t> is_par_;
  int64_t degree_;
  bool is_map_, compact_, padded_;
  size_t n_args_ = 0, n_stack_ = 0, n_outs_ = 0;
  std::mutex mu_;
  std::map<std::string, std::unique_ptr<Variant>> variants_;

  // The arguments as the C ABI takes them (tensors by pointer, sizes and strides; lists and tuples
  // of scalars as their elements) and the signature that selects the region variant.  `dry`:
  // tensors stand for their types only (no device, no pointer).
  void flatten(at::ArrayRef<c10::IValue> inputs, size_t first, int64_t degree, bool dry, std::vector<fx_arg>& args,
               Signature& sig, c10::Device& device, bool& have_device) {
    sig << degree;
    auto addTensor = [&](const at::Tensor& t) {
      TORCH_CHECK(dry || t.is_cuda(), "tssa::ParallelFunctor runs on the GPU only; got a ", t.device(), " tensor");
      TORCH_CHECK(t.dim() <= FX_ARG_MAX_RANK, "tensor rank above ", FX_ARG_MAX_RANK);
      if (!have_device) { device = t.device(); have_device = true; }
      fx_arg a;
      memset(&a, 0, sizeof(a));
      a.kind = 0;
      a.dtype = fxDtype(t.scalar_type());
      a.ptr = dry ? nullptr : t.data_ptr();
      a.rank = (int32_t)t.dim();
      for (int64_t d = 0; d < t.dim(); ++d) { a.sizes[d] = t.size(d); a.strides[d] = t.stride(d); }
      args.push_back(a);
      sig << "|t" << a.dtype << "r" << a.rank;
    };
    auto addScalar = [&](const c10::IValue& v) {
      fx_arg a;
      memset(&a, 0, sizeof(a));
      if (v.isDouble()) { a.kind = 2; a.fval = v.toDouble(); sig << "|f"; }
      else if (v.isBool()) { a.kind = 3; a.ival = v.toBool(); sig << "|b"; }
      else if (v.isInt()) { a.kind = 1; a.ival = v.toInt(); sig << "|i"; }
      else if (v.isDevice() || v.isNone()) { a.kind = 1; a.ival = 0; sig << "|d"; }  // placement only: outputs follow the tensors
      else TORCH_CHECK(false, "ParallelFunctor: unsupported scalar argument ", v.tagKind());
      args.push_back(a);
    };
    // A value that is itself a list or tuple of scalars (int[], float[], bool[], Tuple[int, ...];
    // per task: List[List[int]], List[Tuple[int, int]] ..., graph_builder.cpp:736-857) travels as
    // its elements; their number is part of the signature.  All tasks must agree on it.
    auto addValue = [&](const c10::IValue& v, size_t k, int64_t* n_elems) {
      if (v.isTensor()) { addTensor(v.toTensor()); return; }
      if (v.isList() || v.isTuple()) {
        const auto elems = v.isList() ? v.toListRef() : at::ArrayRef<c10::IValue>(v.toTupleRef().elements());
        TORCH_CHECK(*n_elems < 0 || *n_elems == (int64_t)elems.size(), "ParallelFunctor: argument ", k,
                    ": the tasks' lists differ in length");
        if (*n_elems < 0) sig << "|L" << elems.size();
        *n_elems = (int64_t)elems.size();
        for (const c10::IValue& e : elems) {
          TORCH_CHECK(!e.isTensor() && !e.isList() && !e.isTuple(), "ParallelFunctor: argument ", k,
                      ": nested lists of this kind are not supported");
          addScalar(e);
        }
        return;
      }
      addScalar(v);
    };
    for (size_t k = 0; k < n_args_; ++k) {
      const c10::IValue& v = inputs[first + k];
      const bool per_task = is_map_ && is_par_[k] != 0;
      int64_t n_elems = -1;
      if (per_task) {
        TORCH_CHECK(v.isList(), "ParallelFunctor: argument ", k, " must be a list with one entry per task");
        auto lst = v.toListRef();
        TORCH_CHECK((int64_t)lst.size() >= degree, "ParallelFunctor: list argument ", k, " is shorter than the trip count");
        // element-major: all tasks' first elements, then all second elements ... (one region input each)
        if (degree > 0 && (lst[0].isList() || lst[0].isTuple())) {
          const auto first_elems = lst[0].isList() ? lst[0].toListRef() : at::ArrayRef<c10::IValue>(lst[0].toTupleRef().elements());
          const size_t n = first_elems.size();
          sig << "|L" << n;
          for (size_t e = 0; e < n; ++e)
            for (int64_t t = 0; t < degree; ++t) {
              const auto elems = lst[t].isList() ? lst[t].toListRef() : at::ArrayRef<c10::IValue>(lst[t].toTupleRef().elements());
              TORCH_CHECK(elems.size() == n, "ParallelFunctor: argument ", k, ": the tasks' lists differ in length");
              TORCH_CHECK(!elems[e].isTensor() && !elems[e].isList() && !elems[e].isTuple(), "ParallelFunctor: argument ",
                          k, ": nested lists of this kind are not supported");
              addScalar(elems[e]);
            }
        } else {
          for (int64_t t = 0; t < degree; ++t) addValue(lst[t], k, &n_elems);
        }
      } else {
        addValue(v, k, &n_elems);
      }
    }
  }

  void build(Variant& var, int64_t degree, at::ArrayRef<c10::IValue> inputs, size_t first);
};

// --- subgraph -> region -----------------------------------------------------
struct Translator {
  fx_region* r;
  std::unordered_map<const Value*, int> ids;
  // list- or tuple-valued subgraph parameters: the region inputs that carry their elements
  std::unordered_map<const Value*, std::vector<int>> elements;

  int cint(int64_t v) { int id; FX_OK_OR_THROW(fx_region_const_int(r, v, &id)); return id; }
  int cfloat(double v) { int id; FX_OK_OR_THROW(fx_region_const_float(r, v, &id)); return id; }
  int cbool(bool v) { int id; FX_OK_OR_THROW(fx_region_const_bool(r, v, &id)); return id; }
  int cnone() { int id; FX_OK_OR_THROW(fx_region_const_none(r, &id)); return id; }
  int ilist(const std::vector<int>& v) { int id; FX_OK_OR_THROW(fx_region_int_list(r, v.data(), (int)v.size(), &id)); return id; }
  int tlist(const std::vector<int>& v) { int id; FX_OK_OR_THROW(fx_region_tensor_list(r, v.data(), (int)v.size(), &id)); return id; }
  int op(int code, std::vector<int> args, int dtype = -1) {
    int id;
    FX_OK_OR_THROW(fx_region_op(r, code, args.data(), (int)args.size(), dtype, &id));
    return id;
  }

  int get(const Value* v) {
    auto it = ids.find(v);
    if (it != ids.end()) return it->second;
    const Node* n = v->node();
    TORCH_CHECK(n->kind() == c10::prim::Constant, "ParallelFunctor: value %", v->debugName(), " has no region value");
    auto iv = toIValue(v);
    TORCH_CHECK(iv, "bad constant");
    int id;
    if (iv->isNone()) id = cnone();
    else if (iv->isBool()) id = cbool(iv->toBool());
    else if (iv->isInt()) id = cint(iv->toInt());
    else if (iv->isDouble()) id = cfloat(iv->toDouble());
    else if (iv->isIntList()) {
      std::vector<int> e;
      for (int64_t x : iv->toIntVector()) e.push_back(cint(x));
      id = ilist(e);
    } else if (iv->isDevice() || iv->isString()) id = cnone();
    else TORCH_CHECK(false, "ParallelFunctor: constant of type ", iv->tagKind(), " inside a fused region");
    ids[v] = id;
    return id;
  }

  // dtype argument (ScalarType constant or None) -> fx dtype or -1
  int dtypeArg(const Value* v) {
    auto iv = toIValue(v);
    TORCH_CHECK(iv, "ParallelFunctor: a dtype operand inside a fused region must be a constant");
    if (iv->isNone()) return -1;
    return fxDtype(static_cast<c10::ScalarType>(iv->toInt()));
  }

  void node(const Node* n);
  void block(const Block* b) {
    for (const Node* n : b->nodes()) node(n);
  }
};

void Translator::node(const Node* n) {
  using namespace c10;
  const Symbol k = n->kind();
  auto in = [&](size_t i) { return get(n->input(i)); };
  auto out = [&](int id) { ids[n->output(0)] = id; };
  const size_t ni = n->inputs().size();
  if (k == prim::Constant) return;  // created on demand
  if (k == aten::size && ni == 1) {  // all sizes: the tensor itself stands for them
    out(in(0));
    return;
  }
  if (k == prim::TupleUnpack || k == prim::ListUnpack) {
    auto it = elements.find(n->input(0));
    TORCH_CHECK(it != elements.end() && it->second.size() == n->outputs().size(),
                "ParallelFunctor: ", k.toQualString(), " of a value that is not a region argument");
    for (size_t i = 0; i < n->outputs().size(); ++i) ids[n->output(i)] = it->second[i];
    return;
  }
  if (k == aten::__getitem__ && elements.count(n->input(0))) {  // list[const]
    auto idx = constant_as<int64_t>(n->input(1));
    const auto& e = elements.at(n->input(0));
    TORCH_CHECK(idx, "ParallelFunctor: a list argument can only be read at a constant position inside a region");
    const int64_t i = *idx < 0 ? *idx + (int64_t)e.size() : *idx;
    TORCH_CHECK(i >= 0 && i < (int64_t)e.size(), "ParallelFunctor: list index out of range");
    out(e[(size_t)i]);
    return;
  }
  if (k == prim::ListConstruct) {
    std::vector<int> e;
    for (const Value* v : n->inputs()) e.push_back(get(v));
    auto lt = n->output()->type()->cast<ListType>();
    bool ints = lt && lt->getElementType()->kind() == TypeKind::IntType;
    out(ints ? ilist(e) : tlist(e));
    return;
  }
  struct Simple { Symbol s; int code; };
  static const std::vector<Simple> unary{
      {aten::exp, FX_OP_EXP}, {aten::log, FX_OP_LOG}, {aten::sqrt, FX_OP_SQRT}, {aten::rsqrt, FX_OP_RSQRT},
      {aten::sigmoid, FX_OP_SIGMOID}, {aten::tanh, FX_OP_TANH}, {aten::relu, FX_OP_RELU}, {aten::abs, FX_OP_ABS},
      {aten::floor, FX_OP_FLOOR}, {aten::ceil, FX_OP_CEIL}, {aten::round, FX_OP_ROUND}, {aten::sin, FX_OP_SIN},
      {aten::cos, FX_OP_COS}, {aten::erf, FX_OP_ERF}, {aten::reciprocal, FX_OP_RECIPROCAL},
      {aten::logical_not, FX_OP_LOGICAL_NOT}, {sym::Access(), FX_OP_ACCESS}};
  for (auto& u : unary)
    if (u.s == k) { out(op(u.code, {in(0)})); return; }
  static const std::vector<Simple> binary{
      {aten::mul, FX_OP_MUL}, {aten::div, FX_OP_DIV}, {aten::maximum, FX_OP_MAXIMUM}, {aten::minimum, FX_OP_MINIMUM},
      {aten::pow, FX_OP_POW}, {aten::eq, FX_OP_EQ}, {aten::ne, FX_OP_NE}, {aten::lt, FX_OP_LT}, {aten::le, FX_OP_LE},
      {aten::gt, FX_OP_GT}, {aten::ge, FX_OP_GE}, {aten::__and__, FX_OP_AND}, {aten::__or__, FX_OP_OR},
      {aten::__xor__, FX_OP_XOR}};
  const bool tensor_out = isTensorValue(n->output(0));
  if (!tensor_out && n->output(0)->type()->kind() == TypeKind::IntType) {
    // integer scalar arithmetic on index values
    if (k == aten::add) { out(op(FX_OP_INT_ADD, {in(0), in(1)})); return; }
    if (k == aten::sub) { out(op(FX_OP_INT_SUB, {in(0), in(1)})); return; }
    if (k == aten::mul) { out(op(FX_OP_INT_MUL, {in(0), in(1)})); return; }
    if (k == aten::neg) { out(op(FX_OP_INT_NEG, {in(0)})); return; }
    if (k == aten::size && ni == 2) { out(op(FX_OP_SIZE, {in(0), in(1)})); return; }
    if (k == aten::__derive_index) {  // start + index * step
      out(op(FX_OP_INT_ADD, {in(1), op(FX_OP_INT_MUL, {in(0), in(2)})}));
      return;
    }
  }
  for (auto& b : binary)
    if (b.s == k) { out(op(b.code, {in(0), in(1)})); return; }
  if (k == aten::add || k == aten::sub || k == aten::rsub) {
    int code = k == aten::add ? FX_OP_ADD : (k == aten::sub ? FX_OP_SUB : FX_OP_RSUB);
    out(ni > 2 ? op(code, {in(0), in(1), in(2)}) : op(code, {in(0), in(1)}));
    return;
  }
  if (k == aten::neg) { out(op(FX_OP_NEG, {in(0)})); return; }
  if (k == aten::clone || k == aten::contiguous) { out(op(FX_OP_CLONE, {in(0)})); return; }
  if (k == sym::Assign()) { out(op(FX_OP_ASSIGN, {in(0), in(1)})); return; }
  if (k == aten::select || k == sym::Select()) { out(op(FX_OP_SELECT, {in(0), in(1), in(2)})); return; }
  if (k == sym::SelectRev()) { out(op(FX_OP_SELECT_REV, {in(0), in(1), in(2), in(3)})); return; }
  if (k == aten::slice || k == sym::Slice()) { out(op(FX_OP_SLICE, {in(0), in(1), in(2), in(3), in(4)})); return; }
  if (k == sym::SliceRev()) { out(op(FX_OP_SLICE_REV, {in(0), in(1), in(2), in(3), in(4), in(5)})); return; }
  if (k == aten::squeeze || k == sym::Squeeze()) {
    TORCH_CHECK(ni == 2, "squeeze without a dim inside a fused region");
    out(op(FX_OP_SQUEEZE, {in(0), in(1)}));
    return;
  }
  if (k == aten::unsqueeze || k == sym::Unsqueeze()) { out(op(FX_OP_UNSQUEEZE, {in(0), in(1)})); return; }
  if (k == aten::view || k == aten::reshape || k == sym::View() || k == sym::Reshape()) {
    out(op(FX_OP_VIEW, {in(0), in(1)}));
    return;
  }
  if (k == aten::permute || k == sym::Permute()) { out(op(FX_OP_PERMUTE, {in(0), in(1)})); return; }
  if (k == aten::transpose) { out(op(FX_OP_TRANSPOSE, {in(0), in(1), in(2)})); return; }
  if (k == aten::expand || k == sym::Expand()) { out(op(FX_OP_EXPAND, {in(0), in(1)})); return; }
  if (k == aten::expand_as || k == sym::ExpandAs()) { out(op(FX_OP_EXPAND_AS, {in(0), in(1)})); return; }
  if (k == aten::repeat || k == sym::Repeat()) { out(op(FX_OP_REPEAT, {in(0), in(1)})); return; }
  if (k == aten::index || k == sym::Index()) { out(op(FX_OP_INDEX, {in(0), in(1)})); return; }
  if (k == aten::cat) { out(op(FX_OP_CAT, {in(0), in(1)})); return; }
  if (k == aten::stack) { out(op(FX_OP_STACK, {in(0), in(1)})); return; }
  if (k == aten::triu) { out(op(FX_OP_TRIU, {in(0), in(1)})); return; }
  if (k == aten::tril) { out(op(FX_OP_TRIL, {in(0), in(1)})); return; }
  if (k == aten::clamp) { out(op(FX_OP_CLAMP, {in(0), in(1), in(2)})); return; }
  if (k == aten::where) { out(op(FX_OP_WHERE, {in(0), in(1), in(2)})); return; }
  if (k == aten::softmax) { out(op(FX_OP_SOFTMAX, {in(0), in(1)})); return; }
  if (k == aten::max) {
    TORCH_CHECK(ni >= 2 && n->outputs().size() == 2 && !n->output(1)->hasUses(),
                "aten::max.dim: only the values output can be fused");
    out(op(FX_OP_MAX_DIM, {in(0), in(1), ni > 2 ? in(2) : cbool(false)}));
    return;
  }
  if (k == aten::zeros || k == aten::ones) {
    int dt = dtypeArg(n->input(1));
    out(op(FX_OP_FULL, {in(0), cfloat(k == aten::ones ? 1.0 : 0.0)}, dt < 0 ? FX_DT_F32 : dt));
    return;
  }
  if (k == aten::full) {
    int dt = dtypeArg(n->input(2));
    out(op(FX_OP_FULL, {in(0), in(1)}, dt < 0 ? FX_DT_F32 : dt));
    return;
  }
  if (k == aten::zeros_like || k == aten::ones_like) {
    out(op(FX_OP_FULL, {in(0), cfloat(k == aten::ones_like ? 1.0 : 0.0)}, dtypeArg(n->input(1))));
    return;
  }
  if (k == aten::full_like) {
    out(op(FX_OP_FULL, {in(0), in(1)}, dtypeArg(n->input(2))));
    return;
  }
  if (k == aten::arange) {
    TORCH_CHECK(ni >= 3, "aten::arange: only the (start, end, ...) form can be fused");
    int dt = dtypeArg(n->input(2));
    out(op(FX_OP_ARANGE, {in(0), in(1)}, dt < 0 ? FX_DT_I64 : dt));
    return;
  }
  if (k == aten::tensor) {
    int dt = dtypeArg(n->input(1));
    // a short constant list (torch.tensor([0.1, 0.1, 0.2, 0.2])): its elements stacked
    auto iv = toIValue(n->input(0));
    if (iv && (iv->isDoubleList() || iv->isIntList() || iv->isBoolList())) {
      std::vector<int> elems;
      if (iv->isDoubleList())
        for (double x : iv->toDoubleVector()) elems.push_back(op(FX_OP_SCALAR_TENSOR, {cfloat(x)}, dt < 0 ? FX_DT_F32 : dt));
      else if (iv->isIntList())
        for (int64_t x : iv->toIntVector()) elems.push_back(op(FX_OP_SCALAR_TENSOR, {cint(x)}, dt < 0 ? FX_DT_I64 : dt));
      else
        for (bool x : iv->toBoolList()) elems.push_back(op(FX_OP_SCALAR_TENSOR, {cbool(x)}, dt < 0 ? FX_DT_BOOL : dt));
      TORCH_CHECK(!elems.empty() && elems.size() <= 64, "aten::tensor of ", elems.size(), " constants inside a fused region");
      out(op(FX_OP_STACK, {tlist(elems), cint(0)}));
      return;
    }
    out(op(FX_OP_SCALAR_TENSOR, {in(0)}, dt));
    return;
  }
  if (k == aten::to) {
    // to.dtype(self, dtype, ...) / to.device(self, device, dtype, ...)
    int dt = -1;
    for (size_t i = 1; i < ni && dt < 0; ++i)
      if (n->input(i)->type()->kind() == TypeKind::IntType) dt = dtypeArg(n->input(i));
    TORCH_CHECK(dt >= 0, "aten::to without a dtype inside a fused region");
    out(op(FX_OP_TO, {in(0)}, dt));
    return;
  }
  if (k == sym::ForallSelectRev()) {
    // (T0, dim, lo, hi, captured...) { block(i, T, captured'...) -> src }
    const Block* b = n->blocks()[0];
    int lv;
    FX_OK_OR_THROW(fx_region_loop_var(r, &lv));
    ids[b->inputs()[0]] = lv;
    ids[b->inputs()[1]] = in(0);
    for (size_t c = 2; c < b->inputs().size(); ++c) ids[b->inputs()[c]] = in(2 + c);
    block(b);
    out(op(FX_OP_FORALL_SELECT_REV, {in(0), get(b->outputs()[0]), in(1), in(2), in(3)}));
    return;
  }
  TORCH_CHECK(false, "ParallelFunctor: no lowering for ", k.toQualString());  // graph_builder.cpp:409-414
}

void RegionRunner::build(Variant& var, int64_t degree, at::ArrayRef<c10::IValue> inputs, size_t first) {
  FX_OK_OR_THROW(fx_region_create((int)degree, is_map_ ? 1 : 0, &var.region));
  Translator tr{var.region, {}};
  // input 0: the task index
  const Value* idx = graph_->inputs()[0];
  if (idx->type()->kind() == c10::TypeKind::IntType) {
    int id;
    FX_OK_OR_THROW(fx_region_task_index(var.region, &id));
    tr.ids[idx] = id;
  }
  for (size_t k = 0; k < n_args_; ++k) {
    const Value* p = graph_->inputs()[k + 1];
    const c10::IValue& v = inputs[first + k];
    const bool per_task = is_map_ && is_par_[k] != 0;
    c10::IValue sample = v;
    if (per_task) sample = v.toListRef().at(0);
    int id;
    auto scalarInput = [&](const c10::IValue& e) {
      int sid;
      const int kind = e.isDouble() ? 2 : (e.isBool() ? 3 : 1);
      FX_OK_OR_THROW(fx_region_input_scalar(var.region, kind, per_task, &sid));
      return sid;
    };
    if (sample.isTensor()) {
      const at::Tensor& t = sample.toTensor();
      FX_OK_OR_THROW(fx_region_input_tensor(var.region, fxDtype(t.scalar_type()), (int)t.dim(), per_task, &id));
    } else if (sample.isList() || sample.isTuple()) {
      // one scalar input per element; an int[] becomes a size list, a tuple waits for its TupleUnpack
      const auto elems = sample.isList() ? sample.toListRef() : at::ArrayRef<c10::IValue>(sample.toTupleRef().elements());
      std::vector<int> eids;
      bool ints = true;
      for (const c10::IValue& e : elems) {
        eids.push_back(scalarInput(e));
        ints = ints && e.isInt();
      }
      tr.elements[p] = eids;
      if (sample.isList() && ints) tr.ids[p] = tr.ilist(eids);
      continue;
    } else {
      id = scalarInput(sample);
    }
    tr.ids[p] = id;
  }
  tr.block(graph_->block());
  const size_t n_sub_out = graph_->outputs().size();
  for (size_t o = 0; o < n_sub_out; ++o) {
    int id = tr.get(graph_->outputs()[o]);
    if (compact_ && o + 1 == n_sub_out) FX_OK_OR_THROW(fx_region_compact_rows(var.region, id));
    else FX_OK_OR_THROW(fx_region_output(var.region, id));
  }
  FX_OK_OR_THROW(fx_region_finalize(var.region));
}

// --- fx::lstm_stack -----------------------------------------------------------
// Control words and the h exchange buffer of the persistent kernel, one per (device, stream) and
// shape (batch, hidden, layers): cleared when allocated, and every launch that ends without error
// leaves them ready for the next one (include/fxhip.h fx_lstm_stack), so a call costs the one launch.
struct LstmWorkspaces {
  std::mutex mu;
  std::map<std::tuple<int, void*, int64_t, int64_t, int64_t>, at::Tensor> by_stream;
  at::Tensor get(c10::Device dev, void* stream, int64_t B, int64_t H, int64_t L) {
    std::lock_guard<std::mutex> lock(mu);
    at::Tensor& t = by_stream[{(int)dev.index(), stream, B, H, L}];
    if (!t.defined()) {
      const size_t bytes = fx_lstm_stack_workspace_bytes((int)B, (int)H, (int)L);
      t = at::zeros({(int64_t)bytes}, at::TensorOptions().dtype(at::kByte).device(dev));   // on the current stream
    }
    return t;
  }
  void reset() {
    std::lock_guard<std::mutex> lock(mu);
    by_stream.clear();
  }
};
LstmWorkspaces& lstmWorkspaces() {
  static LstmWorkspaces* w = new LstmWorkspaces();   // tensors must not outlive the HIP runtime's teardown order
  return *w;
}
void resetLstmWorkspaces() { lstmWorkspaces().reset(); }

// fx::lstm_stack(x, wih, whh, bih, bhh, out?, state_h?, state_c?, T, L) -> (out, state_h, state_c)
// is the loop nest
//   for t in range(T): cur = x[t]
//     for j in range(L): (the LSTM cell of layer j on cur, state_h[j], state_c[j]); cur = h
//     out[t] = cur
// in functional form: the results are new tensors, rows [0, T) of out and layers [0, L) of the
// states rewritten, the rest copied from the operands.  None for out means a [T, B, H] buffer that
// the loops fill completely, None for a state means zeros [L, B, H].
void runLstmStack(Stack& stack) {
  auto in = last(stack, 10);
  auto tensorArg = [&](size_t i, const char* name) {
    TORCH_CHECK(in[i].isTensor(), "fx::lstm_stack: ", name, " must be a tensor");
    at::Tensor t = in[i].toTensor();
    TORCH_CHECK(t.is_cuda(), "fx::lstm_stack runs on the GPU only; ", name, " is a ", t.device(), " tensor");
    TORCH_CHECK(t.scalar_type() == at::kFloat, "fx::lstm_stack: ", name, " must be float32");
    return t.contiguous();
  };
  auto optionalArg = [&](size_t i, const char* name) { return in[i].isNone() ? at::Tensor() : tensorArg(i, name); };
  const at::Tensor x = tensorArg(0, "x"), wih = tensorArg(1, "wih"), whh = tensorArg(2, "whh"), bih = tensorArg(3, "bih"),
                   bhh = tensorArg(4, "bhh");
  const at::Tensor out0 = optionalArg(5, "out"), h0 = optionalArg(6, "state_h"), c0 = optionalArg(7, "state_c");
  const int64_t T = std::max<int64_t>(in[8].toInt(), 0), L = std::max<int64_t>(in[9].toInt(), 0);   // a negative trip count runs no iteration
  TORCH_CHECK(x.dim() == 3, "fx::lstm_stack: x must be [T, B, H]");
  const int64_t B = x.size(1), H = x.size(2);
  TORCH_CHECK(T <= x.size(0), "fx::lstm_stack: index ", x.size(0), " is out of bounds for dimension 0 of x with size ", x.size(0));
  auto weightArg = [&](const at::Tensor& w, const char* name, int64_t rows) {
    TORCH_CHECK(w.dim() == 4 && w.size(1) == 4 && w.size(2) == rows && w.size(3) == H && w.size(0) >= L,
                "fx::lstm_stack: ", name, " must be [layers >= ", L, ", 4, ", rows, ", ", H, "], got ", w.sizes());
  };
  weightArg(wih, "wih", H);
  weightArg(whh, "whh", H);
  weightArg(bih, "bih", 1);
  weightArg(bhh, "bhh", 1);
  TORCH_CHECK(wih.size(0) == L || L == 0 || (wih.size(0) == whh.size(0) && bih.size(0) == bhh.size(0)),
              "fx::lstm_stack: the weights disagree on the number of layers");
  auto rowsArg = [&](const at::Tensor& t, const char* name, int64_t need) {
    if (!t.defined()) return need;
    TORCH_CHECK(t.dim() == 3 && t.size(1) == B && t.size(2) == H && t.size(0) >= need, "fx::lstm_stack: ", name,
                " must be [>= ", need, ", ", B, ", ", H, "], got ", t.sizes());
    return t.size(0);
  };
  const int64_t To = rowsArg(out0, "out", T), Lh = rowsArg(h0, "state_h", L), Lc = rowsArg(c0, "state_c", L);
  if (!out0.defined() || !h0.defined() || !c0.defined())
    TORCH_CHECK(c10::get_default_dtype_as_scalartype() == at::kFloat,
                "fx::lstm_stack: the program creates its buffers with the default dtype, which must be float32");
  c10::DeviceGuard guard(x.device());
  const auto opts = x.options();
  const bool runs = T > 0 && L > 0;
  // a result whose every element the kernel writes starts uninitialised, any other one as a copy
  auto result = [&](const at::Tensor& init, int64_t rows, bool all_written) {
    if (all_written) return at::empty({rows, B, H}, opts);
    return init.defined() ? init.clone() : at::zeros({rows, B, H}, opts);
  };
  at::Tensor out = result(out0, To, runs && To == T);
  at::Tensor sh = result(h0, Lh, runs && Lh == L);
  at::Tensor sc = result(c0, Lc, runs && Lc == L);
  if (T > 0 && L == 0) out.narrow(0, 0, T).copy_(x.narrow(0, 0, T));   // no layer: out[t] = x[t]
  if (runs) {
    checkAsyncError();
    TORCH_CHECK(T <= INT32_MAX && B <= INT32_MAX && H <= INT32_MAX, "fx::lstm_stack: sizes beyond 32 bits");
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(x.device().index());
    at::Tensor ws = lstmWorkspaces().get(x.device(), (void*)stream.stream(), B, H, L);
    TORCH_CHECK(((uintptr_t)ws.data_ptr() & 255u) == 0, "fx::lstm_stack: workspace is not 256-byte aligned");
    FX_OK_OR_THROW(fx_lstm_stack(x.data_ptr<float>(), wih.data_ptr<float>(), whh.data_ptr<float>(), bih.data_ptr<float>(),
                                 bhh.data_ptr<float>(), h0.defined() ? h0.data_ptr<float>() : nullptr,
                                 c0.defined() ? c0.data_ptr<float>() : nullptr, out.data_ptr<float>(), sh.data_ptr<float>(),
                                 sc.data_ptr<float>(), (int)T, (int)B, (int)H, (int)L, ws.data_ptr(), (size_t)ws.numel(),
                                 (void*)stream.stream()));
  }
  drop(stack, 10);
  push(stack, std::move(out));
  push(stack, std::move(sh));
  push(stack, std::move(sc));
}

// the region of a functor made by functorFromLstmStack: one fx::lstm_stack node over the arguments
const Node* loneLstmStack(const Graph& sub) {
  const Node* found = nullptr;
  for (const Node* n : sub.nodes()) {
    if (n->kind() == c10::prim::Constant) continue;
    if (n->kind() != sym::LstmStack() || found) return nullptr;
    found = n;
  }
  return found;
}

Operation createParallelFunctor(const Node* node) {
  auto sub = node->g(c10::attr::Subgraph);
  if (const Node* k = loneLstmStack(*sub)) {
    // operand i of the node: argument number (position among the functor's inputs) or a constant
    struct Operand { int arg; c10::IValue constant; };
    std::vector<Operand> operands;
    for (const Value* v : k->inputs()) {
      if (v->node()->kind() == c10::prim::Constant) {
        operands.push_back({-1, *toIValue(v)});
        continue;
      }
      size_t pos = 0;
      while (pos < sub->inputs().size() && sub->inputs()[pos] != v) ++pos;
      TORCH_CHECK(pos >= 1 && pos < sub->inputs().size(), "ParallelFunctor: fx::lstm_stack operand is not an argument");
      operands.push_back({(int)pos - 1, c10::IValue()});
    }
    const size_t n_args = sub->inputs().size() - 1;
    return [operands, n_args](Stack& stack) {
      std::vector<c10::IValue> args;
      for (const c10::IValue& v : last(stack, n_args)) args.push_back(v);
      drop(stack, n_args);
      for (const Operand& o : operands) stack.push_back(o.arg < 0 ? o.constant : args[(size_t)o.arg]);
      runLstmStack(stack);
    };
  }
  auto runner = std::make_shared<RegionRunner>(node);
  return [runner](Stack& stack) { runner->run(stack); };
}

RegisterOperators registerFunctor({
    Operator(sym::ParallelFunctor(), createParallelFunctor, c10::AliasAnalysisKind::PURE_FUNCTION),
    // the collapsed node itself is an operator too: graphs that hold it outside a functor (between
    // the passes, or when ToParallelFunctor is not run) analyse and execute
    Operator("fx::lstm_stack(Tensor x, Tensor wih, Tensor whh, Tensor bih, Tensor bhh, Tensor? out, Tensor? state_h, "
             "Tensor? state_c, int T, int L) -> (Tensor, Tensor, Tensor)",
             [](Stack& stack) { runLstmStack(stack); }, c10::AliasAnalysisKind::PURE_FUNCTION),
});


// ---------------------------------------------------------------------------
// pass: a dense producer sinks into the class map that consumes it
// ---------------------------------------------------------------------------
std::atomic<bool> g_sink_producers{true};

bool isPlainFunctor(const Node* n) {
  return n->kind() == sym::ParallelFunctor() && n->i(sym::is_parallel_map()) == 0 &&
         (!n->hasAttribute(sym::compact_rows()) || n->i(sym::compact_rows()) == 0);
}

// The dry runs of the passes plan regions that the built graph may not keep (a producer before it
// sinks, a merged functor that is not taken): those leave no sources in a capture directory.
struct NoSourceDump {
  int before;
  NoSourceDump() : before(fx_spec_dump_what(0)) {}
  ~NoSourceDump() { fx_spec_dump_what(before); }
};

// a meta tensor of a complete static type
bool sampleOf(const c10::TypePtr& type, c10::IValue* out) {
  auto tt = type->cast<c10::TensorType>();
  if (!tt || !tt->scalarType()) return false;
  auto sizes = tt->sizes().concrete_sizes();
  if (!sizes) return false;
  // a type without strides stands for the contiguous layout (another layout at run time gets its
  // own plan, as always)
  auto strides = tt->strides().concrete_sizes();
  const auto options = at::TensorOptions().dtype(*tt->scalarType()).device(c10::kMeta);
  *out = strides ? at::empty_strided(*sizes, *strides, options) : at::empty(*sizes, options);
  return true;
}

// what stands for a functor argument when the region is only lowered: a meta tensor of its static
// type, the value of a constant, any device for a device (placement does not enter the lowering)
bool sampleOfArg(const c10::TypePtr& type, Value* v, c10::IValue* out) {
  if (sampleOf(type, out)) return true;
  if (auto c = toIValue(v)) {
    *out = *c;
    return true;
  }
  if (v->type()->kind() == c10::TypeKind::DeviceObjType) {
    *out = c10::IValue(c10::Device(c10::kCPU));
    return true;
  }
  return false;
}

// F1 = plain functor, F2 = compacting map functor that reads F1's results as shared arguments.
// Returns true if the graph changed.
bool trySinkProducer(Node* f2, Node* f1);

bool trySink(Node* f2) {
  const auto par2 = f2->is(sym::is_parallel_args());
  const size_t first2 = f2->i(sym::parallel_degree()) < 0 ? 1 : 0;
  // the plain functors among the producers of F2's shared arguments, the last one first: of a
  // chain of producers the one next to the map sinks first, then the one that fed it
  std::vector<Node*> producers;
  for (size_t k = first2; k < f2->inputs().size(); ++k) {
    Node* p = f2->input(k)->node();
    if (par2[k - first2] != 0 || !isPlainFunctor(p) || p->owningBlock() != f2->owningBlock()) continue;
    if (std::find(producers.begin(), producers.end(), p) == producers.end()) producers.push_back(p);
  }
  std::sort(producers.begin(), producers.end(), [](Node* a, Node* b) { return b->isBefore(a); });
  for (Node* f1 : producers)
    if (trySinkProducer(f2, f1)) return true;
  return false;
}

bool trySinkProducer(Node* f2, Node* f1) {
  Graph* g = f2->owningGraph();
  const auto par2 = f2->is(sym::is_parallel_args());
  const size_t first2 = f2->i(sym::parallel_degree()) < 0 ? 1 : 0;
  for (Node* n : f1->g(c10::attr::Subgraph)->nodes())
    if (n->kind() == sym::LstmStack() || n->kind() == sym::ForallSelectRev()) return false;
  // F1's results may only feed F2 and size queries with a constant dimension
  for (Value* o : f1->outputs())
    for (const Use& u : o->uses()) {
      if (u.user == f2) continue;
      if (u.user->kind() == c10::aten::size && u.user->inputs().size() == 2 && constant_as<int64_t>(u.user->input(1))) continue;
      if (u.user->kind() == c10::prim::device) continue;   // answered by F1's own arguments, below
      return false;
    }
  // where F1's results live is where its tensor arguments live
  {
    Value* some_tensor = nullptr;
    for (Value* in : f1->inputs())
      if (!some_tensor && isTensorValue(in)) some_tensor = in;
    for (Value* o : f1->outputs()) {
      const auto uses = o->uses();
      for (const Use& u : uses) {
        if (u.user->kind() != c10::prim::device) continue;
        if (!some_tensor) return false;
        u.user->replaceInput(0, some_tensor);
      }
    }
  }
  // static types of F1's arguments, and what F1 returns for them
  std::vector<c10::IValue> samples1;
  {
    const auto types1 = f1->tys(sym::input_refine_types());
    if (types1.size() != f1->inputs().size()) return false;
    for (size_t k = 0; k < types1.size(); ++k) {
      c10::IValue v;
      if (!sampleOfArg(types1[k], f1->input(k), &v)) return false;
      samples1.push_back(v);
    }
  }
  std::vector<std::vector<int64_t>> shapes1;
  try {
    NoSourceDump quiet;
    int64_t kind1 = 0;
    RegionRunner r1(f1);
    r1.dryRun(samples1, &kind1, &shapes1);
  } catch (const c10::Error&) {
    return false;
  }
  if (shapes1.size() != f1->outputs().size()) return false;
  // size queries on F1's results become constants (the pipeline works on static shapes)
  bool changed = false;
  for (size_t o = 0; o < f1->outputs().size(); ++o) {
    const auto uses = f1->output(o)->uses();
    for (const Use& u : uses) {
      if (u.user == f2) continue;
      if (u.user->kind() != c10::aten::size) continue;
      int64_t d = *constant_as<int64_t>(u.user->input(1));
      const int64_t rank = (int64_t)shapes1[o].size();
      if (d < 0) d += rank;
      if (d < 0 || d >= rank) return changed;
      WithInsertPoint guard(u.user);
      u.user->output()->replaceAllUsesWith(g->insertConstant(shapes1[o][d]));
      u.user->destroy();
      changed = true;
    }
  }
  // the trip count: a constant, or a node of constants
  int64_t degree = f2->i(sym::parallel_degree());
  if (degree < 0) {
    Value* len = f2->input(0);
    auto c = constant_as<int64_t>(len);
    if (!c && len->node()->kind() != c10::prim::Param) {
      auto st = runNodeIfInputsAreConstant(len->node());
      if (st && st->size() == 1 && (*st)[0].isInt()) c = (*st)[0].toInt();
    }
    if (!c) return changed;
    degree = *c;
  }
  if (degree < 1) return changed;
  // the merged functor: F1's arguments (shared), then F2's other arguments
  Node* f = g->createWithSubgraph(sym::ParallelFunctor());
  auto sub = f->g(c10::attr::Subgraph);
  auto sub1 = f1->g(c10::attr::Subgraph);
  auto sub2 = f2->g(c10::attr::Subgraph);
  std::vector<int64_t> par;
  std::vector<c10::TypePtr> types;
  std::vector<c10::IValue> samples;
  std::unordered_map<Value*, Value*> map1, map2;
  Value* idx = sub->addInput()->setType(c10::IntType::get());
  map2[sub2->inputs()[0]] = idx;
  const auto types1 = f1->tys(sym::input_refine_types());
  for (size_t k = 0; k < f1->inputs().size(); ++k) {
    f->addInput(f1->input(k));
    types.push_back(types1[k]);
    par.push_back(0);
    samples.push_back(samples1[k]);
    map1[sub1->inputs()[k + 1]] = sub->addInput()->copyMetadata(sub1->inputs()[k + 1]);
  }
  {
    // F1's placeholder for the task index
    WithInsertPoint guard(sub->block());
    map1[sub1->inputs()[0]] = sub->insertConstant(c10::IValue());
  }
  auto destroyMerged = [&]() { f->destroy(); };
  const auto types2 = f2->tys(sym::input_refine_types());
  for (size_t k = first2; k < f2->inputs().size(); ++k) {
    Value* in = f2->input(k);
    Value* p = sub2->inputs()[k - first2 + 1];
    if (in->node() == f1) continue;   // bound below, once F1's nodes are in
    c10::IValue v;
    if (par2[k - first2] != 0 || !sampleOfArg(types2[k - first2], in, &v)) { destroyMerged(); return changed; }
    f->addInput(in);
    types.push_back(types2[k - first2]);
    par.push_back(0);
    samples.push_back(v);
    map2[p] = sub->addInput()->copyMetadata(p);
  }
  std::vector<Value*> no_returns;
  cloneBlockInto(sub1->block(), sub.get(), map1, &no_returns);
  for (size_t k = first2; k < f2->inputs().size(); ++k) {
    Value* in = f2->input(k);
    if (in->node() == f1) map2[sub2->inputs()[k - first2 + 1]] = map1.at(sub1->outputs()[in->offset()]);
  }
  cloneBlockInto(sub2->block(), sub.get(), map2);
  cseRegion(sub);
  EliminateDeadCode(sub);
  f->i_(sym::parallel_degree(), degree);
  f->i_(sym::is_parallel_map(), 1);
  f->i_(sym::compact_rows(), 1);
  f->is_(sym::is_parallel_args(), par);
  f->tys_(sym::input_refine_types(), types);
  for (Value* out : f2->outputs()) f->addOutput()->copyMetadata(out);
  // only when the library runs the merged region as one of its hand-written kernels: lowered
  // generically every task would redo the producer
  int64_t kind = 0, rs[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  try {
    NoSourceDump quiet;
    std::vector<std::vector<int64_t>> shapes;
    RegionRunner rm(f);
    rm.dryRun(samples, &kind, &shapes, rs);
  } catch (const c10::Error&) {
    kind = 0;
    rs[0] = 0;
  }
  // ... or as a row-stream kernel: then the merged region is a row compaction whose programs stay
  // inside the rows of one task (no reduction, most of every row of the widest input used), so a
  // task evaluates the producer for its own kept rows only and nothing is done twice
  if (kind == 0 && rs[0] == 0) { destroyMerged(); return changed; }
  f->insertBefore(f2);
  for (size_t k = 0; k < f2->outputs().size(); ++k) f2->output(k)->replaceAllUsesWith(f->output(k));
  f2->destroy();
  f1->destroy();
  return true;
}

bool sinkIn(Block* b) {
  bool changed = false;
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* n = *it;
    ++it;
    for (Block* inner : n->blocks()) changed |= sinkIn(inner);
    if (n->kind() != sym::ParallelFunctor() || n->i(sym::is_parallel_map()) == 0 || !n->hasAttribute(sym::compact_rows()) ||
        n->i(sym::compact_rows()) == 0)
      continue;
    if (trySink(n)) return true;   // the block changed under the walk: the caller starts over
  }
  return changed;
}

}  // namespace

void ToParallelFunctor(std::shared_ptr<Graph> graph) { toFunctorIn(graph->block()); }

bool SinkProducersIntoMaps(std::shared_ptr<Graph> graph) {
  if (!g_sink_producers.load()) return false;
  bool changed = false;
  for (int round = 0; round < 64 && sinkIn(graph->block()); ++round) {   // a chain of producers sinks one by one
    changed = true;
    EliminateDeadCode(graph);
  }
  return changed;
}
void setSinkProducers(bool on) { g_sink_producers.store(on); }

// ---------------------------------------------------------------------------
// static shapes of intermediate values
// ---------------------------------------------------------------------------
namespace {

bool completeTensorType(const c10::TypePtr& t) {
  auto tt = t->cast<c10::TensorType>();
  return tt && tt->scalarType() && tt->sizes().concrete_sizes();
}

c10::TypePtr typeOfSample(const at::Tensor& t, const c10::optional<c10::Device>& device) {
  return c10::TensorType::create(t.scalar_type(), device, c10::VaryingShape<int64_t>(t.sizes().vec()),
                                 c10::VaryingShape<int64_t>(t.strides().vec()), false);
}

// The node run on meta tensors of its arguments' static types: what it returns carries the
// shapes of its results.  Only nodes whose other arguments are constants, and only operators
// (nodes with blocks are walked, not run).
bool inferNode(Node* n) {
  // an element of a list argument with a refined type, at a constant index: the element's type
  if (n->kind() == c10::aten::__getitem__ && isTensorValue(n->output()) && !completeTensorType(n->output()->type())) {
    auto it = refinedTypes().find(n->input(0));
    auto idx = constant_as<int64_t>(n->input(1));
    if (it == refinedTypes().end() || !idx) return false;
    const auto& elems = it->second->expectRef<c10::TupleType>().elements();
    const int64_t i = *idx < 0 ? *idx + (int64_t)elems.size() : *idx;
    if (i < 0 || i >= (int64_t)elems.size() || !completeTensorType(elems[i])) return false;
    n->output()->setType(elems[i]);
    return true;
  }
  if (n->blocks().size() != 0 || n->kind() == c10::prim::Constant || n->kind() == c10::prim::ListConstruct ||
      n->kind() == c10::prim::TupleConstruct || n->kind().is_prim() && n->kind() != c10::prim::NumToTensor)
    return false;
  bool wanted = false;
  for (Value* o : n->outputs()) wanted = wanted || (isTensorValue(o) && !completeTensorType(o->type()));
  if (!wanted || !n->maybeOperator()) return false;
  const std::string ns = n->kind().ns().toUnqualString();
  if (ns != "aten" && ns != "immut") return false;
  Stack stack;
  c10::optional<c10::Device> device;
  for (Value* in : n->inputs()) {
    c10::IValue v;
    if (isTensorValue(in)) {
      if (auto c = toIValue(in)) {
        if (!c->isTensor() || !c->toTensor().defined()) return false;
        const at::Tensor t = c->toTensor();
        if (!device) device = t.device();
        stack.emplace_back(at::empty_strided(t.sizes(), t.strides(), t.options().device(c10::kMeta)));
        continue;
      }
      if (!sampleOf(in->type(), &v)) return false;
      if (!device) device = in->type()->expectRef<c10::TensorType>().device();
      stack.push_back(v);
    } else if (in->type()->kind() == c10::TypeKind::ListType && in->node()->kind() == c10::prim::ListConstruct &&
               in->type()->expectRef<c10::ListType>().getElementType()->kind() == c10::TypeKind::TensorType) {
      c10::List<at::Tensor> lst;
      for (Value* e : in->node()->inputs()) {
        if (!sampleOf(e->type(), &v)) return false;
        if (!device) device = e->type()->expectRef<c10::TensorType>().device();
        lst.push_back(v.toTensor());
      }
      stack.emplace_back(lst);
    } else if (auto c = toIValue(in)) {
      stack.push_back(*c);
    } else if (in->type()->kind() == c10::TypeKind::DeviceObjType) {
      stack.emplace_back(c10::Device(c10::kMeta));   // where a tensor is created does not change its shape
    } else {
      return false;
    }
  }
  try {
    n->getOperation()(stack);
  } catch (const std::exception&) {
    return false;   // shapes that depend on data, arguments the operator refuses on this device
  }
  if (stack.size() != n->outputs().size()) return false;
  bool changed = false;
  for (size_t k = 0; k < n->outputs().size(); ++k) {
    Value* o = n->output(k);
    if (!isTensorValue(o) || !stack[k].isTensor() || !stack[k].toTensor().defined() || completeTensorType(o->type())) continue;
    o->setType(typeOfSample(stack[k].toTensor(), device));
    changed = true;
  }
  return changed;
}

// A functor lowered for the static types of its arguments (nothing runs): types of its results,
// and its input_refine_types brought up to date.
bool inferFunctor(Node* n) {
  if (n->i(sym::parallel_degree()) < 0) return false;
  for (Node* k : n->g(c10::attr::Subgraph)->nodes())
    if (k->kind() == sym::LstmStack()) return false;
  const bool is_map = n->i(sym::is_parallel_map()) != 0;
  const auto par = n->is(sym::is_parallel_args());
  auto types = n->tys(sym::input_refine_types());
  if (types.size() != n->inputs().size() || par.size() != types.size()) return false;
  std::vector<c10::IValue> samples;
  c10::optional<c10::Device> device;
  bool refreshed = false;
  for (size_t k = 0; k < types.size(); ++k) {
    c10::IValue v;
    if (is_map && par[k] != 0) {
      auto et = types[k];
      if (auto lt = et->cast<c10::ListType>()) et = lt->getElementType();
      if (!sampleOf(et, &v)) return false;
      c10::List<at::Tensor> lst;
      for (int64_t t = 0; t < n->i(sym::parallel_degree()); ++t) lst.push_back(v.toTensor());
      samples.emplace_back(lst);
      continue;
    }
    // the value's own type, when the walk has given it one, is newer than the attribute
    if (isTensorValue(n->input(k)) && completeTensorType(n->input(k)->type()) && !completeTensorType(types[k])) {
      types[k] = n->input(k)->type();
      refreshed = true;
    }
    if (!sampleOfArg(types[k], n->input(k), &v)) return false;
    if (v.isTensor() && !device) device = types[k]->expectRef<c10::TensorType>().device();
    samples.push_back(v);
  }
  if (refreshed) n->tys_(sym::input_refine_types(), types);
  if (is_map) return refreshed;   // results are lists
  bool wanted = false;
  for (Value* o : n->outputs()) wanted = wanted || !completeTensorType(o->type());
  if (!wanted) return refreshed;
  std::vector<std::vector<int64_t>> shapes;
  std::vector<c10::ScalarType> dtypes;
  try {
    NoSourceDump quiet;
    int64_t kind = 0;
    RegionRunner r(n);
    r.dryRun(samples, &kind, &shapes, nullptr, nullptr, &dtypes);
  } catch (const c10::Error&) {
    return refreshed;
  }
  if (shapes.size() != n->outputs().size()) return refreshed;
  for (size_t k = 0; k < shapes.size(); ++k)
    n->output(k)->setType(c10::TensorType::createContiguous(dtypes[k], device ? *device : c10::Device(c10::kCPU), shapes[k]));
  return true;
}

bool inferIn(Block* b) {
  bool changed = false;
  for (Node* n : b->nodes()) {
    if (n->kind() == sym::ParallelFunctor()) changed |= inferFunctor(n);
    else changed |= inferNode(n);
    for (Block* inner : n->blocks()) changed |= inferIn(inner);
  }
  return changed;
}

}  // namespace

bool InferStaticShapes(std::shared_ptr<Graph> graph) { return inferIn(graph->block()); }

// ---------------------------------------------------------------------------
// every functor of a built graph planned for its static argument types
// ---------------------------------------------------------------------------
namespace {
void planIn(Block* b, std::vector<std::string>* report) {
  for (Node* n : b->nodes()) {
    for (Block* inner : n->blocks()) planIn(inner, report);
    if (n->kind() != sym::ParallelFunctor()) continue;
    std::ostringstream line;
    const auto sub = n->g(c10::attr::Subgraph);
    bool special = false;
    for (Node* k : sub->nodes())
      if (k->kind() == sym::LstmStack()) special = true;
    if (special) { report->push_back("lstm_stack functor: a kernel of its own, nothing to plan"); continue; }
    const auto types = n->tys(sym::input_refine_types());
    const auto par = n->is(sym::is_parallel_args());
    const int64_t degree = n->i(sym::parallel_degree());
    const bool is_map = n->i(sym::is_parallel_map()) != 0;
    if (degree < 0) { report->push_back("functor with a run-time trip count: planned when it runs"); continue; }
    std::vector<c10::IValue> samples;
    bool ok = types.size() == n->inputs().size() && par.size() == types.size();
    for (size_t k = 0; ok && k < types.size(); ++k) {
      c10::IValue v;
      if (is_map && par[k] != 0) {
        // the unified element type of a per-task list
        auto et = types[k];
        if (auto lt = et->cast<c10::ListType>()) et = lt->getElementType();
        if (!sampleOf(et, &v)) { ok = false; break; }
        c10::List<at::Tensor> lst;
        for (int64_t t = 0; t < degree; ++t) lst.push_back(v.toTensor());
        samples.emplace_back(lst);
      } else if (sampleOfArg(types[k], n->input(k), &v)) {
        samples.push_back(v);
      } else {
        ok = false;
      }
    }
    if (!ok) { report->push_back("functor with arguments without a static type: planned when it runs"); continue; }
    try {
      int64_t kind = 0, rs[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      std::vector<std::vector<int64_t>> shapes;
      std::string why;
      RegionRunner r(n);
      int64_t kernels[2] = {0, 0};
      r.dryRun(samples, &kind, &shapes, rs, &why, nullptr, kernels);
      line << "functor planned: " << shapes.size() << " output(s)";
      if (!(n->hasAttribute(sym::compact_rows()) && n->i(sym::compact_rows()) != 0))
        line << (kernels[1] ? ", compiled (lean dense kernel)" : kernels[0] ? ", compiled" : ", interpreted");
      if (n->hasAttribute(sym::compact_rows()) && n->i(sym::compact_rows()) != 0) {
        if (rs[0]) {
          char hx[32];
          snprintf(hx, sizeof hx, "%08llx%08llx", (unsigned long long)rs[3], (unsigned long long)rs[2]);
          line << ", row-stream key " << hx << (rs[1] ? " (kernel linked)" : " (no kernel linked)");
        } else {
          line << ", no row-stream form: " << why;
        }
        if (kind) line << ", hand-written kernel " << kind;
      }
    } catch (const c10::Error& e) {
      line << "functor not planned: " << e.what_without_backtrace();
    }
    report->push_back(line.str());
  }
}
}  // namespace

std::vector<std::string> PlanFunctors(std::shared_ptr<Graph> graph) {
  std::vector<std::string> report;
  planIn(graph->block(), &report);
  return report;
}

void setEarlyResultsHook(EarlyResultsHook* hook) { t_early_hook = hook; }

void functorHostTiming(bool on) {
  if (on) {
    for (auto& v : g_host_ns) v.store(0);
    g_host_calls.store(0);
  }
  g_host_timing.store(on);
}

std::vector<std::pair<std::string, double>> functorHostTimes() {
  std::vector<std::pair<std::string, double>> out;
  const uint64_t calls = g_host_calls.load();
  out.emplace_back("calls", (double)calls);
  for (int s = 0; s < HS_COUNT; ++s)
    out.emplace_back(kHostSectionNames[s], calls ? (double)g_host_ns[s].load() / 1e3 / (double)calls : 0.0);
  return out;
}

std::string fxhipLibraryPath() { return "functs_amd/lib/libfxhip.so"; }

}  // namespace functs
