// functs:: detection-tail operators (score threshold, sort, class-aware greedy NMS, top-k as ONE
// launch of the library's fx_sort_nms) and the pass that joins a compacting map functor with the
// tail behind it.
//
// The reference's detection programs call torchvision::nms from a chain of ATen operators with
// host synchronisations in between (functs/benchmark/ai_model/yolov3/yolov3_bbox.py:104-179,
// functs/benchmark/ai_model/ssd/ssd_bbox.py:163-214).  A program written for this backend calls
//   functs::nms(dets, scores, iou_threshold)                       torchvision::nms's schema
//   functs::batched_nms(boxes, scores, idxs, iou_threshold)        ssd_bbox.py:175-206
//   functs::multiclass_nms(boxes, scores, factors, ...)            yolov3_bbox.py:104-138
// where the reference's program calls the Python functions of those names.  Each is one launch
// followed by one wait for the number of kept boxes (their results have data-dependent shapes).
// FuseDetectionTail rewrites a per-image loop of functs::multiclass_nms over the lists of a
// compacting map functor into
//   functor[padded_outputs] -> functs::multiclass_nms_batched -> functs::unbatch_detections
// two launches on one stream (the second reads the kept-row counts from memory) and ONE wait at
// the end, for all images together.
#include <ATen/ATen.h>
#include <ATen/core/CachingHostAllocator.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/DeviceGuard.h>
#include <torch/csrc/jit/ir/constants.h>
#include <torch/csrc/jit/passes/dead_code_elimination.h>
#include <torch/csrc/jit/runtime/custom_operator.h>
#include <torch/library.h>

#include <atomic>
#include <chrono>
#include <map>
#include <mutex>
#include <tuple>

#include "../../../include/fxhip.h"
#include "passes.h"
#include "symbols.h"

namespace functs {
using namespace torch::jit;

namespace {
using at::Tensor;

#define FX_OK_OR_THROW(expr)                                             \
  do {                                                                   \
    int rc__ = (expr);                                                   \
    TORCH_CHECK(rc__ >= 0, "fxhip: ", fx_last_error(), " (", #expr, ")"); \
  } while (0)

// Counters and key buffers of the kernel, one per (device, stream) and layout (number of images,
// key capacity): cleared when allocated, every launch leaves the counters clear.
struct NmsWorkspaces {
  std::mutex mu;
  std::map<std::tuple<int, void*, int64_t, int64_t>, Tensor> by_stream;
  Tensor get(c10::Device dev, void* stream, int64_t n_tasks, int64_t key_capacity) {
    std::lock_guard<std::mutex> lock(mu);
    Tensor& t = by_stream[{(int)dev.index(), stream, n_tasks, key_capacity}];
    if (!t.defined()) {
      const size_t bytes = fx_sort_nms_workspace_bytes((int)n_tasks, (uint32_t)key_capacity);
      t = at::zeros({(int64_t)std::max<size_t>(bytes, 256)}, at::TensorOptions().dtype(at::kByte).device(dev));   // on the current stream
    }
    return t;
  }
};
NmsWorkspaces& nmsWorkspaces() {
  static NmsWorkspaces* w = new NmsWorkspaces();   // tensors must not outlive the HIP runtime's teardown order
  return *w;
}

// images may lie at any distance from each other (dimension 0), each one contiguous
Tensor imagesContiguous(const Tensor& t, const char* op, const char* name) {
  TORCH_CHECK(t.is_cuda(), op, " runs on the GPU only; ", name, " is a ", t.device(), " tensor");
  TORCH_CHECK(t.scalar_type() == at::kFloat, op, ": ", name, " must be float32");
  if (t.dim() >= 2 && t.size(0) > 0 && t.select(0, 0).is_contiguous() && t.stride(0) >= t.select(0, 0).numel()) return t;
  return t.contiguous();
}

struct Batched { Tensor dets, labels, index, n; };
constexpr int32_t kPending = INT32_MIN + 1;   // no count and not FX_NMS_OVERFLOW (-1)

// One launch for all images.  boxes [T, K, 4]; mode 1: scores [T, K, row], of which the first
// n_classes columns are class scores, factors [T, K] or undefined; mode 0: scores [T, K], labels
// [T, K] int64 or undefined.  counts: int32 [T] on the device or in pinned host memory, or undefined.
Batched launch(const char* op, int mode, const Tensor& boxes_, const Tensor& scores_, const Tensor& factors_, const Tensor& labels_,
               const Tensor& counts_, int64_t n_classes, double score_thr, double iou_thr, int64_t max_num) {
  const Tensor boxes = imagesContiguous(boxes_, op, "boxes"), scores = imagesContiguous(scores_, op, "scores");
  TORCH_CHECK(boxes.dim() == 3 && boxes.size(2) == 4, op, ": boxes must be [images, rows, 4], got ", boxes.sizes());
  const int64_t T = boxes.size(0), K = boxes.size(1);
  TORCH_CHECK(max_num >= 1 && max_num <= FX_NMS_MAX_OUT, op, ": max_num must be 1..", FX_NMS_MAX_OUT);
  c10::DeviceGuard guard(boxes.device());
  const auto dev = boxes.device();
  fx_nms_desc d;
  memset(&d, 0, sizeof d);
  d.mode = mode;
  d.n_tasks = (int32_t)T;
  d.rows = (uint32_t)K;
  d.boxes = boxes.data_ptr<float>();
  d.boxes_task_stride = boxes.stride(0);
  d.scores = scores.data_ptr<float>();
  d.scores_task_stride = scores.stride(0);
  Tensor factors, labels, counts;
  if (mode == 1) {
    TORCH_CHECK(scores.dim() == 3 && scores.size(0) == T && scores.size(1) == K && n_classes >= 1 && n_classes <= scores.size(2), op,
                ": scores must be [images, rows, >= classes], got ", scores.sizes(), " for ", n_classes, " classes");
    d.n_classes = (uint32_t)n_classes;
    d.scores_row_stride = (uint32_t)scores.size(2);
    if (factors_.defined()) {
      factors = imagesContiguous(factors_, op, "score_factors");
      TORCH_CHECK(factors.dim() == 2 && factors.size(0) == T && factors.size(1) == K, op, ": score_factors must be [images, rows]");
      d.factors = factors.data_ptr<float>();
      d.factors_task_stride = factors.stride(0);
    }
  } else {
    TORCH_CHECK(scores.dim() == 2 && scores.size(0) == T && scores.size(1) == K, op, ": scores must be [images, rows], got ", scores.sizes());
    d.n_classes = 1;
    if (labels_.defined()) {
      TORCH_CHECK(labels_.is_cuda() && labels_.scalar_type() == at::kLong && labels_.sizes() == scores.sizes(), op,
                  ": idxs must be int64 on the GPU, one per box");
      labels = labels_.contiguous();
      d.labels = labels.data_ptr<int64_t>();
      d.labels_task_stride = labels.stride(0);
    }
  }
  if (counts_.defined()) {
    TORCH_CHECK(counts_.scalar_type() == at::kInt && counts_.numel() == T && (counts_.is_cuda() || counts_.is_pinned()), op,
                ": counts must be ", T, " int32 values on the device or in pinned host memory");
    counts = counts_.contiguous();
    d.counts = (const uint32_t*)counts.data_ptr<int32_t>();
  }
  d.score_thr = (float)score_thr;
  d.iou_thr = (float)iou_thr;
  d.max_num = (uint32_t)max_num;
  d.key_capacity = FX_NMS_MAX_CANDIDATES;
  Batched r;
  const auto f32 = at::TensorOptions().dtype(at::kFloat).device(dev);
  r.dets = at::empty({T, max_num, 5}, f32);
  r.labels = at::empty({T, max_num}, f32.dtype(at::kLong));
  r.index = at::empty({T, max_num}, f32.dtype(at::kLong));
  // the kept counts land in pinned host memory, marked pending until the kernel stores them: the
  // one wait of the tail is a poll of these words, not a synchronisation of the stream
  r.n = at::empty({T}, at::TensorOptions().dtype(at::kInt).pinned_memory(true));
  for (int64_t t = 0; t < T; ++t) r.n.data_ptr<int32_t>()[t] = kPending;
  d.dets = r.dets.data_ptr<float>();
  d.out_labels = r.labels.data_ptr<int64_t>();
  d.out_index = r.index.data_ptr<int64_t>();
  d.n_out = (uint32_t*)r.n.data_ptr<int32_t>();
  if (T > 0) {
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(dev.index());
    Tensor ws = nmsWorkspaces().get(dev, (void*)stream.stream(), T, d.key_capacity);
    d.workspace = ws.data_ptr();
    d.workspace_bytes = (size_t)ws.numel();
    FX_OK_OR_THROW(fx_sort_nms(&d, (void*)stream.stream()));
    // pinned blocks must not be handed out again before the launch has read / written them
    if (counts.defined() && counts.is_pinned())
      at::getHostAllocator(at::kCUDA)->record_event(counts.data_ptr(), counts.storage().data_ptr().get_context(), stream.unwrap());
    at::getHostAllocator(at::kCUDA)->record_event(r.n.data_ptr(), r.n.storage().data_ptr().get_context(), stream.unwrap());
  } else {
    r.n.zero_();
  }
  return r;
}

// The one wait: the number of kept boxes per image comes to the host, the results are cut to size.
// An image with more candidates than the launch holds is an error, not a shorter result: the
// reference takes its per-class branch from 10000 candidates on (yolov3_bbox.py:148-166), here one
// pass serves up to FX_NMS_MAX_CANDIDATES and nothing serves more.
std::vector<int64_t> keptCounts(const char* op, const Tensor& n, c10::Device dev) {
  Tensor host = n;
  if (n.is_pinned() && n.is_contiguous()) {
    // Usually the counts are here when the kernel ends or shortly before.  The runtime is asked
    // rarely (a query takes its locks); when the stream has drained and a word is still pending,
    // the launch never ran to its end.
    const volatile int32_t* p = n.data_ptr<int32_t>();
    auto pending = [&]() {
      for (int64_t t = 0; t < n.numel(); ++t)
        if (p[t] == kPending) return true;
      return false;
    };
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(dev.index());
    using clock = std::chrono::steady_clock;
    clock::time_point next_query = clock::now() + std::chrono::microseconds(100);
    while (pending()) {
      __builtin_ia32_pause();
      if (clock::now() < next_query) continue;
      if (stream.query()) {
        // drained and still pending: the launch ran on another stream than the current one, or not at all
        stream.synchronize();
        if (pending()) {
          const hipError_t e = hipDeviceSynchronize();
          TORCH_CHECK(e == hipSuccess, op, ": hipDeviceSynchronize: ", hipGetErrorString(e));
        }
        TORCH_CHECK(!pending(), op, ": the kept counts of a launch were never written");
        break;
      }
      next_query = clock::now() + std::chrono::microseconds(100);
    }
    std::atomic_thread_fence(std::memory_order_acquire);
  } else {
    host = n.to(at::kCPU);
  }
  std::vector<int64_t> out((size_t)host.numel());
  const int32_t* p = host.data_ptr<int32_t>();
  bool overflow = false;
  for (size_t t = 0; t < out.size(); ++t) {
    overflow = overflow || p[t] < 0;
    out[t] = p[t];
  }
  if (overflow) {
    fx_async_error_take(FX_ASYNC_NMS_CAPACITY);   // this report is raised here
    TORCH_CHECK(false, op, ": an image has more than ", FX_NMS_MAX_CANDIDATES, " candidates above the score threshold; the "
                "per-class pass that the reference takes for that many is not built, raise the threshold");
  }
  return out;
}

// rows [0, k) of image t of a contiguous [T, M, ...] tensor, without a trip through the dispatcher
Tensor imageRows(const Tensor& all, int64_t t, int64_t k) {
  std::vector<int64_t> sizes{k}, strides{all.stride(1)};
  for (int64_t d = 2; d < all.dim(); ++d) {
    sizes.push_back(all.size(d));
    strides.push_back(all.stride(d));
  }
  auto impl = c10::make_intrusive<c10::TensorImpl>(c10::TensorImpl::VIEW, c10::Storage(all.storage()), all.key_set(), all.dtype());
  impl->set_storage_offset(all.storage_offset() + t * all.stride(0));
  impl->set_sizes_and_strides(sizes, strides);
  return Tensor(std::move(impl));
}

// torchvision::nms: indices of the kept boxes by descending score
Tensor nms(const Tensor& dets, const Tensor& scores, double iou_threshold) {
  TORCH_CHECK(dets.dim() == 2 && dets.size(1) == 4 && scores.dim() == 1 && scores.size(0) == dets.size(0),
              "functs::nms: boxes [N, 4] and scores [N] expected, got ", dets.sizes(), " and ", scores.sizes());
  const int64_t N = dets.size(0);
  if (N == 0) return at::empty({0}, dets.options().dtype(at::kLong));
  TORCH_CHECK(N <= FX_NMS_MAX_CANDIDATES, "functs::nms: at most ", FX_NMS_MAX_CANDIDATES, " boxes, got ", N);
  const int64_t max_num = std::min<int64_t>(N, FX_NMS_MAX_OUT);
  Batched r = launch("functs::nms", 0, dets.unsqueeze(0), scores.unsqueeze(0), Tensor(), Tensor(), Tensor(), 1,
                     -std::numeric_limits<double>::infinity(), iou_threshold, max_num);
  const int64_t k = keptCounts("functs::nms", r.n, dets.device())[0];
  TORCH_CHECK(k < FX_NMS_MAX_OUT || N <= FX_NMS_MAX_OUT, "functs::nms: more than ", FX_NMS_MAX_OUT,
              " boxes are kept, which is the most one launch returns");
  return r.index.select(0, 0).narrow(0, 0, k);
}

// ssd_bbox.py:175-206: (dets [K, 5], keep [K])
std::tuple<Tensor, Tensor> batchedNms(const Tensor& boxes, const Tensor& scores, const Tensor& idxs, double iou_threshold) {
  TORCH_CHECK(boxes.dim() == 2 && boxes.size(1) == 4 && scores.dim() == 1 && scores.size(0) == boxes.size(0) && idxs.sizes() == scores.sizes(),
              "functs::batched_nms: boxes [N, 4], scores [N] and idxs [N] expected");
  const int64_t N = boxes.size(0);
  if (N == 0) return {at::empty({0, 5}, boxes.options()), at::empty({0}, boxes.options().dtype(at::kLong))};
  TORCH_CHECK(N <= FX_NMS_MAX_CANDIDATES, "functs::batched_nms: at most ", FX_NMS_MAX_CANDIDATES, " boxes, got ", N);
  const int64_t max_num = std::min<int64_t>(N, FX_NMS_MAX_OUT);
  Batched r = launch("functs::batched_nms", 0, boxes.unsqueeze(0), scores.unsqueeze(0), Tensor(), idxs.unsqueeze(0), Tensor(), 1,
                     -std::numeric_limits<double>::infinity(), iou_threshold, max_num);
  const int64_t k = keptCounts("functs::batched_nms", r.n, boxes.device())[0];
  TORCH_CHECK(k < FX_NMS_MAX_OUT || N <= FX_NMS_MAX_OUT, "functs::batched_nms: more than ", FX_NMS_MAX_OUT,
              " boxes are kept, which is the most one launch returns");
  return {r.dets.select(0, 0).narrow(0, 0, k), r.index.select(0, 0).narrow(0, 0, k)};
}

int64_t classesOf(const Tensor& multi_scores, bool padded) {
  TORCH_CHECK(multi_scores.dim() >= 2, "multiclass_nms: scores without a class dimension");
  return multi_scores.size(-1) - (padded ? 1 : 0);   // yolov3_bbox.py:110: the last column is padding
}

// yolov3_bbox.py:104-138: (dets [<= max_num, 5], labels)
std::tuple<Tensor, Tensor> multiclassNms(const Tensor& multi_bboxes, const Tensor& multi_scores, const Tensor& score_factors,
                                         double score_thr, double iou_threshold, int64_t max_num, bool padded) {
  TORCH_CHECK(multi_bboxes.dim() == 2 && multi_scores.dim() == 2 && score_factors.dim() == 1,
              "functs::multiclass_nms: boxes [K, 4], scores [K, C] and score factors [K] expected");
  Batched r = launch("functs::multiclass_nms", 1, multi_bboxes.unsqueeze(0), multi_scores.unsqueeze(0), score_factors.unsqueeze(0), Tensor(),
                     Tensor(), classesOf(multi_scores, padded), score_thr, iou_threshold, max_num);
  const int64_t k = keptCounts("functs::multiclass_nms", r.n, multi_bboxes.device())[0];
  return {r.dets.select(0, 0).narrow(0, 0, k), r.labels.select(0, 0).narrow(0, 0, k)};
}

// every image at once, nothing waits: (dets [T, max_num, 5], labels [T, max_num], n [T] int32)
std::tuple<Tensor, Tensor, Tensor> multiclassNmsBatched(const Tensor& multi_bboxes, const Tensor& multi_scores, const Tensor& score_factors,
                                                        const std::optional<Tensor>& counts, double score_thr, double iou_threshold,
                                                        int64_t max_num, bool padded) {
  Batched r = launch("functs::multiclass_nms_batched", 1, multi_bboxes, multi_scores, score_factors, Tensor(),
                     counts ? *counts : Tensor(), classesOf(multi_scores, padded), score_thr, iou_threshold, max_num);
  return {r.dets, r.labels, r.n};
}

// the wait behind multiclass_nms_batched: per image the first n[t] rows
std::tuple<std::vector<Tensor>, std::vector<Tensor>> unbatchDetections(const Tensor& dets, const Tensor& labels, const Tensor& n) {
  TORCH_CHECK(dets.dim() == 3 && labels.dim() == 2 && n.dim() == 1 && dets.size(0) == n.size(0) && labels.size(0) == n.size(0),
              "functs::unbatch_detections: dets [T, M, 5], labels [T, M] and n [T] expected");
  TORCH_CHECK(dets.is_cuda() && labels.is_cuda(), "functs::unbatch_detections runs on the GPU only");
  const std::vector<int64_t> k = keptCounts("functs::unbatch_detections", n, dets.device());
  std::vector<Tensor> d, l;
  for (size_t t = 0; t < k.size(); ++t) {
    d.push_back(imageRows(dets, (int64_t)t, k[t]));
    l.push_back(imageRows(labels, (int64_t)t, k[t]));
  }
  return {d, l};
}

// the same as one list of (dets, labels) per image, the shape of the reference's result
// (yolov3_bbox.py:232-243)
// (the schema language has no list of tuples: the operator is registered with a schema object)
c10::TypePtr pairListType() {
  return c10::ListType::create(c10::TupleType::create({c10::TensorType::get(), c10::TensorType::get()}));
}
void unbatchDetectionPairs(Stack& stack) {
  const Tensor n = pop(stack).toTensor(), labels = pop(stack).toTensor(), dets = pop(stack).toTensor();
  auto lists = unbatchDetections(dets, labels, n);
  c10::impl::GenericList out(pairListType()->expectRef<c10::ListType>().getElementType());
  for (size_t t = 0; t < std::get<0>(lists).size(); ++t)
    out.push_back(c10::ivalue::Tuple::create(std::get<0>(lists)[t], std::get<1>(lists)[t]));
  push(stack, std::move(out));
}
RegisterOperators registerPairs({Operator(
    "functs::unbatch_detection_pairs", "",
    {c10::Argument("dets", c10::TensorType::get()), c10::Argument("labels", c10::TensorType::get()), c10::Argument("n", c10::TensorType::get())},
    {c10::Argument("", pairListType())}, Operation(unbatchDetectionPairs), c10::AliasAnalysisKind::PURE_FUNCTION)});

// ---------------------------------------------------------------------------
// pass: compacting map functor + per-image loop of functs::multiclass_nms
// ---------------------------------------------------------------------------
const Symbol& symMulticlassNms() {
  static const Symbol s = Symbol::fromQualString("functs::multiclass_nms");
  return s;
}

bool constantTrue(Value* v) {
  auto c = toIValue(v);
  return c && c->isBool() && c->toBool();
}

bool tryFuseTail(Node* loop) {
  if (loop->inputs().size() != 2 || !loop->outputs().empty()) return false;
  Block* body = loop->blocks()[0];
  if (!constantTrue(loop->input(1)) || !constantTrue(body->outputs()[0])) return false;
  Value* i = body->inputs()[0];
  Node* tail = nullptr;
  for (Node* n : body->nodes()) {
    if (n->kind() != symMulticlassNms()) continue;
    if (tail) return false;
    tail = n;
  }
  if (!tail) return false;
  // boxes, scores and score factors are list[i] of three results of ONE compacting map functor
  Node* functor = nullptr;
  Node* reads[3];
  size_t which[3];
  for (int k = 0; k < 3; ++k) {
    Node* r = tail->input(k)->node();
    if (r->kind() != c10::aten::__getitem__ || r->owningBlock() != body || r->input(1) != i || r->output()->uses().size() != 1) return false;
    Value* list = r->input(0);
    Node* f = list->node();
    if (f->kind() != sym::ParallelFunctor() || (functor && f != functor) || list->uses().size() != 1) return false;
    functor = f;
    reads[k] = r;
    which[k] = list->offset();
  }
  if (which[0] == which[1] || which[0] == which[2] || which[1] == which[2]) return false;
  if (functor->owningBlock() != loop->owningBlock() || !functor->isBefore(loop)) return false;
  if (functor->i(sym::is_parallel_map()) == 0 || !functor->hasAttribute(sym::compact_rows()) || functor->i(sym::compact_rows()) == 0 ||
      functor->hasAttribute(sym::padded_outputs()))
    return false;
  for (Value* o : functor->outputs())
    if (o->offset() != which[0] && o->offset() != which[1] && o->offset() != which[2] && o->hasUses()) return false;
  // one iteration per task
  const int64_t degree = functor->i(sym::parallel_degree());
  if (degree >= 0) {
    auto trip = toIValue(loop->input(0));
    if (!trip || !trip->isInt() || trip->toInt() != degree || degree < 1) return false;
  } else if (loop->input(0) != functor->input(0)) {
    return false;
  }
  // thresholds and limits are constants
  std::vector<c10::IValue> consts;
  for (size_t k = 3; k < tail->inputs().size(); ++k) {
    auto c = toIValue(tail->input(k));
    if (!c) return false;
    consts.push_back(*c);
  }

  Graph* g = loop->owningGraph();
  Node *batched = nullptr, *lists = nullptr;
  {
  WithInsertPoint guard(loop);
  Node* padded = g->create(sym::ParallelFunctor(), functor->inputs(), functor->outputs().size() + 1);
  padded->copyAttributes(*functor);
  padded->i_(sym::padded_outputs(), 1);
  padded->setSourceRange(functor->sourceRange());
  for (Value* o : padded->outputs()) o->setType(c10::TensorType::get());
  g->insertNode(padded);
  std::vector<Value*> args{padded->output(which[0]), padded->output(which[1]), padded->output(which[2]),
                           padded->output(functor->outputs().size())};
  for (const c10::IValue& c : consts) args.push_back(g->insertConstant(c));
  batched = g->create(Symbol::fromQualString("functs::multiclass_nms_batched"), args, 3);
  batched->setSourceRange(tail->sourceRange());
  for (Value* o : batched->outputs()) o->setType(c10::TensorType::get());
  g->insertNode(batched);
  lists = g->create(Symbol::fromQualString("functs::unbatch_detections"), batched->outputs(), 2);
  lists->setSourceRange(tail->sourceRange());
  for (Value* o : lists->outputs()) o->setType(c10::ListType::ofTensors());
  g->insertNode(lists);
  {
    WithInsertPoint in_body(tail);
    for (int k = 0; k < 2; ++k) {
      Node* r = g->create(c10::aten::__getitem__, {lists->output(k), i}, 1);
      r->output()->setType(c10::TensorType::get());
      g->insertNode(r);
      tail->output(k)->replaceAllUsesWith(r->output());
    }
  }
  }
  tail->destroy();
  for (Node* r : reads) r->destroy();
  functor->destroy();
  // What is left of the loop is often only results.append((dets_l[i], labels_l[i])): the list of
  // pairs then comes from one operator and the loop goes.
  Node *tuple = nullptr, *append = nullptr;
  bool only_pairs = true;
  for (Node* n : body->nodes()) {
    if (n->kind() == c10::prim::Constant) continue;
    if (n->kind() == c10::aten::__getitem__ && n->input(1) == i && (n->input(0) == lists->output(0) || n->input(0) == lists->output(1))) continue;
    if (n->kind() == c10::prim::TupleConstruct && !tuple) { tuple = n; continue; }
    if (n->kind() == c10::aten::append && !append) { append = n; continue; }
    only_pairs = false;
  }
  auto itemOf = [&](Value* v, size_t k) {
    return v->node()->kind() == c10::aten::__getitem__ && v->node()->owningBlock() == body && v->node()->input(0) == lists->output(k);
  };
  if (only_pairs && tuple && append && tuple->inputs().size() == 2 && itemOf(tuple->input(0), 0) && itemOf(tuple->input(1), 1) &&
      append->input(1) == tuple->output() && tuple->output()->uses().size() == 1 && !append->output()->hasUses()) {
    Value* list = append->input(0);
    Node* def = list->node();
    bool fresh = def->kind() == c10::prim::ListConstruct && def->inputs().empty() && def->owningBlock() == loop->owningBlock();
    for (const Use& u : list->uses()) fresh = fresh && (u.user == append || u.user->isAfter(loop));
    if (fresh) {
      Node* pairs = g->create(Symbol::fromQualString("functs::unbatch_detection_pairs"), batched->outputs(), 1);
      pairs->setSourceRange(lists->sourceRange());
      pairs->output()->setType(list->type());
      pairs->insertBefore(loop);
      list->replaceAllUsesAfterNodeWith(loop, pairs->output());
      loop->destroy();
      if (!lists->hasUses()) lists->destroy();
      if (!def->hasUses()) def->destroy();
    }
  }
  return true;
}

bool fuseTailsIn(Block* b) {
  bool changed = false;
  for (auto it = b->nodes().begin(); it != b->nodes().end();) {
    Node* n = *it;
    ++it;
    for (Block* inner : n->blocks()) changed = fuseTailsIn(inner) || changed;
    if (n->kind() == c10::prim::Loop) changed = tryFuseTail(n) || changed;
  }
  return changed;
}

}  // namespace

bool FuseDetectionTail(std::shared_ptr<Graph> graph) { return fuseTailsIn(graph->block()); }

bool PadCompactedResults(std::shared_ptr<Graph> graph) {
  if (graph->outputs().size() != 1) return false;
  Node* ret = graph->outputs()[0]->node();
  if (ret->kind() != c10::prim::TupleConstruct || ret->owningBlock() != graph->block() || ret->output()->uses().size() != 1) return false;
  bool changed = false;
  for (auto it = graph->nodes().begin(); it != graph->nodes().end();) {
    Node* f = *it;
    ++it;
    if (f->kind() != sym::ParallelFunctor() || !f->hasAttribute(sym::compact_rows()) || f->i(sym::compact_rows()) == 0 ||
        f->hasAttribute(sym::padded_outputs()))
      continue;
    if (f->i(sym::is_parallel_map()) != 0 && f->i(sym::parallel_degree()) < 1) continue;   // (an empty map has no padded form)
    bool only_returned = true;
    for (Value* o : f->outputs())
      for (const Use& u : o->uses()) only_returned = only_returned && u.user == ret;
    if (!only_returned) continue;
    Node* padded = graph->create(sym::ParallelFunctor(), f->inputs(), f->outputs().size() + 1);
    padded->copyAttributes(*f);
    padded->i_(sym::padded_outputs(), 1);
    padded->setSourceRange(f->sourceRange());
    for (Value* o : padded->outputs()) o->setType(c10::TensorType::get());
    padded->insertBefore(f);
    for (size_t k = 0; k < f->outputs().size(); ++k) f->output(k)->replaceAllUsesWith(padded->output(k));
    ret->addInput(padded->output(f->outputs().size()));
    f->destroy();
    changed = true;
  }
  if (changed) {
    std::vector<c10::TypePtr> types;
    for (Value* v : ret->inputs()) types.push_back(v->type());
    ret->output()->setType(c10::TupleType::create(std::move(types)));
  }
  return changed;
}

TORCH_LIBRARY(functs, m) {
  m.def("nms(Tensor dets, Tensor scores, float iou_threshold) -> Tensor", nms);
  m.def("batched_nms(Tensor boxes, Tensor scores, Tensor idxs, float iou_threshold=0.45) -> (Tensor, Tensor)", batchedNms);
  m.def("multiclass_nms(Tensor multi_bboxes, Tensor multi_scores, Tensor score_factors, float score_thr=0.05, "
        "float iou_threshold=0.45, int max_num=100, bool padded=True) -> (Tensor, Tensor)", multiclassNms);
  m.def("multiclass_nms_batched(Tensor multi_bboxes, Tensor multi_scores, Tensor score_factors, Tensor? counts=None, "
        "float score_thr=0.05, float iou_threshold=0.45, int max_num=100, bool padded=True) -> (Tensor, Tensor, Tensor)",
        multiclassNmsBatched);
  m.def("unbatch_detections(Tensor dets, Tensor labels, Tensor n) -> (Tensor[], Tensor[])", unbatchDetections);

}

}  // namespace functs
