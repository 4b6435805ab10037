// Region formation on functionalized graphs and the tssa::ParallelFunctor
// operator.  Interfaces of fait/passes/fuse_ops.h, parallelize_loops.h, te_op.h,
// validate_graph.h and functs/csrc/jit/passes/fait/fait_pipeline.h.
#pragma once
#include <torch/csrc/jit/ir/ir.h>

#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

namespace functs {

// fait/passes/fuse_ops.cpp:506-527: group fusable operators of every block
// into prim::FusionGroup nodes (block-bodied).
void FuseOps(std::shared_ptr<torch::jit::Graph> graph);

// A prim::Loop whose single carried tensor T is read only through
// immut::select(T, d, i) and written back through immut::select_rev(T, ., d, i)
// touches a different slab in every iteration: the loop becomes one
// fx::forall_select_rev node that a FusionGroup can absorb.  The reference never
// parallelises loops with carried values (parallelize_loops.cpp:17).
void CollapseAssignLoops(std::shared_ptr<torch::jit::Graph> graph);

// The (time, layer) loop nest of a stacked LSTM (functs/benchmark/ai_model/lstm/lstm.py:79-133),
// whose loops carry the states, becomes one fx::lstm_stack node when the static shapes fit the
// persistent kernel; true if the graph changed.
bool CollapseRecurrentLoops(std::shared_ptr<torch::jit::Graph> graph);

// fait/passes/canonicalize.cpp:148-157 (on a functionalized graph): one spelling per meaning
// (arange(end), max.other, new_zeros, pow with a constant exponent, empty slices, t(), to.dtype /
// to.other, view).
void CanonicalizeOps(std::shared_ptr<torch::jit::Graph> graph);
// Queries that the static types answer become constants: size(x, d), size(x), numel, dim, dtype of
// a value whose type (an argument's example, or an element of a list argument with a refined
// type) says so; device only when the type names a GPU.  With them the index arithmetic that a
// model runs on its shapes (anchor and prior generators: arange, repeat, stack over feature-map
// sizes) is folded by constant propagation when the function is built.  The reference gets there
// through InferShape + constant folding (fait_pipeline.cpp:47-49).  True if the graph changed.
bool FoldStaticTypeQueries(std::shared_ptr<torch::jit::Graph> graph);
// Tensor constants of 16 or more elements that all hold one value become zeros / full nodes again
// (run behind every constant propagation of the pipeline, which folds fills over static shapes).
bool UniformConstantsToFills(std::shared_ptr<torch::jit::Graph> graph);
// fait/passes/licm.cpp:55-66: scalar-valued pure nodes of loop and map bodies whose operands are
// defined outside move in front of the loop; true if the graph changed.
bool HoistLoopInvariants(std::shared_ptr<torch::jit::Graph> graph);

// fait/passes/parallelize_loops.cpp:12-145: loops without carried values whose
// list reads are list[i] and whose list writes are one append per list become
// prim::ParallelMap(len, lists...){block(i, elems...) -> rets}.
void ParallelizeLoops(std::shared_ptr<torch::jit::Graph> graph);
// fait/passes/parallelize_loops.cpp:152-293: every fusion group of a map body gets a map of its own
void SplitParallelMaps(std::shared_ptr<torch::jit::Graph> graph);
// fait/passes/parallelize_loops.cpp:458-502: the group of a fusable map takes the map index, the
// map's parameters in their order, then the values from outside; results in the group's order
void CanonicalizeFusableMaps(std::shared_ptr<torch::jit::Graph> graph);
// fait/passes/unroll_loops.cpp:11-77, parallelize_loops.cpp:372-456; true if the graph changed
bool UnrollLoopsWithDeps(std::shared_ptr<torch::jit::Graph> graph);
bool UnrollSimpleMaps(std::shared_ptr<torch::jit::Graph> graph);

// Fold `x[mask]` consumers of a FusionGroup into the group when the bool mask is
// produced by the same group (row compaction fused into the region).  The
// reference leaves these to ATen (convert_to_tensorssa.cpp:422-443,
// fuse_ops.cpp:173-200).
void FuseMaskedSelect(std::shared_ptr<torch::jit::Graph> graph);

// fait/passes/te_op.cpp:135-236: FusionGroup / ParallelMap{FusionGroup} ->
// tssa::ParallelFunctor (Subgraph + parallel_degree, is_parallel_map,
// is_parallel_args, input_refine_types).
void ToParallelFunctor(std::shared_ptr<torch::jit::Graph> graph);

// A plain functor whose results only feed a compacting map functor (as shared arguments) and size
// queries sinks into the map, when the library then runs the merged region as one hand-written
// kernel (SSD-style heads: decode + softmax, then one score filter per class); size queries on the
// producer's results become constants of the static shapes.  The reference keeps the two functors
// (fait/passes/te_op.cpp:135-236).  True if the graph changed; setSinkProducers(false) switches
// the pass off for the process.
bool SinkProducersIntoMaps(std::shared_ptr<torch::jit::Graph> graph);
void setSinkProducers(bool on);

// A per-image loop of functs::multiclass_nms(list_b[i], list_s[i], list_f[i], constants...) over
// three result lists of one compacting map functor becomes
//   functor[padded_outputs=1] -> functs::multiclass_nms_batched -> functs::unbatch_detections
// (detection_ops.cpp): the functor returns its outputs at full size and the kept-row counts as a
// tensor without waiting for them, the tail of all images is one launch behind it on the stream,
// and the only wait is the one that cuts the final results to size.  The reference runs the tail
// per image, as ATen and torchvision kernels with host synchronisations in between
// (yolov3_bbox.py:104-179, 233-243).  True if the graph changed.
bool FuseDetectionTail(std::shared_ptr<torch::jit::Graph> graph);

// Opt-in (functs_amd.jit.build(..., padded_outputs=True)): every compacting functor whose results
// are only returned gets padded_outputs=1, i.e. it returns each result at its full size (a map:
// one tensor [tasks, rows, ...]) and does NOT wait for the kept-row counts, which it returns as
// one more tensor (int32 in pinned host memory, written by the kernels) at the end of the
// function's result tuple, one per such functor.  Rows from counts[task] on hold no values.  For
// callers that feed the results to further work on the same stream and never need the sizes on
// the host.  True if the graph changed.
bool PadCompactedResults(std::shared_ptr<torch::jit::Graph> graph);

// Static types of intermediate values (the reference's InferShape, fait/passes/refine_types.cpp:
// 420-685, run at fait_pipeline.cpp:47): every operator node whose tensor arguments have complete
// static types and whose other arguments are constants is run on meta tensors of those types, and
// its results take the types of what comes back; a tssa::ParallelFunctor is lowered for its
// argument types instead (nothing runs) and its input_refine_types are brought up to date.  Shapes
// that depend on data stay unknown.  True if a type was set.
bool InferStaticShapes(std::shared_ptr<torch::jit::Graph> graph);

// Plans the region of every tssa::ParallelFunctor of a built graph for the static types in its
// input_refine_types (meta tensors stand for them; nothing runs, no device is needed), as the
// reference compiles every functor when its operator is created (fait/fuser/graph_builder.cpp:
// 259-712).  With a dump directory set in the library (fx_spec_dump_dir) the regions without
// compiled kernels leave their sources there.  Returns one line per functor: what was planned and
// which kernels serve it.
std::vector<std::string> PlanFunctors(std::shared_ptr<torch::jit::Graph> graph);

// Host time of tssa::ParallelFunctor by section (flatten, plan, alloc, launch, views, wait_counts,
// resize, push): switching on clears the sums; the read gives "calls" and the mean microseconds per
// operator call of every section.
// A caller of tssa::ParallelFunctor that holds the Python interpreter's lock through the call
// (functs_amd._C.DirectFunctor) installs one of these for its thread: the operator hands over the
// tensors of a map's list results as soon as they exist - views of the output block, made while
// the kernels run, their first dimension still at full size and cut in place once the kept-row
// counts are known - so that the wrapper objects of a call's results are made in the kernels'
// shadow and not behind the wait; and it tells before it blocks for longer than a short poll.
struct EarlyResultsHook {
  virtual ~EarlyResultsHook() = default;
  virtual void tensorsReady(size_t n_lists, int64_t degree, const at::Tensor* flat /* [list][task] */) = 0;
  virtual void beforeBlocking() = 0;
  virtual void afterBlocking() = 0;
};
void setEarlyResultsHook(EarlyResultsHook* hook);   // of the calling thread; nullptr removes it
void functorHostTiming(bool on);
std::vector<std::pair<std::string, double>> functorHostTimes();

// fait/passes/validate_graph.cpp:6-38: every use is dominated by its definition.
void Validate(std::shared_ptr<torch::jit::Graph> graph);

// functs/csrc/jit/passes/fait/fait_pipeline.cpp:31-68 (the passes of it that the
// fused-region path needs), on an already functionalized graph.
// Returns true when the graph now holds constants taken from the example's shapes (size, len,
// dtype or device queries folded): the built function then serves arguments of those shapes only,
// and the caller keys its built functions by shape (functs_amd/jit.py).
bool FaitPipeline(std::shared_ptr<torch::jit::Graph> graph, std::vector<c10::TypePtr> input_types);

// Refined list types (fait/passes/refine_types.cpp:57-81, 175-195): a list argument whose example
// is a tuple of tensors keeps that tuple type beside its List[Tensor] type while the pipeline runs.
// A map functor then records the unified element type for the argument
// (fait/passes/te_op.cpp:43-59), and len() of such a list is the constant of the example.
using ValueTypeMap = std::unordered_map<const torch::jit::Value*, c10::TypePtr>;
ValueTypeMap& refinedTypes();   // of the pipeline run in progress on this thread

std::string fxhipLibraryPath();

// shared by the passes
bool isFusableNode(torch::jit::Node* node);

// fait/passes/profile_ops.cpp:16-30: `print(label, True / False)` with constant arguments becomes
// prof::Begin(label) / prof::End(label); fait/util/profile.cpp:133-245: the timers behind them.
void ConvertProfilingInstrumentation(std::shared_ptr<torch::jit::Graph> graph);
void profBegin(const std::string& label);
void profEnd(const std::string& label);
std::string profilingResults(size_t count);   // what printProfilingResults writes
void resetProfiling();

}  // namespace functs
