// Python module functs_amd._C: same entry-point names as the reference's
// functs._C (functs/csrc/jit/python/init.cpp:31-76, script_init.cpp:83-95).
#include <torch/csrc/jit/passes/constant_propagation.h>
#include <torch/csrc/jit/passes/freeze_module.h>
#include <torch/csrc/jit/passes/shape_analysis.h>
#include <torch/csrc/jit/python/pybind_utils.h>
#include <torch/extension.h>

#include <torch/csrc/autograd/python_variable.h>

#include "passes.h"
#include "tensorssa.h"

namespace py = pybind11;
using namespace functs;
using torch::jit::Graph;

namespace {
// A built graph that is nothing but ONE tssa::ParallelFunctor over the function's arguments (what
// the pipeline makes of a program that fuses completely) is called without the TorchScript
// interpreter: the arguments go to the operator's stack, its results come back.  Same operator,
// same results; what is saved is the executor's per-call work around a single node.
// A List[Tensor] result that stays the operator's list: elements become Python objects when they
// are asked for.  A map over many tasks returns hundreds of tensors, and a caller that looks at a
// few of them (or hands the list on) does not pay for a wrapper per element on every call.
struct TensorList {
  c10::List<at::Tensor> list;
  py::list tolist() const {
    py::list out(list.size());
    for (size_t k = 0; k < list.size(); ++k) out[k] = py::reinterpret_steal<py::object>(THPVariable_Wrap(list.get(k)));
    return out;
  }
};

// The hook of a direct call (passes.h): the caller keeps the interpreter's lock through the
// operator, so the Python lists of a map's results can be made while the kernels run; the lock is
// given up only around a wait that outlasts the operator's short poll.
struct DirectCallHook final : functs::EarlyResultsHook {
  std::vector<py::object> lists;   // per operator output: its Python list, made early
  PyThreadState* saved = nullptr;
  void tensorsReady(size_t n_lists, int64_t degree, const at::Tensor* flat) override {
    lists.clear();
    lists.reserve(n_lists);
    for (size_t o = 0; o < n_lists; ++o) {
      py::list l((size_t)degree);
      for (int64_t t = 0; t < degree; ++t) {
        PyObject* item = THPVariable_Wrap(flat[o * (size_t)degree + (size_t)t]);
        if (!item) throw py::error_already_set();
        PyList_SET_ITEM(l.ptr(), (Py_ssize_t)t, item);
      }
      lists.push_back(std::move(l));
    }
  }
  void beforeBlocking() override { saved = PyEval_SaveThread(); }
  void afterBlocking() override {
    if (saved) PyEval_RestoreThread(saved);
    saved = nullptr;
  }
};

struct DirectFunctor {
  bool lazy_lists = false;                      // List[Tensor] results come back as TensorList
  std::shared_ptr<Graph> graph;                 // owns the node
  mutable std::optional<torch::jit::Operation> op;   // (Operation's call operator is not const)
  std::vector<int> source;                      // per operator input: graph input number, or -1 - k for constants[k]
  std::vector<c10::IValue> constants;
  std::vector<c10::TypePtr> arg_types;          // of the graph inputs
  std::vector<int> results;                     // per returned value: operator output number
  size_t n_op_outputs = 0;
  bool tuple_result = false;

  static std::shared_ptr<DirectFunctor> match(const std::shared_ptr<Graph>& graph) {
    using namespace torch::jit;
    Node* functor = nullptr;
    Node* tuple = nullptr;
    for (Node* n : graph->nodes()) {
      if (n->kind() == c10::prim::Constant) continue;
      if (n->kind() == c10::Symbol::fromQualString("tssa::ParallelFunctor") && !functor) { functor = n; continue; }
      if (n->kind() == c10::prim::TupleConstruct && functor && !tuple) { tuple = n; continue; }
      return nullptr;
    }
    if (!functor || graph->outputs().size() != 1) return nullptr;
    auto d = std::make_shared<DirectFunctor>();
    d->graph = graph;
    for (Value* in : functor->inputs()) {
      if (auto c = toIValue(in)) {
        d->source.push_back(-1 - (int)d->constants.size());
        d->constants.push_back(*c);
        continue;
      }
      size_t k = 0;
      while (k < graph->inputs().size() && graph->inputs()[k] != in) ++k;
      if (k == graph->inputs().size()) return nullptr;
      d->source.push_back((int)k);
    }
    for (Value* in : graph->inputs()) d->arg_types.push_back(in->type());
    Value* ret = graph->outputs()[0];
    std::vector<Value*> returned;
    if (tuple) {
      if (ret != tuple->output() || tuple->output()->uses().size() != 1) return nullptr;
      for (Value* v : tuple->inputs()) returned.push_back(v);
      d->tuple_result = true;
    } else {
      returned.push_back(ret);
    }
    for (Value* v : returned) {
      if (v->node() != functor) return nullptr;
      for (int seen : d->results)
        if (seen == (int)v->offset()) return nullptr;   // (results are moved out of the stack one by one)
      d->results.push_back((int)v->offset());
    }
    d->n_op_outputs = functor->outputs().size();
    d->op = functor->getOperation();
    return d;
  }

  py::object call(const py::args& args) const {
    TORCH_CHECK(args.size() == arg_types.size(), "expected ", arg_types.size(), " arguments, got ", args.size());
    torch::jit::Stack stack;
    stack.reserve(source.size() + n_op_outputs);
    for (int s : source) {
      if (s < 0) stack.push_back(constants[(size_t)(-1 - s)]);
      else stack.push_back(torch::jit::toIValue(args[(size_t)s], arg_types[(size_t)s]));
    }
    DirectCallHook hook;
    if (lazy_lists) {
      py::gil_scoped_release release;
      (*op)(stack);
    } else {
      struct Installed {
        explicit Installed(functs::EarlyResultsHook* h) { functs::setEarlyResultsHook(h); }
        ~Installed() { functs::setEarlyResultsHook(nullptr); }
      } installed(&hook);
      (*op)(stack);
    }
    TORCH_CHECK(stack.size() == n_op_outputs, "the operator left ", stack.size(), " values for ", n_op_outputs, " results");
    auto convert = [this, &hook](c10::IValue&& v, size_t output) -> py::object {
      if (lazy_lists && v.isTensorList()) return py::cast(TensorList{std::move(v).toTensorList()});
      // (the list made while the kernels ran holds the very tensors of the operator's list)
      if (output < hook.lists.size() && v.isTensorList()) return std::move(hook.lists[output]);
      return torch::jit::toPyObject(std::move(v));
    };
    if (!tuple_result) return convert(std::move(stack[(size_t)results[0]]), (size_t)results[0]);
    py::tuple out(results.size());
    for (size_t k = 0; k < results.size(); ++k) out[k] = convert(std::move(stack[(size_t)results[k]]), (size_t)results[k]);
    return std::move(out);
  }
};
}  // namespace

PYBIND11_MODULE(_C, m) {
  m.doc() = "MI355X backend of FuncTs/FAIT fused functionalized regions";
  py::class_<TensorSSAMutateInfo, std::shared_ptr<TensorSSAMutateInfo>>(m, "TensorSSAMutateInfo")
      .def(py::init<>())
      .def_property_readonly("mutNodes", [](TensorSSAMutateInfo& self) { return self.mutNodes; })
      .def_property_readonly("mutValues", [](TensorSSAMutateInfo& self) { return self.mutValues; });
  m.def("_jit_pass_remove_inplace", RemoveInplace);
  m.def("_jit_pass_dumb_remove_inter_precedure_mutation", DumbRemoveInterPrecedureMutation);
  m.def("_jit_pass_rewrite_mutation", TensorSSARewriteMutation);
  m.def("_jit_pass_block_propagation", TensorSSAPropagation);
  m.def("_jit_pass_rename", TensorSSARename);
  m.def("_jit_pass_tensorssa_remove_update", TensorSSARemoveUpdate);
  m.def("_jit_pass_convert_to_tensorssa", ConvertToTensorSSA);
  m.def("_jit_pass_fait_fuse_ops", FuseOps);
  m.def("_jit_pass_fait_canonicalize_fusable_maps", CanonicalizeFusableMaps);
  m.def("_jit_pass_collapse_assign_loops", CollapseAssignLoops);
  m.def("_jit_pass_collapse_recurrent_loops", CollapseRecurrentLoops);
  m.def("_jit_pass_canonicalize_ops", CanonicalizeOps);
  m.def("_jit_pass_fold_static_type_queries", FoldStaticTypeQueries);
  m.def("_jit_pass_uniform_constants_to_fills", UniformConstantsToFills);
  m.def("_jit_pass_hoist_loop_invariants", HoistLoopInvariants);
  m.def("_jit_pass_parallelize_loops", ParallelizeLoops);
  m.def("_jit_pass_split_parallel_maps", SplitParallelMaps);
  m.def("_jit_pass_unroll_loops_with_deps", UnrollLoopsWithDeps);
  m.def("_jit_pass_unroll_simple_maps", UnrollSimpleMaps);
  m.def("_jit_pass_fuse_masked_select", FuseMaskedSelect);
  m.def("_jit_pass_to_parallel_functor", ToParallelFunctor);
  m.def("_jit_pass_fait_pipeline", FaitPipeline);
  // functs/csrc/jit/python/init.cpp:45: FaitGetRefineType (fait_pipeline.cpp:19-29) gives the graph
  // inputs the types of the examples and propagates dtype / device / shape.  The propagation is
  // libtorch's own; regions specialise on the shapes they are called with, so nothing downstream
  // depends on it.  `refined_types` (per-value types of list elements in the reference) is accepted
  // and left alone: a Python dict crosses this boundary by value in the reference as well.
  m.def("_jit_pass_fait_shape_infer",
        [](std::shared_ptr<Graph> g, std::vector<c10::TypePtr> type_hint, py::object /*refined_types*/) {
          auto inputs = g->inputs();
          TORCH_CHECK(type_hint.size() <= inputs.size(), "_jit_pass_fait_shape_infer: ", type_hint.size(),
                      " type hints for ", inputs.size(), " graph inputs");
          const size_t off = inputs.size() - type_hint.size();   // a leading `self` of a module graph
          for (size_t i = 0; i < type_hint.size(); ++i) {
            auto tt = type_hint[i]->cast<c10::TensorType>();
            if (!tt) continue;
            // the propagation wants complete types: contiguous strides for a hint that carries sizes only
            auto sizes = tt->sizes().concrete_sizes();
            if (sizes && tt->scalarType() && tt->device() && !tt->strides().concrete_sizes())
              inputs[off + i]->setType(c10::TensorType::createContiguous(*tt->scalarType(), *tt->device(), *sizes));
            else
              inputs[off + i]->setType(tt);
          }
          torch::jit::ConstantPropagation(g);   // int[] arguments become constants the shape rules can read
          torch::jit::PropagateInputShapes(g);
        },
        py::arg("graph"), py::arg("type_hint"), py::arg("refined_types") = py::dict());
  // init.cpp:47-48: Freeze(Module*) folds attributes into the graph in place, Clone(Module*) copies
  // (fait/passes/freeze_module.cpp:954-960).  Stock libtorch does both.
  m.def("_jit_pass_freeze", [](torch::jit::Module& module) { module = torch::jit::freeze_module(module); });
  m.def("_jit_pass_clone", [](torch::jit::Module& module) { return module.clone(); });
  m.def("_jit_pass_validate", Validate);
  m.def("_jit_pass_convert_profiling_instrumentation", ConvertProfilingInstrumentation);
  m.def("_prof_begin", profBegin);
  m.def("_prof_end", profEnd);
  m.def("_prof_results", profilingResults);
  m.def("_prof_reset", resetProfiling);
  m.def("_create_function_from_graph", [](const std::string& name, std::shared_ptr<Graph> graph) {
    // script_init.cpp:87-95; the stock GraphFunction + interpreter run the graph
    auto cu = std::make_shared<torch::jit::CompilationUnit>();
    auto* fn = cu->create_function(c10::QualifiedName(name), std::move(graph));
    return torch::jit::StrongFunctionPtr(std::move(cu), fn);
  });
  m.def("_jit_pass_sink_producers_into_maps", SinkProducersIntoMaps);
  m.def("_set_sink_producers", setSinkProducers);
  m.def("_plan_functors", PlanFunctors);
  m.def("_jit_pass_infer_static_shapes", InferStaticShapes);
  m.def("_jit_pass_fuse_detection_tail", FuseDetectionTail);
  m.def("_jit_pass_pad_compacted_results", PadCompactedResults);
  m.def("_functor_host_timing", functorHostTiming);
  m.def("_functor_host_times", []() {
    py::dict d;
    for (const auto& kv : functorHostTimes()) d[py::str(kv.first)] = kv.second;
    return d;
  });
  // Hash of the shapes, dtypes and devices of the tensor arguments (lists and tuples of tensors
  // element by element) and of the kind of every other argument: the key under which
  // functs_amd.jit keeps the graphs it has built for a function.  The device is part of it because
  // a built graph holds folded prim::device constants and constant tensors on its example's device.
  m.def("_shape_key", [](const py::args& args) -> uint64_t {
    uint64_t h = 1469598103934665603ull;
    auto mix = [&h](uint64_t v) {
      h ^= v;
      h *= 1099511628211ull;
    };
    auto tensor = [&mix](PyObject* o) {
      const at::Tensor& t = THPVariable_Unpack(o);
      mix(0x7e50ull + (uint64_t)t.dim());
      for (int64_t d : t.sizes()) mix((uint64_t)d);
      mix((uint64_t)t.scalar_type());
      mix(0xde71ceull + ((uint64_t)(uint8_t)t.device().type() << 8) + (uint64_t)(uint8_t)t.device().index());
    };
    auto other = [&mix](PyObject* o) {   // bool before int: a Python bool is an int
      mix(o == Py_None ? 0x5ca1a0ull : PyBool_Check(o) ? 0x5ca1a1ull : PyLong_Check(o) ? 0x5ca1a2ull : PyFloat_Check(o) ? 0x5ca1a3ull
          : PyUnicode_Check(o) ? 0x5ca1a4ull : 0x5ca1a7ull);
    };
    for (const py::handle& a : args) {
      PyObject* o = a.ptr();
      if (THPVariable_Check(o)) {
        tensor(o);
      } else if (PyList_Check(o) || PyTuple_Check(o)) {
        const Py_ssize_t n = PySequence_Fast_GET_SIZE(o);
        mix(0x115700ull + (uint64_t)n);
        for (Py_ssize_t i = 0; i < n; ++i) {
          PyObject* e = PySequence_Fast_GET_ITEM(o, i);
          if (THPVariable_Check(e)) tensor(e);
          else other(e);
        }
      } else {
        other(o);
      }
    }
    return h;
  });
  m.def("_fxhip_library", []() { return functs::fxhipLibraryPath(); });
  py::class_<TensorList>(m, "TensorList")
      .def("__len__", [](const TensorList& self) { return self.list.size(); })
      .def("__getitem__",
           [](const TensorList& self, int64_t k) {
             const int64_t n = (int64_t)self.list.size();
             if (k < -n || k >= n) throw py::index_error("TensorList index out of range");
             return py::reinterpret_steal<py::object>(THPVariable_Wrap(self.list.get((size_t)(k < 0 ? k + n : k))));
           })
      .def("__getitem__", [](const TensorList& self, const py::slice& s) -> py::object { return py::object(self.tolist()[s]); })
      .def("__iter__", [](const TensorList& self) -> py::object { return py::iter(self.tolist()); })
      .def("tolist", &TensorList::tolist)
      .def("__repr__", [](const TensorList& self) { return "TensorList(" + std::to_string(self.list.size()) + " tensors)"; });
  // (a TensorList over given tensors: what a lazy result is, without running a functor)
  m.def("_tensor_list", [](const std::vector<at::Tensor>& tensors) { return TensorList{c10::List<at::Tensor>(tensors)}; });
  py::class_<DirectFunctor, std::shared_ptr<DirectFunctor>>(m, "DirectFunctor")
      .def_readwrite("lazy_lists", &DirectFunctor::lazy_lists)
      .def("__call__", [](const DirectFunctor& self, const py::args& args) { return self.call(args); });
  // the direct form of a built graph, or None when the graph is more than one functor
  m.def("_direct_functor", [](std::shared_ptr<Graph> graph) { return DirectFunctor::match(graph); });
}
