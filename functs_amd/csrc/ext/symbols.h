// Symbols and operator tables of the functionalized (TensorSSA) dialect.
// Same names as the reference so that graphs, printed IR and user scripts
// carry over: functs/csrc/jit/ir/symbol_ext.h:11-85, fait/passes/te_op.h:13-23,
// fait/passes/parallelize_loops.h:11.
#pragma once
#include <ATen/core/interned_strings.h>
#include <ATen/core/symbol.h>
#include <torch/csrc/jit/ir/ir.h>

#include <unordered_map>

namespace functs {
using c10::Symbol;
namespace aten = c10::aten;
namespace prim = c10::prim;
namespace attr = c10::attr;

namespace sym {
inline Symbol q(const char* s) { return Symbol::fromQualString(s); }
#define FUNCTS_SYM(name, text) \
  inline Symbol name() {       \
    static Symbol s = q(text); \
    return s;                  \
  }
FUNCTS_SYM(Update, "tssa::update")
FUNCTS_SYM(ParallelFunctor, "tssa::ParallelFunctor")
FUNCTS_SYM(Access, "immut::access")
FUNCTS_SYM(Assign, "immut::assign")
FUNCTS_SYM(Select, "immut::select")
FUNCTS_SYM(SelectRev, "immut::select_rev")
FUNCTS_SYM(Slice, "immut::slice")
FUNCTS_SYM(SliceRev, "immut::slice_rev")
FUNCTS_SYM(Squeeze, "immut::squeeze")
FUNCTS_SYM(Unsqueeze, "immut::unsqueeze")
FUNCTS_SYM(View, "immut::view")
FUNCTS_SYM(Reshape, "immut::reshape")
FUNCTS_SYM(Permute, "immut::permute")
FUNCTS_SYM(PermuteRev, "immut::permute_rev")
FUNCTS_SYM(Expand, "immut::expand")
FUNCTS_SYM(ExpandRev, "immut::expand_rev")
FUNCTS_SYM(ExpandAs, "immut::expand_as")
FUNCTS_SYM(ExpandAsRev, "immut::expand_as_rev")
FUNCTS_SYM(Repeat, "immut::repeat")
FUNCTS_SYM(RepeatRev, "immut::repeat_rev")
FUNCTS_SYM(Index, "immut::index")
FUNCTS_SYM(ParallelMap, "prim::ParallelMap")
// a prim::Loop whose carried tensor is read and written only through slab i,
// collapsed to one node (no reference counterpart, see fuse_ops.cpp)
FUNCTS_SYM(ForallSelectRev, "fx::forall_select_rev")
// the (time, layer) loop nest of a stacked LSTM collapsed to one node (recurrent.cpp)
FUNCTS_SYM(LstmStack, "fx::lstm_stack")
// attributes of tssa::ParallelFunctor
FUNCTS_SYM(parallel_degree, "attr::parallel_degree")
FUNCTS_SYM(is_parallel_args, "attr::is_parallel_args")
FUNCTS_SYM(input_refine_types, "attr::input_refine_types")
FUNCTS_SYM(is_parallel_map, "attr::is_parallel_map")
FUNCTS_SYM(compact_rows, "attr::compact_rows")
// a compacting functor that returns every output at its full size (one tensor [tasks, rows, ...])
// and the kept-row counts as one more tensor, without waiting for them (detection_ops.cpp)
FUNCTS_SYM(padded_outputs, "attr::padded_outputs")
#undef FUNCTS_SYM
}  // namespace sym

// aten view / copy operator -> immutable twin (symbol_ext.h:55-70; the
// reference enables the second half only with ENABLE_NNC_INT_LIST)
const std::unordered_map<Symbol, Symbol>& immutableVersion();
// immutable access operator -> the assign operator that writes back through it
// (symbol_ext.h:72-85)
const std::unordered_map<Symbol, Symbol>& reverseVersion();

}  // namespace functs
