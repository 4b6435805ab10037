// Schemas and eager (ATen) bodies of the immut:: operator family.
// Reference: functs/csrc/jit/ir/symbol_ext.cpp:9-199.  Same schemas, same
// values.  One deliberate difference: the reference's *_rev bodies write into
// `self` in place although the operators are registered as pure functions
// (symbol_ext.cpp:21-29, 40-50); here they work on a copy, so that the operators
// really are pure and graphs stay correct under CSE / reordering.
#include <ATen/ATen.h>
#include <torch/csrc/jit/runtime/custom_operator.h>
#include <torch/library.h>

#include "symbols.h"

namespace functs {

const std::unordered_map<Symbol, Symbol>& immutableVersion() {
  static const std::unordered_map<Symbol, Symbol> m{
      {c10::aten::copy_, sym::Assign()},         {c10::aten::select, sym::Select()},
      {c10::aten::slice, sym::Slice()},          {c10::aten::permute, sym::Permute()},
      {c10::aten::squeeze, sym::Squeeze()},      {c10::aten::unsqueeze, sym::Unsqueeze()},
      {c10::aten::view, sym::View()},            {c10::aten::reshape, sym::Reshape()},
      {c10::aten::expand, sym::Expand()},        {c10::aten::expand_as, sym::ExpandAs()},
  };
  return m;
}

const std::unordered_map<Symbol, Symbol>& reverseVersion() {
  static const std::unordered_map<Symbol, Symbol> m{
      {sym::Assign(), sym::Assign()},       {sym::Select(), sym::SelectRev()},   {sym::Slice(), sym::SliceRev()},
      {sym::Permute(), sym::PermuteRev()},  {sym::Squeeze(), sym::Unsqueeze()},  {sym::Unsqueeze(), sym::Squeeze()},
      {sym::View(), sym::View()},           {sym::Reshape(), sym::View()},       {sym::Expand(), sym::ExpandRev()},
      {sym::ExpandAs(), sym::ExpandAsRev()}, {sym::Repeat(), sym::RepeatRev()},
  };
  return m;
}

namespace {
using at::Tensor;

Tensor access(Tensor src) { return src; }
Tensor assign(Tensor self, Tensor src, std::optional<bool>) { return src; }
Tensor select(Tensor src, int64_t dim, int64_t index) { return src.select(dim, index); }
Tensor select_rev(Tensor self, Tensor src, int64_t dim, int64_t index) {
  Tensor out = self.clone();
  out.select(dim, index).copy_(src);
  return out;
}
Tensor slice(Tensor src, int64_t dim, std::optional<int64_t> start, std::optional<int64_t> end, int64_t step) {
  return src.slice(dim, start, end, step);
}
Tensor slice_rev(Tensor self, Tensor src, int64_t dim, std::optional<int64_t> start, std::optional<int64_t> end,
                 int64_t step) {
  Tensor out = self.clone();
  out.slice(dim, start, end, step).copy_(src);
  return out;
}
Tensor squeeze(Tensor src, int64_t dim) { return src.squeeze(dim); }
Tensor unsqueeze(Tensor src, int64_t dim) { return src.unsqueeze(dim); }
Tensor view(Tensor src, at::IntArrayRef dims) { return src.reshape(dims); }
Tensor reshape(Tensor src, at::IntArrayRef dims) { return src.reshape(dims); }
Tensor permute(Tensor src, at::IntArrayRef dims) { return src.permute(dims); }
// writes `src` (shaped like self.permute(dims)) back: the inverse permutation
Tensor permute_rev(Tensor self, Tensor src, at::IntArrayRef dims) {
  std::vector<int64_t> inv(dims.size());
  for (size_t i = 0; i < dims.size(); ++i) inv[at::maybe_wrap_dim(dims[i], (int64_t)dims.size())] = (int64_t)i;
  return src.permute(inv).expand_as(self).contiguous();
}
Tensor expand(Tensor src, at::IntArrayRef sizes, bool implicit) { return src.expand(sizes, implicit); }
Tensor expand_as(Tensor src, Tensor other) { return src.expand_as(other); }
Tensor repeat(Tensor self, at::IntArrayRef sizes) { return self.repeat(sizes); }
Tensor index(Tensor src, c10::List<std::optional<Tensor>> indices) { return src.index(indices); }

// The three operators below are in the reference's registry (symbol_ext.cpp:83-111, 176-195)
// but none of its passes emits them.  The bodies give the results the reference's bodies give,
// on a fresh tensor instead of through `self`.
Tensor expand_rev(Tensor src, at::IntArrayRef sizes, bool implicit) { return src.expand(sizes, implicit); }
// reference: self.repeat(sizes).copy_(src) writes into the temporary that repeat returns, so
// the result is `self` as it was
Tensor repeat_rev(Tensor self, Tensor src, at::IntArrayRef sizes) {
  TORCH_CHECK(at::is_expandable_to(src.sizes(), self.repeat(sizes).sizes()),
              "immut::repeat_rev: src does not broadcast to self.repeat(size)");
  return self.clone();
}
// reference: self.expand_as(other).copy_(src); ATen refuses the copy as soon as the view
// really expands (one element would be written more than once)
Tensor expand_as_rev(Tensor self, Tensor src, Tensor other) {
  TORCH_CHECK(self.sizes() == other.sizes(),
              "immut::expand_as_rev: more than one element of the written-to tensor refers to a single memory "
              "location (self ", self.sizes(), " expanded as ", other.sizes(), ")");
  return src.expand_as(self).to(self.scalar_type()).contiguous();
}

}  // namespace

// immut:: schemas as functs/csrc/jit/ir/symbol_ext.cpp:9-199 registers them; no alias
// annotations, so alias analysis treats every operator as a pure function.
TORCH_LIBRARY(immut, m) {
  m.def("access(Tensor src) -> Tensor", access);
  m.def("assign(Tensor self, Tensor src, bool? n=None) -> Tensor", assign);
  m.def("select(Tensor src, int dim, int index) -> Tensor", select);
  m.def("select_rev(Tensor self, Tensor src, int dim, int index) -> Tensor", select_rev);
  m.def("slice(Tensor src, int dim=0, int? start=None, int? end=None, int step=1) -> Tensor", slice);
  m.def("slice_rev(Tensor self, Tensor src, int dim=0, int? start=None, int? end=None, int step=1) -> Tensor",
        slice_rev);
  m.def("squeeze(Tensor self, int dim) -> Tensor", squeeze);
  m.def("unsqueeze(Tensor self, int dim) -> Tensor", unsqueeze);
  m.def("view(Tensor self, int[] size) -> Tensor", view);
  m.def("reshape(Tensor self, int[] size) -> Tensor", reshape);
  m.def("permute(Tensor self, int[] sizes) -> Tensor", permute);
  m.def("permute_rev(Tensor self, Tensor src, int[] sizes) -> Tensor", permute_rev);
  m.def("expand(Tensor self, int[] size, *, bool implicit=False) -> Tensor", expand);
  m.def("expand_as(Tensor self, Tensor other) -> Tensor", expand_as);
  m.def("repeat(Tensor self, int[] size) -> Tensor", repeat);
  m.def("index.Tensor(Tensor self, Tensor?[] indices) -> Tensor", index);
  m.def("expand_rev(Tensor self, int[] size, *, bool implicit=False) -> Tensor", expand_rev);
  m.def("repeat_rev(Tensor self, Tensor src, int[] size) -> Tensor", repeat_rev);
  m.def("expand_as_rev(Tensor self, Tensor src, Tensor other) -> Tensor", expand_as_rev);
}

}  // namespace functs
