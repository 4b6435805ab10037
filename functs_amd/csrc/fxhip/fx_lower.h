// Host-side region IR, shape functions and lowering to VM bytecode.
// Pure C++ (no HIP): everything here runs without a device.
//
// Plays the role of fait/fuser/graph_builder.cpp:259-712 (GraphBuilder::compile),
// the shape tables fait/fuser/shape_func.cpp:9-374 and the lowering functions
// functs/csrc/jit/tensorexpr/nnc_ext.cpp:62-392 /
// fait/fuser/custom_lowering_func.cpp:17-498, but emits descriptors for
// hand-written kernels instead of NNC statements.
#pragma once
#include <stdint.h>

#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../../include/fxhip.h"
#include "fx_bytecode.h"
#include "fx_cmap.h"
#include "fx_head.h"
#include "fx_rs.h"

namespace fx {

struct Error : std::runtime_error {
  int code;
  Error(int c, const std::string& m) : std::runtime_error(m), code(c) {}
};

enum VKind { VK_TENSOR, VK_INT, VK_FLOAT, VK_BOOL, VK_NONE, VK_INT_LIST, VK_TENSOR_LIST };
enum Prod { P_INPUT, P_CONST, P_TASK, P_LOOPVAR, P_LIST, P_OP };

struct Value {
  VKind kind = VK_NONE;
  Prod prod = P_CONST;
  int dtype = -1;  // FX_DT_* for tensors
  int rank = -1;
  int op = 0;
  std::vector<int> args;
  int64_t ival = 0;
  double fval = 0;
  int input_index = -1;
  bool per_task = false;
};

struct Plan;

struct Region {
  int degree = 1;
  bool is_map = false;
  bool finalized = false;
  std::vector<Value> vals;
  std::vector<int> inputs;   // value ids, declaration order
  std::vector<int> outputs;  // value ids
  int mask = -1;             // row-compaction mask value id
  // per-task int inputs (by input index) whose values shapes or index arithmetic depend on:
  // found out while lowering; their values are part of the plan key and split the tasks
  // into classes (all other per-task scalars are plain run-time data)
  std::vector<char> index_ints;
  std::map<std::vector<int64_t>, std::unique_ptr<Plan>> plans;

  int add(const Value& v) {
    vals.push_back(v);
    return (int)vals.size() - 1;
  }
  int addOp(int opcode, const std::vector<int>& args, int out_dtype);
};

// where a dynamic pointer / scalar slot is filled from at run time
struct PtrSrc {
  enum Kind { INPUT, OUTPUT, FLAGS, COUNTS, TOTALS, ERRWORD, STATUS } kind;
  int index;  // region input index / output index
};
struct ScalSrc {
  int input;      // region input index
  bool as_float;  // store float(value) instead of int32(value)
};

// Streaming (one-pass) form of a row compaction, available when the region has one task class
// and its widest row-major input is read row by row by every program (fx_compact_stream).
struct StreamInfo {
  bool ok = false;
  uint32_t tile_rows = 0;       // rows per workgroup
  uint32_t tiles_per_task = 0;
  uint32_t rows = 0;            // rows per task
  uint32_t grid = 0;
  uint32_t win_slot = 0;        // pointer slot of the window input
  uint32_t win_stride = 0;      // elements per row
  int32_t win_tcoef = 0;        // element offset per task
  int32_t win_lo = 0;           // smallest element offset the programs read inside a row
  uint32_t win_span = 0;        // elements from there to the largest one, inclusive
  uint32_t win_words = 0;       // LDS words of the window (multiple of 4)
  // narrow inputs read row by row as well (at most 256 16-byte lines per tile): staged beside it
  uint32_t n_side = 0;
  uint32_t side_slot[2] = {0, 0}, side_stride[2] = {0, 0}, side_span[2] = {0, 0}, side_words[2] = {0, 0};
  int32_t side_tcoef[2] = {0, 0}, side_lo[2] = {0, 0};
};

struct Plan {
  const Region* region = nullptr;
  std::vector<uint32_t> blob;  // static part (FxHeader ...)
  uint32_t mode = FX_MODE_DENSE;
  uint32_t grid = 0;           // dense grid, or scatter grid in compaction mode
  uint32_t grid_count = 0;     // compaction pass 1
  uint32_t lds_bytes = 0;
  // A call with more pointers or scalars than the kernel argument block holds (a map of many
  // tasks): the tables are written to device memory at wide_off of the caller's scratch by small
  // upload launches ahead of the kernels, which stage them from there.  Such a plan runs the
  // general kernels only.
  bool wide = false;
  size_t wide_off = 0, wide_bytes = 0;
  bool needs_compiled = false;   // the interpreter's temporaries exceed the LDS of a workgroup
  StreamInfo stream;
  FxHeadInfo head;               // the plan is the decode + score filter of a detection head (fx_head.h)
  FxCmapInfo cmap;               // the plan is the decode + per-class score filter of an SSD-style head (fx_cmap.h)
  FxRsInfo rs;                   // the plan has a row-stream form (fx_rs.h): key of the generated kernel that serves it
  bool uses_guard = false;       // some load checks int64 data against 32 bits and reports to the error word
  uint32_t n_temps = 0;
  int max_rank = 1;
  std::vector<PtrSrc> sptr, tptr;
  std::vector<ScalSrc> sscal, tscal;
  std::vector<int> out_dtype;                                 // per output
  std::vector<std::vector<std::vector<int64_t>>> out_shape;   // [out][task][dim]
  size_t scratch_bytes = 0, flags_off = 0, counts_off = 0;
  int launches = 0;
  int64_t alg_bytes = 0;
  std::vector<int> arg_base;  // first fx_arg of each region input
  int n_args = 0;
  // device copy of blob, created on first run
  uint64_t spec_key = 0;       // spec_hash of this plan
  void* dev_blob = nullptr;
  int dev_id = -1;
  // streaming compaction: tile status words, one buffer per launch stream (zero when allocated,
  // never reset: every call tags its words with the next epoch)
  struct Status { void* stream; void* ptr; uint32_t epoch; int dev; };
  std::vector<Status> status;
  // the same for the chunks of the detection-head kernel, and the workgroups of it the device holds at once
  std::vector<Status> head_status;
  uint32_t head_resident = 0;
  uint32_t cmap_resident_wide = 0;   // class-map head kernel: workgroups of its wide form
  FxLeanArgs lean{};           // dense regions that fit the lean kernel: its argument block but for the per-call parts (n_outs 0: none)
  uint32_t lean_slot_err = 0;  // as FxHeader::slot_err
  uint32_t rs_lean = 0, rs_side_lds = 0, rs_sub_rows = 0, rs_chunk_rows = 0, rs_grid_cap = 0;   // row-stream kernel: geometry of a launch (chosen at the first one)
};

// Fills p->head: does the plan compute the decode + score filter of a detection head (fx_head_match.cpp)?
void match_head(Plan* p);
// Fills p->cmap: does the plan compute the decode + per-class score filter of an SSD-style head (fx_cmap_match.cpp)?
void match_classmap(Plan* p);

// Builds (or fetches from the cache) the plan of `r` for these arguments.
const Plan* plan_region(Region& r, const fx_arg* args, int n_args);
std::string disasm(const Plan& p);
// Rank the region kernels are instantiated for (1, 2, 3, 4 or FX_MAXR).
int kernel_rank(int rank);
// Key of the compile-time part of a plan (programs, entry points, kernel rank); 0 if the plan
// cannot be specialised.  spec_source writes the translation unit that specialises it.
uint64_t spec_hash(const Plan& p);
std::string spec_source(const Plan& p, const std::string& label);
// Row-stream form of a compacting plan (fx_rs.h, fx_rs_gen.cpp): rs_analyze fills p->rs,
// rs_source writes the translation unit of the kernel that serves every plan with that key.
void rs_analyze(Plan* p);
std::string rs_source(const Plan& p, const std::string& label);
const char* opname(uint32_t op);

int dtype_size(int dt);

}  // namespace fx
