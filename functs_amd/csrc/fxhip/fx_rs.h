// Row-stream kernels: a row compaction whose widest input is a row-major matrix read row by
// row, run as ONE launch of a kernel that is GENERATED from the region's own lowered programs.
//
// The generator (fx_rs_gen.cpp) executes the bytecode of the mask and of every output
// symbolically, once per output column with the column index a constant, into ONE expression
// graph per row: predicates of select_rev / slice_rev / cat / stack chains that depend on the
// column fold away, loads and sub-expressions that several columns share exist once (the
// decoded centre and half size of a box serve its four corners), loads of neighbouring elements
// become one wide load.  Long runs of columns that execute the same instructions (the class
// scores of a detection head) become a vector form, four columns per lane.  The result is a
// HIP translation unit (spec/fx_rs_<key>.hip) holding a policy class for the skeleton of
// fx_rowstream.h; built into the library, it serves every plan whose programs produce the same
// key: any number of rows and tasks, any pointers, any per-task offsets, and any VALUES of the
// floating-point constants (thresholds, scale factors) as long as equal constants stay equal.
//
// This is the counterpart of the reference's per-subgraph code generator
// (fait/tensorexpr/cuda_codegen_tssa.cpp:881-1121); the compiler runs when the library is
// built instead of when the operator is created (CompileToNVRTC, :1319-1414).
#pragma once
#include <stdint.h>

#include <string>
#include <vector>

#include "fx_bytecode.h"

#define FX_RS_VERSION 3u
#define FX_RS_MAX_IN 8u         // input buffers of a region
#define FX_RS_MAX_OUT 8u        // outputs
#define FX_RS_MAX_FIMM 24u      // distinct floating-point constants
#define FX_RS_SUB 64u           // most rows of a sub-tile (one ballot)
#define FX_RS_NSUB 4u           // most sub-tiles of a chunk: a chunk holds at most FX_BLOCK rows
#define FX_RS_KV 6u             // most 128-bit loads per lane that carry a sub-tile
#define FX_RS_KV_LEAN 5u        // every kernel is also built for five (four registers less: 70 instead of 77 on the
                                // benchmark's region, 22.5 against 23.2 us); the host takes it where it costs no sub-tile
#define FX_RS_STATUS_BITS 9u    // a chunk's count is at most FX_BLOCK
#define FX_RS_MIN_CHUNK 64u     // fewest rows of a chunk unless a task has fewer
#define FX_RS_FLOOD_BYTES (8u << 20)   // first sub-tiles of a launch from which on the counts are sent ahead of the rows
#define FX_RS_BULK_DELAY 128u          // by this many units of 64 clocks
#define FX_RS_OCC 6              // waves per SIMD the register budget of a generated kernel is set for (80 registers)
#define FX_RS_VEC_MIN 8u        // shortest run of alike columns that takes the vector form
#define FX_RS_MAX_UNROLL 64u    // most columns evaluated one by one per row
#define FX_RS_MAX_SIDE 16u      // most words per row that a chunk keeps in LDS of what its rows read besides the window

// What the analysis of a plan found (host).
struct FxRsInfo {
  bool ok = false;
  std::string why;              // when not ok: what rules the region out
  uint64_t key = 0;             // of the generated kernel that serves this plan
  uint32_t S = 0;               // elements per row of the window input
  uint32_t n_rows = 0, n_tasks = 0;
  uint32_t n_in = 0;
  uint32_t in_slot[FX_RS_MAX_IN] = {};     // pointer slot of each input (FX_SLOT_TASK: per-task table); 0 is the window
  int32_t in_tcoef[FX_RS_MAX_IN] = {};     // element offset per task
  uint32_t n_out = 0;
  uint32_t out_slot[FX_RS_MAX_OUT] = {};
  uint32_t out_tstride[FX_RS_MAX_OUT] = {};
  uint32_t n_fimm = 0;
  uint32_t fimm[FX_RS_MAX_FIMM] = {};      // values (float bits) of this plan's floating-point constants
  uint32_t slot_err = 0;        // 1 + shared pointer slot of the error word of guarded int64 loads (0: none)
};

// Kernel arguments (by value, followed by the FxDyn block in the argument segment).
struct FxRsLaunch {
  uint32_t n_rows, n_tasks;
  uint32_t chunks, chunk_rows;  // workgroups per task and rows of each (<= FX_BLOCK)
  uint32_t sub_rows;            // rows of a sub-tile (<= FX_RS_SUB; the window holds them)
  uint32_t epoch, spin_limit;
  uint32_t n_sptr, n_tptr, n_sscal, n_tscal;
  uint32_t bulk_delay;          // big launches: waves without a gather wait this long (units of 64 clocks) before they ask for rows
  uint32_t in_slot[FX_RS_MAX_IN];
  int32_t in_tcoef[FX_RS_MAX_IN];
  uint32_t out_slot[FX_RS_MAX_OUT], out_tstride[FX_RS_MAX_OUT];
  uint32_t fimm[FX_RS_MAX_FIMM];
  uint32_t slot_err;
  uint32_t side_lds;            // the chunk keeps a table of its rows' side values in LDS (0: a row loads them when its turn comes)
  uint32_t late_tell;           // tuning aid: the task's last chunk looks back where the others do (the host hears the total later)
  uint32_t pad0;
  // what a workgroup would otherwise divide for: b / chunks by multiplication, and the sub-tiles
  // (equal in size, at most sub_rows rows) of a whole chunk and of a task's last chunk
  uint32_t chunks_magic, chunks_shift;
  uint32_t sub_rows_whole, n_sub_whole;
  uint32_t rows_last, sub_rows_last, n_sub_last;
  uint32_t pad1;
  uint32_t* status;             // one word per chunk, tagged with the epoch
  uint32_t* totals;             // pinned host memory: kept rows per task
  uint64_t wide;                // 0, or the device address of the call's tables (pointers, then scalars) where the FxDyn block is too small for them
};
static_assert(sizeof(FxRsLaunch) % 8 == 0, "the FxDyn block follows at an 8-byte boundary");
// the derived fields of a launch block whose n_rows, chunk_rows, chunks and sub_rows are set
static inline void fx_rs_finish_geometry(FxRsLaunch* rl) {
  fx_fastdiv_make(rl->chunks ? rl->chunks : 1u, &rl->chunks_magic, &rl->chunks_shift);
  auto split = [&](uint32_t rows, uint32_t* sub_rows, uint32_t* n_sub) {
    const uint32_t cap = rl->sub_rows ? rl->sub_rows : 1u;
    const uint32_t n0 = rows ? (rows + cap - 1u) / cap : 1u;
    *sub_rows = rows ? (rows + n0 - 1u) / n0 : 1u;
    *n_sub = rows ? (rows + *sub_rows - 1u) / *sub_rows : 0u;
  };
  const uint32_t whole = rl->chunk_rows;
  rl->rows_last = rl->chunks ? rl->n_rows - (rl->chunks - 1u) * whole : 0u;
  split(whole, &rl->sub_rows_whole, &rl->n_sub_whole);
  split(rl->rows_last, &rl->sub_rows_last, &rl->n_sub_last);
}

// ---- host side: generated kernels linked into the library ----
struct FxRsKernel {
  const void* fn = nullptr;     // fx_rs_kernel<P, FX_RS_KV, false>
  const void* fn_lean = nullptr; // fx_rs_kernel<P, FX_RS_KV_LEAN, false>
  const void* fn_persist = nullptr; // fx_rs_kernel<P, FX_RS_KV, true>: workgroups that take several chunks in turn
  const void* fn_wide = nullptr;    // fx_rs_kernel<P, FX_RS_KV, true, true>: the same, reading the call's tables from device memory (FxRsLaunch::wide)
  uint32_t S = 0;               // row length the kernel is generated for
  uint32_t stage_row_words = 0; // elements per kept row that the kernel puts together in LDS before they leave
  uint32_t n_staged = 0;        // outputs that take that route
  uint32_t side_row_words = 0;  // words per row of the chunk's table of what the rows read besides the window
};
void fx_rs_register(uint64_t key, const FxRsKernel& k);
const FxRsKernel* fx_rs_find(uint64_t key);
int fx_rs_count();
