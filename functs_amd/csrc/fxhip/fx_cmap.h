// Hand-written kernel for one region shape: the decode + per-class score filter of an SSD-style
// detection head (functs/benchmark/ai_model/ssd/ssd_bbox.py:163-214 in the reference: prior /
// variance decode of the boxes, softmax over the class scores of every prior, then for every
// foreground class the rows whose score exceeds a threshold, as boxes [K, 4] and scores [K]).
// The region is a ParallelMap over the classes whose body holds the whole computation; lowered
// generically every task would redo the decode and the softmax.  A plan whose lowered programs
// ARE that computation (fx::match_classmap compares them instruction by instruction, whatever
// the slot numbering, the number of priors and classes, the first class, the threshold and the
// two variances) runs as ONE launch of fx_classmap_head that computes every row once and serves
// all classes from it.  The arithmetic is that of the region split in two (a dense region for
// decode + softmax whose rows are reduced across the lanes of a wave, and a class map over its
// results): same device functions, same order of operations, bit-identical results.
#pragma once
#include <stdint.h>

#include "fx_bytecode.h"

#define FX_CMAP_MAX_CLS 128u      // floats of a score row: 32 lanes hold four each
#define FX_CMAP_MAX_TASKS 128u
#define FX_CMAP_STATUS_BITS 9u    // a chunk's count per class is at most 64
// hash of the normalised programs of the region (fx_cmap_match.cpp)
#define FX_CMAP_NORM_HASH 0x6daa91ac9f5380ebull

// What the matcher found (host).
struct FxCmapInfo {
  bool ok = false;
  uint64_t norm_hash = 0;          // reported also when the programs do not match
  uint32_t conf_slot = 0, loc_slot = 0, pri_slot = 0;   // pointer slots
  uint32_t C = 0;                  // floats per score row
  uint32_t first = 0;              // task t filters class first + t
  uint32_t thr_bits = 0;           // score threshold (float bits)
  uint32_t var_xy_bits = 0, var_wh_bits = 0;   // the two variances (float bits)
  uint32_t n_rows = 0, n_tasks = 0;
  uint32_t out_slot[2] = {0, 0};     // scores [K], boxes [K, 4]
  uint32_t out_tstride[2] = {0, 0};  // element offset per task
};

// Kernel arguments (by value, followed by the FxDyn block in the argument segment).
struct FxCmapLaunch {
  uint32_t n_rows, n_tasks;
  uint32_t chunks, chunk_rows;     // workgroups and rows of each (32 or 64)
  uint32_t C, first;
  uint32_t thr_bits, var_xy_bits, var_wh_bits;
  uint32_t epoch, spin_limit;
  uint32_t n_sptr, n_tptr;
  uint32_t conf_slot, loc_slot, pri_slot;
  uint32_t out_slot[2], out_tstride[2];
  uint32_t* status;                // n_tasks x chunks words (class-major), tagged with the epoch
  uint32_t* totals;                // pinned host memory: kept rows per task
};
static_assert(sizeof(FxCmapLaunch) % 8 == 0, "the FxDyn block follows at an 8-byte boundary");
