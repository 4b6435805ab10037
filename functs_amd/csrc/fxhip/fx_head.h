// Hand-written kernel for one region shape: the decode + score filter of a YOLO-style detection
// head (functs/benchmark/ai_model/yolov3/yolov3_bbox.py:12-23, 104-130 in the reference: sigmoid
// of the centre offsets, exp of the sizes, anchors and strides, objectness threshold, kept rows
// of boxes / class scores / objectness).  A plan whose lowered programs ARE that computation
// (fx::match_head compares them instruction by instruction, whatever the slot numbering, the
// number of classes, rows and images and the threshold) can run as ONE launch of
// fx_head_stream instead of the two passes of the generic row compaction; every other region
// is untouched.  Results are bit-identical to the generic kernels: same device functions, same
// order of operations.
#pragma once
#include <stdint.h>

#include "fx_bytecode.h"

#define FX_HEAD_SUB 64u        // most rows of a sub-tile (one ballot)
#define FX_HEAD_NSUB 4u        // most sub-tiles of a chunk: a chunk holds at most FX_BLOCK rows
#define FX_HEAD_KV 6u          // 128-bit loads per lane that carry a sub-tile
#define FX_HEAD_STATUS_BITS 9u // a chunk's count is at most FX_BLOCK
#define FX_HEAD_FLOOD_BYTES (8u << 20)   // first sub-tiles of a launch from which on the counts are sent ahead of the rows
#define FX_HEAD_BULK_DELAY 128u           // by this many units of 64 clocks
#define FX_HEAD_MIN_CHUNK 64u  // fewest rows of a chunk unless the image has fewer
// hash of the normalised programs of the detection-head region (fx_head_match.cpp)
#define FX_HEAD_NORM_HASH 0xed6ab9314c50ff65ull
// the same region with the anchors folded into box centres [N, 2] and half sizes [N, 2] and the
// strides as [N, 1] (what constant propagation leaves of anchors generated from static shapes)
#define FX_HEAD_NORM_HASH_FOLDED 0x680166c2c9e835ddull

// What the matcher found (host).
struct FxHeadInfo {
  bool ok = false;
  uint64_t norm_hash = 0;        // hash of the normalised programs (reported also when they do not match)
  uint32_t pred_slot = 0, anc_slot = 0, strd_slot = 0;   // pointer slots (FX_SLOT_TASK: per-task table)
  int32_t pred_tcoef = 0, anc_tcoef = 0, strd_tcoef = 0; // element offset per task
  bool folded = false;           // centres and half sizes instead of anchors: anc_* is the centres', half_* the half sizes'
  uint32_t half_slot = 0;
  int32_t half_tcoef = 0;
  uint32_t S = 0, C = 0;         // floats per prediction row (5 + C), classes
  uint32_t thr_bits = 0;         // objectness threshold (float bits)
  uint32_t n_rows = 0, n_tasks = 0;
  uint32_t out_slot[3] = {0, 0, 0};      // objectness [K], boxes [K, 4], class scores [K, C]
  uint32_t out_tstride[3] = {0, 0, 0};   // element offset per task
  uint32_t slot_total = 0;
};

// Kernel arguments (by value, followed by the FxDyn block in the argument segment).
struct FxHeadLaunch {
  uint32_t n_rows, n_tasks;
  uint32_t chunks, chunk_rows;   // workgroups per task and rows of each (<= FX_BLOCK)
  uint32_t sub_rows;             // rows of a sub-tile (<= FX_HEAD_SUB; the window holds them)
  uint32_t S, C;
  uint32_t g_magic, g_shift;     // fast division by C / 4 (groups of four class scores per row)
  uint32_t thr_bits;
  uint32_t epoch, spin_limit;
  uint32_t n_sptr, n_tptr;
  uint32_t pred_slot, anc_slot, strd_slot;
  int32_t pred_tcoef, anc_tcoef, strd_tcoef;
  uint32_t out_slot[3], out_tstride[3];
  uint32_t bulk_delay;           // big launches: waves without a gather wait this long (units of 64 clocks) before they ask for rows
  uint32_t folded;               // 1: anc_slot holds box centres [N, 2], half_slot half sizes [N, 2]
  uint32_t half_slot;
  int32_t half_tcoef;
  uint32_t* status;              // one word per chunk, tagged with the epoch
  uint32_t* totals;              // pinned host memory: kept rows per task
};
static_assert(sizeof(FxHeadLaunch) % 8 == 0, "the FxDyn block follows at an 8-byte boundary");
