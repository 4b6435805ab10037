// Region bytecode shared by the host lowering (fx_lower.cpp), the gfx950 VM
// kernels (fx_kernels.hip) and the test-only scalar emulator.
//
// A fused functionalized region (the body of a prim::FusionGroup, possibly
// replicated over the tasks of a prim::ParallelMap) is lowered on the host to
// one small accumulator-machine program per region output.  The program
// computes ONE output element from its output coordinates; the kernel runs it
// for FX_V elements per lane at once so that instruction decode (scalar,
// wave-uniform) is amortised over 4 x 64 elements per wave.
//
// This replaces the CUDA-C text the reference generates per region
// (fait/tensorexpr/cuda_codegen_tssa.cpp:881-1121) and the per-element index
// arithmetic of its lowerings (functs/csrc/jit/tensorexpr/nnc_ext.cpp:62-392,
// fait/fuser/custom_lowering_func.cpp:17-498).
#pragma once
#include <stddef.h>
#include <stdint.h>

#define FX_MAXR 6        // max rank of a region output (root coordinates)
#define FX_V 4           // elements per lane
#define FX_BLOCK 256     // threads per workgroup (4 wavefronts of 64)
#define FX_STATIC_MAX_ROWS (1 << 22)  // most rows fx_compact_rows_static takes (64 KiB of tile counts per GPU)
#define FX_TILE (FX_V * FX_BLOCK)
#define FX_ITEM (FX_V * 64)  // elements one wave processes per work item
#define FX_UNIT (16 * FX_ITEM)  // dense kernel: elements of the largest work unit (4 waves x 4 items)
#define FX_MAX_TEMPS 24  // LDS temp slots per lane (each FX_V wide)
#define FX_MASK_DEPTH 16 // nesting depth of predicated regions (4 bits each in a u64)
#define FX_DYN_P 320     // 8-byte dynamic words passed by value (pointers)
#define FX_DYN_S 176     // 4-byte dynamic words passed by value (scalars)
#define FX_WIDE_P 4096   // most pointers of a call whose tables travel through device memory (maps of many tasks)
#define FX_WIDE_S 4096   // most scalars of such a call
#define FX_MAX_TPTR 32   // per-task pointers staged in LDS
#define FX_MAX_TSCAL 32  // per-task scalars staged in LDS
#define FX_MAGIC 0x46585231u  // "FXR1"

// storage dtypes of buffers
enum FxDtype : uint32_t {
  FX_F32 = 0,
  FX_I64 = 1,
  FX_I32 = 2,
  FX_U8 = 3,   // uint8 and bool
  FX_F16 = 4,
  FX_BF16 = 5,
  // One 32-bit word of an int64 element, for programs that only move int64 data (select,
  // slice, index, where, compaction ...): such an output is lowered twice, once per word, and
  // is exact for every value.  FX_I64 itself stands for int64 data that takes part in 32-bit
  // integer arithmetic: its loads check that the value fits (a value that does not sets the
  // library's error word, fx_async_error) and its stores sign-extend; a load with FX_F_I2F
  // converts the whole 64-bit value.
  FX_I64LO = 6,
  FX_I64HI = 7,
};

// value classes inside the VM (32-bit registers)
enum FxVt : uint32_t { FX_VT_F = 0, FX_VT_I = 1 };

enum FxOp : uint32_t {
  FX_NOP = 0,
  // ---- register moves / loads (writes are predicated by the lane mask) ----
  FX_LDA,    // A = buf[a] at affine[b](coords); dt = storage dtype
  FX_LDB,    // B = ...
  FX_LDXA,   // A = buf[a] at element offset (int)A + imm
  FX_AFFA,   // A = (int) affine[b](coords)
  FX_AFFB,
  FX_IMMA,   // A = imm (raw 32 bits)
  FX_IMMB,
  FX_SCLA,   // A = scalar slot a (bit 30 set: per-task table)
  FX_SCLB,
  FX_STT,    // temp[a] = A
  FX_LDTA,   // A = temp[a]
  FX_LDTB,   // B = temp[a]
  FX_MOVBA,  // B = A
  FX_SWAP,   // A <-> B
  // ---- predication ----
  FX_MIF,    // push mask; mask &= (A != 0); if no lane of the wave is live jump to a
  FX_MELSE,  // mask = saved & ~mask; if no lane live jump to a
  FX_MMERGE, // A = live ? A : temp[a]; pop mask
  FX_MEND,   // pop mask (both sides wrote A with predicated moves)
  FX_MIFR,   // x = (int) affine[b](coords); A = (0 <= x < imm >> 8 && x % (imm & 255) == 0); then as MIF
  // ---- unary float (A = f(A)) ----
  FX_FNEG, FX_FABS, FX_EXP, FX_LOG, FX_SQRT, FX_RSQRT, FX_RCP, FX_SIGMOID,
  FX_TANH, FX_RELU, FX_FLOOR, FX_CEIL, FX_ROUND, FX_TRUNC, FX_SIN, FX_COS,
  FX_ERF, FX_LOG2, FX_EXP2, FX_EXPM1, FX_LOG1P,
  // ---- unary int / conversions ----
  FX_INEG, FX_LNOT, FX_INZ, FX_FNZ, FX_F2I, FX_I2F, FX_IABS,
  // ---- binary: A = A op X, X = B or imm (flags & FX_F_IMM).  With FX_F_MEMB / FX_F_TMPB the
  //      instruction first loads B like LDB (fields a, b, dt) / LDTB (field a) ----
  FX_FADD, FX_FSUB, FX_FRSUB, FX_FMUL, FX_FDIV, FX_FRDIV, FX_FMIN, FX_FMAX,
  FX_FPOW, FX_FMOD, FX_ATAN2,
  FX_IADD, FX_ISUB, FX_IRSUB, FX_IMUL, FX_IFDIV, FX_ITDIV, FX_IPMOD, FX_ITMOD,
  FX_IMIN, FX_IMAX, FX_IAND, FX_IOR, FX_IXOR,
  FX_FLT, FX_FLE, FX_FGT, FX_FGE, FX_FEQ, FX_FNE,
  FX_ILT, FX_ILE, FX_IGT, FX_IGE, FX_IEQ, FX_INE,
  // ---- misc ----
  FX_IRANGE, // A = (A >= a && A < b && (A - a) % imm == 0)
  FX_WHERE,  // A = temp[a] != 0 ? A : B
  // ---- serial reduction over an extra coordinate ----
  FX_RBEGIN, // push loop: counter = 0, extent = imm, acc slot = temp[a] preset by program
  FX_RNEXT,  // counter += 1; if counter < extent jump to a
  FX_RIDX,   // A = (int) loop counter of depth a
  // ---- reductions across the wave (row-per-wave mapping, FxOut::rowwave) ----
  FX_WMAX,   // A = max of A over every live element of the wave (NaN-propagating)
  FX_WSUM,   // A = sum of A over every live element of the wave
  FX_OP_COUNT
};

// instructions the batched "pure" interpreter implements (binary ones only with FX_F_IMM)
static inline bool fx_op_is_pure_unary(uint32_t op) {
  switch (op) {
    case FX_FNEG: case FX_FABS: case FX_EXP: case FX_SQRT: case FX_RSQRT: case FX_RCP: case FX_SIGMOID:
    case FX_RELU: case FX_F2I: case FX_I2F:
      return true;
    default: return false;
  }
}
static inline bool fx_op_is_pure_binary(uint32_t op) {
  switch (op) {
    case FX_FADD: case FX_FSUB: case FX_FRSUB: case FX_FMUL: case FX_FDIV: case FX_FMIN: case FX_FMAX:
    case FX_IADD: case FX_IMUL: case FX_FLT: case FX_FLE: case FX_FGT: case FX_FGE: case FX_FEQ: case FX_FNE:
      return true;
    default: return false;
  }
}

#define FX_F_IMM 1u  // binary op takes its second operand from imm
#define FX_F_I2F 2u  // LDA/LDB/AFFA/AFFB/SCLA/SCLB: convert the int result to float
#define FX_F_MEMB 4u // before the operation: B = buf[a] at affine[b](coords), dt = storage dtype (always set on LDB)
#define FX_F_TMPB 8u // before the operation: B = temp[a] (always set on LDTB)
static inline bool fx_op_is_binary(uint32_t op) { return op >= FX_FADD && op <= FX_INE; }

struct FxInsn {
  uint16_t op;
  uint8_t flags;
  uint8_t dt;
  int32_t a;
  int32_t b;
  uint32_t imm;
};

// element offset = base + tcoef * task + sum_k coef[k] * coord[k] + sum_d rcoef[d] * loop_counter[d]
#define FX_MAXLOOP 2
struct FxAffine {
  int32_t coef03[4];          // coefficients of root coordinates 0..3
  int32_t tcoef;
  int32_t base;
  int32_t rcoef[FX_MAXLOOP];
  int32_t coef45[2];          // coefficients of root coordinates 4, 5
  int32_t pad[2];
};
#define FX_AFF_WORDS 12
static inline int32_t fx_aff_coef(const struct FxAffine* a, int k) { return k < 4 ? a->coef03[k] : a->coef45[k - 4]; }
static inline void fx_aff_set_coef(struct FxAffine* a, int k, int32_t v) {
  if (k < 4) a->coef03[k] = v; else a->coef45[k - 4] = v;
}

// what a launcher needs to know about a lowered region besides the blob itself
struct FxLaunchInfo {
  uint32_t blob_words;  // multiple of 4
  uint32_t n_p;         // pointer slots in use
  uint32_t n_s;         // scalar slots in use
  uint32_t n_temps;     // LDS temp slots per lane
  uint32_t total_units; // dense kernel: number of FX_UNIT work units
  // streaming compaction (zero otherwise): see FxLaunch in fx_device.h
  uint32_t epoch, spin_limit, win_words;
  uint32_t s_tiles, s_rows, s_tile_rows, s_win_slot, s_win_stride;
  int32_t s_win_tcoef, s_win_lo;
  uint32_t s_win_span, n_sptr, n_tptr;
  uint32_t n_side;
  uint32_t side_slot[2], side_stride[2];
  int32_t side_tcoef[2], side_lo[2];
  uint32_t side_span[2], side_words[2];
  uint64_t wide;        // device address of the call's uploaded tables, or 0 (see FxLaunch)
};

#define FX_SLOT_TASK 0x40000000  // buffer/scalar slot lives in the per-task table

struct FxOut {
  uint32_t prog_begin, prog_end;  // instruction range, relative to the class base
  uint32_t rank;
  uint32_t numel;                 // dense: elements per task. compaction: rowlen * n_rows
  uint32_t dim[FX_MAXR];
  uint32_t magic[FX_MAXR];        // fast division by dim[k]
  uint32_t shift[FX_MAXR];
  uint32_t dtype;
  uint32_t ptr_slot;              // may carry FX_SLOT_TASK
  uint32_t task_stride;           // element offset added per task (shared output buffer)
  uint32_t block_begin;           // first block of this output inside one task
  uint32_t n_blocks;
  uint32_t rowlen;                // compaction: elements per row (numel / dim[0])
  uint32_t rl_magic, rl_shift;    // fast division by rowlen
  uint32_t vt;                    // FxVt of the program result
  uint32_t colmajor;              // compaction: iterate (column, row chunk) instead of flat elements
  uint32_t lead;                  // program starts with an unconditional affine load (batched by the kernels)
  uint32_t unit_items;            // dense: items per wave and work unit (1 or FX_K)
  uint32_t rowwave;               // dense: one item = one row of dim[rank-1] elements (needed by FX_WMAX/FX_WSUM)
  // A lane works on a group of FX_V consecutive elements along the last dimension
  // (coordinate vd); rows are padded to whole groups.
  uint32_t inner;                 // extent of the last dimension (1 for a scalar)
  uint32_t vd;                    // index of that dimension: max(rank, 1) - 1
  uint32_t gpr;                   // groups per run of `inner` elements: ceil(inner / FX_V)
  uint32_t gp_magic, gp_shift;    // fast division by gpr
  uint32_t gprow;                 // compaction: groups per kept row: rowlen / inner * gpr
  uint32_t gr_magic, gr_shift;    // fast division by gprow
  uint32_t n_groups;              // dense: groups per task: numel / inner * gpr
  uint32_t pure;                  // after the leading load only coordinate-free elementwise instructions with
                                  // immediate operands follow: FX_K items are interpreted as one batch
  uint32_t rowseg;                // rowwave: lanes per row (16, 32 or 64); a wave holds 64 / rowseg rows and
                                  // FX_WMAX / FX_WSUM reduce inside each segment of rowseg lanes
  uint32_t pad[2];
};


struct FxClass {
  uint32_t block_begin, block_end;  // grid range covered by this class (dense / scatter pass)
  uint32_t first_task;              // index into the task map
  uint32_t n_tasks;
  uint32_t blocks_per_task;
  uint32_t n_outs;
  uint32_t off_outs;                // word offset of FxOut[n_outs]
  uint32_t off_insn;                // word offset of FxInsn[]
  uint32_t off_aff;                 // word offset of FxAffine[]
  uint32_t n_temps;
  // row compaction (mode 1)
  uint32_t mask_begin, mask_end;    // mask program
  uint32_t n_rows;
  uint32_t n_rowtiles;              // ceil(n_rows / row_tile)
  uint32_t mask_vt;
  uint32_t cnt_block_begin, cnt_block_end;  // grid range in the count pass
  uint32_t cnt_blocks_per_task;
  uint32_t pad2[2];
};

enum FxMode : uint32_t { FX_MODE_DENSE = 0, FX_MODE_COMPACT = 1 };

struct FxHeader {
  uint32_t magic;
  uint32_t mode;
  uint32_t n_classes;
  uint32_t n_tasks;
  uint32_t n_sptr, n_tptr, n_sscal, n_tscal;
  uint32_t off_class;    // word offset of FxClass[n_classes]
  uint32_t off_taskmap;  // word offset of uint32 task ids grouped by class
  uint32_t row_tile;     // rows per compaction tile (<= FX_BLOCK)
  uint32_t max_rowtiles; // stride of the per-task tile-count table
  uint32_t slot_flags, slot_counts, slot_total;  // shared pointer slots used by compaction
  uint32_t total_words;
  uint32_t max_rows;     // stride of the per-task row-flag table
  uint32_t slot_err;     // 1 + shared pointer slot of the error word that FX_I64 loads report to (0: none)
  uint32_t slot_status;  // streaming compaction: shared pointer slot of the tile status words
  uint32_t pad[1];
};

// Dense regions with ONE task class of one or two outputs per task (the usual case) whose
// programs are compiled: the lean dense kernel (fx_dense_lean in fx_spec.h) takes what a
// workgroup needs in front of its first load from a short argument block, copied out of the
// descriptor at plan time, and stages the descriptor only if a program reads it.  A kernel start
// costs a trip to the argument segment per line of it that is read and per level of dependent
// reads, and about as much again per jump to code that has not been fetched yet, so the block is
// small, read in one go, and the kernel short; regions that do not fit take the general kernel.
#define FX_FAST_OUTS 2
#define FX_LEAN_P 24     // pointers and
#define FX_LEAN_S 16     // scalars of a region that the lean kernel's argument block holds
// One output of the region: the fields of FxOut that place a work item, the leading load's
// affine map, and the two buffers.  160 bytes, laid out so that a kernel for rank <= 3 reads the
// first 128 only; the records start at a multiple of 64 bytes in the argument segment.
struct FxLeanOut {
  uint64_t out_ptr;             // the output's buffer and the leading load's, resolved at launch when
  uint64_t lead_ptr;            // they do not change with the task (0: look the slot up in p[])
  uint32_t ptr_slot, lead_slot; // may carry FX_SLOT_TASK
  uint32_t lead;                // as FxOut::lead
  uint32_t block_begin, task_stride, unit_items, inner, vd, gpr, gp_magic, gp_shift, n_groups;   // as in FxOut
  int32_t lead_base, lead_tcoef;
  int32_t lead_cf[FX_MAXR];
  uint32_t rowseg;              // 0, or as FxOut::rowseg of an output whose items are whole rows (FxOut::rowwave); then
                                // n_groups holds the number of rows
  uint32_t dms[FX_MAXR - 1][3]; // FxOut::dim, magic, shift of dimensions 1 .. FX_MAXR - 1
};
struct FxLeanArgs {
  uint32_t blob_words, n_p, n_s, total_units;   // as in FxLaunchInfo
  uint32_t n_outs;              // 0: the region does not fit the lean kernel
  uint32_t bpt;                 // work units per task, and the division by it
  uint32_t bpt_magic, bpt_shift;
  uint32_t n_sptr, n_tptr;
  uint32_t cls_off;             // word offset of the class record in the descriptor
  uint32_t second_begin;        // first unit of a task that belongs to the second output
  uint64_t err_ptr;             // the error word of guarded loads (0: none), resolved at launch
  struct FxLeanOut out[FX_FAST_OUTS];
  uint64_t p[FX_LEAN_P];        // the first n_p words of FxDyn::p
  uint32_t s[FX_LEAN_S];        // the first n_s words of FxDyn::s
};
#ifdef __cplusplus
static_assert(sizeof(FxLeanOut) == 160 && offsetof(FxLeanArgs, out) == 56, "the records of FxLeanArgs start on a line of the argument segment (behind the 8-byte descriptor pointer)");
#endif

// dynamic (per call) arguments, passed by value in the kernarg segment
struct FxDyn {
  uint64_t p[FX_DYN_P];  // [shared ptrs][task 0 ptrs][task 1 ptrs]...
  uint32_t s[FX_DYN_S];  // [shared scalars][task 0 scalars]...
};

// fast unsigned division n / d for n < 2^31: q = (umulhi(n, magic) + n) >> shift
static inline void fx_fastdiv_make(uint32_t d, uint32_t* magic, uint32_t* shift) {
  uint32_t s = 0;
  while ((1ull << s) < d) ++s;
  uint64_t one = 1;
  uint64_t m = ((one << 32) * ((one << s) - d)) / d + 1;
  *magic = (uint32_t)m;
  *shift = s;
}
