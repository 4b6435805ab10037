// gfx950 kernels of the fused-region backend.
//
//   fx_region_dense   : one launch evaluates every output of a fused
//                       functionalized region for every ParallelMap task.
//   fx_compact_count  : pass 1 of row compaction (mask program -> row flags +
//                       per-tile keep counts, wave ballot + popcount).
//   fx_compact_scatter: pass 2 (per-tile exclusive offset, ballot/prefix row
//                       map in LDS, region programs evaluated only for kept
//                       rows, results written densely in source order).
//
// The kernels are templates (fx_device.h) over the way a program is run: this file
// instantiates them with the bytecode interpreter (fx_run); spec/*.hip instantiate them with
// the programs of one region as compile-time constants (fx_spec.h).  A workgroup first copies
// the whole region descriptor (programs, affine maps, output descriptors, task classes) and the
// per-call pointer / scalar tables of all tasks into LDS with one round of coalesced 128-bit
// loads; from then on every table access is an LDS broadcast read, so no dependent chain of
// cold global loads sits in front of the data traffic.  Instruction decode is wave-uniform
// (the opcode word goes through readfirstlane, the switch is a scalar branch); every
// instruction then operates on FX_V consecutive elements per lane along the last output
// dimension: a contiguous source is read with one 128-bit load per lane and results are written
// with one 128-bit store, so a global access of a wave covers 1 KB of contiguous memory.
//
// Replaces the NVRTC-generated kernels of the reference
// (fait/tensorexpr/cuda_codegen_tssa.cpp:881-1121, launch shape
// fait/fuser/graph_builder.cpp:463-499, per-task code cloning
// fait/tensorexpr/functor_parallization.cpp:93-108) and, for the
// data-dependent part, the ATen nonzero/index calls the reference leaves
// unfused (functs/csrc/jit/passes/convert_to_tensorssa.cpp:422-443).
#include <algorithm>
#include <cstring>
#include "fx_spec.h"

#include <mutex>
#include <unordered_map>

// --------------------------------------------------------------------------
// stand-alone order-preserving row compaction: out_c = col_c[mask] for up to
// 8 columns that share one byte mask.  Tiles of FX_BLOCK rows.
//   pass 1: per-tile keep counts (ballot + popcount)
//   pass 2 (only above FX_SCAN_DIRECT tiles): exclusive scan of the counts
//   pass 3: ballot/prefix row map in LDS, coalesced row copies
// --------------------------------------------------------------------------
// (up to here a tile sums the counts in front of it itself: 32 loads per lane at most, against a
// third launch whose one workgroup walks the counts 256 at a time)
#define FX_SCAN_DIRECT 8192
struct FxCols {
  const void* src[8];
  void* dst[8];
  int32_t words[8];   // 4-byte words per row (elsize 4/8) or bytes per row (elsize 1)
  int32_t bytes[8];   // 1 = byte column, 0 = word column
  int32_t vec[8];     // word column whose rows are whole 16-byte groups at 16-byte aligned addresses
  uint32_t magic[8], shift[8];   // division by the units of a row (groups when vec, else words / bytes)
  int32_t n;
};

__global__ __launch_bounds__(FX_BLOCK) void fx_rows_count(const uint8_t* __restrict__ mask, uint32_t n,
                                                          uint32_t* __restrict__ counts) {
  __shared__ uint32_t s_w[FX_BLOCK / 64];
  const uint32_t row = blockIdx.x * FX_BLOCK + threadIdx.x;
  const bool keep = row < n && mask[row] != 0;
  const uint64_t bal = __builtin_amdgcn_ballot_w64(keep);
  if ((threadIdx.x & 63u) == 0) s_w[threadIdx.x >> 6] = (uint32_t)__popcll(bal);
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t s = 0;
    for (int k = 0; k < FX_BLOCK / 64; ++k) s += s_w[k];
    counts[blockIdx.x] = s;
  }
}

// in-place exclusive scan of counts[0..t) by one workgroup; counts[t] = total
__global__ __launch_bounds__(FX_BLOCK) void fx_rows_scan(uint32_t* __restrict__ counts, uint32_t t) {
  __shared__ uint32_t s_w[FX_BLOCK / 64];
  __shared__ uint32_t s_carry;
  if (threadIdx.x == 0) s_carry = 0;
  __syncthreads();
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  for (uint32_t base = 0; base < t; base += FX_BLOCK) {
    const uint32_t i = base + threadIdx.x;
    const uint32_t v = i < t ? counts[i] : 0u;
    uint32_t x = v;  // inclusive wave scan
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      uint32_t y = __shfl_up(x, o, 64);
      if (lane >= (uint32_t)o) x += y;
    }
    if (lane == 63) s_w[wave] = x;
    __syncthreads();
    uint32_t woff = 0;
    for (uint32_t k = 0; k < wave; ++k) woff += s_w[k];
    const uint32_t carry = s_carry;
    if (i < t) counts[i] = carry + woff + x - v;
    __syncthreads();
    if (threadIdx.x == FX_BLOCK - 1) s_carry = carry + woff + x;
    __syncthreads();
  }
  if (threadIdx.x == 0) counts[t] = s_carry;
}

template <bool SCANNED>
__global__ __launch_bounds__(FX_BLOCK) void fx_rows_scatter(const uint8_t* __restrict__ mask, uint32_t n,
                                                            const uint32_t* __restrict__ counts, const FxCols cols,
                                                            uint32_t* __restrict__ total_host) {
  __shared__ uint32_t s_rowmap[FX_BLOCK];
  __shared__ uint32_t s_wsum[FX_BLOCK / 64];
  __shared__ uint32_t s_woff[FX_BLOCK / 64 + 1];
  __shared__ uint32_t s_prefix;
  const uint32_t tile = blockIdx.x;
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  uint32_t part = 0;
  if (!SCANNED) {
    for (uint32_t t = threadIdx.x; t < tile; t += FX_BLOCK) part += counts[t];
    part = fx_wave_sum(part, lane);
    if (lane == 0) s_wsum[wave] = part;
  }
  const uint32_t row = tile * FX_BLOCK + threadIdx.x;
  const bool keep = row < n && mask[row] != 0;
  const uint64_t bal = __builtin_amdgcn_ballot_w64(keep);
  const uint32_t before = (uint32_t)__popcll(bal & ((1ull << lane) - 1ull));
  if (lane == 0) s_woff[wave + 1] = (uint32_t)__popcll(bal);
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t p = 0;
    if (SCANNED) p = counts[tile];
    else for (int k = 0; k < FX_BLOCK / 64; ++k) p += s_wsum[k];
    s_prefix = p;
    uint32_t acc = 0;
    s_woff[0] = 0;
    for (int k = 1; k <= FX_BLOCK / 64; ++k) { acc += s_woff[k]; s_woff[k] = acc; }
  }
  __syncthreads();
  if (keep) s_rowmap[s_woff[wave] + before] = row;
  __syncthreads();
  const uint32_t n_kept = s_woff[FX_BLOCK / 64];
  const uint32_t prefix = s_prefix;
  // system scope: the caller may poll the word in host memory while the kernel runs
  if (tile + 1 == gridDim.x && threadIdx.x == 0)
    __hip_atomic_store(total_host, prefix + n_kept, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  if (n_kept == 0) return;
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    if (c >= cols.n) break;
    const uint32_t w = (uint32_t)cols.words[c];
    const uint32_t n_el = n_kept * w;
    const uint32_t magic = cols.magic[c], shift = cols.shift[c];
    if (cols.bytes[c]) {
      const FX_AS1 uint8_t* src = (const FX_AS1 uint8_t*)cols.src[c];
      FX_AS1 uint8_t* dst = (FX_AS1 uint8_t*)cols.dst[c] + (size_t)prefix * w;
      for (uint32_t e = threadIdx.x; e < n_el; e += FX_BLOCK) {
        const uint32_t r = fx_fastdiv(e, magic, shift), k = e - r * w;
        dst[e] = src[(size_t)s_rowmap[r] * w + k];
      }
    } else if (cols.vec[c]) {
      // a lane moves one 16-byte group; four groups per lane are in flight
      const uint32_t g = w >> 2, n_g = n_kept * g;
      const FX_AS1 fx_u32x4* src = (const FX_AS1 fx_u32x4*)cols.src[c];
      FX_AS1 fx_u32x4* dst = (FX_AS1 fx_u32x4*)cols.dst[c] + (size_t)prefix * g;
      for (uint32_t e0 = threadIdx.x; e0 < n_g; e0 += 4u * FX_BLOCK) {
        fx_u32x4 v[4];
#pragma unroll
        for (uint32_t u = 0; u < 4u; ++u) {
          const uint32_t e = e0 + u * FX_BLOCK;
          if (e < n_g) {
            const uint32_t r = fx_fastdiv(e, magic, shift), k = e - r * g;
            v[u] = src[(size_t)s_rowmap[r] * g + k];
          }
        }
#pragma unroll
        for (uint32_t u = 0; u < 4u; ++u) {
          const uint32_t e = e0 + u * FX_BLOCK;
          if (e < n_g) dst[e] = v[u];
        }
      }
    } else if (w == 1u) {
      const FX_AS1 uint32_t* src = (const FX_AS1 uint32_t*)cols.src[c];
      FX_AS1 uint32_t* dst = (FX_AS1 uint32_t*)cols.dst[c] + (size_t)prefix;
      for (uint32_t e = threadIdx.x; e < n_kept; e += FX_BLOCK) dst[e] = src[s_rowmap[e]];
    } else {
      const FX_AS1 uint32_t* src = (const FX_AS1 uint32_t*)cols.src[c];
      FX_AS1 uint32_t* dst = (FX_AS1 uint32_t*)cols.dst[c] + (size_t)prefix * w;
      for (uint32_t e = threadIdx.x; e < n_el; e += FX_BLOCK) {
        const uint32_t r = fx_fastdiv(e, magic, shift), k = e - r * w;
        dst[e] = src[(size_t)s_rowmap[r] * w + k];
      }
    }
  }
}

// --------------------------------------------------------------------------
// plain copy kernel of known size: calibration of the HBM counters and the
// bandwidth ceiling a kernel of this launch shape can reach.
// --------------------------------------------------------------------------
__global__ __launch_bounds__(FX_BLOCK) void fx_copy_f4(const float4* __restrict__ src, float4* __restrict__ dst, size_t n4) {
  size_t i = (size_t)blockIdx.x * FX_BLOCK + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * FX_BLOCK;
  for (; i < n4; i += stride) dst[i] = src[i];
}

// --------------------------------------------------------------------------
// host-callable launchers (C++ linkage inside the library; the C ABI is in
// fx_api.cpp)
// --------------------------------------------------------------------------
// Specialised kernels register themselves from static initialisers of their translation
// units (spec/*.hip), before any plan is made.
static std::unordered_map<uint64_t, FxSpecKernels>& spec_table() {
  static std::unordered_map<uint64_t, FxSpecKernels> t;
  return t;
}
static std::mutex& spec_mutex() {
  static std::mutex m;
  return m;
}
void fx_spec_register(uint64_t hash, const FxSpecKernels& k) {
  std::lock_guard<std::mutex> g(spec_mutex());
  spec_table()[hash] = k;
}
const FxSpecKernels* fx_spec_find(uint64_t hash) {
  std::lock_guard<std::mutex> g(spec_mutex());
  auto it = spec_table().find(hash);
  return it == spec_table().end() ? nullptr : &it->second;   // entries are never erased
}
bool fx_spec_has_stream(const FxSpecKernels* spec) { return spec && spec->stream != nullptr; }
bool fx_spec_has_lean(const FxSpecKernels* spec) { return spec && spec->lean != nullptr; }
int fx_spec_count() {
  std::lock_guard<std::mutex> g(spec_mutex());
  return (int)spec_table().size();
}

// a specialised kernel takes the arguments of the generic one
static hipError_t launch_spec(const void* fn, const uint32_t* sb, const FxLaunch& la, const FxDyn* dyn, uint32_t grid,
                              uint32_t lds, hipStream_t stream, uint32_t threads = FX_BLOCK) {
  void* args[3] = {(void*)&sb, (void*)&la, (void*)dyn};
  return hipLaunchKernel(fn, dim3(grid), dim3(threads), args, lds, stream);
}

// The tables of a call that the kernel argument block cannot hold (a map of many tasks) travel
// to device memory in pieces: each launch carries one piece by value and stores it.  In stream
// order like the kernels that read the tables, nothing for the host to keep alive, and a
// captured graph replays it.
__global__ __launch_bounds__(FX_BLOCK) void fx_store_words(const FxDyn piece, uint64_t* dst, uint32_t n_words) {
  (void)piece;   // read through the argument segment: indexing a by-value aggregate would copy it to per-lane memory
  const uint64_t* src = (const uint64_t*)((const uint8_t*)__builtin_amdgcn_kernarg_segment_ptr());
  for (uint32_t i = threadIdx.x; i < n_words; i += FX_BLOCK) dst[i] = src[i];
}
hipError_t fx_upload_words(const uint64_t* words, size_t n_words, void* dst, hipStream_t stream) {
  static_assert(sizeof(FxDyn) % 8 == 0, "pieces are whole 8-byte words");
  const size_t per = sizeof(FxDyn) / 8;
  FxDyn piece;
  memset(&piece, 0, sizeof piece);
  for (size_t at = 0; at < n_words; at += per) {
    const uint32_t n = (uint32_t)std::min(per, n_words - at);
    memcpy(&piece, words + at, (size_t)n * 8);
    uint64_t* d = (uint64_t*)dst + at;
    void* args[3] = {(void*)&piece, (void*)&d, (void*)&n};
    const hipError_t e = hipLaunchKernel((const void*)&fx_store_words, dim3(1), dim3(FX_BLOCK), args, 0, stream);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

static FxLaunch make_launch(const FxLaunchInfo& li) {
  FxLaunch la;
  la.wide = li.wide;
  la.blob_words = li.blob_words;
  la.n_p = li.n_p;
  la.n_s = li.n_s;
  la.temps_off = (li.blob_words + 2 * li.n_p + li.n_s + 3u) & ~3u;
  la.total_units = li.total_units;
  la.epoch = li.epoch;
  la.win_off = la.temps_off;   // compiled kernels; the interpreter's launcher moves it behind the temporaries
  la.spin_limit = li.spin_limit;
  la.s_tiles = li.s_tiles;
  la.s_rows = li.s_rows;
  la.s_tile_rows = li.s_tile_rows;
  la.s_win_slot = li.s_win_slot;
  la.s_win_stride = li.s_win_stride;
  la.s_win_tcoef = li.s_win_tcoef;
  la.s_win_lo = li.s_win_lo;
  la.s_win_span = li.s_win_span;
  la.n_sptr = li.n_sptr;
  la.n_tptr = li.n_tptr;
  la.win_buf = li.win_words;
  la.n_side = li.n_side;
  uint32_t off = la.win_off + li.win_words;
  for (int i = 0; i < FX_SIDE_WIN; ++i) {
    la.side_slot[i] = li.side_slot[i];
    la.side_stride[i] = li.side_stride[i];
    la.side_tcoef[i] = li.side_tcoef[i];
    la.side_lo[i] = li.side_lo[i];
    la.side_span[i] = li.side_span[i];
    la.side_off[i] = off;
    off += li.side_words[i];
  }
  return la;
}

uint32_t fx_lds_bytes(const FxLaunchInfo& li) {
  FxLaunch la = make_launch(li);
  return (la.temps_off + li.n_temps * FX_V * FX_BLOCK) * 4u;
}
// compiled kernels keep their temporaries in registers
static uint32_t lds_bytes_compiled(const FxLaunchInfo& li) { return make_launch(li).temps_off * 4u; }

// A workgroup may take all 160 KB of a CU's LDS on this device; more than the default 64 KB has
// to be granted per kernel (and device) before the launch.  The interpreter's temporaries (4 KB
// each per workgroup) are what needs it.
template <class K>
static hipError_t allow_lds(K kernel, uint32_t bytes) {
  if (bytes <= 64u * 1024u) return hipSuccess;
  static std::mutex mu;
  static std::unordered_map<uint64_t, uint32_t> granted;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t key = ((uint64_t)(uintptr_t)(const void*)kernel << 6) ^ (uint64_t)dev;
  std::lock_guard<std::mutex> g(mu);
  uint32_t& have = granted[key];
  if (have >= bytes) return hipSuccess;
  e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e == hipSuccess) have = bytes;
  return e;
}
#define FX_LAUNCH_LDS(kernel, grid, lds, stream, ...)          \
  do {                                                         \
    const hipError_t e__ = allow_lds(&kernel, lds);            \
    if (e__ != hipSuccess) return e__;                         \
    kernel<<<grid, FX_BLOCK, lds, stream>>>(__VA_ARGS__);      \
  } while (0)

hipError_t fx_launch_dense(int rank, const uint32_t* sb, const FxLaunchInfo& li, const FxDyn* dyn, uint32_t grid,
                           hipStream_t stream, const FxSpecKernels* spec, const FxLeanArgs* lean, uint32_t slot_err) {
  if (grid == 0) return hipSuccess;
  if (spec && spec->lean && lean && lean->n_outs != 0) {
    // the lean kernel: a short argument block instead of FxLaunch + FxDyn
    FxLeanArgs a = *lean;
    a.err_ptr = slot_err ? dyn->p[slot_err - 1u] : 0;
    for (uint32_t o = 0; o < a.n_outs; ++o) {
      FxLeanOut& lo = a.out[o];
      lo.out_ptr = (lo.ptr_slot & FX_SLOT_TASK) ? 0 : dyn->p[lo.ptr_slot & 0xffffu];
      lo.lead_ptr = (!lo.lead || (lo.lead_slot & FX_SLOT_TASK)) ? 0 : dyn->p[lo.lead_slot & 0xffffu];
    }
    memcpy(a.p, dyn->p, sizeof(uint64_t) * a.n_p);
    memcpy(a.s, dyn->s, sizeof(uint32_t) * a.n_s);
    void* args[2] = {(void*)&sb, (void*)&a};
    return hipLaunchKernel(spec->lean, dim3(grid), dim3(FX_BLOCK), args, spec->lean_stages ? lds_bytes_compiled(li) : 0u,
                           stream);
  }
  const FxLaunch la = make_launch(li);
  const uint32_t lds = fx_lds_bytes(li);
  if (spec && spec->dense) return launch_spec(spec->dense, sb, la, dyn, grid, lds_bytes_compiled(li), stream);
  switch (rank) {
    case 0:
    case 1: FX_LAUNCH_LDS(fx_region_dense<1>, grid, lds, stream, sb, la, *dyn); break;
    case 2: FX_LAUNCH_LDS(fx_region_dense<2>, grid, lds, stream, sb, la, *dyn); break;
    case 3: FX_LAUNCH_LDS(fx_region_dense<3>, grid, lds, stream, sb, la, *dyn); break;
    case 4: FX_LAUNCH_LDS(fx_region_dense<4>, grid, lds, stream, sb, la, *dyn); break;
    default: FX_LAUNCH_LDS(fx_region_dense<FX_MAXR>, grid, lds, stream, sb, la, *dyn); break;
  }
  return hipGetLastError();
}

hipError_t fx_launch_compact_count(const uint32_t* sb, const FxLaunchInfo& li, const FxDyn* dyn, uint32_t grid,
                                   hipStream_t stream, const FxSpecKernels* spec) {
  if (grid == 0) return hipSuccess;
  if (spec && spec->count) return launch_spec(spec->count, sb, make_launch(li), dyn, grid, lds_bytes_compiled(li), stream);
  FX_LAUNCH_LDS(fx_compact_count<FxInterp>, grid, fx_lds_bytes(li), stream, sb, make_launch(li), *dyn);
  return hipGetLastError();
}

hipError_t fx_launch_compact_scatter(int rank, const uint32_t* sb, const FxLaunchInfo& li, const FxDyn* dyn,
                                     uint32_t grid, hipStream_t stream, const FxSpecKernels* spec) {
  if (grid == 0) return hipSuccess;
  const FxLaunch la = make_launch(li);
  const uint32_t lds = fx_lds_bytes(li);
  if (spec && spec->scatter)
    return launch_spec(spec->scatter, sb, la, dyn, grid, lds_bytes_compiled(li), stream, spec->scatter_threads);
  switch (rank) {
    case 0:
    case 1: FX_LAUNCH_LDS(fx_compact_scatter<1>, grid, lds, stream, sb, la, *dyn); break;
    case 2: FX_LAUNCH_LDS(fx_compact_scatter<2>, grid, lds, stream, sb, la, *dyn); break;
    case 3: FX_LAUNCH_LDS(fx_compact_scatter<3>, grid, lds, stream, sb, la, *dyn); break;
    case 4: FX_LAUNCH_LDS(fx_compact_scatter<4>, grid, lds, stream, sb, la, *dyn); break;
    default: FX_LAUNCH_LDS(fx_compact_scatter<FX_MAXR>, grid, lds, stream, sb, la, *dyn); break;
  }
  return hipGetLastError();
}

// LDS a streaming launch needs: descriptor and tables, the interpreter's temporaries, the window
uint32_t fx_stream_lds_bytes(const FxLaunchInfo& li, bool compiled) {
  const FxLaunch la = make_launch(li);
  const uint32_t temps = compiled ? 0u : li.n_temps * FX_V * FX_BLOCK;
  return (la.temps_off + temps + li.win_words + li.side_words[0] + li.side_words[1]) * 4u;
}

hipError_t fx_launch_compact_stream(int rank, const uint32_t* sb, const FxLaunchInfo& li, const FxDyn* dyn, uint32_t grid,
                                    hipStream_t stream, const FxSpecKernels* spec) {
  if (grid == 0) return hipSuccess;
  FxLaunch la = make_launch(li);
  if (spec && spec->stream) return launch_spec(spec->stream, sb, la, dyn, grid, fx_stream_lds_bytes(li, true), stream);
  {
    // the interpreter's temporaries sit between the tables and the windows
    const uint32_t shift = li.n_temps * FX_V * FX_BLOCK;
    la.win_off += shift;
    for (int i = 0; i < FX_SIDE_WIN; ++i) la.side_off[i] += shift;
  }
  const uint32_t lds = fx_stream_lds_bytes(li, false);
  switch (rank) {
    case 0:
    case 1: fx_compact_stream<1><<<grid, FX_BLOCK, lds, stream>>>(sb, la, *dyn); break;
    case 2: fx_compact_stream<2><<<grid, FX_BLOCK, lds, stream>>>(sb, la, *dyn); break;
    case 3: fx_compact_stream<3><<<grid, FX_BLOCK, lds, stream>>>(sb, la, *dyn); break;
    case 4: fx_compact_stream<4><<<grid, FX_BLOCK, lds, stream>>>(sb, la, *dyn); break;
    default: fx_compact_stream<FX_MAXR><<<grid, FX_BLOCK, lds, stream>>>(sb, la, *dyn); break;
  }
  return hipGetLastError();
}

hipError_t fx_launch_compact_rows(const uint8_t* mask, int64_t n, const void* const* cols, void* const* outs,
                                  const int32_t* rowlen, const int32_t* elsize, int n_cols, uint32_t* counts,
                                  uint32_t* total_host, hipStream_t stream) {
  FxCols c;
  for (int i = 0; i < 8; ++i) {
    c.src[i] = nullptr; c.dst[i] = nullptr; c.words[i] = 0; c.bytes[i] = 0; c.vec[i] = 0; c.magic[i] = 0; c.shift[i] = 0;
  }
  c.n = n_cols;
  for (int i = 0; i < n_cols; ++i) {
    c.src[i] = cols[i];
    c.dst[i] = outs[i];
    c.bytes[i] = elsize[i] == 1 ? 1 : 0;
    c.words[i] = elsize[i] == 1 ? rowlen[i] : rowlen[i] * (elsize[i] / 4);
    c.vec[i] = !c.bytes[i] && c.words[i] >= 4 && (c.words[i] & 3) == 0 && (((uintptr_t)cols[i] | (uintptr_t)outs[i]) & 15u) == 0;
    fx_fastdiv_make((uint32_t)std::max(c.vec[i] ? c.words[i] / 4 : c.words[i], 1), &c.magic[i], &c.shift[i]);
  }
  const uint32_t tiles = (uint32_t)((n + FX_BLOCK - 1) / FX_BLOCK);
  fx_rows_count<<<tiles, FX_BLOCK, 0, stream>>>(mask, (uint32_t)n, counts);
  if (tiles > FX_SCAN_DIRECT) {
    fx_rows_scan<<<1, FX_BLOCK, 0, stream>>>(counts, tiles);
    fx_rows_scatter<true><<<tiles, FX_BLOCK, 0, stream>>>(mask, (uint32_t)n, counts, c, total_host);
  } else {
    fx_rows_scatter<false><<<tiles, FX_BLOCK, 0, stream>>>(mask, (uint32_t)n, counts, c, total_host);
  }
  return hipGetLastError();
}

// --------------------------------------------------------------------------
// Tile counts of fx_compact_rows_static: device memory that exists from the moment the code
// object is loaded, so the call allocates nothing.  One copy per GPU, at its own address;
// every call on a GPU shares it.  Nothing in it has to start at zero: fx_rows_count writes
// the count of every tile of the call and fx_rows_scan the word behind them before anything
// reads them.
// --------------------------------------------------------------------------
#define FX_STATIC_SCRATCH_WORDS (FX_STATIC_MAX_ROWS / FX_BLOCK + 2)
static __device__ __align__(256) uint32_t fx_static_scratch[FX_STATIC_SCRATCH_WORDS];

#define FX_STATIC_MAX_DEVICES 64
static std::mutex g_static_mu;
static uint32_t* g_static_ptr[FX_STATIC_MAX_DEVICES];  // device address of the array, per GPU

// The array's name is a host-side handle, not a device address: the address on the current
// device is looked up once and kept.
static hipError_t static_scratch(uint32_t** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= FX_STATIC_MAX_DEVICES) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> g(g_static_mu);
  if (!g_static_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(fx_static_scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_static_ptr[dev] = (uint32_t*)p;
  }
  *out = g_static_ptr[dev];
  return hipSuccess;
}

hipError_t fx_launch_compact_rows_static(const uint8_t* mask, int64_t n, const void* const* cols, void* const* outs,
                                         const int32_t* rowlen, const int32_t* elsize, int n_cols,
                                         uint32_t* total_host, hipStream_t stream) {
  uint32_t* counts = nullptr;
  hipError_t e = static_scratch(&counts);
  if (e != hipSuccess) return e;
  return fx_launch_compact_rows(mask, n, cols, outs, rowlen, elsize, n_cols, counts, total_host, stream);
}

hipError_t fx_launch_copy(const void* src, void* dst, size_t bytes, uint32_t grid, hipStream_t stream) {
  fx_copy_f4<<<grid, FX_BLOCK, 0, stream>>>((const float4*)src, (float4*)dst, bytes / 16);
  return hipGetLastError();
}


