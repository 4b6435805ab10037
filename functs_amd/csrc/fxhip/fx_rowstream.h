// Skeleton of the generated row-stream kernels (fx_rs.h): a row compaction in ONE launch.
//
// A workgroup owns a CHUNK: a run of up to 256 consecutive rows of one task.  The host sizes
// the chunks so that all workgroups of the launch are resident together whenever the input
// allows it.
//   1. Wave 0 evaluates the mask of every row of the chunk from memory (the few words a row's
//      mask needs, gathered before anything else) and publishes the chunk's kept-row count in a
//      status word tagged with the call's epoch.
//   2. Meanwhile all waves ask for the rows of the first sub-tile of the window input (up to 64
//      rows: one contiguous run of memory, coalesced 128-bit loads; the lines travel in
//      registers and are parked in an LDS window; the next sub-tile is requested as soon as the
//      current one is parked).
//   3. One look-back per workgroup (wave 1): the write offset of the chunk is the sum of the
//      counts of the earlier chunks of its task, read from their status words as they appear.
//      Earlier chunks never wait for later ones, and every poll loop is bounded: when a word does
//      not show up within spin_limit polls the workgroup counts the kept rows in front of its
//      chunk itself, from memory, so the kernel ends whatever the order in which workgroups are
//      started.
//   4. Per sub-tile: row map from the kept flags (ballot + popcount), then the generated code:
//      P::row once per kept row (one lane each: every column that needs code of its own), and
//      per vector segment four columns per lane (V::elem), written to the compacted rows.  Rows
//      are loaded and results stored as streaming (non-temporal) accesses.
// P is the policy class a generated translation unit defines (fx_rs_gen.cpp).
// Status words belong to the library (one per chunk, zero when allocated, never reset: a word
// of an earlier call carries an older epoch).
//
// This replaces the launch of generated CUDA of the reference for such a subgraph
// (fait/tensorexpr/cuda_codegen_tssa.cpp:1167-1306) and the ATen kernels it leaves x[mask] to
// (functs/csrc/jit/passes/convert_to_tensorssa.cpp:422-443).
#pragma once
#include <hip/hip_runtime.h>

#include "fx_device.h"
#include "fx_rs.h"

#define FX_RS_FN __device__ __forceinline__

namespace {

typedef uint32_t fx_u32x2_a4 __attribute__((ext_vector_type(2), aligned(4)));   // 64 bits, 4-byte aligned

FX_RS_FN float rs_sigmoid(float x) { return fx_sigmoid(x); }
FX_RS_FN float rs_exp(float x) { return fx_exp(x); }
FX_RS_FN float rs_tanh(float x) { return fx_tanh(x); }

// Run-time side of generated code: pointers, per-task offsets, constants.
struct FxRsRt {
  const FxRsLaunch& la;
  uint32_t task;
  uint32_t* stg[FX_RS_MAX_OUT];   // LDS: where a staged output's kept rows of the sub-tile are put together
  uint32_t ph[FX_RS_MAX_OUT];     // and the phase of the run in memory (first element's index mod 4)
  // the call's tables: the FxDyn block behind the launch block in the argument segment, or (the
  // build for maps of many tasks) where the launch block says they were uploaded
  bool wide;
  FX_RS_FN const uint32_t* staged(int k) const { return stg[k]; }
  FX_RS_FN uint64_t ptr(uint32_t slot) const {
    const uint8_t* ka = (const uint8_t*)__builtin_amdgcn_kernarg_segment_ptr();
    const uint64_t* gp = wide ? (const uint64_t*)la.wide : (const uint64_t*)(ka + sizeof(FxRsLaunch));
    const uint32_t pi = (slot & FX_SLOT_TASK) ? la.n_sptr + task * la.n_tptr + (slot & 0xffffu) : (slot & 0xffffu);
    return gp[pi];
  }
  FX_RS_FN uint32_t scal(int32_t slot) const {
    const uint8_t* ka = (const uint8_t*)__builtin_amdgcn_kernarg_segment_ptr();
    const uint32_t* gs = wide ? (const uint32_t*)((const uint64_t*)la.wide + la.n_sptr + la.n_tasks * la.n_tptr)
                              : (const uint32_t*)(ka + sizeof(FxRsLaunch) + offsetof(FxDyn, s));
    const uint32_t si = ((uint32_t)slot & FX_SLOT_TASK) ? la.n_sscal + task * la.n_tscal + ((uint32_t)slot & 0xffffu) : ((uint32_t)slot & 0xffffu);
    return gs[si];
  }
  FX_RS_FN uint32_t fimm(int k) const { return la.fimm[k]; }
  // input k of this task: base address, and the element offset of the task inside it
  FX_RS_FN uint64_t in(int k) const { return ptr(la.in_slot[k]); }
  FX_RS_FN uint32_t toff(int k) const { return (uint32_t)(la.in_tcoef[k] * (int32_t)task); }
  FX_RS_FN uint64_t out(int k) const { return ptr(la.out_slot[k]); }
  FX_RS_FN uint32_t ooff(int k) const { return la.out_tstride[k] * task; }
  FX_RS_FN uint64_t err() const { return la.slot_err ? ptr(la.slot_err - 1u) : 0ull; }
};

template <int CVT>
FX_RS_FN uint32_t rs_scal(const FxRsRt& rt, int32_t slot) {
  const uint32_t s = rt.scal(slot);
  return CVT ? f2u((float)(int32_t)s) : s;
}

// element `off` (+ the task's offset) of input k, as the region's loads read it (fx_load_vec)
template <uint32_t DT, int CVT>
FX_RS_FN uint32_t rs_ldx_at(const FxRsRt& rt, int k, uint32_t o) {
  const FX_AS1 uint8_t* base = (const FX_AS1 uint8_t*)rt.in(k);
  uint32_t v;
  if constexpr (DT == FX_F32 || DT == FX_I32) {
    v = *(const FX_AS1 uint32_t*)(base + (o << 2));
  } else if constexpr (DT == FX_I64) {
    const uint64_t w = *(const FX_AS1 uint64_t*)(base + (o << 3));
    if constexpr (CVT != 0) return f2u((float)(int64_t)w);
    v = (uint32_t)w;
    if ((int64_t)w != (int64_t)(int32_t)(uint32_t)w) {
      const uint64_t e = rt.err();
      if (e) __hip_atomic_store((uint32_t*)e, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  } else if constexpr (DT == FX_I64LO) {
    v = *(const FX_AS1 uint32_t*)(base + (o << 3));
  } else if constexpr (DT == FX_I64HI) {
    v = *(const FX_AS1 uint32_t*)(base + (o << 3) + 4u);
  } else if constexpr (DT == FX_U8) {
    v = base[o];
  } else if constexpr (DT == FX_F16) {
    v = f2u(__half2float(__ushort_as_half(*(const FX_AS1 uint16_t*)(base + (o << 1)))));
  } else {
    v = (uint32_t)(*(const FX_AS1 uint16_t*)(base + (o << 1))) << 16;
  }
  if constexpr (CVT != 0) v = f2u((float)(int32_t)v);
  return v;
}
template <uint32_t DT, int CVT>
FX_RS_FN uint32_t rs_ld(const FxRsRt& rt, int k, uint32_t off) {
  return rs_ldx_at<DT, CVT>(rt, k, off + rt.toff(k));
}
// a load through a computed index (FX_LDXA): no per-task offset
template <uint32_t DT>
FX_RS_FN uint32_t rs_ldx(const FxRsRt& rt, int k, uint32_t off) {
  return rs_ldx_at<DT, 0>(rt, k, off);
}
FX_RS_FN void rs_ld2(const FxRsRt& rt, int k, uint32_t off, uint32_t& a, uint32_t& b) {
  const FX_AS1 uint8_t* base = (const FX_AS1 uint8_t*)rt.in(k);
  const fx_u32x2_a4 v = *(const FX_AS1 fx_u32x2_a4*)(base + ((off + rt.toff(k)) << 2));
  a = v.x; b = v.y;
}
FX_RS_FN void rs_ld4(const FxRsRt& rt, int k, uint32_t off, uint32_t& a, uint32_t& b, uint32_t& c, uint32_t& d) {
  const FX_AS1 uint8_t* base = (const FX_AS1 uint8_t*)rt.in(k);
  const fx_u32x4_a4 v = *(const FX_AS1 fx_u32x4_a4*)(base + ((off + rt.toff(k)) << 2));
  a = v.x; b = v.y; c = v.z; d = v.w;
}
template <uint32_t DT, uint32_t VT>
FX_RS_FN void rs_st(const FxRsRt& rt, int k, uint32_t off, uint32_t v) {
  const uint32_t o = off + rt.ooff(k);
  if constexpr ((DT == FX_F32 && VT == FX_VT_F) || (DT == FX_I32 && VT == FX_VT_I))
    __builtin_nontemporal_store(v, (FX_AS1 uint32_t*)((FX_AS1 uint8_t*)rt.out(k) + (o << 2)));
  else
    fx_store(rt.out(k), o, DT, VT, v);
}
FX_RS_FN void rs_st4(const FxRsRt& rt, int k, uint32_t off, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  fx_u32x4 v;
  v.x = a; v.y = b; v.z = c; v.w = d;
  __builtin_nontemporal_store(v, (FX_AS1 fx_u32x4_a4*)((FX_AS1 uint8_t*)rt.out(k) + ((off + rt.ooff(k)) << 2)));
}
// staged outputs (plain 32-bit elements): into LDS, and from there to element `e` of the output
// buffer (the task's offset included; e a multiple of four for the group)
FX_RS_FN void rs_stl(const FxRsRt& rt, int k, uint32_t off, uint32_t v) { rt.stg[k][rt.ph[k] + off] = v; }
FX_RS_FN void rs_st_at(const FxRsRt& rt, int k, uint32_t e, uint32_t v) {
  __builtin_nontemporal_store(v, (FX_AS1 uint32_t*)((FX_AS1 uint8_t*)rt.out(k) + (e << 2)));
}
FX_RS_FN void rs_st4_at(const FxRsRt& rt, int k, uint32_t e, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  fx_u32x4 v;
  v.x = a; v.y = b; v.z = c; v.w = d;
  __builtin_nontemporal_store(v, (FX_AS1 fx_u32x4*)((FX_AS1 uint8_t*)rt.out(k) + (e << 2)));
}

}  // namespace
#include "fx_rs_ops.h"
namespace {

// (WIDE, the build that reads the call's tables from device memory, is compiled for one workgroup
// per CU less: at the others' occupancy it spills, 194 against 182 us for the head on 128 images)
template <class P, uint32_t KV, bool PERSIST, bool WIDE = false>
__global__ __launch_bounds__(FX_BLOCK, (WIDE ? FX_RS_OCC - 1u : FX_RS_OCC)) void fx_rs_kernel(const FxRsLaunch la, const FxDyn) {
  constexpr uint32_t NT = FX_BLOCK, NW = NT / 64u, NSUB = FX_RS_NSUB, S = P::S;
  extern __shared__ __attribute__((aligned(16))) uint32_t L[];   // the window: sub_rows rows of S elements
  __shared__ uint32_t s_rowmap[FX_RS_SUB];
  __shared__ uint8_t s_keep[FX_BLOCK];
  __shared__ uint32_t s_wsum[NW];
  __shared__ uint32_t s_prefix, s_ok, s_nk, s_total, s_told;
  const uint32_t lane = threadIdx.x & 63u, wave = uni(threadIdx.x >> 6);
  // A launch that fits the device has a workgroup per chunk.  PERSIST: a launch with more chunks
  // than the device holds workgroups has as many workgroups as it holds, and workgroup w takes
  // the chunks w, w + gridDim.x, ... in that order (chunks are numbered task by task).  A chunk
  // waits for chunks with smaller numbers only, and those are in the hands of workgroups that are
  // running: no chunk waits for one that has not been started.  (A build of its own: the loop
  // costs registers, which the launches that fit do not pay.)
  const uint32_t n_chunks_all = la.chunks * la.n_tasks;
  for (uint32_t b = blockIdx.x;;) {
    const uint32_t task = fx_fastdiv(b, la.chunks_magic, la.chunks_shift), chunk = b - task * la.chunks;
    const uint32_t c_r0 = chunk * la.chunk_rows;
    // rows of the chunk (>= 1) and its sub-tiles of equal size, at most la.sub_rows rows each: the
    // host has divided (fx_rs_finish_geometry)
    const bool last_chunk = chunk + 1u == la.chunks;
    const uint32_t c_rows = last_chunk ? la.rows_last : la.chunk_rows;
    const uint32_t sub_rows = last_chunk ? la.sub_rows_last : la.sub_rows_whole;
    const uint32_t n_sub = last_chunk ? la.n_sub_last : la.n_sub_whole;
    FxRsRt rt{la, task, {}, {}, WIDE};
    // What the rows' own code reads from memory besides the window (a few words per row: anchors,
    // strides ...) is fetched for all rows of the chunk before the first sub-tile, into a table in LDS.
    const bool SIDE_LDS = P::n_row_cols != 0u && P::n_side != 0u && P::n_side <= FX_RS_MAX_SIDE && la.side_lds != 0u;
    uint32_t* side = nullptr;
    {
      // staged outputs behind the window, each sub_rows rows and a group of slack
      uint32_t* sp = L + ((((la.sub_rows * S + 3u + 3u) >> 2) + 1u) << 2);
  #pragma unroll
      for (uint32_t k = 0; k < FX_RS_MAX_OUT; ++k) {
        rt.stg[k] = sp;
        rt.ph[k] = 0u;
        if (k < P::n_out && P::stage_rowlen[k] != 0u) sp += la.sub_rows * P::stage_rowlen[k] + 8u;
      }
      side = sp;   // la.chunk_rows rows of P::n_side words
    }
    // element 0 of this task's rows of the window input
    const FX_AS1 uint32_t* win = (const FX_AS1 uint32_t*)rt.in(0) + (int64_t)la.in_tcoef[0] * task;

    fx_u32x4 wr[KV];
    uint32_t shift = 0, n_vec = 0;
    auto request = [&](uint32_t s) {
      const uint32_t r0 = c_r0 + s * sub_rows, rows = min(sub_rows, c_rows - s * sub_rows);
      const uint64_t a0 = (uint64_t)(win + (size_t)r0 * S);
      shift = ((uint32_t)a0 & 15u) >> 2;   // elements between the 16-byte line and the first row
      const FX_AS1 fx_u32x4* g4 = (const FX_AS1 fx_u32x4*)(a0 & ~(uint64_t)15);
      n_vec = (shift + rows * S + 3u) >> 2;   // <= KV * NT (host)
      // every line is used once; lanes past the end ask for the last line again rather than branch,
      // so that the requests leave back to back; a load of which no lane of the wave has a part is
      // left out (a branch on a value that all lanes share)
      const uint32_t n_vec_u = uni(n_vec);
  #pragma unroll
      for (uint32_t k = 0; k < KV; ++k)
        if (k * NT + wave * 64u < n_vec_u) wr[k] = __builtin_nontemporal_load(&g4[min(threadIdx.x + k * NT, n_vec - 1u)]);
    };
    const bool teller = chunk + 1u == la.chunks && la.late_tell == 0u;   // the task's last chunk tells the host the task's total
    uint32_t pw[2] = {0, 0};   // wave 1: what its first look at the earlier chunks found
    // One look-back per workgroup (wave 1): the sum of the counts of the earlier chunks of the task.
    auto look_back = [&]() {
      const uint32_t first = b - chunk;
      // A lane watches the words of chunks lane, lane + 64, ..., four at a time: what is still
      // missing of the four is asked for again in one go, so a round of polls costs one trip
      // however many of the words a lane has.
      constexpr uint32_t NG = 4u;
      uint32_t part = 0;
      bool ok = true;
      for (uint32_t base = 0; base < chunk && ok; base += NG * 64u) {
        uint32_t wv[NG], polls = 0;
  #pragma unroll
        for (uint32_t j = 0; j < NG; ++j) wv[j] = (base == 0u && j < 2u) ? pw[j] : 0u;
        for (;;) {
          bool missing = false;
  #pragma unroll
          for (uint32_t j = 0; j < NG; ++j)
            missing = missing || (base + j * 64u + lane < chunk && (wv[j] >> FX_RS_STATUS_BITS) != la.epoch);
          if (!missing) break;
          if (polls >= la.spin_limit) { ok = false; break; }
          ++polls;
          __builtin_amdgcn_s_sleep(1);
  #pragma unroll
          for (uint32_t j = 0; j < NG; ++j)
            if (base + j * 64u + lane < chunk && (wv[j] >> FX_RS_STATUS_BITS) != la.epoch)
              wv[j] = __hip_atomic_load(la.status + first + base + j * 64u + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
  #pragma unroll
        for (uint32_t j = 0; j < NG; ++j)
          part += (ok && base + j * 64u + lane < chunk) ? (wv[j] & ((1u << FX_RS_STATUS_BITS) - 1u)) : 0u;
      }
      part = fx_wave_sum(part, lane);
      const bool all_ok = __builtin_amdgcn_ballot_w64(!ok) == 0ull;
      if (lane == 0) { s_prefix = part; s_ok = all_ok ? 1u : 0u; }
      // The task's last chunk tells the host the task's total as soon as it is known: its own
      // count comes from its status word (wave 0 publishes it right after the gather).  The host
      // polls the word while the kernel still runs: a system-scope store goes through to host
      // memory instead of waiting in L2 for the end of the kernel.
      if (chunk + 1u == la.chunks && all_ok) {
        uint32_t wv = 0, polls = 0;
        bool own = true;
        for (;;) {
          wv = __hip_atomic_load(la.status + b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if ((wv >> FX_RS_STATUS_BITS) == la.epoch) break;
          if (polls >= la.spin_limit) { own = false; break; }
          ++polls;
          __builtin_amdgcn_s_sleep(1);
        }
        if (own && lane == 0) {
          __hip_atomic_store(la.totals + task, part + (wv & ((1u << FX_RS_STATUS_BITS) - 1u)), __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_SYSTEM);
          s_told = 1u;
        }
      }
    };
    // ---- requests: mask of the chunk's rows (wave 0), first look at the earlier chunks (wave 1),
    // rows of the first sub-tile (everybody).  In a launch that floods the memory system
    // (la.bulk_delay) the waves that carry no gather hold their requests back for a moment: the
    // counts, a few bytes per row that every later workgroup of the task waits for, then reach the
    // memory system ahead of the bulk instead of somewhere in a queue of tens of megabytes.
    if (wave == 0) {
      bool keep[NSUB];
  #pragma unroll
      for (uint32_t j = 0; j < NSUB; ++j) {
        const uint32_t r = j * 64u + lane;
        // rows past the chunk evaluate the chunk's last row (a valid address) and are dropped
        keep[j] = P::template mask<FxRsRt>(rt, c_r0 + min(r, c_rows - 1u)) && r < c_rows;
      }
      request(0);
      uint32_t nk = 0;
  #pragma unroll
      for (uint32_t j = 0; j < NSUB; ++j) {
        s_keep[j * 64u + lane] = keep[j] ? 1u : 0u;
        nk += (uint32_t)__popcll(__builtin_amdgcn_ballot_w64(keep[j]));
      }
      if (lane == 0) {
        __hip_atomic_store(la.status + b, (la.epoch << FX_RS_STATUS_BITS) | nk, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_total = nk;
      }
    } else {
      if (wave == 1) {
        if (lane == 0) s_told = 0u;
  #pragma unroll
        for (uint32_t j = 0; j < 2; ++j)
          if (j * 64u + lane < chunk)
            pw[j] = __hip_atomic_load(la.status + b - chunk + j * 64u + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      if (SIDE_LDS) {
        // (these waves hold their rows back anyway, and the table is shared by the tasks: cache hits)
        for (uint32_t r = threadIdx.x - 64u; r < c_rows; r += NT - 64u) {
          typename P::Side sd;
          P::template row_side<FxRsRt>(rt, c_r0 + r, sd);
  #pragma unroll
          for (uint32_t k = 0; k < P::n_side; ++k) side[r * P::n_side + k] = sd.s[k];
        }
      }
      if (wave == 1 && teller) {
        // The host waits for this wave's word: it looks back before it asks for any rows (its polls
        // would wait for them: loads return in order), so the task's total leaves as soon as the
        // counts of the task's chunks are known, not when the first sub-tile has arrived.
        look_back();
        request(0);
      } else {
        if (!PERSIST || b == blockIdx.x)   // (the first chunks of a launch start together; later ones are spread out)
        for (uint32_t d = 0; d < la.bulk_delay; d += 32u) __builtin_amdgcn_s_sleep(32);
        request(0);
      }
    }

    uint32_t prefix = 0, before = 0, staged_kept = 0, staged_orow = 0;
    for (uint32_t s = 0; s < n_sub; ++s) {
      if (s) __syncthreads();   // the window and the row map of the sub-tile before are no longer read
      // Outputs that the sub-tile before put together in LDS leave now, as aligned runs, while the
      // next window is parked: behind the barrier above everything is in place, and the barrier
      // below keeps this sub-tile's values out of the buffers until everything has left.
      if (P::n_staged != 0u && s) fx_rs_copy_out<P, 0u>(rt, staged_kept, staged_orow, threadIdx.x, NT);
      const uint32_t sh = shift;
  #pragma unroll
      for (uint32_t k = 0; k < KV; ++k) {
        const uint32_t v = threadIdx.x + k * NT;
        if (v < n_vec) ((fx_u32x4*)L)[v] = wr[k];
      }
      // all of the sub-tile is parked before the next one is asked for: interleaved, every new
      // request would be waited for where the next old line is parked
      asm volatile("" ::: "memory");
      // (wave 1 looks back first where it does: its polls wait for everything it has asked for)
      const bool looks_back = wave == 1u && s == 0u && !teller;
      if (s + 1u < n_sub && !looks_back) request(s + 1u);
      const uint32_t t_r0 = s * sub_rows, t_rows = min(sub_rows, c_rows - t_r0);
      if (wave == 0) {
        const bool keep = lane < t_rows && s_keep[t_r0 + lane] != 0u;
        const uint64_t bal = __builtin_amdgcn_ballot_w64(keep);
        if (keep) s_rowmap[__popcll(bal & ((1ull << lane) - 1ull))] = lane;
        if (lane == 0) s_nk = (uint32_t)__popcll(bal);
      } else if (looks_back) {
        look_back();
        if (s + 1u < n_sub) request(s + 1u);
      }
      __syncthreads();
      if (s == 0) {
        if (uni(s_ok) == 0u) {
          // an earlier chunk has not reported in time: count the kept rows in front of this chunk
          // here, from memory
          uint32_t cnt = 0;
          for (uint32_t r = threadIdx.x; r < c_r0 + ((NT - c_r0 % NT) % NT); r += NT) {
            const bool k2 = P::template mask<FxRsRt>(rt, min(r, c_r0 - 1u)) && r < c_r0;
            cnt += (uint32_t)__popcll(__builtin_amdgcn_ballot_w64(k2));
          }
          if (lane == 0) s_wsum[wave] = cnt;
          __syncthreads();
          if (threadIdx.x == 0) {
            uint32_t p = 0;
            for (uint32_t k = 0; k < NW; ++k) p += s_wsum[k];
            s_prefix = p;
          }
          __syncthreads();
        }
        prefix = uni(s_prefix);
        // (the total of the task, unless wave 1 has told the host already)
        if (chunk + 1u == la.chunks && threadIdx.x == 0 && s_told == 0u)
          __hip_atomic_store(la.totals + task, prefix + s_total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      }
      const uint32_t n_kept = uni(s_nk);
      const uint32_t* Wb = L + sh;
      const uint32_t orow = prefix + before;          // first compacted row of this sub-tile
      const uint32_t rs0 = c_r0 + t_r0;               // first source row of this sub-tile
      fx_rs_phases<P, 0u>(rt, orow);
      // ---- the columns with code of their own: one kept row per lane
      if (P::n_row_cols != 0u && threadIdx.x < n_kept) {
        const uint32_t src = s_rowmap[threadIdx.x];
        // What the row reads besides the window: from the chunk's table in LDS.  (Loaded here, the
        // words would arrive behind the next sub-tile, which this wave has asked for already: loads
        // return in order.)
        typename P::Side sd;
        if (SIDE_LDS) {
  #pragma unroll
          for (uint32_t k = 0; k < P::n_side; ++k) sd.s[k] = side[(t_r0 + src) * P::n_side + k];
        } else {
          P::template row_side<FxRsRt>(rt, rs0 + src, sd);
        }
        P::template row<FxRsRt>(rt, Wb + src * S, sd, rs0 + src, orow + threadIdx.x, threadIdx.x);
      }
      // ---- vector segments: four columns per lane
      fx_rs_segments<P>(typename P::Vecs{}, rt, Wb, s_rowmap, n_kept, rs0, orow, threadIdx.x, NT);
      staged_kept = n_kept;
      staged_orow = orow;
      before += n_kept;
    }
    if (P::n_staged != 0u) {
      __syncthreads();
      fx_rs_copy_out<P, 0u>(rt, staged_kept, staged_orow, threadIdx.x, NT);
    }
    if constexpr (!PERSIST) {
      break;
    } else {
      b += gridDim.x;
      if (b >= n_chunks_all) break;
      __syncthreads();   // the window, the row map and the tables are written again by the next chunk
    }
  }
}

struct FxRsRegistrar {
  FxRsRegistrar(uint64_t key, const void* fn, const void* fn_lean, const void* fn_persist, const void* fn_wide, uint32_t S,
                uint32_t stage_row_words, uint32_t n_staged, uint32_t side_row_words) {
    FxRsKernel k;
    k.fn = fn;
    k.fn_lean = fn_lean;
    k.fn_persist = fn_persist;
    k.fn_wide = fn_wide;
    k.S = S;
    k.stage_row_words = stage_row_words;
    k.n_staged = n_staged;
    k.side_row_words = side_row_words;
    fx_rs_register(key, k);
  }
};

}  // namespace

#define FX_RS_REGISTER(P) \
  static FxRsRegistrar fx_rs_registrar_##P(P::key, (const void*)&fx_rs_kernel<P, FX_RS_KV, false>,                          \
                                           (const void*)&fx_rs_kernel<P, FX_RS_KV_LEAN, false>,                             \
                                           (const void*)&fx_rs_kernel<P, FX_RS_KV, true>,                                   \
                                           (const void*)&fx_rs_kernel<P, FX_RS_KV, true, true>, P::S, P::stage_row_words,   \
                                           P::n_staged, (P::n_row_cols != 0u && P::n_side <= FX_RS_MAX_SIDE) ? P::n_side : 0u);
