// fx_head_stream: decode + score filter of a YOLO-style detection head in one launch (see
// fx_head.h for what it stands in for and when it is chosen).
//
// A workgroup owns a CHUNK: a run of up to 256 consecutive prediction rows of one image.  The
// host sizes the chunks so that all workgroups of the launch are resident together whenever the
// input allows it.
//   1. Wave 0 gathers the objectness of every row of the chunk (one float per row, issued before
//      anything else), evaluates the threshold and publishes the chunk's kept-row count in a
//      status word tagged with the call's epoch.
//   2. Meanwhile all waves ask for the rows of the first sub-tile (up to 64 rows: one contiguous
//      run of memory, coalesced 128-bit loads; the lines travel in registers and are parked in an
//      LDS window; the next sub-tile is requested as soon as the current one is parked).
//   3. One look-back per workgroup (wave 1): the write offset of the chunk is the sum of the
//      counts of the earlier chunks of its image, read from their status words as they appear.
//      Earlier chunks never wait for later ones, and every poll loop is bounded: when a word does
//      not show up within spin_limit polls the workgroup counts the kept rows of the earlier
//      chunks itself, from memory, so the kernel ends whatever the order in which workgroups
//      are started.
//   4. Per sub-tile: row map from the kept flags (ballot + popcount), then from LDS only:
//      boxes and objectness one kept row per lane, class scores four per lane, written to their
//      compacted rows with 128-bit stores.  Rows are loaded and results stored as streaming
//      (non-temporal) accesses: every line is touched once, and the 46 MB a large launch writes
//      leave for memory while the kernel runs instead of sitting in the caches until its end
//      (27.5 -> 21 us on cold lines for 16 images).
// The arithmetic repeats the lowered programs of the region operation for operation (fx_sigmoid,
// fx_exp, no contraction), so the results are bit-identical to the generic kernels.
// Status words belong to the library (one per chunk, zero when allocated, never reset: a word
// of an earlier call carries an older epoch).
#include <hip/hip_runtime.h>

#include "fx_device.h"
#include "fx_head.h"

namespace {

#define FX_HEAD_DYN_OFF sizeof(FxHeadLaunch)
typedef uint32_t fx_u32x2_a4 __attribute__((ext_vector_type(2), aligned(4)));   // 64 bits, 4-byte aligned

__device__ __forceinline__ uint64_t fxh_ptr(const FxHeadLaunch& hl, uint32_t slot, uint32_t task) {
  const uint8_t* ka = (const uint8_t*)__builtin_amdgcn_kernarg_segment_ptr();
  const uint64_t* gp = (const uint64_t*)(ka + FX_HEAD_DYN_OFF);
  const uint32_t pi = (slot & FX_SLOT_TASK) ? hl.n_sptr + task * hl.n_tptr + (slot & 0xffffu) : (slot & 0xffffu);
  return gp[pi];
}

__global__ __launch_bounds__(FX_BLOCK) void fx_head_stream(const FxHeadLaunch hl, const FxDyn) {
  constexpr uint32_t NT = FX_BLOCK, NW = NT / 64u, KV = FX_HEAD_KV, NSUB = FX_HEAD_NSUB;
  extern __shared__ __attribute__((aligned(16))) uint32_t L[];   // the window: sub_rows rows of S floats
  __shared__ uint32_t s_rowmap[FX_HEAD_SUB];
  __shared__ uint8_t s_keep[FX_BLOCK];
  __shared__ uint32_t s_wsum[NW];
  __shared__ uint32_t s_prefix, s_ok, s_nk, s_total, s_told;
  const uint32_t lane = threadIdx.x & 63u, wave = uni(threadIdx.x >> 6);
  const uint32_t b = blockIdx.x;
  const uint32_t task = b / hl.chunks, chunk = b - task * hl.chunks;
  const uint32_t c_r0 = chunk * hl.chunk_rows;
  const uint32_t c_rows = min(hl.chunk_rows, hl.n_rows - c_r0);   // >= 1 (host)
  // sub-tiles of equal size, at most hl.sub_rows rows each
  const uint32_t n_sub0 = (c_rows + hl.sub_rows - 1u) / hl.sub_rows;
  const uint32_t sub_rows = (c_rows + n_sub0 - 1u) / n_sub0;
  const uint32_t n_sub = (c_rows + sub_rows - 1u) / sub_rows;
  const uint32_t S = hl.S;
  const float thr = u2f(hl.thr_bits);
  // element 0 of this task's rows
  const FX_AS1 float* pred = (const FX_AS1 float*)fxh_ptr(hl, hl.pred_slot, task) + (int64_t)hl.pred_tcoef * task;

  fx_u32x4 wr[KV];
  uint32_t shift = 0, n_vec = 0;
  auto request = [&](uint32_t s) {
    const uint32_t r0 = c_r0 + s * sub_rows, rows = min(sub_rows, c_rows - s * sub_rows);
    const uint64_t a0 = (uint64_t)(pred + (size_t)r0 * S);
    shift = ((uint32_t)a0 & 15u) >> 2;   // floats between the 16-byte line and the first row
    const FX_AS1 fx_u32x4* g4 = (const FX_AS1 fx_u32x4*)(a0 & ~(uint64_t)15);
    n_vec = (shift + rows * S + 3u) >> 2;   // <= KV * NT (host)
#pragma unroll
    for (uint32_t k = 0; k < KV; ++k) {
      const uint32_t v = threadIdx.x + k * NT;
      if (v < n_vec) wr[k] = __builtin_nontemporal_load(&g4[v]);   // every line is used once
    }
  };
  uint32_t pw[2] = {0, 0};   // wave 1: what its first look at the earlier chunks found
  // One look-back per workgroup (wave 1): the sum of the counts of the earlier chunks of the image.
  auto look_back = [&]() {
    const uint32_t first = b - chunk;
    uint32_t part = 0;
    bool ok = true;
    for (uint32_t i = lane; i < chunk; i += 64u) {
      uint32_t wv = i < 64u ? pw[0] : (i < 128u ? pw[1] : 0u), polls = 0;
      while ((wv >> FX_HEAD_STATUS_BITS) != hl.epoch) {
        if (polls >= hl.spin_limit) { ok = false; break; }
        ++polls;
        __builtin_amdgcn_s_sleep(1);
        wv = __hip_atomic_load(hl.status + first + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      part += ok ? (wv & ((1u << FX_HEAD_STATUS_BITS) - 1u)) : 0u;
    }
    part = fx_wave_sum(part, lane);
    const bool all_ok = __builtin_amdgcn_ballot_w64(!ok) == 0ull;
    if (lane == 0) { s_prefix = part; s_ok = all_ok ? 1u : 0u; }
    // The image's last chunk tells the host the image's total as soon as it is known: its own
    // count comes from its status word (wave 0 publishes it right after the gather).  The host polls the word while the kernel still runs: a
    // system-scope store goes through to host memory instead of waiting in L2 for the end of
    // the kernel.
    if (chunk + 1u == hl.chunks && all_ok) {
      uint32_t wv = 0, polls = 0;
      bool own = true;
      for (;;) {
        wv = __hip_atomic_load(hl.status + b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((wv >> FX_HEAD_STATUS_BITS) == hl.epoch) break;
        if (polls >= hl.spin_limit) { own = false; break; }
        ++polls;
        __builtin_amdgcn_s_sleep(1);
      }
      if (own && lane == 0) {
        __hip_atomic_store(hl.totals + task, part + (wv & ((1u << FX_HEAD_STATUS_BITS) - 1u)), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_SYSTEM);
        s_told = 1u;
      }
    }
  };
  // ---- requests: objectness of the chunk (wave 0), first look at the earlier chunks (wave 1),
  // rows of the first sub-tile (everybody).  In a launch that floods the memory system
  // (hl.bulk_delay) the waves that carry no gather hold their requests back for a moment: the
  // counts, a few bytes per row that every later workgroup of the image waits for, then reach the
  // memory system ahead of the bulk instead of somewhere in a queue of tens of megabytes.
  float o[NSUB];
  if (wave == 0) {
#pragma unroll
    for (uint32_t j = 0; j < NSUB; ++j) {
      const uint32_t r = j * 64u + lane;
      o[j] = r < c_rows ? pred[(size_t)(c_r0 + r) * S + 4u] : 0.0f;
    }
  } else {
    if (wave == 1) {
      if (lane == 0) s_told = 0u;
#pragma unroll
      for (uint32_t j = 0; j < 2; ++j)
        if (j * 64u + lane < chunk)
          pw[j] = __hip_atomic_load(hl.status + b - chunk + j * 64u + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    for (uint32_t d = 0; d < hl.bulk_delay; d += 32u) __builtin_amdgcn_s_sleep(32);
  }
  request(0);

  // ---- kept flags and count of the chunk; published at once
  if (wave == 0) {
    uint32_t nk = 0;
#pragma unroll
    for (uint32_t j = 0; j < NSUB; ++j) {
      const uint32_t r = j * 64u + lane;
      const bool keep = r < c_rows && fx_sigmoid(o[j]) >= thr;
      s_keep[r] = keep ? 1u : 0u;
      nk += (uint32_t)__popcll(__builtin_amdgcn_ballot_w64(keep));
    }
    if (lane == 0) {
      __hip_atomic_store(hl.status + b, (hl.epoch << FX_HEAD_STATUS_BITS) | nk, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_total = nk;
    }
  }

  uint32_t prefix = 0, before = 0;
  for (uint32_t s = 0; s < n_sub; ++s) {
    if (s) __syncthreads();   // the window and the row map of the sub-tile before are no longer read
    const uint32_t sh = shift;
#pragma unroll
    for (uint32_t k = 0; k < KV; ++k) {
      const uint32_t v = threadIdx.x + k * NT;
      if (v < n_vec) ((fx_u32x4*)L)[v] = wr[k];
    }
    if (s + 1u < n_sub) request(s + 1u);
    const uint32_t t_r0 = s * sub_rows, t_rows = min(sub_rows, c_rows - t_r0);
    if (wave == 0) {
      const bool keep = lane < t_rows && s_keep[t_r0 + lane] != 0u;
      const uint64_t bal = __builtin_amdgcn_ballot_w64(keep);
      if (keep) s_rowmap[__popcll(bal & ((1ull << lane) - 1ull))] = lane;
      if (lane == 0) s_nk = (uint32_t)__popcll(bal);
    } else if (wave == 1 && s == 0) {
      look_back();
    }
    __syncthreads();
    if (s == 0) {
      if (uni(s_ok) == 0u) {
        // an earlier chunk has not reported in time: count the kept rows in front of this chunk
        // here, from memory
        uint32_t cnt = 0;
        for (uint32_t r = threadIdx.x; r < c_r0 + ((NT - c_r0 % NT) % NT); r += NT) {
          const bool k2 = r < c_r0 && fx_sigmoid(pred[(size_t)r * S + 4u]) >= thr;
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
      // (the total of the image, unless wave 1 has told the host already)
      if (chunk + 1u == hl.chunks && threadIdx.x == 0 && s_told == 0u)
        __hip_atomic_store(hl.totals + task, prefix + s_total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    const uint32_t n_kept = uni(s_nk);
    const uint32_t* W = L + sh;
    const uint32_t orow = prefix + before;          // first compacted row of this sub-tile
    const uint32_t rs0 = c_r0 + t_r0;               // first source row of this sub-tile
    // ---- boxes and objectness: one kept row per lane
    if (threadIdx.x < n_kept) {
      const uint32_t r = threadIdx.x, src = s_rowmap[r], row = rs0 + src;
      const FX_AS1 float* anc = (const FX_AS1 float*)fxh_ptr(hl, hl.anc_slot, task) + (int64_t)hl.anc_tcoef * task;
      const FX_AS1 float* strd = (const FX_AS1 float*)fxh_ptr(hl, hl.strd_slot, task) + (int64_t)hl.strd_tcoef * task;
      const float st = strd[row];
      // base of the centre and of the half size: from the anchor corners, or folded ahead of time
      float bcx, bcy, bhw, bhh;
      if (hl.folded) {
        const FX_AS1 float* hf = (const FX_AS1 float*)fxh_ptr(hl, hl.half_slot, task) + (int64_t)hl.half_tcoef * task;
        const fx_u32x2_a4 c2 = *(const FX_AS1 fx_u32x2_a4*)(anc + (size_t)row * 2u);
        const fx_u32x2_a4 h2 = *(const FX_AS1 fx_u32x2_a4*)(hf + (size_t)row * 2u);
        bcx = u2f(c2.x); bcy = u2f(c2.y); bhw = u2f(h2.x); bhh = u2f(h2.y);
      } else {
        const fx_u32x4_a4 an = *(const FX_AS1 fx_u32x4_a4*)(anc + (size_t)row * 4u);
        const float a0 = u2f(an.x), a1 = u2f(an.y), a2 = u2f(an.z), a3 = u2f(an.w);
        bcx = (a0 + a2) * 0.5f; bcy = (a1 + a3) * 0.5f; bhw = (a2 - a0) * 0.5f; bhh = (a3 - a1) * 0.5f;
      }
      const uint32_t* p = W + src * S;
      const float p0 = u2f(p[0]), p1 = u2f(p[1]), p2 = u2f(p[2]), p3 = u2f(p[3]), p4 = u2f(p[4]);
      // half sizes ((hi - lo) * 0.5) * exp(p), centres ((lo + hi) * 0.5) + ((sigmoid(p) - 0.5) * stride)
      const float hw = bhw * fx_exp(p2), hh = bhh * fx_exp(p3);
      const float cx = bcx + ((fx_sigmoid(p0) - 0.5f) * st);
      const float cy = bcy + ((fx_sigmoid(p1) - 0.5f) * st);
      fx_u32x4 ob;
      ob.x = f2u(cx - hw); ob.y = f2u(cy - hh); ob.z = f2u(cx + hw); ob.w = f2u(cy + hh);
      FX_AS1 float* box = (FX_AS1 float*)fxh_ptr(hl, hl.out_slot[1], task) + (size_t)hl.out_tstride[1] * task;
      FX_AS1 float* obj = (FX_AS1 float*)fxh_ptr(hl, hl.out_slot[0], task) + (size_t)hl.out_tstride[0] * task;
      __builtin_nontemporal_store(ob, (FX_AS1 fx_u32x4_a4*)(box + (size_t)(orow + r) * 4u));
      __builtin_nontemporal_store(fx_sigmoid(p4), obj + orow + r);
    }
    // ---- class scores: four per lane
    {
      const uint32_t G = hl.C >> 2, ng = n_kept * G;
      FX_AS1 float* cls = (FX_AS1 float*)fxh_ptr(hl, hl.out_slot[2], task) + (size_t)hl.out_tstride[2] * task + (size_t)orow * hl.C;
#pragma unroll 2
      for (uint32_t g = threadIdx.x; g < ng; g += NT) {
        const uint32_t r = fx_fastdiv(g, hl.g_magic, hl.g_shift);
        const uint32_t c = g - r * G;
        const uint32_t* p = W + s_rowmap[r] * S + 5u + c * 4u;
        fx_u32x4 v;
        v.x = f2u(fx_sigmoid(u2f(p[0]))); v.y = f2u(fx_sigmoid(u2f(p[1])));
        v.z = f2u(fx_sigmoid(u2f(p[2]))); v.w = f2u(fx_sigmoid(u2f(p[3])));
        __builtin_nontemporal_store(v, (FX_AS1 fx_u32x4_a4*)(cls + (size_t)g * 4u));
      }
    }
    before += n_kept;
  }
}

}  // namespace

uint32_t fx_head_lds_bytes(const FxHeadLaunch& hl) {
  return (((hl.sub_rows * hl.S + 3u + 3u) >> 2) + 1u) * 16u;
}

// Workgroups of the kernel that the current device holds at once.
hipError_t fx_head_resident(uint32_t lds_bytes, uint32_t* workgroups, uint32_t* per_cu_out) {
  int dev = 0, cus = 0, per_cu = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return e;
  e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)&fx_head_stream, (int)FX_BLOCK, (size_t)lds_bytes);
  if (e != hipSuccess) return e;
  *workgroups = (uint32_t)std::max(per_cu, 1) * (uint32_t)std::max(cus, 1);
  *per_cu_out = (uint32_t)std::max(per_cu, 1);
  return hipSuccess;
}

hipError_t fx_launch_head_stream(const FxHeadLaunch& hl, const FxDyn* dyn, hipStream_t stream) {
  const uint32_t grid = hl.chunks * hl.n_tasks;
  if (grid == 0) return hipSuccess;
  void* args[2] = {(void*)&hl, (void*)dyn};
  return hipLaunchKernel((const void*)&fx_head_stream, dim3(grid), dim3(FX_BLOCK), args, fx_head_lds_bytes(hl), stream);
}
