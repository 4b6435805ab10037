// Detection tail in ONE launch for all tasks (images): candidate selection by score threshold,
// sort by descending score, class-aware greedy NMS, top-k.  What the reference runs after its row
// compaction as a chain of ATen / torchvision kernels with host synchronisations in between
// (nonzero, index, max, sort, torchvision::nms, slicing: functs/benchmark/ai_model/yolov3/
// yolov3_bbox.py:104-179, functs/benchmark/ai_model/ssd/ssd_bbox.py:163-214).
//
// `slices` workgroups of 1024 threads per task share the scan of its scores; the last of them to
// finish (a ticket counter: nobody waits for anybody) does the rest alone, in LDS:
//   1. candidates whose score passes the threshold become 64-bit keys (inverted orderable score
//      bits : candidate index), collected in LDS by each workgroup and appended to the task's
//      key buffer in the workspace - their order of arrival does not matter, the index in the
//      key restores it;
//   2. bitonic sort of the keys: descending score, equal scores by ascending index (a stable
//      descending sort);
//   3. candidates are taken 64 at a time in that order.  Each is tested against the kept list
//      (16 threads per candidate), the 64 x 64 overlaps inside the chunk become one 64-bit word
//      per candidate (its overlapping predecessors), and one wave resolves the chunk: all
//      candidates decide together in rounds, as many as the longest chain of overlaps.  The
//      walk ends when max_num boxes are kept: later candidates cannot change earlier decisions.
// The workspace counters are zero when a launch starts and zero again when it ends.
// The number of valid rows per task is read from memory (device or pinned host), so the count a
// preceding compaction produced never has to reach the host.
// Arithmetic of an overlap test, in float32 and in this order (no contraction):
//   box + label * (max coordinate + 1);  area = (x2 - x1) * (y2 - y1);
//   inter = max(0, min(x2) - max(x1)) * max(0, min(y2) - max(y1));  iou = inter / ((area_i + area_j) - inter) > thr
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>
#include <mutex>

#include "../../../include/fxhip.h"
#include "fx_device.h"

// a hook for timing the phases of a task's last workgroup from a test program; nothing in the library
#ifndef FX_NMS_STAMP
#define FX_NMS_STAMP(k)
#endif

#define FX_NMS_THREADS 1024u
#define FX_NMS_CHUNK 64u

namespace {

__device__ __forceinline__ uint32_t orderable(float f) {   // monotone map float -> uint32
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float from_orderable(uint32_t o) {
  return __uint_as_float((o & 0x80000000u) ? (o & 0x7fffffffu) : ~o);
}

// one stage of the bitonic network on a key a lane, partners J lanes apart: the lower lane keeps
// the smaller key where the run ascends
template <uint32_t J>
__device__ __forceinline__ uint64_t bitonic_step(uint64_t key, bool up, uint32_t lane) {
  const uint64_t other = ((uint64_t)fx_lane_xor<J>((uint32_t)(key >> 32), lane) << 32) | (uint64_t)fx_lane_xor<J>((uint32_t)key, lane);
  const bool keep_min = ((lane & J) == 0u) == up;
  return ((key < other) == keep_min) ? key : other;
}

struct Box { float x1, y1, x2, y2; };

__device__ __forceinline__ bool overlaps(const Box& a, float area_a, const Box& b, float area_b, float thr) {
  const float xx1 = fmaxf(a.x1, b.x1), yy1 = fmaxf(a.y1, b.y1);
  const float xx2 = fminf(a.x2, b.x2), yy2 = fminf(a.y2, b.y2);
  const float w = fmaxf(0.0f, xx2 - xx1), h = fmaxf(0.0f, yy2 - yy1);
  const float inter = w * h;
  const float iou = inter / ((area_a + area_b) - inter);
  return iou > thr;
}

// workspace: per task FX_NMS_WS_WORDS counters (candidates, finished slices, largest coordinate,
// row count + 1; zero between launches) in front of all tasks' key buffers
#define FX_NMS_WS_WORDS 64u
__global__ __launch_bounds__(FX_NMS_THREADS) void fx_sort_nms_kernel(const fx_nms_desc d, const uint32_t key_cap,
                                                                    const uint32_t slices, uint32_t* const ws,
                                                                    uint32_t* err_host) {
  extern __shared__ __attribute__((aligned(16))) uint64_t s_keys[];   // key_cap (a power of two)
  __shared__ float s_kbox[FX_NMS_MAX_OUT][4];
  __shared__ float s_karea[FX_NMS_MAX_OUT];
  __shared__ float s_cbox[FX_NMS_CHUNK][4];     // chunk: original boxes
  __shared__ float s_obox[FX_NMS_CHUNK][4];     // chunk: boxes moved by their class offset
  __shared__ float s_carea[FX_NMS_CHUNK];
  __shared__ uint32_t s_cidx[FX_NMS_CHUNK], s_clabel[FX_NMS_CHUNK];
  __shared__ float s_cscore[FX_NMS_CHUNK];
  __shared__ uint32_t s_in[FX_NMS_CHUNK][2];    // earlier candidates of the chunk that overlap candidate j
  __shared__ uint32_t s_dead[2];                // candidates of the chunk that the kept list overlaps
  __shared__ uint32_t s_count, s_maxc, s_nk, s_base, s_ticket;

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t task = blockIdx.x / slices, slice = blockIdx.x - task * slices;
  uint32_t* const ctr = ws + (size_t)task * FX_NMS_WS_WORDS;   // [0] candidates, [1] finished slices, [2] largest coordinate
  uint64_t* const g_keys = (uint64_t*)(ws + (size_t)d.n_tasks * FX_NMS_WS_WORDS) + (size_t)task * key_cap;
  // NC classes, in rows of C elements (C > NC: columns behind the class scores that are not candidates)
  const uint32_t NC = d.mode == 1 ? d.n_classes : 1u;
  const uint32_t C = (d.mode == 1 && d.scores_row_stride != 0u) ? d.scores_row_stride : NC;
  const float* boxes = d.boxes + (int64_t)task * d.boxes_task_stride;
  const float* scores = d.scores + (int64_t)task * d.scores_task_stride;
  const float* factors = d.factors ? d.factors + (int64_t)task * d.factors_task_stride : nullptr;
  const int64_t* labels = d.labels ? d.labels + (int64_t)task * d.labels_task_stride : nullptr;
  float* dets = d.dets + (size_t)task * d.max_num * 5u;
  int64_t* out_labels = d.out_labels + (size_t)task * d.max_num;
  int64_t* out_index = d.out_index ? d.out_index + (size_t)task * d.max_num : nullptr;

  // The task's row count may lie in host memory, where a read costs a trip over the bus and the
  // reads of many workgroups queue up: slice 0 reads it and passes it on through the workspace
  // (count + 1 in ctr[3]); a slice that does not see it within its polls reads it itself.
  if (tid == 0) {
    s_count = 0u;
    s_maxc = 0u;
    uint32_t rows = d.rows;
    if (d.counts) {
      uint32_t seen = 0u;
      if (slice != 0u)
        for (uint32_t polls = 0; polls < 4096u && seen == 0u; ++polls) {
          seen = __hip_atomic_load(&ctr[3], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (seen == 0u) __builtin_amdgcn_s_sleep(2);
        }
      if (seen == 0u) {
        seen = min(d.rows, __hip_atomic_load(d.counts + task, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM)) + 1u;
        if (slice == 0u) __hip_atomic_store(&ctr[3], seen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      rows = seen - 1u;
    }
    s_base = rows;
  }
  __syncthreads();
  const uint32_t rows = s_base;
  __syncthreads();   // s_base is used again below

  FX_NMS_STAMP(0);
  // 1. candidates: four 128-bit loads per thread in flight
  const uint32_t all_items = rows * C;   // < 2^32 (host)
  // this workgroup's share: a multiple of four items, so that its 128-bit loads stay aligned
  const uint32_t share = (((all_items + slices - 1u) / slices) + 3u) & ~3u;
  const uint32_t first = min(slice * share, all_items);
  const uint32_t n_items = min(first + share, all_items);   // end of the share
  const bool vec = (((uintptr_t)scores) & 15u) == 0u;
  constexpr uint32_t U = 4u, PER_ROUND = FX_NMS_THREADS * U * 4u;
  for (uint32_t base = first; base < n_items; base += PER_ROUND) {
    float v[U][4];
#pragma unroll
    for (uint32_t u = 0; u < U; ++u) {
      const uint32_t i0 = base + (u * FX_NMS_THREADS + tid) * 4u;
      if (vec && i0 + 3u < n_items) {
        const float4 q = *(const float4*)(scores + i0);
        v[u][0] = q.x; v[u][1] = q.y; v[u][2] = q.z; v[u][3] = q.w;
      } else {
#pragma unroll
        for (uint32_t e = 0; e < 4u; ++e) v[u][e] = i0 + e < n_items ? scores[i0 + e] : d.score_thr;   // the threshold itself never passes
      }
    }
    uint32_t mine = 0u;   // bit u * 4 + e: element passes
#pragma unroll
    for (uint32_t u = 0; u < U; ++u)
#pragma unroll
      for (uint32_t e = 0; e < 4u; ++e)
        if (v[u][e] > d.score_thr) mine |= 1u << (u * 4u + e);
    // few elements pass a detector's threshold: a lane that has some takes its places with one LDS
    // atomic (the order of arrival does not matter), the others go straight on to the next loads
    if (mine == 0u) continue;
    if (C != NC) {   // columns behind the class scores are no candidates
#pragma unroll
      for (uint32_t u = 0; u < U; ++u)
#pragma unroll
        for (uint32_t e = 0; e < 4u; ++e)
          if (((mine >> (u * 4u + e)) & 1u) && (base + (u * FX_NMS_THREADS + tid) * 4u + e) % C >= NC) mine &= ~(1u << (u * 4u + e));
      if (mine == 0u) continue;
    }
    uint32_t slot = atomicAdd(&s_count, (uint32_t)__popc(mine));
#pragma unroll
    for (uint32_t u = 0; u < U; ++u)
#pragma unroll
      for (uint32_t e = 0; e < 4u; ++e) {
        if ((mine >> (u * 4u + e)) & 1u) {
          const uint32_t i = base + (u * FX_NMS_THREADS + tid) * 4u + e;
          // (the raw score for now: the row's factor is applied by the finishing workgroup)
          if (slot < key_cap) s_keys[slot] = ((uint64_t)(~orderable(v[u][e])) << 32) | (uint64_t)i;
          ++slot;
        }
      }
  }
  __syncthreads();
  FX_NMS_STAMP(1);
  {
    // hand this workgroup's keys over and take a ticket
    const uint32_t mine = min(s_count, key_cap);
    if (tid == 0) s_base = atomicAdd(&ctr[0], s_count);
    __syncthreads();
    const uint32_t gbase = s_base;
    // Keys and counters are written with device-scope atomic accesses, which go through to the
    // memory side of the caches, and the ticket is taken only after they have been acknowledged:
    // no release / acquire fence, which on this device would write back and invalidate whole
    // caches once per workgroup.  This rests on the device: a relaxed device-scope store is
    // performed at the memory side of the caches by the time it is acknowledged (vmcnt).  The
    // compiler is told the order explicitly: nothing moves across the signal fences.
    for (uint32_t k = tid; k < mine; k += FX_NMS_THREADS)
      if (gbase + k < key_cap) __hip_atomic_store(&g_keys[gbase + k], s_keys[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __syncthreads();
    if (tid == 0) s_ticket = atomicAdd(&ctr[1], 1u);
    __syncthreads();
    if (s_ticket != slices - 1u) return;   // somebody else finishes the task
  }
  FX_NMS_STAMP(2);
  // the last workgroup of the task: everything the others wrote is visible
  const uint32_t count = __hip_atomic_load(&ctr[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  if (tid == 0) {   // the counters are zero again for the next launch
    __hip_atomic_store(&ctr[0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&ctr[1], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&ctr[2], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&ctr[3], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (count > key_cap) {   // more candidates than the launch was sized for: reported, nothing returned
    if (tid == 0) {
      __hip_atomic_store(d.n_out + task, FX_NMS_OVERFLOW, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      if (err_host) __hip_atomic_store(err_host, (uint32_t)FX_ASYNC_NMS_CAPACITY, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    for (uint32_t k = tid; k < d.max_num * 5u; k += FX_NMS_THREADS) dets[k] = 0.0f;
    for (uint32_t k = tid; k < d.max_num; k += FX_NMS_THREADS) {
      out_labels[k] = 0;
      if (out_index) out_index[k] = 0;
    }
    return;
  }
  // The largest coordinate of the candidates' boxes (classes are told apart by moving boxes by a
  // multiple of it): taken here, one box per thread, not in the scan, where a gather per
  // candidate would sit between the rounds of loads.
  uint32_t my_max = 0u;                // below orderable() of every value
  for (uint32_t k = tid; k < count; k += FX_NMS_THREADS) {
    uint64_t key = __hip_atomic_load(&g_keys[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t r = (uint32_t)key / C;
    if (d.mode == 1 && factors) {
      const float sc = from_orderable(~(uint32_t)(key >> 32)) * factors[r];
      key = ((uint64_t)(~orderable(sc)) << 32) | (uint64_t)(uint32_t)key;
    }
    s_keys[k] = key;
    const float4 b = *(const float4*)(boxes + (size_t)r * 4u);
    my_max = max(my_max, max(max(orderable(b.x), orderable(b.y)), max(orderable(b.z), orderable(b.w))));
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) my_max = max(my_max, (uint32_t)__shfl_xor((int)my_max, o, 64));
  if (lane == 0u) atomicMax(&s_maxc, my_max);
  __syncthreads();
  const float class_step = from_orderable(s_maxc) + 1.0f;

  // 2. bitonic sort (ascending keys = descending score, ascending index); the tail is padding.
  // Stages whose partners lie at most 64 apart stay inside aligned blocks of 128 keys: a wave
  // runs all of them on its blocks without a workgroup barrier (LDS accesses of one wave are
  // performed in order), so a phase costs one barrier per wider stage plus one.
  FX_NMS_STAMP(3);
  uint32_t n2 = 128u;
  while (n2 < count) n2 <<= 1;
  for (uint32_t i = count + tid; i < n2; i += FX_NMS_THREADS) s_keys[i] = ~0ull;
  __syncthreads();
  auto exchange = [&](uint32_t i, uint32_t j, uint32_t k) {
    const uint32_t l = i | j;
    const uint64_t a = s_keys[i], b = s_keys[l];
    const bool up = (i & k) == 0u;
    if ((a > b) == up) { s_keys[i] = b; s_keys[l] = a; }
  };
  auto narrow_stages = [&](uint32_t k_first, uint32_t k_last) {   // every stage j <= 64 of phases k_first .. k_last
    for (uint32_t blk = wave; blk < (n2 >> 7); blk += FX_NMS_THREADS / 64u) {
      // the block's 128 keys in registers, two a lane (positions lane and lane + 64): the stages
      // exchange them between lanes, LDS is read and written once per call
      const uint32_t p0 = (blk << 7) + lane;
      uint64_t ka = s_keys[p0], kb = s_keys[p0 + 64u];
      for (uint32_t k = k_first; k <= k_last; k <<= 1) {
        const bool up_a = (p0 & k) == 0u, up_b = ((p0 + 64u) & k) == 0u;
        if (k >= 128u) {   // partners 64 apart: the lane's own two keys (up_a == up_b here)
          const bool sw = (ka > kb) == up_a;
          const uint64_t lo = sw ? kb : ka, hi = sw ? ka : kb;
          ka = lo; kb = hi;
        }
        if (k >= 64u) { ka = bitonic_step<32>(ka, up_a, lane); kb = bitonic_step<32>(kb, up_b, lane); }
        if (k >= 32u) { ka = bitonic_step<16>(ka, up_a, lane); kb = bitonic_step<16>(kb, up_b, lane); }
        if (k >= 16u) { ka = bitonic_step<8>(ka, up_a, lane); kb = bitonic_step<8>(kb, up_b, lane); }
        if (k >= 8u) { ka = bitonic_step<4>(ka, up_a, lane); kb = bitonic_step<4>(kb, up_b, lane); }
        if (k >= 4u) { ka = bitonic_step<2>(ka, up_a, lane); kb = bitonic_step<2>(kb, up_b, lane); }
        ka = bitonic_step<1>(ka, up_a, lane); kb = bitonic_step<1>(kb, up_b, lane);
      }
      s_keys[p0] = ka; s_keys[p0 + 64u] = kb;
    }
  };
  narrow_stages(2u, 128u);
  __syncthreads();
  for (uint32_t k = 256u; k <= n2; k <<= 1) {
    for (uint32_t j = k >> 1; j >= 128u; j >>= 1) {
      for (uint32_t p = tid; p < (n2 >> 1); p += FX_NMS_THREADS) exchange(((p & ~(j - 1u)) << 1) | (p & (j - 1u)), j, k);
      __syncthreads();
    }
    narrow_stages(k, k);
    __syncthreads();
  }

  FX_NMS_STAMP(4);
  // 3. greedy walk
  if (tid == 0) s_nk = 0u;
  __syncthreads();
  uint32_t nk = 0u;
  for (uint32_t pos = 0; pos < count && nk < d.max_num; pos += FX_NMS_CHUNK) {
    const uint32_t m = min(FX_NMS_CHUNK, count - pos);
    if (tid < FX_NMS_CHUNK) {
      s_in[tid][0] = 0u; s_in[tid][1] = 0u;
      if (tid < 2u) s_dead[tid] = 0u;
      if (tid < m) {
        const uint64_t key = s_keys[pos + tid];
        const uint32_t idx = (uint32_t)key;
        const uint32_t r = idx / C;
        const uint32_t label = d.mode == 1 ? idx - r * C : (labels ? (uint32_t)labels[idx] : 0u);
        const float4 b = *(const float4*)(boxes + (size_t)r * 4u);
        const float off = (float)label * class_step;
        const float x1 = b.x + off, y1 = b.y + off, x2 = b.z + off, y2 = b.w + off;
        s_cbox[tid][0] = b.x; s_cbox[tid][1] = b.y; s_cbox[tid][2] = b.z; s_cbox[tid][3] = b.w;
        s_obox[tid][0] = x1; s_obox[tid][1] = y1; s_obox[tid][2] = x2; s_obox[tid][3] = y2;
        s_carea[tid] = (x2 - x1) * (y2 - y1);
        s_cidx[tid] = d.mode == 1 ? r * NC + label : idx;   // position among the candidates proper
        s_clabel[tid] = label;
        s_cscore[tid] = from_orderable(~(uint32_t)(key >> 32));
      }
    }
    __syncthreads();
    {
      // against the kept list: candidate c, every 16th kept box
      const uint32_t c = tid & 63u, part = tid >> 6;
      if (c < m) {
        const Box cb{s_obox[c][0], s_obox[c][1], s_obox[c][2], s_obox[c][3]};
        const float ca = s_carea[c];
        bool dead = false;
        for (uint32_t k = part; k < nk && !dead; k += FX_NMS_THREADS / 64u) {
          const Box kb{s_kbox[k][0], s_kbox[k][1], s_kbox[k][2], s_kbox[k][3]};
          dead = overlaps(kb, s_karea[k], cb, ca, d.iou_thr);
        }
        if (dead) atomicOr(&s_dead[c >> 5], 1u << (c & 31u));
      }
      // inside the chunk: candidate i against four later candidates
      const uint32_t i = tid >> 4, j0 = (tid & 15u) * 4u;
      if (i < m) {
        const Box ib{s_obox[i][0], s_obox[i][1], s_obox[i][2], s_obox[i][3]};
        const float ia = s_carea[i];
#pragma unroll
        for (uint32_t jj = 0; jj < 4u; ++jj) {
          const uint32_t j = j0 + jj;
          if (j > i && j < m) {
            const Box jb{s_obox[j][0], s_obox[j][1], s_obox[j][2], s_obox[j][3]};
            if (overlaps(ib, ia, jb, s_carea[j], d.iou_thr)) atomicOr(&s_in[j][i >> 5], 1u << (i & 31u));
          }
        }
      }
    }
    __syncthreads();
    if (wave == 0u) {
      // In order, candidate i is kept unless a kept one before it overlaps it.  All candidates
      // decide together, round after round: one with a kept overlapping predecessor is dead, one
      // whose overlapping predecessors are all dead is kept, the others wait; the first undecided
      // candidate always decides, and with few overlaps two or three rounds settle the chunk
      // (a walk from candidate to candidate costs 64 dependent steps).
      const uint64_t in = ((uint64_t)s_in[lane][1] << 32) | (uint64_t)s_in[lane][0];
      const uint64_t valid = m >= 64u ? ~0ull : (1ull << m) - 1ull;
      uint64_t deadm = (((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)s_dead[1]) << 32) |
                        (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)s_dead[0])) | ~valid;
      uint64_t keptm = 0ull;
      bool decided = ((deadm >> lane) & 1ull) != 0ull;
      for (;;) {
        const bool now_dead = !decided && (in & keptm) != 0ull;
        const bool now_kept = !decided && !now_dead && (in & ~deadm) == 0ull;
        const uint64_t nd = __ballot(now_dead), nkp = __ballot(now_kept);
        if ((nd | nkp) == 0ull) break;
        deadm |= nd;
        keptm |= nkp;
        decided = decided || now_dead || now_kept;
      }
      // the walk ends when max_num are kept: the first `room` of them in order
      const uint32_t room = d.max_num - nk;
      const uint32_t rank = (uint32_t)__popcll(keptm & ((1ull << lane) - 1ull));
      const uint64_t keep = __ballot(((keptm >> lane) & 1ull) != 0ull && rank < room);
      const uint32_t kept_now = (uint32_t)__popcll(keep);
      if ((keep >> lane) & 1ull) {
        const uint32_t slot = nk + rank;
        s_kbox[slot][0] = s_obox[lane][0]; s_kbox[slot][1] = s_obox[lane][1];
        s_kbox[slot][2] = s_obox[lane][2]; s_kbox[slot][3] = s_obox[lane][3];
        s_karea[slot] = s_carea[lane];
        float* o = dets + (size_t)slot * 5u;
        o[0] = s_cbox[lane][0]; o[1] = s_cbox[lane][1]; o[2] = s_cbox[lane][2]; o[3] = s_cbox[lane][3];
        o[4] = s_cscore[lane];
        out_labels[slot] = (int64_t)s_clabel[lane];
        if (out_index) out_index[slot] = (int64_t)s_cidx[lane];
      }
      if (lane == 0u) s_nk = nk + kept_now;
    }
    __syncthreads();
    nk = s_nk;
  }
  FX_NMS_STAMP(5);
  // rows past the kept ones are zero: the outputs have a fixed shape
  for (uint32_t k = nk * 5u + tid; k < d.max_num * 5u; k += FX_NMS_THREADS) dets[k] = 0.0f;
  for (uint32_t k = nk + tid; k < d.max_num; k += FX_NMS_THREADS) {
    out_labels[k] = 0;
    if (out_index) out_index[k] = 0;
  }
  // (system scope: a count in pinned host memory goes through to the host, which may be polling it)
  if (tid == 0) __hip_atomic_store(d.n_out + task, nk, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

}  // namespace

// slices of a task: a workgroup per CU over all tasks (a CU takes one workgroup of 1024 threads at
// a time: with two per CU the second half of the launch starts when the first ends, 16 us into
// the kernel for 16 images), none with less than one round of loads
uint32_t fx_nms_slices(const fx_nms_desc& d) {
  const uint64_t items = (uint64_t)d.rows * (d.mode == 1 ? std::max(d.n_classes, d.scores_row_stride) : 1u);
  const uint64_t per_round = (uint64_t)FX_NMS_THREADS * 16u;
  uint64_t s = (items + per_round - 1) / per_round;
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) cus = n;
    else cus = 256;
  }
  const uint64_t want = d.n_tasks > 0 ? std::max<uint32_t>((uint32_t)cus / (uint32_t)d.n_tasks, 1u) : 1u;
  if (s > want) s = want;
  if (s > 64) s = 64;
  return s < 1 ? 1u : (uint32_t)s;
}

size_t fx_nms_workspace_bytes(int n_tasks, uint32_t key_cap) {
  return (size_t)n_tasks * ((size_t)FX_NMS_WS_WORDS * 4 + (size_t)key_cap * 8);
}
size_t fx_nms_workspace_clear_bytes(int n_tasks) { return (size_t)n_tasks * FX_NMS_WS_WORDS * 4; }

// 0: launched; otherwise a HIP error code + 100
int fx_launch_sort_nms(const fx_nms_desc& d, uint32_t key_cap, void* workspace, uint32_t* err_host, hipStream_t stream) {
  const size_t lds = (size_t)key_cap * sizeof(uint64_t);
  hipError_t e = hipSuccess;
  if (lds > 32768) {   // beyond what a kernel gets without asking: raised once per device, to the most a launch may need
    static std::mutex mu;
    static bool raised[64] = {};
    int dev = 0;
    e = hipGetDevice(&dev);
    if (e != hipSuccess) return 100 + (int)e;
    std::lock_guard<std::mutex> lock(mu);
    if (dev < 0 || dev >= 64 || !raised[dev]) {
      e = hipFuncSetAttribute((const void*)fx_sort_nms_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)(FX_NMS_MAX_CANDIDATES * sizeof(uint64_t)));
      if (e != hipSuccess) return 100 + (int)e;
      if (dev >= 0 && dev < 64) raised[dev] = true;
    }
  }
  const uint32_t slices = fx_nms_slices(d);
  hipLaunchKernelGGL(fx_sort_nms_kernel, dim3((uint32_t)d.n_tasks * slices), dim3(FX_NMS_THREADS), lds, stream, d, key_cap,
                     slices, (uint32_t*)workspace, err_host);
  e = hipGetLastError();
  return e == hipSuccess ? 0 : 100 + (int)e;
}
