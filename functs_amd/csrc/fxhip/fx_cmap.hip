// fx_classmap_head: decode + per-class score filter of an SSD-style detection head in one launch
// (see fx_cmap.h for what it stands in for and when it is chosen).
//
// A workgroup owns a CHUNK of 32 consecutive priors; the host launches it only when all
// workgroups are resident together.  The work of a chunk is a chain of short dependent steps, so
// the workgroup is wide (512 threads, two rows per half-wave: two waves on every SIMD hide each
// other's latencies; with 1024 threads a CU took one workgroup only and the launch of 273 ran in
// two rounds) or, when only that launch fits the device at once, 256 threads and four rows per
// half-wave.
//   1. Every half-wave takes its rows of class scores (a lane holds four consecutive floats,
//      one 128-bit load per row) and computes their softmax with butterfly reductions inside the
//      half-wave; the first 32 threads also decode the chunk's boxes.  Results stay in LDS.
//   2. Per class, the rows above the threshold are one ballot (two classes per ballot: 32 rows
//      each).  The chunk publishes its counts in status words of 64 bits: eight 6-bit counts and
//      the call's epoch, so that one load brings eight classes of an earlier chunk.
//   3. The write offset of the chunk for every class is the sum of the counts of the earlier
//      chunks: all threads read those words (several loads in flight per lane) and ask again,
//      together, for the ones that are not there yet.  Every poll loop is bounded: when a word does not show up within
//      spin_limit polls the workgroup computes the earlier chunks itself, so the kernel ends
//      whatever the order in which workgroups are started.  The last chunk tells the host the
//      totals as soon as it knows them (system-scope stores to pinned memory).
//   4. Kept rows go to their compacted places: the score, and the box as one 128-bit store.
// The arithmetic repeats the lowered programs operation for operation (fx_exp, fx_fmax, no
// contraction; the reductions in the order of the row-per-wave-segment softmax of the dense
// kernel), so the results are bit-identical to the generic kernels on the region split in two.
// Status words belong to the library (zero when allocated, never reset between calls: a word
// of an earlier call carries an older epoch).
#include <hip/hip_runtime.h>

#include <algorithm>

#include "fx_cmap.h"
#include "fx_device.h"

// a hook for timing the phases of a workgroup from a test program; nothing in the library
#ifndef FX_CMAP_STAMP
#define FX_CMAP_STAMP(k)
#endif

namespace {

#define FX_CMAP_DYN_OFF sizeof(FxCmapLaunch)
#define FX_CMAP_R 32u         // rows of a chunk
#define FX_CMAP_WIDE 512u     // threads of a workgroup: two rows per half-wave ...
#ifndef FX_CMAP_FIRST_LOOK_DELAY
#define FX_CMAP_FIRST_LOOK_DELAY 8   // units of 64 clocks between publishing the counts and reading the others'
#endif
#define FX_CMAP_NARROW 256u   // ... or four rows per half-wave, when the device cannot hold the wide launch at once

__device__ __forceinline__ uint64_t fxc_ptr(const FxCmapLaunch& hl, uint32_t slot, uint32_t task) {
  const uint8_t* ka = (const uint8_t*)__builtin_amdgcn_kernarg_segment_ptr();
  const uint64_t* gp = (const uint64_t*)(ka + FX_CMAP_DYN_OFF);
  const uint32_t pi = (slot & FX_SLOT_TASK) ? hl.n_sptr + task * hl.n_tptr + (slot & 0xffffu) : (slot & 0xffffu);
  return gp[pi];
}

template <uint32_t NT>
__global__ __launch_bounds__(NT) void fx_classmap_head(const FxCmapLaunch hl, const FxDyn) {
  // RPH rows per half-wave; U status words a lane asks for at once
  constexpr uint32_t R = FX_CMAP_R, RPH = R * 32u / NT, U = NT >= 512u ? 6u : 12u;
  extern __shared__ __attribute__((aligned(16))) float s_y[];   // R rows of CP floats: the softmax of the chunk
  __shared__ fx_u32x4 s_box[R];
  __shared__ uint32_t s_cnt[FX_CMAP_MAX_TASKS], s_prefix[FX_CMAP_MAX_TASKS];
  __shared__ uint32_t s_ok;
  __shared__ uint64_t s_sc[FX_CMAP_MAX_TASKS], s_bx[FX_CMAP_MAX_TASKS];   // where every task's scores and boxes go
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = uni(tid >> 6);
  const uint32_t b = blockIdx.x;
  const uint32_t C = hl.C, CP = C | 1u, T = hl.n_tasks, NG = (T + 7u) >> 3;
  const float thr = u2f(hl.thr_bits), var_xy = u2f(hl.var_xy_bits), var_wh = u2f(hl.var_wh_bits);
  const FX_AS1 float* conf = (const FX_AS1 float*)fxc_ptr(hl, hl.conf_slot, 0);
  const FX_AS1 float* loc = (const FX_AS1 float*)fxc_ptr(hl, hl.loc_slot, 0);
  const FX_AS1 float* pri = (const FX_AS1 float*)fxc_ptr(hl, hl.pri_slot, 0);
  uint64_t* status = (uint64_t*)hl.status;

  // ---- softmax (and boxes) of chunk cb into LDS; the counts per class into s_cnt.  With
  // `publish` the counts also go to the chunk's status words.
  auto compute_chunk = [&](uint32_t cb, bool boxes, bool publish) {
    const uint32_t r0 = cb * R, rows = min(R, hl.n_rows - r0);
    const uint32_t hw = tid >> 5, l = tid & 31u, c0 = l * 4u;
    float x[RPH][4];
#pragma unroll
    for (uint32_t k = 0; k < RPH; ++k) {
      const uint32_t row = hw + k * (NT / 32u);
      const FX_AS1 float* src = conf + (size_t)(r0 + row) * C + c0;
      if (row < rows && c0 + 3u < C) {
        const fx_u32x4_a4 v = *(const FX_AS1 fx_u32x4_a4*)src;
        x[k][0] = u2f(v.x); x[k][1] = u2f(v.y); x[k][2] = u2f(v.z); x[k][3] = u2f(v.w);
      } else {
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) x[k][j] = (row < rows && c0 + j < C) ? src[j] : 0.0f;
      }
    }
    fx_u32x4_a4 lv = {0u, 0u, 0u, 0u}, pv = {0u, 0u, 0u, 0u};
    if (boxes && tid < rows) {
      lv = *(const FX_AS1 fx_u32x4_a4*)(loc + (size_t)(r0 + tid) * 4u);
      pv = *(const FX_AS1 fx_u32x4_a4*)(pri + (size_t)(r0 + tid) * 4u);
    }
    // The argument segment lies in host memory: a load from it with an address that differs from
    // lane to lane costs a trip over the bus.  Every task's destinations are fetched once, behind
    // the loads of the scores (loads return in order), and parked in LDS after the softmax.
    uint64_t q_sc = 0, q_bx = 0;
    if (publish && tid < T) {
      q_sc = fxc_ptr(hl, hl.out_slot[0], tid);
      q_bx = fxc_ptr(hl, hl.out_slot[1], tid);
    }
    if (publish) FX_CMAP_STAMP(6);
    // The four rows of a half-wave go through every step together: their reductions are
    // independent, so four lane exchanges are in flight at a time instead of one.
    float m[RPH], v[RPH], e[RPH][4];
#pragma unroll
    for (uint32_t k = 0; k < RPH; ++k) {
      m[k] = -__builtin_inff();
#pragma unroll
      for (uint32_t j = 0; j < 4; ++j)
        if (c0 + j < C) m[k] = fx_fmax(m[k], x[k][j]);
    }
#define FX_CMAP_STEP(O)                                                              \
  {                                                                                  \
    float t[RPH];                                                                    \
    _Pragma("unroll") for (uint32_t k = 0; k < RPH; ++k) t[k] = fx_lane_xor_f<(O)>(m[k], lane); \
    _Pragma("unroll") for (uint32_t k = 0; k < RPH; ++k) m[k] = fx_fmax(m[k], t[k]); \
  }
    FX_CMAP_STEP(16u) FX_CMAP_STEP(8u) FX_CMAP_STEP(4u) FX_CMAP_STEP(2u) FX_CMAP_STEP(1u)
#undef FX_CMAP_STEP
#pragma unroll
    for (uint32_t k = 0; k < RPH; ++k) {
      v[k] = 0.0f;
#pragma unroll
      for (uint32_t j = 0; j < 4; ++j) {
        e[k][j] = fx_exp(x[k][j] - m[k]);
        if (c0 + j < C) v[k] = v[k] + e[k][j];
      }
    }
#define FX_CMAP_STEP(O)                                                              \
  {                                                                                  \
    float t[RPH];                                                                    \
    _Pragma("unroll") for (uint32_t k = 0; k < RPH; ++k) t[k] = fx_lane_xor_f<(O)>(v[k], lane); \
    _Pragma("unroll") for (uint32_t k = 0; k < RPH; ++k) v[k] = v[k] + t[k];         \
  }
    FX_CMAP_STEP(16u) FX_CMAP_STEP(8u) FX_CMAP_STEP(4u) FX_CMAP_STEP(2u) FX_CMAP_STEP(1u)
#undef FX_CMAP_STEP
#pragma unroll
    for (uint32_t k = 0; k < RPH; ++k) {
      const uint32_t row = hw + k * (NT / 32u);
      if (row < rows) {
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j)
          if (c0 + j < C) s_y[row * CP + c0 + j] = e[k][j] / v[k];
      }
    }
    if (boxes && tid < rows) {
      const float l0 = u2f(lv.x), l1 = u2f(lv.y), l2 = u2f(lv.z), l3 = u2f(lv.w);
      const float p0 = u2f(pv.x), p1 = u2f(pv.y), p2 = u2f(pv.z), p3 = u2f(pv.w);
      // half sizes (p * exp(l * var_wh)) / 2, centres p + (l * var_xy) * p_size
      const float hx = (p2 * fx_exp(l2 * var_wh)) / 2.0f, hy = (p3 * fx_exp(l3 * var_wh)) / 2.0f;
      const float cx = p0 + (l0 * var_xy) * p2, cy = p1 + (l1 * var_xy) * p3;
      fx_u32x4 ob;
      ob.x = f2u(cx - hx); ob.y = f2u(cy - hy); ob.z = f2u(cx + hx); ob.w = f2u(cy + hy);
      s_box[tid] = ob;
    }
    if (publish) FX_CMAP_STAMP(1);
    if (publish && tid < T) {
      s_sc[tid] = q_sc + (uint64_t)hl.out_tstride[0] * tid * 4u;
      s_bx[tid] = q_bx + (uint64_t)hl.out_tstride[1] * tid * 4u;
    }
    __syncthreads();
    // counts: a wave takes groups of eight classes, two classes per ballot
    const uint32_t row = lane & 31u, sub = lane >> 5;
    for (uint32_t g = wave; g < NG; g += NT / 64u) {
      uint64_t word = 0;
      float yk[4];
#pragma unroll
      for (uint32_t k = 0; k < 4; ++k) {
        const uint32_t t = g * 8u + k * 2u + sub;
        yk[k] = (t < T && row < rows) ? s_y[row * CP + hl.first + t] : -__builtin_inff();
      }
#pragma unroll
      for (uint32_t k = 0; k < 4; ++k) {
        const uint32_t t = g * 8u + k * 2u + sub;
        const bool keep = t < T && row < rows && yk[k] > thr;
        const uint64_t bal = __builtin_amdgcn_ballot_w64(keep);
        const uint32_t n0 = (uint32_t)__popc((uint32_t)bal), n1 = (uint32_t)__popc((uint32_t)(bal >> 32));
        word |= ((uint64_t)n0 << (12u * k)) | ((uint64_t)n1 << (12u * k + 6u));
        if (row == 0 && t < T) s_cnt[t] = sub ? n1 : n0;
      }
      if (publish && lane == 0)
        __hip_atomic_store(status + (size_t)cb * NG + g, ((uint64_t)hl.epoch << 48) | word, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
  };

  FX_CMAP_STAMP(0);
  if (tid < FX_CMAP_MAX_TASKS) s_prefix[tid] = 0u;
  if (tid == 0) s_ok = 1u;
  compute_chunk(b, true, true);
  FX_CMAP_STAMP(2);   // (its barrier also orders the stores above)

  // ---- look-back: thread (i0, g) sums the counts of classes 8g .. 8g+7 over chunks i0, i0 + rp, ...
  {
    const uint32_t g = tid % NG, i0 = tid / NG, rp = NT / NG;   // rp rows of status words side by side
    uint32_t acc[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
    bool ok = true;
    // a quarter of a microsecond before the first look: the neighbours publish at the same moment
    // as this chunk, and a look that leaves at once finds half of their words still old (10.2 ->
    // 9.5 us for 273 chunks; twice as long a pause gains nothing more, four times loses it again)
    if (b > 0) __builtin_amdgcn_s_sleep(FX_CMAP_FIRST_LOOK_DELAY);
    if (i0 < rp) {
      for (uint32_t ib = i0; ib < b && ok; ib += rp * U) {
        // The words of a batch are asked for together, and asked for again together as long as
        // some of them still carry an older epoch: workgroups run in step, so the first look
        // usually comes a moment before the neighbours' counts land.
        uint64_t w[U];
        uint32_t pending = 0, polls = 0;
#pragma unroll
        for (uint32_t u = 0; u < U; ++u)
          if (ib + u * rp < b) pending |= 1u << u;
        while (pending) {
#pragma unroll
          for (uint32_t u = 0; u < U; ++u)
            if ((pending >> u) & 1u)
              w[u] = __hip_atomic_load(status + (size_t)(ib + u * rp) * NG + g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
          for (uint32_t u = 0; u < U; ++u)
            if (((pending >> u) & 1u) && (uint32_t)(w[u] >> 48) == hl.epoch) {
              pending &= ~(1u << u);
#pragma unroll
              for (uint32_t k = 0; k < 8; ++k) acc[k] += (uint32_t)(w[u] >> (6u * k)) & 63u;
            }
          if (pending) {
            if (polls >= hl.spin_limit) { ok = false; break; }
            ++polls;
            __builtin_amdgcn_s_sleep(2);
          }
        }
      }
    }
    if (!ok) s_ok = 0u;
    if (i0 < rp && b > 0) {
#pragma unroll
      for (uint32_t k = 0; k < 8; ++k)
        if (acc[k] != 0u) atomicAdd(&s_prefix[g * 8u + k], acc[k]);   // (entries behind the last class stay unused)
    }
  }
  __syncthreads();
  FX_CMAP_STAMP(3);
  if (uni(s_ok) == 0u) {
    // an earlier chunk has not reported in time: compute the earlier chunks here
    __syncthreads();
    if (tid < FX_CMAP_MAX_TASKS) s_prefix[tid] = 0u;
    for (uint32_t cb = 0; cb < b; ++cb) {
      __syncthreads();   // s_y and s_cnt of the round before are no longer read
      compute_chunk(cb, false, false);
      __syncthreads();
      if (tid < T) s_prefix[tid] += s_cnt[tid];
    }
    __syncthreads();
    compute_chunk(b, true, false);
    __syncthreads();
  }
  // the totals, as soon as they are known
  if (b + 1u == hl.chunks && tid < T)
    __hip_atomic_store(hl.totals + tid, s_prefix[tid] + s_cnt[tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);

  FX_CMAP_STAMP(4);
  // ---- kept rows to their compacted places
  {
    const uint32_t rows = min(R, hl.n_rows - b * R);
    const uint32_t row = lane & 31u, sub = lane >> 5;
    const fx_u32x4 box = s_box[row];
    for (uint32_t g = wave; g < NG; g += NT / 64u) {
      // everything a class needs is read before the first store of the group is issued
      float yk[4];
      uint32_t pk[4];
      uint64_t sk[4], bk[4];
#pragma unroll
      for (uint32_t k = 0; k < 4; ++k) {
        const uint32_t t = min(g * 8u + k * 2u + sub, T - 1u);
        yk[k] = s_y[min(row, rows - 1u) * CP + hl.first + t];
        pk[k] = s_prefix[t];
        sk[k] = s_sc[t];
        bk[k] = s_bx[t];
      }
#pragma unroll
      for (uint32_t k = 0; k < 4; ++k) {
        const uint32_t t = g * 8u + k * 2u + sub;
        const bool keep = t < T && row < rows && yk[k] > thr;
        const uint64_t bal = __builtin_amdgcn_ballot_w64(keep);
        if (keep) {
          const uint32_t half = sub ? (uint32_t)(bal >> 32) : (uint32_t)bal;
          const uint32_t dst = pk[k] + (uint32_t)__popc(half & ((1u << row) - 1u));
          ((FX_AS1 float*)sk[k])[dst] = yk[k];
          *(FX_AS1 fx_u32x4_a4*)((FX_AS1 float*)bk[k] + (size_t)dst * 4u) = box;
        }
      }
    }
  }
  FX_CMAP_STAMP(5);
}

}  // namespace

uint32_t fx_cmap_lds_bytes(const FxCmapLaunch& hl) { return FX_CMAP_R * (hl.C | 1u) * 4u; }
uint32_t fx_cmap_chunk_rows() { return FX_CMAP_R; }

// Workgroups of the kernel that the current device holds at once: of the wide form, of the narrow form.
hipError_t fx_cmap_resident(uint32_t lds_bytes, uint32_t* wide, uint32_t* narrow) {
  int dev = 0, cus = 0, per_cu = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return e;
  e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)&fx_classmap_head<FX_CMAP_WIDE>, (int)FX_CMAP_WIDE,
                                                   (size_t)lds_bytes);
  if (e != hipSuccess) return e;
  *wide = (uint32_t)std::max(per_cu, 0) * (uint32_t)std::max(cus, 1);
  e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)&fx_classmap_head<FX_CMAP_NARROW>, (int)FX_CMAP_NARROW,
                                                   (size_t)lds_bytes);
  if (e != hipSuccess) return e;
  *narrow = (uint32_t)std::max(per_cu, 0) * (uint32_t)std::max(cus, 1);
  return hipSuccess;
}

hipError_t fx_launch_classmap_head(const FxCmapLaunch& hl, const FxDyn* dyn, bool wide, hipStream_t stream) {
  if (hl.chunks == 0) return hipSuccess;
  void* args[2] = {(void*)&hl, (void*)dyn};
  if (wide)
    return hipLaunchKernel((const void*)&fx_classmap_head<FX_CMAP_WIDE>, dim3(hl.chunks), dim3(FX_CMAP_WIDE), args,
                           fx_cmap_lds_bytes(hl), stream);
  return hipLaunchKernel((const void*)&fx_classmap_head<FX_CMAP_NARROW>, dim3(hl.chunks), dim3(FX_CMAP_NARROW), args,
                         fx_cmap_lds_bytes(hl), stream);
}
