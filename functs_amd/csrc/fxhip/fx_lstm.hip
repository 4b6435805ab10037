// Persistent stacked-LSTM kernel: the whole (time, layer) loop nest of
//   for t: cur = x[t]; for j: gates = cur @ Wih[j] + bih[j] + h[j] @ Whh[j] + bhh[j];
//          c[j] = f * c[j] + i * g; h[j] = o * tanh(c[j]); cur = h[j];  out[t] = cur
// (functs/benchmark/ai_model/lstm/lstm.py:79-133) as ONE launch.  The reference runs this loop on
// the host, one fused kernel and two library GEMMs per (t, j).
//
// A workgroup owns FX_LSTM_UPW hidden units, i.e. 4 * FX_LSTM_UPW gate columns of every layer's
// two weight matrices.  The inner dimension is split over its threads: thread k holds row k of
// those columns, for every layer, IN REGISTERS for the whole sequence (the 16.8 MB of weights of
// the benchmark configuration are read from memory once), and in every step it fetches element k
// of the step's vectors itself: x[t][k] and, per layer, element k of the h written in the step
// before.  Nothing is staged: the products stay in the thread, 16 partial sums a thread (two
// layers) are summed over the wave by a butterfly that halves the number of values as it doubles
// the lanes summed (lane-swap and data-parallel-primitive instructions, no LDS), the waves' sums
// meet in LDS behind the step's one barrier, and sixteen lanes of the first wave add the biases,
// apply the gates and update the cells; the cell state never leaves its lane.
// Steps are the diagonals t + j of the loop nest.  There is no barrier between workgroups: an h
// value travels with the tag of the step that wrote it and readers poll for the tag they expect
// (fx_lstm_sched.h), with bounded waits.
#include <hip/hip_runtime.h>

#define FX_LSTM_HD __host__ __device__
#include "../../../include/fxhip.h"
#include "fx_device.h"
#include "fx_lstm_sched.h"

#define FX_LSTM_BLOCK 256
#define FX_LSTM_MAXB 16
#define FX_LSTM_UPW 2   // hidden units per workgroup
#ifndef FX_LSTM_FIRST_LOOK
#define FX_LSTM_FIRST_LOOK 8   // units of 64 clocks; 7 to 10 are within 4 % of each other on the benchmark shape, 0 and 16 cost 40 and 8 %
#endif
// hooks for timing the phases of a step in a test build; nothing in the library
#ifndef FX_LSTM_STAMP
#define FX_LSTM_STAMP(k)
#define FX_LSTM_PSTAMP(k)
#define FX_LSTM_STAMP_END()
#define FX_LSTM_STAMP_DECL
#endif

namespace {
// Everything that crosses workgroups (the tagged h values, the control words) is written and read
// with device-scope atomic accesses, which go through to the memory side of the caches: no
// release / acquire fences, which on this device would write back and invalidate whole caches
// once per step.  A tagged value is one 64-bit store, so a reader never sees a value without
// its tag.
struct DevAtomics {
  static __device__ __forceinline__ uint32_t add(uint32_t* p) {
    return __hip_atomic_fetch_add(p, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  static __device__ __forceinline__ uint32_t load(uint32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  static __device__ __forceinline__ void store(uint32_t* p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  static __device__ __forceinline__ void store64(uint64_t* p, uint64_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
};

template <int CTRL>
__device__ __forceinline__ float dpp_get(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
// the value of lane K of the caller's group of four lanes
template <int K>
__device__ __forceinline__ float quad_lane(float v) { return dpp_get<K * 0x55>(v); }

typedef unsigned fx_u32x2v __attribute__((ext_vector_type(2)));
// Sixteen values a lane in, one out: lane l gets the sum over the wave of value l >> 2.  Every
// stage adds a value across two lanes that differ in one bit of the lane number and keeps only
// half of the values in each of them, so the work halves from stage to stage:
//   lanes l and l ^ 32 (the upper half keeps values 8-15), rows of 16 lanes r and r ^ 1 (odd rows
//   keep the upper half of what is left), lanes l and l ^ 8, lanes l and the mirrored lane of
//   their group of eight, and at last the four lanes of a group, which hold the same value.
__device__ __forceinline__ float wave_sum16(const float (&p)[16], int lane) {
  float q[8], r[4], s2[2];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const fx_u32x2v t = __builtin_amdgcn_permlane32_swap(__float_as_uint(p[i]), __float_as_uint(p[i + 8]), false, false);
    q[i] = __uint_as_float(t.x) + __uint_as_float(t.y);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const fx_u32x2v t = __builtin_amdgcn_permlane16_swap(__float_as_uint(q[i]), __float_as_uint(q[i + 4]), false, false);
    r[i] = __uint_as_float(t.x) + __uint_as_float(t.y);
  }
  const bool b3 = (lane & 8) != 0, b2 = (lane & 4) != 0;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const float keep = b3 ? r[i + 2] : r[i], send = b3 ? r[i] : r[i + 2];
    s2[i] = keep + dpp_get<0x128>(send);   // row_ror:8: from lane l ^ 8
  }
  const float keep = b2 ? s2[1] : s2[0], send = b2 ? s2[0] : s2[1];
  float v = keep + dpp_get<0x141>(send);   // row_half_mirror: from lane 7 - l of the group of eight
  v = v + dpp_get<0xB1>(v);                // quad_perm [1, 0, 3, 2]
  v = v + dpp_get<0x4E>(v);                // quad_perm [2, 3, 0, 1]
  return v;
}
}  // namespace

// 1024 hidden units (two elements a thread) are resident together only at four waves per SIMD,
// i.e. within 128 registers a lane; the smaller sizes need two
template <int L, int HPT, int UPW>
__global__ __launch_bounds__(FX_LSTM_BLOCK * UPW, HPT >= 32 ? 4 : 2) void fx_lstm_stack_kernel(const FxLstmArgs a) {
  static_assert(UPW == 2, "the butterfly sums 16 values: two layers of four gates of two units");
  constexpr int NT = FX_LSTM_BLOCK * UPW;                             // threads
  constexpr int NW = NT / 64;                                         // waves
  constexpr int HH = HPT * 32;                                        // H
  constexpr int EPT = (HH + NT - 1) / NT;                             // rows of the weights per thread
  constexpr int NG = (L + 1) / 2;                                     // pairs of layers: 16 values each
  __shared__ float s_part[2][NG][NW][16];   // the waves' sums, by parity of the (step, batch row) pair: read behind the
                                            // pair's barrier, written again two barriers later
  __shared__ float s_c[FX_LSTM_MAXB][64];   // cell states: [batch row][owner lane]
  __shared__ uint32_t s_abort;
  FX_LSTM_STAMP_DECL
  const int H = a.H, B = a.B, T = a.T;
  const int tid = (int)threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  FX_LSTM_PSTAMP(0);
  // Workgroups go to the chip's eight dies in turn, and every die has a cache of its own: the
  // workgroups of a die take neighbouring hidden units, so that a die fetches its eighth of every
  // weight row once (lines of a row are shared by 32 units) instead of every die fetching all of it.
  const int n_wg = (int)gridDim.x;
  const int wg = (n_wg % 8 == 0) ? ((int)blockIdx.x % 8) * (n_wg / 8) + (int)blockIdx.x / 8 : (int)blockIdx.x;
  const int u0 = wg * UPW;
  // a workspace that still carries a given-up wait is refused (below, behind the first barrier)
  if (tid == 0) s_abort = fx_lstm_refused<DevAtomics>(a.ctl) ? 1u : 0u;
  // tags of this launch start behind those of every launch before it
  const uint32_t base = DevAtomics::load(a.ctl + FX_LSTM_W_BASE);

  // rows k = tid + e * NT of the workgroup's columns: [layer][gate][unit], input and recurrent matrix
  float w_ih[L][4][UPW][EPT], w_hh[L][4][UPW][EPT];
#pragma unroll
  for (int j = 0; j < L; ++j)
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
      for (int e = 0; e < EPT; ++e) {
        const int k = tid + e * NT;
        float2 wi = make_float2(0.0f, 0.0f), wh = wi;
        if (k < HH) {
          const size_t at = ((size_t)(j * 4 + g) * H + k) * H + u0;   // u0 is even: 8-byte aligned
          wi = *(const float2*)(a.wih + at);
          wh = *(const float2*)(a.whh + at);
        }
        w_ih[j][g][0][e] = wi.x; w_ih[j][g][1][e] = wi.y;
        w_hh[j][g][0][e] = wh.x; w_hh[j][g][1][e] = wh.y;
      }
  // Lane 4 * v + gate of the first wave ends up with the gate sum of value v = (layer in its pair,
  // unit) of every pair of layers; the lane of gate 0 owns the cell.
  const int f_v = lane >> 2, f_gate = lane & 3, f_ul = f_v & 1, f_jl = f_v >> 1;
  float f_bias_ih[NG], f_bias_hh[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const int j = 2 * g + f_jl;
    const bool live = wave == 0 && lane < 16 && j < L;
    f_bias_ih[g] = live ? a.bih[(size_t)(j * 4 + f_gate) * H + u0 + f_ul] : 0.0f;
    f_bias_hh[g] = live ? a.bhh[(size_t)(j * 4 + f_gate) * H + u0 + f_ul] : 0.0f;
  }
  if (wave == 0) {
    for (int b = 0; b < B; ++b) {
      float c = 0.0f;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        // one lane owns at most one cell per pair of layers; with two pairs the second pair's cells
        // live in lanes 16-31
        const int j = 2 * g + ((lane & 15) >> 3), ul = ((lane & 15) >> 2) & 1;
        if ((lane >> 4) == g && (lane & 3) == 0 && j < L && a.c0) c = a.c0[((size_t)j * B + b) * H + u0 + ul];
      }
      s_c[b][lane] = c;
    }
  }
  __syncthreads();
  if (s_abort != 0u) {   // uniform: written once, ahead of the barrier
    if (tid == 0 && a.err_host) __hip_atomic_store(a.err_host, (uint32_t)FX_ASYNC_BARRIER, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    fx_lstm_poison(a, L, (uint32_t)tid, (uint32_t)NT);
    return;
  }
  FX_LSTM_PSTAMP(1);

  const int n_steps = fx_lstm_steps(T, L);
  // x of the next (step, batch row) is asked for at the top of a step, ahead of the polls, and is
  // in its register long before it is used
  float x_cur[EPT], x_next[EPT];
  auto fetch_x = [&](int d, int b, float (&dst)[EPT]) {
    const int t0 = (d < n_steps) ? fx_lstm_time(d, 0, T) : -1;
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int k = tid + e * NT;
      dst[e] = (t0 >= 0 && k < HH) ? a.x[((size_t)t0 * B + b) * H + k] : 0.0f;
    }
  };
  fetch_x(0, 0, x_cur);
  int it = 0;   // (step, batch row) pairs so far: its parity picks the buffer of the waves' sums
  for (int d = 0; d < n_steps; ++d) {
    const int rp = (d + 1) & 1;   // parity written by step d - 1
    const uint32_t want = fx_lstm_tag_read(base, d);
    for (int b = 0; b < B; ++b) {
      FX_LSTM_STAMP(0);
      if (b + 1 < B) fetch_x(d, b + 1, x_next);
      else fetch_x(d + 1, 0, x_next);
      // --- element k of what every layer wrote in the step before ---
      // hv[j]: what layer j reads as its own previous h, which is also what layer j + 1 reads as its
      // input: h0[j] at the layer's first step (not tagged), else the h that layer j wrote in step
      // d - 1 (tagged).  A slot that is not tagged or not needed is loaded all the same (and ignored):
      // the loads of a round are then issued together, without a branch and a wait between them, and
      // a round takes one trip to the memory side instead of one per layer.
      bool need[L];
      float hv[L][EPT] = {};
      const uint64_t* src[L];
#pragma unroll
      for (int j = 0; j < L; ++j) {
        const int tj = fx_lstm_time(d, j, T);
        const bool next_active = j + 1 < L && fx_lstm_time(d, j + 1, T) >= 0;
        need[j] = tj != 0 && (tj > 0 || next_active);
        src[j] = a.hbuf + fx_lstm_hoff(rp, j, b, 0, L, B, H);
        if (tj == 0) {
          const float* hr = a.h0 ? a.h0 + ((size_t)j * B + b) * H : nullptr;
#pragma unroll
          for (int e = 0; e < EPT; ++e) hv[j][e] = (hr && tid + e * NT < HH) ? hr[tid + e * NT] : 0.0f;
        }
      }
      {
        uint32_t polls = 0;
        // the waves that are not busy with the cells arrive here while the owners still write: looking
        // at once would only add reads of the very lines the writes are on their way to
        __builtin_amdgcn_s_sleep(FX_LSTM_FIRST_LOOK);
        for (;;) {
          bool ready = true;
          uint64_t el[L][EPT];
#pragma unroll
          for (int j = 0; j < L; ++j)
#pragma unroll
            for (int e = 0; e < EPT; ++e)
              el[j][e] = __hip_atomic_load(src[j] + min(tid + e * NT, HH - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
          for (int j = 0; j < L; ++j)
#pragma unroll
            for (int e = 0; e < EPT; ++e) {
              ready = ready && (!need[j] || tid + e * NT >= HH || fx_lstm_tag_of(el[j][e]) == want);
              if (need[j]) hv[j][e] = (tid + e * NT < HH) ? __uint_as_float((uint32_t)el[j][e]) : 0.0f;
            }
          if (ready) break;
          if (++polls > a.spin_limit || ((polls & 255u) == 0u && DevAtomics::load(a.ctl + FX_LSTM_W_ERR) != 0u)) {
            // given up (or somebody else has): the workgroup leaves behind this step's barrier
            DevAtomics::store(a.ctl + FX_LSTM_W_ERR, 1u);
            if (a.err_host) __hip_atomic_store(a.err_host, (uint32_t)FX_ASYNC_BARRIER, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            s_abort = 1u;
            break;
          }
          __builtin_amdgcn_s_sleep(1);
        }
      }
      FX_LSTM_STAMP(2);
      // --- this thread's share of every gate sum, and the sums over the wave ---
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        float p[16];   // value (jl * 2 + ul) * 4 + gate
#pragma unroll
        for (int jl = 0; jl < 2; ++jl) {
          const int j = 2 * g + jl;
          const bool active = j < L && fx_lstm_time(d, j < L ? j : 0, T) >= 0;
#pragma unroll
          for (int ul = 0; ul < UPW; ++ul)
#pragma unroll
            for (int gt = 0; gt < 4; ++gt) {
              float s = 0.0f;
              if (j < L) {
#pragma unroll
                for (int e = 0; e < EPT; ++e) {
                  const float in = (j == 0) ? x_cur[e] : hv[j > 0 ? j - 1 : 0][e];
                  s = __builtin_fmaf(w_ih[j < L ? j : 0][gt][ul][e], in, s);
                  s = __builtin_fmaf(w_hh[j < L ? j : 0][gt][ul][e], hv[j < L ? j : 0][e], s);
                }
              }
              p[(jl * 2 + ul) * 4 + gt] = active ? s : 0.0f;
            }
        }
        const float total = wave_sum16(p, lane);   // lane l: the wave's sum of value l >> 2
        if ((lane & 3) == 0) s_part[it & 1][g][wave][lane >> 2] = total;
      }
      FX_LSTM_STAMP(4);
      // the cell states of this batch row, read ahead of the barrier (a lane reads what it wrote itself)
      float c_prev[NG];
#pragma unroll
      for (int g = 0; g < NG; ++g) c_prev[g] = wave == 0 ? s_c[b][(lane & 15) + 16 * g] : 0.0f;
      __syncthreads();
      FX_LSTM_STAMP(5);
      // A wait that was given up: every wave of the workgroup leaves, nothing is checked out.  The
      // first wave looks at the word together with the waves' sums and leaves before it would store.
      if (wave != 0) {
        if (s_abort != 0u) {   // the results are not to be used: the waves without cells say so in the data
          fx_lstm_poison(a, L, (uint32_t)(tid - 64), (uint32_t)(NT - 64));
          return;
        }
      } else {
        // --- sixteen lanes a pair of layers: biases, gates, cells ---
        float part[NG][NW];
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
          for (int w = 0; w < NW; ++w) part[g][w] = s_part[it & 1][g][w][lane & 15];
        const uint32_t aborted = s_abort;
#pragma unroll
        for (int g = 0; g < NG; ++g) {
#pragma unroll
          for (int span = 1; span < NW; span *= 2)
#pragma unroll
            for (int w = 0; w + span < NW; w += 2 * span) part[g][w] += part[g][w + span];
          // the value of a lane here is lane & 15 = (layer in the pair * 2 + unit) * 4 + gate, as for the biases
          const int v = lane & 15, gt = v & 3, ul = (v >> 2) & 1, j = 2 * g + (v >> 3);
          const float pre = (part[g][0] + f_bias_ih[g]) + f_bias_hh[g];
          const float act = gt == 2 ? fx_tanh(pre) : fx_sigmoid(pre);
          const float fg = quad_lane<1>(act), gg = quad_lane<2>(act), og = quad_lane<3>(act);
          const int t = (j < L) ? fx_lstm_time(d, j, T) : -1;
          if (g == 0 && aborted != 0u) return;
          if (lane < 16 && gt == 0 && t >= 0) {
            const float c = (fg * c_prev[g]) + (act * gg);
            s_c[b][lane + 16 * g] = c;
            const float h = og * fx_tanh(c);
            const int u = u0 + ul;
            DevAtomics::store64(a.hbuf + fx_lstm_hoff(d & 1, j, b, u, L, B, H),
                                fx_lstm_pack(__float_as_uint(h), fx_lstm_tag_written(base, d)));
            if (j == L - 1) a.out[((size_t)t * B + b) * H + u] = h;
            if (t == T - 1) {
              a.state_h[((size_t)j * B + b) * H + u] = h;
              a.state_c[((size_t)j * B + b) * H + u] = c;
            }
          }
        }
      }
      FX_LSTM_STAMP(6);
#pragma unroll
      for (int e = 0; e < EPT; ++e) x_cur[e] = x_next[e];
      ++it;
    }
  }
  FX_LSTM_STAMP_END();
  if (threadIdx.x == 0)
    fx_lstm_leave<DevAtomics>(a.ctl, gridDim.x, base, (uint32_t)n_steps, a.hbuf, (uint32_t)(2 * L * B * H));
}

typedef void (*fx_lstm_kernel_t)(const FxLstmArgs);
template <int L, int UPW>
static fx_lstm_kernel_t pick_hpt(int hpt) {
  switch (hpt) {
    case 1: return fx_lstm_stack_kernel<L, 1, UPW>;
    case 2: return fx_lstm_stack_kernel<L, 2, UPW>;
    case 4: return fx_lstm_stack_kernel<L, 4, UPW>;
    case 8: return fx_lstm_stack_kernel<L, 8, UPW>;
    case 16: return fx_lstm_stack_kernel<L, 16, UPW>;
    case 32: return fx_lstm_stack_kernel<L, 32, UPW>;
    default: return nullptr;
  }
}
template <int UPW>
static fx_lstm_kernel_t pick_layers(int L, int hpt) {
  switch (L) {
    case 1: return pick_hpt<1, UPW>(hpt);
    case 2: return pick_hpt<2, UPW>(hpt);
    case 3: return pick_hpt<3, UPW>(hpt);
    case 4: return pick_hpt<4, UPW>(hpt);
    default: return nullptr;
  }
}

// 0: launched; 1: shape outside what the kernel is built for; 2: the grid would not be resident
// all at once (every workgroup waits for values that all the others write); otherwise a HIP error code + 100.
int fx_launch_lstm_stack(const FxLstmArgs& a, int L, hipStream_t stream) {
  if (a.H < 32 || a.H % 32 != 0 || a.B < 1 || a.B > FX_LSTM_MAXB || L * a.B > FX_LSTM_BLOCK) return 1;
  // two hidden units per workgroup: every workgroup fetches the step's vectors from the memory
  // side once, so fewer, larger workgroups fetch less, and sixteen gate sums fill the butterfly
  constexpr int upw = FX_LSTM_UPW;
  fx_lstm_kernel_t k = pick_layers<FX_LSTM_UPW>(L, a.H / 32);
  if (!k) return 1;
  int dev = 0, per_cu = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  const size_t lds = 0;
  const int threads = FX_LSTM_BLOCK * upw, grid = a.H / upw;
  if (e == hipSuccess) e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)k, threads, lds);
  if (e != hipSuccess) return 100 + (int)e;
  if ((long)per_cu * cus < grid) return 2;
  void* args[1] = {(void*)&a};
  e = hipLaunchKernel((const void*)k, dim3((uint32_t)grid), dim3((uint32_t)threads), args, lds, stream);
  return e == hipSuccess ? 0 : 100 + (int)e;
}
