// Persistent stacked-LSTM kernel: the whole (time, layer) loop nest of
//   for t: cur = x[t]; for j: gates = cur @ Wih[j] + bih[j] + h[j] @ Whh[j] + bhh[j];
//          c[j] = f * c[j] + i * g; h[j] = o * tanh(c[j]); cur = h[j];  out[t] = cur
// (functs/benchmark/ai_model/lstm/lstm.py:79-133) as ONE launch.  The reference runs this loop on
// the host, one fused kernel and two library GEMMs per (t, j).
//
// One workgroup per hidden unit u.  Its 4 waves are the 4 gates (i, f, g, o); in a wave, lanes
// 0-31 hold column u of Wih[j][gate] and lanes 32-63 column u of Whh[j][gate] for every layer j,
// H / 32 elements per lane, IN REGISTERS for the whole sequence: the 16.8 MB of weights of the
// benchmark configuration are read from memory once.  A step reads the input vectors (x[t] and
// the h of the previous step, a few KB that every workgroup shares), does H / 32 fused
// multiply-adds per lane and layer, reduces over the half wave, and one thread per (layer, batch
// row) applies the gates; the cell state never leaves its register.  The workgroup fetches the
// vectors once into LDS for its four waves: coherent reads bypass the caches, so what a step
// costs is above all how often the same few KB are fetched from the memory side.  Steps are the diagonals
// t + j of the loop nest.  There is no barrier between them: an h value travels with the tag of
// the step that wrote it and readers poll for the tag they expect (fx_lstm_sched.h), with bounded
// waits.
#include <hip/hip_runtime.h>

#define FX_LSTM_HD __host__ __device__
#include "../../../include/fxhip.h"
#include "fx_device.h"
#include "fx_lstm_sched.h"

#define FX_LSTM_BLOCK 256
#define FX_LSTM_MAXB 16
#define FX_LSTM_UPW 2   // hidden units per workgroup
#ifndef FX_LSTM_FIRST_LOOK
#define FX_LSTM_FIRST_LOOK 8
#endif
// hooks for timing the phases of a step in a test build; nothing in the library
#ifndef FX_LSTM_STAMP
#define FX_LSTM_STAMP(k)
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
__device__ __forceinline__ float dpp_add(float v) {
  return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
// every lane gets the sum over its row of 16 lanes: neighbours, pairs, then the mirrored half rows and rows
__device__ __forceinline__ float row_sum(float v) {
  v = dpp_add<0xB1>(v);    // quad_perm [1, 0, 3, 2]
  v = dpp_add<0x4E>(v);    // quad_perm [2, 3, 0, 1]
  v = dpp_add<0x141>(v);   // row_half_mirror
  v = dpp_add<0x140>(v);   // row_mirror
  return v;
}
__device__ __forceinline__ float lane_value(float v, int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l)); }
}  // namespace

// 1024 workgroups (HPT = 32) are resident together only at four waves per SIMD, i.e. within 128
// registers a lane; the smaller sizes need two
template <int L, int HPT, int UPW>
__global__ __launch_bounds__(FX_LSTM_BLOCK * UPW, HPT >= 32 ? 4 : 2) void fx_lstm_stack_kernel(const FxLstmArgs a) {
  // the input vectors of one batch row of a step: x[t] and, per layer, the h it reads
  extern __shared__ __attribute__((aligned(16))) float s_vec[];   // [L + 1][H]
  __shared__ float s_gate[2][UPW][L][FX_LSTM_MAXB][4];   // activated gates, by parity of the step
  __shared__ uint32_t s_abort;
  FX_LSTM_STAMP_DECL
  constexpr int NT = FX_LSTM_BLOCK * UPW;                             // threads: four waves per hidden unit
  constexpr int HH = HPT * 32;                                        // H
  constexpr int EPT = (HH + NT - 1) / NT;                             // elements of a vector per thread
  const int H = a.H, B = a.B, T = a.T;
  const int tid = (int)threadIdx.x;
  const int ul = tid / FX_LSTM_BLOCK;                                 // which of the workgroup's units
  // Workgroups go to the chip's eight dies in turn, and every die has a cache of its own: the
  // workgroups of a die take neighbouring hidden units, so that a die fetches its eighth of every
  // weight row once (lines of a row are shared by 32 units) instead of every die fetching all of it.
  const int n_wg = (int)gridDim.x;
  const int wg = (n_wg % 8 == 0) ? ((int)blockIdx.x % 8) * (n_wg / 8) + (int)blockIdx.x / 8 : (int)blockIdx.x;
  const int u = wg * UPW + ul;
  const int lane = (int)(threadIdx.x & 63u), gate = (int)((threadIdx.x >> 6) & 3u);
  const int half = lane >> 5, sub = lane & 31;
  if (threadIdx.x == 0) s_abort = 0u;
  // tags of this launch start behind those of every launch before it
  const uint32_t base = DevAtomics::load(a.ctl + FX_LSTM_W_BASE);

  // this lane's slice of the weights, and the biases of (layer, gate, unit)
  float w[L][HPT];
  float b_ih[L], b_hh[L];
#pragma unroll
  for (int j = 0; j < L; ++j) {
    const float* W = (half ? a.whh : a.wih) + ((size_t)(j * 4 + gate) * H) * H + u;
#pragma unroll
    for (int m = 0; m < HPT; ++m) w[j][m] = W[(size_t)(sub + 32 * m) * H];
    b_ih[j] = a.bih[(size_t)(j * 4 + gate) * H + u];
    b_hh[j] = a.bhh[(size_t)(j * 4 + gate) * H + u];
  }
  // thread (j, b) of a unit's four waves owns the cell state of its layer and batch row
  const int own_j = (tid % FX_LSTM_BLOCK) / B, own_b = (tid % FX_LSTM_BLOCK) % B;
  const bool owner = own_j < L;
  float c_reg = (owner && a.c0) ? a.c0[((size_t)own_j * B + own_b) * H + u] : 0.0f;
  __syncthreads();

  const int n_steps = fx_lstm_steps(T, L);
  for (int d = 0; d < n_steps; ++d) {
    const int rp = (d + 1) & 1;   // parity written by step d - 1
    const uint32_t want = fx_lstm_tag_read(base, d);
    FX_LSTM_STAMP(0);
    for (int b = 0; b < B; ++b) {
      // --- the workgroup fetches the vectors of a batch row once, for all its waves ---
      // slot 0: x[t] (layer 0 active); slot j + 1: what layer j reads as its own previous h, which
      // is also what layer j + 1 reads as its input: h0[j] at the layer's first step (not tagged),
      // else the h that layer j wrote in step d - 1 (tagged).
      {
        const int t0 = fx_lstm_time(d, 0, T);
        if (t0 >= 0) {
          const float* xr = a.x + ((size_t)t0 * B + b) * H;
#pragma unroll
          for (int k = 0; k < EPT; ++k)
            if (tid + k * NT < HH) s_vec[tid + k * NT] = xr[tid + k * NT];
        }
      }
      FX_LSTM_STAMP(1);
      // tagged sources of this step.  A slot that is not tagged or not needed is loaded all the same
      // (and ignored): the loads of a round are then issued together, without a branch and a wait
      // between them, and a round takes one trip to the memory side instead of one per layer.
      bool need[L];
      const uint64_t* src[L];
#pragma unroll
      for (int j = 0; j < L; ++j) {
        const int tj = fx_lstm_time(d, j, T);
        const bool next_active = j + 1 < L && fx_lstm_time(d, j + 1, T) >= 0;
        need[j] = false;
        src[j] = a.hbuf + fx_lstm_hoff(rp, j, b, 0, L, B, H);
        if (tj == 0) {
          const float* hr = a.h0 ? a.h0 + ((size_t)j * B + b) * H : nullptr;
#pragma unroll
          for (int k = 0; k < EPT; ++k)
            if (tid + k * NT < HH) s_vec[(j + 1) * HH + tid + k * NT] = hr ? hr[tid + k * NT] : 0.0f;
        } else if (tj > 0 || next_active) {
          need[j] = true;
        }
      }
      {
        float val[L][EPT];
        uint32_t polls = 0;
        __builtin_amdgcn_s_sleep(FX_LSTM_FIRST_LOOK);
        for (;;) {
          bool ready = true;
          uint64_t e[L][EPT];
#pragma unroll
          for (int j = 0; j < L; ++j)
#pragma unroll
            for (int k = 0; k < EPT; ++k)
              e[j][k] = __hip_atomic_load(src[j] + min(tid + k * NT, HH - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
          for (int j = 0; j < L; ++j)
#pragma unroll
            for (int k = 0; k < EPT; ++k) {
              ready = ready && (!need[j] || tid + k * NT >= HH || fx_lstm_tag_of(e[j][k]) == want);
              val[j][k] = __uint_as_float((uint32_t)e[j][k]);
            }
          if (ready) break;
          if (++polls > a.spin_limit || ((polls & 255u) == 0u && DevAtomics::load(a.ctl + FX_LSTM_W_ERR) != 0u)) {
            // given up (or somebody else has): the workgroup leaves at the end of this step's reads
            DevAtomics::store(a.ctl + FX_LSTM_W_ERR, 1u);
            if (a.err_host) __hip_atomic_store(a.err_host, (uint32_t)FX_ASYNC_BARRIER, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            s_abort = 1u;
            break;
          }
          __builtin_amdgcn_s_sleep(1);
        }
        FX_LSTM_STAMP(2);
#pragma unroll
        for (int j = 0; j < L; ++j) {
          if (!need[j]) continue;
#pragma unroll
          for (int k = 0; k < EPT; ++k)
            if (tid + k * NT < HH) s_vec[(j + 1) * HH + tid + k * NT] = val[j][k];
        }
      }
      __syncthreads();
      FX_LSTM_STAMP(3);
      // --- dot products: lanes 0-31 the layer's input, lanes 32-63 its own previous h ---
#pragma unroll
      for (int j = 0; j < L; ++j) {
        if (fx_lstm_time(d, j, T) < 0) continue;
        const float* vsrc = s_vec + (half == 0 ? j : j + 1) * HH;
        float s = 0.0f;
#pragma unroll
        for (int m = 0; m < HPT; ++m) s = __builtin_fmaf(w[j][m], vsrc[sub + 32 * m], s);
        // sums over the rows of 16 lanes inside the vector unit, then the four row sums through
        // scalar registers: lanes 0-31 are the input's half, lanes 32-63 the half of the own h
        s = row_sum(s);
        const float ih = lane_value(s, 0) + lane_value(s, 16);
        const float hh = lane_value(s, 32) + lane_value(s, 48);
        const float g = (ih + b_ih[j]) + (hh + b_hh[j]);
        // every gate's wave applies its own activation; the owner is left with the cell update
        if (lane == 0) s_gate[d & 1][ul][j][b][gate] = gate == 2 ? fx_tanh(g) : fx_sigmoid(g);
      }
      FX_LSTM_STAMP(4);
      __syncthreads();   // the vectors are overwritten by the next batch row; the gates are complete
      FX_LSTM_STAMP(5);
    }
    if (s_abort != 0u) return;   // a wait was given up: every wave of the workgroup leaves, nothing is checked out
    if (owner) {
      const int t = fx_lstm_time(d, own_j, T);
      if (t >= 0) {
        const float* gt = s_gate[d & 1][ul][own_j][own_b];
        const float ig = gt[0], fg = gt[1], gg = gt[2], og = gt[3];
        c_reg = (fg * c_reg) + (ig * gg);
        const float h = og * fx_tanh(c_reg);
        DevAtomics::store64(a.hbuf + fx_lstm_hoff(d & 1, own_j, own_b, u, L, B, H),
                            fx_lstm_pack(__float_as_uint(h), fx_lstm_tag_written(base, d)));
        if (own_j == L - 1) a.out[((size_t)t * B + own_b) * H + u] = h;
        if (t == T - 1) {
          a.state_h[((size_t)own_j * B + own_b) * H + u] = h;
          a.state_c[((size_t)own_j * B + own_b) * H + u] = c_reg;
        }
      }
    }
    // no barrier here: the next step writes the gates of the other parity, and the one after it
    // comes behind two barriers that the owners pass only after they have read these
    FX_LSTM_STAMP(6);
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
  // hidden units per workgroup: every workgroup fetches the step's vectors from the memory side
  // once, so fewer, larger workgroups fetch less
  // (measured on the benchmark shape: 248 us with one unit per workgroup, 223 with two, 291 with four)
  constexpr int upw = FX_LSTM_UPW;
  fx_lstm_kernel_t k = pick_layers<FX_LSTM_UPW>(L, a.H / 32);
  if (!k) return 1;
  int dev = 0, per_cu = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  const size_t lds = (size_t)(L + 1) * a.H * sizeof(float);   // the staged vectors
  const int threads = FX_LSTM_BLOCK * upw, grid = a.H / upw;
  if (e == hipSuccess) e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)k, threads, lds);
  if (e != hipSuccess) return 100 + (int)e;
  if ((long)per_cu * cus < grid) return 2;
  void* args[1] = {(void*)&a};
  e = hipLaunchKernel((const void*)k, dim3((uint32_t)grid), dim3((uint32_t)threads), args, lds, stream);
  return e == hipSuccess ? 0 : 100 + (int)e;
}
