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
// the h of the previous step, a few KB that every workgroup shares) from L2, does H / 32 fused
// multiply-adds per lane and layer, reduces over the half wave, and one thread per (layer, batch
// row) applies the gates; the cell state never leaves its register.  Steps are the diagonals
// t + j of the loop nest, separated by a device-wide barrier (fx_lstm_sched.h) whose waits are
// bounded.
#include <hip/hip_runtime.h>

#define FX_LSTM_HD __host__ __device__
#include "fx_device.h"
#include "fx_lstm_sched.h"

#define FX_LSTM_BLOCK 256
#define FX_LSTM_MAXB 16

namespace {
// Every value that crosses the barrier (the h vectors) is written and read with device-scope
// atomic accesses, which go through to the memory side of the caches, and a workgroup arrives only
// after its stores have been acknowledged (the wait in front of the barrier below).  The
// counters therefore need no release / acquire fences of their own, which on this device would
// write back and invalidate whole caches once per step.
struct DevAtomics {
  static __device__ __forceinline__ uint32_t add_release(uint32_t* p) {
    return __hip_atomic_fetch_add(p, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  static __device__ __forceinline__ uint32_t load(uint32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  static __device__ __forceinline__ void store(uint32_t* p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  static __device__ __forceinline__ void acquire() {}
  static __device__ __forceinline__ void pause() { __builtin_amdgcn_s_sleep(2); }
};
}  // namespace

template <int L, int HPT>
__global__ __launch_bounds__(FX_LSTM_BLOCK) void fx_lstm_stack_kernel(const FxLstmArgs a) {
  __shared__ float s_gate[L][FX_LSTM_MAXB][4];
  __shared__ uint32_t s_go;
  const int H = a.H, B = a.B, T = a.T;
  const int u = (int)blockIdx.x;
  const int lane = (int)(threadIdx.x & 63u), gate = (int)(threadIdx.x >> 6);
  const int half = lane >> 5, sub = lane & 31;

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
  // thread (j, b) owns the cell state of its layer and batch row
  const int own_j = (int)threadIdx.x / B, own_b = (int)threadIdx.x % B;
  const bool owner = own_j < L;
  float c_reg = (owner && a.c0) ? a.c0[((size_t)own_j * B + own_b) * H + u] : 0.0f;

  const int n_steps = fx_lstm_steps(T, L);
  for (int d = 0; d < n_steps; ++d) {
    const int rp = (d + 1) & 1;   // parity written by step d - 1
#pragma unroll
    for (int j = 0; j < L; ++j) {
      const int t = fx_lstm_time(d, j, T);
      if (t < 0) continue;
      for (int b = 0; b < B; ++b) {
        const float* src;   // null: zeros (no initial state given)
        bool coherent;      // written by other workgroups during this launch
        if (half == 0) {
          if (j == 0) { src = a.x + ((size_t)t * B + b) * H; coherent = false; }
          else { src = a.hbuf + fx_lstm_hoff(rp, j - 1, b, 0, L, B, H); coherent = true; }
        } else {
          if (t == 0) { src = a.h0 ? a.h0 + ((size_t)j * B + b) * H : nullptr; coherent = false; }
          else { src = a.hbuf + fx_lstm_hoff(rp, j, b, 0, L, B, H); coherent = true; }
        }
        float v[HPT];
#pragma unroll
        for (int m = 0; m < HPT; ++m)
          v[m] = coherent ? __hip_atomic_load(src + sub + 32 * m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                          : (src ? src[sub + 32 * m] : 0.0f);
        float s = 0.0f;
#pragma unroll
        for (int m = 0; m < HPT; ++m) s = __builtin_fmaf(w[j][m], v[m], s);
#pragma unroll
        for (int o = 16; o >= 1; o >>= 1) s += __shfl_xor(s, o, 64);
        const float other = __shfl(s, 32, 64);   // the hh half's sum, for lane 0
        if (lane == 0) s_gate[j][b][gate] = (s + b_ih[j]) + (other + b_hh[j]);
      }
    }
    __syncthreads();
    if (owner) {
      const int t = fx_lstm_time(d, own_j, T);
      if (t >= 0) {
        const float ig = fx_sigmoid(s_gate[own_j][own_b][0]);
        const float fg = fx_sigmoid(s_gate[own_j][own_b][1]);
        const float gg = fx_tanh(s_gate[own_j][own_b][2]);
        const float og = fx_sigmoid(s_gate[own_j][own_b][3]);
        c_reg = (fg * c_reg) + (ig * gg);
        const float h = og * fx_tanh(c_reg);
        __hip_atomic_store(a.hbuf + fx_lstm_hoff(d & 1, own_j, own_b, u, L, B, H), h, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
        if (own_j == L - 1) a.out[((size_t)t * B + own_b) * H + u] = h;
        if (t == T - 1) {
          a.state_h[((size_t)own_j * B + own_b) * H + u] = h;
          a.state_c[((size_t)own_j * B + own_b) * H + u] = c_reg;
        }
      }
    }
    if (d + 1 < n_steps) {
      __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this thread's h store has been acknowledged
      __syncthreads();   // the gates have been read, h has been stored by this workgroup's owners
      if (threadIdx.x == 0) {
        const bool ok = fx_lstm_barrier<DevAtomics>(a.bar, (uint32_t)(d + 1), blockIdx.x, gridDim.x, a.spin_limit);
        if (!ok && a.err_host) __hip_atomic_store(a.err_host, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        s_go = ok ? 1u : 0u;
      }
      __syncthreads();
      if (s_go == 0u) return;   // a wait was given up somewhere: every workgroup leaves
    }
  }
  if (threadIdx.x == 0) fx_lstm_leave<DevAtomics>(a.bar, gridDim.x);
}

typedef void (*fx_lstm_kernel_t)(const FxLstmArgs);
template <int L>
static fx_lstm_kernel_t pick_hpt(int hpt) {
  switch (hpt) {
    case 1: return fx_lstm_stack_kernel<L, 1>;
    case 2: return fx_lstm_stack_kernel<L, 2>;
    case 4: return fx_lstm_stack_kernel<L, 4>;
    case 8: return fx_lstm_stack_kernel<L, 8>;
    case 16: return fx_lstm_stack_kernel<L, 16>;
    case 32: return fx_lstm_stack_kernel<L, 32>;
    default: return nullptr;
  }
}

// 0: launched; 1: shape outside what the kernel is built for; 2: the grid would not be resident
// all at once (the barrier needs that); otherwise a HIP error code + 100.
int fx_launch_lstm_stack(const FxLstmArgs& a, int L, hipStream_t stream) {
  if (a.H < 32 || a.H % 32 != 0 || a.B < 1 || a.B > FX_LSTM_MAXB || L * a.B > FX_LSTM_BLOCK) return 1;
  fx_lstm_kernel_t k = nullptr;
  switch (L) {
    case 1: k = pick_hpt<1>(a.H / 32); break;
    case 2: k = pick_hpt<2>(a.H / 32); break;
    case 3: k = pick_hpt<3>(a.H / 32); break;
    case 4: k = pick_hpt<4>(a.H / 32); break;
    default: break;
  }
  if (!k) return 1;
  int dev = 0, per_cu = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e == hipSuccess) e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)k, FX_LSTM_BLOCK, 0);
  if (e != hipSuccess) return 100 + (int)e;
  if ((long)per_cu * cus < a.H) return 2;
  void* args[1] = {(void*)&a};
  e = hipLaunchKernel((const void*)k, dim3((uint32_t)a.H), dim3(FX_LSTM_BLOCK), args, 0, stream);
  return e == hipSuccess ? 0 : 100 + (int)e;
}
