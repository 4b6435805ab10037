// TEST INFRASTRUCTURE ONLY - never linked into or loaded by the product.
//
// CPU build of the persistent stacked-LSTM kernel's schedule and barrier
// (functs_amd/csrc/fxhip/fx_lstm_sched.h): one host thread per workgroup (hidden unit), the
// diagonal schedule, the two parities of the h buffer and the two-level barrier with bounded
// waits, exactly as the GPU kernel walks them; only the arithmetic inside a workgroup is written
// as plain loops.  Checks, without a GPU, that no cell reads a value that has not been written
// yet or has already been overwritten, and that a wait that cannot end is given up.
#include <math.h>
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <thread>
#include <vector>

#include "../../functs_amd/csrc/fxhip/fx_lstm_sched.h"

namespace {
struct HostAtomics {
  static uint32_t add_release(uint32_t* p) { return __atomic_fetch_add(p, 1u, __ATOMIC_RELEASE); }
  static uint32_t load(uint32_t* p) { return __atomic_load_n(p, __ATOMIC_RELAXED); }
  static void store(uint32_t* p, uint32_t v) { __atomic_store_n(p, v, __ATOMIC_RELAXED); }
  static void acquire() { __atomic_thread_fence(__ATOMIC_ACQUIRE); }
  static void pause() { std::this_thread::yield(); }
};
float sigmoidf(float x) { return 1.0f / (1.0f + expf(-x)); }

// what one workgroup (hidden unit u) does; skip_wg: that workgroup never arrives at a barrier
void workgroup(const FxLstmArgs& a, int L, int u, int n_wg, int skip_wg) {
  const int H = a.H, B = a.B, T = a.T;
  std::vector<float> c((size_t)L * B);
  for (int j = 0; j < L; ++j)
    for (int b = 0; b < B; ++b) c[j * B + b] = a.c0 ? a.c0[((size_t)j * B + b) * H + u] : 0.0f;
  const int n_steps = fx_lstm_steps(T, L);
  for (int d = 0; d < n_steps; ++d) {
    const int rp = (d + 1) & 1;
    for (int j = 0; j < L; ++j) {
      const int t = fx_lstm_time(d, j, T);
      if (t < 0) continue;
      for (int b = 0; b < B; ++b) {
        const float* cur = j == 0 ? a.x + ((size_t)t * B + b) * H : a.hbuf + fx_lstm_hoff(rp, j - 1, b, 0, L, B, H);
        const float* hp = t == 0 ? (a.h0 ? a.h0 + ((size_t)j * B + b) * H : nullptr) : a.hbuf + fx_lstm_hoff(rp, j, b, 0, L, B, H);
        float g[4];
        for (int k = 0; k < 4; ++k) {
          const float* wi = a.wih + ((size_t)(j * 4 + k) * H) * H + u;
          const float* wh = a.whh + ((size_t)(j * 4 + k) * H) * H + u;
          float si = 0.f, sh = 0.f;
          for (int i = 0; i < H; ++i) {
            si += wi[(size_t)i * H] * cur[i];
            sh += wh[(size_t)i * H] * (hp ? hp[i] : 0.0f);
          }
          g[k] = (si + a.bih[(size_t)(j * 4 + k) * H + u]) + (sh + a.bhh[(size_t)(j * 4 + k) * H + u]);
        }
        float& cc = c[j * B + b];
        cc = sigmoidf(g[1]) * cc + sigmoidf(g[0]) * tanhf(g[2]);
        const float h = sigmoidf(g[3]) * tanhf(cc);
        a.hbuf[fx_lstm_hoff(d & 1, j, b, u, L, B, H)] = h;
        if (j == L - 1) a.out[((size_t)t * B + b) * H + u] = h;
        if (t == T - 1) {
          a.state_h[((size_t)j * B + b) * H + u] = h;
          a.state_c[((size_t)j * B + b) * H + u] = cc;
        }
      }
    }
    if (d + 1 < n_steps) {
      if (u == skip_wg) return;
      if (!fx_lstm_barrier<HostAtomics>(a.bar, (uint32_t)(d + 1), (uint32_t)u, (uint32_t)n_wg, a.spin_limit)) return;
    }
  }
  fx_lstm_leave<HostAtomics>(a.bar, (uint32_t)n_wg);
}
}  // namespace

// `launches` runs of the same sequence, one after the other, on barrier words that are cleared only
// once (h0 / c0 may be null: zero initial state).  Returns the error word (0: every barrier was
// passed), or -1 when a run without error did not leave every barrier word at zero.
extern "C" int fx_lstm_emul(const float* x, const float* wih, const float* whh, const float* bih, const float* bhh,
                            const float* h0, const float* c0, float* out, float* state_h, float* state_c, int T, int B,
                            int H, int L, uint32_t spin_limit, int skip_wg, int launches) {
  std::vector<uint32_t> bar(FX_LSTM_BAR_WORDS, 0u);
  std::vector<float> hbuf((size_t)2 * L * B * H, NAN);   // a value read before it is written poisons the result
  FxLstmArgs a;
  a.x = x; a.wih = wih; a.whh = whh; a.bih = bih; a.bhh = bhh; a.h0 = h0; a.c0 = c0;
  a.out = out; a.state_h = state_h; a.state_c = state_c;
  a.hbuf = hbuf.data(); a.bar = bar.data(); a.err_host = nullptr;
  a.T = T; a.B = B; a.H = H; a.spin_limit = spin_limit;
  for (int n = 0; n < launches; ++n) {
    std::fill(hbuf.begin(), hbuf.end(), NAN);
    std::vector<std::thread> th;
    for (int u = 0; u < H; ++u) th.emplace_back(workgroup, std::cref(a), L, u, H, skip_wg);
    for (auto& t : th) t.join();
    const int err = (int)bar[(FX_LSTM_GROUPS + 1u) * FX_LSTM_LINE];
    if (err) return err;
    for (uint32_t w : bar)
      if (w != 0u) return -1;
  }
  return 0;
}
