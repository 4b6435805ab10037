// TEST INFRASTRUCTURE ONLY - never linked into or loaded by the product.
//
// CPU build of the persistent stacked-LSTM kernel's schedule and hand-over protocol
// (functs_amd/csrc/fxhip/fx_lstm_sched.h): one host thread per workgroup (hidden unit), the
// diagonal schedule, the two parities of the h buffer, values that travel with the tag of their
// step, bounded polls and the tag base that the last workgroup advances, as the GPU kernel has
// them; only the arithmetic inside a workgroup is written as plain loops.  Checks, without a GPU,
// that no cell reads a value that has not been written yet or has already been overwritten, that
// launches in a row on one workspace do not see each other's values, and that a wait that
// cannot end is given up.
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
  static uint32_t add(uint32_t* p) { return __atomic_fetch_add(p, 1u, __ATOMIC_ACQ_REL); }
  static uint32_t load(uint32_t* p) { return __atomic_load_n(p, __ATOMIC_ACQUIRE); }
  static void store(uint32_t* p, uint32_t v) { __atomic_store_n(p, v, __ATOMIC_RELEASE); }
  static void store64(uint64_t* p, uint64_t v) { __atomic_store_n(p, v, __ATOMIC_RELEASE); }
  static uint64_t load64(const uint64_t* p) { return __atomic_load_n(p, __ATOMIC_ACQUIRE); }
};
float sigmoidf(float x) { return 1.0f / (1.0f + expf(-x)); }
float bits_to_float(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }
uint32_t float_to_bits(float f) { uint32_t b; memcpy(&b, &f, 4); return b; }

// element i of a tagged vector, polled until it carries `want`; false: given up (the results
// are filled with NaN, as the kernel's workgroup does on its way out)
bool read_tagged(const FxLstmArgs& a, int L, const uint64_t* p, uint32_t want, float* out) {
  for (uint32_t polls = 0;; ++polls) {
    const uint64_t e = HostAtomics::load64(p);
    if (fx_lstm_tag_of(e) == want) { *out = bits_to_float((uint32_t)e); return true; }
    if (polls > a.spin_limit || ((polls & 255u) == 255u && HostAtomics::load(a.ctl + FX_LSTM_W_ERR) != 0u)) {
      HostAtomics::store(a.ctl + FX_LSTM_W_ERR, 1u);
      fx_lstm_poison(a, L, 0u, 1u);
      return false;
    }
    std::this_thread::yield();
  }
}

// what one workgroup (hidden unit u) does; skip_wg: that workgroup stops writing after step 0
void workgroup(const FxLstmArgs& a, int L, int u, int n_wg, int skip_wg) {
  const int H = a.H, B = a.B, T = a.T;
  if (fx_lstm_refused<HostAtomics>(a.ctl)) {   // the workspace carries a given-up wait
    fx_lstm_poison(a, L, (uint32_t)u, (uint32_t)n_wg);
    return;
  }
  const uint32_t base = HostAtomics::load(a.ctl + FX_LSTM_W_BASE);
  std::vector<float> c((size_t)L * B), cur(H), hp(H), hnew((size_t)L * B);
  for (int j = 0; j < L; ++j)
    for (int b = 0; b < B; ++b) c[j * B + b] = a.c0 ? a.c0[((size_t)j * B + b) * H + u] : 0.0f;
  const int n_steps = fx_lstm_steps(T, L);
  for (int d = 0; d < n_steps; ++d) {
    if (u == skip_wg && d > 0) return;
    const int rp = (d + 1) & 1;
    const uint32_t want = fx_lstm_tag_read(base, d);
    // all reads of the step, then all its writes (as the kernel: dot products, barrier, owners)
    for (int j = 0; j < L; ++j) {
      const int t = fx_lstm_time(d, j, T);
      if (t < 0) continue;
      for (int b = 0; b < B; ++b) {
        for (int i = 0; i < H; ++i) {
          if (j == 0) cur[i] = a.x[((size_t)t * B + b) * H + i];
          else if (!read_tagged(a, L, a.hbuf + fx_lstm_hoff(rp, j - 1, b, i, L, B, H), want, &cur[i])) return;
          if (t == 0) hp[i] = a.h0 ? a.h0[((size_t)j * B + b) * H + i] : 0.0f;
          else if (!read_tagged(a, L, a.hbuf + fx_lstm_hoff(rp, j, b, i, L, B, H), want, &hp[i])) return;
        }
        float g[4];
        for (int k = 0; k < 4; ++k) {
          const float* wi = a.wih + ((size_t)(j * 4 + k) * H) * H + u;
          const float* wh = a.whh + ((size_t)(j * 4 + k) * H) * H + u;
          float si = 0.f, sh = 0.f;
          for (int i = 0; i < H; ++i) {
            si += wi[(size_t)i * H] * cur[i];
            sh += wh[(size_t)i * H] * hp[i];
          }
          g[k] = (si + a.bih[(size_t)(j * 4 + k) * H + u]) + (sh + a.bhh[(size_t)(j * 4 + k) * H + u]);
        }
        float& cc = c[j * B + b];
        cc = sigmoidf(g[1]) * cc + sigmoidf(g[0]) * tanhf(g[2]);
        hnew[j * B + b] = sigmoidf(g[3]) * tanhf(cc);
      }
    }
    for (int j = 0; j < L; ++j) {
      const int t = fx_lstm_time(d, j, T);
      if (t < 0) continue;
      for (int b = 0; b < B; ++b) {
        const float h = hnew[j * B + b];
        HostAtomics::store64(a.hbuf + fx_lstm_hoff(d & 1, j, b, u, L, B, H), fx_lstm_pack(float_to_bits(h), fx_lstm_tag_written(base, d)));
        if (j == L - 1) a.out[((size_t)t * B + b) * H + u] = h;
        if (t == T - 1) {
          a.state_h[((size_t)j * B + b) * H + u] = h;
          a.state_c[((size_t)j * B + b) * H + u] = c[j * B + b];
        }
      }
    }
  }
  fx_lstm_leave<HostAtomics>(a.ctl, (uint32_t)n_wg, base, (uint32_t)n_steps, a.hbuf, (uint32_t)(2 * L * B * H));
}
}  // namespace

// `launches` runs of the same sequence, one after the other, on a workspace that is cleared only
// once and whose tag base starts at `base0` (h0 / c0 may be null: zero initial state).  Before
// every run after the first, out / state_h / state_c are filled with NaN.  Returns the error
// word (0: no wait was given up), or -1 when a run without error did not leave the control words
// as the next launch needs them.
extern "C" int fx_lstm_emul(const float* x, const float* wih, const float* whh, const float* bih, const float* bhh,
                            const float* h0, const float* c0, float* out, float* state_h, float* state_c, int T, int B,
                            int H, int L, uint32_t spin_limit, int skip_wg, int launches, uint32_t base0) {
  std::vector<uint32_t> ctl(FX_LSTM_CTL_WORDS, 0u);
  std::vector<uint64_t> hbuf((size_t)2 * L * B * H, 0ull);
  ctl[FX_LSTM_W_BASE] = base0;
  FxLstmArgs a;
  a.x = x; a.wih = wih; a.whh = whh; a.bih = bih; a.bhh = bhh; a.h0 = h0; a.c0 = c0;
  a.out = out; a.state_h = state_h; a.state_c = state_c;
  a.hbuf = hbuf.data(); a.ctl = ctl.data(); a.err_host = nullptr;
  a.T = T; a.B = B; a.H = H; a.spin_limit = spin_limit;
  uint32_t expect_base = base0;
  for (int n = 0; n < launches; ++n) {
    if (n > 0) {
      std::fill(out, out + (size_t)T * B * H, NAN);
      std::fill(state_h, state_h + (size_t)L * B * H, NAN);
      std::fill(state_c, state_c + (size_t)L * B * H, NAN);
    }
    std::vector<std::thread> th;
    for (int u = 0; u < H; ++u) th.emplace_back(workgroup, std::cref(a), L, u, H, skip_wg);
    for (auto& t : th) t.join();
    const int err = (int)ctl[FX_LSTM_W_ERR];
    if (err) return err;
    expect_base += (uint32_t)fx_lstm_steps(T, L);
    if (expect_base >= FX_LSTM_TAG_WRAP) {
      expect_base = 0u;
      for (uint64_t e : hbuf)
        if (e != 0ull) return -1;
    }
    if (ctl[FX_LSTM_W_BASE] != expect_base || ctl[FX_LSTM_W_LEAVE] != 0u) return -1;
  }
  return 0;
}

// A wait that is given up, and what comes after it on the same workspace.  Three launches:
//   1: workgroup `skip_wg` stops writing, the others give up;
//   2: the same workspace, not cleared, every workgroup at work: must be refused;
//   3: the workspace cleared: must run.
// Before each launch the results are filled with 0.5.  Returns bits: 1 launch 1 set the error
// word, 2 its results hold no value other than NaN or what the stopped workgroup wrote,
// 4 launch 2 left the error word set, 8 its results are all NaN, 16 launch 3 ended without error
// (its results are in out / state_h / state_c).
extern "C" int fx_lstm_emul_give_up(const float* x, const float* wih, const float* whh, const float* bih, const float* bhh,
                                    const float* h0, const float* c0, float* out, float* state_h, float* state_c, int T,
                                    int B, int H, int L, uint32_t spin_limit, int skip_wg) {
  std::vector<uint32_t> ctl(FX_LSTM_CTL_WORDS, 0u);
  std::vector<uint64_t> hbuf((size_t)2 * L * B * H, 0ull);
  FxLstmArgs a;
  a.x = x; a.wih = wih; a.whh = whh; a.bih = bih; a.bhh = bhh; a.h0 = h0; a.c0 = c0;
  a.out = out; a.state_h = state_h; a.state_c = state_c;
  a.hbuf = hbuf.data(); a.ctl = ctl.data(); a.err_host = nullptr;
  a.T = T; a.B = B; a.H = H; a.spin_limit = spin_limit;
  const size_t n_out = (size_t)T * B * H, n_state = (size_t)L * B * H;
  auto launch = [&](int skip) {
    std::fill(out, out + n_out, 0.5f);
    std::fill(state_h, state_h + n_state, 0.5f);
    std::fill(state_c, state_c + n_state, 0.5f);
    std::vector<std::thread> th;
    for (int u = 0; u < H; ++u) th.emplace_back(workgroup, std::cref(a), L, u, H, skip);
    for (auto& t : th) t.join();
  };
  // every element NaN, except (when given) those of hidden unit `but`
  auto poisoned = [&](int but) {
    auto all_nan = [&](const float* p, size_t n) {
      for (size_t i = 0; i < n; ++i)
        if (!std::isnan(p[i]) && (int)(i % (size_t)H) != but) return false;
      return true;
    };
    return all_nan(out, n_out) && all_nan(state_h, n_state) && all_nan(state_c, n_state);
  };
  int bits = 0;
  launch(skip_wg);
  if (ctl[FX_LSTM_W_ERR] != 0u) bits |= 1;
  if (poisoned(skip_wg)) bits |= 2;
  launch(-1);
  if (ctl[FX_LSTM_W_ERR] != 0u) bits |= 4;
  if (poisoned(-1)) bits |= 8;
  std::fill(ctl.begin(), ctl.end(), 0u);
  std::fill(hbuf.begin(), hbuf.end(), 0ull);
  // (this launch has every workgroup: it must not give up because the host's threads, more than
  // it has cores, took long to be scheduled)
  a.spin_limit = 0x7fffffffu;
  launch(-1);
  if (ctl[FX_LSTM_W_ERR] == 0u) bits |= 16;
  return bits;
}
