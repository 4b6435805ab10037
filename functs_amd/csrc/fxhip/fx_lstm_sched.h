// Schedule and device-wide barrier of the persistent stacked-LSTM kernel (fx_lstm.hip), written
// so that the same text also builds for the CPU, where tests run it with one host thread per
// workgroup (tests/support/lstm_emul.cpp) to check the schedule, the buffer parities and the
// barrier protocol without a GPU.
//
// The recurrence (functs/benchmark/ai_model/lstm/lstm.py:79-133): for t in [0, T), for layer j in
// [0, L): gates(t, j) need the output of layer j - 1 at time t and the state of layer j at time
// t - 1.  Cells (t, j) with the same d = t + j are independent, so the kernel walks the
// T + L - 1 diagonals d and computes every active layer of a diagonal between two barriers.
//   h of (t, j), computed in step d, is written to hbuf[d & 1][j]; step d reads its inputs from
//   hbuf[(d - 1) & 1] (layer j - 1 at time t and layer j at time t - 1 were both computed in
//   step d - 1), from x (layer 0) and from h0 (t == 0).  Writing parity d & 1 in step d while
//   parity (d - 1) & 1 is read needs one barrier per step and no other ordering.
#pragma once
#include <stdint.h>

#ifndef FX_LSTM_HD
#define FX_LSTM_HD
#endif

#define FX_LSTM_GROUPS 16u         // first-level barrier counters
#define FX_LSTM_LINE 64u           // words between counters: one 256-byte line each
#define FX_LSTM_BAR_WORDS ((FX_LSTM_GROUPS + 3u) * FX_LSTM_LINE)   // groups, top counter, error word, leave counter

// arguments of the kernel (contiguous fp32 tensors; see fx_lstm_stack in include/fxhip.h)
struct FxLstmArgs {
  const float *x, *wih, *whh, *bih, *bhh;
  const float *h0, *c0;   // null: zero initial state
  float *out, *state_h, *state_c;
  float* hbuf;         // [2][L][B][H]: h of the cells of the last two steps
  uint32_t* bar;       // FX_LSTM_BAR_WORDS words, zero when the kernel starts (and again when it ends without error)
  uint32_t* err_host;  // pinned word that a given-up wait reports to as well (may be null)
  int T, B, H;
  uint32_t spin_limit;
};

FX_LSTM_HD inline int fx_lstm_steps(int T, int L) { return T > 0 ? T + L - 1 : 0; }
FX_LSTM_HD inline int fx_lstm_time(int d, int j, int T) {
  const int t = d - j;
  return (t >= 0 && t < T) ? t : -1;
}
// element offset of h of (layer j, batch b, unit u) in parity p of hbuf[2][L][B][H]
FX_LSTM_HD inline uint32_t fx_lstm_hoff(int p, int j, int b, int u, int L, int B, int H) {
  return (uint32_t)((((p * L + j) * B + b) * H) + u);
}

// Arrival at the barrier that closes step `gen` (1-based) and the wait for everybody else.
// Counters only grow during a launch and start from zero (fx_lstm_leave puts them back).  Two levels: a workgroup
// adds to its group's counter, the last arrival of a group adds to the top counter, everybody
// polls the top counter.  Returns false when the wait was given up (poll limit reached, or another
// workgroup had already given up): the error word is set and the caller must leave the kernel.
//   A: atomics policy { add_release(uint32_t*) -> old value, load(uint32_t*), store(uint32_t*, v),
//                       acquire(), pause() }
template <class A>
FX_LSTM_HD inline bool fx_lstm_barrier(uint32_t* bar, uint32_t gen, uint32_t wg, uint32_t n_wg, uint32_t spin_limit) {
  const uint32_t n_groups = n_wg < FX_LSTM_GROUPS ? n_wg : FX_LSTM_GROUPS;
  const uint32_t grp = wg % n_groups;
  const uint32_t members = n_wg / n_groups + (grp < n_wg % n_groups ? 1u : 0u);
  uint32_t* top = bar + FX_LSTM_GROUPS * FX_LSTM_LINE;
  uint32_t* err = bar + (FX_LSTM_GROUPS + 1u) * FX_LSTM_LINE;
  const uint32_t old = A::add_release(bar + grp * FX_LSTM_LINE);
  if (old + 1u == gen * members) (void)A::add_release(top);
  const uint32_t want = gen * n_groups;
  uint32_t polls = 0;
  for (;;) {
    if (A::load(top) >= want) break;
    if (A::load(err) != 0u || polls >= spin_limit) {
      A::store(err, 1u);
      return false;
    }
    ++polls;
    A::pause();
  }
  A::acquire();
  return true;
}

// A workgroup that has passed its last barrier of the launch checks out; the last one to do so
// puts every counter back to zero, so the same words serve the next launch on the stream without
// a clear in between.  Nobody polls any more at that point: a workgroup checks out only after its
// own last wait has ended.  A workgroup that gave up a wait does not check out: the error word
// stays set and the counters stay as they are until the host clears the words.
template <class A>
FX_LSTM_HD inline void fx_lstm_leave(uint32_t* bar, uint32_t n_wg) {
  uint32_t* leave = bar + (FX_LSTM_GROUPS + 2u) * FX_LSTM_LINE;
  if (A::add_release(leave) + 1u != n_wg) return;
  for (uint32_t g = 0; g <= FX_LSTM_GROUPS; ++g) A::store(bar + g * FX_LSTM_LINE, 0u);
  A::store(leave, 0u);
}
