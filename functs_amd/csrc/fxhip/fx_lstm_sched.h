// Schedule and hand-over protocol of the persistent stacked-LSTM kernel (fx_lstm.hip), written so
// that the same text also builds for the CPU, where tests run it with one host thread per
// workgroup (tests/support/lstm_emul.cpp) to check the schedule, the buffer parities and the
// protocol without a GPU.
//
// The recurrence (functs/benchmark/ai_model/lstm/lstm.py:79-133): for t in [0, T), for layer j in
// [0, L): gates(t, j) need the output of layer j - 1 at time t and the state of layer j at time
// t - 1.  Cells (t, j) with the same d = t + j are independent, so the kernel walks the
// T + L - 1 diagonals d and computes every active layer of a diagonal in one step.
//   h of (t, j), computed in step d, is written to hbuf[d & 1][j]; step d reads its inputs from
//   hbuf[(d - 1) & 1] (layer j - 1 at time t and layer j at time t - 1 were both computed in
//   step d - 1), from x (layer 0) and from h0 (t == 0).
// Hand-over without a barrier: every element of hbuf is 64 bits, the value and the TAG of the
// step that wrote it (one atomic store), and a reader polls the elements it needs until they
// carry the tag of the step it expects.  A workgroup writes step d only after it has read all
// it needs of step d - 1, and nobody can be in step d + 1, whose writes land on the parity that
// step d reads, before every workgroup has written step d: the two parities suffice.
// Tags are base + d + 1, where base is a word of the workspace that the last workgroup to leave
// advances past the tags of the launch, so the elements a launch finds from earlier launches
// never carry a tag it waits for (a zeroed workspace carries tag 0, which no step has).
// Every poll loop is bounded: a reader that gives up sets the error word and its workgroup
// leaves; the others give up in turn.
#pragma once
#include <stdint.h>

#ifndef FX_LSTM_HD
#define FX_LSTM_HD
#endif

#define FX_LSTM_LINE 64u                          // words between the control words: one 256-byte line each
#define FX_LSTM_W_BASE 0u                         // tag base of the next launch
#define FX_LSTM_W_LEAVE (1u * FX_LSTM_LINE)       // workgroups that have left
#define FX_LSTM_W_ERR (2u * FX_LSTM_LINE)         // a wait was given up
#define FX_LSTM_CTL_WORDS (3u * FX_LSTM_LINE)
#define FX_LSTM_TAG_WRAP 0x80000000u              // the base starts over (and the tags are cleared) beyond this

// arguments of the kernel (contiguous fp32 tensors; see fx_lstm_stack in include/fxhip.h)
struct FxLstmArgs {
  const float *x, *wih, *whh, *bih, *bhh;
  const float *h0, *c0;   // null: zero initial state
  float *out, *state_h, *state_c;
  uint64_t* hbuf;      // [2][L][B][H] (value, tag): h of the cells of the last two steps
  uint32_t* ctl;       // FX_LSTM_CTL_WORDS control words
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
FX_LSTM_HD inline uint64_t fx_lstm_pack(uint32_t value_bits, uint32_t tag) { return ((uint64_t)tag << 32) | value_bits; }
FX_LSTM_HD inline uint32_t fx_lstm_tag_of(uint64_t e) { return (uint32_t)(e >> 32); }
// tag of what step d writes / of what step d reads (written by step d - 1)
FX_LSTM_HD inline uint32_t fx_lstm_tag_written(uint32_t base, int d) { return base + (uint32_t)d + 1u; }
FX_LSTM_HD inline uint32_t fx_lstm_tag_read(uint32_t base, int d) { return base + (uint32_t)d; }

// A wait that was given up: the launch's results are not to be used, and its workspace stays
// marked (the error word) until the host clears it.  Two rules make that visible in the data
// itself, whatever the caller does with the error report:
//   a workgroup that gives up fills out, state_h and state_c with NaN before it leaves (a
//   workgroup that has already finished may write a few values after that; the report still says
//   that the launch failed);
//   a launch that finds the error word set does no step at all: every workgroup reports the
//   error again, fills the results with NaN and leaves.
template <class A>
FX_LSTM_HD inline bool fx_lstm_refused(uint32_t* ctl) { return A::load(ctl + FX_LSTM_W_ERR) != 0u; }
// element first, first + stride, ... of the three results
FX_LSTM_HD inline void fx_lstm_poison(const FxLstmArgs& a, int L, uint32_t first, uint32_t stride) {
  const float nan = __builtin_nanf("");
  const uint32_t n_out = (uint32_t)a.T * (uint32_t)a.B * (uint32_t)a.H, n_state = (uint32_t)L * (uint32_t)a.B * (uint32_t)a.H;
  for (uint32_t i = first; i < n_out; i += stride) a.out[i] = nan;
  for (uint32_t i = first; i < n_state; i += stride) {
    a.state_h[i] = nan;
    a.state_c[i] = nan;
  }
}

// A workgroup that has finished its last step checks out; the last one to do so (nobody reads
// or writes hbuf any more) moves the tag base past this launch's tags and puts the counter back
// to zero, so the same workspace serves the next launch on the stream without a clear in
// between.  Past FX_LSTM_TAG_WRAP the base starts over at zero and the tags in hbuf are cleared
// first.  A workgroup that gave up a wait does not check out: the error word stays set and the
// host clears the whole workspace before it is used again.
//   A: atomics policy { add(uint32_t*) -> old value, load(uint32_t*), store(uint32_t*, v), store64(uint64_t*, v) }
template <class A>
FX_LSTM_HD inline void fx_lstm_leave(uint32_t* ctl, uint32_t n_wg, uint32_t base, uint32_t n_steps, uint64_t* hbuf,
                                     uint32_t n_elems) {
  if (A::add(ctl + FX_LSTM_W_LEAVE) + 1u != n_wg) return;
  uint32_t next = base + n_steps;
  if (next >= FX_LSTM_TAG_WRAP) {
    for (uint32_t i = 0; i < n_elems; ++i) A::store64(hbuf + i, 0ull);
    next = 0u;
  }
  A::store(ctl + FX_LSTM_W_BASE, next);
  A::store(ctl + FX_LSTM_W_LEAVE, 0u);
}
