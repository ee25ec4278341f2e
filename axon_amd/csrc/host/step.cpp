// The host side of a step before anything runs on the device: the entries of a step are checked
// and their tokens laid side by side, in one native call (the reference validates a whole step
// before it runs anything and builds its rows natively: src/cuda/qwen2/slots.rs:393-438,
// src/cuda/qwen2/batch.rs:2942-2963).
//
// An entry is (tokens it brings, positions its request already holds, its slot, the places among
// its tokens whose logits are wanted).  The layout is what the device is given: for each token of
// the step its id, its position and its request's slot (three rows of `meta`), and the rows whose
// logits are wanted.  Nothing is written if the step is refused.
#include <stdint.h>
#include <stdio.h>

extern "C" {

// tokens: the entries' tokens one after the other (counts[e] each); want: likewise the wanted
// places (want_counts[e] each, relative to the entry's first token).  meta: [3][stride] int32,
// rows = token ids, positions, slots.  Returns the number of tokens laid out, or a negative code
// with a message in err: -1 an entry without tokens, -2 a token outside the vocabulary, -3 a
// wanted place outside the entry's tokens, -4 a request that would pass max_seq_len, -5 more
// tokens than meta has room for.  *entry says which entry was refused.
long axh_step_layout(int n_entries, const int32_t* slots, const long* n_cached, const long* counts, const int64_t* tokens,
                     const long* want, const long* want_counts, long vocab, long max_seq_len, int32_t* meta, long stride,
                     int32_t* want_rows, int* entry, char* err, int err_len) {
  long total = 0, at = 0, w_at = 0;
  for (int e = 0; e < n_entries; ++e) {
    *entry = e;
    if (counts[e] <= 0) {
      snprintf(err, err_len, "brings no tokens");
      return -1;
    }
    for (long i = 0; i < counts[e]; ++i) {
      const int64_t t = tokens[at + i];
      if (t < 0 || t >= vocab) {
        snprintf(err, err_len, "token %lld is outside the vocabulary of %ld", (long long)t, vocab);
        return -2;
      }
    }
    for (long i = 0; i < want_counts[e]; ++i) {
      const long w = want[w_at + i];
      if (w < 0 || w >= counts[e]) {
        snprintf(err, err_len, "wanted place %ld is outside its %ld tokens", w, counts[e]);
        return -3;
      }
    }
    if (n_cached[e] + counts[e] > max_seq_len) {
      snprintf(err, err_len, "would reach %ld positions, at most %ld", n_cached[e] + counts[e], max_seq_len);
      return -4;
    }
    at += counts[e];
    w_at += want_counts[e];
    total += counts[e];
  }
  *entry = -1;
  if (total > stride) {
    snprintf(err, err_len, "%ld tokens, room for %ld", total, stride);
    return -5;
  }
  at = 0;
  w_at = 0;
  long n_want = 0;
  for (int e = 0; e < n_entries; ++e) {
    for (long i = 0; i < counts[e]; ++i) {
      meta[at + i] = (int32_t)tokens[at + i];
      meta[stride + at + i] = (int32_t)(n_cached[e] + i);
      meta[2 * stride + at + i] = slots[e];
    }
    for (long i = 0; i < want_counts[e]; ++i) want_rows[n_want++] = (int32_t)(at + want[w_at + i]);
    at += counts[e];
    w_at += want_counts[e];
  }
  return total;
}

}  // extern "C"
