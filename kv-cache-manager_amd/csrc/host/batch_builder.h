// Turns "these sequences run these token ranges" into the flat int32 arrays the device step
// reads, written into one caller-owned buffer so that a single host-to-device copy moves them.
// The reference packs the same kind of arrays per step (src/engine/engine.cpp:50-71,
// src/model/llama.cpp:65-81); per-group slot maps and tables, per-sequence row ranges, state slots
// and padding to a fixed shape are additions.
#pragma once
#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "kv_manager.h"

namespace kvcm {

struct BatchEntry {
  const Sequence* seq;
  int start;
  int count;
  std::vector<int32_t> want;  // offsets inside [0, count) whose logits are asked for
  // how a token is drawn from each wanted row (the sampling kernel reads them from the same buffer)
  float temperature = 0.f;
  uint64_t sampler_seed = 0;
  int64_t request_id = 0;
  int32_t token_index = 0;
};

// Index of each field in the descriptor array.
enum BatchDesc : int {
  kRows = 0, kSeqs, kLogitRows, kMaxContext, kMaxRun, kTotalInts,
  kOffTokens, kOffPositions, kOffContextLens, kOffRowSeq, kOffRunStart, kOffSeqStart, kOffSeqEnd,
  kOffLogitRows, kOffStateSlots, kRowsPadded, kSeqsPadded, kLogitRowsPadded,
  // sampling parameters per (padded) logit row, starting at an even offset so that the 64-bit
  // arrays are aligned: float temperature[Rp], int32 token_index[Rp], uint64 seed[Rp], int64 request_id[Rp]
  kOffSampling,
  kGroupBase = 20,  // per group: slots offset, tables offset, table stride, (spare)
  kGroupStride = 4,
};

inline int batch_desc_len(int num_groups) { return kGroupBase + kGroupStride * num_groups; }

// Padding rows have token 0, position 0, context length 0 and slot -1: they write no key and
// attend to nothing.  Padding sequences have empty runs and tables of zeros.
// `pad_leading` brings the step's leading single-token runs up to that many: the entries before the
// first one with more than one token are followed by padding sequences of one padding row each, so
// that a step recorded for "D single rows, then prompt portions" fits every step with at most D.
inline void build_batch(const KVManager& kv, const std::vector<BatchEntry>& entries, int pad_rows,
                        int pad_seqs, int pad_logit_rows, int table_stride, int32_t* out, int64_t cap,
                        int32_t* desc, int pad_leading = 0) {
  const int G = kv.num_groups();
  const int B = kv.block_size();
  int T = 0, R = 0, max_ctx = 0, max_run = 0;
  std::vector<int> widest(G, 0);
  for (const auto& e : entries) {
    if (e.count <= 0) throw std::invalid_argument("build_batch: an entry without tokens");
    if (e.start < 0 || e.start + e.count > e.seq->size())
      throw std::invalid_argument("build_batch: the run leaves the sequence's tokens");
    if (static_cast<int>(e.seq->tables.size()) != G)
      throw std::invalid_argument("build_batch: sequence " + std::to_string(e.seq->id) + " holds no pages");
    T += e.count;
    R += static_cast<int>(e.want.size());
    max_ctx = std::max(max_ctx, e.start + e.count);
    max_run = std::max(max_run, e.count);
    for (int g = 0; g < G; ++g) {
      if (kv.group(g).kind == GroupKind::State) continue;
      const int need = (e.start + e.count + B - 1) / B;
      if (static_cast<int>(e.seq->tables[g].size()) < need)
        throw std::invalid_argument("build_batch: sequence " + std::to_string(e.seq->id) + " has no page for its tokens");
      widest[g] = std::max(widest[g], need);
    }
  }
  int leading = 0;
  while (leading < static_cast<int>(entries.size()) && entries[leading].count == 1) ++leading;
  const int filler = std::max(pad_leading - leading, 0);   // padding sequences after the leading single rows
  T += filler;
  const int S = static_cast<int>(entries.size()) + filler;
  const int Tp = std::max(T, pad_rows), Sp = std::max(S, pad_seqs), Rp = std::max(R, pad_logit_rows);
  for (int g = 0; g < G; ++g) {
    if (table_stride > 0) {
      if (widest[g] > table_stride) throw std::invalid_argument("build_batch: table_stride is too small");
      widest[g] = table_stride;
    }
    widest[g] = std::max(widest[g], 1);
  }

  int64_t cursor = 0;
  auto take = [&](int64_t n) { const int64_t at = cursor; cursor += n; return at; };
  for (int i = 0; i < batch_desc_len(G); ++i) desc[i] = 0;
  desc[kRows] = T; desc[kSeqs] = S; desc[kLogitRows] = R;
  desc[kMaxContext] = max_ctx; desc[kMaxRun] = max_run;
  desc[kRowsPadded] = Tp; desc[kSeqsPadded] = Sp; desc[kLogitRowsPadded] = Rp;
  const int64_t o_tok = take(Tp), o_pos = take(Tp), o_ctx = take(Tp), o_rseq = take(Tp);
  const int64_t o_run = take(Sp + 1), o_sstart = take(Sp), o_send = take(Sp);
  const int64_t o_lrow = take(Rp), o_state = take(Sp);
  std::vector<int64_t> o_slots(G), o_tables(G);
  for (int g = 0; g < G; ++g) {
    const bool paged = kv.group(g).kind != GroupKind::State;
    o_slots[g] = take(paged ? Tp : 0);
    o_tables[g] = take(paged ? int64_t(Sp) * widest[g] : 0);
    desc[kGroupBase + kGroupStride * g + 0] = static_cast<int32_t>(o_slots[g]);
    desc[kGroupBase + kGroupStride * g + 1] = static_cast<int32_t>(o_tables[g]);
    desc[kGroupBase + kGroupStride * g + 2] = paged ? widest[g] : 0;
  }
  cursor += cursor & 1;
  const int64_t o_samp = take(6 * int64_t(Rp));
  desc[kOffSampling] = static_cast<int32_t>(o_samp);
  if (cursor > cap) throw std::length_error("build_batch: the metadata buffer is too small");
  if (cursor > INT32_MAX) throw std::length_error("build_batch: metadata exceeds 2^31 ints");
  desc[kTotalInts] = static_cast<int32_t>(cursor);
  desc[kOffTokens] = static_cast<int32_t>(o_tok); desc[kOffPositions] = static_cast<int32_t>(o_pos);
  desc[kOffContextLens] = static_cast<int32_t>(o_ctx); desc[kOffRowSeq] = static_cast<int32_t>(o_rseq);
  desc[kOffRunStart] = static_cast<int32_t>(o_run); desc[kOffSeqStart] = static_cast<int32_t>(o_sstart);
  desc[kOffSeqEnd] = static_cast<int32_t>(o_send); desc[kOffLogitRows] = static_cast<int32_t>(o_lrow);
  desc[kOffStateSlots] = static_cast<int32_t>(o_state);

  for (int64_t i = 0; i < cursor; ++i) out[i] = 0;
  for (int g = 0; g < G; ++g)
    if (kv.group(g).kind != GroupKind::State)
      for (int t = 0; t < Tp; ++t) out[o_slots[g] + t] = -1;
  for (int s = 0; s < Sp; ++s) out[o_state + s] = -1;

  int row = 0, lrow = 0;
  for (int s = 0, next = 0; s < S; ++s) {
    if (s >= leading && s < leading + filler) {   // a padding sequence of one padding row
      out[o_run + s] = row;
      out[o_rseq + row] = s;
      ++row;
      continue;
    }
    const BatchEntry& e = entries[next++];
    const Sequence& q = *e.seq;
    out[o_run + s] = row;
    out[o_sstart + s] = e.start;
    out[o_send + s] = e.start + e.count;
    out[o_state + s] = q.state_slot;
    for (int g = 0; g < G; ++g) {
      if (kv.group(g).kind == GroupKind::State) continue;
      const auto& tab = q.tables[g];
      const int n = std::min<int>(static_cast<int>(tab.size()), widest[g]);
      for (int b = 0; b < n; ++b) out[o_tables[g] + int64_t(s) * widest[g] + b] = tab[b];
    }
    for (int j = 0; j < e.count; ++j, ++row) {
      const int pos = e.start + j;
      out[o_tok + row] = q.tokens[pos];
      out[o_pos + row] = pos;
      out[o_ctx + row] = pos + 1;
      out[o_rseq + row] = s;
      for (int g = 0; g < G; ++g) {
        if (kv.group(g).kind == GroupKind::State) continue;
        const int page = q.tables[g][pos / B];
        if (page < 0) throw std::logic_error("build_batch: token's page was already given back");
        out[o_slots[g] + row] = page * B + pos % B;
      }
    }
    for (int w : e.want) {
      if (w < 0 || w >= e.count) throw std::invalid_argument("build_batch: wanted place outside the run");
      static_assert(sizeof(float) == 4, "the buffer holds 32-bit floats");
      std::memcpy(out + o_samp + lrow, &e.temperature, 4);
      out[o_samp + Rp + lrow] = e.token_index;
      std::memcpy(out + o_samp + 2 * int64_t(Rp) + 2 * int64_t(lrow), &e.sampler_seed, 8);
      std::memcpy(out + o_samp + 4 * int64_t(Rp) + 2 * int64_t(lrow), &e.request_id, 8);
      out[o_lrow + lrow++] = out[o_run + s] + w;
    }
  }
  for (int s = S; s <= Sp; ++s) out[o_run + s] = row;
}

}  // namespace kvcm
