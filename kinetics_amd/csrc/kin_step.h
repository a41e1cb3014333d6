// Parameters of the fused decode-step kernel (kin_step.hip: one workgroup, or a team of
// workgroups, per list).
#pragma once

#include "kin_common.h"

namespace kin {

struct StepParams {
  const uint16_t* q;
  const uint32_t* k;  // new token's K/V rows as dwords; null = no append
  const uint32_t* v;
  uint16_t* kv;
  uint16_t* kbar;
  const int32_t* page_indices;
  const int32_t* page_indptr;
  const int32_t* last_page_len;
  int32_t* sel_pages;  // optional HBM copy of the page lists
  int32_t* sel_count;  // optional
  uint16_t* out;
  float* lse;  // optional
  int batch, num_q_heads, num_kv_heads, group;
  int kbar_pages, sel_stride, topk, sink_pages, local_tokens, first_page_offset, sort_cap, page_size;
  int table_cap;      // LDS entries for the copy of a sequence's page table (0: none)
  int region0_bytes;  // LDS: max(attend staging, select scratch); the page list follows it
  // Teams.  The lists 0 .. head_lists-1 have one workgroup each (the first head_blocks workgroups
  // of the grid); every later list has a team of `team` consecutive workgroups.  Each member
  // scores a slice of the candidates into ws_keys and counts in on ws_count; the members
  // 0 .. parts-1 (parts <= team) then wait for the whole team -- a bounded wait: when it runs out
  // the member scores the whole list itself -- load all the keys, select (identical results),
  // attend their share of the page list and leave a partial result; the member that counts in
  // last on ws_count2 merges the parts.  Counters are zero at launch (a fill kernel in front).
  int head_lists, head_blocks, team, parts;
  int spin_limit;      // polls (a fraction of a microsecond each) a member waits for its team
  int32_t* ws_count;   // [team lists] members that have scored
  int32_t* ws_count2;  // [team lists] parts that have attended
  uint32_t* ws_keys;   // [team lists, score_key_stride(kbar_pages)]
  uint32_t* ws_po;     // [team lists, parts, group, 128] fp32 bits: normalised partial outputs
  uint32_t* ws_plse;   // [team lists, parts, group] fp32 bits: base-2 log-sum-exp of the parts
  const int32_t* slot_ids;  // kbar row block of each sequence (null: the sequence's own index)
  int num_slots;
  int32_t* slot_lens;       // optional [num_slots]: token count of each slot, advanced by one per appended token
  int64_t num_pages;
  float scale_log2;
  int deep_score;      // few lists: more mean-key loads in flight per lane (see the kernel)
  int rotate;          // attend_rotates(lists)
};

// Polls (about a third of a microsecond each) after which a team member stops waiting for the
// others' keys and scores the whole list itself: some 100 us, several times what a slice takes.
// The default of kin_set_team_spin_limit().
constexpr int kTeamSpinLimit = 300;
// The limit the next launches use (kin_api.hip).
int team_spin_limit();

}  // namespace kin
