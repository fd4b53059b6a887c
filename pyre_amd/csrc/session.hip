// Host-side request loop over one resident state: prefill on the absolute chunk grid with a prefix cache of state
// snapshots, then greedy generation.  Follows engine_qn::run, src/engine_qn.rs:92-170 of the reference (prefix cache
// :92-99, state / snapshot choice :107-116, chunk grid and the cut at the previous prompt's common prefix :127-146).
#include "common.h"
#include <algorithm>
#include <memory>
#include <vector>

struct pyre_session {
  pyre_ctx* ctx = nullptr; const pyre_model* m = nullptr; pyre_state* st = nullptr;
  int max_ctx = 0, chunk = 256; size_t cap_bytes = 0;
  std::vector<uint32_t> tokens;          // what the state has consumed (State::tokens)
  std::vector<uint32_t> last_prompt;     // LASTP, :129
  struct Entry { std::vector<uint32_t> tokens; pyre_snap* snap; };
  std::vector<Entry> pc;                 // oldest first
  bool have_state = false;
};

namespace {
bool starts_with(const uint32_t* p, int n, const std::vector<uint32_t>& pre) { return (int)pre.size() <= n && std::equal(pre.begin(), pre.end(), p); }
size_t cache_bytes(const pyre_session* s) { size_t b = 0; for (auto& e : s->pc) b += pyre_snap_bytes(e.snap); return b; }
}

extern "C" {

int pyre_session_create(pyre_ctx* ctx, const pyre_model* m, int max_ctx, int prefill_chunk, size_t cache_bytes_cap, pyre_session** out) {
  if (!ctx || !m || !out || max_ctx < 2) return pyre_fail(ctx, PYRE_E_ARG, "pyre_session_create: bad argument");
  *out = nullptr;
  std::unique_ptr<pyre_session> s(new pyre_session()); s->ctx = ctx; s->m = m; s->max_ctx = max_ctx; s->chunk = prefill_chunk > 0 ? prefill_chunk : 256; s->cap_bytes = cache_bytes_cap;
  int rc = pyre_state_create(ctx, m, max_ctx, &s->st); if (rc) return rc;
  *out = s.release(); return PYRE_OK;
}
void pyre_session_destroy(pyre_session* s) {
  if (!s) return;
  for (auto& e : s->pc) pyre_snap_destroy(e.snap);
  pyre_state_destroy(s->st); delete s;
}
pyre_state* pyre_session_state(pyre_session* s) { return s ? s->st : nullptr; }

int pyre_session_prefill(pyre_ctx* ctx, pyre_session* s, const uint32_t* prompt, int n, float* logits_host, int* cached_out, int* from_snapshot) {
  if (!ctx || !s || !prompt || !logits_host) return pyre_fail(ctx, PYRE_E_ARG, "pyre_session_prefill: null argument");
  if (n < 1) return pyre_fail(ctx, PYRE_E_ARG, "pyre_session_prefill: empty prompt");
  if (n >= s->max_ctx) return pyre_fail(ctx, PYRE_E_STATE, "prompt (%d tokens) exceeds context size %d", n, s->max_ctx);                // :104
  const bool pcache = s->cap_bytes > 0;
  // reuse the previous state only when the new prompt strictly extends it (:106); longest snapshot the prompt strictly extends (:108)
  const int ext = (s->have_state && (int)s->tokens.size() < n && starts_with(prompt, n, s->tokens)) ? (int)s->tokens.size() : 0;
  int best = -1, best_n = 0;
  if (pcache) for (size_t i = 0; i < s->pc.size(); ++i) { int ln = (int)s->pc[i].tokens.size(); if (ln < n && starts_with(prompt, n, s->pc[i].tokens) && (best < 0 || ln >= best_n)) { best = (int)i; best_n = ln; } }
  int cached = 0, rc; bool snap_used = false;
  if (ext > 0 && (best < 0 || best_n <= ext)) cached = ext;
  else if (best >= 0) {
    pyre_session::Entry e = std::move(s->pc[best]); s->pc.erase(s->pc.begin() + best);
    rc = pyre_state_restore(ctx, s->st, e.snap);
    s->tokens = e.tokens; s->pc.push_back(std::move(e));          // most recently used goes to the young end (:113)
    if (rc) { s->have_state = false; return rc; }
    cached = best_n; snap_used = true;
  } else { if ((rc = pyre_state_reset(ctx, s->st))) return rc; s->tokens.clear(); }
  s->have_state = true;
  // absolute chunk grid: the first piece runs up to the next multiple of `chunk`, so a prompt resumed from a grid snapshot is
  // split exactly like a full prefill of the same tokens; also cut (and snapshot) where this prompt leaves the previous one
  int lcp = 0; { int lim = std::min<int>((int)s->last_prompt.size(), n); while (lcp < lim && s->last_prompt[lcp] == prompt[lcp]) ++lcp; }
  const int cut = (pcache && lcp > cached && lcp < n) ? lcp : INT32_MAX;
  s->last_prompt.assign(prompt, prompt + n);
  int pos = cached;
  while (pos < n) {
    int end = std::min((pos / s->chunk + 1) * s->chunk, n); if (pos < cut && cut < end) end = cut;
    rc = pyre_forward(ctx, s->m, s->st, prompt + pos, end - pos, end == n ? logits_host : nullptr);
    if (rc) { s->have_state = false; return rc; }
    s->tokens.insert(s->tokens.end(), prompt + pos, prompt + end); pos = end;
    if (pcache && (end % s->chunk == 0 || end == cut) && end < n) {
      bool have = false; for (auto& e : s->pc) if ((int)e.tokens.size() == end && std::equal(e.tokens.begin(), e.tokens.end(), prompt)) { have = true; break; }
      if (!have) {
        pyre_snap* sn = nullptr;
        if (pyre_state_snapshot(ctx, s->st, &sn) == PYRE_OK) {       // a snapshot that cannot be taken (memory) is skipped, as Model::snapshot returning None (:141)
          s->pc.push_back(pyre_session::Entry{std::vector<uint32_t>(prompt, prompt + end), sn});
          while (s->pc.size() > 1 && cache_bytes(s) > s->cap_bytes) { pyre_snap_destroy(s->pc.front().snap); s->pc.erase(s->pc.begin()); }     // oldest dropped first (:141)
        }
      }
    }
  }
  if (cached_out) *cached_out = cached; if (from_snapshot) *from_snapshot = snap_used ? 1 : 0;
  return PYRE_OK;
}

int pyre_session_generate_greedy(pyre_ctx* ctx, pyre_session* s, const float* first_logits_host, int n_out, uint32_t* out, int n_draft, const uint32_t* draft_stream, int* rounds) {
  if (!ctx || !s || !s->have_state) return pyre_fail(ctx, PYRE_E_STATE, "pyre_session_generate_greedy: no prefilled state");
  if ((int)s->tokens.size() + n_out > s->max_ctx) return pyre_fail(ctx, PYRE_E_STATE, "pyre_session_generate_greedy: %d more tokens exceed the context size %d", n_out, s->max_ctx);
  int rc = pyre_generate_greedy(ctx, s->m, s->st, first_logits_host, n_out, out, n_draft, draft_stream, rounds);
  if (rc) { s->have_state = false; return rc; }
  s->tokens.insert(s->tokens.end(), out, out + (n_out > 0 ? n_out - 1 : 0));      // the last emitted token is pending: the state has not consumed it
  if ((int)s->tokens.size() != pyre_state_len(s->st)) { s->have_state = false; return pyre_fail(ctx, PYRE_E_STATE, "pyre_session_generate_greedy: token record (%zu) and state length (%d) differ", s->tokens.size(), pyre_state_len(s->st)); }
  return PYRE_OK;
}

int pyre_session_stats(const pyre_session* s, int* n_snapshots, size_t* snapshot_bytes, int* state_len) {
  if (!s) return PYRE_E_ARG;
  if (n_snapshots) *n_snapshots = (int)s->pc.size(); if (snapshot_bytes) *snapshot_bytes = cache_bytes(s); if (state_len) *state_len = s->have_state ? (int)s->tokens.size() : 0;
  return PYRE_OK;
}
int pyre_session_snapshot_len(const pyre_session* s, int i) { return (s && i >= 0 && i < (int)s->pc.size()) ? (int)s->pc[i].tokens.size() : -1; }

}  // extern "C"
