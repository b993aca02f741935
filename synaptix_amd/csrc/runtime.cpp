// Host-side runtime (no device code): the bookkeeping of cache pages and sequence slots, the
// integer tables of a step as the kernels read them, and the sampler's random stream.
//
// The reference keeps these in Rust beside its kernels: one dense cache per layer with a single
// length for the whole batch (crates/synaptix-models/llm/common/src/model.rs:349-368,998-1050),
// per-row device arrays for its graph decode (model.rs:519-553), and Philox-4x32-10 for sampling
// (crates/synaptix-ops/src/rng.rs:16-25,32-36,50-58,82-97).  Here every sequence has a length of
// its own, so storage is cut into pages of 64 tokens and every step carries a sequence table.
//
// All functions return 0, or 1 (nothing free: pages or slots; nothing was taken) or 2 (misuse),
// with a text for syn_rt_last_error().  Handles are plain pointers owned by the caller.
#include <algorithm>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <queue>
#include <vector>

#define RT_API extern "C" __attribute__((visibility("default")))

namespace {

constexpr int OK = 0, FULL = 1, MISUSE = 2;
constexpr int PAGE_TOKENS = 64;

thread_local char g_error[512];

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

inline long pages_for(long n_tokens) { return (n_tokens + PAGE_TOKENS - 1) / PAGE_TOKENS; }

// ------------------------------------------------------------------ pages
struct PagePool {
  int n_pages;
  std::vector<int> free_list;   // back() is handed out next: 0, 1, 2, ... at first
  std::vector<uint8_t> held;

  explicit PagePool(int n) : n_pages(n), held(n, 0) {
    free_list.reserve(n);
    for (int p = n - 1; p >= 0; --p) free_list.push_back(p);
  }
  int free_pages() const { return (int)free_list.size(); }

  int take(int n, int* out) {
    if (n > free_pages()) return fail(FULL, "%d pages wanted, %d of %d free", n, free_pages(), n_pages);
    for (int i = 0; i < n; ++i) {
      const int p = free_list.back();
      free_list.pop_back();
      held[p] = 1;
      out[i] = p;
    }
    return OK;
  }
  int give_back(const int* pages, int n) {
    for (int i = 0; i < n; ++i) {
      const int p = pages[i];
      if (p < 0 || p >= n_pages || !held[p]) return fail(MISUSE, "page %d is not held", p);
      held[p] = 0;
      free_list.push_back(p);
    }
    return OK;
  }
  // every page is either free once or held: none lost, none twice
  int check() const {
    std::vector<uint8_t> seen(n_pages, 0);
    for (int p : free_list) {
      if (p < 0 || p >= n_pages) return fail(MISUSE, "page %d in the free list does not exist", p);
      if (seen[p]) return fail(MISUSE, "a page is in the free list twice");
      seen[p] = 1;
    }
    for (int p = 0; p < n_pages; ++p)
      if ((held[p] != 0) == (seen[p] != 0))
        return fail(MISUSE, "page %d is %s", p, held[p] ? "both held and free" : "lost");
    return OK;
  }
};

// ------------------------------------------------------------------ slots
struct Slot {
  bool live = false;
  long length = 0;     // tokens written
  long reserved = 0;   // tokens for which pages are held (>= length)
  std::vector<std::vector<int>> pages;   // [group][logical page] -> page id, -1 once given back
};

struct Cache {
  std::vector<PagePool> pools;   // one for each group
  std::vector<long> windows;     // keys a query sees, or -1 for all of them
  int n_pages, max_slots;
  long max_positions;            // -1: no limit
  std::vector<Slot> slots;
  std::vector<int> free_slots;

  Slot* live_slot(int sid) {
    if (sid < 0 || sid >= max_slots || !slots[sid].live) {
      fail(MISUSE, "slot %d is not live", sid);
      return nullptr;
    }
    return &slots[sid];
  }
};

// ------------------------------------------------------------------ random stream
struct Philox {
  uint32_t key[2];
  uint32_t counter[4] = {0, 0, 0, 0};
  uint32_t buf[4];
  int left = 0;
};

void philox_block(const uint32_t c_in[4], const uint32_t k_in[2], uint32_t out[4]) {
  uint32_t c0 = c_in[0], c1 = c_in[1], c2 = c_in[2], c3 = c_in[3], k0 = k_in[0], k1 = k_in[1];
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
    c0 = n0, c1 = n1, c2 = n2, c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0, out[1] = c1, out[2] = c2, out[3] = c3;
}

uint32_t philox_next(Philox* p) {
  if (p->left == 0) {
    philox_block(p->counter, p->key, p->buf);
    for (int i = 0; i < 4; ++i)
      if (++p->counter[i]) break;
    p->left = 4;
  }
  return p->buf[4 - p->left--];
}

// ------------------------------------------------------------------ the tables of a step
// One int32 buffer: tokens[N] tok_seq[N] tok_pos[N] seq_start[B+1] seq_past[B] seq_len[B] seq_slot[B]
// want[n_want], then a page table [B, width_g] for each group.
struct Layout {
  long tokens, tok_seq, tok_pos, seq_start, seq_past, seq_len, seq_slot, want, total;
  std::vector<long> tables;
};

Layout make_layout(long N, long B, long n_want, int n_groups, const int* widths) {
  Layout l;
  long off = 0;
  l.tokens = off, off += N;
  l.tok_seq = off, off += N;
  l.tok_pos = off, off += N;
  l.seq_start = off, off += B + 1;
  l.seq_past = off, off += B;
  l.seq_len = off, off += B;
  l.seq_slot = off, off += B;
  l.want = off, off += n_want;
  for (int g = 0; g < n_groups; ++g) {
    l.tables.push_back(off);
    off += B * widths[g];
  }
  l.total = std::max(off, 1L);
  return l;
}

int fill_table(Cache* c, int group, const int* sids, int n, int width, int fill, int* out) {
  for (int i = 0; i < n; ++i) {
    Slot* s = c->live_slot(sids[i]);
    if (!s) return MISUSE;
    const std::vector<int>& pages = s->pages[group];
    if ((int)pages.size() > width)
      return fail(MISUSE, "page table width %d is less than %d", width, (int)pages.size());
    int* row = out + (size_t)i * width;
    for (int j = 0; j < width; ++j) row[j] = j < (int)pages.size() ? std::max(pages[j], 0) : fill;
  }
  return OK;
}

}  // namespace

RT_API const char* syn_rt_last_error() { return g_error; }
RT_API int syn_rt_page_tokens() { return PAGE_TOKENS; }

// ------------------------------------------------------------------ cache bookkeeping
// group_pages: the pages of each group's pool (a group that keeps a window needs fewer than one that keeps every
// key), or null: n_pages for every group
RT_API void* syn_cache_new(int n_groups, const long* windows, int n_pages, const int* group_pages, int max_slots,
                           long max_positions) {
  if (n_groups < 0 || n_pages <= 0 || max_slots <= 0) {
    fail(MISUSE, "a cache needs pages and slots (%d pages, %d slots)", n_pages, max_slots);
    return nullptr;
  }
  for (int g = 0; group_pages && g < n_groups; ++g)
    if (group_pages[g] <= 0) {
      fail(MISUSE, "group %d of the cache has %d pages", g, group_pages[g]);
      return nullptr;
    }
  Cache* c = new Cache;
  c->n_pages = n_pages, c->max_slots = max_slots, c->max_positions = max_positions;
  for (int g = 0; g < n_groups; ++g) {
    c->pools.emplace_back(group_pages ? group_pages[g] : n_pages);
    c->windows.push_back(windows[g]);
  }
  c->slots.resize(max_slots);
  for (int s = max_slots - 1; s >= 0; --s) c->free_slots.push_back(s);
  return c;
}
RT_API void syn_cache_delete(void* h) { delete (Cache*)h; }
RT_API int syn_cache_free_slots(void* h) { return (int)((Cache*)h)->free_slots.size(); }
RT_API int syn_cache_free_pages(void* h, int group) { return ((Cache*)h)->pools[group].free_pages(); }
RT_API int syn_cache_is_live(void* h, int sid) {
  Cache* c = (Cache*)h;
  return sid >= 0 && sid < c->max_slots && c->slots[sid].live;
}

RT_API int syn_cache_acquire(void* h, int* sid_out) {
  Cache* c = (Cache*)h;
  if (c->free_slots.empty()) return fail(FULL, "all %d slots are taken", c->max_slots);
  const int sid = c->free_slots.back();
  c->free_slots.pop_back();
  Slot& s = c->slots[sid];
  s.live = true, s.length = 0, s.reserved = 0;
  s.pages.assign(c->pools.size(), {});
  *sid_out = sid;
  return OK;
}

RT_API int syn_cache_release(void* h, int sid) {
  Cache* c = (Cache*)h;
  Slot* s = c->live_slot(sid);
  if (!s) return MISUSE;
  for (size_t g = 0; g < c->pools.size(); ++g) {
    std::vector<int> held;
    for (int p : s->pages[g])
      if (p >= 0) held.push_back(p);
    const int rc = c->pools[g].give_back(held.data(), (int)held.size());
    if (rc) return rc;
  }
  s->live = false, s->length = 0, s->reserved = 0;
  s->pages.clear();
  c->free_slots.push_back(sid);
  return OK;
}

RT_API int syn_cache_length(void* h, int sid, long* out) {
  Slot* s = ((Cache*)h)->live_slot(sid);
  if (!s) return MISUSE;
  *out = s->length;
  return OK;
}

// pages that reserve(sid, n_new) would take from every group
RT_API int syn_cache_pages_needed(void* h, int sid, long n_new, long* out) {
  Slot* s = ((Cache*)h)->live_slot(sid);
  if (!s) return MISUSE;
  *out = std::max(0L, pages_for(s->length + n_new) - pages_for(s->reserved));
  return OK;
}

// hold pages for n_new more tokens in every group, or FULL and nothing changed
RT_API int syn_cache_reserve(void* h, int sid, long n_new) {
  Cache* c = (Cache*)h;
  Slot* s = c->live_slot(sid);
  if (!s) return MISUSE;
  if (n_new <= 0) return fail(MISUSE, "a step brings at least one token for each of its sequences");
  const long total = s->length + n_new;
  if (c->max_positions >= 0 && total > c->max_positions)
    return fail(MISUSE, "KV overflow: %ld + %ld tokens exceed the position range %ld", s->length, n_new,
                c->max_positions);
  const long want = pages_for(total) - pages_for(s->reserved);
  if (want > 0) {
    for (PagePool& p : c->pools)
      if (p.free_pages() < want) return fail(FULL, "%ld pages wanted, %d of %d free", want, p.free_pages(), p.n_pages);
    std::vector<int> got(want);
    for (size_t g = 0; g < c->pools.size(); ++g) {
      c->pools[g].take((int)want, got.data());
      s->pages[g].insert(s->pages[g].end(), got.begin(), got.end());
    }
  }
  s->reserved = std::max(s->reserved, total);
  return OK;
}

// all pages that a step's sequences need, or FULL and nothing changed
RT_API int syn_cache_reserve_step(void* h, int n, const int* sids, const long* counts) {
  Cache* c = (Cache*)h;
  long need = 0;
  for (int i = 0; i < n; ++i) {
    Slot* s = c->live_slot(sids[i]);
    if (!s) return MISUSE;
    if (counts[i] <= 0) return fail(MISUSE, "a step brings at least one token for each of its sequences");
    if (c->max_positions >= 0 && s->length + counts[i] > c->max_positions)
      return fail(MISUSE, "KV overflow: slot %d holds %ld tokens, %ld more exceed the position range %ld", sids[i],
                  s->length, counts[i], c->max_positions);
    need += std::max(0L, pages_for(s->length + counts[i]) - pages_for(s->reserved));
  }
  for (PagePool& p : c->pools)
    if (p.free_pages() < need)
      return fail(FULL, "the step needs %ld more pages, %d of %d are free", need, p.free_pages(), p.n_pages);
  for (int i = 0; i < n; ++i) {
    const int rc = syn_cache_reserve(h, sids[i], counts[i]);
    if (rc) return rc;
  }
  return OK;
}

// the step has written n_new tokens; windows give back the pages that fell out of reach
RT_API int syn_cache_commit(void* h, int sid, long n_new) {
  Cache* c = (Cache*)h;
  Slot* s = c->live_slot(sid);
  if (!s) return MISUSE;
  if (s->length + n_new > s->reserved) return fail(MISUSE, "commit without reserve");
  s->length += n_new;
  for (size_t g = 0; g < c->pools.size(); ++g) {
    const long w = c->windows[g];
    if (w < 0) continue;
    // the next query sits at position `length`; it sees keys > length - w
    const long first_needed = std::max(0L, s->length - w + 1) / PAGE_TOKENS;
    std::vector<int>& pages = s->pages[g];
    for (long i = 0; i < first_needed && i < (long)pages.size(); ++i)
      if (pages[i] >= 0) {
        const int rc = c->pools[g].give_back(&pages[i], 1);
        if (rc) return rc;
        pages[i] = -1;
      }
  }
  return OK;
}

// Go back to an earlier length of the sequence (what lies behind it is written again).  Pages stay
// held; a group with a window must still hold every page that a query at `length` sees.
RT_API int syn_cache_truncate(void* h, int sid, long length) {
  Cache* c = (Cache*)h;
  Slot* s = c->live_slot(sid);
  if (!s) return MISUSE;
  if (length < 0 || length > s->length)
    return fail(MISUSE, "slot %d holds %ld tokens and cannot go back to %ld", sid, s->length, length);
  for (size_t g = 0; g < c->pools.size(); ++g) {
    const long w = c->windows[g];
    if (w < 0) continue;
    const long first_needed = std::max(0L, length - w + 1) / PAGE_TOKENS;
    const std::vector<int>& pages = s->pages[g];
    for (long i = first_needed; i < pages_for(length) && i < (long)pages.size(); ++i)
      if (pages[i] < 0)
        return fail(MISUSE, "slot %d: the window of group %d has given back a page that length %ld needs", sid,
                    (int)g, length);
  }
  s->length = length;
  return OK;
}

RT_API int syn_cache_table_width(void* h, int group, const int* sids, int n, int* out) {
  Cache* c = (Cache*)h;
  int w = 1;
  for (int i = 0; i < n; ++i) {
    Slot* s = c->live_slot(sids[i]);
    if (!s) return MISUSE;
    w = std::max(w, (int)s->pages[group].size());
  }
  *out = w;
  return OK;
}

// int32 [n, width]: the page of each logical page of each sequence (0 where none)
RT_API int syn_cache_page_table(void* h, int group, const int* sids, int n, int width, int* out) {
  return fill_table((Cache*)h, group, sids, n, width, 0, out);
}

RT_API int syn_cache_live_slots(void* h, int* out) {
  Cache* c = (Cache*)h;
  int n = 0;
  for (int s = 0; s < c->max_slots; ++s)
    if (c->slots[s].live) out[n++] = s;
  return n;
}

// no slot or page lost, held twice or free twice
RT_API int syn_cache_check(void* h) {
  Cache* c = (Cache*)h;
  std::vector<uint8_t> free_seen(c->max_slots, 0);
  for (int s : c->free_slots) {
    if (free_seen[s]) return fail(MISUSE, "a slot is in the free list twice");
    free_seen[s] = 1;
  }
  for (int s = 0; s < c->max_slots; ++s)
    if (c->slots[s].live == (free_seen[s] != 0))
      return fail(MISUSE, "slot %d is %s", s, c->slots[s].live ? "both live and free" : "lost");
  for (size_t g = 0; g < c->pools.size(); ++g) {
    const int rc = c->pools[g].check();
    if (rc) return rc;
    const int pool_pages = c->pools[g].n_pages;
    std::vector<uint8_t> owned(pool_pages, 0);
    long held = 0;
    for (const Slot& s : c->slots) {
      if (!s.live) continue;
      for (int p : s.pages[g]) {
        if (p < 0) continue;
        if (p >= pool_pages) return fail(MISUSE, "group %d: page %d does not exist", (int)g, p);
        if (owned[p]) return fail(MISUSE, "group %d: a page is held by two sequences", (int)g);
        owned[p] = 1;
        ++held;
      }
    }
    if (held + c->pools[g].free_pages() != pool_pages)
      return fail(MISUSE, "group %d: %ld pages lost", (int)g, pool_pages - held - c->pools[g].free_pages());
  }
  return OK;
}

// ------------------------------------------------------------------ the tables of a step
// offsets[0..7] = tokens, tok_seq, tok_pos, seq_start, seq_past, seq_len, seq_slot, want;
// offsets[8 + g] = page table of group g; returns the buffer's length in int32
RT_API long syn_step_layout(long N, long B, long n_want, int n_groups, const int* widths, long* offsets) {
  const Layout l = make_layout(N, B, n_want, n_groups, widths);
  const long o[8] = {l.tokens, l.tok_seq, l.tok_pos, l.seq_start, l.seq_past, l.seq_len, l.seq_slot, l.want};
  std::memcpy(offsets, o, sizeof(o));
  for (int g = 0; g < n_groups; ++g) offsets[8 + g] = l.tables[g];
  return l.total;
}

// Sequences one after another without padding: tokens of sequence i at positions past_i, past_i + 1, ...
// (past_i = the slot's length).  host has room for syn_step_layout's total.
RT_API int syn_step_fill(void* h, int B, const int* sids, const long* counts, const int* tokens, long n_want,
                         const int* want_rows, int n_groups, const int* widths, int* host) {
  Cache* c = (Cache*)h;
  long N = 0;
  for (int i = 0; i < B; ++i) N += counts[i];
  const Layout l = make_layout(N, B, n_want, n_groups, widths);
  long pos = 0;
  for (int i = 0; i < B; ++i) {
    Slot* s = c->live_slot(sids[i]);
    if (!s) return MISUSE;
    const long past = s->length, n = counts[i];
    host[l.seq_start + i] = (int)pos;
    host[l.seq_past + i] = (int)past;
    host[l.seq_len + i] = (int)(past + n);
    host[l.seq_slot + i] = sids[i];
    for (long t = 0; t < n; ++t) {
      host[l.tokens + pos + t] = tokens[pos + t];
      host[l.tok_seq + pos + t] = i;
      host[l.tok_pos + pos + t] = (int)(past + t);
    }
    pos += n;
  }
  host[l.seq_start + B] = (int)pos;
  for (long i = 0; i < n_want; ++i) host[l.want + i] = want_rows[i];
  for (int g = 0; g < n_groups; ++g) {
    const int rc = fill_table(c, g, sids, B, widths[g], 0, host + l.tables[g]);
    if (rc) return rc;
  }
  return OK;
}

// The same for a step that is replayed from a captured graph and therefore has fixed counts: N_pad tokens,
// B_pad sequences, want_pad wanted rows.  The step's own B sequences and N tokens come first; the tokens up
// to N_pad are padding (token 0 at positions 0, 1, ... of sequence B, which owns no slot and whose table
// row names only a spare page that no sequence owns); sequences beyond it are empty; wanted rows beyond the
// step's own name row 0.  B < B_pad unless N == N_pad; a table row of widths[g] pages must hold N_pad - N tokens.
RT_API int syn_step_fill_padded(void* h, int B, const int* sids, const long* counts, const int* tokens, long n_want,
                                const int* want_rows, int n_groups, const int* widths, const int* spare_pages,
                                long N_pad, int B_pad, long want_pad, int* host) {
  Cache* c = (Cache*)h;
  long N = 0;
  for (int i = 0; i < B; ++i) N += counts[i];
  if (N > N_pad || B > B_pad || n_want > want_pad || (N < N_pad && B == B_pad))
    return fail(MISUSE, "a step of %ld tokens, %d sequences, %ld wanted rows for a table of %ld, %d, %ld", N, B, n_want,
                N_pad, B_pad, want_pad);
  for (int g = 0; g < n_groups; ++g)
    if ((N_pad - N + PAGE_TOKENS - 1) / PAGE_TOKENS > widths[g])
      return fail(MISUSE, "page table width %d of group %d is less than the %ld padding tokens need", widths[g], g, N_pad - N);
  const Layout l = make_layout(N_pad, B_pad, want_pad, n_groups, widths);
  long pos = 0;
  for (int i = 0; i < B_pad; ++i) {
    long past = 0, n = 0;
    int sid = -1;
    if (i < B) {
      Slot* s = c->live_slot(sids[i]);
      if (!s) return MISUSE;
      past = s->length, n = counts[i], sid = sids[i];
    } else if (i == B) {
      n = N_pad - N;
    }
    host[l.seq_start + i] = (int)pos;
    host[l.seq_past + i] = (int)past;
    host[l.seq_len + i] = (int)(past + n);
    host[l.seq_slot + i] = sid;
    for (long t = 0; t < n; ++t) {
      host[l.tokens + pos + t] = i < B ? tokens[pos + t] : 0;
      host[l.tok_seq + pos + t] = i;
      host[l.tok_pos + pos + t] = (int)(past + t);
    }
    pos += n;
  }
  host[l.seq_start + B_pad] = (int)pos;
  for (long i = 0; i < want_pad; ++i) host[l.want + i] = i < n_want ? want_rows[i] : 0;
  for (int g = 0; g < n_groups; ++g) {
    int* tab = host + l.tables[g];
    const int rc = fill_table(c, g, sids, B, widths[g], spare_pages[g], tab);
    if (rc) return rc;
    for (long j = (long)B * widths[g]; j < (long)B_pad * widths[g]; ++j) tab[j] = spare_pages[g];
  }
  return OK;
}

// The work list of a decode step's attention over one group of layers: rows * n_splits items
// {sequence, split | splits of the sequence << 16, first, the sequence's length}, where `first` + split is
// the place of the split's partial result.  Every sequence gets one split; the others go one by one to the sequence whose splits
// are longest, while a split keeps at least MIN_UNITS units of 32 keys (a window bounds the keys that
// count); sequences of one length get equal shares.  The items lie in rounds (every sequence's first split, then
// the second of those that have one, ...), in each round the longest pieces first; spare items {-1, 0, 0, 0} last.
// Behind the items lie rows x {first, splits}, the same by sequence, for a kernel that merges the splits afterwards:
// `items` has room for 4 * rows * n_splits + 2 * rows ints.
RT_API int syn_decode_items(const int* seq_len, int rows, int n_splits, long window, int* items) {
  if (rows <= 0 || n_splits <= 0) return fail(MISUSE, "a work list for %d rows x %d splits", rows, n_splits);
  constexpr long UNIT = 32, MIN_UNITS = 8;
  constexpr int MAX_SPLITS = 64;
  const long T = (long)rows * n_splits;
  std::vector<long> units(rows);
  std::vector<int> splits(rows, 1);
  for (int i = 0; i < rows; ++i) {
    long keys = std::max(1, seq_len[i]);
    if (window > 0) keys = std::min(keys, window);
    units[i] = (keys + UNIT - 1) / UNIT;
  }
  // (units * other splits compared, not quotients: exact, and ties go to the earlier row)
  auto longer = [&](int a, int b) {
    const long l = units[a] * splits[b], r = units[b] * splits[a];
    return l != r ? l < r : a > b;   // priority_queue keeps the greatest on top
  };
  auto may_grow = [&](int i) { return splits[i] < MAX_SPLITS && units[i] >= MIN_UNITS * (splits[i] + 1); };
  std::priority_queue<int, std::vector<int>, decltype(longer)> heap(longer);
  for (int i = 0; i < rows; ++i)
    if (may_grow(i)) heap.push(i);
  for (long left = T - rows; left > 0 && !heap.empty(); --left) {
    const int i = heap.top();
    heap.pop();
    ++splits[i];
    if (may_grow(i)) heap.push(i);
  }
  std::vector<int> order(rows);
  for (int i = 0; i < rows; ++i) order[i] = i;
  auto piece = [&](int i) { return (units[i] + splits[i] - 1) / splits[i]; };
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return piece(a) > piece(b); });
  // the places of the partial results: a sequence's splits side by side; the items themselves in rounds (split 0 of
  // every sequence, then split 1 of those that have one, ...), so that the workgroups that run at one time belong
  // to many sequences, as they do when every sequence has the same number of splits
  std::vector<long> first(rows);
  long at = 0;
  int most = 1;
  for (int i : order) {
    first[i] = at;
    at += splits[i];
    most = std::max(most, splits[i]);
  }
  at = 0;
  for (int sp = 0; sp < most; ++sp)
    for (int i : order) {
      if (sp >= splits[i]) continue;
      int* it = items + 4 * at++;
      it[0] = i, it[1] = sp | (splits[i] << 16), it[2] = (int)first[i], it[3] = seq_len[i];
    }
  for (; at < T; ++at) {
    int* it = items + 4 * at;
    it[0] = -1, it[1] = 0, it[2] = 0, it[3] = 0;
  }
  for (int i = 0; i < rows; ++i) items[4 * T + 2 * i] = (int)first[i], items[4 * T + 2 * i + 1] = splits[i];
  return OK;
}

// A decode step of `rows` rows of which the first B are sequences (one token each) and the rest
// padding: token 0 at position 0 against a spare page that no sequence owns.  After the integer
// tables lie 2 * rows floats: temperatures and uniform numbers (0 where none are given); after
// them, for each group with item_splits[g] > 0 (item_splits may be null), the work list of the
// group's attention: rows * item_splits[g] items of four ints and rows pairs (syn_decode_items).
RT_API int syn_decode_fill(void* h, int rows, int B, const int* sids, const int* tokens, int n_groups,
                           const int* widths, const int* spare_pages, const float* temps, const float* uniforms,
                           const int* item_splits, int* host) {
  Cache* c = (Cache*)h;
  if (B > rows) return fail(MISUSE, "%d sequences for a table of %d rows", B, rows);
  const Layout l = make_layout(rows, rows, rows, n_groups, widths);
  for (int i = 0; i < rows; ++i) {
    long past = 0;
    if (i < B) {
      Slot* s = c->live_slot(sids[i]);
      if (!s) return MISUSE;
      past = s->length;
    }
    host[l.tokens + i] = i < B ? tokens[i] : 0;
    host[l.tok_seq + i] = i;
    host[l.tok_pos + i] = (int)past;
    host[l.seq_start + i] = i;
    host[l.seq_past + i] = (int)past;
    host[l.seq_len + i] = (int)past + 1;
    host[l.seq_slot + i] = i < B ? sids[i] : -1;
    host[l.want + i] = i;
  }
  host[l.seq_start + rows] = rows;
  for (int g = 0; g < n_groups; ++g) {
    int* tab = host + l.tables[g];
    const int rc = fill_table(c, g, sids, B, widths[g], spare_pages[g], tab);
    if (rc) return rc;
    // logical pages beyond a sequence's own stay inside the spare page as well
    for (long j = (long)B * widths[g]; j < (long)rows * widths[g]; ++j) tab[j] = spare_pages[g];
  }
  float* f = (float*)(host + l.total);
  for (int i = 0; i < 2 * rows; ++i) f[i] = 0.f;
  if (temps)
    for (int i = 0; i < B; ++i) f[i] = temps[i], f[rows + i] = uniforms[i];
  int* items = host + l.total + 2 * rows;
  for (int g = 0; g < n_groups && item_splits; ++g) {
    if (item_splits[g] <= 0) continue;
    const int rc = syn_decode_items(host + l.seq_len, rows, item_splits[g], c->windows[g], items);
    if (rc) return rc;
    items += 4L * rows * item_splits[g] + 2L * rows;
  }
  return OK;
}

// ------------------------------------------------------------------ Philox-4x32-10
RT_API void syn_philox_block(const uint32_t* counter, const uint32_t* key, uint32_t* out) {
  philox_block(counter, key, out);
}
RT_API void* syn_philox_new(uint64_t seed) {
  Philox* p = new Philox;
  p->key[0] = (uint32_t)seed, p->key[1] = (uint32_t)(seed >> 32);
  return p;
}
RT_API void syn_philox_delete(void* h) { delete (Philox*)h; }
RT_API uint32_t syn_philox_next_u32(void* h) { return philox_next((Philox*)h); }
// (u32 >> 8) * 2^-24, in [0, 1) (rng.rs:66-69)
RT_API float syn_philox_next_uniform(void* h) { return (float)(philox_next((Philox*)h) >> 8) * (1.0f / 16777216.0f); }
// (u32 as f32) / (u32::MAX as f32), as the multinomial sampler draws it
// (crates/synaptix-infer/src/sampling/multinomial.rs:30-32); it can be exactly 1
RT_API float syn_philox_next_multinomial_uniform(void* h) {
  return (float)philox_next((Philox*)h) / (float)0xFFFFFFFFu;
}
