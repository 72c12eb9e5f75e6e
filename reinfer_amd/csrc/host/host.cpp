// The engine's host runtime: paged-cache bookkeeping, packing of a step's index
// arrays, and the continuous-batching scheduler. Nothing here touches the GPU.
// Python sees it as the extension module reinfer_amd._host (pybind11); the
// classes in reinfer_amd/cache and reinfer_amd/engine/scheduler are these.
//
// Cache: keys and values live in blocks of block_size tokens. Layers with the
// same needs form a group (all earlier keys, or a window of them); every group
// has a pool of its own and every request one block table per group. Blocks are
// taken lazily, when a step's tokens need them, given back when the request ends
// or, in a window group, when the window has passed them, and used again, last
// freed first (the reference's PagePool is LIFO the same way,
// crates/memory/src/pool.rs:61-155). Beside the pools: slots for per-request
// state of fixed size.
//
// Scheduler: each call of schedule() decides one step: every decoding request
// takes one token first; what is left of the token budget goes to prompt
// portions, requests already running before waiting ones, resumed ones before
// new arrivals, then first come first served (crates/scheduler/src/batch.rs:69-101,
// policy.rs:30-63). When blocks run out the newest running request that was not
// preempted before is preempted and later recomputed from its prompt plus what
// it generated (crates/scheduler/src/req.rs:340-357), so its output is what it
// would have been. Everything is a pure function of the arrival order
// (crates/scheduler/src/replay.rs:1-7).
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <deque>
#include <limits>
#include <memory>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

namespace py = pybind11;

// exception classes defined in Python (they carry attributes); set once at import, never destroyed
static py::object* E_OutOfBlocks = nullptr;
static py::object* E_OutOfSlots = nullptr;
static py::object* E_RequestRefused = nullptr;
static py::object* E_StepError = nullptr;

[[noreturn]] static void raise_instance(const py::object& cls, const py::object& inst) {
  PyErr_SetObject(cls.ptr(), inst.ptr());
  throw py::error_already_set();
}
[[noreturn]] static void out_of_blocks(int group, int need, int free_) {
  raise_instance(*E_OutOfBlocks, (*E_OutOfBlocks)(group, need, free_));
}
[[noreturn]] static void step_error(const std::string& msg) {
  raise_instance(*E_StepError, (*E_StepError)(msg));
}
[[noreturn]] static void assertion(const std::string& msg) {
  PyErr_SetString(PyExc_AssertionError, msg.c_str());
  throw py::error_already_set();
}
static std::string show(const py::handle& o) { return py::repr(o).cast<std::string>(); }

// ------------------------------------------------------------------- pools
struct BlockPool {
  int num_blocks;
  std::vector<int> free_;          // back() is handed out next
  std::vector<char> held;
  long allocs = 0, frees = 0;
  bool log_freed = false;          // a test's hook: remember which blocks came back, for poisoning them
  std::vector<int> freed_log;

  explicit BlockPool(int n) : num_blocks(n) {
    if (n <= 0) throw py::value_error("a pool needs at least one block");
    free_.reserve(n);
    for (int b = n - 1; b >= 0; --b) free_.push_back(b);      // block 0 first
    held.assign(n, 0);
  }
  int num_free() const { return (int)free_.size(); }
  int num_held() const { return num_blocks - (int)free_.size(); }
  int take() {
    if (free_.empty()) out_of_blocks(-1, 1, 0);
    const int b = free_.back();
    free_.pop_back();
    if (held[b]) assertion("block " + std::to_string(b) + " handed out twice");
    held[b] = 1;
    ++allocs;
    return b;
  }
  void give_back(int b) {
    if (b < 0 || b >= num_blocks) throw py::value_error("block " + std::to_string(b) + " is not of this pool");
    if (!held[b]) throw std::runtime_error("block " + std::to_string(b) + " freed twice");
    held[b] = 0;
    free_.push_back(b);
    ++frees;
    if (log_freed) freed_log.push_back(b);
  }
  void check() const {
    std::vector<char> seen(num_blocks, 0);
    int n_held = 0;
    for (int b : free_) {
      if (seen[b]) assertion("a block is on the free list twice");
      seen[b] = 1;
      if (held[b]) assertion("a free block is marked held");
    }
    for (char h : held) n_held += h;
    if (n_held + (int)free_.size() != num_blocks) assertion("a block is lost");
    if (allocs - frees != num_held()) assertion("allocations and frees do not add up");
  }
};

struct SlotPool {
  int num_slots;
  std::vector<int> free_;
  std::vector<char> held;
  explicit SlotPool(int n) : num_slots(n) {
    for (int s = n - 1; s >= 0; --s) free_.push_back(s);
    held.assign(std::max(n, 0), 0);
  }
  int num_free() const { return (int)free_.size(); }
  int take() {
    if (free_.empty())
      raise_instance(*E_OutOfSlots, (*E_OutOfSlots)("all " + std::to_string(num_slots) + " request slots are in use"));
    const int s = free_.back();
    free_.pop_back();
    held[s] = 1;
    return s;
  }
  void give_back(int s) {
    if (s < 0 || s >= num_slots || !held[s]) throw std::runtime_error("slot " + std::to_string(s) + " freed twice");
    held[s] = 0;
    free_.push_back(s);
  }
};

// A request's part in a step: its next tokens and where logits are wanted (indices into tokens).
struct StepEntry {
  py::object rid;
  std::vector<int> tokens;
  std::vector<int> want;
};
using StepEntryP = std::shared_ptr<StepEntry>;
using StepEntries = std::vector<StepEntryP>;

// ------------------------------------------------------------------ manager
struct RequestCache {
  int slot = 0;
  int num_tokens = 0;                          // tokens whose keys are stored
  std::vector<std::vector<int>> tables;        // per group; -1 = given back
  std::vector<int> first_live;                 // per group: first block still held
  bool fresh = true;                           // no step has run for it yet
  uint64_t serial = 0;                         // distinguishes a request from an earlier one of the same id
};

struct KeyHash {
  size_t operator()(const py::object& o) const { return (size_t)py::hash(o); }
};
struct KeyEq {
  bool operator()(const py::object& a, const py::object& b) const { return a.equal(b); }
};

struct CacheManager {
  py::list groups;                             // the CacheGroupSpec records, as given
  std::vector<int> windows;
  int block_size;
  std::vector<BlockPool> pools;
  SlotPool slots;
  std::unordered_map<py::object, std::shared_ptr<RequestCache>, KeyHash, KeyEq> requests;
  uint64_t next_serial = 1;

  CacheManager(py::list groups_, int block_size_, std::vector<int> num_blocks, int max_seqs)
      : groups(groups_), block_size(block_size_), slots(max_seqs) {
    if (block_size <= 0) throw py::value_error("block_size must be positive");
    if (num_blocks.size() != (size_t)py::len(groups)) throw py::value_error("one block count per cache group");
    for (auto g : groups) windows.push_back(g.attr("window").cast<int>());
    for (int n : num_blocks) pools.emplace_back(n);
  }
  int n_groups() const { return (int)windows.size(); }

  std::shared_ptr<RequestCache> add(const py::object& rid) {
    if (requests.count(rid)) throw py::key_error("request " + show(rid) + " is already live");
    auto rc = std::make_shared<RequestCache>();
    rc->slot = slots.take();
    rc->tables.assign(n_groups(), {});
    rc->first_live.assign(n_groups(), 0);
    rc->serial = next_serial++;
    requests.emplace(rid, rc);
    return rc;
  }
  std::shared_ptr<RequestCache> get(const py::object& rid) const {
    auto it = requests.find(rid);
    if (it == requests.end()) throw py::key_error(show(rid));
    return it->second;
  }
  bool contains(const py::object& rid) const { return requests.count(rid) != 0; }

  // Give back everything a request holds, exactly once (crates/scheduler/src/req.rs:372-378).
  void free(const py::object& rid) {
    auto it = requests.find(rid);
    if (it == requests.end()) throw py::key_error("request " + show(rid) + " is not live (freed twice?)");
    auto rc = it->second;
    requests.erase(it);
    for (int g = 0; g < n_groups(); ++g) {
      auto& t = rc->tables[g];
      for (auto b = t.rbegin(); b != t.rend(); ++b)
        if (*b >= 0) pools[g].give_back(*b);
    }
    slots.give_back(rc->slot);
  }

  // First block a query at first_query_pos can still read in group g.
  int first_needed_block(int g, int first_query_pos) const {
    const int w = windows[g];
    if (w <= 0) return 0;
    const int lo = first_query_pos - w + 1;
    return std::max(0, lo) / block_size;
  }
  // Blocks each group must still take so that tokens [stored, new_total) fit.
  void blocks_needed_into(const RequestCache& rc, int new_total, int* need) const {
    const int want = (new_total + block_size - 1) / block_size;
    for (int g = 0; g < n_groups(); ++g) {
      const int have = (int)rc.tables[g].size();
      // blocks wholly below the window of the first new query are never taken
      const int first = std::max(have, first_needed_block(g, rc.num_tokens));
      need[g] = std::max(0, want - first);
    }
  }
  std::vector<int> blocks_needed(const py::object& rid, int new_total) const {
    std::vector<int> need(n_groups());
    blocks_needed_into(*get(rid), new_total, need.data());
    return need;
  }
  bool can_grow(const std::vector<std::pair<py::object, int>>& growth) const {
    std::vector<int> total(n_groups(), 0), need(n_groups());
    for (auto& [rid, new_total] : growth) {
      blocks_needed_into(*get(rid), new_total, need.data());
      for (int g = 0; g < n_groups(); ++g) total[g] += need[g];
    }
    for (int g = 0; g < n_groups(); ++g)
      if (total[g] > pools[g].num_free()) return false;
    return true;
  }
  // Take the blocks for tokens up to new_total; all groups or none.
  void grow_rc(RequestCache& rc, int new_total) {
    if (new_total < rc.num_tokens) throw py::value_error("a request's cache does not shrink");
    std::vector<int> need(n_groups());
    blocks_needed_into(rc, new_total, need.data());
    for (int g = 0; g < n_groups(); ++g)
      if (need[g] > pools[g].num_free()) out_of_blocks(g, need[g], pools[g].num_free());
    const int want = (new_total + block_size - 1) / block_size;
    for (int g = 0; g < n_groups(); ++g) {
      auto& table = rc.tables[g];
      const int first = first_needed_block(g, rc.num_tokens);
      while ((int)table.size() < want) {
        if ((int)table.size() < first) {
          table.push_back(-1);                 // below the window from the start: never held
          rc.first_live[g] = (int)table.size();
        } else {
          table.push_back(pools[g].take());
        }
      }
    }
  }
  void grow(const py::object& rid, int new_total) { grow_rc(*get(rid), new_total); }

  // The step has stored tokens up to new_total; give back what every later query's window has passed.
  void commit_rc(RequestCache& rc, int new_total) {
    rc.num_tokens = new_total;
    rc.fresh = false;
    for (int g = 0; g < n_groups(); ++g) {
      const int first = first_needed_block(g, new_total);       // the next query sits at new_total
      auto& table = rc.tables[g];
      const int end = std::min(first, (int)table.size());
      for (int b = rc.first_live[g]; b < end; ++b)
        if (table[b] >= 0) {
          pools[g].give_back(table[b]);
          table[b] = -1;
        }
      rc.first_live[g] = std::max(rc.first_live[g], end);
    }
  }
  void commit(const py::object& rid, int new_total) { commit_rc(*get(rid), new_total); }

  // Flat cache slot (block * block_size + offset) of position pos; -1 if not held.
  int slot_of(const py::object& rid, int group, int pos) const {
    auto rc = get(rid);
    const int b = rc->tables.at(group).at(pos / block_size);
    return b < 0 ? -1 : b * block_size + pos % block_size;
  }

  // No block lost, held twice or free while held.
  void check() const {
    for (int g = 0; g < n_groups(); ++g) {
      pools[g].check();
      std::vector<char> seen(pools[g].num_blocks, 0);
      int n = 0;
      for (auto& kv : requests)
        for (int b : kv.second->tables[g])
          if (b >= 0) {
            if (seen[b]) assertion("group " + std::to_string(g) + ": a block is held by two requests");
            if (!pools[g].held[b]) assertion("group " + std::to_string(g) + ": a table names a free block");
            seen[b] = 1;
            ++n;
          }
      if (n != pools[g].num_held())
        assertion("group " + std::to_string(g) + ": " + std::to_string(pools[g].num_held()) + " held, " +
                  std::to_string(n) + " in tables");
    }
    std::vector<char> seen(std::max(slots.num_slots, 0), 0);
    for (auto& kv : requests) {
      if (seen[kv.second->slot]) assertion("a state slot is held twice");
      seen[kv.second->slot] = 1;
    }
    if ((int)requests.size() + slots.num_free() != slots.num_slots) assertion("a state slot is lost");
  }

  // A hook for tests: from now on every block given back is remembered; take_freed() hands the list of
  // each group over and forgets it. (A test fills those blocks with NaN, so that a kernel that reads a
  // slot its request no longer holds shows.)
  void log_freed(bool on) {
    for (auto& p : pools) {
      p.log_freed = on;
      p.freed_log.clear();
    }
  }
  std::vector<std::vector<int>> take_freed() {
    std::vector<std::vector<int>> out;
    for (auto& p : pools) {
      out.push_back(p.freed_log);
      p.freed_log.clear();
    }
    return out;
  }

  py::dict stats() const {
    py::dict d;
    py::list total, free_, allocs, frees;
    for (auto& p : pools) {
      total.append(p.num_blocks);
      free_.append(p.num_free());
      allocs.append(p.allocs);
      frees.append(p.frees);
    }
    d["block_size"] = block_size;
    d["live_requests"] = (int)requests.size();
    d["blocks_total"] = total;
    d["blocks_free"] = free_;
    d["allocs"] = allocs;
    d["frees"] = frees;
    return d;
  }

  // ------------------------------------------------------ a step's index arrays
  // Sizes of the packed int32 buffer of a step over `entries` (objects with rid, tokens, want):
  // -> (q_lens, starts, widths per group, wanted rows). The layout itself is the caller's.
  py::tuple step_shape(const StepEntries& entries) const {
    std::vector<int> q_lens, starts, widths(n_groups(), 1);
    int n_out = 0;
    for (auto& e : entries) {
      auto rc = get(e->rid);
      q_lens.push_back((int)e->tokens.size());
      starts.push_back(rc->num_tokens);
      n_out += (int)e->want.size();
      for (int g = 0; g < n_groups(); ++g) widths[g] = std::max(widths[g], (int)rc->tables[g].size());
    }
    return py::make_tuple(q_lens, starts, widths, n_out);
  }

  // Fill the packed buffer. `offs` holds the first element of: tokens, positions, request of each
  // token, first token of each request (n + 1), start, context length, state slot, fresh flag,
  // wanted rows, "store nothing" slots, then per group the block tables [n, width] and after all
  // tables per group the cache slot of each token.
  void fill_step(const StepEntries& entries, py::array_t<int32_t, py::array::c_style> buffer,
                 const std::vector<long>& offs, const std::vector<int>& widths) const {
    int32_t* h = buffer.mutable_data();
    const int n = (int)entries.size(), G = n_groups();
    if ((int)offs.size() != 10 + 2 * G || (int)widths.size() != G) throw py::value_error("fill_step: bad layout");
    const long o_tok = offs[0], o_pos = offs[1], o_seq = offs[2], o_cu = offs[3], o_start = offs[4], o_ctx = offs[5],
               o_state = offs[6], o_fresh = offs[7], o_rows = offs[8], o_noslot = offs[9];
    long t = 0, r = 0;
    for (int i = 0; i < n; ++i) {
      const StepEntry& e = *entries[i];
      auto rc = get(e.rid);
      const int start = rc->num_tokens, q = (int)e.tokens.size();
      for (int j = 0; j < q; ++j) {
        h[o_tok + t + j] = e.tokens[j];
        h[o_pos + t + j] = start + j;
        h[o_seq + t + j] = i;
        h[o_noslot + t + j] = -1;
      }
      h[o_cu + i] = (int32_t)t;
      h[o_start + i] = start;
      h[o_ctx + i] = start + q;
      h[o_state + i] = rc->slot;
      h[o_fresh + i] = rc->fresh ? 1 : 0;
      for (int w : e.want) h[o_rows + r++] = (int32_t)(t + w);
      for (int g = 0; g < G; ++g) {
        const auto& table = rc->tables[g];
        const long row = offs[10 + g] + (long)i * widths[g];
        // entries given back (-1) are never read by a kernel; 0 keeps every index valid
        for (size_t b = 0; b < table.size(); ++b) h[row + (long)b] = table[b] >= 0 ? table[b] : 0;
        const long o_slot = offs[10 + G + g];
        for (int j = 0; j < q; ++j) {
          const int pos = start + j;
          const int blk = table.at(pos / block_size);
          h[o_slot + t + j] = blk < 0 ? -1 : blk * block_size + pos % block_size;
        }
      }
      t += q;
    }
    h[o_cu + n] = (int32_t)t;
  }

  // Before a step: check the entries (the reference's step checks the same on the host,
  // crates/cuda/src/engine.rs:5854-5943), then take the blocks their tokens need, all or none.
  // -> (every entry brings one token, every entry wants one row, the longest context after the step)
  py::tuple begin_step(const StepEntries& entries, int vocab, int max_model_len) {
    bool one_token = true, one_want = true;
    int longest = 0;
    if (entries.empty()) step_error("a step needs at least one request");
    std::vector<RequestCache*> rcs;
    const int G = n_groups();
    std::vector<int> total(G, 0), need(G);
    for (size_t i = 0; i < entries.size(); ++i) {
      const StepEntry& e = *entries[i];
      for (size_t k = 0; k < i; ++k)
        if (entries[k]->rid.equal(e.rid)) step_error("request " + show(e.rid) + " appears twice in one step");
      auto it = requests.find(e.rid);
      if (it == requests.end()) step_error("request " + show(e.rid) + " is not live");
      if (e.tokens.empty()) step_error("request " + show(e.rid) + " brings no tokens");
      for (int tok : e.tokens)
        if (tok < 0 || tok >= vocab)
          step_error("request " + show(e.rid) + ": token " + std::to_string(tok) + " outside the vocabulary of " + std::to_string(vocab));
      for (int w : e.want)
        if (w < 0 || w >= (int)e.tokens.size())
          step_error("request " + show(e.rid) + ": logits wanted at " + std::to_string(w) + " of " + std::to_string(e.tokens.size()) + " tokens");
      RequestCache* rc = it->second.get();
      const int new_total = rc->num_tokens + (int)e.tokens.size();
      if (new_total > max_model_len)
        step_error("request " + show(e.rid) + ": " + std::to_string(new_total) + " tokens exceed the context of " + std::to_string(max_model_len));
      blocks_needed_into(*rc, new_total, need.data());
      for (int g = 0; g < G; ++g) total[g] += need[g];
      rcs.push_back(rc);
      one_token = one_token && e.tokens.size() == 1;
      one_want = one_want && e.want.size() == 1;
      longest = std::max(longest, new_total);
    }
    int worst = -1;
    for (int g = 0; g < G; ++g)
      if (total[g] > pools[g].num_free() && (worst < 0 || total[g] - pools[g].num_free() > total[worst] - pools[worst].num_free()))
        worst = g;
    if (worst >= 0) out_of_blocks(worst, total[worst], pools[worst].num_free());
    for (size_t i = 0; i < entries.size(); ++i) grow_rc(*rcs[i], rcs[i]->num_tokens + (int)entries[i]->tokens.size());
    return py::make_tuple(one_token, one_want, longest);
  }
  // After the step: its tokens are stored.
  void end_step(const StepEntries& entries) {
    for (auto& e : entries) {
      auto rc = get(e->rid);
      commit_rc(*rc, rc->num_tokens + (int)e->tokens.size());
    }
  }
};

// Rows of a captured decode step: which request sits in which row of the static buffers, and how
// much of its block tables is already there, so that a step writes only what changed.
struct DecodeRows {
  std::shared_ptr<CacheManager> manager;
  int B, W;
  std::vector<long> offs;       // token_ids, positions, start_pos, ctx_lens, state_slots, fresh, sample_pos,
                                // temps, seeds (in int32 units), then per group: table, slots
  std::vector<uint64_t> owner;  // serial of the request in each row, 0 = padding
  std::vector<std::vector<int>> row_len;

  DecodeRows(std::shared_ptr<CacheManager> m, int B_, int W_, std::vector<long> offs_)
      : manager(std::move(m)), B(B_), W(W_), offs(std::move(offs_)) {
    if ((int)offs.size() != 9 + 2 * manager->n_groups()) throw py::value_error("DecodeRows: bad layout");
    owner.assign(B, 0);
    row_len.assign(manager->n_groups(), std::vector<int>(B, 0));
  }

  void pad(int32_t* h, int lo, int hi) {
    const int G = manager->n_groups();
    for (int i = lo; i < hi; ++i) {
      h[offs[0] + i] = 0;       // token 0 at position 0 that stores nothing
      h[offs[1] + i] = 0;
      h[offs[2] + i] = 0;
      h[offs[3] + i] = 1;
      h[offs[4] + i] = -1;
      h[offs[5] + i] = 0;
      h[offs[6] + i] = 0;
      h[offs[7] + i] = 0;       // temperature 0.0f
      h[offs[8] + 2 * i] = 0;
      h[offs[8] + 2 * i + 1] = 0;
      for (int g = 0; g < G; ++g) h[offs[9 + 2 * g + 1] + i] = -1;
      owner[i] = 0;
    }
  }

  // entries: objects with rid and tokens (one each); sampling: None or (temperatures, seeds, positions)
  // The entries' blocks are already taken (begin_step): a token's position is the request's length before
  // the step.
  void fill(const StepEntries& entries, py::array_t<int32_t, py::array::c_style> buffer, const py::object& sampling) {
    int32_t* h = buffer.mutable_data();
    const int n = (int)entries.size(), G = manager->n_groups(), bs = manager->block_size;
    if (n > B) throw py::value_error("DecodeRows: more entries than rows");
    for (int i = 0; i < n; ++i) {
      const StepEntry& e = *entries[i];
      auto rc = manager->get(e.rid);
      const int p = rc->num_tokens;
      h[offs[0] + i] = e.tokens.at(0);
      h[offs[1] + i] = p;
      h[offs[2] + i] = p;
      h[offs[3] + i] = p + 1;
      h[offs[4] + i] = rc->slot;
      h[offs[5] + i] = rc->fresh ? 1 : 0;
      const bool same = owner[i] == rc->serial;
      for (int g = 0; g < G; ++g) {
        const auto& table = rc->tables[g];
        if ((int)table.size() > W) throw py::value_error("DecodeRows: block table longer than the static row");
        const int have = same ? row_len[g][i] : 0;
        int32_t* row = h + offs[9 + 2 * g] + (long)i * W;
        // entries given back (-1) are never read; 0 keeps every index valid
        for (int b = have; b < (int)table.size(); ++b) row[b] = table[b] >= 0 ? table[b] : 0;
        row_len[g][i] = (int)table.size();
        const int blk = table.at(p / bs);
        h[offs[9 + 2 * g + 1] + i] = blk < 0 ? -1 : blk * bs + p % bs;
      }
      owner[i] = rc->serial;
    }
    if (!sampling.is_none()) {
      auto s = sampling.cast<py::tuple>();
      int k = 0;
      for (auto v : s[0]) {
        const float f = v.cast<float>();
        std::memcpy(h + offs[7] + k++, &f, 4);
      }
      k = 0;
      for (auto v : s[1]) {
        const int64_t x = v.cast<int64_t>();
        std::memcpy(h + offs[8] + 2 * k++, &x, 8);
      }
      k = 0;
      for (auto v : s[2]) h[offs[6] + k++] = v.cast<int32_t>();
    } else {
      for (int k = 0; k < n; ++k) {
        h[offs[6] + k] = 0;
        h[offs[7] + k] = 0;
        h[offs[8] + 2 * k] = 0;
        h[offs[8] + 2 * k + 1] = 0;
      }
    }
    int hi = n;
    for (int k = B - 1; k >= n; --k)
      if (owner[k] != 0) {
        hi = k + 1;
        break;
      }
    if (hi > n) pad(h, n, hi);
  }
  void pad_all(py::array_t<int32_t, py::array::c_style> buffer) { pad(buffer.mutable_data(), 0, B); }
};

// --------------------------------------------------------------- scheduler
static const char* WAITING = "waiting";
static const char* RUNNING = "running";
static const char* FINISHED = "finished";

struct Request {
  py::object rid;
  std::vector<int> prompt;
  py::object params;
  py::object seed;
  long arrival = 0;
  std::string state = WAITING;
  std::vector<int> output;
  int num_computed = 0;            // tokens of prompt + output whose keys are in the cache
  bool resumed = false;            // preempted at least once
  bool aborted = false;
  py::object finish_reason = py::none();
  int preemptions = 0;
  // read once from params
  int max_tokens = 0;
  bool ignore_eos = false;
  bool filters = false;            // anything beside temperature shapes the distribution
  float temperature = 0.f;
  int64_t seed64 = 0;              // the seed's low 64 bits as the kernels take them
  std::vector<int> stop_ids;
  std::vector<std::vector<int>> stop_seqs;       // token sequences that end the request

  int num_tokens() const { return (int)(prompt.size() + output.size()); }
  int remaining() const { return num_tokens() - num_computed; }
  // in the cache up to its last token, which is a generated one
  bool decoding() const { return state == RUNNING && !output.empty() && remaining() == 1; }
  std::vector<int> tokens() const {
    std::vector<int> t(prompt);
    t.insert(t.end(), output.begin(), output.end());
    return t;
  }
  int token_at(int i) const {
    if (i < 0 || i >= num_tokens()) throw py::index_error("token index out of range");
    return i < (int)prompt.size() ? prompt[i] : output[i - prompt.size()];
  }
  std::vector<int> tokens_slice(int start, int n) const {
    std::vector<int> t;
    t.reserve(std::max(n, 0));
    for (int i = start; i < start + n; ++i) t.push_back(token_at(i));
    return t;
  }
};
using RequestP = std::shared_ptr<Request>;

struct Portion {
  RequestP request;
  int start, length;
  // where in the request's output the token of this portion goes, once the step has been launched and
  // until its token has been read (Scheduler::advance_blind / resolve); -1 otherwise
  int out_index = -1;
  // the portion reaches the request's current end: its last logits give a token (asked before the step is
  // launched: afterwards the request has grown by the token's place)
  bool samples() const { return start + length == request->num_tokens(); }
};

struct StepPlan {
  std::vector<Portion> portions;
  std::vector<RequestP> preempted;
  std::vector<RequestP> finished;      // ended without running (cache)
  int num_tokens() const {
    int n = 0;
    for (auto& p : portions) n += p.length;
    return n;
  }
};

struct Scheduler {
  std::shared_ptr<CacheManager> manager;
  int max_num_seqs, budget, max_model_len, max_chunk;
  std::vector<int> eos;
  std::deque<RequestP> waiting;
  std::vector<RequestP> running;
  std::unordered_map<py::object, RequestP, KeyHash, KeyEq> requests;
  long arrivals = 0;
  long c_steps = 0, c_preemptions = 0, c_finished = 0, c_refused = 0, c_tokens = 0, c_held_back = 0;
  // Admission by estimate (crates/scheduler/src/admission.rs:1-27): a request is let in only while the
  // peak of what the running set is expected to hold fits the pool. Without it ("blocks") a request is
  // let in as soon as its first portion's blocks are free, and a full pool preempts its way out.
  bool peak_admission = true;
  double ema_out = 2048.0;                  // output length of finished requests (admission.rs:34-37)
  static constexpr double EMA_FLOOR = 64.0, BUSY_RATIO = 0.8;     // sched_loop.rs:749
  static constexpr int ADDED_OUTPUT_LEN = 16;                     // admission.rs:31

  Scheduler(std::shared_ptr<CacheManager> m, int max_num_seqs_, int max_num_batched_tokens, int max_model_len_,
            py::object max_chunk_, std::vector<int> eos_ids, const std::string& admission)
      : manager(std::move(m)), budget(max_num_batched_tokens), max_model_len(max_model_len_), eos(std::move(eos_ids)) {
    if (max_num_seqs_ < 1 || max_num_batched_tokens < 1)
      throw py::value_error("max_num_seqs and max_num_batched_tokens must be positive");
    if (admission != "peak" && admission != "blocks")
      throw py::value_error("admission is \"peak\" (by the estimated peak of the running set) or \"blocks\" (by free blocks alone)");
    peak_admission = admission == "peak";
    max_num_seqs = std::min(max_num_seqs_, manager->slots.num_slots);
    max_chunk = (max_chunk_.is_none() || max_chunk_.cast<int>() <= 0) ? max_num_batched_tokens : max_chunk_.cast<int>();
  }

  [[noreturn]] void refuse(const std::string& why, bool count = true) {
    if (count) ++c_refused;
    raise_instance(*E_RequestRefused, (*E_RequestRefused)(why));
  }
  // Tokens the smallest pool holds. A model none of whose layers keeps keys has no pool at all: its
  // requests hold a state slot each and nothing that grows, so only the slots (and the context) bound it.
  int pool_tokens() const {
    if (manager->pools.empty()) return std::numeric_limits<int>::max() / 2;
    long n = manager->pools.at(0).num_blocks;
    for (auto& p : manager->pools) n = std::min<long>(n, p.num_blocks);
    return (int)std::min<long>(n * manager->block_size, std::numeric_limits<int>::max() / 2);
  }

  RequestP add(const py::object& rid, const std::vector<int>& prompt, const py::object& params, const py::object& seed) {
    auto it = requests.find(rid);
    if (it != requests.end() && it->second->state != FINISHED) refuse("request " + show(rid) + " is already live", false);
    const int n = (int)prompt.size();
    if (n == 0) refuse("empty prompt");
    if (n + 1 > max_model_len)
      refuse("prompt of " + std::to_string(n) + " tokens leaves no room in a context of " + std::to_string(max_model_len));
    if (n + 1 > pool_tokens())
      refuse("prompt of " + std::to_string(n) + " tokens can never fit a cache of " + std::to_string(pool_tokens()) + " tokens");
    auto req = std::make_shared<Request>();
    req->rid = rid;
    req->prompt = prompt;
    req->params = params;
    req->seed = seed;
    {
      py::int_ mask((uint64_t)0xFFFFFFFFFFFFFFFFull);
      req->seed64 = (int64_t)py::reinterpret_steal<py::int_>(PyNumber_And(seed.ptr(), mask.ptr())).cast<uint64_t>();
    }
    req->arrival = arrivals++;
    req->max_tokens = params.attr("max_tokens").cast<int>();
    req->ignore_eos = params.attr("ignore_eos").cast<bool>();
    req->filters = params.attr("filters").cast<bool>();
    req->temperature = std::max(0.f, params.attr("temperature").cast<float>());
    for (auto t : params.attr("stop_token_ids")) req->stop_ids.push_back(t.cast<int>());
    for (auto seq : params.attr("stop_sequences")) {
      std::vector<int> v;
      for (auto t : seq) v.push_back(t.cast<int>());
      if (!v.empty()) req->stop_seqs.push_back(std::move(v));      // an empty pattern never matches
    }
    requests[rid] = req;
    waiting.push_back(req);
    return req;
  }

  // Idempotent; frees once (crates/scheduler/src/req.rs:326-338).
  bool abort(const py::object& rid) {
    auto it = requests.find(rid);
    if (it == requests.end() || it->second->state == FINISHED) return false;
    auto req = it->second;
    if (req->state == RUNNING) {
      running.erase(std::find(running.begin(), running.end(), req));
      manager->free(rid);
    } else {
      waiting.erase(std::find(waiting.begin(), waiting.end(), req));
    }
    req->state = FINISHED;
    req->aborted = true;
    req->finish_reason = py::str("abort");
    forget(req);
    return true;
  }
  // A finished request leaves the table: whoever holds the Request object keeps it alive, the
  // scheduler keeps nothing of it (a long-running engine's memory does not grow with requests served).
  void forget(const RequestP& req) {
    auto it = requests.find(req->rid);
    if (it != requests.end() && it->second == req) requests.erase(it);
  }
  bool has_work() const { return !waiting.empty() || !running.empty(); }

  // (a, b) of a request: a = tokens it holds once its current tokens are in the cache, plus one;
  // b = new tokens it is expected to add yet: all it may when the pool is busy, else up to the
  // larger of 1.1 x what it has generated and the running mean of finished requests' lengths, plus a
  // slack of 16 (admission.rs:72-86; the reference counts the generated tokens in a and again in b,
  // here b is what is still to come; its term for steps that a portioned prompt waits between
  // portions is left out: no step here runs without the waiting portions).
  std::pair<long, long> estimate(const Request& r, bool busy) const {
    const long gen = (long)r.output.size();
    const long a = (long)r.num_tokens() + 1;
    long total = r.max_tokens;
    if (!busy) total = std::min<long>(total, std::max<long>((long)std::ceil(1.1 * gen), (long)ema_out));
    total = std::min<long>(total, std::max(0, max_model_len - (int)r.prompt.size()));
    return {a, std::max<long>(0, total - gen) + ADDED_OUTPUT_LEN};
  }
  // The most tokens the set will hold at one time if every request adds its b and then leaves: sorted
  // by b descending, max over k of b[k] * (k + 1) + a[0] + ... + a[k] (admission.rs:138-148).
  static long peak_tokens(std::vector<std::pair<long, long>> set) {
    std::stable_sort(set.begin(), set.end(), [](const std::pair<long, long>& x, const std::pair<long, long>& y) { return x.second > y.second; });
    long peak = 0, cur = 0;
    for (size_t k = 0; k < set.size(); ++k) {
      cur += set[k].first;
      peak = std::max(peak, set[k].second * (long)(k + 1) + cur);
    }
    return peak;
  }
  bool busy() const {
    double worst = 0.0;
    for (auto& p : manager->pools)
      worst = std::max(worst, 1.0 - (double)p.num_free() / std::max(1, p.num_blocks));
    return worst >= BUSY_RATIO;
  }
  // May `cand` join `set` (estimates of the running requests)? Busy: everything at once must fit;
  // otherwise the peak must (admission.rs:211-240). A request's last block may be partly empty.
  bool estimate_admits(const std::vector<std::pair<long, long>>& set, const std::pair<long, long>& cand, bool is_busy) const {
    std::vector<std::pair<long, long>> all(set);
    all.push_back(cand);
    const long pool = (long)pool_tokens() - (long)all.size() * (manager->block_size - 1);
    if (is_busy) {
      long sum = 0;
      for (auto& e : all) sum += e.first + e.second;
      if (sum > pool) return false;
    }
    return peak_tokens(std::move(all)) <= pool;
  }
  void observe_output(long n) {
    // running mean of output lengths: slow to fall, quicker to rise, never below 64 (admission.rs:113-126)
    const double alpha = (double)n > ema_out ? 0.9 : 0.6;
    ema_out = std::max(EMA_FLOOR, alpha * ema_out + (1.0 - alpha) * (double)n);
  }

  void preempt(const RequestP& req, StepPlan& plan) {
    running.erase(std::find(running.begin(), running.end(), req));
    manager->free(req->rid);
    req->state = WAITING;
    req->num_computed = 0;
    req->resumed = true;
    ++req->preemptions;
    ++c_preemptions;
    waiting.push_front(req);
    plan.preempted.push_back(req);
  }

  StepPlan schedule() {
    StepPlan plan;
    const int G = manager->n_groups();
    int left = budget;
    std::vector<int> need(G), one(G), free_(G);
    auto read_free = [&]() {
      for (int g = 0; g < G; ++g) free_[g] = manager->pools[g].num_free();
    };

    // 1. decoding requests: one token each; make room by preempting the newest
    while (true) {
      std::fill(need.begin(), need.end(), 0);
      int n_dec = 0;
      for (auto& r : running)
        if (r->decoding()) {
          ++n_dec;
          manager->blocks_needed_into(*manager->get(r->rid), r->num_computed + 1, one.data());
          for (int g = 0; g < G; ++g) need[g] += one[g];
        }
      read_free();
      bool is_short = n_dec > left;
      for (int g = 0; g < G; ++g) is_short = is_short || need[g] > free_[g];
      if (!is_short) break;
      if (running.size() == 1) {
        auto lone = running[0];
        running.clear();
        manager->free(lone->rid);
        lone->state = FINISHED;
        lone->finish_reason = py::str("cache");
        ++c_finished;
        forget(lone);
        plan.finished.push_back(lone);
        break;
      }
      // victims: not yet preempted first, newest arrival first (policy.rs:59-63)
      RequestP victim = running[0];
      for (auto& r : running)
        if (std::make_pair(r->resumed, -r->arrival) < std::make_pair(victim->resumed, -victim->arrival)) victim = r;
      preempt(victim, plan);
    }
    std::vector<RequestP> by_arrival(running);
    std::sort(by_arrival.begin(), by_arrival.end(), [](const RequestP& a, const RequestP& b) { return a->arrival < b->arrival; });
    read_free();
    for (auto& r : by_arrival)
      if (r->decoding()) {
        manager->blocks_needed_into(*manager->get(r->rid), r->num_computed + 1, one.data());
        for (int g = 0; g < G; ++g) free_[g] -= one[g];
        plan.portions.push_back(Portion{r, r->num_computed, 1});
        --left;
      }

    // Largest portion <= want whose blocks are free (leaving `reserve` blocks in every group); takes them from free_.
    const int bs = manager->block_size;
    auto fit = [&](const RequestP& req, int start, int want, bool live, int reserve) {
      int n = want;
      while (n > 0) {
        if (live) {
          manager->blocks_needed_into(*manager->get(req->rid), start + n, one.data());
        } else {
          for (int g = 0; g < G; ++g) one[g] = (start + n + bs - 1) / bs;
        }
        bool ok = true;
        for (int g = 0; g < G; ++g) ok = ok && one[g] + reserve <= free_[g];
        if (ok) {
          for (int g = 0; g < G; ++g) free_[g] -= one[g];
          return n;
        }
        // shrink to the last block edge that fits
        n = std::min(n - 1, ((start + n - 1) / bs) * bs - start);
      }
      return 0;
    };

    // 2. prompt portions of running requests, oldest first. If nothing at all can be placed (every
    // running request is in the middle of its prompt and the pool is full, so that step 1 had nobody to
    // make room for), the newest request that was not preempted before goes back to the queue and its
    // blocks serve the others; a lone request that cannot get a block ends with reason `cache`.
    while (true) {
      for (auto& r : by_arrival) {
        if (r->decoding()) continue;
        if (left <= 0) break;
        const int n = fit(r, r->num_computed, std::min({r->remaining(), max_chunk, left}), true, 0);
        if (n > 0) {
          plan.portions.push_back(Portion{r, r->num_computed, n});
          left -= n;
        }
      }
      if (!plan.portions.empty() || running.empty() || left <= 0) break;
      if (running.size() == 1) {
        // it may still be admitted again below if it was the pool's only holder: only a request that
        // holds the whole pool and still needs more ends here
        auto lone = running[0];
        running.clear();
        manager->free(lone->rid);
        lone->state = FINISHED;
        lone->finish_reason = py::str("cache");
        ++c_finished;
        forget(lone);
        plan.finished.push_back(lone);
        break;
      }
      RequestP victim = running[0];
      for (auto& r : running)
        if (std::make_pair(r->resumed, -r->arrival) < std::make_pair(victim->resumed, -victim->arrival)) victim = r;
      preempt(victim, plan);
      by_arrival.erase(std::find(by_arrival.begin(), by_arrival.end(), victim));
      read_free();
    }

    // 3. admissions: resumed first (they sit at the head), then arrival order
    std::vector<std::pair<long, long>> working;
    const bool is_busy = peak_admission && busy();
    if (peak_admission && !waiting.empty())
      for (auto& r : running) working.push_back(estimate(*r, is_busy));
    while (!waiting.empty() && left > 0 && (int)running.size() < max_num_seqs) {
      auto r = waiting.front();
      if (std::find(plan.preempted.begin(), plan.preempted.end(), r) != plan.preempted.end())
        break;                      // preempted in this very step: not before the next
      if (peak_admission && !running.empty()) {      // a lone request always runs: add() saw that it can fit
        const auto e = estimate(*r, is_busy);
        if (!estimate_admits(working, e, is_busy)) {
          ++c_held_back;
          break;
        }
        working.push_back(e);
      } else if (peak_admission) {
        working.push_back(estimate(*r, is_busy));
      }
      // a block of headroom for every running request, so that an admission does not force a
      // preemption at the very next step
      const int n = fit(r, 0, std::min({r->remaining(), max_chunk, left}), false, (int)running.size());
      if (n == 0) break;            // first come first served: nobody overtakes
      waiting.pop_front();
      manager->add(r->rid);
      r->state = RUNNING;
      running.push_back(r);
      plan.portions.push_back(Portion{r, 0, n});
      left -= n;
    }

    // requests keep their order in the batch: by arrival (batch.rs:13-15 sorts by id)
    std::stable_sort(plan.portions.begin(), plan.portions.end(),
                     [](const Portion& a, const Portion& b) { return a.request->arrival < b.request->arrival; });
    ++c_steps;
    c_tokens += plan.num_tokens();
    return plan;
  }

  // The step ran: advance cursors, append sampled tokens, finish and free. Order of the checks:
  // stop ids, then the cap on new tokens, then the context (crates/scheduler/src/req.rs:281-314);
  // the stop token is consumed, not emitted.
  std::vector<RequestP> complete(StepPlan& plan, const py::dict& sampled) {
    std::vector<int> tokens;
    for (auto& p : plan.portions)
      if (p.samples()) tokens.push_back(sampled[p.request->rid].cast<int>());
    return complete_tokens(plan, tokens);
  }
  // The same with the sampled tokens as a list in the order of the portions that sample.
  std::vector<RequestP> complete_tokens(StepPlan& plan, const std::vector<int>& tokens) {
    advance_blind(plan);
    return resolve(plan, tokens);
  }

  // The two halves of complete_tokens, for a caller that launches the next step before it has read this
  // one's tokens. advance_blind: the step has been launched; cursors move, every request that samples
  // grows by the place of its token (its value comes later), and what does not depend on the value is
  // decided now: the cap on new tokens and the context end a request here, and its blocks go back at once
  // (work queued on the GPU's stream before this moment is done before anything a later step launches).
  // resolve: the tokens have been read; they take their places, and a token that stops its request (an
  // end-of-sequence id, a stop id, the last of a stop sequence) cuts the output off before itself, together
  // with whatever place a later step already added behind it: that step computed a row for a request that
  // had ended, and the row is dropped. -> the requests whose end is known now, in the order of the portions.
  static constexpr int TOKEN_PLACE = 0;        // what stands in an output until its token is read
  void retire(const RequestP& r) {
    if (r->state == RUNNING) {
      running.erase(std::find(running.begin(), running.end(), r));
      manager->free(r->rid);
    } else if (r->state == WAITING) {            // preempted since: it holds nothing
      auto it = std::find(waiting.begin(), waiting.end(), r);
      if (it != waiting.end()) waiting.erase(it);
    }
    r->state = FINISHED;
    ++c_finished;
    forget(r);
  }
  void advance_blind(StepPlan& plan) {
    for (auto& p : plan.portions) {
      auto& r = p.request;
      if (r->state != RUNNING) continue;         // aborted, or ended by an earlier token, since the plan was made
      const bool samples = p.samples();          // before the cursor and the output move
      r->num_computed = p.start + p.length;
      if (!samples) continue;
      p.out_index = (int)r->output.size();
      r->output.push_back(TOKEN_PLACE);
      if ((int)r->output.size() >= r->max_tokens || r->num_tokens() >= max_model_len) {
        r->finish_reason = py::str("length");
        retire(r);
      }
    }
  }
  std::vector<RequestP> resolve(StepPlan& plan, const std::vector<int>& tokens) {
    std::vector<RequestP> done;
    size_t next = 0;
    for (auto& p : plan.portions) {
      if (p.out_index < 0) continue;
      if (next >= tokens.size()) throw py::value_error("complete: fewer tokens than portions that sample");
      const int tok = tokens[next++];
      auto& r = p.request;
      const int idx = p.out_index;
      p.out_index = -1;
      if (r->aborted || idx >= (int)r->output.size()) continue;     // gone, or cut off by an earlier step's stop
      r->output[idx] = tok;
      const bool is_eos = std::find(eos.begin(), eos.end(), tok) != eos.end();
      // A stop sequence fires the moment it is a suffix of the generated stream; its last token is
      // consumed like a stop id, the ones before it were emitted (crates/scheduler/src/stop.rs:1-12,
      // req.rs:281-300).
      bool seq_stop = false;
      for (auto& pat : r->stop_seqs) {
        const size_t L = pat.size();
        if (tok != pat[L - 1] || (size_t)idx + 1 < L) continue;
        if (std::equal(pat.begin(), pat.end() - 1, r->output.begin() + (idx + 1 - L))) {
          seq_stop = true;
          break;
        }
      }
      const bool stop = seq_stop || (is_eos && !r->ignore_eos) ||
                        std::find(r->stop_ids.begin(), r->stop_ids.end(), tok) != r->stop_ids.end();
      if (stop) {
        r->output.resize(idx);
        r->finish_reason = py::str("stop");
        if (r->state != FINISHED) retire(r);     // (ended by the cap already: the stop wins, as it is checked first)
      } else if (!(r->state == FINISHED && idx == (int)r->output.size() - 1)) {
        continue;                                // goes on; or ended by the cap with a later token still to come
      }
      observe_output((long)r->output.size());
      done.push_back(r);
    }
    return done;
  }

  // The plan as the step function takes it: one entry per portion, logits wanted at a portion's last
  // token where it reaches the request's end. -> (entries, requests that sample in entry order,
  // (temperatures, seeds, positions) if every entry samples and none uses filters, else None)
  py::tuple entries_for(const StepPlan& plan) const {
    StepEntries entries;
    std::vector<RequestP> rows;
    bool plain = true;
    for (auto& p : plan.portions) {
      if (p.request->state != RUNNING) continue;      // ended by a token that was read after the plan was made
      auto e = std::make_shared<StepEntry>();
      e->rid = p.request->rid;
      e->tokens = p.request->tokens_slice(p.start, p.length);
      if (p.samples()) {
        e->want.push_back(p.length - 1);
        rows.push_back(p.request);
        plain = plain && !p.request->filters;
      } else {
        plain = false;
      }
      entries.push_back(std::move(e));
    }
    py::object sampling = py::none();
    if (plain && !rows.empty()) {
      py::list temps, seeds, positions;
      for (auto& r : rows) {
        temps.append(r->temperature);
        seeds.append(r->seed64);
        positions.append(r->num_tokens());
      }
      sampling = py::make_tuple(temps, seeds, positions);
    }
    return py::make_tuple(entries, rows, sampling);
  }

  // Whether `next` is `prev` over again: the same requests in the same rows, one token each, every token drawn
  // without a filter. Such a step can be launched before the tokens of `prev` have been read.
  bool repeats(const StepPlan& prev, const StepPlan& next) const {
    if (next.portions.empty() || next.portions.size() != prev.portions.size()) return false;
    for (size_t i = 0; i < next.portions.size(); ++i) {
      const Portion& p = next.portions[i];
      if (p.request != prev.portions[i].request || p.length != 1 || !p.samples() || p.request->filters ||
          p.request->state != RUNNING)
        return false;
    }
    return true;
  }

  py::dict counters() const {
    py::dict d;
    d["steps"] = c_steps;
    d["preemptions"] = c_preemptions;
    d["finished"] = c_finished;
    d["refused"] = c_refused;
    d["tokens"] = c_tokens;
    d["held_back"] = c_held_back;
    return d;
  }
};

PYBIND11_MODULE(_host, m) {
  m.doc() = "host runtime of reinfer_amd: cache bookkeeping, step packing, scheduler";
  m.def("set_exceptions", [](py::object oob, py::object oos, py::object refused, py::object step) {
    E_OutOfBlocks = new py::object(std::move(oob));
    E_OutOfSlots = new py::object(std::move(oos));
    E_RequestRefused = new py::object(std::move(refused));
    E_StepError = new py::object(std::move(step));
  });

  py::class_<StepEntry, StepEntryP>(m, "StepEntry", "A request's part in a step: its next tokens and where logits are wanted.")
      .def(py::init([](py::object rid, std::vector<int> tokens, std::vector<int> want) {
             auto e = std::make_shared<StepEntry>();
             e->rid = std::move(rid);
             e->tokens = std::move(tokens);
             e->want = std::move(want);
             return e;
           }),
           py::arg("rid"), py::arg("tokens"), py::arg("want") = std::vector<int>())
      .def_readonly("rid", &StepEntry::rid)
      .def_readonly("tokens", &StepEntry::tokens)
      .def_readonly("want", &StepEntry::want)
      .def_property_readonly("num_tokens", [](const StepEntry& e) { return e.tokens.size(); })
      .def("__repr__", [](const StepEntry& e) {
        return "StepEntry(" + show(e.rid) + ", " + std::to_string(e.tokens.size()) + " tokens, " +
               std::to_string(e.want.size()) + " wanted)";
      });
  m.attr("WAITING") = WAITING;
  m.attr("RUNNING") = RUNNING;
  m.attr("FINISHED") = FINISHED;

  py::class_<BlockPool>(m, "BlockPool", "Fixed set of block ids with a LIFO free list; every misuse is an error.")
      .def(py::init<int>(), py::arg("num_blocks"))
      .def_readonly("num_blocks", &BlockPool::num_blocks)
      .def_property_readonly("num_free", &BlockPool::num_free)
      .def_property_readonly("num_held", &BlockPool::num_held)
      .def_readonly("allocs", &BlockPool::allocs)
      .def_readonly("frees", &BlockPool::frees)
      .def("take", &BlockPool::take)
      .def("give_back", &BlockPool::give_back)
      .def("is_held", [](const BlockPool& p, int b) { return b >= 0 && b < p.num_blocks && p.held[b]; })
      .def("check", &BlockPool::check);

  py::class_<SlotPool>(m, "SlotPool", "Ids for per-request state of fixed size.")
      .def(py::init<int>(), py::arg("num_slots"))
      .def_readonly("num_slots", &SlotPool::num_slots)
      .def_property_readonly("num_free", &SlotPool::num_free)
      .def("take", &SlotPool::take)
      .def("give_back", &SlotPool::give_back);

  py::class_<RequestCache, std::shared_ptr<RequestCache>>(m, "RequestCache")
      .def_readonly("slot", &RequestCache::slot)
      .def_readwrite("num_tokens", &RequestCache::num_tokens)
      .def_readonly("tables", &RequestCache::tables)
      .def_readonly("first_live", &RequestCache::first_live)
      .def_readwrite("fresh", &RequestCache::fresh);

  py::class_<CacheManager, std::shared_ptr<CacheManager>>(m, "CacheManager")
      .def(py::init<py::list, int, std::vector<int>, int>(), py::arg("groups"), py::arg("block_size"),
           py::arg("num_blocks"), py::arg("max_seqs"))
      .def_readonly("groups", &CacheManager::groups)
      .def_readonly("block_size", &CacheManager::block_size)
      .def_property_readonly("pools", [](py::object self) {
        auto& c = self.cast<CacheManager&>();
        py::list out;                  // every element keeps the manager alive
        for (auto& p : c.pools) out.append(py::cast(&p, py::return_value_policy::reference_internal, self));
        return out;
      })
      .def_property_readonly("slots", [](CacheManager& c) { return &c.slots; }, py::return_value_policy::reference_internal)
      .def("add", &CacheManager::add, py::arg("rid"))
      .def("get", &CacheManager::get, py::arg("rid"))
      .def("__contains__", &CacheManager::contains)
      .def("free", &CacheManager::free)
      .def("blocks_needed", &CacheManager::blocks_needed)
      .def("can_grow", &CacheManager::can_grow)
      .def("grow", &CacheManager::grow)
      .def("commit", &CacheManager::commit)
      .def("slot_of", &CacheManager::slot_of)
      .def("check", &CacheManager::check)
      .def("stats", &CacheManager::stats)
      .def("log_freed", &CacheManager::log_freed, py::arg("on") = true)
      .def("take_freed", &CacheManager::take_freed)
      .def("step_shape", &CacheManager::step_shape)
      .def("fill_step", &CacheManager::fill_step)
      .def("begin_step", &CacheManager::begin_step, py::arg("entries"), py::arg("vocab"), py::arg("max_model_len"))
      .def("end_step", &CacheManager::end_step, py::arg("entries"));

  py::class_<DecodeRows>(m, "DecodeRows")
      .def(py::init<std::shared_ptr<CacheManager>, int, int, std::vector<long>>())
      .def("fill", &DecodeRows::fill)
      .def("pad_all", &DecodeRows::pad_all);

  py::class_<Request, RequestP>(m, "Request")
      .def_readonly("rid", &Request::rid)
      .def_readonly("prompt", &Request::prompt)
      .def_readonly("params", &Request::params)
      .def_readonly("seed", &Request::seed)
      .def_readonly("arrival", &Request::arrival)
      .def_readwrite("state", &Request::state)
      .def_readonly("output", &Request::output)
      .def_readwrite("num_computed", &Request::num_computed)
      .def_readwrite("resumed", &Request::resumed)
      .def_readwrite("finish_reason", &Request::finish_reason)
      .def_readwrite("preemptions", &Request::preemptions)
      .def_property_readonly("prompt_len", [](const Request& r) { return (int)r.prompt.size(); })
      .def_property_readonly("tokens", &Request::tokens)
      .def_property_readonly("num_tokens", &Request::num_tokens)
      .def_property_readonly("remaining", &Request::remaining)
      .def_property_readonly("decoding", &Request::decoding)
      .def("token_at", &Request::token_at)
      .def("tokens_slice", &Request::tokens_slice);

  py::class_<Portion>(m, "Portion")
      .def_readonly("request", &Portion::request)
      .def_readonly("start", &Portion::start)
      .def_readonly("length", &Portion::length)
      .def_property_readonly("samples", &Portion::samples);

  py::class_<StepPlan>(m, "StepPlan")
      .def_readonly("portions", &StepPlan::portions)
      .def_readonly("preempted", &StepPlan::preempted)
      .def_readonly("finished", &StepPlan::finished)
      .def_property_readonly("num_tokens", &StepPlan::num_tokens);

  py::class_<Scheduler>(m, "Scheduler")
      .def(py::init<std::shared_ptr<CacheManager>, int, int, int, py::object, std::vector<int>, const std::string&>(),
           py::arg("manager"), py::kw_only(), py::arg("max_num_seqs"), py::arg("max_num_batched_tokens"),
           py::arg("max_model_len"), py::arg("max_chunk") = py::none(), py::arg("eos_token_ids") = std::vector<int>(),
           py::arg("admission") = "peak")
      .def_readonly("peak_admission", &Scheduler::peak_admission)
      .def_readonly("ema_out", &Scheduler::ema_out)
      .def("estimate", [](const Scheduler& s, const RequestP& r, bool busy) { return s.estimate(*r, busy); }, py::arg("request"), py::arg("busy") = false)
      .def_static("peak_tokens", &Scheduler::peak_tokens, py::arg("estimates"))
      .def("observe_output", &Scheduler::observe_output, py::arg("length"))
      .def_readonly("manager", &Scheduler::manager)
      .def_readonly("max_num_seqs", &Scheduler::max_num_seqs)
      .def_readonly("budget", &Scheduler::budget)
      .def_readonly("max_model_len", &Scheduler::max_model_len)
      .def_readonly("max_chunk", &Scheduler::max_chunk)
      .def_property_readonly("waiting", [](const Scheduler& s) { return std::vector<RequestP>(s.waiting.begin(), s.waiting.end()); })
      .def_readonly("running", &Scheduler::running)
      .def_property_readonly("requests", [](const Scheduler& s) {
        py::dict d;
        for (auto& kv : s.requests) d[kv.first] = kv.second;
        return d;
      })
      .def_property_readonly("num_arrivals", [](const Scheduler& s) { return s.arrivals; })
      .def_property_readonly("counters", &Scheduler::counters)
      .def("pool_tokens", &Scheduler::pool_tokens)
      .def("add", &Scheduler::add, py::arg("rid"), py::arg("prompt"), py::arg("params"), py::arg("seed"))
      .def("abort", &Scheduler::abort, py::arg("rid"))
      .def("has_work", &Scheduler::has_work)
      .def("schedule", &Scheduler::schedule)
      .def("entries_for", &Scheduler::entries_for, py::arg("plan"))
      .def("complete", &Scheduler::complete, py::arg("plan"), py::arg("sampled"))
      .def("complete_tokens", &Scheduler::complete_tokens, py::arg("plan"), py::arg("tokens"))
      .def("advance_blind", &Scheduler::advance_blind, py::arg("plan"))
      .def("repeats", &Scheduler::repeats, py::arg("prev"), py::arg("next"))
      .def("resolve", &Scheduler::resolve, py::arg("plan"), py::arg("tokens"));
}
