#include "step_batch.h"

#include "hip_api.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <set>

#include "errors.h"

namespace mercury {

namespace {
void hip_check(hipError_t e, const char* what) {
  if (e != hipSuccess) throw KernelError(std::string(what) + ": " + hip().error_string(e));
}
}  // namespace

StepView PackedStep::view(const int32_t* device) const {
  StepView v;
  v.num_tokens = num_tokens;
  v.num_seqs = num_seqs;
  v.num_rows = num_rows;
  v.token_ids = device + off_ids;
  v.positions = device + off_positions;
  v.token_seq = device + off_token_seq;
  v.cu_q = device + off_cu_q;
  v.kv_len = device + off_kv_len;
  v.state_slots = device + off_slots;
  v.logit_rows = device + off_rows;
  for (size_t g = 0; g < off_tables.size(); ++g) v.tables.push_back(device + off_tables[g]);
  v.widths = widths;
  v.counts = counts;
  v.max_q_len = max_q_len;
  v.max_kv_len = max_kv_len;
  for (const TileList& t : tiles) {
    mk_tile_list out;
    out.group = t.group;
    out.tile_rows = t.tile_rows;
    out.count = t.count;
    out.seq = device + t.off_seq;
    out.row0 = device + t.off_row0;
    v.tiles.push_back(out);
  }
  return v;
}

int count_tiles(const std::vector<int>& counts, int group, int tile_rows) {
  int total = 0;
  for (int c : counts) total += (c * group + tile_rows - 1) / tile_rows;
  return total;
}

void build_tiles(const std::vector<int>& counts, int group, int tile_rows, std::vector<int>& seq,
                 std::vector<int>& row0) {
  for (int s = 0; s < (int)counts.size(); ++s) {
    const int n = (counts[s] * group + tile_rows - 1) / tile_rows;
    for (int i = 0; i < n; ++i) {
      seq.push_back(s);
      row0.push_back(i * tile_rows);
    }
  }
}

std::vector<int> PackedStep::layout() const {
  std::vector<int> out{num_tokens, num_seqs, num_rows};
  out.insert(out.end(), widths.begin(), widths.end());
  for (const TileList& t : tiles) {
    out.push_back(t.group);
    out.push_back(t.tile_rows);
    out.push_back(t.count);
  }
  return out;
}

StepPacker::StepPacker(std::shared_ptr<CacheManager> manager, int vocab_size, int max_positions)
    : manager_(std::move(manager)), vocab_size_(vocab_size), max_positions_(max_positions) {
  ring_.resize(4);
}

StepPacker::~StepPacker() {
  for (Slot& s : ring_) {
    if (s.event) (void)hip().event_destroy((hipEvent_t)s.event);
    if (s.data) {
      if (s.pinned) (void)hip().host_free(s.data); else std::free(s.data);
    }
  }
}

int32_t* StepPacker::acquire(size_t ints, int& slot_index) {
  slot_index = next_;
  next_ = (next_ + 1) % (int)ring_.size();
  Slot& s = ring_[slot_index];
  if (s.in_flight) {
    hip_check(hip().event_synchronize((hipEvent_t)s.event), "waiting for a step buffer's copy");
    s.in_flight = false;
  }
  if (s.capacity < ints) {
    if (s.data) {
      if (s.pinned) (void)hip().host_free(s.data); else std::free(s.data);
    }
    const size_t capacity = std::max<size_t>(ints + ints / 2, 4096);
    s.pinned = pinned_;
    if (pinned_) {
      void* p = nullptr;
      hip_check(hip().host_malloc(&p, capacity * sizeof(int32_t), hipHostMallocDefault),
                "allocating a pinned step buffer");
      s.data = (int32_t*)p;
    } else {
      s.data = (int32_t*)std::malloc(capacity * sizeof(int32_t));
      if (!s.data) throw std::bad_alloc();
    }
    s.capacity = capacity;
  }
  return s.data;
}

PackedStep StepPacker::pack(const std::vector<SeqInput>& seqs, const Program* program,
                            int table_width, bool check_ids, int kv_bound) {
  if (seqs.empty()) throw BatchError("a step needs at least one sequence");
  PackedStep p;
  const int page = manager_->page_size();
  const int groups = manager_->num_groups();
  p.num_seqs = (int)seqs.size();
  int needed = 0;
  for (const SeqInput& s : seqs) {
    if (s.count <= 0) throw BatchError("every sequence of a step needs at least one token");
    if (s.start < 0 || s.start + s.count > max_positions_) {
      throw BatchError("a sequence would reach " + std::to_string(s.start + s.count) +
                       " tokens; the limit is " + std::to_string(max_positions_));
    }
    p.firsts.push_back(p.num_tokens);
    p.counts.push_back(s.count);
    p.starts.push_back(s.start);
    p.num_tokens += s.count;
    p.num_rows += (int)s.want.size();
    p.max_q_len = std::max(p.max_q_len, s.count);
    p.max_kv_len = std::max(p.max_kv_len, s.start + s.count);
    needed = std::max(needed, (s.start + s.count + page - 1) / page);
  }
  p.max_kv_len = std::max(p.max_kv_len, kv_bound);
  const int width = table_width < 0 ? needed : table_width;
  if (width < needed) {
    throw BatchError("block tables of width " + std::to_string(width) + " cannot hold " +
                     std::to_string(needed) + " pages");
  }
  p.widths.assign((size_t)groups, width);

  std::vector<Program::TileNeed> needs;
  if (program) needs = program->tile_needs(p.counts, p.max_q_len, p.max_kv_len);

  const size_t T = (size_t)p.num_tokens, S = (size_t)p.num_seqs, R = (size_t)p.num_rows;
  size_t at = 0;
  auto take = [&](size_t n) {
    const size_t here = at;
    at += n;
    return here;
  };
  p.off_ids = take(T);
  p.off_positions = take(T);
  p.off_token_seq = take(T);
  p.off_cu_q = take(S + 1);
  p.off_kv_len = take(S);
  p.off_slots = take(S);
  p.off_rows = take(R);
  for (int g = 0; g < groups; ++g) p.off_tables.push_back(take(S * (size_t)width));
  for (const Program::TileNeed& need : needs) {
    PackedStep::TileList t;
    t.group = need.group;
    t.tile_rows = need.tile_rows;
    t.count = count_tiles(p.counts, need.group, need.tile_rows);
    t.off_seq = take((size_t)t.count);
    t.off_row0 = take((size_t)t.count);
    p.tiles.push_back(t);
  }
  p.total = at;

  int32_t* b = acquire(p.total, p.ring_slot);
  p.host = b;
  int32_t* rows = b + p.off_rows;
  size_t row_at = 0;
  for (size_t s = 0; s < S; ++s) {
    const SeqInput& in = seqs[s];
    const int first = p.firsts[s];
    for (int i = 0; i < in.count; ++i) {
      const int32_t id = in.tokens[i];
      if (check_ids && (id < 0 || id >= vocab_size_)) {
        throw BatchError("token id outside [0, " + std::to_string(vocab_size_) + ")");
      }
      b[p.off_ids + first + i] = id;
      b[p.off_positions + first + i] = in.start + i;
      b[p.off_token_seq + first + i] = (int32_t)s;
    }
    b[p.off_cu_q + s] = first;
    b[p.off_kv_len + s] = in.start + in.count;
    std::set<int> seen;
    for (int w : in.want) {
      if (w < 0 || w >= in.count) {
        throw BatchError("wanted index " + std::to_string(w) + " outside the " +
                         std::to_string(in.count) + " tokens of a sequence");
      }
      // The final norm folds the last projection's partial sums into a wanted row of the
      // residual stream; a row named twice would receive them twice.
      if (!seen.insert(w).second) {
        throw BatchError("sequence '" + in.key + "' wants the same place twice");
      }
      rows[row_at++] = first + w;
    }
    const Sequence& record = manager_->sequence(in.key);
    b[p.off_slots + s] = record.state_slot;
    if (in.start == 0) p.fresh_slots.push_back(record.state_slot);
    const int need = (in.start + in.count + page - 1) / page;
    for (int g = 0; g < groups; ++g) {
      const std::vector<int>& pages = record.tables[(size_t)g];
      if ((int)pages.size() < need) {
        throw BatchError("sequence '" + in.key + "' holds " + std::to_string(pages.size()) +
                         " pages in group " + std::to_string(g) + " but needs " + std::to_string(need));
      }
      int32_t* row = b + p.off_tables[(size_t)g] + s * (size_t)width;
      std::copy(pages.begin(), pages.begin() + need, row);
      std::fill(row + need, row + width, -1);
    }
  }
  b[p.off_cu_q + S] = p.num_tokens;
  for (const PackedStep::TileList& t : p.tiles) {
    std::vector<int> seq, row0;
    build_tiles(p.counts, t.group, t.tile_rows, seq, row0);
    std::copy(seq.begin(), seq.end(), b + t.off_seq);
    std::copy(row0.begin(), row0.end(), b + t.off_row0);
  }
  return p;
}

PackedStep StepPacker::pack_plan(const Plan& plan, const Program* program, int table_width,
                                 int kv_bound) {
  std::vector<SeqInput> seqs;
  seqs.reserve(plan.work.size());
  for (const Work& w : plan.work) {
    SeqInput in;
    in.key = w.request->rid;
    in.tokens = w.request->tokens.data() + w.start;
    in.count = w.count;
    in.start = w.start;
    if (w.emits) in.want.push_back(w.count - 1);
    seqs.push_back(std::move(in));
  }
  return pack(seqs, program, table_width, true, kv_bound);
}

void StepPacker::upload(const PackedStep& step, void* device, void* stream) {
  Slot& s = ring_.at((size_t)step.ring_slot);
  hip_check(hip().memcpy_async(device, step.host, step.total * sizeof(int32_t),
                               hipMemcpyHostToDevice, (hipStream_t)stream),
            "copying a step to the device");
  if (!s.event) {
    hipEvent_t e;
    hip_check(hip().event_create(&e, hipEventDisableTiming), "creating an event");
    s.event = e;
  }
  hip_check(hip().event_record((hipEvent_t)s.event, (hipStream_t)stream), "recording an event");
  s.in_flight = true;
}

}  // namespace mercury
