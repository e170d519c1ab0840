// Python bindings of the host core (module `mercury_host`).
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <cmath>

#include "cache_manager.h"
#include "engine_core.h"
#include "fill.h"
#include "hashing.h"
#include "page_pool.h"
#include "scheduler.h"

namespace py = pybind11;
using namespace mercury;

void bind_program(py::module_& m);    // operation kinds, programs, the step packer
void bind_ops(py::module_& m);        // the built-in operations (csrc/ops)

namespace {

py::int_ hash_to_py(const PageHash& h) {
  if (h.hi == 0) return py::int_(h.lo);
  return py::reinterpret_steal<py::int_>(
      PyNumber_Or(py::int_(h.lo).ptr(),
                  py::reinterpret_steal<py::object>(
                      PyNumber_Lshift(py::int_(h.hi).ptr(), py::int_(64).ptr())).ptr()));
}

PageHash hash_from_py(const py::handle& obj) {
  PageHash h;
  py::int_ value = py::reinterpret_borrow<py::int_>(obj);
  static const py::int_ mask(0xFFFFFFFFFFFFFFFFull);
  h.lo = py::cast<uint64_t>(value.attr("__and__")(mask));
  h.hi = py::cast<uint64_t>(value.attr("__rshift__")(64).attr("__and__")(mask));
  return h;
}

std::vector<PageHash> chain_from_py(const py::handle& seq) {
  std::vector<PageHash> out;
  for (const py::handle& item : seq) out.push_back(hash_from_py(item));
  return out;
}

py::list chain_to_py(const std::vector<PageHash>& chain) {
  py::list out;
  for (const PageHash& h : chain) out.append(hash_to_py(h));
  return out;
}

std::vector<int32_t> tokens_from_py(const py::handle& seq) {
  std::vector<int32_t> out;
  out.reserve((size_t)py::len(seq));
  for (const py::handle& item : seq) out.push_back(py::cast<int32_t>(item));
  return out;
}

std::string key_of(const py::handle& key) { return py::cast<std::string>(py::str(key)); }

py::object time_or_none(double t) {
  if (std::isnan(t)) return py::none();
  return py::float_(t);
}

py::dict pool_snapshot(const PagePool& pool) {
  py::dict d;
  const PagePool::Stats& s = pool.stats();
  d["num_blocks"] = pool.num_pages();
  d["block_size"] = pool.page_size();
  d["free_blocks"] = pool.num_free();
  d["evictable_blocks"] = pool.num_idle();
  d["available_blocks"] = pool.available();
  d["cached_blocks"] = pool.num_indexed();
  d["hit_rate"] = pool.hit_rate();
  d["hit_tokens"] = s.hit_tokens;
  d["query_tokens"] = s.query_tokens;
  d["evictions"] = s.evictions;
  d["prefills"] = s.prefills;
  d["allocation_failures"] = s.allocation_failures;
  return d;
}

py::dict pool_stats(const PagePool& pool) {
  py::dict d;
  const PagePool::Stats& s = pool.stats();
  d["hit_tokens"] = s.hit_tokens;
  d["query_tokens"] = s.query_tokens;
  d["evictions"] = s.evictions;
  d["prefills"] = s.prefills;
  d["allocation_failures"] = s.allocation_failures;
  return d;
}

GroupSpec spec_from_py(const py::handle& obj) {
  py::tuple t = py::hasattr(obj, "as_tuple") ? py::tuple(obj.attr("as_tuple")())
                                              : py::reinterpret_borrow<py::tuple>(obj);
  if (t.size() != 5) throw py::value_error("a cache need is (kv_heads, k_dim, v_dim, dtype, window)");
  GroupSpec s;
  s.kv_heads = py::cast<int>(t[0]);
  s.k_dim = py::cast<int>(t[1]);
  s.v_dim = py::cast<int>(t[2]);
  s.dtype = py::cast<int>(t[3]);
  s.window = py::cast<int>(t[4]);
  return s;
}

py::tuple spec_to_py(const GroupSpec& s) {
  return py::make_tuple(s.kv_heads, s.k_dim, s.v_dim, s.dtype, s.window);
}

SchedulerOptions scheduler_options(const std::string& policy, int max_running, int prefill_budget,
                                   double aging, double max_wait, int scan_limit) {
  SchedulerOptions o;
  o.policy = parse_policy(policy);
  o.max_running = max_running;
  o.prefill_budget = prefill_budget;
  o.aging_tokens_per_s = aging;
  o.max_wait_s = max_wait;
  o.scan_limit = scan_limit;
  return o;
}

const char* policy_name(Policy p) {
  return p == Policy::FCFS ? "fcfs" : p == Policy::LPM ? "lpm" : "lpm_aging";
}

py::dict scheduler_stats(const Scheduler& s) {
  py::dict d;
  const Scheduler::Stats& st = s.stats();
  d["steps"] = st.steps;
  d["sched_seconds"] = st.sched_seconds;
  d["preemptions"] = st.preemptions;
  d["admissions"] = st.admissions;
  d["max_waiting"] = st.max_waiting;
  d["scan_limit_exceeded"] = st.scan_limit_exceeded;
  d["scored_requests"] = st.scored_requests;
  return d;
}

py::dict request_record(const RequestRecord& r) {
  py::dict d;
  d["rid"] = r.rid;
  d["session_id"] = r.has_session ? py::object(py::str(r.session_id)) : py::object(py::none());
  d["arrival"] = r.arrival;
  d["admitted_at"] = time_or_none(r.admitted_at);
  d["first_token_at"] = time_or_none(r.first_token_at);
  d["finished_at"] = time_or_none(r.finished_at);
  d["queue_delay"] = std::isnan(r.admitted_at) ? py::object(py::none())
                                               : py::object(py::float_(r.admitted_at - r.arrival));
  d["prompt_tokens"] = r.prompt_tokens;
  d["output_tokens"] = r.output_tokens;
  d["cached_tokens"] = r.cached_tokens;
  d["recomputed_tokens"] = r.recomputed_tokens;
  d["preemptions"] = r.preemptions;
  d["finish_reason"] = r.finish_reason.empty() ? py::object(py::none())
                                               : py::object(py::str(r.finish_reason));
  d["state"] = r.state;
  return d;
}

}  // namespace

PYBIND11_MODULE(mercury_host, m) {
  m.doc() = "Host core of mercury_amd: cache pages, scheduling, step packing, kernel launches";
  py::register_exception<PoolError>(m, "PagePoolError", PyExc_AssertionError);
  py::register_exception<UnknownSequence>(m, "UnknownSequence", PyExc_KeyError);

  m.def("sha256", [](py::bytes data) {
    std::string s = data;
    uint8_t out[32];
    sha256(reinterpret_cast<const uint8_t*>(s.data()), s.size(), out);
    return py::bytes(reinterpret_cast<const char*>(out), 32);
  });
  m.def("fill_normal", [](uintptr_t out, int dtype, int64_t count, uint64_t key, float mean, float std) {
    py::gil_scoped_release release;
    fill_normal(reinterpret_cast<void*>(out), dtype, count, key, mean, std);
  }, "out[i] = mean + std * normal(key, i) in host memory; dtype 0 float32, 1 bfloat16");

  py::class_<PageHasher, std::shared_ptr<PageHasher>>(m, "PageHasher")
      .def(py::init<int, bool>(), py::arg("page_size"), py::arg("cryptographic") = false)
      .def_property_readonly("page_size", &PageHasher::page_size)
      .def_property_readonly("cryptographic", &PageHasher::strong)
      .def("page_hash", [](const PageHasher& h, py::handle parent, py::handle tokens) {
        auto t = tokens_from_py(tokens);
        return hash_to_py(h.page(hash_from_py(parent), t.data(), (int)t.size()));
      })
      .def("hashes", [](const PageHasher& h, py::handle tokens) {
        auto t = tokens_from_py(tokens);
        return chain_to_py(h.chain(t.data(), t.size()));
      }, "One hash per full page of the tokens.")
      .def("extend", [](const PageHasher& h, py::list hashes, py::handle tokens) {
        auto t = tokens_from_py(tokens);
        auto chain = chain_from_py(hashes);
        const size_t before = chain.size();
        const int added = h.extend(chain, t.data(), t.size());
        for (size_t i = before; i < chain.size(); ++i) hashes.append(hash_to_py(chain[i]));
        return added;
      }, "Grow `hashes` in place to cover every full page of the tokens; returns pages added.");

  py::class_<PagePool>(m, "PagePool")
      .def(py::init<int, int>(), py::arg("num_pages"), py::arg("page_size"))
      .def_property_readonly("num_pages", &PagePool::num_pages)
      .def_property_readonly("page_size", &PagePool::page_size)
      .def("num_available", &PagePool::available)
      .def("num_cached_pages", &PagePool::num_indexed)
      .def("hit_rate", &PagePool::hit_rate)
      .def_property_readonly("holders", [](const PagePool& p) {
        py::list out;
        for (int i = 0; i < p.num_pages(); ++i) out.append(p.holders(i));
        return out;
      })
      .def("hash_of", [](const PagePool& p, int page) -> py::object {
        if (page < 0 || page >= p.num_pages()) throw py::index_error("no such page");
        if (!p.hashed(page)) return py::none();
        return hash_to_py(p.hash_of(page));
      })
      .def("page_for", [](const PagePool& p, py::handle h) -> py::object {
        const int page = p.page_for(hash_from_py(h));
        if (page < 0) return py::none();
        return py::int_(page);
      })
      .def_property_readonly("free", &PagePool::free_order)
      .def_property_readonly("idle", &PagePool::idle_order)
      .def_property_readonly("stats", &pool_stats)
      .def("reset_stats", &PagePool::reset_stats)
      .def("match", [](const PagePool& p, py::handle chain) { return p.match(chain_from_py(chain)); })
      .def("reusable", [](const PagePool& p, py::handle chain, int num_tokens, int cap) {
        return p.reusable(chain_from_py(chain), num_tokens, cap);
      }, py::arg("hashes"), py::arg("num_tokens"), py::arg("cap") = -1)
      .def("reserve", [](PagePool& p, py::handle chain, int num_tokens, int cap) -> py::object {
        std::vector<int> pages;
        int reused = 0;
        if (!p.reserve(chain_from_py(chain), num_tokens, cap, pages, reused)) return py::none();
        return py::make_tuple(pages, reused);
      }, py::arg("hashes"), py::arg("num_tokens"), py::arg("cap") = -1)
      .def("take", [](PagePool& p) -> py::object {
        const int page = p.take();
        if (page < 0) return py::none();
        return py::int_(page);
      })
      .def("publish", [](PagePool& p, int page, py::handle h) { p.publish(page, hash_from_py(h)); })
      .def("give_back", [](PagePool& p, const std::vector<int>& pages) {
        p.give_back(pages.data(), (int)pages.size());
      })
      .def("snapshot", &pool_snapshot)
      .def("check_invariants", &PagePool::audit);

  py::class_<StateSlots>(m, "StateSlotPool")
      .def(py::init<int>())
      .def_property_readonly("num_slots", &StateSlots::count)
      .def("num_available", &StateSlots::available)
      .def("take", [](StateSlots& s, py::handle key) -> py::object {
        const int slot = s.take(key_of(key));
        if (slot < 0) return py::none();
        return py::int_(slot);
      })
      .def("give", [](StateSlots& s, py::handle key) { s.give(key_of(key)); })
      .def("slot_of", [](const StateSlots& s, py::handle key) { return s.slot_of(key_of(key)); })
      .def("check_invariants", &StateSlots::audit);

  py::class_<Sequence>(m, "SequencePages")
      .def_readonly("tables", &Sequence::tables)
      .def_readonly("first_live", &Sequence::first_live)
      .def_readonly("state_slot", &Sequence::state_slot)
      .def_readonly("cached_tokens", &Sequence::cached_tokens)
      .def_readonly("committed", &Sequence::committed);

  py::class_<CacheManager::Group>(m, "CacheGroup")
      .def_property_readonly("spec", [](const CacheManager::Group& g) { return spec_to_py(g.spec); })
      .def_property_readonly("window", [](const CacheManager::Group& g) -> py::object {
        if (g.spec.window == 0) return py::none();
        return py::int_(g.spec.window);
      })
      .def_readonly("slots", &CacheManager::Group::slots)
      .def_property_readonly("pool", [](CacheManager::Group& g) { return g.pool.get(); },
                             py::return_value_policy::reference_internal);

  py::class_<CacheManager, std::shared_ptr<CacheManager>>(m, "CacheManager")
      .def(py::init([](py::dict cache_slots, int num_pages, int page_size, int max_requests,
                       bool has_state) {
        std::vector<std::pair<int, GroupSpec>> slots;
        for (auto item : cache_slots) {
          slots.emplace_back(py::cast<int>(item.first), spec_from_py(item.second));
        }
        return std::make_shared<CacheManager>(slots, num_pages, page_size, max_requests, has_state);
      }), py::arg("cache_slots"), py::arg("num_pages"), py::arg("page_size"),
           py::arg("max_requests"), py::arg("has_state") = false)
      .def_property_readonly("page_size", &CacheManager::page_size)
      .def_property_readonly("prefix_sharing", &CacheManager::prefix_sharing)
      .def_property_readonly("has_state", &CacheManager::has_state)
      .def_property_readonly("groups", [](py::object self) {
        CacheManager& m = py::cast<CacheManager&>(self);
        py::list out;
        for (int g = 0; g < m.num_groups(); ++g) {
          out.append(py::cast(&m.group(g), py::return_value_policy::reference_internal, self));
        }
        return out;
      })
      .def_property_readonly("num_groups", &CacheManager::num_groups)
      .def("group_of", &CacheManager::group_of_slot, "The group a cache slot belongs to.")
      .def_property_readonly("state_slots", [](CacheManager& m) { return &m.state_slots(); },
                             py::return_value_policy::reference_internal)
      .def_property_readonly("main_pool", [](CacheManager& m) { return m.main_pool(); },
                             py::return_value_policy::reference_internal)
      .def("num_available", &CacheManager::available)
      .def("capacity_tokens", &CacheManager::capacity_tokens)
      .def("cached_prefix_tokens", [](const CacheManager& m, py::handle chain) {
        return m.cached_prefix_tokens(chain_from_py(chain));
      })
      .def("leaked_pages", &CacheManager::leaked_pages)
      .def("holds", [](const CacheManager& m, py::handle key) { return m.holds(key_of(key)); })
      .def("keys", &CacheManager::keys)
      .def("sequence", [](const CacheManager& m, py::handle key) { return m.sequence(key_of(key)); })
      .def("table", [](const CacheManager& m, py::handle key, int group) {
        return m.sequence(key_of(key)).tables.at((size_t)group);
      })
      .def("admit", [](CacheManager& m, py::handle key, py::handle chain, int num_tokens) -> py::object {
        const int cached = m.admit(key_of(key), chain_from_py(chain), num_tokens);
        if (cached < 0) return py::none();
        return py::int_(cached);
      })
      .def("grow", [](CacheManager& m, py::handle key, int start, int new_len) {
        return m.grow(key_of(key), start, new_len);
      })
      .def("trim", [](CacheManager& m, py::handle key, int n) { return m.trim(key_of(key), n); })
      .def("commit", [](CacheManager& m, py::handle key, py::handle chain, int full_pages) {
        m.commit(key_of(key), chain_from_py(chain), full_pages);
      })
      .def("free", [](CacheManager& m, py::handle key) { m.release(key_of(key)); })
      .def("check_invariants", &CacheManager::audit)
      .def("snapshot", [](CacheManager& m) {
        PagePool* pool = m.main_pool();
        py::dict out = pool ? pool_snapshot(*pool) : py::dict();
        py::list groups;
        for (int g = 0; g < m.num_groups(); ++g) {
          const CacheManager::Group& group = m.group(g);
          py::dict d;
          d["slots"] = group.slots.size();
          d["kv_heads"] = group.spec.kv_heads;
          d["head_dim"] = group.spec.k_dim;
          d["value_dim"] = group.spec.v_dim;
          d["window"] = group.spec.window ? py::object(py::int_(group.spec.window)) : py::object(py::none());
          d["available_blocks"] = group.pool->available();
          groups.append(d);
        }
        out["groups"] = groups;
        out["state_slots_free"] = m.state_slots().available();
        return out;
      });

  py::enum_<RequestState>(m, "RequestState")
      .value("WAITING", RequestState::WAITING)
      .value("RUNNING", RequestState::RUNNING)
      .value("FINISHED", RequestState::FINISHED)
      .value("ABORTED", RequestState::ABORTED);

  py::class_<SamplingParams>(m, "SamplingParams")
      .def(py::init([](double temperature, double top_p, bool ignore_eos, py::object seed) {
        SamplingParams p;
        p.temperature = temperature;
        p.top_p = top_p;
        p.ignore_eos = ignore_eos;
        if (!seed.is_none()) {
          p.has_seed = true;
          p.seed = py::cast<int64_t>(seed);
        }
        return p;
      }), py::arg("temperature") = 0.0, py::arg("top_p") = 1.0, py::arg("ignore_eos") = false,
           py::arg("seed") = py::none())
      .def_readwrite("temperature", &SamplingParams::temperature)
      .def_readwrite("top_p", &SamplingParams::top_p)
      .def_readwrite("ignore_eos", &SamplingParams::ignore_eos)
      .def_property("seed", [](const SamplingParams& p) -> py::object {
        if (!p.has_seed) return py::none();
        return py::int_(p.seed);
      }, [](SamplingParams& p, py::object seed) {
        p.has_seed = !seed.is_none();
        p.seed = p.has_seed ? py::cast<int64_t>(seed) : 0;
      })
      .def_property_readonly("greedy", &SamplingParams::greedy)
      .def("__repr__", [](const SamplingParams& p) {
        return "SamplingParams(temperature=" + std::to_string(p.temperature) + ", top_p=" +
               std::to_string(p.top_p) + ", ignore_eos=" + (p.ignore_eos ? "True" : "False") + ")";
      });

  py::class_<Request, RequestPtr>(m, "Request")
      .def(py::init([](const std::string& rid, py::handle prompt, int max_tokens, double arrival,
                       py::handle hashes, py::object params, py::object session_id) {
        auto r = std::make_shared<Request>();
        r->rid = rid;
        r->tokens = tokens_from_py(prompt);
        r->prompt_len = (int)r->tokens.size();
        r->max_tokens = max_tokens;
        r->arrival = arrival;
        r->chain = chain_from_py(hashes);
        if (!params.is_none()) r->params = py::cast<SamplingParams>(params);
        if (!session_id.is_none()) {
          r->has_session = true;
          r->session_id = py::cast<std::string>(session_id);
        }
        return r;
      }), py::arg("rid"), py::arg("prompt"), py::arg("max_tokens"), py::arg("arrival"),
           py::arg("hashes"), py::arg("params") = py::none(), py::arg("session_id") = py::none())
      .def_readonly("rid", &Request::rid)
      .def_readonly("max_tokens", &Request::max_tokens)
      .def_readonly("arrival", &Request::arrival)
      .def_readonly("params", &Request::params)
      .def_readonly("prompt_len", &Request::prompt_len)
      .def_property_readonly("tokens", [](const Request& r) { return r.tokens; })
      .def_property_readonly("prompt", [](const Request& r) {
        return std::vector<int32_t>(r.tokens.begin(), r.tokens.begin() + r.prompt_len);
      })
      .def_property_readonly("out", [](const Request& r) {
        return std::vector<int32_t>(r.tokens.begin() + r.prompt_len, r.tokens.end());
      })
      .def_property_readonly("num_out", &Request::num_out)
      .def("token_at", [](const Request& r, int index) { return r.tokens.at((size_t)index); })
      .def_property_readonly("hashes", [](const Request& r) { return chain_to_py(r.chain); })
      .def_property_readonly("session_id", [](const Request& r) -> py::object {
        if (!r.has_session) return py::none();
        return py::str(r.session_id);
      })
      .def_readwrite("num_computed", &Request::num_computed)
      .def_readwrite("num_cached", &Request::num_cached)
      .def_readwrite("state", &Request::state)
      .def_readwrite("preemptions", &Request::preemptions)
      .def_readwrite("recomputed_tokens", &Request::recomputed_tokens)
      .def_property_readonly("admitted_at", [](const Request& r) { return time_or_none(r.admitted_at); })
      .def_property_readonly("last_admitted_at", [](const Request& r) { return time_or_none(r.last_admitted_at); })
      .def_property_readonly("first_token_at", [](const Request& r) { return time_or_none(r.first_token_at); })
      .def_property_readonly("finished_at", [](const Request& r) { return time_or_none(r.finished_at); })
      .def_property_readonly("finish_reason", [](const Request& r) -> py::object {
        if (r.finish_reason.empty()) return py::none();
        return py::str(r.finish_reason);
      })
      .def_property_readonly("seq_len", &Request::seq_len)
      .def_property_readonly("remaining", &Request::remaining)
      .def_property_readonly("running", &Request::running)
      .def_property_readonly("done", &Request::done)
      .def("append", &Request::append, "Take a generated token.")
      .def("queue_delay", [](const Request& r) -> py::object {
        if (std::isnan(r.admitted_at)) return py::none();
        return py::float_(r.admitted_at - r.arrival);
      })
      .def("record", [](const Request& r) { return request_record(record_of(r)); });

  py::class_<Work>(m, "Work")
      .def_readonly("request", &Work::request)
      .def_readonly("start", &Work::start)
      .def_readonly("count", &Work::count)
      .def_readonly("emits", &Work::emits);

  py::class_<Plan>(m, "Plan")
      .def(py::init<>())
      .def_readonly("work", &Plan::work)
      .def_readonly("preempted", &Plan::preempted)
      .def_readonly("admitted", &Plan::admitted)
      .def_readonly("sched_seconds", &Plan::sched_seconds)
      .def_readonly("steady", &Plan::steady)
      .def("__bool__", [](const Plan& p) { return !p.work.empty(); })
      .def("__len__", [](const Plan& p) { return p.work.size(); })
      .def_property_readonly("prefill", [](const Plan& p) {
        std::vector<RequestPtr> out;
        for (const Work& w : p.work) {
          if (!w.decode()) out.push_back(w.request);
        }
        return out;
      })
      .def_property_readonly("decode", [](const Plan& p) {
        std::vector<RequestPtr> out;
        for (const Work& w : p.work) {
          if (w.decode()) out.push_back(w.request);
        }
        return out;
      })
      .def_property_readonly("num_decode", &Plan::num_decode)
      .def_property_readonly("num_prefill", &Plan::num_prefill)
      .def_property_readonly("num_prefill_tokens", &Plan::num_prefill_tokens)
      .def_property_readonly("emitting", [](const Plan& p) {
        std::vector<RequestPtr> out;
        for (const Work& w : p.work) {
          if (w.emits) out.push_back(w.request);
        }
        return out;
      });

  py::class_<Scheduler>(m, "Scheduler")
      .def(py::init([](std::shared_ptr<CacheManager> manager, std::shared_ptr<PageHasher> hasher,
                       const std::string& policy, int max_running, int prefill_budget,
                       double aging, double max_wait, int scan_limit) {
        return new Scheduler(manager, hasher, scheduler_options(policy, max_running, prefill_budget,
                                                                aging, max_wait, scan_limit));
      }), py::arg("manager"), py::arg("hasher"), py::arg("policy") = "fcfs",
           py::arg("max_running") = 64, py::arg("prefill_budget") = 8192,
           py::arg("aging_tokens_per_s") = 2000.0, py::arg("max_wait_s") = 5.0,
           py::arg("scan_limit") = 128)
      .def_property_readonly("waiting", &Scheduler::waiting)
      .def_property_readonly("running", &Scheduler::running)
      .def_property_readonly("policy", [](const Scheduler& s) { return policy_name(s.options().policy); })
      .def_property("max_running", [](const Scheduler& s) { return s.options().max_running; },
                    [](Scheduler& s, int n) { s.mutable_options().max_running = n; })
      .def_property("max_wait_s", [](const Scheduler& s) { return s.options().max_wait_s; },
                    [](Scheduler& s, double v) { s.mutable_options().max_wait_s = v; })
      .def_property("prefill_budget", [](const Scheduler& s) { return s.options().prefill_budget; },
                    [](Scheduler& s, int n) { s.mutable_options().prefill_budget = n; })
      .def_property_readonly("stats", &scheduler_stats)
      .def("has_work", &Scheduler::has_work)
      .def("add", &Scheduler::add)
      .def("abort", &Scheduler::abort)
      .def("drop", &Scheduler::drop)
      .def("schedule", &Scheduler::schedule)
      .def("score", [](const Scheduler& s, const RequestPtr& r, double now) { return s.score(*r, now); })
      .def("snapshot", [](const Scheduler& s) {
        py::dict d = scheduler_stats(s);
        const double steps = (double)std::max<int64_t>(1, s.stats().steps);
        d["policy"] = policy_name(s.options().policy);
        d["waiting"] = s.waiting().size();
        d["running"] = s.running().size();
        d["mean_sched_seconds"] = s.stats().sched_seconds / steps;
        return d;
      });

  py::class_<Event>(m, "StreamEvent")
      .def(py::init([](const std::string& rid, const std::string& kind, py::object token, int index,
                       py::object finish_reason, py::object message, double t) {
        Event e;
        e.rid = rid;
        e.kind = kind;
        e.token = token.is_none() ? -1 : py::cast<int>(token);
        e.index = index;
        if (!finish_reason.is_none()) e.finish_reason = py::cast<std::string>(finish_reason);
        if (!message.is_none()) e.message = py::cast<std::string>(message);
        e.t = t;
        return e;
      }), py::arg("rid"), py::arg("kind"), py::arg("token") = py::none(), py::arg("index") = 0,
           py::arg("finish_reason") = py::none(), py::arg("message") = py::none(), py::arg("t") = 0.0)
      .def_readonly("rid", &Event::rid)
      .def_readonly("kind", &Event::kind)
      .def_property_readonly("token", [](const Event& e) -> py::object {
        if (e.token < 0) return py::none();
        return py::int_(e.token);
      })
      .def_readonly("index", &Event::index)
      .def_property_readonly("finish_reason", [](const Event& e) -> py::object {
        if (e.finish_reason.empty()) return py::none();
        return py::str(e.finish_reason);
      })
      .def_property_readonly("message", [](const Event& e) -> py::object {
        if (e.message.empty()) return py::none();
        return py::str(e.message);
      })
      .def_readonly("t", &Event::t)
      .def("__repr__", [](const Event& e) {
        return "StreamEvent(rid='" + e.rid + "', kind='" + e.kind + "', token=" +
               std::to_string(e.token) + ", index=" + std::to_string(e.index) + ")";
      });

  py::class_<StepRecord>(m, "StepRecord")
      .def_readonly("t", &StepRecord::t)
      .def_readonly("num_prefill", &StepRecord::num_prefill)
      .def_readonly("num_decode", &StepRecord::num_decode)
      .def_readonly("prefill_tokens", &StepRecord::prefill_tokens)
      .def_readonly("sched_s", &StepRecord::sched_s)
      .def_readonly("prepare_s", &StepRecord::prepare_s)
      .def_readonly("forward_s", &StepRecord::forward_s)
      .def_readonly("device_s", &StepRecord::device_s)
      .def_readonly("step_s", &StepRecord::step_s)
      .def_readonly("waiting", &StepRecord::waiting)
      .def_readonly("running", &StepRecord::running)
      .def_readonly("free_blocks", &StepRecord::free_blocks)
      .def_readonly("preempted", &StepRecord::preempted);

  py::class_<EngineCore>(m, "EngineCore")
      .def(py::init([](std::shared_ptr<CacheManager> manager, std::shared_ptr<PageHasher> hasher,
                       const std::string& policy, int max_running, int prefill_budget, double aging,
                       double max_wait, int scan_limit, int max_model_len, std::vector<int> eos_ids,
                       size_t max_step_records, size_t max_request_records) {
        return new EngineCore(manager, hasher,
                              scheduler_options(policy, max_running, prefill_budget, aging, max_wait,
                                                scan_limit),
                              max_model_len, eos_ids, max_step_records, max_request_records);
      }), py::arg("manager"), py::arg("hasher"), py::arg("policy"), py::arg("max_running"),
           py::arg("prefill_budget"), py::arg("aging_tokens_per_s"), py::arg("max_wait_s"),
           py::arg("scan_limit"), py::arg("max_model_len"), py::arg("eos_ids"),
           py::arg("max_step_records") = 500000, py::arg("max_request_records") = 200000)
      .def_property_readonly("scheduler", [](EngineCore& c) { return &c.scheduler(); },
                             py::return_value_policy::reference_internal)
      .def_property("eos_ids", [](const EngineCore& c) { return c.eos_ids(); },
                    [](EngineCore& c, const std::vector<int>& ids) { c.set_eos_ids(ids); })
      .def("refusal", [](const EngineCore& c, size_t prompt_len, int max_tokens) -> py::object {
        std::string why = c.refusal(prompt_len, max_tokens);
        if (why.empty()) return py::none();
        return py::str(why);
      })
      .def("make_request", [](EngineCore& c, const std::string& rid, py::handle prompt, int max_tokens,
                              double arrival, py::object params, py::object session) {
        SamplingParams p;
        if (!params.is_none()) p = py::cast<SamplingParams>(params);
        std::string s;
        const bool has = !session.is_none();
        if (has) s = py::cast<std::string>(session);
        return c.make_request(rid, tokens_from_py(prompt), max_tokens, arrival, p, has ? &s : nullptr);
      })
      .def("count_rejected", &EngineCore::count_rejected)
      .def("count_idle", &EngineCore::count_idle)
      .def("add", &EngineCore::add)
      .def("abort", &EngineCore::abort)
      .def("schedule", [](EngineCore& c, double now) {
        std::vector<Event> events;
        Plan plan = c.schedule(now, events);
        return py::make_tuple(plan, events);
      })
      .def("advance", [](EngineCore& c, const Plan& plan, py::handle tokens, double now) {
        std::vector<int> t;
        for (const py::handle& item : tokens) t.push_back(item.is_none() ? -1 : py::cast<int>(item));
        return c.advance(plan, t, now);
      })
      .def("log_step", [](EngineCore& c, const Plan& plan, double now, double prepare_s,
                          double forward_s, double device_s, double step_s) {
        c.log_step(plan, now, prepare_s, forward_s, device_s, step_s);
        return c.steps().back();
      })
      .def_property_readonly("num_step_records", [](const EngineCore& c) { return c.steps().size(); })
      .def("step_records", [](const EngineCore& c) {
        return std::vector<StepRecord>(c.steps().begin(), c.steps().end());
      })
      .def_property_readonly("counters", [](const EngineCore& c) { return c.counters(); })
      .def("summary", [](const EngineCore& c) {
        py::dict d;
        for (const auto& kv : c.summary()) d[py::str(kv.first)] = kv.second;
        for (const auto& kv : c.counters()) d[py::str(kv.first)] = kv.second;
        return d;
      })
      .def("drain_finished", [](EngineCore& c) {
        py::list out;
        for (const RequestRecord& r : c.drain_finished()) out.append(request_record(r));
        return out;
      });

  bind_program(m);
  bind_ops(m);
}
