// Bindings of the step side of the host core: the registry of operation kinds, programs, and
// the step packer.
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <cstddef>

#include "program.h"
#include "step_batch.h"

namespace py = pybind11;
using namespace mercury;

namespace {

template <typename T>
T* as_ptr(uintptr_t p) {
  return reinterpret_cast<T*>(p);
}

// Chunks as Python gives them: (key, token ids, start, wanted indices).
struct Chunks {
  std::vector<std::vector<int32_t>> tokens;
  std::vector<SeqInput> seqs;
  explicit Chunks(const py::handle& list) {
    const size_t n = (size_t)py::len(list);
    tokens.resize(n);
    seqs.resize(n);
    size_t i = 0;
    for (const py::handle& item : list) {
      py::object key, toks, start, want;
      if (py::isinstance<py::tuple>(item)) {
        py::tuple t = py::reinterpret_borrow<py::tuple>(item);
        key = t[0]; toks = t[1]; start = t[2]; want = t[3];
      } else {
        key = item.attr("key"); toks = item.attr("tokens");
        start = item.attr("start"); want = item.attr("want");
      }
      for (const py::handle& tok : toks) tokens[i].push_back(py::cast<int32_t>(tok));
      SeqInput& s = seqs[i];
      s.key = py::cast<std::string>(py::str(key));
      s.tokens = tokens[i].data();
      s.count = (int)tokens[i].size();
      s.start = py::cast<int>(start);
      for (const py::handle& w : want) s.want.push_back(py::cast<int>(w));
      ++i;
    }
  }
};

}  // namespace

void bind_program(py::module_& m) {
  py::register_exception<KernelError>(m, "KernelError", PyExc_RuntimeError);
  py::register_exception<BatchError>(m, "BatchError", PyExc_ValueError);

  // ---- operation kinds
  m.def("register_op", [](const std::string& name, uintptr_t run, uintptr_t tiles, int flags) {
    OpKind kind;
    kind.name = name;
    kind.run = reinterpret_cast<mk_op_run_fn>(run);
    kind.tiles = reinterpret_cast<mk_op_tiles_fn>(tiles);
    kind.flags = flags;
    OpRegistry::instance().add(kind);
  }, py::arg("name"), py::arg("run"), py::arg("tiles") = 0, py::arg("flags") = 0,
        "Register an operation kind: `run` and `tiles` are addresses of C functions with the "
        "signatures of op_abi.h (mk_op_run_fn, mk_op_tiles_fn); whoever registers keeps them alive.");
  m.def("op_kinds", []() { return OpRegistry::instance().names(); });
  m.def("op_abi_layout", []() {
    py::dict d;
    d["context_size"] = sizeof(mk_op_context);
    d["step_size"] = sizeof(mk_step_view);
    d["tile_list_size"] = sizeof(mk_tile_list);
    d["context_error_offset"] = offsetof(mk_op_context, error);
    d["context_alloc_offset"] = offsetof(mk_op_context, alloc);
    d["context_out_x_offset"] = offsetof(mk_op_context, out_x);
    d["step_tables_offset"] = offsetof(mk_step_view, tables);
    return d;
  }, "Sizes and a few offsets of the structures of op_abi.h, for mirrors of them to check.");
  m.attr("OP_READS_X") = (int)MK_OP_READS_X;
  m.attr("OP_FOLDS_PENDING") = (int)MK_OP_FOLDS_PENDING;
  m.attr("OP_FIXED_STREAM") = (int)MK_OP_FIXED_STREAM;
  m.def("set_fixed_stream_limit", [](int limit) {
    OpRegistry& r = OpRegistry::instance();
    const int before = r.fixed_stream_limit;
    r.fixed_stream_limit = limit;
    return before;
  }, py::arg("limit"),
        "Steps of up to `limit` tokens keep their residual stream in fixed point where every "
        "operation of the program can (0: none do; negative: the kernels' own rule).  Returns "
        "the limit set before.");

  m.def("build_tiles", [](const std::vector<int>& counts, int group, int tile_rows) {
    std::vector<int> seq, row0;
    build_tiles(counts, group, tile_rows, seq, row0);
    return py::make_tuple(seq, row0);
  });
  m.def("count_tiles", &count_tiles);

  // ---- programs
  py::class_<Program, std::shared_ptr<Program>>(m, "Program")
      .def(py::init<int, int, int>(), py::arg("dtype"), py::arg("hidden"), py::arg("vocab"))
      .def_property_readonly("num_ops", [](const Program& p) { return p.size(); })
      .def_property_readonly("kinds", [](const Program& p) {
        std::vector<std::string> out;
        for (size_t i = 0; i < p.size(); ++i) out.push_back(p.kind_of(i));
        return out;
      })
      .def("append", [](Program& p, const std::string& kind, const py::bytes& params) {
        const std::string blob = params;
        p.append(kind, blob.data(), blob.size());
      }, py::arg("kind"), py::arg("params"),
           "Append an operation of a registered kind with its parameter block (copied).")
      .def("host", [](Program& p, int index, bool gives_x) { p.append_caller_step(index, gives_x); },
           py::arg("index"), py::arg("gives_x") = false,
           "Append a step the caller runs itself between two calls of run().")
      .def("host_index", [](const Program& p, int op) { return p.caller_index((size_t)op); })
      .def("tile_needs", [](const Program& p, const std::vector<int>& counts, int max_q_len,
                            int max_kv_len) {
        py::list out;
        for (const Program::TileNeed& t : p.tile_needs(counts, max_q_len, max_kv_len)) {
          out.append(py::make_tuple(t.group, t.tile_rows));
        }
        return out;
      })
      .def("fixed_stream", [](const Program& p, int num_tokens) { return p.fixed_stream(num_tokens); },
           py::arg("num_tokens"),
           "Whether a step of this many tokens keeps its residual stream in fixed point.")
      .def("workspace_bytes", [](const Program& p, const PackedStep& step) {
        return p.measure(step.view(nullptr)).total();
      })
      .def("workspace_bytes_for", [](const Program& p, const std::vector<int>& counts, int num_rows,
                                     int max_kv_len, int num_groups, int x_rows, bool own_stream) {
        return p.measure(StepView::shape_only(counts, num_rows, max_kv_len, num_groups), x_rows,
                         own_stream).total();
      }, py::arg("counts"), py::arg("num_rows"), py::arg("max_kv_len"), py::arg("num_groups") = 1,
           py::arg("x_rows") = 0, py::arg("own_stream") = false,
           "What a step of this shape (tokens per sequence, wanted rows, longest sequence) needs "
           "of its workspace; also the check that the operations fit together.")
      .def("run", [](const Program& p, const PackedStep& step, uintptr_t ints, uintptr_t workspace,
                     size_t workspace_bytes, uintptr_t stream, int begin, uintptr_t x, int x_rows,
                     uintptr_t pending, int pending_count) {
        RunState state;
        state.begin = begin;
        state.x = as_ptr<const void>(x);
        state.x_rows = x_rows;
        state.pending = as_ptr<const float>(pending);
        state.pending_count = pending_count;
        p.run(step.view(as_ptr<const int32_t>(ints)), as_ptr<char>(workspace), workspace_bytes,
              as_ptr<void>(stream), state);
        return py::make_tuple(state.stopped_at, (uintptr_t)state.h, (uintptr_t)state.logits,
                              (uintptr_t)state.x, state.x_rows, (uintptr_t)state.pending,
                              state.pending_count);
      }, py::arg("step"), py::arg("ints"), py::arg("workspace"), py::arg("workspace_bytes"),
           py::arg("stream"), py::arg("begin") = 0, py::arg("x") = 0, py::arg("x_rows") = 0,
           py::arg("pending") = 0, py::arg("pending_count") = 0,
           "Launch the operations from `begin` to the end or to the next caller-run step; "
           "returns (stopped_at, h, logits, x, x_rows, pending, pending_count), device addresses.")
      .def("run_on", [](const Program& p, const py::dict& v, uintptr_t workspace,
                        size_t workspace_bytes, uintptr_t stream, uintptr_t h, uintptr_t logits,
                        uintptr_t x, int x_rows, uintptr_t pending, int pending_count) {
        // A step described by device addresses (a step context of the caller's), and a
        // residual stream of the caller's own: how a single operation is run on tensors.
        auto at = [&](const char* key) {
          return v.contains(key) && !v[key].is_none() ? as_ptr<const int>(py::cast<uintptr_t>(v[key]))
                                                      : nullptr;
        };
        StepView step;
        step.counts = py::cast<std::vector<int>>(v["counts"]);
        step.num_seqs = (int)step.counts.size();
        for (int c : step.counts) step.num_tokens += c;
        step.num_rows = py::cast<int>(v["num_rows"]);
        step.max_q_len = py::cast<int>(v["max_q_len"]);
        step.max_kv_len = py::cast<int>(v["max_kv_len"]);
        step.token_ids = at("token_ids");
        step.positions = at("positions");
        step.token_seq = at("token_seq");
        step.cu_q = at("cu_q");
        step.kv_len = at("kv_len");
        step.state_slots = at("state_slots");
        step.logit_rows = at("logit_rows");
        for (const py::handle& item : v["tables"]) {
          const py::tuple t = py::reinterpret_borrow<py::tuple>(item);
          step.tables.push_back(as_ptr<const int>(py::cast<uintptr_t>(t[0])));
          step.widths.push_back(py::cast<int>(t[1]));
        }
        for (const py::handle& item : v["tiles"]) {
          const py::tuple t = py::reinterpret_borrow<py::tuple>(item);
          mk_tile_list list;
          list.group = py::cast<int>(t[0]);
          list.tile_rows = py::cast<int>(t[1]);
          list.seq = as_ptr<const int>(py::cast<uintptr_t>(t[2]));
          list.row0 = as_ptr<const int>(py::cast<uintptr_t>(t[3]));
          list.count = py::cast<int>(t[4]);
          step.tiles.push_back(list);
        }
        RunState state;
        state.own_h = as_ptr<float>(h);
        state.own_logits = as_ptr<float>(logits);
        state.x = as_ptr<const void>(x);
        state.x_rows = x_rows;
        state.pending = as_ptr<const float>(pending);
        state.pending_count = pending_count;
        if (!state.own_h) throw KernelError("run_on needs the caller's residual stream");
        p.run(step, as_ptr<char>(workspace), workspace_bytes, as_ptr<void>(stream), state);
        if (state.stopped_at != (int)p.size()) {
          throw KernelError("run_on runs programs without caller-run steps");
        }
        return py::make_tuple((uintptr_t)state.logits, (uintptr_t)state.x, state.x_rows,
                              (uintptr_t)state.pending, state.pending_count);
      }, py::arg("view"), py::arg("workspace"), py::arg("workspace_bytes"), py::arg("stream"),
           py::arg("h"), py::arg("logits") = 0, py::arg("x") = 0, py::arg("x_rows") = 0,
           py::arg("pending") = 0, py::arg("pending_count") = 0,
           "Run the whole program on a step given by device addresses and on a residual stream "
           "of the caller's; returns (logits, x, x_rows, pending, pending_count).");

  py::class_<PackedStep>(m, "PackedStep")
      .def_readonly("num_tokens", &PackedStep::num_tokens)
      .def_readonly("num_seqs", &PackedStep::num_seqs)
      .def_readonly("num_rows", &PackedStep::num_rows)
      .def_readonly("max_q_len", &PackedStep::max_q_len)
      .def_readonly("max_kv_len", &PackedStep::max_kv_len)
      .def_readonly("counts", &PackedStep::counts)
      .def_readonly("starts", &PackedStep::starts)
      .def_readonly("widths", &PackedStep::widths)
      .def_readonly("fresh_slots", &PackedStep::fresh_slots)
      .def_readonly("total", &PackedStep::total)
      .def_property_readonly("host_address", [](const PackedStep& p) { return (uintptr_t)p.host; })
      .def_property_readonly("spans", [](const PackedStep& p) {
        py::list out;
        for (size_t s = 0; s < p.counts.size(); ++s) {
          out.append(py::make_tuple(p.firsts[s], p.counts[s], p.starts[s]));
        }
        return out;
      })
      .def_property_readonly("offsets", [](const PackedStep& p) {
        py::dict d;
        d["token_ids"] = py::make_tuple(p.off_ids, p.num_tokens);
        d["positions"] = py::make_tuple(p.off_positions, p.num_tokens);
        d["token_seq"] = py::make_tuple(p.off_token_seq, p.num_tokens);
        d["cu_q"] = py::make_tuple(p.off_cu_q, p.num_seqs + 1);
        d["kv_len"] = py::make_tuple(p.off_kv_len, p.num_seqs);
        d["state_slots"] = py::make_tuple(p.off_slots, p.num_seqs);
        d["logit_rows"] = py::make_tuple(p.off_rows, p.num_rows);
        py::list tables;
        for (size_t g = 0; g < p.off_tables.size(); ++g) {
          tables.append(py::make_tuple(p.off_tables[g], p.num_seqs, p.widths[g]));
        }
        d["tables"] = tables;
        py::list tiles;
        for (const PackedStep::TileList& t : p.tiles) {
          tiles.append(py::make_tuple(t.group, t.tile_rows, t.count, t.off_seq, t.off_row0));
        }
        d["tiles"] = tiles;
        return d;
      })
      .def("layout", [](const PackedStep& p) { return py::tuple(py::cast(p.layout())); })
      .def("host_list", [](const PackedStep& p) {
        return std::vector<int32_t>(p.host, p.host + p.total);
      });

  py::class_<StepPacker>(m, "StepPacker")
      .def(py::init([](std::shared_ptr<CacheManager> manager, int vocab, int max_positions,
                       bool pinned) {
        auto* packer = new StepPacker(manager, vocab, max_positions);
        packer->set_pinned(pinned);
        return packer;
      }), py::arg("manager"), py::arg("vocab_size"), py::arg("max_positions"),
           py::arg("pinned") = true)
      .def("pack", [](StepPacker& packer, py::handle chunks, std::shared_ptr<Program> program,
                      int table_width, bool check_ids, int kv_bound) {
        Chunks c(chunks);
        return packer.pack(c.seqs, program.get(), table_width, check_ids, kv_bound);
      }, py::keep_alive<0, 1>(), py::arg("chunks"), py::arg("program") = nullptr,
           py::arg("table_width") = -1, py::arg("check_ids") = true, py::arg("kv_bound") = 0)
      .def("pack_plan", [](StepPacker& packer, const Plan& plan, std::shared_ptr<Program> program,
                           int table_width, int kv_bound) {
        return packer.pack_plan(plan, program.get(), table_width, kv_bound);
      }, py::keep_alive<0, 1>(), py::arg("plan"), py::arg("program") = nullptr,
           py::arg("table_width") = -1, py::arg("kv_bound") = 0)
      .def("upload", [](StepPacker& packer, const PackedStep& step, uintptr_t device,
                        uintptr_t stream) {
        packer.upload(step, as_ptr<void>(device), as_ptr<void>(stream));
      });
}
