// Bindings of what talks to the GPU: the kernel libraries, the decisions which kernel runs
// what, programs, and the step packer.
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include "dispatch.h"
#include "kernels.h"
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

py::dict plan_to_py(const AttentionPlan& p) {
  py::dict d;
  d["mfma"] = p.mfma;
  d["rows"] = p.rows;
  d["staged"] = p.staged;
  d["splits"] = p.splits;
  d["split_blocks"] = p.split_blocks;
  d["tile_rows"] = p.tile_rows;
  d["num_tiles"] = p.num_tiles;
  return d;
}

}  // namespace

void bind_device(py::module_& m) {
  py::register_exception<KernelError>(m, "KernelError", PyExc_RuntimeError);
  py::register_exception<BatchError>(m, "BatchError", PyExc_ValueError);

  m.def("load_kernels", &load_kernel_library, py::arg("name"), py::arg("path"));
  m.def("kernels_loaded", [](const std::string& name) {
    return name == "core" ? kernels().has_core() : kernels().has_mfma();
  });

  // ---- decisions (pure functions of sizes and element types)
  m.def("mfma_eligible", &mfma_eligible);
  m.def("wants_partials", &wants_partials);
  m.def("plan_partials", [](int rows, int n, int k) {
    const PartialsPlan p = plan_partials(rows, n, k);
    return py::make_tuple(p.skinny, p.slices);
  });
  m.def("choose_linear", [](int x_dtype, int rows, int n, int k, bool has_bias, bool accumulate,
                            int out_dtype, int force) {
    return (int)choose_linear(x_dtype, rows, n, k, has_bias, accumulate, out_dtype, force);
  }, "0 float32-arithmetic kernel, 1 skinny, 2 skinny accumulating, 3 tiled");
  m.def("fuses_gating", &fuses_gating);
  m.def("gated_is_skinny", &gated_is_skinny);
  m.def("qkv_fusable", &qkv_fusable);
  m.def("choose_qkv", [](int x_dtype, int w_dtype, int rows, int width, int k, int head_dim,
                         int rotary_dim, int page_size, bool half_layout) {
    return (int)choose_qkv(x_dtype, w_dtype, rows, width, k, head_dim, rotary_dim, page_size,
                           half_layout);
  }, "0 fused skinny, 1 fused tiled, 2 partial sums then the finishing kernel, 3 projection then rotation");
  m.def("plan_attention", [](int dtype, int head_dim, int page_size, int n_q, int n_kv, int window,
                             const std::vector<int>& counts, int max_q_len, int max_kv_len,
                             int force, int tile_rows, int staged, int splits, int split_blocks) {
    return plan_to_py(plan_attention(dtype, head_dim, page_size, n_q, n_kv, window, counts,
                                     max_q_len, max_kv_len, force, tile_rows, staged, splits,
                                     split_blocks));
  }, py::arg("dtype"), py::arg("head_dim"), py::arg("page_size"), py::arg("n_q"), py::arg("n_kv"),
        py::arg("window"), py::arg("counts"), py::arg("max_q_len"), py::arg("max_kv_len"),
        py::arg("force") = 0, py::arg("tile_rows") = -1, py::arg("staged") = -1,
        py::arg("splits") = 0, py::arg("split_blocks") = 0);
  m.def("build_tiles", [](const std::vector<int>& counts, int group, int tile_rows) {
    std::vector<int> seq, row0;
    build_tiles(counts, group, tile_rows, seq, row0);
    return py::make_tuple(seq, row0);
  });

  // ---- programs
  py::class_<Program, std::shared_ptr<Program>>(m, "Program")
      .def(py::init<int, int, int>(), py::arg("dtype"), py::arg("hidden"), py::arg("vocab"))
      .def_property_readonly("num_ops", [](const Program& p) { return p.ops().size(); })
      .def_property_readonly("kinds", [](const Program& p) {
        static const char* names[] = {"embed", "norm", "attention", "gated_mlp", "head", "host"};
        std::vector<std::string> out;
        for (const Op& op : p.ops()) out.push_back(names[(int)op.kind]);
        return out;
      })
      .def("embed", [](Program& p, uintptr_t table, int dtype, int vocab) {
        Op op;
        op.kind = OpKind::EMBED;
        op.table = as_ptr<void>(table);
        op.table_dtype = dtype;
        op.vocab = vocab;
        p.ops().push_back(op);
      })
      .def("norm", [](Program& p, uintptr_t weight, int dtype, float eps) {
        Op op;
        op.kind = OpKind::NORM;
        op.norm_w = as_ptr<void>(weight);
        op.norm_w_dtype = dtype;
        op.eps = eps;
        p.ops().push_back(op);
      })
      .def("attention", [](Program& p, uintptr_t w_qkv, uintptr_t b_qkv, int b_qkv_dtype,
                           uintptr_t w_o, uintptr_t b_o, int b_o_dtype, int n_q, int n_kv,
                           int head_dim, int rotary_dim, uintptr_t cos, uintptr_t sin,
                           int table_positions, bool interleaved, uintptr_t k_cache,
                           uintptr_t v_cache, int group, int page_size, float scale, int window,
                           bool writes) {
        Op op;
        op.kind = OpKind::ATTENTION;
        op.w_qkv = as_ptr<void>(w_qkv);
        op.b_qkv = as_ptr<void>(b_qkv);
        op.b_qkv_dtype = b_qkv_dtype;
        op.w_o = as_ptr<void>(w_o);
        op.b_o = as_ptr<void>(b_o);
        op.b_o_dtype = b_o_dtype;
        op.n_q = n_q;
        op.n_kv = n_kv;
        op.head_dim = head_dim;
        op.pos.rotary_dim = rotary_dim;
        op.pos.cos = as_ptr<float>(cos);
        op.pos.sin = as_ptr<float>(sin);
        op.pos.table_positions = table_positions;
        op.pos.interleaved = interleaved;
        op.k_cache = as_ptr<void>(k_cache);
        op.v_cache = as_ptr<void>(v_cache);
        op.group = group;
        op.page_size = page_size;
        op.scale = scale;
        op.window = window;
        op.writes = writes;
        p.ops().push_back(op);
      }, py::arg("w_qkv"), py::arg("b_qkv"), py::arg("b_qkv_dtype"), py::arg("w_o"), py::arg("b_o"),
           py::arg("b_o_dtype"), py::arg("n_q"), py::arg("n_kv"), py::arg("head_dim"),
           py::arg("rotary_dim"), py::arg("cos"), py::arg("sin"), py::arg("table_positions"),
           py::arg("interleaved"), py::arg("k_cache"), py::arg("v_cache"), py::arg("group"),
           py::arg("page_size"), py::arg("scale"), py::arg("window"), py::arg("writes"))
      .def("gated_mlp", [](Program& p, uintptr_t w_gate_up, uintptr_t w_down, int inter) {
        Op op;
        op.kind = OpKind::GATED_MLP;
        op.w_gate_up = as_ptr<void>(w_gate_up);
        op.w_down = as_ptr<void>(w_down);
        op.inter = inter;
        p.ops().push_back(op);
      })
      .def("head", [](Program& p, uintptr_t norm_w, int norm_dtype, float eps, uintptr_t head_w) {
        Op op;
        op.kind = OpKind::HEAD;
        op.norm_w = as_ptr<void>(norm_w);
        op.norm_w_dtype = norm_dtype;
        op.eps = eps;
        op.head_w = as_ptr<void>(head_w);
        p.ops().push_back(op);
      })
      .def("host", [](Program& p, int index) {
        Op op;
        op.kind = OpKind::HOST;
        op.host_index = index;
        p.ops().push_back(op);
      })
      .def("host_index", [](const Program& p, int op) { return p.ops().at((size_t)op).host_index; })
      .def("workspace_bytes", [](const Program& p, const PackedStep& step) {
        return p.measure(step.view(nullptr)).total();
      })
      .def("run", [](const Program& p, const PackedStep& step, uintptr_t ints, uintptr_t workspace,
                     size_t workspace_bytes, uintptr_t stream, int begin, uintptr_t pending,
                     int pending_count) {
        RunState state;
        state.begin = begin;
        state.pending = as_ptr<const float>(pending);
        state.pending_count = pending_count;
        p.run(step.view(as_ptr<const int32_t>(ints)), as_ptr<char>(workspace), workspace_bytes,
              as_ptr<void>(stream), state);
        return py::make_tuple(state.stopped_at, (uintptr_t)state.h, (uintptr_t)state.logits,
                              (uintptr_t)state.pending, state.pending_count);
      }, py::arg("step"), py::arg("ints"), py::arg("workspace"), py::arg("workspace_bytes"),
           py::arg("stream"), py::arg("begin") = 0, py::arg("pending") = 0,
           py::arg("pending_count") = 0,
           "Launch the operations from `begin` to the end or to the next caller-run layer; "
           "returns (stopped_at, h, logits, pending, pending_count) as device addresses.");

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
