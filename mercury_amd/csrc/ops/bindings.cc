// Bindings of the built-in operations: the kernel libraries, the decisions which kernel runs
// what, the parameter blocks of the built-in operation kinds, and the launch sequences as
// functions of device addresses (what the Python faces of the kernels call, so that a kernel
// test and a step's program go through the same code).
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <cstring>

#include "../host/program.h"
#include "builtin.h"
#include "dispatch.h"
#include "kernels.h"
#include "launch.h"

namespace py = pybind11;
using namespace mercury;

namespace {

template <typename T>
T* as_ptr(uintptr_t p) {
  return reinterpret_cast<T*>(p);
}

template <typename T>
T get(const py::dict& d, const char* key, T fallback) {
  return d.contains(key) && !d[key].is_none() ? py::cast<T>(d[key]) : fallback;
}

template <typename T>
T* ptr_of(const py::dict& d, const char* key) {
  return as_ptr<T>(get<uintptr_t>(d, key, 0));
}

template <typename P>
py::bytes blob(const P& params) {
  return py::bytes(reinterpret_cast<const char*>(&params), sizeof params);
}

py::dict plan_to_py(const AttentionPlan& p) {
  py::dict d;
  d["mfma"] = p.mfma;
  d["rows"] = p.rows;
  d["staged"] = p.staged;
  d["direct"] = p.direct;
  d["splits"] = p.splits;
  d["split_blocks"] = p.split_blocks;
  d["tile_rows"] = p.tile_rows;
  d["num_tiles"] = p.num_tiles;
  return d;
}

// The q/k/v side of an attention as Python describes it: addresses and sizes by name.
QkvArgs qkv_from(const py::dict& d) {
  QkvArgs a;
  a.w = ptr_of<const void>(d, "w_qkv");
  a.bias = ptr_of<const void>(d, "b_qkv");
  a.bias_dtype = get<int>(d, "b_qkv_dtype", kF32);
  a.n_q = get<int>(d, "n_q", 0);
  a.n_kv = get<int>(d, "n_kv", 0);
  a.head_dim = get<int>(d, "head_dim", 0);
  a.pos.rotary_dim = get<int>(d, "rotary_dim", 0);
  a.pos.cos = ptr_of<const float>(d, "cos");
  a.pos.sin = ptr_of<const float>(d, "sin");
  a.pos.table_positions = get<int>(d, "table_positions", 0);
  a.pos.interleaved = get<bool>(d, "interleaved", false) ? 1 : 0;
  a.k_cache = ptr_of<void>(d, "k_cache");
  a.v_cache = ptr_of<void>(d, "v_cache");
  a.page_size = get<int>(d, "page_size", 1);
  a.writes = get<bool>(d, "writes", true);
  if (a.n_q <= 0 || a.n_kv <= 0 || a.head_dim <= 0 || a.n_q % a.n_kv) {
    throw KernelError("attention: bad head counts or head size");
  }
  return a;
}

AttendArgs attend_from(const py::dict& d) {
  AttendArgs a;
  a.n_q = get<int>(d, "n_q", 0);
  a.n_kv = get<int>(d, "n_kv", 0);
  a.head_dim = get<int>(d, "head_dim", 0);
  a.page_size = get<int>(d, "page_size", 0);
  a.window = get<int>(d, "window", 0);
  a.scale = get<float>(d, "scale", 0.f);
  a.k_cache = ptr_of<const void>(d, "k_cache");
  a.v_cache = ptr_of<const void>(d, "v_cache");
  a.score_cap = get<float>(d, "score_cap", 0.f);
  a.distance_slopes = ptr_of<const float>(d, "distance_slopes");
  return a;
}

StepArrays arrays_from(const py::dict& d) {
  StepArrays s;
  s.positions = ptr_of<const int>(d, "positions");
  s.token_seq = ptr_of<const int>(d, "token_seq");
  s.cu_q = ptr_of<const int>(d, "cu_q");
  s.kv_len = ptr_of<const int>(d, "kv_len");
  s.table = ptr_of<const int>(d, "table");
  s.table_stride = get<int>(d, "table_stride", 0);
  return s;
}

void* scratch_alloc(void* arena, size_t bytes) { return static_cast<Arena*>(arena)->alloc(bytes); }

// An operation context over memory the Python caller provides.
struct Face {
  Arena arena;
  mk_op_context ctx;
  Face(int dtype, uintptr_t stream, char* base, size_t size, bool dry) {
    arena.reset(base, size, dry);
    std::memset(&ctx, 0, sizeof ctx);
    ctx.stream = as_ptr<void>(stream);
    ctx.dry = dry ? 1 : 0;
    ctx.dtype = dtype;
    ctx.arena = &arena;
    ctx.alloc = &scratch_alloc;
  }
};

// Run a launch sequence over scratch memory of the caller's: once dry, to learn how much it
// allocates; `alloc(bytes) -> address` is then asked for that much; then for real.
template <typename F>
auto with_scratch(int dtype, uintptr_t stream, const py::object& alloc, F body) {
  Face dry(dtype, stream, nullptr, 0, true);
  Launch measure(&dry.ctx);
  body(measure);
  const size_t need = dry.arena.peak();
  uintptr_t base = 0;
  if (need) {
    if (alloc.is_none()) throw KernelError("this launch needs scratch memory and was given none");
    base = py::cast<uintptr_t>(alloc(need));
  }
  Face wet(dtype, stream, as_ptr<char>(base), need, false);
  Launch launch(&wet.ctx);
  return body(launch);
}

}  // namespace

void bind_ops(py::module_& m) {
  register_builtin_ops();

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
  m.def("validate_attention_plan", [](const py::dict& plan, int head_dim, int page_size, int n_q,
                                      int n_kv) {
    AttentionPlan p;
    p.mfma = py::cast<bool>(plan["mfma"]);
    p.rows = py::cast<int>(plan["rows"]);
    p.staged = py::cast<int>(plan["staged"]);
    p.direct = plan.contains("direct") && py::cast<bool>(plan["direct"]);
    p.splits = py::cast<int>(plan["splits"]);
    p.split_blocks = py::cast<int>(plan["split_blocks"]);
    p.tile_rows = py::cast<int>(plan["tile_rows"]);
    p.num_tiles = py::cast<int>(plan["num_tiles"]);
    return plan_defect(p, head_dim, page_size, n_q, n_kv);
  }, "Why the matrix-core attention would refuse this plan, or an empty string.");

  // ---- parameter blocks of the built-in operation kinds
  m.def("embed_params", [](uintptr_t table, int table_dtype, int vocab, float scale) {
    EmbedParams p;
    p.table = as_ptr<const void>(table);
    p.table_dtype = table_dtype;
    p.vocab = vocab;
    p.scale = scale;
    return blob(p);
  }, py::arg("table"), py::arg("table_dtype"), py::arg("vocab"), py::arg("scale") = 1.f);
  m.def("norm_params", [](uintptr_t weight, int weight_dtype, float eps, bool select_rows) {
    NormParams p;
    p.weight = as_ptr<const void>(weight);
    p.weight_dtype = weight_dtype;
    p.eps = eps;
    p.select_rows = select_rows ? 1 : 0;
    return blob(p);
  }, py::arg("weight"), py::arg("weight_dtype"), py::arg("eps"), py::arg("select_rows") = false);
  m.def("attention_params", [](const py::kwargs& kw) {
    const py::dict d = kw;
    AttentionParams p;
    p.qkv = qkv_from(d);
    p.w_o = ptr_of<const void>(d, "w_o");
    p.b_o = ptr_of<const void>(d, "b_o");
    p.b_o_dtype = get<int>(d, "b_o_dtype", kF32);
    p.group = get<int>(d, "group", 0);
    p.window = get<int>(d, "window", 0);
    p.scale = get<float>(d, "scale", 0.f);
    p.score_cap = get<float>(d, "score_cap", 0.f);
    p.distance_slopes = ptr_of<const float>(d, "distance_slopes");
    return blob(p);
  });
  m.def("gated_mlp_params", [](uintptr_t w_gate_up, uintptr_t w_down, int inter) {
    GatedMlpParams p;
    p.w_gate_up = as_ptr<const void>(w_gate_up);
    p.w_down = as_ptr<const void>(w_down);
    p.inter = inter;
    return blob(p);
  });
  m.def("head_params", [](uintptr_t weight, uintptr_t bias, int bias_dtype, float cap) {
    HeadParams p;
    p.weight = as_ptr<const void>(weight);
    p.bias = as_ptr<const void>(bias);
    p.bias_dtype = bias_dtype;
    p.cap = cap;
    return blob(p);
  }, py::arg("weight"), py::arg("bias") = 0, py::arg("bias_dtype") = 0, py::arg("cap") = 0.f);

  // ---- the launch sequences, by device address
  m.def("launch_embed", [](uintptr_t ids, uintptr_t table, int table_dtype, uintptr_t out,
                           int tokens, int hidden, int vocab, float scale, uintptr_t stream) {
    Face f(kF32, stream, nullptr, 0, false);
    Launch l(&f.ctx);
    embed(l, as_ptr<const int>(ids), as_ptr<const void>(table), table_dtype, as_ptr<float>(out),
          tokens, hidden, vocab, scale);
  });
  m.def("launch_rmsnorm", [](uintptr_t h, int tokens, int hidden, uintptr_t pending,
                             int pending_count, uintptr_t weight, int weight_dtype, float eps,
                             uintptr_t rows, int out_rows, uintptr_t out, int out_dtype,
                             uintptr_t stream) {
    Face f(out_dtype, stream, nullptr, 0, false);
    Launch l(&f.ctx);
    rmsnorm(l, as_ptr<float>(h), tokens, hidden, as_ptr<const float>(pending), pending_count,
            as_ptr<const void>(weight), weight_dtype, eps, as_ptr<const int>(rows), out_rows,
            as_ptr<void>(out));
  });
  m.def("launch_silu_mul", [](uintptr_t gate_up, uintptr_t out, int dtype, int tokens, int inter,
                              uintptr_t stream) {
    Face f(dtype, stream, nullptr, 0, false);
    Launch l(&f.ctx);
    silu_mul(l, as_ptr<const void>(gate_up), tokens, inter, as_ptr<void>(out));
  });
  m.def("launch_logit_cap", [](uintptr_t logits, long long count, float cap, uintptr_t stream) {
    Face f(kF32, stream, nullptr, 0, false);
    Launch l(&f.ctx);
    logit_cap(l, as_ptr<float>(logits), count, cap);
  });
  m.def("launch_linear", [](uintptr_t x, int m_, uintptr_t w, int n, int k, int dtype,
                            uintptr_t bias, int bias_dtype, uintptr_t out, int out_dtype,
                            bool accumulate, int kernel, int tile_config, uintptr_t stream) {
    Face f(dtype, stream, nullptr, 0, false);
    Launch l(&f.ctx);
    LinearForce force;
    force.kernel = kernel;
    force.tile_config = tile_config;
    linear(l, as_ptr<const void>(x), m_, as_ptr<const void>(w), n, k, as_ptr<const void>(bias),
           bias_dtype, as_ptr<void>(out), out_dtype, accumulate, force);
  });
  m.def("launch_linear_partials", [](uintptr_t x, int m_, uintptr_t w, int n, int k, int dtype,
                                     const py::object& alloc, uintptr_t stream) {
    int slices = 0;
    float* out = with_scratch(dtype, stream, alloc, [&](Launch& l) {
      return linear_partials(l, as_ptr<const void>(x), m_, as_ptr<const void>(w), n, k, slices);
    });
    return py::make_tuple((uintptr_t)out, slices);
  });
  m.def("launch_project", [](uintptr_t x, int m_, uintptr_t w, int n, int k, int dtype,
                             uintptr_t bias, int bias_dtype, uintptr_t h, const py::object& alloc,
                             uintptr_t stream) {
    const float* pending = nullptr;
    int count = 0;
    with_scratch(dtype, stream, alloc, [&](Launch& l) {
      project_into_stream(l, as_ptr<const void>(x), m_, as_ptr<const void>(w), n, k,
                          as_ptr<const void>(bias), bias_dtype, as_ptr<float>(h), pending, count);
      return 0;
    });
    return py::make_tuple((uintptr_t)pending, count);
  }, "h += x W^T (+ bias), or partial sums left for the next norm: (address, how many).");
  m.def("launch_gated", [](uintptr_t x, int m_, int k, uintptr_t w, int inter, int dtype,
                           int tile_config, const py::object& alloc, uintptr_t stream) {
    void* act = with_scratch(dtype, stream, alloc, [&](Launch& l) {
      return gated(l, as_ptr<const void>(x), m_, k, as_ptr<const void>(w), inter, tile_config);
    });
    return (uintptr_t)act;
  });
  m.def("launch_qkv_project", [](uintptr_t x, int m_, int k, int dtype, const py::dict& args,
                                 const py::dict& arrays, int kind, int tile_config,
                                 const py::object& alloc, uintptr_t stream) {
    const QkvArgs a = qkv_from(args);
    const StepArrays s = arrays_from(arrays);
    QkvForce force;
    force.kind = kind;
    force.tile_config = tile_config;
    const Queries q = with_scratch(dtype, stream, alloc, [&](Launch& l) {
      return qkv_project(l, as_ptr<const void>(x), m_, k, a, s, force);
    });
    return py::make_tuple((uintptr_t)q.q, q.stride);
  }, "Returns (address of the rotated queries, their row stride in elements).");
  m.def("launch_rope_kv_write", [](uintptr_t qkv, int row_stride, int m_, int dtype,
                                   const py::dict& args, const py::dict& arrays, uintptr_t stream) {
    Face f(dtype, stream, nullptr, 0, false);
    Launch l(&f.ctx);
    rope_kv_write(l, as_ptr<void>(qkv), row_stride, m_, qkv_from(args), arrays_from(arrays));
  });
  m.def("launch_qkv_finish", [](uintptr_t parts, int slices, int m_, int out_dtype,
                                const py::dict& args, const py::dict& arrays,
                                const py::object& alloc, uintptr_t stream) {
    const QkvArgs a = qkv_from(args);
    const StepArrays s = arrays_from(arrays);
    void* q = with_scratch(out_dtype, stream, alloc, [&](Launch& l) {
      return qkv_finish(l, as_ptr<const float>(parts), slices, m_, a, s, out_dtype);
    });
    return (uintptr_t)q;
  });
  m.def("launch_attention_project", [](uintptr_t q, int q_stride, int dtype, const py::dict& args,
                                       const py::dict& arrays, const std::vector<int>& counts,
                                       int max_q_len, int max_kv_len, const py::object& tiles,
                                       uintptr_t w_o, uintptr_t b_o, int b_o_dtype, int hidden,
                                       uintptr_t h, int fold, const py::object& alloc,
                                       uintptr_t stream) {
    const AttendArgs a = attend_from(args);
    const StepArrays s = arrays_from(arrays);
    mk_step_view view;
    std::memset(&view, 0, sizeof view);
    view.num_seqs = (int)counts.size();
    view.counts = counts.data();
    for (int c : counts) view.num_tokens += c;
    view.max_q_len = max_q_len;
    view.max_kv_len = max_kv_len;
    const AttentionPlan plan = plan_for(dtype, a, view);
    mk_tile_list list;
    std::memset(&list, 0, sizeof list);
    if (plan.mfma) {
      const py::tuple t = tiles(a.n_q / a.n_kv, plan.tile_rows);
      list.group = a.n_q / a.n_kv;
      list.tile_rows = plan.tile_rows;
      list.seq = as_ptr<const int>(py::cast<uintptr_t>(t[0]));
      list.row0 = as_ptr<const int>(py::cast<uintptr_t>(t[1]));
      list.count = py::cast<int>(t[2]);
      view.num_tile_lists = 1;
      view.tile_lists = &list;
    }
    const float* pending = nullptr;
    int count = 0;
    with_scratch(dtype, stream, alloc, [&](Launch& l) {
      attend_and_project(l, Queries{as_ptr<const void>(q), q_stride}, a, s, view,
                         as_ptr<const void>(w_o), as_ptr<const void>(b_o), b_o_dtype, hidden,
                         as_ptr<float>(h), pending, count, AttendForce{}, fold);
      return 0;
    });
    return py::make_tuple((uintptr_t)pending, count);
  }, "The attention and its output projection into h; (address, count) of partial sums left.");
  m.def("launch_attention", [](uintptr_t q, int q_stride, int dtype, const py::dict& args,
                               const py::dict& arrays, const std::vector<int>& counts,
                               int max_q_len, int max_kv_len, const py::dict& force_in,
                               const py::object& tiles, uintptr_t out, const py::object& alloc,
                               uintptr_t stream) {
    const AttendArgs a = attend_from(args);
    const StepArrays s = arrays_from(arrays);
    AttendForce force;
    force.kernel = get<int>(force_in, "kernel", 0);
    force.tile_rows = get<int>(force_in, "tile_rows", -1);
    force.staged = get<int>(force_in, "staged", -1);
    force.splits = get<int>(force_in, "splits", 0);
    force.split_blocks = get<int>(force_in, "split_blocks", 0);
    mk_step_view view;
    std::memset(&view, 0, sizeof view);
    view.num_seqs = (int)counts.size();
    view.counts = counts.data();
    for (int c : counts) view.num_tokens += c;
    view.max_q_len = max_q_len;
    view.max_kv_len = max_kv_len;
    // the tile list the plan will walk, from the caller
    const AttentionPlan plan = plan_for(dtype, a, view, force);
    mk_tile_list list;
    std::memset(&list, 0, sizeof list);
    if (plan.mfma) {
      const py::tuple t = tiles(a.n_q / a.n_kv, plan.tile_rows);
      list.group = a.n_q / a.n_kv;
      list.tile_rows = plan.tile_rows;
      list.seq = as_ptr<const int>(py::cast<uintptr_t>(t[0]));
      list.row0 = as_ptr<const int>(py::cast<uintptr_t>(t[1]));
      list.count = py::cast<int>(t[2]);
      view.num_tile_lists = 1;
      view.tile_lists = &list;
    }
    void* result = with_scratch(dtype, stream, alloc, [&](Launch& l) {
      return attend(l, Queries{as_ptr<const void>(q), q_stride}, a, s, view, force,
                    as_ptr<void>(out));
    });
    return (uintptr_t)result;
  });
}
