// Python module `fluidml`: the reference's surface (src/python/pybind.cpp:23-109;
// checklist test/python/import_test.py:10-61) over the MI355X backend, plus
// read-only inspection helpers (names starting with a lower-case verb on
// Executor, and module functions starting with "_") that the tests and the
// benchmark use to look at plans, layouts and per-kernel times.
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <optional>
#include <string_view>

#include "evaluation/dp.h"
#include "evaluation/eval.h"
#include "structure/context/context.h"
#include "structure/flow/flow.h"
#include "structure/graph/graph.h"
#include "structure/memory/memory.h"
#include "structure/tensor/meta.h"
#include "utils/utils.h"
#include "worker/builder.h"
#include "worker/converter.h"
#include "optimization/graph_passes.h"
#include "worker/executor.h"
#include "worker/launcher.h"
#include "worker/lower.h"
#include "worker/parser.h"
#include "worker/planner.h"
#include "worker/runner.h"

namespace py = pybind11;
using namespace fluidml;

namespace {

py::dict OperandOf(const worker::Operand &op) {
  static const char *kSpaces[] = {"arena", "interface", "constant", "private"};
  py::dict d;
  d["name"] = op.name;
  d["space"] = kSpaces[static_cast<int>(op.space)];
  d["offset"] = op.offset;
  d["pool"] = op.pool;
  d["bytes"] = op.meta.GetSize();
  d["shape"] = op.meta.GetShape();
  d["layout"] = op.layout;
  return d;
}

py::dict StepsOf(worker::LaunchPlan &plan) {
  py::list steps;
  for (const worker::Step &s : plan.GetSteps()) {
    py::dict d;
    py::list inputs;
    inputs.append(OperandOf(s.in0));
    if (s.node->IsDoubleInputs()) inputs.append(OperandOf(s.in1));
    d["inputs"] = inputs;
    d["out"] = OperandOf(s.out);
    d["node"] = s.node->GetName();
    d["kernel"] = s.kernel->GetKernelName();
    d["bytes"] = s.bytes;
    d["flops"] = s.flops;
    d["output"] = s.out.name;
    d["output_layout"] = s.out.layout;
    steps.append(d);
  }
  py::dict out;
  out["name"] = plan.GetName();
  out["arena_bytes"] = plan.GetArenaBytes();
  out["constant_bytes"] = plan.GetConstantBytes();
  out["interface_bytes"] = plan.GetInterfaceBytes();
  out["private_bytes"] = plan.GetPrivateBytes();
  out["peak_device_bytes"] = plan.GetPeakDeviceBytes();
  out["steps"] = steps;
  py::list launches;
  for (const worker::Launch &l : plan.GetSchedule()) {
    py::dict d;
    d["kind"] = worker::LaunchKindName(l.kind);
    d["members"] = l.members;
    // members whose output tensor the launch writes (the rest are elided intermediates)
    std::vector<size_t> written;
    if (l.kind == worker::Launch::Kind::View) {
      // nothing runs and nothing is written: the readers address `source` (bytes of another tensor) instead
      py::dict src = OperandOf(l.out);
      src["bytes"] = l.out.Extent();
      src["view_offset"] = l.out.view_offset;
      src["view_strides"] = l.out.view_strides;
      d["source"] = src;
    } else if (l.kind == worker::Launch::Kind::Placed) {
      // a Concat2 whose inputs were written in place, or a Reshape behind a Concat2 that wrote into its buffer: nothing runs
    } else if (l.group.empty()) {
      // (a launch with a second output writes the tensor its last member reads as well: the member before it)
      if (l.has_out2 && l.members.size() >= 2) written.push_back(l.members[l.members.size() - 2]);
      written.push_back(l.members.back());
    }
    // a launch that writes into a part of another tensor (an input of a Concat2 placed in its output)
    // (a launch that writes its own result through other strides -- a Transpose it absorbed -- is not meant)
    auto padded = [&](const std::string &name) {  // the output of a Pad step (written in place by its input's producer)?
      for (const worker::Step &st : plan.GetSteps()) {
        if (st.out.name == name && !st.out.viewed) return st.node->GetKind() == flow::OpKind::Pad;
      }
      return false;
    };
    if (l.kind != worker::Launch::Kind::View && l.kind != worker::Launch::Kind::Placed && l.out.viewed && l.group.empty() &&
        !padded(l.out.name) &&
        (l.members.empty() || l.kind == worker::Launch::Kind::CopyInto ||
         l.out.name != plan.GetSteps()[l.members.back()].out.name)) {
      py::dict into = OperandOf(l.out);
      into["bytes"] = l.out.Extent();
      d["writes_into"] = into;
    }
    // results written into the interior of another tensor's buffer (a zero Pad that does not run: the padded tensor
    // lives outside the arena, its border is never written), per member of a group as well
    {
      py::list inside;
      auto note = [&](const worker::Operand &out, size_t step) {
        const worker::Step &producer = plan.GetSteps()[step];
        if (!out.viewed || !padded(out.name) || l.kind == worker::Launch::Kind::CopyInto) return;
        (void)producer;
        py::dict w;
        w["step"] = step;
        py::dict into = OperandOf(out);
        into["bytes"] = out.Extent();
        into["view_offset"] = out.view_offset;
        into["view_strides"] = out.view_strides;
        w["into"] = into;
        inside.append(w);
      };
      if (l.kind != worker::Launch::Kind::View && l.kind != worker::Launch::Kind::Placed) {
        if (l.group.empty() && !l.members.empty()) note(l.out, l.members.back());
        for (const worker::Launch &m : l.group) note(m.out, m.members.back());
      }
      d["writes_inside"] = inside;
    }
    for (const worker::Launch &m : l.group) written.push_back(m.members.back());
    d["written"] = written;
    // what the launch reads and writes as it is issued (operands of a side branch point at buffers of their own)
    py::list reads, writes;
    if (l.kind != worker::Launch::Kind::View && l.kind != worker::Launch::Kind::Placed) {
      auto add_reads = [&](const worker::Launch &x) {
        for (const worker::Operand *op : {&x.a, &x.b, &x.c, &x.d, &x.e}) {
          if (!op->name.empty() && (x.kind != worker::Launch::Kind::Step || x.rewired)) {
            py::dict o = OperandOf(*op);
            o["bytes"] = op->Extent();
            reads.append(o);
          }
        }
      };
      auto add_write = [&](const worker::Operand &op) {
        py::dict o = OperandOf(op);
        o["bytes"] = op.Extent();
        writes.append(o);
      };
      add_reads(l);
      for (const worker::Launch &m : l.group) add_reads(m);
      if (l.kind != worker::Launch::Kind::Step || l.rewired) {
        if (l.group.empty()) add_write(l.out);
        for (const worker::Launch &m : l.group) add_write(m.out);
        if (l.has_out2) add_write(l.out2);
      }
    }
    d["reads"] = reads;
    d["writes"] = writes;
    // a LayerNormalization kept out of memory: 1 = the launch normalises its left operand on the fly, 2 = its addend;
    // "norm_emits": the launch absorbed a LayerNormalization step and leaves row statistics for its readers
    d["norm_mode"] = l.norm_mode;
    d["norm_emits"] = !l.norm_stats_out.empty();
    // tensors this launch writes into buffers of their own although the memory plan holds bytes for them (the
    // planned bytes are in use when the fused launch writes or reads them)
    {
      py::list moved;
      auto note = [&](const worker::Operand &out, size_t step) {
        if (out.space == worker::Operand::Space::Private && out.pool.empty() &&
            plan.GetSteps()[step].out.space != worker::Operand::Space::Private) {
          py::dict o = OperandOf(out);
          o["bytes"] = out.Extent();
          moved.append(o);
        }
      };
      if (l.kind != worker::Launch::Kind::View && l.kind != worker::Launch::Kind::Placed &&
          (l.kind != worker::Launch::Kind::Step || l.rewired)) {
        if (l.group.empty() && !l.members.empty()) note(l.out, l.members.back());
        if (l.has_out2 && l.members.size() >= 2) note(l.out2, l.members[l.members.size() - 2]);
        for (const worker::Launch &m : l.group) note(m.out, m.members.back());
      }
      d["moved_out"] = moved;
    }
    d["position"] = l.group.empty() ? l.members.back() : l.position;
    d["bytes"] = l.bytes;
    d["flops"] = l.flops;
    launches.append(d);
  }
  out["launches"] = launches;
  // runs of launches issued side by side: launches [a_begin, b_begin) on the plan's stream, [b_begin, end) beside them
  py::list regions;
  for (const worker::LaunchPlan::Region &r : plan.GetRegions()) regions.append(py::make_tuple(r.a_begin, r.b_begin, r.end));
  out["regions"] = regions;
  py::list arguments;
  for (const worker::Argument &arg : plan.GetArguments()) {
    py::dict d;
    d["name"] = arg.name;
    d["kind"] = arg.type == worker::Argument::Type::Input ? "input" : "output";
    d["dtype"] = static_cast<int>(arg.meta.GetType());
    d["shape"] = arg.meta.GetShape();
    d["bytes"] = arg.meta.GetSize();
    arguments.append(d);
  }
  out["arguments"] = arguments;
  return out;
}

std::optional<Meta> MetaOf(const std::vector<int64_t> &shape) { return Meta(Type::kFloat32, shape); }

}  // namespace

PYBIND11_MODULE(fluidml, m) {
  m.doc() = "FluidML on MI355X: compile an ONNX graph into a HIP launch plan over one HBM arena and run it";

  py::class_<context::Context>(m, "Context")
      .def(py::init<>())
      .def("make_plain_general_builder", &context::Context::MakePlainGeneralBuilder, py::arg("function_name"))
      .def("make_dp_general_builder", &context::Context::MakeDPGeneralBuilder, py::arg("function_name"))
      .def("make_kernel_builder", &context::Context::MakeKernelBuilder, py::arg("function_name"))
      .def("make_plain_linear_planner", &context::Context::MakePlainLinearPlanner)
      .def("make_plain_greedy_planner", &context::Context::MakePlainGreedyPlanner)
      .def("make_dp_greedy_planner", &context::Context::MakeDPGreedyPlanner)
      .def("make_lower", &context::Context::MakeLower)
      .def("make_runner", &context::Context::MakeRunner)
      .def("set_cost_mode",
           [](context::Context &c, const std::string &mode) {
             c->cost_model.reset();
             if (mode == "constant") {
               c->cost_mode = context::CostMode::Constant;
             } else if (mode == "measure") {
               c->cost_mode = context::CostMode::Measure;
             } else {
               c->cost_mode = context::CostMode::Table;
               c->cost_table_path = mode;
             }
           },
           py::arg("mode"), "\"measure\", \"constant\" or the path of a saved cost table")
      .def("set_ref_flags", [](context::Context &c, uint32_t flags) { c->ref_flags = flags; }, py::arg("flags"))
      .def("set_use_graph", [](context::Context &c, bool use) { c->use_graph = use; }, py::arg("use"))
      .def("set_fuse", [](context::Context &c, bool fuse) { c->fuse = fuse; }, py::arg("fuse"))
      .def("set_graph_passes", [](context::Context &c, bool on) { c->graph_passes = on; }, py::arg("on"))
      .def("set_bf16", [](context::Context &c, bool on) { c->bf16 = on; }, py::arg("on"))
      .def("set_branch_min_us", [](context::Context &c, double us) { c->branch_min_us = us; }, py::arg("us"))
      .def("set_branch_check", [](context::Context &c, bool on) { c->branch_check = on; }, py::arg("on"))
      .def("set_branch_decision", [](context::Context &c, int keep) { c->branch_decision = keep; }, py::arg("keep"),
           "1 / 0: keep / drop the side branches without timing them; negative: decide by timing")
      .def("set_tune",
           [](context::Context &c, const std::string &mode) {
             using Mode = kernel::ContractionTable::Mode;
             if (mode == "off") {
               c->contraction_table->SetMode(Mode::Off);
             } else if (mode == "measure") {
               c->contraction_table->SetMode(Mode::Measure);
             } else if (mode == "replay") {
               c->contraction_table->SetMode(Mode::Replay);
             } else {
               c->LoadSavedDecisions(mode);
               c->contraction_table->SetMode(Mode::Replay);
             }
           },
           py::arg("mode"),
           "tile configuration of the contractions: \"measure\" (time unknown problems at compile), \"off\" (the "
           "library's rule), \"replay\" (only what the table holds), or the path of a JSON file an earlier compile wrote")
      .def("load_contraction_table",
           [](context::Context &c, const std::string &json_text) { c->contraction_table->LoadJsonText(json_text); },
           py::arg("json_text"))
      .def("contraction_table_json", [](context::Context &c) { return c->contraction_table->ToJson(); })
      .def("plan_text", [](context::Context &c) { return c->GetModule().ToText(); });

  py::class_<flow::Flow, std::unique_ptr<flow::Flow>>(m, "Flow")
      .def("node_names", [](const flow::Flow &f) {
        std::vector<std::string> names;
        for (const auto &n : f.GetNodes()) names.push_back(n->GetName());
        return names;
      });

  py::class_<flow::Sequence, std::unique_ptr<flow::Sequence>>(m, "Sequence")
      .def("node_names",
           [](const flow::Sequence &s) {
             std::vector<std::string> names;
             for (const auto &n : s.GetNodes()) names.push_back(n->GetName());
             return names;
           })
      .def("kernel_names",
           [](const flow::Sequence &s) {
             std::vector<std::string> names;
             for (const auto &n : s.GetNodes()) names.push_back(std::string(n->GetKindName()) + "Kernel");
             return names;
           })
      .def("region_names",
           [](const flow::Sequence &s) {
             std::vector<std::string> names;
             for (const auto &r : s.GetRegions()) names.push_back(r->GetName());
             return names;
           })
      .def("buffer_sizes",
           [](const flow::Sequence &s) {
             std::vector<size_t> sizes;
             for (const auto &n : s.GetNodes()) sizes.push_back(n->GetBufferSize());
             return sizes;
           })
      .def("layouts", [](const flow::Sequence &s) {
        std::map<std::string, std::vector<size_t>> out;
        for (const auto &r : s.GetRegions()) out[r->GetName()] = r->GetLayout();
        return out;
      });

  py::class_<graph::Graph, std::unique_ptr<graph::Graph>>(m, "Graph")
      .def("nodes",
           [](const graph::Graph &g) {
             py::list out;
             for (const std::shared_ptr<graph::Node> &n : g.GetAllNodes()) {
               py::dict d;
               d["name"] = n->GetName();
               d["op"] = graph::OpToString(n->GetOp());
               std::vector<std::string> ins, outs;
               for (const auto &e : g.GetNodeFrom(n->GetName())) ins.push_back(e->GetName());
               for (const auto &e : g.GetNodeTo(n->GetName())) outs.push_back(e->GetName());
               d["inputs"] = ins;
               d["outputs"] = outs;
               out.append(d);
             }
             return out;
           },
           "nodes in container order: name, op, input and output value names");

  py::class_<optimization::GraphPassesManager>(m, "GraphPassesManager")
      .def(py::init<>())
      .def("register_all_passes", &optimization::GraphPassesManager::RegisterAllPasses)
      .def("run", &optimization::GraphPassesManager::Run, py::arg("graph"));

  py::class_<memory::Index, std::unique_ptr<memory::Index>>(m, "Index")
      .def("get", &memory::Index::Get, py::arg("name"))
      .def("get_maximum", &memory::Index::GetMaximum)
      .def("items", [](const memory::Index &index) {
        std::map<std::string, std::pair<size_t, size_t>> out;
        for (const auto &kv : index.GetAll()) out[kv.first] = {std::get<0>(kv.second), std::get<1>(kv.second)};
        return out;
      });

  py::class_<worker::Builder, std::unique_ptr<worker::Builder>>(m, "Builder");

  py::class_<worker::GeneralBuilder, worker::Builder, std::unique_ptr<worker::GeneralBuilder>>(m, "GeneralBuilder")
      .def("run", &worker::GeneralBuilder::Run, py::arg("sequence"), py::arg("index"));

  py::class_<worker::KernelBuilder, worker::Builder, std::unique_ptr<worker::KernelBuilder>>(m, "KernelBuilder");

  py::class_<worker::Converter, std::unique_ptr<worker::Converter>>(m, "Converter")
      .def("run", &worker::Converter::Run, py::arg("graph"))
      .def_static("make", &worker::Converter::Make);

  py::class_<worker::Executor, std::unique_ptr<worker::Executor>>(m, "Executor")
      .def("compile",
           py::overload_cast<std::string_view, std::optional<std::string_view>, std::optional<std::string_view>,
                             std::optional<std::string_view>>(&worker::Executor::Compile),
           py::arg("input"), py::arg("mlir") = std::nullopt, py::arg("llvm") = std::nullopt,
           py::arg("json") = std::nullopt)
      .def("invoke",
           py::overload_cast<const std::unordered_map<std::string, py::array> &>(&worker::Executor::Invoke),
           py::arg("args"))
      .def_static("make_plain_linear", &worker::Executor::MakePlainLinear, py::arg("name"), py::arg("epoch") = 1)
      .def_static("make_plain_greedy", &worker::Executor::MakePlainGreedy, py::arg("name"), py::arg("epoch") = 1)
      .def_static("make_dp_greedy", &worker::Executor::MakeDPGreedy, py::arg("name"), py::arg("epoch") = 1)
      // ---- inspection (not in the reference) ----
      .def("context", [](worker::Executor &e) { return e.GetContext(); })
      .def("plan", [](worker::Executor &e) { return StepsOf(e.GetContext()->GetModule()); },
           "launch plan summary: arena/constant/interface bytes and one dict per step")
      .def("plan_text", [](worker::Executor &e) { return e.GetContext()->GetModule().ToText(); })
      .def("profile",
           [](worker::Executor &e, size_t warmup, size_t iters) {
             py::list out;
             for (const worker::StepTime &t : e.GetContext()->GetModule().Profile(warmup, iters)) {
               py::dict d;
               d["node"] = t.node;
               d["kernel"] = t.kernel;
               d["ns"] = t.ns;
               d["bytes"] = t.bytes;
               d["flops"] = t.flops;
               out.append(d);
             }
             return out;
           },
           py::arg("warmup") = 3, py::arg("iters") = 20, "median hipEvent nanoseconds of every step")
      .def("time_replay_ns",
           [](worker::Executor &e, size_t warmup, size_t iters) {
             return e.GetContext()->GetModule().TimeReplayNs(warmup, iters);
           },
           py::arg("warmup") = 3, py::arg("iters") = 20,
           "mean device nanoseconds of one replay of the whole plan (inputs resident in HBM)")
      .def("replay_times_ns",
           [](worker::Executor &e, size_t warmup, size_t iters) {
             return e.GetContext()->GetModule().ReplayTimesNs(warmup, iters);
           },
           py::arg("warmup") = 3, py::arg("iters") = 100,
           "device nanoseconds of each of `iters` consecutive replays (events on the plan's stream)")
      .def("replay", [](worker::Executor &e, size_t n) { e.GetContext()->GetModule().ReplayResident(n); }, py::arg("n") = 1,
           "n replays of the plan on the tensors already in HBM, then a stream wait (no host copies)")
      .def("materialize", [](worker::Executor &e) { e.GetContext()->GetModule().Materialize(); })
      .def("contraction_choices",
           [](worker::Executor &e) {
             py::list out;
             for (const auto &c : e.GetContext()->GetModule().GetContractionChoices()) {
               const uint32_t tile = (c.second >> FL_CONTRACT_TILE_SHIFT) & 0xfu, splits = (c.second >> FL_CONTRACT_SPLIT_SHIFT) & 0x3fu;
               out.append(py::make_tuple(c.first, tile, splits));
             }
             return out;
           },
           "(signature, tile, splits) of every MatMul / Gemm launch of the schedule; 0 = the library's rule")
      .def("branch_decision", [](worker::Executor &e) { return e.GetContext()->GetModule().GetBranchDecision(); });

  py::class_<worker::Lower, std::unique_ptr<worker::Lower>>(m, "Lower").def("run", &worker::Lower::Run);

  py::class_<worker::Parser, std::unique_ptr<worker::Parser>>(m, "Parser")
      .def("run", py::overload_cast<std::string_view>(&worker::Parser::Run), py::arg("input"))
      .def_static("make", &worker::Parser::Make);

  py::class_<worker::Planner, std::unique_ptr<worker::Planner>>(m, "Planner")
      .def("run", &worker::Planner::Run, py::arg("flow"));

  py::class_<worker::Runner, std::unique_ptr<worker::Runner>>(m, "Runner")
      .def("run",
           py::overload_cast<const std::unordered_map<std::string, py::array> &, size_t>(&worker::Runner::Run),
           py::arg("args"), py::arg("epoch") = 1);

  // ---- module-level helpers for tests of the planning core ----
  m.def(
      "_plan_memory",
      [](int kind, const std::vector<size_t> &starts, const std::vector<size_t> &ends, const std::vector<size_t> &sizes) {
        std::unique_ptr<memory::Infos> infos;
        std::unique_ptr<memory::Plan> plan;
        if (kind == 0) {
          infos = std::make_unique<memory::PlainInfos>();
          plan = std::make_unique<memory::LinearPlan>();
        } else {
          infos = std::make_unique<memory::GreedyInfos>();
          plan = std::make_unique<memory::GreedyPlan>();
        }
        for (size_t i = 0; i < sizes.size(); ++i) infos->Push(memory::Info("t" + std::to_string(i), starts[i], ends[i], sizes[i]));
        memory::Index index = plan->Run(*infos);
        std::vector<size_t> offsets;
        for (size_t i = 0; i < sizes.size(); ++i) offsets.push_back(index.Get("t" + std::to_string(i)));
        return std::make_pair(offsets, index.GetMaximum());
      },
      py::arg("kind"), py::arg("starts"), py::arg("ends"), py::arg("sizes"),
      "kind 0 = PlainInfos+LinearPlan, 1 = GreedyInfos+GreedyPlan; tensors are named t0, t1, ... in push order");
  m.def("_kernel_names", [] {
    // GetKernelName() of every kernel class, in the order of flow::OpKind
    std::vector<std::string> names;
    for (int k = 0; k <= static_cast<int>(flow::OpKind::WhereConstantCondConstantTensorY); ++k) {
      names.push_back(kernel::KernelNameOf(static_cast<flow::OpKind>(k)));
    }
    return names;
  });
  m.def("_contraction_candidates", &kernel::ContractionTable::Candidates, py::arg("full"));
  m.def(
      "_contraction_measure",
      [](const std::vector<std::pair<int, int>> &candidates, const py::function &launch, const py::function &elapsed,
         int rounds, double margin) {
        const kernel::ContractPick p = kernel::ContractionTable::Measure(
            candidates, [&](uint32_t bits) { return launch(bits).cast<int>(); }, [&]() { return elapsed().cast<double>(); },
            rounds, margin);
        return py::make_tuple(p.tile, p.splits, p.ns, p.rule_ns);
      },
      py::arg("candidates"), py::arg("launch"), py::arg("elapsed_ns"), py::arg("rounds") = 3, py::arg("margin") = 0.015,
      "the tuner's selection rule on caller-supplied launch and timing functions");
  m.def(
      "_contraction_signature",
      [](const std::string &path, const std::string &node_name, const std::vector<size_t> &lhs_layout,
         const std::vector<size_t> &rhs_layout, const std::vector<size_t> &out_layout) {
        std::unique_ptr<worker::Parser> parser = worker::Parser::Make();
        std::unique_ptr<worker::Converter> converter = worker::Converter::Make();
        graph::Graph graph = parser->Run(std::string_view(path));
        flow::Flow flow = converter->Run(graph);
        for (const std::shared_ptr<flow::Node> &node : flow.GetNodes()) {
          if (node->GetName() == node_name) {
            kernel::KernelGenerator g(*node);
            return g.GetContractionSignature(lhs_layout, rhs_layout, out_layout);
          }
        }
        throw std::out_of_range("no node named " + node_name);
      },
      py::arg("onnx_path"), py::arg("node"), py::arg("lhs_layout"), py::arg("rhs_layout"), py::arg("out_layout"),
      "ContractionTable key of a MatMul / Gemm node's standalone kernel under the given layouts");
  m.def(
      "_pack_constant_f32",
      [](std::vector<float64_t> values, std::vector<int64_t> shape, const std::vector<size_t> &layout, bool gathered) {
        const Tensor t(Type::kFloat32, std::move(shape), std::move(values));
        const std::vector<uint8_t> bytes = t.Pack(layout, gathered);
        return py::bytes(reinterpret_cast<const char *>(bytes.data()), bytes.size());
      },
      py::arg("values"), py::arg("shape"), py::arg("layout"), py::arg("gathered") = false,
      "the bytes uploaded for a float32 constant stored with `layout` (gathered: FL_REF_CONSTANT_GATHERED)");
  m.def("_gen_all_orders", &utils::GenAllOrders);
  m.def("_gen_all_indices_in_order", &utils::GenAllIndicesInOrder);
  m.def("_gen_physical_shape", &utils::GenPhysicalShape);
  m.def("_gen_strides", py::overload_cast<const std::vector<int64_t> &>(&utils::GenStrides));
  m.def("_gen_strides_layout",
        py::overload_cast<const std::vector<int64_t> &, const std::vector<size_t> &>(&utils::GenStrides));
  m.def("_broadcast_shape", [](const std::vector<int64_t> &a, const std::vector<int64_t> &b) {
    std::optional<Meta> r = BroadcastShape(*MetaOf(a), *MetaOf(b), Type::kFloat32);
    return r ? std::optional<std::vector<int64_t>>(r->GetShape()) : std::nullopt;
  });
  m.def("_broadcast_matmul_shape", [](const std::vector<int64_t> &a, const std::vector<int64_t> &b) {
    std::optional<Meta> r = BroadcastMatMulShape(*MetaOf(a), *MetaOf(b), Type::kFloat32);
    return r ? std::optional<std::vector<int64_t>>(r->GetShape()) : std::nullopt;
  });
  m.def(
      "_dp_layouts",
      [](const flow::Flow &flow, const std::string &cost) {
        std::shared_ptr<evaluation::CostModel> model = cost == "constant" ? evaluation::CostModel::MakeConstant()
                                                                          : evaluation::CostModel::MakeFromTable(cost);
        auto table = evaluation::DynamicProgrammingTable::Make(model);
        evaluation::DynamicProgrammingPlan plan = table->Run(flow);
        return std::map<std::string, std::vector<size_t>>(plan.GetAll().begin(), plan.GetAll().end());
      },
      py::arg("flow"), py::arg("cost") = "constant",
      "layout DP on a flow with constant costs or with the JSON text of a cost table");
}
