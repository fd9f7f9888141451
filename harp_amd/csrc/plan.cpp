// plan_program: the passes in order, then a schedule for every kernel that is left.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <mutex>
#include <set>
#include <sstream>

#include "codegen_parts.hpp"

namespace eh {

ProgramPlan plan_program(const Node& program, const GenOptions& opt) {
  if (program.op != Op::Program) throw Error("expected a program node");
  g_guard_branches = opt.guard_branches;
  g_ranged_loads = opt.ranged_loads;
  validate_sizes(program);
  Planning st(opt);
  ProgramPlan& plan = st.plan;
  std::vector<const Node*>& kernels = st.kernels;
  std::vector<NodePtr>& rewritten = st.rewritten;
  std::map<std::string, size_t>& elems = st.elems;
  bool& have_table = st.have_table;
  auto& readers = st.readers;
  auto& nests = st.nests;
  auto& absorbed = st.absorbed;
  auto& absorbed_name = st.absorbed_name;
  auto& folded = st.folded;
  auto& folded_kernels = st.folded_kernels;
  auto& windows = st.windows;
  auto& scattered = st.scattered;
  auto& partly_written = st.partly_written;
  for (const auto& f : program.args) {
    if (f->op == Op::Kernel) kernels.push_back(f.get());
    else if (f->op == Op::Function) throw Error("helper functions in a program are not supported by this backend");
  }
  if (kernels.empty()) throw Error("program holds no kernel");
  // what the reference's AST optimiser did to the lowered loop nests is undone first
  if (opt.normalize)
    for (size_t q = 0; q < kernels.size(); ++q)
      for (const auto& f : program.args)
        if (f.get() == kernels[q]) {
          NodePtr nk = normalize_kernel(f);
          if (nk != f) {
            rewritten.push_back(nk);
            kernels[q] = nk.get();
          }
        }

  // buffer table: given, or synthesised from the kernels' pointer parameters
  plan.buffers = program.buffers;
  if (!plan.buffers.empty() && opt.fuse) {
    std::vector<const Node*> out;
    for (const Node* k : kernels) {
      auto nk = extract_nest(*k);
      auto rs = nk ? split_long_rows(*nk) : std::nullopt;
      if (!rs) { out.push_back(k); continue; }
      rewritten.push_back(rs->part);
      rewritten.push_back(rs->final_);
      out.push_back(rs->part.get());
      out.push_back(rs->final_.get());
      plan.buffers.push_back(rs->scratch);
    }
    kernels = out;
  }
  if (!plan.buffers.empty() && opt.fuse && opt.reindex) rewrite_for_readers(program, opt, &kernels, &rewritten, &plan);
  move_elementwise_behind_producers(st);
  have_table = !plan.buffers.empty();
  if (have_table) {
    for (const auto& b : plan.buffers) elems[b.name] = b.numel();
  } else {
    std::set<std::string> seen;
    for (const Node* k : kernels)
      for (const auto& p : k->params)
        if (p.dtype.is_ptr() && seen.insert(p.name).second) {
          BufferInfo bi;
          bi.name = p.name;
          bi.dtype = p.dtype.elem();
          bi.role = p.mut_ ? "output" : "input";
          bi.shape_known = false;
          plan.buffers.push_back(bi);
        } else if (p.dtype.is_ptr() && p.mut_) {
          for (auto& b : plan.buffers)
            if (b.name == p.name) b.role = "output";
        }
  }
  auto role_of = [&](const std::string& name) { return st.role_of(name); };
  for (const Node* k : kernels)
    for (const auto& p : k->params)
      if (p.dtype.is_ptr()) role_of(p.name);

  // consumers per buffer (kernel indices)
  for (size_t i = 0; i < kernels.size(); ++i)
    for (const auto& p : kernels[i]->params)
      if (p.dtype.is_ptr() && !p.mut_) readers[p.name].push_back(i);

  // inputs the executor itself fills with a constant (role ones / zeros): reads of them are
  // folded into literals wherever a kernel is recognised, so they cost no memory traffic
  std::map<std::string, double> consts;
  for (const auto& b : plan.buffers) {
    if (b.role == "ones") consts[b.name] = 1.0;
    if (b.role == "zeros") consts[b.name] = 0.0;
  }
  std::function<NodePtr(const NodePtr&)> fold = [&](const NodePtr& n) -> NodePtr {
    if (n->op == Op::Load && n->args[0]->op == Op::Var && consts.count(n->args[0]->name) && n->count == 1) {
      auto c = std::make_shared<Node>(Op::Const);
      c->dtype = n->dtype;
      c->fval = consts.at(n->args[0]->name);
      c->ival = static_cast<int64_t>(c->fval);
      return c;
    }
    bool changed = false;
    std::vector<NodePtr> args;
    for (const auto& a : n->args) {
      NodePtr r = fold(a);
      changed = changed || r != a;
      args.push_back(std::move(r));
    }
    if (!changed) return n;
    auto c = std::make_shared<Node>(*n);
    c->args = std::move(args);
    return c;
  };

  for (const Node* k : kernels) {
    nests.push_back(extract_nest(*k));
    if (nests.back() && nests.back()->rkind == ReduceKind::None) {
      // An elementwise nest has no loop-carried dependence, so its loops may run in any order:
      // walk the output in address order (largest stride outermost).  A kernel lowered through
      // a transposing view otherwise strides through memory with its innermost loop, and it
      // would not share an index space with the kernel that produced its operand.
      NestKernel& nk = *nests.back();
      const Affine& oa = *nk.out_aff;
      bool all_used = true;
      for (const auto& l : nk.loops) all_used = all_used && (l.extent == 1 || oa.of(l.var) != 0);
      if (all_used) {
        std::vector<Loop> wide;                       // loops of extent 1 keep their places
        for (const auto& l : nk.loops)
          if (l.extent > 1) wide.push_back(l);
        std::stable_sort(wide.begin(), wide.end(), [&](const Loop& a, const Loop& b) {
          return std::llabs(oa.of(a.var)) > std::llabs(oa.of(b.var));
        });
        size_t w = 0;
        for (auto& l : nk.loops)
          if (l.extent > 1) l = wide[w++];
      }
    }
    if (nests.back() && !consts.empty()) {
      NestKernel& nk = *nests.back();
      nk.value = fold(nk.value);
      std::vector<LoadRef> loads;
      collect_loads(*nk.value, loads);
      std::set<std::string> used;
      for (const auto& lr : loads) used.insert(lr.load->args[0]->name);
      std::vector<Param> kept;
      for (const auto& p : nk.params)
        if (p.mut_ || used.count(p.name) || !consts.count(p.name)) kept.push_back(p);
      nk.params = kept;
    }
  }

  merge_batch_sums_into_contractions(st);

  merge_sums_over_neighbouring_axes(st);

  fold_gathers_into_contractions(st);

  read_windows_through_their_gathers(st);

  join_shifted_sums_with_their_contraction(st);

  // Elementwise kernels that follow kernel i (a reduce with a dense output of `total` elements)
  // over the same dense index space and feed on its result: the function that applies them to
  // one element while it is still in a register.  `k0r`: k0 with its output laid out as a
  // consumer that reads it through a permutation wants it, when that applies and is allowed.
  auto build_epilogue = [&](size_t i, const NestKernel& k0, int64_t total, bool allow_relayout, NestKernel& k0r,
                            EpilogueSpec& epi, size_t& after) -> bool {
    bool have_epi = false;
    const bool small = total < (int64_t{1} << 30);
    std::map<std::string, DType> avail;          // values held in registers: C and stage outputs
    avail[k0.out_buf] = k0.out_dtype;
    bool c_relaid = false;
    size_t relaid_pos = 0;                       // position in `taken` of the stage that reads through a permutation
    Affine relaid_read;                          // ... and the index it reads at, over its own loops
    std::set<std::string> old_space;             // values produced before that stage
    std::set<size_t> independent;                // taken stages that read no value of the chain
    std::vector<size_t> taken;
    size_t j = i + 1;
    for (; j < kernels.size(); ++j) {
      if (absorbed.count(j)) continue;
      if (!nests[j] || folded_kernels.count(j) || nests[j]->rkind != ReduceKind::None) break;
      const NestKernel& sk = *nests[j];
      int64_t numel = 0;
      auto strides = dense_strides(sk, &numel);
      if (!strides || numel != total || avail.count(sk.out_buf)) break;
      std::vector<LoadRef> loads;
      collect_loads(*sk.value, loads);
      bool feeds = false, ok = true;
      std::optional<Affine> permuted;            // the one index all values of the chain are read at, if not the aligned one
      for (const auto& lr : loads) {
        if (lr.load->args[0]->op != Op::Var || lr.load->count != 1) { ok = false; break; }
        const std::string& b = lr.load->args[0]->name;
        if (!avail.count(b)) continue;
        auto a = affine_of(*lr.load->args[1]);
        if (!a) { ok = false; break; }
        const bool aligned = *a == *sk.out_aff;
        if (c_relaid && (old_space.count(b) || !aligned)) { ok = false; break; }
        if (!aligned) {
          if (feeds && !permuted) { ok = false; break; }          // the stage reads the chain both ways
          if (permuted && !(*permuted == *a)) { ok = false; break; }
          permuted = *a;
        } else if (permuted) {
          ok = false;
          break;
        }
        feeds = true;
      }
      if (!ok) break;
      // a stage over the same index space that reads nothing of the chain (the square of a
      // saved activation, say) rides along when a later stage combines it with the chain
      if (!feeds) independent.insert(j);
      if (permuted) {
        // A consumer may read the chain's values through a permutation (a transposed weight
        // gradient and its update, NHWC -> NCHW after a convolution).  If nothing computed so
        // far is needed outside the chain, the contraction can put each element where this
        // consumer wants it: C takes the consumer's index space, the stages before it are
        // evaluated at the element's original position, and the read becomes the aligned one.
        bool sole = true;
        for (const auto& kv : avail) {
          sole = sole && role_of(kv.first) == "temp";
          for (size_t r : readers[kv.first]) sole = sole && r > i && r <= j;
        }
        auto na = sole && allow_relayout ? relayout(k0, sk, *permuted) : std::nullopt;
        if (!na) break;
        k0r.out_aff = *na;
        if (!gemm_shaped(k0r, opt)) { k0r.out_aff = k0.out_aff; break; }
        c_relaid = true;
        relaid_pos = taken.size();
        relaid_read = *permuted;
        for (const auto& kv : avail) old_space.insert(kv.first);
      }
      avail[sk.out_buf] = sk.out_dtype;
      taken.push_back(j);
    }
    while (!taken.empty() && independent.count(taken.back())) {
      avail.erase(nests[taken.back()]->out_buf);      // nothing after it uses the chain: leave it out
      independent.erase(taken.back());
      taken.pop_back();
    }
    if (!taken.empty()) {
      after = taken.back() + 1;
      auto needed = [&](const std::string& buf) {
        if (role_of(buf) != "temp") return true;
        for (size_t r : readers[buf])
          if (r <= i || r >= after) return true;
        return false;
      };
      std::ostringstream fn, body;
      // the same function in two parts, for schedules that finish many elements per work-item in a
      // row: everything read from memory first (eh_epilogue_load), the arithmetic and the stores
      // after (eh_epilogue_apply); only when no read sits under a guard
      std::ostringstream load_body, apply_body;
      std::vector<std::string> slot_types;
      bool split_ok = true;
      // ... and for four elements in a row (eh_e a multiple of four): what does not move inside the
      // four is read once, what is read at the element itself as one vector, stores as vectors
      std::ostringstream quad_load, quad_apply;
      std::vector<std::string> quad_slots;         // declarations of EhEpiLoads4's members
      int quad_regs = 0;
      bool quad_ok = !(c_relaid && relaid_pos > 0);
      std::vector<std::string> ext_order;
      std::map<std::string, std::pair<std::string, size_t>> ext;   // name -> (declaration, min bytes)
      epi.store_c = needed(k0.out_buf);
      if (!epi.store_c) plan.elided.insert(k0.out_buf);
      const std::string IT = small ? "int" : "long long";
      const std::string UT = small ? "unsigned" : "unsigned long long";
      body << "  const " << IT << " eh_l = (" << IT << ")eh_e;\n";
      load_body << "  const " << IT << " eh_l = (" << IT << ")eh_e;\n  (void)eh_l;\n";
      body << "  const " << ctype(k0.out_dtype) << " eh_v_" << k0.out_buf << " = eh_acc;\n";
      if (epi.store_c) body << "  " << k0.out_buf << "[eh_e] = eh_acc;\n";
      apply_body << body.str();
      quad_load << "  const " << IT << " eh_l = (" << IT << ")eh_e;\n  (void)eh_l;\n";
      quad_apply << "  const " << IT << " eh_l = (" << IT << ")eh_e;\n  (void)eh_l;\n  " << ctype(k0.out_dtype) << " eh_v_" << k0.out_buf
                 << "[4] = {eh_acc[0], eh_acc[1], eh_acc[2], eh_acc[3]};\n";
      if (epi.store_c)
        quad_apply << "  *reinterpret_cast<EhQ<float>*>(" << k0.out_buf << " + eh_e) = EhQ<float>{eh_acc[0], eh_acc[1], eh_acc[2], eh_acc[3]};\n";
      auto decode_to = [&](std::ostringstream& to, const NestKernel& sk, const std::string& from) {
        int64_t numel = 0;
        auto strides = *dense_strides(sk, &numel);
        for (size_t li = 0; li < sk.loops.size(); ++li) {
          const Loop& l = sk.loops[li];
          if (l.extent == 1) to << "    const " << IT << " " << l.var << " = 0;\n";
          else to << "    const " << IT << " " << l.var << " = (" << IT << ")(((" << UT << ")" << from << " / " << strides[li] << "u) % "
                  << l.extent << "u);\n";    // (never negative: the unsigned division is the cheaper one)
        }
      };
      auto decode = [&](const NestKernel& sk, const std::string& from) { decode_to(body, sk, from); };
      if (c_relaid && relaid_pos > 0) {
        // where this element sat before C took the later consumer's layout: the stages
        // ahead of that consumer index their other operands with it
        if (epi.store_c) throw Error("internal: relaid contraction '" + k0.name + "' must not store C");
        split_ok = false;
        body << "  " << IT << " eh_lo;\n  {\n";
        decode(*nests[taken[relaid_pos]], "eh_l");
        body << "    eh_lo = ";
        bool first_term = true;
        for (const auto& kv : relaid_read.coef) {
          if (kv.second == 0) continue;
          body << (first_term ? "" : " + ") << kv.first << " * " << kv.second;
          first_term = false;
        }
        if (first_term) body << "0";
        body << ";\n  }\n";
      }
      for (size_t ti = 0; ti < taken.size(); ++ti) {
        const size_t j2 = taken[ti];
        const NestKernel& sk = *nests[j2];
        epi.kernels.push_back(sk.name);
        body << "  " << ctype(sk.out_dtype) << " eh_v_" << sk.out_buf << ";\n  {\n";
        decode(sk, (c_relaid && ti < relaid_pos) ? "eh_lo" : "eh_l");
        ExprRenderer er;
        er.load_hook = [&](const Node& ld, std::string* out) {
          const std::string& b = ld.args[0]->name;
          if (!avail.count(b)) return false;
          *out = "eh_v_" + b;
          return true;
        };
        std::vector<LoadRef> loads;
        collect_loads(*sk.value, loads);
        for (const auto& lr : loads) {
          const std::string& b = lr.load->args[0]->name;
          if (avail.count(b) || ext.count(b)) {
            if (ext.count(b) && !lr.guarded) {
              if (auto a = affine_of(*lr.load->args[1]))
                ext[b].second = std::max(ext[b].second, static_cast<size_t>(max_abs_index(*a, sk.loops, nullptr) + 1) *
                                                             lr.load->dtype.itemsize());
            }
            continue;
          }
          size_t mb = 0;
          if (!lr.guarded)
            if (auto a = affine_of(*lr.load->args[1]))
              mb = static_cast<size_t>(max_abs_index(*a, sk.loops, nullptr) + 1) * lr.load->dtype.itemsize();
          DType et = lr.load->dtype;
          for (const auto& pp : sk.params)
            if (pp.name == b) et = pp.dtype.elem();
          ext[b] = {"const " + ctype(et) + "* __restrict__ " + b, mb};
          ext_order.push_back(b);
          epi.bytes += static_cast<double>(elems.count(b) ? elems.at(b) : 0) * et.itemsize();
        }
        body << "    eh_v_" << sk.out_buf << " = (" << ctype(sk.out_dtype) << ")(" << er.expr(*sk.value) << ");\n";
        {
          // the two-part form of this stage
          std::set<const Node*> guarded;
          for (const auto& lr : loads)
            if (lr.guarded) guarded.insert(lr.load);
          apply_body << "  " << ctype(sk.out_dtype) << " eh_v_" << sk.out_buf << ";\n  {\n";
          decode_to(apply_body, sk, "eh_l");
          load_body << "  {\n";
          decode_to(load_body, sk, "eh_l");
          ExprRenderer er2;
          er2.load_hook = [&](const Node& ld, std::string* out) {
            const std::string& lb = ld.args[0]->name;
            if (avail.count(lb)) {
              *out = "eh_v_" + lb;
              return true;
            }
            if (guarded.count(&ld)) split_ok = false;
            ExprRenderer plain;
            const std::string slot = "eh_p.v" + std::to_string(slot_types.size());
            load_body << "    " << slot << " = " << plain.expr(ld) << ";\n";
            slot_types.push_back(ctype(ld.dtype));
            *out = slot;
            return true;
          };
          apply_body << "    eh_v_" << sk.out_buf << " = (" << ctype(sk.out_dtype) << ")(" << er2.expr(*sk.value) << ");\n";
          load_body << "  }\n";
          if (needed(sk.out_buf)) apply_body << "    " << sk.out_buf << "[eh_e] = eh_v_" << sk.out_buf << ";\n";
          apply_body << "  }\n";
        }
        if (quad_ok) {
          int64_t numel4 = 0;
          const auto strides4 = *dense_strides(sk, &numel4);
          std::set<std::string> still, vars;      // loops that keep their value over four aligned elements; all loops
          for (size_t li = 0; li < sk.loops.size(); ++li) {
            vars.insert(sk.loops[li].var);
            if (sk.loops[li].extent == 1 || strides4[li] % 4 == 0) still.insert(sk.loops[li].var);
          }
          std::function<bool(const Node&)> as_value = [&](const Node& n) {
            if (n.op == Op::Load) return false;
            if ((n.op == Op::Var || n.op == Op::Wildcard) && vars.count(n.name)) return true;
            for (const auto& a : n.args)
              if (a && as_value(*a)) return true;
            return false;
          };
          if (as_value(*sk.value) || (needed(sk.out_buf) && sk.out_dtype.itemsize() != 4)) quad_ok = false;
          quad_load << "  {\n";
          decode_to(quad_load, sk, "eh_l");
          quad_apply << "  " << ctype(sk.out_dtype) << " eh_v_" << sk.out_buf << "[4];\n  {\n";
          std::map<const Node*, std::string> slot_of;
          for (int c = 0; c < 4 && quad_ok; ++c) {
            ExprRenderer er4;
            er4.load_hook = [&](const Node& ld, std::string* out) {
              const std::string& lb = ld.args[0]->name;
              const std::string comp = "[" + std::to_string(c) + "]";
              if (avail.count(lb)) {
                *out = "eh_v_" + lb + comp;
                return true;
              }
              auto known = slot_of.find(&ld);
              if (known == slot_of.end()) {
                auto a = affine_of(*ld.args[1]);
                bool uniform = a.has_value();
                if (a)
                  for (const auto& kv : a->coef) uniform = uniform && (kv.second == 0 || still.count(kv.first));
                const bool at_element = a && sk.out_aff && *a == *sk.out_aff && ld.dtype.itemsize() == 4;
                for (const auto& lr : loads)
                  if (lr.load == &ld && lr.guarded) uniform = false;
                const std::string name = "eh_p.s" + std::to_string(quad_slots.size());
                if (uniform) {
                  ExprRenderer plain;
                  quad_load << "    " << name << " = " << plain.expr(ld) << ";\n";
                  quad_slots.push_back(ctype(ld.dtype) + " s" + std::to_string(quad_slots.size()));
                  quad_regs += 1;
                  known = slot_of.emplace(&ld, name).first;
                } else if (at_element) {
                  quad_load << "    " << name << " = *reinterpret_cast<const EhQ<" << ctype(ld.dtype) << ">*>(" << lb << " + eh_e);\n";
                  quad_slots.push_back("EhQ<" + ctype(ld.dtype) + "> s" + std::to_string(quad_slots.size()));
                  quad_regs += 4;
                  known = slot_of.emplace(&ld, name + "[]").first;
                } else {
                  quad_ok = false;
                  *out = "0";
                  return true;
                }
              }
              const std::string& sl = known->second;
              *out = sl.size() > 2 && sl.compare(sl.size() - 2, 2, "[]") == 0 ? sl.substr(0, sl.size() - 2) + comp : sl;
              return true;
            };
            quad_apply << "    eh_v_" << sk.out_buf << "[" << c << "] = (" << ctype(sk.out_dtype) << ")(" << er4.expr(*sk.value) << ");\n";
          }
          quad_load << "  }\n";
          if (needed(sk.out_buf))
            quad_apply << "    *reinterpret_cast<EhQ<" << ctype(sk.out_dtype) << ">*>(" << sk.out_buf << " + eh_e) = EhQ<" << ctype(sk.out_dtype)
                       << ">{eh_v_" << sk.out_buf << "[0], eh_v_" << sk.out_buf << "[1], eh_v_" << sk.out_buf << "[2], eh_v_" << sk.out_buf
                       << "[3]};\n";
          quad_apply << "  }\n";
        }
        if (needed(sk.out_buf)) {
          body << "    " << sk.out_buf << "[eh_e] = eh_v_" << sk.out_buf << ";\n";
          ext[sk.out_buf] = {ctype(sk.out_dtype) + "* __restrict__ " + sk.out_buf,
                             static_cast<size_t>(total) * sk.out_dtype.itemsize()};
          ext_order.push_back(sk.out_buf);
          epi.bytes += static_cast<double>(total) * sk.out_dtype.itemsize();
        } else {
          plan.elided.insert(sk.out_buf);
        }
        body << "  }\n";
      }
      for (const auto& b : ext_order) {
        epi.params += ", " + ext[b].first;
        epi.args += ", " + b;
        epi.bufs.push_back(b);
        epi.min_bytes.push_back(ext[b].second);
      }
      fn << "// what kernels";
      for (const auto& n : epi.kernels) fn << " " << n;
      fn << " do to element eh_e of " << k0.out_buf << "\n";
      fn << "__device__ __forceinline__ void eh_epilogue(long long eh_e, float eh_acc"
         << (epi.store_c ? ", " + ctype(k0.out_dtype) + "* __restrict__ " + k0.out_buf : std::string()) << epi.params
         << ") {\n" << body.str() << "}\n";
      epi.function = fn.str();
      if (split_ok && !slot_types.empty() && slot_types.size() <= 8) {
        std::ostringstream sp;
        sp << "// the same in two parts: what it reads from memory, then the rest\nstruct EhEpiLoads {\n";
        for (size_t q = 0; q < slot_types.size(); ++q) sp << "  " << slot_types[q] << " v" << q << ";\n";
        sp << "};\n__device__ __forceinline__ void eh_epilogue_load(long long eh_e, EhEpiLoads& eh_p" << epi.params << ") {\n"
           << load_body.str() << "}\n";
        sp << "__device__ __forceinline__ void eh_epilogue_apply(long long eh_e, float eh_acc, const EhEpiLoads& eh_p"
           << (epi.store_c ? ", " + ctype(k0.out_dtype) + "* __restrict__ " + k0.out_buf : std::string()) << epi.params << ") {\n"
           << apply_body.str() << "}\n";
        epi.split_functions = sp.str();
        epi.n_loads = static_cast<int>(slot_types.size());
      }
      if (quad_ok && total % 4 == 0 && quad_regs <= 24) {
        std::ostringstream qd;
        qd << "// the same for four elements in a row (eh_e a multiple of four), reads first\n"
              "template <typename T> using EhQ = T __attribute__((ext_vector_type(4)));\nstruct EhEpiLoads4 {\n";
        for (const auto& d : quad_slots) qd << "  " << d << ";\n";
        qd << "};\n__device__ __forceinline__ void eh_epilogue_load4(long long eh_e, EhEpiLoads4& eh_p" << epi.params << ") {\n"
           << quad_load.str() << "}\n";
        qd << "__device__ __forceinline__ void eh_epilogue_apply4(long long eh_e, const float (&eh_acc)[4], const EhEpiLoads4& eh_p"
           << (epi.store_c ? ", " + ctype(k0.out_dtype) + "* __restrict__ " + k0.out_buf : std::string()) << epi.params << ") {\n"
           << quad_apply.str() << "}\n";
        epi.quad_functions = qd.str();
        epi.quad_regs = quad_regs;
      }
      have_epi = true;
    }
    return have_epi;
  };

  std::vector<LaunchSpec> held_back;       // independent final reductions, issued together at the end
  // The launch just planned for kernels [i, next) (the last of them, when there are two) can run
  // whenever its inputs are ready if nothing later reads what it writes or writes what it reads
  // (a parameter's update at the end of its gradient's chain): it is taken out of the sequence.
  auto hold_back_if_sink = [&](size_t i, size_t next) {
    if (!(opt.fuse && opt.reindex && opt.merge_launches && have_table) || plan.launches.empty()) return;
    const LaunchSpec& ls = plan.launches.back();
    if (ls.grid[1] != 1 || ls.grid[2] != 1 || ls.lds_bytes || ls.block[0] % 64 || ls.source.rfind(kernel_header(), 0) != 0) return;
    std::set<std::string> written;
    for (size_t q = i; q < next; ++q)
      if (nests[q]) written.insert(nests[q]->out_buf);
      else return;
    bool sink = true;
    for (const auto& b : written)
      for (size_t r : readers[b]) sink = sink && r < next;
    for (size_t m = next; m < kernels.size() && sink; ++m)
      for (const auto& pm : kernels[m]->params)
        if (pm.dtype.is_ptr() && pm.mut_)
          sink = sink && std::find(ls.arg_bufs.begin(), ls.arg_bufs.end(), pm.name) == ls.arg_bufs.end();
    if (!sink) return;
    held_back.push_back(plan.launches.back());
    plan.launches.pop_back();
  };
  // every launch carries the key of the kernel its planning started from; options filed under that
  // key (GenOptions::launch_options) apply while it is planned
  size_t stamped = 0, stamped_held = 0, anchor = 0;
  auto stamp = [&] {
    const unsigned long long key = anchor < kernels.size() ? launch_tune_key(*kernels[anchor]) : 0;
    for (size_t q = std::min(stamped, plan.launches.size()); q < plan.launches.size(); ++q)
      if (!plan.launches[q].tune_key) plan.launches[q].tune_key = key;
    for (size_t q = std::min(stamped_held, held_back.size()); q < held_back.size(); ++q)
      if (!held_back[q].tune_key) held_back[q].tune_key = key;
    stamped = plan.launches.size();
    stamped_held = held_back.size();
  };
  size_t i = 0;
  while (i < kernels.size()) {
    stamp();
    anchor = i;
    if (folded_kernels.count(i) || absorbed.count(i)) {
      ++i;
      continue;
    }
    const GenOptions lopt = options_for_launch(opt, *kernels[i]);
    if (auto sw = scattered.find(i); sw != scattered.end()) {
      for (auto& ls : sw->second.launches) plan.launches.push_back(std::move(ls));
      i = sw->second.next;
      continue;
    }
    if (auto w = windows.find(i); w != windows.end()) {
      std::vector<const NestKernel*> chain;
      for (size_t q : w->second) chain.push_back(&*nests[q]);
      plan.launches.push_back(emit_window_reduce(*nests[i], chain, lopt, elems));
      ++i;
      continue;
    }
    if (!nests[i]) {
      auto spread = render_kernel_outer_parallel(*kernels[i], lopt, have_table && opt.fuse ? &plan.buffers : nullptr);
      if (spread.empty()) plan.launches.push_back(render_kernel_as_written(*kernels[i], lopt));
      else for (auto& ls : spread) plan.launches.push_back(std::move(ls));
      ++i;
      continue;
    }
    const NestKernel& k0 = *nests[i];
    // contraction (matmul-shaped reduce) -> MFMA schedule
    if (k0.rkind == ReduceKind::Sum && opt.gemm) {
      // elementwise kernels that follow over the same dense index space and feed on the
      // result become the contraction's epilogue
      EpilogueSpec epi;
      size_t after = i + 1;
      bool have_epi = false;
      NestKernel k0r = k0;          // k0 with C laid out as its consumer wants it, when that applies
      if (opt.gemm_epilogue && opt.fuse && have_table && gemm_shaped(k0, opt)) {
        auto gs = match_gemm(k0);
        if (gs && gemm_output_dense(*gs)) {
          have_epi = build_epilogue(i, k0, gs->batch * gs->M * gs->N, true, k0r, epi, after);
        }
      }
      // A pooling reduce over what the epilogue stores (read through its gathers) is offered to the
      // contraction as a tail: a schedule whose workgroups each store a closed share of that buffer
      // lets them compute the reduce's outputs over their share, and the reduce's launch goes.
      size_t tail_of = kernels.size();
      if (have_epi && opt.fuse && opt.window && opt.reindex && opt.gemm_tail) {
        for (const auto& w : windows) {
          const size_t ri = w.first;
          if (ri < after || folded_kernels.count(ri) || absorbed.count(ri) || !nests[ri]) continue;
          std::vector<const NestKernel*> chain;
          for (size_t q : w.second) chain.push_back(&*nests[q]);
          // nothing between here and the reduce may write what it writes or read it
          bool free_to_move = true;
          for (size_t m = after; m < ri && free_to_move; ++m) {
            if (folded_kernels.count(m) || absorbed.count(m)) continue;
            for (const auto& pm : kernels[m]->params) free_to_move = free_to_move && pm.name != nests[ri]->out_buf;
          }
          if (!free_to_move) continue;
          if (window_reduce_tail(*nests[ri], chain, elems, &epi)) {
            tail_of = ri;
            break;
          }
        }
      }
      auto gl = try_emit_gemm(have_epi ? k0r : k0, lopt, &plan.buffers, &folded, have_epi ? &epi : nullptr);
      if (!gl.empty() && tail_of < kernels.size()) {
        // taken when the launch lists the reduce among its kernels
        const auto& ks = gl.back().kernels;
        if (std::find(ks.begin(), ks.end(), nests[tail_of]->name) != ks.end()) {
          folded_kernels.insert(tail_of);
          windows.erase(tail_of);
        }
      }
      if (!gl.empty()) {
        if (absorbed_name.count(i)) gl.back().kernels.push_back(absorbed_name[i]);
        // K was split and the next kernel only sums the (dense) result over the batch axis: it
        // sums the partial tiles of all chunks and all batch elements in one go (chunks lie
        // above the batch in the scratch buffer, so the two walk as one axis), and the launch
        // that would add the chunks up goes
        if (gl.size() == 2 && !have_epi && !absorbed_name.count(i) && opt.fuse && opt.reindex && have_table) {
          size_t j = i + 1;
          while (j < kernels.size() && (absorbed.count(j) || folded_kernels.count(j))) ++j;
          auto gs = match_gemm(k0);
          const std::string& scratch = gl[0].arg_bufs.back();
          if (j < kernels.size() && nests[j] && gs && gs->batch > 1 && gemm_output_dense(*gs) &&
              gl[0].grid[1] > 1 && scratch.rfind("eh_part_", 0) == 0) {
            NestKernel& r2 = *nests[j];
            const Node& v2 = *r2.value;
            auto ra = v2.op == Op::Load && v2.count == 1 && v2.args[0]->op == Op::Var && v2.args[0]->name == k0.out_buf
                          ? affine_of(*v2.args[1]) : std::nullopt;
            const int64_t tile = gs->M * gs->N;
            bool ok = r2.rkind == ReduceKind::Sum && ra && ra->c == 0 && r2.acc_dtype.ty == Ty::F32 &&
                      r2.rloop.extent == gs->batch && ra->of(r2.rloop.var) == tile && role_of(k0.out_buf) == "temp" &&
                      readers[k0.out_buf] == std::vector<size_t>{j} && !(opt.gemm && gemm_shaped(r2, opt));
            // the other loops of r2 stay inside one tile
            int64_t reach = 0;
            if (ok)
              for (const auto& l : r2.loops) {
                if (l.extent <= 1) continue;
                ok = ok && ra->of(l.var) > 0;
                reach += ra->of(l.var) * (l.extent - 1);
              }
            if (ok && reach < tile) {
              const int64_t S = gl[0].grid[1];
              std::map<std::string, NodePtr> to_scratch{{k0.out_buf, make_var(scratch)}};
              r2.value = rename(r2.value, to_scratch);
              r2.rloop.extent *= S;
              for (auto& pp : r2.params)
                if (pp.name == k0.out_buf) pp.name = scratch;
              plan.elided.insert(k0.out_buf);
              gl.pop_back();
            }
          }
        }
        const bool two = gl.size() == 2;
        for (auto& ls : gl) plan.launches.push_back(std::move(ls));
        if (two && !absorbed_name.count(i)) hold_back_if_sink(i, have_epi ? after : i + 1);   // the launch that sums the chunks (and updates the weight)
        i = have_epi ? after : i + 1;
        continue;
      }
      if (have_epi) throw Error("internal: contraction '" + k0.name + "' matched but could not be emitted");
    }
    if (k0.rkind != ReduceKind::None && !reduce_is_rowwise(k0)) {
      // elementwise kernels over the reduce's (dense) output that feed on it ride along: a
      // parameter's update in the launch that finishes its gradient's sum
      EpilogueSpec epi;
      size_t after = i + 1;
      NestKernel k0r = k0;
      int64_t numel = 0;
      bool have_epi = false;
      if (opt.gemm_epilogue && opt.fuse && have_table && k0.acc_dtype.ty == Ty::F32 && k0.out_dtype.ty == Ty::F32 &&
          dense_strides(k0, &numel))
        have_epi = build_epilogue(i, k0, numel, false, k0r, epi, after);
      emit_serial_reduce(k0, lopt, &plan, have_epi ? &epi : nullptr);
      // A one-launch reduce at the end of its chain (nothing later reads what it writes or
      // writes what it reads: a parameter's update) can run whenever its inputs are ready:
      // it is held back and issued together with the others of its kind as one launch.
      hold_back_if_sink(i, have_epi ? after : i + 1);
      i = have_epi ? after : i + 1;
      continue;
    }
    // start a group with kernel i and extend it while the next kernels fit
    Group g;
    size_t first = i;
    {
      Canon c = canon_as(k0, k0.rkind == ReduceKind::None ? StageKind::Wide : StageKind::Reduce);
      if (!c.ok) {
        plan.launches.push_back(render_kernel_as_written(*kernels[i], lopt));
        ++i;
        continue;
      }
      g.rows = c.rows;
      g.C = c.C;
      g.stages.push_back(c.stage);
    }
    ++i;
    // kernel k as the group's next stage, if it fits
    auto stage_for = [&](const NestKernel& k) {
      Canon pick;
      if (k.rkind == ReduceKind::Sum && opt.gemm && gemm_shaped(k, opt)) return pick;
      if (k.rkind != ReduceKind::None) {
        if (!reduce_is_rowwise(k)) return pick;
        Canon c = canon_as(k, StageKind::Reduce);
        if (c.ok && c.rows == g.rows && c.C == g.C) pick = c;
      } else {
        Canon w = canon_as(k, StageKind::Wide);
        if (w.ok && w.rows == g.rows && w.C == g.C) pick = w;
        else {
          Canon s = canon_as(k, StageKind::Scalar);
          if (s.ok && s.rows == g.rows && g.has_reduce()) pick = s;
        }
      }
      // a buffer may be written once per group
      if (pick.ok && (!aligned_with_group(g, pick.stage) || g.producer(pick.stage.out_buf))) pick.ok = false;
      return pick;
    };
    // (a reduce that reads through its gathers, or a contraction with its shifted sums, has a
    // launch of its own planned: its operands are not in memory for a stage of this group to read)
    while (opt.fuse && i < kernels.size() && nests[i] && !folded_kernels.count(i) && !windows.count(i) && !scattered.count(i)) {
      if (absorbed.count(i)) {
        ++i;
        continue;
      }
      Canon pick = stage_for(*nests[i]);
      if (!pick.ok) break;
      g.stages.push_back(pick.stage);
      ++i;
    }
    // Kernels further down that carry on with this group's rows on a few thousand elements (the
    // bookkeeping of a loss, lowered behind the kernels of another root) join it when nothing in
    // between has a hand in what they read or write: one launch less on the way, and no large
    // value has to be kept for them.
    if (opt.fuse && opt.reindex && opt.merge_launches && have_table && g.has_reduce()) {
      auto tiny = [&](const Node* k) {
        for (const auto& p : k->params) {
          if (!p.dtype.is_ptr()) continue;
          auto e = elems.find(p.name);
          if (e == elems.end() || e->second > (size_t{1} << 12)) return false;
        }
        return true;
      };
      for (size_t j = i; j < kernels.size() && j < i + 200; ++j) {
        if (absorbed.count(j) || folded_kernels.count(j) || windows.count(j) || scattered.count(j) || absorbed_name.count(j)) continue;
        if (!nests[j] || !tiny(kernels[j])) continue;
        bool feeds = false;
        for (const auto& p : kernels[j]->params)
          feeds = feeds || (p.dtype.is_ptr() && !p.mut_ && g.producer(p.name));
        if (!feeds) continue;
        bool free_to_move = true;
        for (size_t m = i; m < j && free_to_move; ++m) {
          if (absorbed.count(m)) continue;              // (already part of an earlier launch, this group's included)
          for (const auto& pm : kernels[m]->params)
            for (const auto& pj : kernels[j]->params)
              if (pm.dtype.is_ptr() && pj.dtype.is_ptr() && pm.name == pj.name && (pm.mut_ || pj.mut_)) free_to_move = false;
        }
        if (!free_to_move) continue;
        Canon pick = stage_for(*nests[j]);
        if (!pick.ok) continue;
        g.stages.push_back(pick.stage);
        absorbed.insert(j);
      }
    }
    // which stage outputs must reach memory
    for (size_t s = 0; s < g.stages.size(); ++s) {
      Stage& st = g.stages[s];
      bool needed = role_of(st.out_buf) != "temp";
      for (size_t r : readers[st.out_buf])
        if (r < first || r >= i) needed = true;
      st.store = needed;
      if (!needed) plan.elided.insert(st.out_buf);
    }
    plan.launches.push_back(emit_group(g, lopt, elems));
  }
  stamp();
  // what was held back goes to the end one by one: the pass that issues independent launches together
  // (below) merges it with whatever else is still waiting there, by workgroup size (a part's surplus
  // work-items leave at once, but they are launched all the same)
  for (auto& ls : held_back) plan.launches.push_back(std::move(ls));
  // constant inputs no launch binds any more need not exist
  for (const auto& c : consts) {
    bool bound = false;
    for (const auto& ls : plan.launches)
      for (const auto& a : ls.arg_bufs) bound = bound || a == c.first;
    if (!bound) plan.elided.insert(c.first);
  }
  // a launch that covers a kernel which took another one in covers that one too
  // (before launches are merged: the covered kernels decide which buffers a launch writes)
  for (auto& ls : plan.launches) {
    const std::vector<std::string> covered = ls.kernels;
    for (const auto& kn : covered)
      for (const auto& an : absorbed_name)
        if (nests[an.first] && nests[an.first]->name == kn &&
            std::find(ls.kernels.begin(), ls.kernels.end(), an.second) == ls.kernels.end())
          ls.kernels.push_back(an.second);
  }
  issue_independent_launches_together(&plan, kernels, opt);
  // A lowered kernel whose output index is the dense index of its loops writes every element of
  // its output; the launch that stores it overwrites a buffer of exactly that size, whatever it
  // held (the executor need not have zero-filled it first).
  {
    std::map<std::string, std::pair<std::string, size_t>> dense_out;     // kernel -> (buffer, bytes)
    for (const auto& nk : nests) {
      int64_t numel = 0;
      if (nk && !partly_written.count(nk->name) && dense_strides(*nk, &numel))
        dense_out[nk->name] = {nk->out_buf, static_cast<size_t>(numel) * nk->out_dtype.itemsize()};
    }
    for (auto& ls : plan.launches) {
      ls.arg_full_bytes.assign(ls.arg_bufs.size(), 0);
      for (const auto& kn : ls.kernels) {
        auto it = dense_out.find(kn);
        if (it == dense_out.end()) continue;
        for (size_t a = 0; a < ls.arg_bufs.size(); ++a)
          if (ls.arg_bufs[a] == it->second.first) ls.arg_full_bytes[a] = it->second.second;
      }
    }
  }
  assign_lanes(&plan, kernels, opt);
  return plan;
}

}  // namespace eh
