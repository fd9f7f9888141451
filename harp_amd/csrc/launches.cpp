// Passes over the planned launches: what each writes, which go out together, lanes.
#include <cctype>
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

// Which buffers each launch writes, and which launches may run beside each other.
//
// A program's launches are planned in an order that is valid one after the other.  Many of them
// do not depend on each other, though: in a training step the gradient of every parameter and
// its update hang off the chain that carries the gradient back through the layers, and most of
// them are small launches that cost their few microseconds of launch latency whatever they
// compute.  Launches are therefore given lanes: lane 0 (the device's stream) takes the chain of
// dependent launches with the largest estimated duration, the others go to side lanes that run
// concurrently; a launch waits for the launches on other lanes whose buffers it reads or
// overwrites (`waits`), and the executor joins the lanes at the end of the program.  The results
// do not depend on the lanes: every launch still sees exactly the inputs it would have seen.
// Which of its buffers each launch writes: the outputs of the lowered kernels it covers; a scratch
// buffer the plan added is written by the first launch that binds it and read by the later ones.
void mark_written(ProgramPlan* plan, const std::vector<const Node*>& kernels) {
  auto& L = plan->launches;
  std::map<std::string, const Node*> by_name;
  for (const Node* k : kernels) by_name[k->name] = k;
  // written: outputs of the lowered kernels a launch covers; a scratch buffer the plan added is
  // written by the first launch that binds it and read by the later ones
  std::set<std::string> scratch_seen;
  for (auto& ls : L) {
    std::set<std::string> outs;
    bool known = !ls.kernels.empty();
    for (const auto& kn : ls.kernels) {
      auto it = by_name.find(kn);
      if (it == by_name.end()) { known = false; continue; }
      for (const auto& p : it->second->params)
        if (p.dtype.is_ptr() && p.mut_) outs.insert(p.name);
    }
    // a launch whose kernels cannot be looked up is taken to write everything it binds
    ls.arg_written.assign(ls.arg_bufs.size(), known ? 0 : 1);
    for (size_t a = 0; a < ls.arg_bufs.size() && known; ++a) {
      const std::string& b = ls.arg_bufs[a];
      bool declared = false;
      for (const Node* k : kernels)
        for (const auto& p : k->params) declared = declared || p.name == b;
      if (outs.count(b)) ls.arg_written[a] = 1;
      else if (!declared && scratch_seen.insert(b).second) ls.arg_written[a] = 1;
    }
  }
}

// Launches of the elementwise / reduce schedules that do not depend on each other are issued as one
// launch (merge_launches).  A launch that could be merged is held until a launch that depends on it
// (reads what it writes, writes what it reads or writes) comes up; launches that depend on nothing
// held pass it by, which only changes the order among independent launches.  What is held at
// that point goes out together, grouped by workgroup size.
void issue_independent_launches_together(ProgramPlan* plan, const std::vector<const Node*>& kernels, const GenOptions& opt) {
  if (!(opt.fuse && opt.reindex && opt.merge_launches) || plan->launches.size() < 3) return;
  mark_written(plan, kernels);
  const std::string head = kernel_header();
  // A contraction built from a kernel template can be compiled as a part of a larger launch.
  // Only the small ones are: four waves a workgroup, at most 4 GFLOP -- the weight gradients of a
  // small network, each a few microseconds above the cost of a launch.  A part's LDS is the
  // launch's, so these go out among themselves, never with kernels that want many workgroups a CU.
  auto template_part = [&](const LaunchSpec& ls) {
    return !ls.part_params.empty() && ls.block[0] == 256 && ls.block[1] == 1 && ls.block[2] == 1 && !ls.lds_bytes &&
           ls.flops <= 4e9 && !ls.kernels.empty() && opt.merge_templates && ls.schedule.find(",tail=") == std::string::npos;
  };
  auto size_class = [&](const LaunchSpec& ls) { return ls.block[0] * 2 + (template_part(ls) ? 1u : 0u); };
  auto mergeable = [&](const LaunchSpec& ls) {
    if (template_part(ls)) return true;
    if (ls.grid[1] != 1 || ls.grid[2] != 1 || ls.block[1] != 1 || ls.block[2] != 1 || ls.block[0] % 64 || ls.lds_bytes) return false;
    if (ls.source.rfind(head, 0) != 0 || ls.schedule.rfind("together(", 0) == 0 || ls.kernels.empty()) return false;
    const std::string open = "extern \"C\" __global__ void __launch_bounds__(" + std::to_string(ls.block[0]) + ") " + ls.entry + "(";
    const size_t at = ls.source.find(open);
    return at != std::string::npos && ls.source.find("__global__", at + open.size()) == std::string::npos &&
           ls.source.find("blockIdx.y") == std::string::npos && ls.source.find("blockDim") == std::string::npos;
  };
  auto conflict = [](const LaunchSpec& a, const LaunchSpec& b) {
    for (size_t i = 0; i < a.arg_bufs.size(); ++i)
      for (size_t j = 0; j < b.arg_bufs.size(); ++j)
        if (a.arg_bufs[i] == b.arg_bufs[j] && (a.arg_written[i] || b.arg_written[j])) return true;
    return false;
  };
  std::vector<LaunchSpec> in = std::move(plan->launches), out, held;
  std::vector<char> taken(in.size(), 0);       // pulled forward into an earlier launch
  // The held launches of every workgroup size that has one in the way of `trigger` (all of them
  // at the end) go out as one launch per size.  Each takes along what further down the list could
  // run here just as well: launches of its size that depend on nothing between here and there
  // (the final launches of a training step, which nothing reads, were put at the end of the list).
  auto flush = [&](size_t next, const LaunchSpec* trigger) {
    std::map<unsigned, std::vector<LaunchSpec>> by_block;
    std::vector<LaunchSpec> stay;
    std::set<unsigned> go;
    for (const auto& h : held)
      if (!trigger || conflict(*trigger, h)) go.insert(size_class(h));
    for (auto& h : held) {
      if (go.count(size_class(h))) by_block[size_class(h)].push_back(std::move(h));
      else stay.push_back(std::move(h));
    }
    held = std::move(stay);
    for (auto& kv : by_block) {
      for (size_t q = next; q < in.size(); ++q) {
        if (taken[q] || !mergeable(in[q]) || size_class(in[q]) != kv.first) continue;
        bool free_to_move = true;
        for (size_t p = next; p < q && free_to_move; ++p) free_to_move = taken[p] || !conflict(in[q], in[p]);
        for (const auto& h : held) free_to_move = free_to_move && !conflict(in[q], h);
        for (const auto& g : by_block)
          for (const auto& m : g.second) free_to_move = free_to_move && !conflict(in[q], m);
        if (!free_to_move) continue;
        kv.second.push_back(std::move(in[q]));
        taken[q] = 1;
      }
      if (kv.second.size() >= 2) out.push_back(merge_launches(kv.second, opt));
      else out.push_back(std::move(kv.second.front()));
    }
  };
  for (size_t q = 0; q < in.size(); ++q) {
    if (taken[q]) continue;
    LaunchSpec& ls = in[q];
    bool dep = false;
    for (const auto& h : held) dep = dep || conflict(ls, h);
    if (dep) flush(q, &ls);
    if (mergeable(ls)) held.push_back(std::move(ls));
    else out.push_back(std::move(ls));
    taken[q] = 1;
  }
  flush(in.size(), nullptr);
  plan->launches = std::move(out);
}

void assign_lanes(ProgramPlan* plan, const std::vector<const Node*>& kernels, const GenOptions& opt) {
  auto& L = plan->launches;
  const size_t n = L.size();
  mark_written(plan, kernels);
  plan->lanes = 1;
  for (auto& ls : L) { ls.lane = 0; ls.waits.clear(); }
  if (opt.lanes < 2 || n < 8) return;
  // dependences: read after write, write after write, write after read
  std::vector<std::vector<int>> deps(n);
  for (size_t j = 0; j < n; ++j)
    for (size_t i = 0; i < j; ++i) {
      bool dep = false;
      for (size_t a = 0; a < L[i].arg_bufs.size() && !dep; ++a)
        for (size_t b = 0; b < L[j].arg_bufs.size() && !dep; ++b)
          dep = L[i].arg_bufs[a] == L[j].arg_bufs[b] && (L[i].arg_written[a] || L[j].arg_written[b]);
      if (dep) deps[j].push_back(static_cast<int>(i));
    }
  // estimated microseconds: a launch floor plus traffic at half the memory rate or the matrix
  // cores at a third of theirs
  std::vector<double> est(n), path(n);
  std::vector<int> prev(n, -1);
  for (size_t j = 0; j < n; ++j) {
    est[j] = 4.0 + std::max(L[j].algo_bytes / 4.0e6, L[j].flops / 5.0e7);
    path[j] = est[j];
    for (int i : deps[j])
      if (path[static_cast<size_t>(i)] + est[j] > path[j]) {
        path[j] = path[static_cast<size_t>(i)] + est[j];
        prev[j] = i;
      }
  }
  size_t end = 0;
  for (size_t j = 0; j < n; ++j)
    if (path[j] > path[end]) end = j;
  std::vector<char> on_main(n, 0);
  for (int j = static_cast<int>(end); j >= 0; j = prev[static_cast<size_t>(j)]) on_main[static_cast<size_t>(j)] = 1;
  // a launch that fills the chip for long gains nothing from company and slows down in it
  if (opt.lane_us > 0)
    for (size_t j = 0; j < n; ++j)
      if (est[j] > opt.lane_us) on_main[j] = 1;
  // lane 0 never waits for a side lane: whatever a launch of lane 0 depends on is on lane 0 too
  for (size_t j = n; j-- > 0;)
    if (on_main[j])
      for (int i : deps[j]) on_main[static_cast<size_t>(i)] = 1;
  double side_us = 0;
  for (size_t j = 0; j < n; ++j)
    if (!on_main[j]) side_us += est[j];
  if (side_us < 24.0) return;                       // not worth a fork and a join
  const int lanes = std::min(opt.lanes, 4);
  // bottom level: what still has to run behind a launch, the launch included
  std::vector<double> tail(n);
  for (size_t j = n; j-- > 0;) {
    tail[j] = std::max(tail[j], est[j]);
    for (int i : deps[j]) tail[static_cast<size_t>(i)] = std::max(tail[static_cast<size_t>(i)], est[static_cast<size_t>(i)] + tail[j]);
  }
  // List scheduling: of the launches whose producers are placed, the one that can start first
  // goes next (the longer tail on a tie); chain launches on lane 0, the others on the side lane
  // that is free first.  The order of placement is the order of issue: a lane runs in order, so
  // a side lane must be handed its launches in the order in which their inputs become ready.
  std::vector<double> lane_free(static_cast<size_t>(lanes), 0.0), finish(n, 0.0);
  std::vector<char> placed(n, 0);
  std::vector<int> lane_of(n, 0);
  std::vector<size_t> order;
  while (order.size() < n) {
    int best = -1, best_lane = 0;
    double best_start = 0;
    for (size_t j = 0; j < n; ++j) {
      if (placed[j]) continue;
      bool ok = true;
      double ready = 0;
      int dep_lane = -1;
      for (int i : deps[j]) {
        ok = ok && placed[static_cast<size_t>(i)];
        if (finish[static_cast<size_t>(i)] >= ready) {
          ready = finish[static_cast<size_t>(i)];
          dep_lane = lane_of[static_cast<size_t>(i)];
        }
      }
      if (!ok) continue;
      int lane = 0;
      if (!on_main[j]) {
        lane = 1;
        for (int t = 2; t < lanes; ++t)
          if (lane_free[static_cast<size_t>(t)] < lane_free[static_cast<size_t>(lane)]) lane = t;
        // behind its last producer when that costs nothing: no wait across lanes then
        if (dep_lane > 0 && lane_free[static_cast<size_t>(dep_lane)] <= std::max(ready, lane_free[static_cast<size_t>(lane)])) lane = dep_lane;
      }
      const double start = std::max(ready, lane_free[static_cast<size_t>(lane)]);
      if (best < 0 || start < best_start - 1e-9 || (start < best_start + 1e-9 && tail[j] > tail[static_cast<size_t>(best)])) {
        best = static_cast<int>(j);
        best_lane = lane;
        best_start = start;
      }
    }
    const size_t j = static_cast<size_t>(best);
    placed[j] = 1;
    lane_of[j] = best_lane;
    finish[j] = best_start + est[j];
    lane_free[static_cast<size_t>(best_lane)] = finish[j];
    order.push_back(j);
  }
  std::vector<int> position(n);
  for (size_t q = 0; q < n; ++q) position[order[q]] = static_cast<int>(q);
  std::vector<LaunchSpec> sorted;
  sorted.reserve(n);
  for (size_t q = 0; q < n; ++q) {
    sorted.push_back(std::move(L[order[q]]));
    sorted.back().lane = lane_of[order[q]];
    plan->lanes = std::max(plan->lanes, sorted.back().lane + 1);
  }
  // a lane runs its launches in order, so waiting for one launch of a lane covers that lane's
  // earlier launches too
  std::vector<std::vector<int>> waited(static_cast<size_t>(lanes), std::vector<int>(static_cast<size_t>(lanes), -1));
  for (size_t q = 0; q < n; ++q) {
    const size_t lj = static_cast<size_t>(sorted[q].lane);
    std::vector<int> latest(static_cast<size_t>(lanes), -1);
    for (int i : deps[order[q]]) {
      const int pi = position[static_cast<size_t>(i)];
      const size_t li = static_cast<size_t>(sorted[static_cast<size_t>(pi)].lane);
      if (li != lj) latest[li] = std::max(latest[li], pi);
    }
    for (size_t t = 0; t < latest.size(); ++t)
      if (latest[t] > waited[lj][t]) {
        sorted[q].waits.push_back(latest[t]);
        waited[lj][t] = latest[t];
      }
  }
  L = std::move(sorted);
}


LaunchSpec merge_launches(const std::vector<LaunchSpec>& parts_in, const GenOptions& opt) {
  LaunchSpec out;
  const std::string head = hdr(opt);
  // template kernels: the longest first, so that the launch ends on its short parts
  std::vector<LaunchSpec> parts = parts_in;
  const bool templates = !parts.front().part_params.empty();
  if (templates)
    std::stable_sort(parts.begin(), parts.end(), [](const LaunchSpec& x, const LaunchSpec& y) { return x.flops > y.flops; });
  unsigned block = 0;
  for (const auto& p : parts) block = std::max(block, p.block[0]);
  out.entry = parts.front().entry + "_and_" + std::to_string(parts.size() - 1);
  out.tune_key = parts.front().tune_key;
  std::ostringstream os, sig, body, lds;
  os << head;
  unsigned first = 0;
  for (size_t i = 0; i < parts.size(); ++i) {
    const LaunchSpec& p = parts[i];
    const std::string ns = "eh_part" + std::to_string(i);
    std::string params;
    unsigned blocks = p.grid[0];
    if (templates) {
      // the template's EH_PART mode: a device function eh_run(linear workgroup id, LDS block, parameters...)
      if (p.part_params.empty() || p.block[0] != block || p.block[1] != 1 || p.block[2] != 1 || p.lds_bytes)
        throw Error("internal: launch '" + p.entry + "' cannot be merged");
      blocks = p.grid[0] * p.grid[1] * p.grid[2];
      os << "#define EH_PART 1\n#define EH_PART_GX " << p.grid[0] << "u\n#define EH_PART_GY " << p.grid[1] << "u\n";
      os << "namespace " << ns << " {\n" << p.source << "}  // namespace " << ns << "\n";
      // every macro the part defined goes again: the next part defines its own
      std::set<std::string> macros = {"EH_PART", "EH_PART_GX", "EH_PART_GY"};
      for (size_t q = p.source.find("#define "); q != std::string::npos; q = p.source.find("#define ", q + 8)) {
        if (q > 0 && p.source[q - 1] != '\n') continue;
        size_t e = q + 8;
        while (e < p.source.size() && (std::isalnum(static_cast<unsigned char>(p.source[e])) || p.source[e] == '_')) ++e;
        macros.insert(p.source.substr(q + 8, e - q - 8));
      }
      for (const auto& m : macros) os << "#undef " << m << "\n";
      params = p.part_params;
      lds << "eh_max2(" << ns << "::eh_lds_floats, ";
    } else {
      if (p.source.rfind(head, 0) != 0 || p.grid[1] != 1 || p.grid[2] != 1 || p.block[1] != 1 || p.block[2] != 1 || p.block[0] % 64 || p.lds_bytes)
        throw Error("internal: launch '" + p.entry + "' cannot be merged");
      std::string text = p.source.substr(head.size());
      const std::string open = "extern \"C\" __global__ void __launch_bounds__(" + std::to_string(p.block[0]) + ") " + p.entry + "(";
      const size_t at = text.find(open);
      const size_t close = at == std::string::npos ? at : text.find(") {\n", at);
      if (close == std::string::npos) throw Error("internal: launch '" + p.entry + "' has no entry point to merge");
      params = text.substr(at + open.size(), close - at - open.size());
      text.replace(at, open.size(), "__device__ __forceinline__ void eh_run(const unsigned eh_bx, ");
      for (size_t q = text.find("blockIdx.x"); q != std::string::npos; q = text.find("blockIdx.x", q)) text.replace(q, 10, "eh_bx");
      const std::string own_grid = std::to_string(p.grid[0]) + "u";
      for (size_t q = text.find("gridDim.x"); q != std::string::npos; q = text.find("gridDim.x", q)) text.replace(q, 9, own_grid);
      os << "namespace " << ns << " {\n" << text << "}  // namespace " << ns << "\n";
    }
    // the part's parameters, renamed, in the merged signature; the same names in the call
    std::string call;
    size_t from = 0, n = 0;
    while (from < params.size()) {
      size_t comma = params.find(", ", from);
      if (comma == std::string::npos) comma = params.size();
      std::string one = params.substr(from, comma - from);
      while (!one.empty() && one.front() == ' ') one.erase(one.begin());
      while (!one.empty() && one.back() == ' ') one.pop_back();
      from = comma + 2;
      if (one.empty()) continue;
      const size_t sp = one.rfind(' ');
      const std::string name = "p" + std::to_string(i) + "_" + one.substr(sp + 1);
      sig << (sig.tellp() > 0 ? ", " : "") << one.substr(0, sp + 1) << name;
      call += ", " + name;
      ++n;
    }
    if (n != p.arg_bufs.size()) throw Error("internal: launch '" + p.entry + "' lists " + std::to_string(p.arg_bufs.size()) + " buffers for " + std::to_string(n) + " parameters");
    body << "  if (blockIdx.x < " << first + blocks << "u) {\n    if (threadIdx.x < " << p.block[0] << "u) " << ns << "::eh_run(blockIdx.x - "
         << first << "u" << (templates ? ", eh_lds" : "") << call << ");\n    return;\n  }\n";
    first += blocks;
    for (size_t a = 0; a < p.arg_bufs.size(); ++a) {
      out.arg_bufs.push_back(p.arg_bufs[a]);
      out.arg_min_bytes.push_back(a < p.arg_min_bytes.size() ? p.arg_min_bytes[a] : 0);
    }
    for (const auto& kn : p.kernels) out.kernels.push_back(kn);
    out.algo_bytes += p.algo_bytes;
    out.flops += p.flops;
    out.schedule += (i ? " + " : "together(") + p.schedule;
  }
  out.schedule += ")";
  if (templates) {
    os << "namespace {\nconstexpr int eh_max2(int a, int b) { return a > b ? a : b; }\n}\n";
  }
  os << "extern \"C\" __global__ void __launch_bounds__(" << block << ") " << out.entry << "(" << sig.str() << ") {\n";
  if (templates)
    os << "  // the parts' tiles, one part at a time: a workgroup runs exactly one part\n"
       << "  __shared__ __attribute__((aligned(16))) float eh_lds[" << lds.str() << "4" << std::string(parts.size(), ')') << "];\n";
  os << body.str() << "}\n";
  out.source = os.str();
  out.grid[0] = first;
  out.block[0] = block;
  return out;
}


}  // namespace eh
