// Host-side robustness driver for the AST reader, the normaliser and the planner, meant to be
// built with AddressSanitizer and UndefinedBehaviorSanitizer (harp_amd/build.py,
// build_host_fuzz).  No GPU and no HIP runtime involved: it links the generator sources only.
//
//   host_fuzz <corpus file> <mutations per entry> <seed>
//
// The corpus holds one AST text per line.  Every entry is parsed, normalised and planned as it
// is (that must succeed), then mutated `mutations` times -- bytes deleted, inserted and replaced,
// atoms swapped for hostile ones, sub-expressions duplicated, the text truncated -- and pushed
// through the same calls.  A mutated text may be rejected (eh::Error) or accepted; what it may
// not do is crash, read out of bounds, overflow a signed integer or trip any other sanitizer
// check, nor keep the planner busy for more than ten seconds.  Prints a one-line summary and
// exits 0; a sanitizer report aborts the process.
#include <csignal>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <exception>
#include <fstream>
#include <iostream>
#include <string>
#include <vector>

#include <unistd.h>

#include "../harp_amd/csrc/analysis.hpp"
#include "../harp_amd/csrc/ast.hpp"
#include "../harp_amd/csrc/codegen.hpp"
#include "../harp_amd/csrc/normalize.hpp"

namespace {

struct Rng {
  uint64_t s;
  uint64_t next() {
    s ^= s << 13;
    s ^= s >> 7;
    s ^= s << 17;
    return s;
  }
  size_t below(size_t n) { return n ? static_cast<size_t>(next() % n) : 0; }
};

const char* kHostile[] = {
    "0", "-1", "1", "9223372036854775807", "-9223372036854775808", "4611686018427387904", "65536",
    "999999999999", "#ffffffff", "#7fc00000", "#00000000", "nan", "inf", "-inf", "i64", "f32", "f64", "bool",
    "unknown", "void", "(ptr f32 global)", "(vec f32 4)", "range", "store", "load", "block", "assign", "kernel",
    "program", "const", "var", "add", "mul", "idiv", "rem", "shl", "select", "if", "sequential", "openmp",
    "\"ridx0\"", "\"acc\"", "\"\"", "(decls)", "(buffers)", "mut", "imm", "normal", "(group_id 0)", "(local_id 7)"};

// start and end of the s-expression that opens at or after `from` (balanced parentheses)
bool subexpr(const std::string& t, size_t from, size_t* a, size_t* b) {
  size_t i = t.find('(', from);
  if (i == std::string::npos) return false;
  int depth = 0;
  for (size_t j = i; j < t.size(); ++j) {
    if (t[j] == '(') ++depth;
    if (t[j] == ')' && --depth == 0) {
      *a = i;
      *b = j + 1;
      return true;
    }
  }
  return false;
}

std::string mutate(const std::string& in, Rng& r) {
  std::string t = in;
  const int edits = 1 + static_cast<int>(r.below(3));
  for (int e = 0; e < edits && !t.empty(); ++e) {
    switch (r.below(7)) {
      case 0: t.erase(r.below(t.size()), 1 + r.below(4)); break;
      case 1: t.insert(r.below(t.size()), 1, "()\" #-0123456789abcxyz"[r.below(22)]); break;
      case 2: t[r.below(t.size())] = "()\" #-019"[r.below(9)]; break;
      case 3: t.resize(r.below(t.size())); break;
      case 4: {            // an atom replaced by a hostile one
        size_t p = r.below(t.size());
        while (p < t.size() && (t[p] == '(' || t[p] == ')' || t[p] == ' ')) ++p;
        size_t q = p;
        while (q < t.size() && t[q] != '(' && t[q] != ')' && t[q] != ' ') ++q;
        if (p < q) t.replace(p, q - p, kHostile[r.below(sizeof kHostile / sizeof *kHostile)]);
        break;
      }
      case 5: {            // a sub-expression duplicated in place
        size_t a, b;
        if (subexpr(t, r.below(t.size()), &a, &b) && b - a < 4000) t.insert(b, " " + t.substr(a, b - a));
        break;
      }
      default: {           // a sub-expression replaced by another one of the same text
        size_t a, b, c, d;
        if (subexpr(t, r.below(t.size()), &a, &b) && subexpr(t, r.below(t.size()), &c, &d) && d - c < 4000) {
          const std::string other = t.substr(c, d - c);
          t.replace(a, b - a, other);
        }
      }
    }
  }
  return t;
}

// An input that keeps the planner busy for more than ten seconds is a finding too: the alarm
// prints it and ends the run.
const std::string* g_current = nullptr;
void on_alarm(int) {
  static const char msg[] = "host_fuzz: an input took more than 10 s:\n";
  (void)!write(2, msg, sizeof msg - 1);
  if (g_current) (void)!write(2, g_current->data(), g_current->size() < 6000 ? g_current->size() : 6000);
  (void)!write(2, "\n", 1);
  _exit(3);
}

// Parse, normalise, plan.  Returns 0 accepted, 1 rejected with eh::Error, 2 other exception.
int run_one(const std::string& text) {
  g_current = &text;
  alarm(10);
  try {
    eh::NodePtr ast = eh::parse_ast(text);
    if (ast->op == eh::Op::Kernel) ast = eh::make(eh::Op::Program, {ast});
    eh::validate_sizes(*ast);
    if (ast->op == eh::Op::Program)
      for (const auto& f : ast->args)
        if (f->op == eh::Op::Kernel) (void)eh::to_text(*eh::normalize_kernel(f));
    eh::GenOptions opt;
    opt.allow_serial = true;
    (void)eh::plan_program(*ast, opt);
    return 0;
  } catch (const eh::Error&) {
    return 1;
  } catch (const std::exception& e) {
    std::fprintf(stderr, "unexpected exception type: %s\n", e.what());
    return 2;
  }
}

}  // namespace

int main(int argc, char** argv) {
  if (argc < 4) {
    std::fprintf(stderr, "usage: host_fuzz <corpus> <mutations per entry> <seed>\n");
    return 2;
  }
  std::signal(SIGALRM, on_alarm);
  std::ifstream f(argv[1]);
  std::vector<std::string> corpus;
  for (std::string line; std::getline(f, line);)
    if (!line.empty()) corpus.push_back(line);
  const long per_entry = std::atol(argv[2]);
  Rng rng{static_cast<uint64_t>(std::atoll(argv[3])) * 0x9e3779b97f4a7c15ull + 1};
  long accepted = 0, rejected = 0, odd = 0;
  for (size_t i = 0; i < corpus.size(); ++i) {
    if (run_one(corpus[i]) != 0) {
      std::fprintf(stderr, "corpus entry %zu was not accepted as it is\n", i);
      return 1;
    }
    for (long m = 0; m < per_entry; ++m) {
      const int rc = run_one(mutate(corpus[i], rng));
      if (rc == 0) ++accepted;
      else if (rc == 1) ++rejected;
      else ++odd;
    }
  }
  std::printf("host_fuzz: %zu corpus entries, %ld mutations accepted, %ld rejected, %ld odd\n", corpus.size(), accepted,
              rejected, odd);
  return odd ? 1 : 0;
}
