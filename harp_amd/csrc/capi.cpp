// extern "C" surface declared in include/eclat_hip.h.
#include <hip/hip_runtime_api.h>

#include <cstdlib>
#include <cstring>
#include <new>
#include <memory>
#include <string>

#include "../../include/eclat_hip.h"
#include "backend.hpp"
#include "normalize.hpp"
#include "static_scratch.hpp"

using namespace eh;

struct eh_device {
  HipDevice dev;
  explicit eh_device(int i) : dev(i) {}
};
struct eh_buffer {
  HipBuffer buf;
  eh_buffer(HipDevice* d, size_t n) : buf(d, n) {}
};
struct eh_program {
  HipProgram prog;
  eh_program(HipDevice* d, const std::string& t, const GenOptions& o) : prog(d, t, o) {}
};
struct eh_plan {
  ProgramPlan plan;
};
struct eh_graph {
  std::unique_ptr<HipGraph> graph;
  std::vector<eh_buffer*> held;          // the caller's buffers, one reference each
  ~eh_graph() {
    graph.reset();                       // waits for queued replays before the buffers may go
    for (eh_buffer* b : held)
      if (b->buf.release()) delete b;
  }
};
struct eh_module {
  HipDevice* dev;
  std::shared_ptr<HipKernel> kernel;
};
struct eh_event {
  HipDevice* dev;
  hipEvent_t ev;
};

namespace {

thread_local std::string g_err;

int fail(int code, const std::string& msg) {
  g_err = msg;
  return code;
}

int classify(const std::string& m) {
  if (m.rfind("AST text", 0) == 0 || m.rfind("option", 0) == 0 || m.rfind("unknown option", 0) == 0) return EH_ERR_PARSE;
  if (m.find("hiprtc") != std::string::npos) return EH_ERR_COMPILE;
  if (m.find("Buffer size mismatch") != std::string::npos) return EH_ERR_SIZE;
  if (m.find("hip error") != std::string::npos || m.find("no HIP device") != std::string::npos ||
      m.find("device index") != std::string::npos)
    return EH_ERR_DEVICE;
  if (m.find("not supported") != std::string::npos || m.find("cannot render") != std::string::npos)
    return EH_ERR_UNSUPPORTED;
  return EH_ERR_INVALID;
}

template <class F> int guard(F&& f) {
  try {
    f();
    return EH_OK;
  } catch (const Error& e) {
    return fail(classify(e.what()), e.what());
  } catch (const std::bad_alloc&) {
    return fail(EH_ERR_INVALID, "out of host memory");
  } catch (const std::exception& e) {
    return fail(EH_ERR_INVALID, e.what());
  }
}

void fill_info(const LaunchSpec& ls, eh_launch_info* out) {
  out->entry = ls.entry.c_str();
  out->source = ls.source.c_str();
  out->schedule = ls.schedule.c_str();
  for (int i = 0; i < 3; ++i) {
    out->grid[i] = ls.grid[i];
    out->block[i] = ls.block[i];
  }
  out->lds_bytes = ls.lds_bytes;
  out->n_args = static_cast<int>(ls.arg_bufs.size());
  out->n_kernels = static_cast<int>(ls.kernels.size());
  out->algo_bytes = ls.algo_bytes;
  out->flops = ls.flops;
  out->lane = ls.lane;
  out->n_waits = static_cast<int>(ls.waits.size());
  out->tune_key = ls.tune_key;
}

int buffer_entry(const ProgramPlan& p, int i, const char** name, const char** role, size_t* bytes, int* elided) {
  if (i < 0 || i >= static_cast<int>(p.buffers.size())) return fail(EH_ERR_INVALID, "buffer index out of range");
  const BufferInfo& b = p.buffers[static_cast<size_t>(i)];
  if (name) *name = b.name.c_str();
  if (role) *role = b.role.c_str();
  if (bytes) *bytes = b.shape_known ? b.bytes() : 0;
  if (elided) *elided = p.elided.count(b.name) ? 1 : 0;
  return EH_OK;
}

#define REQUIRE(cond, msg) \
  if (!(cond)) return fail(EH_ERR_INVALID, msg)

}  // namespace

extern "C" {

int eh_version(void) { return 100; }
const char* eh_last_error(void) { return g_err.c_str(); }
void eh_free(void* p) { std::free(p); }

int eh_device_count(int* count) {
  REQUIRE(count, "count is NULL");
  *count = HipDevice::count();
  return EH_OK;
}

int eh_device_open(int index, eh_device** out) {
  REQUIRE(out, "out is NULL");
  return guard([&] { *out = new eh_device(index); });
}

int eh_device_close(eh_device* dev) {
  REQUIRE(dev, "device is NULL");
  return guard([&] { delete dev; });
}

int eh_device_get_props(eh_device* dev, eh_device_props* out) {
  REQUIRE(dev && out, "device or out is NULL");
  const DeviceProfile& p = dev->dev.profile();
  std::memset(out, 0, sizeof *out);
  std::strncpy(out->name, p.name.c_str(), sizeof out->name - 1);
  std::strncpy(out->arch, p.arch.c_str(), sizeof out->arch - 1);
  out->compute_units = p.compute_units;
  out->warp_size = p.warp_size;
  out->max_work_group_size = p.max_work_group_size;
  out->local_memory_size = p.local_memory_size;
  out->global_memory_size = p.global_memory_size;
  out->clock_khz = p.clock_khz;
  out->memory_clock_khz = p.memory_clock_khz;
  out->memory_bus_bits = p.memory_bus_bits;
  out->l2_bytes = p.l2_bytes;
  return EH_OK;
}

int eh_device_sync(eh_device* dev) {
  REQUIRE(dev, "device is NULL");
  return guard([&] { dev->dev.synchronize(); });
}

int eh_device_stream(eh_device* dev, void** stream) {
  REQUIRE(dev && stream, "device or stream is NULL");
  return guard([&] { *stream = reinterpret_cast<void*>(dev->dev.stream()); });
}

int eh_device_trim(eh_device* dev, size_t* kept_bytes) {
  REQUIRE(dev, "device is NULL");
  return guard([&] {
    if (kept_bytes) *kept_bytes = dev->dev.pooled_bytes();
    dev->dev.trim();
  });
}

int eh_buffer_alloc(eh_device* dev, size_t bytes, eh_buffer** out) {
  REQUIRE(dev && out, "device or out is NULL");
  return guard([&] { *out = new eh_buffer(&dev->dev, bytes); });
}

int eh_buffer_retain(eh_buffer* buf) {
  REQUIRE(buf, "buffer is NULL");
  buf->buf.retain();
  return EH_OK;
}

int eh_buffer_release(eh_buffer* buf) {
  REQUIRE(buf, "buffer is NULL");
  return guard([&] {
    if (buf->buf.release()) delete buf;
  });
}

int eh_buffer_bytes(eh_buffer* buf, size_t* bytes) {
  REQUIRE(buf && bytes, "buffer or bytes is NULL");
  *bytes = buf->buf.byte_len();
  return EH_OK;
}

int eh_buffer_write(eh_buffer* buf, const void* src, size_t bytes) {
  REQUIRE(buf && (src || bytes == 0), "buffer or src is NULL");
  return guard([&] { buf->buf.write_from_host(src, bytes); });
}

int eh_buffer_read(eh_buffer* buf, void* dst, size_t bytes) {
  REQUIRE(buf && (dst || bytes == 0), "buffer or dst is NULL");
  return guard([&] { buf->buf.read_to_host(dst, bytes); });
}

int eh_buffer_copy(eh_buffer* dst, eh_buffer* src) {
  REQUIRE(dst && src, "buffer is NULL");
  return guard([&] { dst->buf.copy_from(src->buf); });
}

int eh_buffer_device_ptr(eh_buffer* buf, void** ptr) {
  REQUIRE(buf && ptr, "buffer or ptr is NULL");
  return guard([&] {
    buf->buf.settle();               // the caller may read through the pointer
    *ptr = buf->buf.device_ptr();
  });
}

int eh_tune_key(const char* ast_text, unsigned long long* key) {
  REQUIRE(ast_text && key, "ast_text or key is NULL");
  *key = tune_key(ast_text);
  return EH_OK;
}

int eh_render_program(const char* ast_text, const char* options, eh_plan** out) {
  REQUIRE(ast_text && out, "ast_text or out is NULL");
  return guard([&] {
    GenOptions o = options_for(ast_text, options);
    NodePtr ast = parse_ast(ast_text);
    if (ast->op == Op::Kernel) ast = make(Op::Program, {ast});
    auto* p = new eh_plan;
    try {
      p->plan = plan_program(*ast, o);
      dump_plan(p->plan);
    } catch (...) {
      delete p;
      throw;
    }
    *out = p;
  });
}

int eh_normalize_ast(const char* ast_text, char** out_text) {
  REQUIRE(ast_text && out_text, "ast_text or out_text is NULL");
  return guard([&] {
    NodePtr ast = parse_ast(ast_text);
    validate_sizes(*ast);
    std::string text;
    if (ast->op == Op::Kernel) {
      text = to_text(*normalize_kernel(ast));
    } else if (ast->op == Op::Program) {
      auto p = std::make_shared<Node>(*ast);
      for (auto& f : p->args)
        if (f->op == Op::Kernel) f = normalize_kernel(f);
      text = to_text(*p);
    } else {
      throw Error("expected a program or kernel node");
    }
    char* buf = static_cast<char*>(std::malloc(text.size() + 1));
    if (!buf) throw std::bad_alloc();
    std::memcpy(buf, text.c_str(), text.size() + 1);
    *out_text = buf;
  });
}

int eh_plan_num_launches(eh_plan* plan, int* n) {
  REQUIRE(plan && n, "plan or n is NULL");
  *n = static_cast<int>(plan->plan.launches.size());
  return EH_OK;
}

int eh_plan_launch(eh_plan* plan, int launch, eh_launch_info* out) {
  REQUIRE(plan && out, "plan or out is NULL");
  REQUIRE(launch >= 0 && launch < static_cast<int>(plan->plan.launches.size()), "launch index out of range");
  fill_info(plan->plan.launches[static_cast<size_t>(launch)], out);
  return EH_OK;
}

int eh_fit_local_size(const size_t global[3], const size_t preferred[3], size_t max_work_group, size_t local[3]) {
  REQUIRE(global && preferred && local, "global, preferred or local is NULL");
  REQUIRE(max_work_group >= 1, "max_work_group must be at least 1");
  uint64_t g[3], p[3], l[3];
  for (int i = 0; i < 3; ++i) {
    REQUIRE(preferred[i] >= 1, "a preferred local size must be at least 1");
    REQUIRE(global[i] <= (uint64_t{1} << 40) && preferred[i] <= (uint64_t{1} << 40), "size out of range");
    g[i] = global[i];
    p[i] = preferred[i];
  }
  eh::fit_local_size(g, p, max_work_group, l);
  for (int i = 0; i < 3; ++i) local[i] = static_cast<size_t>(l[i]);
  return EH_OK;
}

int eh_plan_launch_arg(eh_plan* plan, int launch, int arg, const char** buffer_name) {
  REQUIRE(plan && buffer_name, "plan or buffer_name is NULL");
  REQUIRE(launch >= 0 && launch < static_cast<int>(plan->plan.launches.size()), "launch index out of range");
  const auto& a = plan->plan.launches[static_cast<size_t>(launch)].arg_bufs;
  REQUIRE(arg >= 0 && arg < static_cast<int>(a.size()), "argument index out of range");
  *buffer_name = a[static_cast<size_t>(arg)].c_str();
  return EH_OK;
}

int eh_plan_launch_arg_written(eh_plan* plan, int launch, int arg, int* written) {
  REQUIRE(plan && written, "plan or written is NULL");
  REQUIRE(launch >= 0 && launch < static_cast<int>(plan->plan.launches.size()), "launch index out of range");
  const auto& a = plan->plan.launches[static_cast<size_t>(launch)].arg_written;
  REQUIRE(arg >= 0 && arg < static_cast<int>(a.size()), "argument index out of range");
  const auto& f = plan->plan.launches[static_cast<size_t>(launch)].arg_full_bytes;
  const bool whole = static_cast<size_t>(arg) < f.size() && f[static_cast<size_t>(arg)] != 0;
  *written = a[static_cast<size_t>(arg)] ? (whole ? 2 : 1) : 0;
  return EH_OK;
}

int eh_plan_launch_wait(eh_plan* plan, int launch, int i, int* waited_launch) {
  REQUIRE(plan && waited_launch, "plan or waited_launch is NULL");
  REQUIRE(launch >= 0 && launch < static_cast<int>(plan->plan.launches.size()), "launch index out of range");
  const auto& w = plan->plan.launches[static_cast<size_t>(launch)].waits;
  REQUIRE(i >= 0 && i < static_cast<int>(w.size()), "wait index out of range");
  *waited_launch = w[static_cast<size_t>(i)];
  return EH_OK;
}

int eh_plan_launch_kernel(eh_plan* plan, int launch, int k, const char** kernel_name) {
  REQUIRE(plan && kernel_name, "plan or kernel_name is NULL");
  REQUIRE(launch >= 0 && launch < static_cast<int>(plan->plan.launches.size()), "launch index out of range");
  const auto& a = plan->plan.launches[static_cast<size_t>(launch)].kernels;
  REQUIRE(k >= 0 && k < static_cast<int>(a.size()), "kernel index out of range");
  *kernel_name = a[static_cast<size_t>(k)].c_str();
  return EH_OK;
}

int eh_plan_num_buffers(eh_plan* plan, int* n) {
  REQUIRE(plan && n, "plan or n is NULL");
  *n = static_cast<int>(plan->plan.buffers.size());
  return EH_OK;
}

int eh_plan_buffer(eh_plan* plan, int i, const char** name, const char** role, size_t* bytes, int* elided) {
  REQUIRE(plan, "plan is NULL");
  return buffer_entry(plan->plan, i, name, role, bytes, elided);
}

int eh_plan_release(eh_plan* plan) {
  REQUIRE(plan, "plan is NULL");
  delete plan;
  return EH_OK;
}

int eh_compile_source(const char* source, const char* arch, void** blob, size_t* len) {
  REQUIRE(source && blob && len, "source, blob or len is NULL");
  return guard([&] {
    Binary b = HipCompiler::compile(source, arch ? arch : "gfx950");
    void* p = std::malloc(b.code.size() ? b.code.size() : 1);
    if (!p) throw std::bad_alloc();
    std::memcpy(p, b.code.data(), b.code.size());
    *blob = p;
    *len = b.code.size();
  });
}

int eh_program_compile(eh_device* dev, const char* ast_text, const char* options, eh_program** out) {
  REQUIRE(dev && ast_text && out, "device, ast_text or out is NULL");
  return guard([&] {
    GenOptions o = options_for(ast_text, options);
    *out = new eh_program(&dev->dev, ast_text, o);
  });
}

int eh_program_release(eh_program* prog) {
  REQUIRE(prog, "program is NULL");
  return guard([&] { delete prog; });
}

int eh_program_num_buffers(eh_program* prog, int* n) {
  REQUIRE(prog && n, "program or n is NULL");
  *n = static_cast<int>(prog->prog.plan().buffers.size());
  return EH_OK;
}

int eh_program_buffer(eh_program* prog, int i, const char** name, const char** role, size_t* bytes, int* elided) {
  REQUIRE(prog, "program is NULL");
  return buffer_entry(prog->prog.plan(), i, name, role, bytes, elided);
}

int eh_program_num_launches(eh_program* prog, int* n) {
  REQUIRE(prog && n, "program or n is NULL");
  *n = static_cast<int>(prog->prog.plan().launches.size());
  return EH_OK;
}

int eh_program_launch(eh_program* prog, int launch, eh_launch_info* out) {
  REQUIRE(prog && out, "program or out is NULL");
  const auto& ls = prog->prog.plan().launches;
  REQUIRE(launch >= 0 && launch < static_cast<int>(ls.size()), "launch index out of range");
  fill_info(ls[static_cast<size_t>(launch)], out);
  return EH_OK;
}

int eh_program_execute(eh_program* prog, eh_buffer* const* bufs, int n_bufs, int sync) {
  REQUIRE(prog && (bufs || n_bufs == 0) && n_bufs >= 0, "program or bufs is NULL");
  return guard([&] {
    std::vector<HipBuffer*> v(static_cast<size_t>(n_bufs), nullptr);
    for (int i = 0; i < n_bufs; ++i) v[static_cast<size_t>(i)] = bufs[i] ? &bufs[i]->buf : nullptr;
    prog->prog.execute(v.data(), v.size(), sync != 0);
  });
}

int eh_program_execute_static(eh_program* prog, eh_buffer* const* bufs, int n_bufs, int sync) {
  REQUIRE(prog && (bufs || n_bufs == 0) && n_bufs >= 0, "program or bufs is NULL");
  return guard([&] {
    std::vector<HipBuffer*> v(static_cast<size_t>(n_bufs), nullptr);
    for (int i = 0; i < n_bufs; ++i) v[static_cast<size_t>(i)] = bufs[i] ? &bufs[i]->buf : nullptr;
    prog->prog.execute_static(v.data(), v.size(), sync != 0);
  });
}

int eh_program_record(eh_program* prog, eh_buffer* const* bufs, int n_bufs, eh_graph** out) {
  REQUIRE(prog && out && (bufs || n_bufs == 0) && n_bufs >= 0, "program, bufs or out is NULL");
  return guard([&] {
    std::vector<HipBuffer*> v(static_cast<size_t>(n_bufs), nullptr);
    for (int i = 0; i < n_bufs; ++i) v[static_cast<size_t>(i)] = bufs[i] ? &bufs[i]->buf : nullptr;
    std::unique_ptr<eh_graph> g(new eh_graph());
    g->graph.reset(new HipGraph(&prog->prog, v.data(), v.size()));
    for (int i = 0; i < n_bufs; ++i)
      if (bufs[i]) {
        bufs[i]->buf.retain();
        g->held.push_back(bufs[i]);
      }
    *out = g.release();
  });
}

int eh_graph_replay(eh_graph* graph, int sync) {
  REQUIRE(graph, "graph is NULL");
  return guard([&] { graph->graph->replay(sync != 0); });
}

int eh_graph_release(eh_graph* graph) {
  REQUIRE(graph, "graph is NULL");
  return guard([&] { delete graph; });
}

int eh_program_execute_positional(eh_program* prog, eh_buffer* const* inputs, int n_inputs, eh_buffer* const* outputs,
                                  int n_outputs, int sync) {
  REQUIRE(prog && n_inputs >= 0 && n_outputs >= 0, "bad arguments");
  REQUIRE((inputs || n_inputs == 0) && (outputs || n_outputs == 0), "inputs or outputs is NULL");
  return guard([&] {
    std::vector<HipBuffer*> in, out;
    for (int i = 0; i < n_inputs; ++i) {
      if (!inputs[i]) throw Error("input buffer " + std::to_string(i) + " is NULL");
      in.push_back(&inputs[i]->buf);
    }
    for (int i = 0; i < n_outputs; ++i) {
      if (!outputs[i]) throw Error("output buffer " + std::to_string(i) + " is NULL");
      out.push_back(&outputs[i]->buf);
    }
    prog->prog.execute_positional(in.data(), in.size(), out.data(), out.size(), sync != 0);
  });
}

int eh_program_binary(eh_program* prog, int launch, const void** blob, size_t* len) {
  REQUIRE(prog && blob && len, "program, blob or len is NULL");
  REQUIRE(launch >= 0 && launch < static_cast<int>(prog->prog.plan().launches.size()), "launch index out of range");
  const auto& b = prog->prog.kernel(static_cast<size_t>(launch)).binary();
  *blob = b.data();
  *len = b.size();
  return EH_OK;
}

int eh_module_load(eh_device* dev, const void* blob, size_t len, const char* entry, eh_module** out) {
  REQUIRE(dev && blob && len > 0 && entry && out, "device, blob, entry or out is NULL");
  return guard([&] {
    Binary b;
    b.code.assign(static_cast<const char*>(blob), static_cast<const char*>(blob) + len);
    if (len < 4 || std::memcmp(b.code.data(), "\x7f" "ELF", 4) != 0)
      throw Error("code object does not start with an ELF header");
    *out = new eh_module{&dev->dev, dev->dev.load(b, entry)};
  });
}

int eh_module_launch(eh_module* mod, const unsigned grid[3], const unsigned block[3], unsigned lds_bytes,
                     eh_buffer* const* args, int n_args, int sync) {
  REQUIRE(mod && grid && block && n_args >= 0 && (args || n_args == 0), "bad arguments");
  return guard([&] {
    unsigned long long threads = 1ull * block[0] * block[1] * block[2];
    if (threads == 0 || threads > 1024 || grid[0] == 0 || grid[1] == 0 || grid[2] == 0)
      throw Error("dispatch size out of range (block of " + std::to_string(threads) + " work-items)");
    if (lds_bytes > 160 * 1024) throw Error("dynamic LDS request exceeds 160 KiB");
    std::vector<void*> ptrs;
    for (int i = 0; i < n_args; ++i) {
      if (!args[i]) throw Error("argument " + std::to_string(i) + " is NULL");
      if (args[i]->buf.device() != mod->dev) throw Error("argument " + std::to_string(i) + " lives on another device");
    }
    auto lk = mod->dev->stream_lock();
    for (int i = 0; i < n_args; ++i) {
      args[i]->buf.settle();         // nothing is known about what the code object reads
      ptrs.push_back(args[i]->buf.device_ptr());
    }
    mod->dev->make_current();
    mod->kernel->launch(grid, block, lds_bytes, ptrs);
    if (sync) mod->dev->synchronize();
  });
}

int eh_module_release(eh_module* mod) {
  REQUIRE(mod, "module is NULL");
  return guard([&] { delete mod; });
}

int eh_event_create(eh_device* dev, eh_event** out) {
  REQUIRE(dev && out, "device or out is NULL");
  return guard([&] {
    dev->dev.make_current();
    hipEvent_t e;
    hipError_t r = hipEventCreate(&e);
    if (r != hipSuccess) throw Error(std::string("hipEventCreate: ") + hipGetErrorString(r) + " (hip error)");
    *out = new eh_event{&dev->dev, e};
  });
}

int eh_event_record(eh_event* ev) {
  REQUIRE(ev, "event is NULL");
  return guard([&] {
    auto lk = ev->dev->stream_lock();
    ev->dev->make_current();
    hipError_t r = hipEventRecord(ev->ev, ev->dev->stream());
    if (r != hipSuccess) throw Error(std::string("hipEventRecord: ") + hipGetErrorString(r) + " (hip error)");
  });
}

int eh_event_sync(eh_event* ev) {
  REQUIRE(ev, "event is NULL");
  return guard([&] {
    hipError_t r = hipEventSynchronize(ev->ev);
    if (r != hipSuccess) throw Error(std::string("hipEventSynchronize: ") + hipGetErrorString(r) + " (hip error)");
  });
}

int eh_event_elapsed_ms(eh_event* start, eh_event* stop, float* ms) {
  REQUIRE(start && stop && ms, "event or ms is NULL");
  return guard([&] {
    hipError_t r = hipEventElapsedTime(ms, start->ev, stop->ev);
    if (r != hipSuccess) throw Error(std::string("hipEventElapsedTime: ") + hipGetErrorString(r) + " (hip error)");
  });
}

int eh_event_release(eh_event* ev) {
  REQUIRE(ev, "event is NULL");
  (void)hipEventDestroy(ev->ev);
  delete ev;
  return EH_OK;
}

}  // extern "C"
