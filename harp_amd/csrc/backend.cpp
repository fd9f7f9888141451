#include "backend.hpp"
#include "static_scratch.hpp"

#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <list>
#include <mutex>
#include <optional>
#include <sstream>
#include <thread>
#include <unordered_map>

namespace eh {

namespace {

void check(hipError_t e, const char* what) {
  if (e != hipSuccess)
    throw Error(std::string(what) + ": " + hipGetErrorString(e) + " (hip error " + std::to_string(static_cast<int>(e)) + ")");
}

uint64_t fnv1a(const std::string& s, uint64_t h) {
  for (unsigned char c : s) {
    h ^= c;
    h *= 1099511628211ull;
  }
  return h;
}

std::string hash_hex(const std::string& s) {
  char buf[40];
  snprintf(buf, sizeof buf, "%016llx%016llx", static_cast<unsigned long long>(fnv1a(s, 14695981039346656037ull)),
           static_cast<unsigned long long>(fnv1a(s, 0x9e3779b97f4a7c15ull)));
  return buf;
}

void mkdirs(const std::string& path) {
  std::string cur;
  for (size_t i = 0; i < path.size(); ++i) {
    cur += path[i];
    if (path[i] == '/' || i + 1 == path.size()) ::mkdir(cur.c_str(), 0755);
  }
}

// In-memory code objects, least recently used first out; the capacity is the reference's
// kernel-cache capacity (src/backend/cache/store.rs:116-168).
class BinaryCache {
 public:
  static constexpr size_t kCapacity = 1024;
  std::shared_ptr<Binary> find(const std::string& key) {
    std::lock_guard<std::mutex> lk(mu_);
    auto it = index_.find(key);
    if (it == index_.end()) return nullptr;
    order_.splice(order_.begin(), order_, it->second);      // now the most recently used
    return it->second->second;
  }
  void insert(const std::string& key, std::shared_ptr<Binary> bin) {
    std::lock_guard<std::mutex> lk(mu_);
    auto it = index_.find(key);
    if (it != index_.end()) {
      it->second->second = std::move(bin);
      order_.splice(order_.begin(), order_, it->second);
      return;
    }
    order_.emplace_front(key, std::move(bin));
    index_[key] = order_.begin();
    while (order_.size() > kCapacity) {
      index_.erase(order_.back().first);
      order_.pop_back();
    }
  }

 private:
  std::mutex mu_;
  std::list<std::pair<std::string, std::shared_ptr<Binary>>> order_;
  std::unordered_map<std::string, std::list<std::pair<std::string, std::shared_ptr<Binary>>>::iterator> index_;
};
BinaryCache g_bin_cache;

}  // namespace

// ---------------------------------------------------------------------------------------------
// HipCompiler
// ---------------------------------------------------------------------------------------------

std::vector<std::string> HipCompiler::options(const std::string& arch) {
  // fp-contract off: `a*b` followed by `+c` in separate graph nodes must round twice, as the C
  // backend's output does.  The target feature keeps packed-fp32 instructions out of the code.
  return {"--offload-arch=" + arch, "-O3", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang",
          "-packed-fp32-ops"};
}

bool HipCompiler::disk_cache_enabled() { return std::getenv("HARP_NO_DISK_CACHE") == nullptr; }

std::string HipCompiler::cache_dir() {
  std::string base;
  if (const char* d = std::getenv("HARP_CACHE_DIR")) base = d;
  else if (const char* h = std::getenv("HOME")) base = std::string(h) + "/.cache/harp";
  else base = "/tmp/harp-cache";
  // not kernels/<DeviceKind>: that is where the reference keeps its own disk cache, with a
  // different side-file schema (src/backend/cache/disk.rs:63-115)
  return base + "/code_objects/gfx950";
}

Binary HipCompiler::compile(const std::string& source, const std::string& arch, bool use_disk_cache, bool refresh) {
  std::vector<std::string> opts = options(arch);
  int maj = 0, min = 0;
  hiprtcVersion(&maj, &min);
  std::string key_text = source;
  for (const auto& o : opts) key_text += "\n" + o;
  key_text += "\nhiprtc " + std::to_string(maj) + "." + std::to_string(min);
  const std::string key = hash_hex(key_text);
  if (!refresh)
    if (auto hit = g_bin_cache.find(key)) return *hit;
  const bool disk = use_disk_cache && disk_cache_enabled();
  const std::string path = cache_dir() + "/" + key + ".bin";
  Binary out;
  const std::string meta_path = cache_dir() + "/" + key + ".json";
  if (disk && !refresh) {
    // a cached code object counts only if its side file vouches for it: same length, same hash
    // (a truncated or half-written file must never reach the module loader)
    std::ifstream f(path, std::ios::binary);
    std::ifstream m(meta_path);
    if (f && m) {
      std::string meta((std::istreambuf_iterator<char>(m)), std::istreambuf_iterator<char>());
      out.code.assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
      const std::string want = "\"fnv1a\": \"" + hash_hex(std::string(out.code.begin(), out.code.end())) + "\"";
      const std::string len = "\"bytes\": " + std::to_string(out.code.size());
      out.from_cache = !out.code.empty() && meta.find(want) != std::string::npos && meta.find(len) != std::string::npos;
      if (!out.from_cache) out.code.clear();
    }
  }
  if (!out.from_cache) {
    hiprtcProgram prog;
    if (hiprtcCreateProgram(&prog, source.c_str(), "eclat_kernel.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS)
      throw Error("hiprtcCreateProgram failed");
    std::vector<const char*> copts;
    for (const auto& o : opts) copts.push_back(o.c_str());
    hiprtcResult r = hiprtcCompileProgram(prog, static_cast<int>(copts.size()), copts.data());
    size_t ls = 0;
    hiprtcGetProgramLogSize(prog, &ls);
    if (ls > 1) {
      out.log.resize(ls);
      hiprtcGetProgramLog(prog, &out.log[0]);
    }
    if (r != HIPRTC_SUCCESS) {
      hiprtcDestroyProgram(&prog);
      throw Error(std::string("hiprtc compilation failed: ") + hiprtcGetErrorString(r) + "\n" + out.log);
    }
    size_t cs = 0;
    hiprtcGetCodeSize(prog, &cs);
    out.code.resize(cs);
    hiprtcGetCode(prog, out.code.data());
    hiprtcDestroyProgram(&prog);
    if (disk) {
      mkdirs(cache_dir());
      // private name, then an atomic rename: concurrent writers of one key never share a file
      const std::string tmp = path + ".tmp" + std::to_string(static_cast<long>(::getpid())) + "_" +
                              std::to_string(std::hash<std::thread::id>{}(std::this_thread::get_id()) & 0xffffff);
      std::ofstream f(tmp, std::ios::binary);
      if (f) {
        f.write(out.code.data(), static_cast<std::streamsize>(out.code.size()));
        f.close();
        std::rename(tmp.c_str(), path.c_str());
        std::ofstream meta(meta_path);
        meta << "{\"arch\": \"" << arch << "\", \"hiprtc\": \"" << maj << "." << min << "\", \"bytes\": "
             << out.code.size() << ", \"fnv1a\": \"" << hash_hex(std::string(out.code.begin(), out.code.end()))
             << "\"}\n";
      }
    }
  }
  g_bin_cache.insert(key, std::make_shared<Binary>(out));
  return out;
}

// ---------------------------------------------------------------------------------------------
// HipDevice / HipBuffer / HipKernel
// ---------------------------------------------------------------------------------------------

int HipDevice::count() {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

HipDevice::HipDevice(int index) : index_(index) {
  int n = count();
  if (n == 0) throw Error("no HIP device is present (hipGetDeviceCount found none)");
  if (index < 0 || index >= n)
    throw Error("device index " + std::to_string(index) + " out of range (" + std::to_string(n) + " device(s))");
  check(hipSetDevice(index), "hipSetDevice");
  hipDeviceProp_t p;
  check(hipGetDeviceProperties(&p, index), "hipGetDeviceProperties");
  profile_.name = p.name;
  profile_.arch = p.gcnArchName;
  profile_.arch = profile_.arch.substr(0, profile_.arch.find(':'));
  profile_.compute_units = p.multiProcessorCount;
  profile_.warp_size = p.warpSize;
  profile_.max_work_group_size = p.maxThreadsPerBlock;
  profile_.local_memory_size = p.maxSharedMemoryPerMultiProcessor ? p.maxSharedMemoryPerMultiProcessor : p.sharedMemPerBlock;
  profile_.global_memory_size = p.totalGlobalMem;
  profile_.clock_khz = p.clockRate;
  profile_.memory_clock_khz = p.memoryClockRate;
  profile_.memory_bus_bits = p.memoryBusWidth;
  profile_.l2_bytes = p.l2CacheSize;
  check(hipStreamCreate(&stream_), "hipStreamCreate");
  pool_limit_ = std::getenv("ECLAT_HIP_NO_POOL") ? 0 : profile_.global_memory_size / 4;
  // resolved here, with this device current, so that the entry point which must not allocate
  // never triggers the load of the library's code object itself
  try {
    static_scratch_ = static_scratch_ptr(index_);
  } catch (const Error& e) {
    static_scratch_error_ = e.what();
  }
}

void* HipDevice::static_scratch() const {
  if (!static_scratch_) throw Error("the static scratch block is not available: " + static_scratch_error_);
  return static_scratch_;
}

HipDevice::~HipDevice() {
  if (stream_) {
    (void)hipSetDevice(index_);
    (void)hipStreamSynchronize(stream_);
    for (hipStream_t st : side_streams_) {
      (void)hipStreamSynchronize(st);
      (void)hipStreamDestroy(st);
    }
    for (auto& kv : pool_) (void)hipFree(kv.second);
    (void)hipStreamDestroy(stream_);
  }
}

hipStream_t HipDevice::lane_stream(int lane) {
  if (lane <= 0) return stream_;
  auto lk = stream_lock();
  make_current();
  while (side_streams_.size() < static_cast<size_t>(lane)) {
    hipStream_t st = nullptr;
    check(hipStreamCreateWithFlags(&st, hipStreamNonBlocking), "hipStreamCreateWithFlags");
    side_streams_.push_back(st);
  }
  return side_streams_[static_cast<size_t>(lane) - 1];
}

void* HipDevice::allocate(size_t bytes) {
  {
    std::lock_guard<std::mutex> lk(pool_mu_);
    auto it = pool_.find(bytes);
    if (it != pool_.end()) {
      void* p = it->second;
      pool_.erase(it);
      pooled_bytes_ -= bytes;
      return p;
    }
  }
  void* p = nullptr;
  hipError_t e = hipMalloc(&p, bytes);
  if (e == hipErrorOutOfMemory) {      // give the kept blocks back and try once more
    (void)hipGetLastError();
    trim();
    e = hipMalloc(&p, bytes);
  }
  check(e, "hipMalloc");
  return p;
}

void HipDevice::release(void* ptr, size_t bytes) {
  {
    std::lock_guard<std::mutex> lk(pool_mu_);
    if (pooled_bytes_ + bytes <= pool_limit_) {
      pool_.emplace(bytes, ptr);
      pooled_bytes_ += bytes;
      return;
    }
  }
  auto lk = stream_lock();
  (void)hipStreamSynchronize(stream_);
  (void)hipFree(ptr);
}

void HipDevice::trim() {
  std::multimap<size_t, void*> blocks;
  {
    std::lock_guard<std::mutex> lk(pool_mu_);
    blocks.swap(pool_);
    pooled_bytes_ = 0;
  }
  if (blocks.empty()) return;
  auto lk = stream_lock();
  (void)hipStreamSynchronize(stream_);
  for (auto& kv : blocks) (void)hipFree(kv.second);
}

void HipDevice::make_current() const { check(hipSetDevice(index_), "hipSetDevice"); }

void HipDevice::synchronize() const {
  auto lk = stream_lock();
  make_current();
  check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
}

std::shared_ptr<HipKernel> HipDevice::load(const Binary& bin, const std::string& entry) {
  return std::make_shared<HipKernel>(this, bin, entry);
}

HipBuffer::HipBuffer(HipDevice* dev, size_t bytes) : dev_(dev), bytes_(bytes) {
  auto lk = dev_->stream_lock();
  dev_->make_current();
  if (bytes_ == 0) return;
  ptr_ = dev_->allocate(bytes_);
  zero_pending_ = true;
}

void HipBuffer::settle() {
  auto lk = dev_->stream_lock();
  if (!zero_pending_) return;
  dev_->make_current();
  // a fill recorded into somebody's graph would run again on every replay, over whatever the
  // buffer holds by then
  hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(dev_->stream(), &cs) == hipSuccess && cs != hipStreamCaptureStatusNone)
    throw Error("a buffer that nothing has written yet is read under stream capture: write it, read it or take its "
                "address once before the capture starts");
  check(hipMemsetAsync(ptr_, 0, bytes_, dev_->stream()), "hipMemsetAsync");
  zero_pending_ = false;
}

HipBuffer::~HipBuffer() {
  if (ptr_) {
    (void)hipSetDevice(dev_->index());
    dev_->release(ptr_, bytes_);
  }
}

void HipBuffer::write_from_host(const void* src, size_t bytes) {
  if (bytes != bytes_)
    throw Error("Buffer size mismatch: expected " + std::to_string(bytes_) + ", got " + std::to_string(bytes));
  if (!bytes_) return;
  auto lk = dev_->stream_lock();
  dev_->make_current();
  check(hipMemcpyAsync(ptr_, src, bytes_, hipMemcpyHostToDevice, dev_->stream()), "hipMemcpyAsync(H2D)");
  check(hipStreamSynchronize(dev_->stream()), "hipStreamSynchronize");
  zero_pending_ = false;
}

void HipBuffer::read_to_host(void* dst, size_t bytes) const {
  if (bytes != bytes_)
    throw Error("Buffer size mismatch: expected " + std::to_string(bytes_) + ", got " + std::to_string(bytes));
  if (!bytes_) return;
  auto lk = dev_->stream_lock();
  if (zero_pending_) {                         // never written: zeros, without touching the device
    std::memset(dst, 0, bytes_);
    return;
  }
  dev_->make_current();
  check(hipMemcpyAsync(dst, ptr_, bytes_, hipMemcpyDeviceToHost, dev_->stream()), "hipMemcpyAsync(D2H)");
  check(hipStreamSynchronize(dev_->stream()), "hipStreamSynchronize");
}

void HipBuffer::copy_from(const HipBuffer& src) {
  if (src.bytes_ != bytes_)
    throw Error("Buffer size mismatch: expected " + std::to_string(bytes_) + ", got " + std::to_string(src.bytes_));
  if (!bytes_) return;
  auto lk = dev_->stream_lock();
  dev_->make_current();
  if (src.zero_pending_) {                     // a copy of zeros
    check(hipMemsetAsync(ptr_, 0, bytes_, dev_->stream()), "hipMemsetAsync");
  } else {
    check(hipMemcpyAsync(ptr_, src.ptr_, bytes_, hipMemcpyDeviceToDevice, dev_->stream()), "hipMemcpyAsync(D2D)");
  }
  zero_pending_ = false;
}

HipKernel::HipKernel(HipDevice* dev, const Binary& bin, const std::string& entry)
    : dev_(dev), binary_(bin.code), entry_(entry) {
  dev_->make_current();
  check(hipModuleLoadData(&module_, binary_.data()), "hipModuleLoadData");
  hipError_t e = hipModuleGetFunction(&fn_, module_, entry.c_str());
  if (e != hipSuccess) {
    (void)hipModuleUnload(module_);
    module_ = nullptr;
    throw Error("entry point '" + entry + "' not found in the code object: " + hipGetErrorString(e));
  }
}

HipKernel::~HipKernel() {
  if (module_) {
    auto lk = dev_->stream_lock();
    (void)hipSetDevice(dev_->index());
    (void)hipStreamSynchronize(dev_->stream());
    (void)hipModuleUnload(module_);
  }
}

void HipKernel::launch(const unsigned grid[3], const unsigned block[3], unsigned lds_bytes,
                       const std::vector<void*>& device_ptrs, hipStream_t stream) const {
  auto lk = dev_->stream_lock();
  std::vector<void*> vals = device_ptrs;
  std::vector<void*> params(vals.size());
  for (size_t i = 0; i < vals.size(); ++i) params[i] = &vals[i];
  check(hipModuleLaunchKernel(fn_, grid[0], grid[1], grid[2], block[0], block[1], block[2], lds_bytes,
                              stream ? stream : dev_->stream(), params.data(), nullptr),
        ("launch of " + entry_).c_str());
}

// ---------------------------------------------------------------------------------------------
// HipProgram
// ---------------------------------------------------------------------------------------------

unsigned long long tune_key(const char* ast_text) {
  // of the canonical text, so that spacing and the like do not matter; text that does not parse is hashed as it is
  std::string text = ast_text ? ast_text : "";
  try {
    text = to_text(*parse_ast(text));
  } catch (const Error&) {
  }
  return fnv1a(text);
}

GenOptions options_for(const char* ast_text, const char* options) {
  const char* path = std::getenv("ECLAT_HIP_TUNE");
  if (!path || !*path || !ast_text) return parse_options(options);
  std::ifstream f(path);
  if (!f) {
    static std::once_flag warned;
    std::call_once(warned, [&] { std::fprintf(stderr, "eclat backend-hip: cannot read the tuned-options file '%s' (ECLAT_HIP_TUNE); defaults are used\n", path); });
    return parse_options(options);
  }
  char key[17];
  std::snprintf(key, sizeof key, "%016llx", tune_key(ast_text));
  std::string line, tuned;
  std::map<std::string, std::string> others;        // lines under other keys: a launch's, if this program has such a launch
  while (std::getline(f, line)) {
    const size_t hash = line.find('#');
    if (hash != std::string::npos) line.resize(hash);
    std::istringstream ls(line);
    std::string k, v;
    if (!(ls >> k >> v)) continue;
    if (k == key) tuned = v;                          // the last entry for a key counts
    else if (k.size() == 16) others[k] = v;
  }
  // a launch's options as "@<key>:<name>=<value>" items, the program's own in front, the caller's last
  std::string all = tuned;
  for (const auto& kv : others) {
    std::stringstream ss(kv.second);
    std::string item;
    while (std::getline(ss, item, ','))
      if (!item.empty()) all += (all.empty() ? "" : ",") + ("@" + kv.first + ":" + item);
  }
  if (options && *options) all += (all.empty() ? "" : ",") + std::string(options);
  return parse_options(all.c_str());
}

void dump_plan(const ProgramPlan& plan) {
  const char* dir = std::getenv("ECLAT_HIP_DUMP");
  if (!dir || !*dir) return;
  mkdirs(dir);
  for (const auto& ls : plan.launches) {
    const std::string base = std::string(dir) + "/" + ls.entry;
    std::ofstream(base + ".hip") << ls.source;
    std::ofstream t(base + ".txt");
    t << "entry: " << ls.entry << "\nschedule: " << ls.schedule << "\ngrid: " << ls.grid[0] << " " << ls.grid[1] << " "
      << ls.grid[2] << "\nblock: " << ls.block[0] << " " << ls.block[1] << " " << ls.block[2]
      << "\nlds_bytes: " << ls.lds_bytes << "\nalgorithmic_bytes: " << ls.algo_bytes << "\nflops: " << ls.flops << "\nbuffers:";
    for (const auto& b : ls.arg_bufs) t << " " << b;
    t << "\nkernels:";
    for (const auto& k : ls.kernels) t << " " << k;
    t << "\n";
  }
}

HipProgram::HipProgram(HipDevice* dev, const std::string& ast_text, const GenOptions& opt) : dev_(dev) {
  NodePtr ast = parse_ast(ast_text);
  if (ast->op == Op::Kernel) ast = make(Op::Program, {ast});
  GenOptions o = opt;
  if (dev_->profile().arch.rfind("gfx", 0) == 0) o.arch = dev_->profile().arch;
  plan_ = plan_program(*ast, o);
  dump_plan(plan_);
  for (size_t i = 0; i < plan_.buffers.size(); ++i) index_[plan_.buffers[i].name] = i;
  temps_.assign(plan_.buffers.size(), nullptr);
  first_full_.assign(plan_.buffers.size(), 0);
  std::vector<char> touched(plan_.buffers.size(), 0);
  for (const auto& ls : plan_.launches) {
    for (const auto& a : ls.arg_bufs)
      if (!index_.count(a)) throw Error("launch '" + ls.entry + "' binds unknown buffer '" + a + "'");
    // (a buffer bound to two parameters of its first launch may be read there: no shortcut)
    for (size_t a = 0; a < ls.arg_bufs.size(); ++a) {
      const size_t i = index_.at(ls.arg_bufs[a]);
      const bool whole = a < ls.arg_written.size() && ls.arg_written[a] && a < ls.arg_full_bytes.size() &&
                         std::count(ls.arg_bufs.begin(), ls.arg_bufs.end(), ls.arg_bufs[a]) == 1;
      if (!touched[i] && whole) first_full_[i] = ls.arg_full_bytes[a];
    }
    for (const auto& a : ls.arg_bufs) touched[index_.at(a)] = 1;
    Binary bin = HipCompiler::compile(ls.source, o.arch);
    try {
      kernels_.push_back(dev_->load(bin, ls.entry));
    } catch (...) {
      // a cached code object the loader rejects: compile afresh, replace it, try once more
      if (!bin.from_cache) throw;
      bin = HipCompiler::compile(ls.source, o.arch, true, true);
      kernels_.push_back(dev_->load(bin, ls.entry));
    }
  }
}

HipProgram::~HipProgram() {
  // every execute joined its lanes back into the device's stream, which the temps' release waits
  // for; an event may be destroyed while work queued behind it is still pending
  for (hipEvent_t e : events_)
    if (e) (void)hipEventDestroy(e);
  for (hipEvent_t e : join_)
    if (e) (void)hipEventDestroy(e);
  if (fork_) (void)hipEventDestroy(fork_);
  for (HipBuffer* b : temps_)
    if (b && b->release()) delete b;
}

std::vector<HipBuffer*> HipProgram::bind(HipBuffer* const* bufs, size_t n, std::vector<HipBuffer*>* cancelled) {
  // the caller's table comes first; scratch temps the plan appended may be left out
  const size_t total = plan_.buffers.size();
  bool enough = n <= total;
  for (size_t i = n; enough && i < total; ++i) enough = plan_.buffers[i].role == "temp";
  if (!enough)
    throw Error("program binds " + std::to_string(total) + " buffers, " + std::to_string(n) + " given");
  dev_->make_current();
  std::vector<HipBuffer*> bound(total, nullptr);
  for (size_t i = 0; i < total; ++i) {
    const BufferInfo& bi = plan_.buffers[i];
    if (plan_.elided.count(bi.name)) continue;
    HipBuffer* b = i < n ? bufs[i] : nullptr;
    if (!b) {
      if (bi.role != "temp")
        throw Error("MissingInput: buffer '" + bi.name + "' (" + bi.role + ") was not provided");
      if (!temps_[i]) temps_[i] = new HipBuffer(dev_, bi.bytes());
      b = temps_[i];
    }
    if (b->device() != dev_) throw Error("buffer '" + bi.name + "' lives on another device");
    if (bi.shape_known) {
      if (b->byte_len() < bi.bytes())
        throw Error("Buffer size mismatch: '" + bi.name + "' needs " + std::to_string(bi.bytes()) + " bytes, has " +
                    std::to_string(b->byte_len()));
    }
    bound[i] = b;
  }
  {
    std::vector<Span> spans(total);
    for (size_t i = 0; i < total; ++i)
      if (bound[i]) spans[i] = {bound[i]->device_ptr(), bound[i]->byte_len(), true};
    refuse_aliases(spans);
  }
  resolve_fills(bound, cancelled);
  return bound;
}

// Zero fills still owed to the buffers of a table: cancelled where the program overwrites the
// whole buffer before it reads it (the caller can take the debt back), queued now otherwise.
void HipProgram::resolve_fills(const std::vector<HipBuffer*>& bound, std::vector<HipBuffer*>* cancelled) {
  for (size_t i = 0; i < bound.size(); ++i) {
    HipBuffer* b = bound[i];
    if (!b || !b->zero_pending()) continue;
    if (cancelled && first_full_[i] != 0 && first_full_[i] == b->byte_len() &&
        std::count(bound.begin(), bound.end(), b) == 1) {
      b->set_zero_pending(false);
      cancelled->push_back(b);
    } else {
      b->settle();
    }
  }
}

// The planner reorders, merges and (with lanes) overlaps launches by the dependences it reads off
// the buffer names, so two table entries must never be the same memory when a launch writes either
// of them: an in-place update (one buffer bound as a parameter and as its updated value) would race
// silently.  Refused here, on the host.
void HipProgram::refuse_aliases(const std::vector<Span>& bound) const {
  if (written_.empty()) {
    written_.assign(plan_.buffers.size(), 0);
    for (const auto& ls : plan_.launches)
      for (size_t a = 0; a < ls.arg_bufs.size(); ++a)
        if (a < ls.arg_written.size() && ls.arg_written[a]) written_[index_.at(ls.arg_bufs[a])] = 1;
  }
  struct Range { const char* lo; const char* hi; size_t i; };
  std::vector<Range> r;
  for (size_t i = 0; i < bound.size(); ++i)
    if (bound[i].bound && bound[i].bytes)
      r.push_back({static_cast<const char*>(bound[i].ptr), static_cast<const char*>(bound[i].ptr) + bound[i].bytes, i});
  std::sort(r.begin(), r.end(), [](const Range& a, const Range& b) { return a.lo < b.lo; });
  // sorted by start: an overlap with anything earlier shows against the furthest end seen so far;
  // among read-only entries sharing is harmless, so the furthest written end is kept apart
  const Range* far = nullptr;      // furthest-reaching entry so far
  const Range* far_w = nullptr;    // furthest-reaching written entry so far
  for (const Range& x : r) {
    const Range* hit = nullptr;
    if (far_w && x.lo < far_w->hi) hit = far_w;
    else if (written_[x.i] && far && x.lo < far->hi) hit = far;
    if (hit)
      throw Error("buffers '" + plan_.buffers[hit->i].name + "' and '" + plan_.buffers[x.i].name +
                  "' of the table are bound to overlapping device memory and the program writes one of them: table "
                  "entries must be distinct buffers (no in-place updates)");
    if (!far || x.hi > far->hi) far = &x;
    if (written_[x.i] && (!far_w || x.hi > far_w->hi)) far_w = &x;
  }
}

void HipProgram::launch_all(const std::vector<HipBuffer*>& bound) {
  std::vector<Span> spans(bound.size());
  for (size_t i = 0; i < bound.size(); ++i)
    if (bound[i]) spans[i] = {bound[i]->device_ptr(), bound[i]->byte_len(), true};
  launch_spans(spans);
}

void HipProgram::launch_spans(const std::vector<Span>& bound) {
  auto lk = dev_->stream_lock();               // the program's launches go out as one run
  const int lanes = plan_.lanes;
  std::vector<hipStream_t> streams(static_cast<size_t>(std::max(lanes, 1)), dev_->stream());
  if (lanes > 1) {
    dev_->make_current();
    if (events_.empty()) {
      // an event behind every launch somebody on another lane waits for
      events_.assign(plan_.launches.size(), nullptr);
      for (const LaunchSpec& ls : plan_.launches)
        for (int w : ls.waits)
          if (!events_[static_cast<size_t>(w)])
            check(hipEventCreateWithFlags(&events_[static_cast<size_t>(w)], hipEventDisableTiming), "hipEventCreateWithFlags");
      join_.assign(static_cast<size_t>(lanes - 1), nullptr);
      for (auto& e : join_) check(hipEventCreateWithFlags(&e, hipEventDisableTiming), "hipEventCreateWithFlags");
      check(hipEventCreateWithFlags(&fork_, hipEventDisableTiming), "hipEventCreateWithFlags");
    }
    // fork: the side lanes start behind everything queued on the device's stream so far
    check(hipEventRecord(fork_, dev_->stream()), "hipEventRecord");
    for (int s = 1; s < lanes; ++s) {
      streams[static_cast<size_t>(s)] = dev_->lane_stream(s);
      check(hipStreamWaitEvent(streams[static_cast<size_t>(s)], fork_, 0), "hipStreamWaitEvent");
    }
  }
  // Whatever happens, the side lanes are joined back: a launch that fails half-way must not
  // leave work on a side stream that later work on the device's stream does not wait for.
  struct Join {
    HipProgram* p;
    const std::vector<hipStream_t>& st;
    int lanes;
    ~Join() {
      for (int s = 1; s < lanes; ++s) {
        hipEvent_t e = p->join_.size() >= static_cast<size_t>(s) ? p->join_[static_cast<size_t>(s) - 1] : nullptr;
        if (!e || st[static_cast<size_t>(s)] == p->dev_->stream()) continue;
        (void)hipEventRecord(e, st[static_cast<size_t>(s)]);
        (void)hipStreamWaitEvent(p->dev_->stream(), e, 0);
      }
    }
  } join{this, streams, lanes};
  for (size_t l = 0; l < plan_.launches.size(); ++l) {
    const LaunchSpec& ls = plan_.launches[l];
    hipStream_t stream = streams[static_cast<size_t>(lanes > 1 ? ls.lane : 0)];
    if (lanes > 1)
      for (int w : ls.waits) check(hipStreamWaitEvent(stream, events_[static_cast<size_t>(w)], 0), "hipStreamWaitEvent");
    std::vector<void*> ptrs;
    for (size_t a = 0; a < ls.arg_bufs.size(); ++a) {
      const Span& b = bound[index_.at(ls.arg_bufs[a])];
      if (!b.bound) throw Error("launch '" + ls.entry + "' needs buffer '" + ls.arg_bufs[a] + "', which is not bound");
      if (a < ls.arg_min_bytes.size() && b.bytes < ls.arg_min_bytes[a])
        throw Error("Buffer size mismatch: '" + ls.arg_bufs[a] + "' needs at least " +
                    std::to_string(ls.arg_min_bytes[a]) + " bytes for '" + ls.entry + "', has " +
                    std::to_string(b.bytes));
      ptrs.push_back(b.ptr);
    }
    kernels_[l]->launch(ls.grid, ls.block, ls.lds_bytes, ptrs, stream);
    if (lanes > 1 && events_[l]) check(hipEventRecord(events_[l], stream), "hipEventRecord");
  }
}

void HipProgram::execute(HipBuffer* const* bufs, size_t n, bool sync) {
  std::lock_guard<std::mutex> lk(mu_);
  auto sl = dev_->stream_lock();               // binding may allocate (and fill) temps
  std::vector<HipBuffer*> cancelled;
  try {
    launch_all(bind(bufs, n, &cancelled));
  } catch (...) {
    // some launch was not queued: what it would have overwritten is owed its zeros again
    for (HipBuffer* b : cancelled) b->set_zero_pending(true);
    throw;
  }
  if (sync) dev_->synchronize();
}

// Scratch temps the plan appended (names starting with "eh_") sit behind the caller's table.
static bool plan_scratch(const ProgramPlan& plan, size_t i) {
  return plan.buffers[i].role == "temp" && plan.buffers[i].name.rfind("eh_", 0) == 0 && !plan.elided.count(plan.buffers[i].name);
}

size_t HipProgram::static_scratch_needed() const {
  size_t need = 0;
  for (size_t i = 0; i < plan_.buffers.size(); ++i)
    if (plan_scratch(plan_, i))
      need += (plan_.buffers[i].bytes() + kStaticScratchAlign - 1) / kStaticScratchAlign * kStaticScratchAlign;
  return need;
}

void HipProgram::execute_static(HipBuffer* const* bufs, size_t n, bool sync) {
  std::lock_guard<std::mutex> lk(mu_);
  auto sl = dev_->stream_lock();
  const size_t total = plan_.buffers.size();
  if (n > total) throw Error("program binds " + std::to_string(total) + " buffers, " + std::to_string(n) + " given");
  const size_t need = static_scratch_needed();
  if (need > kStaticScratchBytes)
    throw Error("Buffer size mismatch: the program's scratch buffers need " + std::to_string(need) +
                " bytes, the static scratch block holds " + std::to_string(kStaticScratchBytes) +
                "; use eh_program_execute, which allocates them");
  dev_->make_current();
  char* block = need ? static_cast<char*>(dev_->static_scratch()) : nullptr;
  std::vector<Span> bound(total);
  std::vector<HipBuffer*> given(total, nullptr);
  size_t off = 0;
  for (size_t i = 0; i < total; ++i) {
    const BufferInfo& bi = plan_.buffers[i];
    if (plan_.elided.count(bi.name)) continue;
    if (plan_scratch(plan_, i) && !(i < n && bufs[i])) {
      bound[i] = {block + off, bi.bytes(), true};
      off += (bi.bytes() + kStaticScratchAlign - 1) / kStaticScratchAlign * kStaticScratchAlign;
      continue;
    }
    HipBuffer* b = i < n ? bufs[i] : nullptr;
    if (!b)
      throw Error("MissingInput: buffer '" + bi.name + "' (" + bi.role + ") was not provided; this entry point allocates nothing");
    if (b->device() != dev_) throw Error("buffer '" + bi.name + "' lives on another device");
    if (bi.shape_known && b->byte_len() < bi.bytes())
      throw Error("Buffer size mismatch: '" + bi.name + "' needs " + std::to_string(bi.bytes()) + " bytes, has " +
                  std::to_string(b->byte_len()));
    given[i] = b;
    bound[i] = {b->device_ptr(), b->byte_len(), true};
  }
  refuse_aliases(bound);
  std::vector<HipBuffer*> cancelled;
  resolve_fills(given, &cancelled);              // (queues fills at most; allocates nothing)
  // another handle on this GPU (its own stream, its own lock) shares the block: take turns
  std::optional<StaticScratchTurn> turn;
  if (need) turn.emplace(dev_->index(), static_cast<void*>(dev_->stream()));
  try {
    launch_spans(bound);
  } catch (...) {
    for (HipBuffer* b : cancelled) b->set_zero_pending(true);
    throw;
  }
  if (sync) dev_->synchronize();
}

// ---------------------------------------------------------------------------------------------
// HipGraph: the launches of one execute, captured once on fixed buffers and replayed as a whole
// ---------------------------------------------------------------------------------------------

HipGraph::HipGraph(HipProgram* prog, HipBuffer* const* bufs, size_t n) : dev_(prog->device()) {
  std::lock_guard<std::mutex> lk(prog->mu_);
  // held across the whole capture: whatever another thread wants to put on this stream (a buffer
  // fill, a copy, another program's launches, a synchronisation) waits until the capture ended
  auto sl = dev_->stream_lock();
  // binding allocates missing temps: all of it happens before the capture starts, the capture
  // itself records kernel launches only (no memset or copy nodes)
  std::vector<HipBuffer*> bound = prog->bind(bufs, n, nullptr);
  launches_ = prog->plan().launches.size();
  kernels_ = prog->kernels_;
  // the program's own temps are shared with it by reference count; the caller's buffers are kept
  // alive by whoever owns their handles
  for (size_t i = 0; i < bound.size(); ++i)
    if (bound[i] && (i >= n || !bufs[i])) {
      bound[i]->retain();
      held_.push_back(bound[i]);
    }
  hipGraph_t graph = nullptr;
  try {
    check(hipStreamBeginCapture(dev_->stream(), hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
    try {
      prog->launch_all(bound);
    } catch (...) {
      (void)hipStreamEndCapture(dev_->stream(), &graph);
      if (graph) (void)hipGraphDestroy(graph);
      throw;
    }
    check(hipStreamEndCapture(dev_->stream(), &graph), "hipStreamEndCapture");
    hipError_t e = hipGraphInstantiate(&exec_, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    check(e, "hipGraphInstantiate");
  } catch (...) {
    drop();
    throw;
  }
}

void HipGraph::drop() {
  for (HipBuffer* b : held_)
    if (b->release()) delete b;
  held_.clear();
}

HipGraph::~HipGraph() {
  auto sl = dev_->stream_lock();
  (void)hipSetDevice(dev_->index());
  (void)hipStreamSynchronize(dev_->stream());
  if (exec_) (void)hipGraphExecDestroy(exec_);
  drop();
}

void HipGraph::replay(bool sync) {
  auto sl = dev_->stream_lock();
  dev_->make_current();
  check(hipGraphLaunch(exec_, dev_->stream()), "hipGraphLaunch");
  if (sync) dev_->synchronize();
}

void HipProgram::execute_positional(HipBuffer* const* inputs, size_t n_in, HipBuffer* const* outputs, size_t n_out,
                                    bool sync) {
  std::vector<HipBuffer*> bufs(plan_.buffers.size(), nullptr);
  size_t ii = 0, oi = 0;
  for (size_t i = 0; i < plan_.buffers.size(); ++i) {
    const std::string& role = plan_.buffers[i].role;
    if (role == "input" || role == "ones" || role == "zeros") {
      if (ii >= n_in) throw Error("kernel takes more inputs than the " + std::to_string(n_in) + " given");
      bufs[i] = inputs[ii++];
    } else if (role == "output") {
      if (oi >= n_out) throw Error("kernel takes more outputs than the " + std::to_string(n_out) + " given");
      bufs[i] = outputs[oi++];
    }
  }
  if (ii != n_in || oi != n_out)
    throw Error("kernel takes " + std::to_string(ii) + " inputs and " + std::to_string(oi) + " outputs, got " +
                std::to_string(n_in) + " and " + std::to_string(n_out));
  execute(bufs.data(), bufs.size(), sync);
}

std::vector<std::string> HipBackendRegistry::list_devices() {
  std::vector<std::string> out;
  int n = HipDevice::count();
  for (int i = 0; i < n; ++i) {
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, i) == hipSuccess) out.push_back(std::string(p.name) + " (" + p.gcnArchName + ")");
  }
  return out;
}

}  // namespace eh
