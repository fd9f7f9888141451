// The backend proper: device, buffers, compiler, kernels, registry -- the C++ counterparts of
// the traits a reference backend crate implements (src/backend/traits.rs: Device :273-306,
// Buffer :455-482, Kernel :531-587, Compiler :592-607; src/backend/device.rs:83-171
// BackendRegistry), shaped after crates/backend-c/src/{device,buffer,compiler,kernel,lib}.rs.
#pragma once

#include <hip/hip_runtime_api.h>

#include <atomic>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "ast.hpp"
#include "codegen.hpp"

namespace eh {

struct DeviceProfile {
  std::string name, arch;
  int compute_units = 0, warp_size = 64, max_work_group_size = 1024;
  size_t local_memory_size = 0, global_memory_size = 0;
  int clock_khz = 0, memory_clock_khz = 0, memory_bus_bits = 0, l2_bytes = 0;
};

class HipKernel;

// Code object produced by hiprtc (or read back from the disk cache).
struct Binary {
  std::vector<char> code;
  std::string log;
  bool from_cache = false;
};

class HipCompiler {
 public:
  // HIP C -> gfx950 code object.  Needs no device.  Throws eh::Error carrying the hiprtc log.
  // `refresh` ignores what the caches hold for this source and overwrites it (used when a
  // cached code object turns out not to load).
  static Binary compile(const std::string& source, const std::string& arch, bool use_disk_cache = true,
                        bool refresh = false);
  static std::vector<std::string> options(const std::string& arch);
  static std::string cache_dir();      // HARP_CACHE_DIR or ~/.cache/harp, + /code_objects/gfx950
  static bool disk_cache_enabled();    // HARP_NO_DISK_CACHE unset
};

class HipDevice {
 public:
  static int count();                  // 0 when no GPU/driver is present
  static bool is_available() { return count() > 0; }
  explicit HipDevice(int index);
  ~HipDevice();
  HipDevice(const HipDevice&) = delete;
  HipDevice& operator=(const HipDevice&) = delete;

  int index() const { return index_; }
  hipStream_t stream() const { return stream_; }
  // Side stream `lane` (1, 2, ...; default priority, created on first use): a program whose plan
  // spreads independent launches over lanes forks them off the device's stream and joins them
  // back before its execute returns, so to everybody else the device still has one stream.
  hipStream_t lane_stream(int lane);
  // Everything that enqueues on (or waits for) the device's one stream holds this lock while it
  // does: buffer fills and copies, launches of a program, graph replays, synchronisation -- and
  // a graph capture holds it from begin to end, so that no other thread's work is recorded into
  // the graph instead of running (or fails for touching a capturing stream).  Recursive: an
  // execute that synchronises at its end takes it twice.
  std::unique_lock<std::recursive_mutex> stream_lock() const { return std::unique_lock<std::recursive_mutex>(stream_mu_); }
  const DeviceProfile& profile() const { return profile_; }
  void make_current() const;
  void synchronize() const;

  // Loads a code object and resolves one entry point; modules are shared per (binary, entry).
  std::shared_ptr<HipKernel> load(const Binary& bin, const std::string& entry);

  // Device memory for buffers.  Released blocks are kept (up to a quarter of the device's
  // memory) and handed out again to requests of the same size without a hipMalloc/hipFree
  // pair and its device-wide wait: every use of a block is queued on this device's one
  // stream, so the next owner's work runs after the previous owner's.  ECLAT_HIP_NO_POOL
  // set in the environment turns the reuse off.
  void* allocate(size_t bytes);
  void release(void* ptr, size_t bytes);
  void trim();                         // returns every kept block to the driver
  size_t pooled_bytes() const { return pooled_bytes_; }
  // This device's static scratch block (static_scratch.hpp), resolved when the device was
  // opened; throws when that failed.
  void* static_scratch() const;

 private:
  int index_;
  hipStream_t stream_ = nullptr;
  std::vector<hipStream_t> side_streams_;
  DeviceProfile profile_;
  mutable std::recursive_mutex stream_mu_;
  std::mutex pool_mu_;
  std::multimap<size_t, void*> pool_;  // size -> free block
  size_t pooled_bytes_ = 0, pool_limit_ = 0;
  void* static_scratch_ = nullptr;
  std::string static_scratch_error_;
};

class HipBuffer {
 public:
  // Reads as zeros until something is written, as the reference's buffers do.  The fill itself
  // is put off until something needs the memory's contents: a kernel that overwrites the whole
  // buffer (the usual fate of an output the executor has just allocated) or a full write from
  // the host cancels it.
  HipBuffer(HipDevice* dev, size_t bytes);
  ~HipBuffer();
  HipBuffer(const HipBuffer&) = delete;
  HipBuffer& operator=(const HipBuffer&) = delete;

  size_t byte_len() const { return bytes_; }
  void* device_ptr() const { return ptr_; }       // the memory as it is: settle() first unless it is about to be overwritten
  bool zero_pending() const { return zero_pending_; }
  void settle();                                   // queues the fill if it is still owed
  void set_zero_pending(bool owed) { zero_pending_ = owed && ptr_; }   // (under the device's stream lock)
  HipDevice* device() const { return dev_; }
  void write_from_host(const void* src, size_t bytes);   // size must match exactly
  void read_to_host(void* dst, size_t bytes) const;
  void copy_from(const HipBuffer& src);                   // clone_buffer
  void retain() { refs_.fetch_add(1); }
  bool release() { return refs_.fetch_sub(1) == 1; }      // true when the last reference went

 private:
  HipDevice* dev_;
  void* ptr_ = nullptr;
  size_t bytes_;
  bool zero_pending_ = false;                      // guarded by the device's stream lock
  std::atomic<int> refs_{1};
};

// One loaded entry point.
class HipKernel {
 public:
  HipKernel(HipDevice* dev, const Binary& bin, const std::string& entry);
  ~HipKernel();
  // Queues the kernel on `stream` (nullptr: the device's stream).
  void launch(const unsigned grid[3], const unsigned block[3], unsigned lds_bytes,
              const std::vector<void*>& device_ptrs, hipStream_t stream = nullptr) const;
  const std::vector<char>& binary() const { return binary_; }   // Kernel::get_binary
  const std::string& entry() const { return entry_; }

 private:
  HipDevice* dev_;
  hipModule_t module_ = nullptr;
  hipFunction_t fn_ = nullptr;
  std::vector<char> binary_;
  std::string entry_;
};

// A Program compiled for a device: the launches in order plus the buffers they bind.
class HipProgram {
 public:
  HipProgram(HipDevice* dev, const std::string& ast_text, const GenOptions& opt);
  ~HipProgram();

  const ProgramPlan& plan() const { return plan_; }
  // `bufs[i]` binds plan().buffers[i]; entries for elided buffers are ignored, missing temps are
  // allocated once and kept.  Launches go to the device's stream; `sync` waits for them.
  void execute(HipBuffer* const* bufs, size_t n, bool sync);
  // Positional form (Kernel::execute): immutable pointer parameters, then mutable ones.
  void execute_positional(HipBuffer* const* inputs, size_t n_in, HipBuffer* const* outputs, size_t n_out, bool sync);
  // execute() without any device allocation: every buffer of the caller's table that reaches
  // memory must be given, and the scratch temps the plan appended (partial sums of split
  // reductions and contractions, chunk totals of scans) are placed in the device's static
  // scratch block instead of buffers of their own.  Throws when they do not fit.
  void execute_static(HipBuffer* const* bufs, size_t n, bool sync);
  size_t static_scratch_needed() const;          // bytes of the block execute_static() would use
  const HipKernel& kernel(size_t launch) const { return *kernels_.at(launch); }
  HipDevice* device() const { return dev_; }

 private:
  friend class HipGraph;
  // checks sizes, allocates missing temps; a buffer still owed its zero fill gets it now, unless
  // the first launch that touches it overwrites all of it (`cancelled` then lists it, so that a
  // failed execute can put the debt back)
  std::vector<HipBuffer*> bind(HipBuffer* const* bufs, size_t n, std::vector<HipBuffer*>* cancelled);
  void resolve_fills(const std::vector<HipBuffer*>& bound, std::vector<HipBuffer*>* cancelled);
  void launch_all(const std::vector<HipBuffer*>& bound);            // queues every launch on the stream
  struct Span {
    void* ptr = nullptr;
    size_t bytes = 0;
    bool bound = false;
  };
  void launch_spans(const std::vector<Span>& bound);                // the same, over plain address ranges
  void refuse_aliases(const std::vector<Span>& bound) const;        // throws when two entries overlap and one is written
  HipDevice* dev_;
  ProgramPlan plan_;
  std::vector<std::shared_ptr<HipKernel>> kernels_;
  std::map<std::string, size_t> index_;          // buffer name -> table index
  mutable std::vector<char> written_;            // by table index: some launch writes the buffer (filled on first use)
  std::vector<size_t> first_full_;               // by table index: size of the buffer the first launch that binds it overwrites whole (0: none)
  std::vector<HipBuffer*> temps_;                // owned, by table index (nullptr if unused)
  // Lanes (plan().lanes > 1): events_[l] is recorded behind launch l when a launch on another
  // lane waits for it; fork_ is recorded on the device's stream before the first launch and
  // join_[s-1] on side lane s behind its last one.  Created on the first execute.
  std::vector<hipEvent_t> events_, join_;
  hipEvent_t fork_ = nullptr;
  std::mutex mu_;
};

// One execute of a program on fixed buffers, captured from the device's stream as a HIP graph of
// kernel nodes: a replay queues all launches with one call.  Holds a reference to the program's
// temps and code objects, so it may outlive the program; the caller keeps its own buffers alive.
class HipGraph {
 public:
  HipGraph(HipProgram* prog, HipBuffer* const* bufs, size_t n);
  ~HipGraph();
  HipGraph(const HipGraph&) = delete;
  HipGraph& operator=(const HipGraph&) = delete;
  void replay(bool sync);
  size_t launches() const { return launches_; }

 private:
  void drop();
  HipDevice* dev_;
  hipGraphExec_t exec_ = nullptr;
  std::vector<HipBuffer*> held_;                 // program temps, by reference count
  std::vector<std::shared_ptr<HipKernel>> kernels_;
  size_t launches_ = 0;
};

// Key under which a program's tuned options are filed: FNV-1a (64 bit) of its AST text.
unsigned long long tune_key(const char* ast_text);
// Options for compiling `ast_text`: what the file named by ECLAT_HIP_TUNE holds for this program
// (lines "<16 hex digits of the key> <key=value,...>"; '#' starts a comment), then `options` on
// top.  Without the variable, or without an entry, just `options`.
GenOptions options_for(const char* ast_text, const char* options);

// With ECLAT_HIP_DUMP=<dir> in the environment, writes every launch of a plan there:
// <entry>.hip (the translation unit handed to hiprtc) and <entry>.txt (schedule, grid, block,
// LDS bytes, bound buffers, the lowered kernels the launch covers).  The counterpart of the
// reference's debug dumps of generated kernels (src/backend/pipeline.rs:150-153).
void dump_plan(const ProgramPlan& plan);

class HipBackendRegistry {
 public:
  static const char* kind() { return "hip"; }
  static const char* name() { return "HIP (gfx950)"; }
  static bool is_available() { return HipDevice::is_available(); }
  static bool supports_runtime() { return true; }
  static bool supports_binary_cache() { return true; }
  static std::vector<std::string> list_devices();
};

}  // namespace eh
