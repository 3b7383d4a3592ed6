// HSA tools library: one fixed SDMA engine per direction of host<->device copies.
//
// Why it exists.  The HIP runtime issues pinned host<->device copies with
// hsa_amd_memory_async_copy_on_engine and re-picks the engine of a stream from
// hsa_amd_memory_copy_engine_status: the lowest engine that is idle at that
// instant.  An engine counts as busy while this very stream's previous copy is
// still running, so a stream that keeps its direction saturated walks up
// through the engines.  On MI355X only SDMA engines 0-3 reach the host link's
// rate (57 GB/s for a 117 MB copy: 2.1 ms); engines 4-7 take 9.2 ms for the same
// copy, 8-11 take 11.7 ms and engine 12 takes 16.5 ms.  When the pick lands on
// the engine the other direction uses, the two directions share one in-order
// ring and the link runs half duplex.  A training step that streams optimizer
// states both ways falls into both traps for hundreds of milliseconds at a time.
//
// What it does.  The ROCr runtime loads every library named in HSA_TOOLS_LIB
// during hsa_init and hands it the API table.  OnLoad swaps the table's
// hsa_amd_memory_async_copy_on_engine for a wrapper that rewrites the engine of
// CPU->GPU copies to one fixed engine and of GPU->CPU copies to another.
// Dependency and completion signals pass through untouched, so the HIP runtime's
// stream ordering is unchanged; copies of one direction simply queue on one ring
// in issue order.  GPU<->GPU copies and everything else are left alone.  If the
// runtime rejects a rewritten call, the original call is made instead, and after
// eight such rejections in a row the rewrite switches itself off.
//
// Scope.  Until a host range is registered (oa_copy_engines_register_range) every
// pinned host<->device copy of the process is rewritten.  From the first
// registration on, only copies whose host side lies inside a registered range
// are: the optimizer's own buffers, which the package's pinned allocator
// registers.  Copies of anybody else in the process (a data loader, torch's
// pinned tensors) then keep the engine the HIP runtime chose and do not queue
// behind 100 MB state transfers on the two fixed rings.
//
// Configuration (read once, at load):
//   OFFLOAD_ADAM_COPY_ENGINES="<h2d mask>,<d2h mask>"   default "0x1,0x2"
//   OFFLOAD_ADAM_COPY_ENGINES=off                       load, but rewrite nothing
//
// The include directory of hsa_api_trace.h is laid out for ROCr's own build
// unless AMD_INTERNAL_BUILD is defined; the build line defines it and adds
// <rocm>/include/hsa to the include path.

#include <hsa.h>
#include <hsa_ext_amd.h>
#include <hsa_api_trace.h>

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <shared_mutex>
#include <vector>

#include "offload_adam_copy_engines.h"

namespace {

decltype(hsa_amd_memory_async_copy_on_engine)* real_copy_on_engine = nullptr;
decltype(hsa_amd_memory_async_copy)* real_copy = nullptr;
decltype(hsa_agent_get_info)* real_agent_get_info = nullptr;

std::atomic<int> loaded{0};
std::atomic<int> active{0};
unsigned h2d_engine = 0x1;
unsigned d2h_engine = 0x2;
std::atomic<unsigned long long> n_h2d{0}, n_d2h{0}, n_rejected{0}, n_unpinned{0};
std::atomic<int> rejected_in_a_row{0};
constexpr int kMaxRejectedInARow = 8;

// Registered host ranges, sorted by base; `scoped` is set by the first registration.
struct Range {
  uintptr_t base, end;
};
std::shared_mutex ranges_mutex;
std::vector<Range> ranges;
std::atomic<int> scoped{0};
std::atomic<unsigned long long> n_passed_by{0};

bool in_registered_range(const void* p) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  std::shared_lock<std::shared_mutex> lock(ranges_mutex);
  auto it = std::upper_bound(ranges.begin(), ranges.end(), a,
                             [](uintptr_t x, const Range& r) { return x < r.base; });
  if (it == ranges.begin()) return false;
  --it;
  return a < it->end;
}

// Which fixed engine a copy goes to: 0 = leave it to the runtime.
unsigned engine_for(const void* dst, bool dst_cpu, const void* src, bool src_cpu) {
  if (src_cpu == dst_cpu) return 0;
  if (scoped.load(std::memory_order_relaxed) && !in_registered_range(src_cpu ? src : dst)) {
    n_passed_by.fetch_add(1, std::memory_order_relaxed);
    return 0;
  }
  return src_cpu ? h2d_engine : d2h_engine;
}

bool single_bit(unsigned m) { return m != 0 && (m & (m - 1)) == 0 && m <= 0x8000u; }

bool is_cpu(hsa_agent_t agent) {
  hsa_device_type_t type = HSA_DEVICE_TYPE_GPU;
  if (real_agent_get_info(agent, HSA_AGENT_INFO_DEVICE, &type) != HSA_STATUS_SUCCESS) return false;
  return type == HSA_DEVICE_TYPE_CPU;
}

hsa_status_t copy_on_fixed_engine(void* dst, hsa_agent_t dst_agent, const void* src,
                                  hsa_agent_t src_agent, size_t size, uint32_t num_dep_signals,
                                  const hsa_signal_t* dep_signals, hsa_signal_t completion_signal,
                                  hsa_amd_sdma_engine_id_t engine_id, bool force_copy_on_sdma) {
  if (active.load(std::memory_order_relaxed)) {
    const bool src_cpu = is_cpu(src_agent), dst_cpu = is_cpu(dst_agent);
    const unsigned want = engine_for(dst, dst_cpu, src, src_cpu);
    if (want != 0) {
      hsa_status_t st = real_copy_on_engine(dst, dst_agent, src, src_agent, size, num_dep_signals,
                                            dep_signals, completion_signal,
                                            static_cast<hsa_amd_sdma_engine_id_t>(want),
                                            force_copy_on_sdma);
      if (st == HSA_STATUS_SUCCESS) {
        (src_cpu ? n_h2d : n_d2h).fetch_add(1, std::memory_order_relaxed);
        rejected_in_a_row.store(0, std::memory_order_relaxed);
        return st;
      }
      n_rejected.fetch_add(1, std::memory_order_relaxed);
      if (rejected_in_a_row.fetch_add(1, std::memory_order_relaxed) + 1 >= kMaxRejectedInARow)
        active.store(0, std::memory_order_relaxed);
    }
  }
  return real_copy_on_engine(dst, dst_agent, src, src_agent, size, num_dep_signals, dep_signals,
                             completion_signal, engine_id, force_copy_on_sdma);
}

// The runtime's other copy call names no engine and lets ROCr choose one (HIP
// falls back to it when the engine status query offers nothing).  Host<->device
// copies that arrive here are sent to the same fixed engines; a rejected rewrite
// falls through to the call as it was made.
hsa_status_t copy_without_engine(void* dst, hsa_agent_t dst_agent, const void* src,
                                 hsa_agent_t src_agent, size_t size, uint32_t num_dep_signals,
                                 const hsa_signal_t* dep_signals,
                                 hsa_signal_t completion_signal) {
  if (active.load(std::memory_order_relaxed)) {
    const bool src_cpu = is_cpu(src_agent), dst_cpu = is_cpu(dst_agent);
    const unsigned want = engine_for(dst, dst_cpu, src, src_cpu);
    if (want != 0) {
      n_unpinned.fetch_add(1, std::memory_order_relaxed);
      hsa_status_t st = real_copy_on_engine(dst, dst_agent, src, src_agent, size, num_dep_signals,
                                            dep_signals, completion_signal,
                                            static_cast<hsa_amd_sdma_engine_id_t>(want), false);
      if (st == HSA_STATUS_SUCCESS) {
        (src_cpu ? n_h2d : n_d2h).fetch_add(1, std::memory_order_relaxed);
        return st;
      }
      n_rejected.fetch_add(1, std::memory_order_relaxed);
    }
  }
  return real_copy(dst, dst_agent, src, src_agent, size, num_dep_signals, dep_signals,
                   completion_signal);
}

// "0x1,0x2" -> masks; anything malformed keeps the defaults.  Returns false for "off".
bool read_config() {
  const char* s = getenv("OFFLOAD_ADAM_COPY_ENGINES");
  if (!s || !*s) return true;
  if (!strcmp(s, "off") || !strcmp(s, "0") || !strcmp(s, "none")) return false;
  char* end = nullptr;
  unsigned long a = strtoul(s, &end, 0);
  if (!end || *end != ',') return true;
  unsigned long b = strtoul(end + 1, &end, 0);
  if (single_bit((unsigned)a) && single_bit((unsigned)b)) {
    h2d_engine = (unsigned)a;
    d2h_engine = (unsigned)b;
  }
  return true;
}

}  // namespace

extern "C" bool OnLoad(HsaApiTable* table, uint64_t /*runtime_version*/,
                       uint64_t /*failed_tool_count*/, const char* const* /*failed_tool_names*/) {
  if (!table || !table->core_ || !table->amd_ext_) return true;
  if (!table->amd_ext_->hsa_amd_memory_async_copy_on_engine_fn) return true;
  const bool rewrite = read_config();
  real_agent_get_info = table->core_->hsa_agent_get_info_fn;
  real_copy_on_engine = table->amd_ext_->hsa_amd_memory_async_copy_on_engine_fn;
  table->amd_ext_->hsa_amd_memory_async_copy_on_engine_fn = copy_on_fixed_engine;
  if (table->amd_ext_->hsa_amd_memory_async_copy_fn) {
    real_copy = table->amd_ext_->hsa_amd_memory_async_copy_fn;
    table->amd_ext_->hsa_amd_memory_async_copy_fn = copy_without_engine;
  }
  active.store(rewrite ? 1 : 0);
  loaded.store(1);
  return true;
}

extern "C" void OnUnload() { active.store(0); }

extern "C" int oa_copy_engines_loaded(void) { return loaded.load(); }

extern "C" int oa_copy_engines_active(void) { return active.load(); }

extern "C" void oa_copy_engines_config(unsigned* h2d_mask, unsigned* d2h_mask) {
  if (h2d_mask) *h2d_mask = h2d_engine;
  if (d2h_mask) *d2h_mask = d2h_engine;
}

extern "C" unsigned long long oa_copy_engines_unpinned_calls(void) { return n_unpinned.load(); }

extern "C" int oa_copy_engines_register_range(const void* base, size_t bytes) {
  if (!base || bytes == 0) return -1;
  const uintptr_t b = reinterpret_cast<uintptr_t>(base);
  std::unique_lock<std::shared_mutex> lock(ranges_mutex);
  auto it = std::lower_bound(ranges.begin(), ranges.end(), b,
                             [](const Range& r, uintptr_t x) { return r.base < x; });
  if (it != ranges.end() && it->base == b) it->end = b + bytes;
  else ranges.insert(it, Range{b, b + bytes});
  scoped.store(1, std::memory_order_relaxed);
  return 0;
}

extern "C" int oa_copy_engines_unregister_range(const void* base) {
  const uintptr_t b = reinterpret_cast<uintptr_t>(base);
  std::unique_lock<std::shared_mutex> lock(ranges_mutex);
  for (auto it = ranges.begin(); it != ranges.end(); ++it) {
    if (it->base == b) {
      ranges.erase(it);
      return 0;
    }
  }
  return -1;
}

extern "C" int oa_copy_engines_scoped(void) { return scoped.load(); }

extern "C" unsigned long long oa_copy_engines_passed_by(void) { return n_passed_by.load(); }

extern "C" void oa_copy_engines_stats(unsigned long long* h2d_copies, unsigned long long* d2h_copies,
                                      unsigned long long* rejected) {
  if (h2d_copies) *h2d_copies = n_h2d.load();
  if (d2h_copies) *d2h_copies = n_d2h.load();
  if (rejected) *rejected = n_rejected.load();
}
