// Host<->device copies of the streaming path on a fixed SDMA engine per direction,
// issued by this library and ordered inside a HIP stream.
//
// Why.  hipMemcpyAsync lets the HIP runtime pick an SDMA engine per copy - the
// lowest one that is idle at that instant - and a stream that keeps its direction
// saturated walks up through the engines.  On MI355X only engines 0-3 reach the
// host link's rate (a 117 MB copy: 2.1 ms on engines 0-3, 9-16 ms on the others),
// and when the pick lands on the engine the other direction uses, the link runs
// half duplex.  The ROCr runtime does take an engine from its caller
// (hsa_amd_memory_async_copy_on_engine), but an HSA copy is ordered by HSA signals
// and a HIP stream does not hand its own out.
//
// How.  hipExtMallocWithFlags(..., hipMallocSignalMemory) returns the value word of an
// HSA signal the HIP runtime created, in host memory the GPU can address
// (amd_signal_t, hsa/amd_hsa_signal.h: the signal's handle is the address of that
// structure, its value the second 8-byte field; the library checks the arithmetic
// against hsa_amd_signal_value_pointer for every signal it uses).  A copy on stream S
// is then three asynchronous steps:
//   1. link_release_kernel on S (dep := 0)     S reaches this point -> the copy may start
//   2. hsa_amd_memory_async_copy_on_engine(..., dep, done, engine)
//   3. link_wait_kernel on S (polls done)      S goes on when the engine has finished
// so the copy starts after everything S was given before and everything S is given
// afterwards starts after the copy: the semantics of hipMemcpyAsync on S.  Events
// and cross-stream waits around it stay ordinary HIP calls.  Nothing here depends
// on the process environment or on when the library was loaded, other streams'
// copies are untouched, and a profiler that traces HSA copies sees these.  (HIP's own
// hipStreamWriteValue64 / hipStreamWaitValue64 are kernels too on this runtime; its
// wait polls without pause, see link_wait_kernel.)  What it costs against a
// hipMemcpyAsync whose engine is fixed from outside: the two one-lane kernels per
// unit, about 4 % of an 8B training step that keeps both directions of the link busy.
//
// oa_link_copy_batch issues several copies of one direction as one unit: one
// dependency signal for all of them (step 1 once), every copy handed to the engine
// before the stream is given its first wait, then step 3 per copy - the engine runs
// them back to back instead of waiting for the stream to come round between copies
// and the stream runs one wait per recorded event instead of one per copy.
//
// Signals come from a ring per GPU; the slots of a unit are reused only after an
// event recorded behind the unit's last wait has completed.  Not for use under stream
// capture.

#include <dlfcn.h>
#include <hsa/amd_hsa_signal.h>
#include <hsa/hsa.h>
#include <hsa/hsa_ext_amd.h>

#include <atomic>
#include <cstddef>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

#include "oa_common.hpp"

namespace {

// The stream-side wait for a copy: one lane polls the completion signal's value word
// (host memory the engine decrements to 0) about every 3 us and returns when it reads
// 0.  hipStreamWaitValue64 does the same with a kernel of the HIP runtime that polls
// without pause; its reads cross the host link the copies are using, and an 8B
// training step that streams 80 GB each way ran 6 % longer with it.  The wait is
// bounded: after `max_polls` (kDefaultPolls: about a minute) the lane gives up, raises
// `*gave_up` for the host to find, and the stream goes on - a copy that never
// completes must not leave a wave spinning for good.
constexpr unsigned kDefaultPolls = 10u * 1000u * 1000u;

__global__ void __launch_bounds__(64)
link_wait_kernel(const int64_t* done, unsigned* gave_up, unsigned max_polls) {
  if (threadIdx.x != 0) return;
  for (unsigned n = 0; n < max_polls; ++n) {
    if (__hip_atomic_load(done, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM) == 0) return;
    __builtin_amdgcn_s_sleep(127);
    __builtin_amdgcn_s_sleep(127);
  }
  __hip_atomic_store(gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// The stream-side release of a unit's copies: writes 0 to the dependency signal.
__global__ void __launch_bounds__(64) link_release_kernel(int64_t* dep) {
  if (threadIdx.x == 0) __hip_atomic_store(dep, (int64_t)0, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

struct HsaApi {
  decltype(hsa_init)* init = nullptr;
  decltype(hsa_iterate_agents)* iterate_agents = nullptr;
  decltype(hsa_agent_get_info)* agent_get_info = nullptr;
  decltype(hsa_signal_store_relaxed)* signal_store = nullptr;
  decltype(hsa_amd_signal_value_pointer)* signal_value_pointer = nullptr;
  decltype(hsa_amd_memory_async_copy_on_engine)* copy_on_engine = nullptr;
};

struct Slot {
  int64_t* dep = nullptr;   // value words of two HIP-owned HSA signals
  int64_t* done = nullptr;
  hsa_signal_t dep_sig{}, done_sig{};
  hipEvent_t passed = nullptr;  // recorded behind a unit whose last slot this was
  int fence = -1;  // slot whose `passed` event covers this slot's last use (its unit's last slot)
  bool used = false;
};

constexpr int kMaxDevices = 64;
constexpr int kRing = 1024;  // copies that may be outstanding per GPU before a caller waits

struct DeviceLink {
  std::mutex mu;
  int state = 0;  // 0 = not set up yet, 1 = ready, < 0 = an OA_LINK_* reason it is not
  hsa_agent_t gpu{}, cpu{};
  std::vector<Slot> ring;
  size_t next = 0;
  unsigned* gave_up = nullptr;  // pinned host word a wait kernel raises when it times out
  unsigned max_polls = kDefaultPolls;  // bound of the waits issued from now on
  std::atomic<unsigned long long> n_h2d{0}, n_d2h{0}, n_fallback{0};
};

DeviceLink g_links[kMaxDevices];
HsaApi g_hsa;
std::once_flag g_hsa_once;
bool g_hsa_ok = false;
unsigned g_h2d_engine = 0x1, g_d2h_engine = 0x2;
bool g_switched_off = false;

bool single_bit(unsigned long m) { return m != 0 && (m & (m - 1)) == 0 && m <= 0x8000ul; }

void load_hsa() {
  // OFFLOAD_ADAM_COPY_ENGINES="<h2d mask>,<d2h mask>" (default "0x1,0x2") or "off"
  if (const char* s = getenv("OFFLOAD_ADAM_COPY_ENGINES")) {
    if (!strcmp(s, "off") || !strcmp(s, "0") || !strcmp(s, "none")) {
      g_switched_off = true;
    } else {
      char* end = nullptr;
      const unsigned long a = strtoul(s, &end, 0);
      if (end && *end == ',') {
        const unsigned long b = strtoul(end + 1, &end, 0);
        if (single_bit(a) && single_bit(b)) {
          g_h2d_engine = (unsigned)a;
          g_d2h_engine = (unsigned)b;
        }
      }
    }
  }
  // the HIP runtime has the ROCr runtime loaded already; take the same instance
  void* h = dlopen("libhsa-runtime64.so.1", RTLD_NOW | RTLD_NOLOAD);
  if (!h) h = dlopen("libhsa-runtime64.so.1", RTLD_NOW);
  if (!h) return;
#define OA_SYM(field, name) \
  g_hsa.field = reinterpret_cast<decltype(g_hsa.field)>(dlsym(h, name)); \
  if (!g_hsa.field) return
  OA_SYM(init, "hsa_init");
  OA_SYM(iterate_agents, "hsa_iterate_agents");
  OA_SYM(agent_get_info, "hsa_agent_get_info");
  OA_SYM(signal_store, "hsa_signal_store_relaxed");
  OA_SYM(signal_value_pointer, "hsa_amd_signal_value_pointer");
  OA_SYM(copy_on_engine, "hsa_amd_memory_async_copy_on_engine");
#undef OA_SYM
  // reference-counted; the HIP runtime holds the first reference for the process's life
  g_hsa_ok = g_hsa.init() == HSA_STATUS_SUCCESS;
}

struct AgentSearch {
  unsigned domain, bus, device;
  hsa_agent_t gpu{}, first_cpu{};
  bool have_gpu = false, have_cpu = false;
};

hsa_status_t visit_agent(hsa_agent_t agent, void* data) {
  auto* want = static_cast<AgentSearch*>(data);
  hsa_device_type_t type = HSA_DEVICE_TYPE_DSP;
  if (g_hsa.agent_get_info(agent, HSA_AGENT_INFO_DEVICE, &type) != HSA_STATUS_SUCCESS)
    return HSA_STATUS_SUCCESS;
  if (type == HSA_DEVICE_TYPE_CPU) {
    if (!want->have_cpu) {
      want->first_cpu = agent;
      want->have_cpu = true;
    }
  } else if (type == HSA_DEVICE_TYPE_GPU && !want->have_gpu) {
    uint32_t bdf = 0, domain = 0;
    const auto bdf_attr = static_cast<hsa_agent_info_t>(HSA_AMD_AGENT_INFO_BDFID);
    const auto dom_attr = static_cast<hsa_agent_info_t>(HSA_AMD_AGENT_INFO_DOMAIN);
    if (g_hsa.agent_get_info(agent, bdf_attr, &bdf) != HSA_STATUS_SUCCESS) return HSA_STATUS_SUCCESS;
    if (g_hsa.agent_get_info(agent, dom_attr, &domain) != HSA_STATUS_SUCCESS) domain = want->domain;
    if (((bdf >> 8) & 0xFF) == want->bus && ((bdf >> 3) & 0x1F) == want->device &&
        domain == want->domain) {
      want->gpu = agent;
      want->have_gpu = true;
    }
  }
  return HSA_STATUS_SUCCESS;
}

// The signal whose value word HIP handed out, checked against the runtime's own answer.
bool signal_of(int64_t* value, hsa_signal_t* out) {
  hsa_signal_t s;
  s.handle = reinterpret_cast<uint64_t>(value) - offsetof(amd_signal_t, value);
  const auto* raw = reinterpret_cast<const amd_signal_t*>(s.handle);
  if (raw->kind != AMD_SIGNAL_KIND_USER) return false;
  volatile hsa_signal_value_t* at = nullptr;
  if (g_hsa.signal_value_pointer(s, &at) != HSA_STATUS_SUCCESS) return false;
  if (reinterpret_cast<const volatile void*>(at) != reinterpret_cast<const volatile void*>(value))
    return false;
  *out = s;
  return true;
}

void release_ring(DeviceLink& link) {
  for (Slot& s : link.ring) {
    if (s.dep) (void)hipFree(s.dep);
    if (s.done) (void)hipFree(s.done);
    if (s.passed) (void)hipEventDestroy(s.passed);
  }
  link.ring.clear();
}

// Called with link.mu held and `dev` current.  Leaves link.state at 1 or at a reason.
void set_up(DeviceLink& link, int dev) {
  std::call_once(g_hsa_once, load_hsa);
  if (g_switched_off) { link.state = OA_LINK_OFF; return; }
  if (!g_hsa_ok) { link.state = OA_LINK_NO_RUNTIME; return; }
  char busid[64] = {0};
  AgentSearch want{};
  if (hipDeviceGetPCIBusId(busid, sizeof(busid), dev) != hipSuccess ||
      sscanf(busid, "%x:%x:%x", &want.domain, &want.bus, &want.device) != 3) {
    link.state = OA_LINK_NO_AGENT;
    return;
  }
  if (g_hsa.iterate_agents(visit_agent, &want) != HSA_STATUS_SUCCESS || !want.have_gpu ||
      !want.have_cpu) {
    link.state = OA_LINK_NO_AGENT;
    return;
  }
  link.gpu = want.gpu;
  link.cpu = want.first_cpu;
  hsa_agent_t nearest{};
  const auto near_attr = static_cast<hsa_agent_info_t>(HSA_AMD_AGENT_INFO_NEAREST_CPU);
  if (g_hsa.agent_get_info(link.gpu, near_attr, &nearest) == HSA_STATUS_SUCCESS && nearest.handle)
    link.cpu = nearest;

  if (hipHostMalloc(reinterpret_cast<void**>(&link.gave_up), sizeof(unsigned), hipHostMallocDefault) !=
      hipSuccess) {
    (void)hipGetLastError();
    link.state = OA_LINK_NO_SIGNALS;
    return;
  }
  *link.gave_up = 0;
  link.ring.resize(kRing);
  for (Slot& s : link.ring) {
    bool ok = hipExtMallocWithFlags(reinterpret_cast<void**>(&s.dep), 8, hipMallocSignalMemory) == hipSuccess &&
              hipExtMallocWithFlags(reinterpret_cast<void**>(&s.done), 8, hipMallocSignalMemory) == hipSuccess &&
              hipEventCreateWithFlags(&s.passed, hipEventDisableTiming) == hipSuccess;
    ok = ok && signal_of(s.dep, &s.dep_sig) && signal_of(s.done, &s.done_sig);
    if (!ok) {
      (void)hipGetLastError();
      release_ring(link);
      link.state = OA_LINK_NO_SIGNALS;
      return;
    }
  }
  link.state = 1;
}

DeviceLink* current_link(int* dev_out, int* rc) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) { *rc = static_cast<int>(err); return nullptr; }
  if (dev < 0 || dev >= kMaxDevices) { *rc = OA_ERANGE; return nullptr; }
  *dev_out = dev;
  *rc = 0;
  return &g_links[dev];
}

// `count` copies of one direction as ONE unit in the stream's order: all of them start
// after the work the stream was given before (one dependency signal, written by the
// stream), run back to back on the direction's engine without returning to the
// stream in between, and the stream observes their completions in order, recording
// record_events[i] (if any) behind copy i.  Called with the link's mutex held.
int issue_batch(DeviceLink& link, int count, void* const* dsts, const void* const* srcs,
                const size_t* bytes, bool h2d, hipStream_t stream, void* const* record_events) {
  hipError_t err;
  // slots of this unit; every one is reusable only after the whole unit has passed
  const size_t first = link.next;
  for (int i = 0; i < count; ++i) {
    Slot& s = link.ring[(first + i) % kRing];
    if (s.used) {
      // The stream that used this slot is past the slot's unit once that unit's event is
      // done.  (Slots are taken in ring order, so the event's own slot - the last of that
      // unit - has not been handed out again, and the event not recorded again, before
      // this one.)
      err = hipEventSynchronize(link.ring[s.fence].passed);
      if (err != hipSuccess) return static_cast<int>(err);
      s.used = false;
    }
    g_hsa.signal_store(s.done_sig, 1);
  }
  link.next = (first + count) % kRing;
  Slot& head = link.ring[first];
  g_hsa.signal_store(head.dep_sig, 1);
  hipLaunchKernelGGL(link_release_kernel, dim3(1), dim3(64), 0, stream, head.dep);
  err = hipGetLastError();
  if (err != hipSuccess) return static_cast<int>(err);  // nothing else was enqueued
  const hsa_agent_t dst_agent = h2d ? link.gpu : link.cpu, src_agent = h2d ? link.cpu : link.gpu;
  const auto engine = static_cast<hsa_amd_sdma_engine_id_t>(h2d ? g_h2d_engine : g_d2h_engine);
  // Engine side first: every copy is in the engine's queue before the stream is given
  // its first wait, so the engine never idles between the copies of a unit.
  int taken = 0;
  for (; taken < count; ++taken) {
    if (bytes[taken] == 0) continue;
    Slot& s = link.ring[(first + taken) % kRing];
    if (g_hsa.copy_on_engine(dsts[taken], dst_agent, srcs[taken], src_agent, bytes[taken], 1,
                             &head.dep_sig, s.done_sig, engine, false) != HSA_STATUS_SUCCESS)
      break;  // the runtime declined: this copy and the rest go through the HIP runtime
  }
  // The engine completes a direction's copies in the order it was given them, so the
  // stream only has to observe the copies something is recorded behind, and the last.
  int last_taken = -1;
  for (int i = 0; i < taken; ++i)
    if (bytes[i] != 0) last_taken = i;
  int rc = 0;
  for (int i = 0; i < count && rc == 0; ++i) {
    Slot& s = link.ring[(first + i) % kRing];
    if (bytes[i] != 0) {
      if (i < taken) {
        err = hipSuccess;
        if (i == last_taken || (record_events && record_events[i])) {
          hipLaunchKernelGGL(link_wait_kernel, dim3(1), dim3(64), 0, stream, s.done, link.gave_up,
                             link.max_polls);
          err = hipGetLastError();
        }
        (h2d ? link.n_h2d : link.n_d2h).fetch_add(1, std::memory_order_relaxed);
      } else {
        link.n_fallback.fetch_add(1, std::memory_order_relaxed);
        err = hipMemcpyAsync(dsts[i], srcs[i], bytes[i],
                             h2d ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost, stream);
      }
      if (err != hipSuccess) rc = static_cast<int>(err);
    }
    if (rc == 0 && record_events && record_events[i]) {
      err = hipEventRecord(static_cast<hipEvent_t>(record_events[i]), stream);
      if (err != hipSuccess) rc = static_cast<int>(err);
    }
  }
  // The unit's signals (its one dependency signal above all) may be written again once
  // the stream is past this point: one event for the unit, in its last slot.
  const int fence = static_cast<int>((first + count - 1) % kRing);
  const bool recorded = hipEventRecord(link.ring[fence].passed, stream) == hipSuccess;
  if (!recorded && rc == 0) rc = static_cast<int>(hipGetLastError());
  for (int i = 0; i < count; ++i) {
    Slot& s = link.ring[(first + i) % kRing];
    s.fence = fence;
    s.used = true;
  }
  if (!recorded) {
    // without the event nothing tells when the slots are free again: wait here, once
    (void)hipStreamSynchronize(stream);
    for (int i = 0; i < count; ++i) link.ring[(first + i) % kRing].used = false;
  }
  return rc;
}

int link_copies(int count, void* const* dsts, const void* const* srcs, const size_t* bytes,
                bool h2d, void* stream_v, void* wait_event, void* const* record_events) {
  if (count < 0) return OA_EINVAL;
  if (count > 0 && (!dsts || !srcs || !bytes)) return OA_EINVAL;
  for (int i = 0; i < count; ++i)
    if (bytes[i] != 0 && (!dsts[i] || !srcs[i])) return OA_EINVAL;
  int dev = -1, rc = 0;
  DeviceLink* link = current_link(&dev, &rc);
  if (!link) return rc;
  hipStream_t stream = static_cast<hipStream_t>(stream_v);
  std::lock_guard<std::mutex> lock(link->mu);
  if (link->state == 0) set_up(*link, dev);
  if (link->state != 1) return OA_EUNAVAILABLE;
  if (*static_cast<volatile unsigned*>(link->gave_up)) return OA_ELINKTIMEOUT;
  if (wait_event) {
    const hipError_t err = hipStreamWaitEvent(stream, static_cast<hipEvent_t>(wait_event), 0);
    if (err != hipSuccess) return static_cast<int>(err);
  }
  // units of at most a quarter of the ring: a unit's slots are reused together
  constexpr int kUnit = kRing / 4;
  for (int at = 0; at < count; at += kUnit) {
    const int n = count - at < kUnit ? count - at : kUnit;
    rc = issue_batch(*link, n, dsts + at, srcs + at, bytes + at, h2d, stream,
                     record_events ? record_events + at : nullptr);
    if (rc) return rc;
  }
  return 0;
}

int link_copy(void* dst, const void* src, size_t bytes, bool h2d, void* stream,
              void* wait_event, void* record_event) {
  void* const rec[1] = {record_event};
  return link_copies(1, &dst, &src, &bytes, h2d, stream, wait_event, rec);
}

}  // namespace

extern "C" int oa_h2d_async(void* dst, const void* src, size_t bytes, void* stream,
                            void* wait_event, void* record_event) {
  return link_copy(dst, src, bytes, true, stream, wait_event, record_event);
}

extern "C" int oa_d2h_async(void* dst, const void* src, size_t bytes, void* stream,
                            void* wait_event, void* record_event) {
  return link_copy(dst, src, bytes, false, stream, wait_event, record_event);
}

extern "C" int oa_link_copy_batch(int count, void* const* dsts, const void* const* srcs,
                                  const size_t* bytes, int kind, void* stream,
                                  void* const* record_events) {
  if (kind != OA_COPY_H2D && kind != OA_COPY_D2H) return OA_EINVAL;
  return link_copies(count, dsts, srcs, bytes, kind == OA_COPY_H2D, stream, nullptr,
                     record_events);
}

extern "C" int oa_link_wait_limit(unsigned long long max_polls, int clear_timeout) {
  if (max_polls > 0xFFFFFFFFull) return OA_ERANGE;
  int dev = -1, rc = 0;
  DeviceLink* link = current_link(&dev, &rc);
  if (!link) return rc;
  std::lock_guard<std::mutex> lock(link->mu);
  if (link->state == 0) set_up(*link, dev);
  if (link->state != 1) return OA_EUNAVAILABLE;
  link->max_polls = max_polls ? static_cast<unsigned>(max_polls) : kDefaultPolls;
  const bool timed_out = *static_cast<volatile unsigned*>(link->gave_up) != 0;
  if (clear_timeout) *static_cast<volatile unsigned*>(link->gave_up) = 0;
  return timed_out ? OA_ELINKTIMEOUT : 0;
}

extern "C" int oa_link_copy_status(unsigned* h2d_engine, unsigned* d2h_engine,
                                   unsigned long long* h2d_copies,
                                   unsigned long long* d2h_copies,
                                   unsigned long long* runtime_copies) {
  int dev = -1, rc = 0;
  DeviceLink* link = current_link(&dev, &rc);
  if (!link) return rc;
  std::lock_guard<std::mutex> lock(link->mu);
  if (link->state == 0) set_up(*link, dev);
  if (h2d_engine) *h2d_engine = g_h2d_engine;
  if (d2h_engine) *d2h_engine = g_d2h_engine;
  if (h2d_copies) *h2d_copies = link->n_h2d.load();
  if (d2h_copies) *d2h_copies = link->n_d2h.load();
  if (runtime_copies) *runtime_copies = link->n_fallback.load();
  return link->state == 1 ? 0 : link->state;
}
