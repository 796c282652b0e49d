// Library lifetime, the single stream, the pooled device allocator with its
// live-block registry, host<->device copies through pinned staging, event
// timing, and recording of a sequence of launches into a HIP graph.
#include <ctype.h>
#include <string.h>

#include <map>
#include <mutex>
#include <set>
#include <unordered_map>
#include <vector>

#include "common.h"

namespace tfhip {
namespace {

constexpr size_t kStagingBytes = size_t(32) << 20;  // per pinned staging buffer
constexpr int kStagingBuffers = 2;

struct RecordedGraph {
  hipGraphExec_t exec = nullptr;
  size_t nodes = 0;
  std::vector<std::pair<void *, size_t>> owned;         // block, class size
  struct Ref {
    uintptr_t base;
    size_t size;
    uint64_t generation;
  };
  std::vector<Ref> refs;   // blocks a recorded kernel names and that were live when the recording ended
  std::vector<uintptr_t> writes;   // of those, the blocks a recorded call writes: a replay changes their contents
};

struct Runtime {
  bool ready = false;
  int device = 0;
  hipStream_t stream = nullptr;
  hipDeviceProp_t prop;
  // live blocks: base address -> usable size. `owned` blocks came from the pool.
  std::map<uintptr_t, size_t> live;
  std::map<uintptr_t, bool> owned;
  // Every hand-out of an address (tfhip_alloc, tfhip_register_external) gets a new
  // number: an address that was freed and handed out again is a different block.
  std::map<uintptr_t, uint64_t> generation;
  uint64_t next_generation = 1;
  std::unordered_map<size_t, std::vector<void *>> free_lists;  // by class size
  size_t live_bytes = 0, pooled_bytes = 0;
  void *staging[kStagingBuffers] = {nullptr, nullptr};
  hipEvent_t staging_done[kStagingBuffers] = {nullptr, nullptr};
  bool staging_busy[kStagingBuffers] = {false, false};
  int next_staging = 0;
  void *workspace = nullptr;
  size_t workspace_bytes = 0;
  hipEvent_t events[TFHIP_MAX_EVENTS] = {};
  bool event_recorded[TFHIP_MAX_EVENTS] = {};
  // Recording (tfhip_capture_begin .. tfhip_capture_end). A recorded graph
  // replays kernels with the addresses they were given, so it keeps what it
  // needs: blocks freed while recording go to `capture_free` (reused by later
  // allocations of the same recording, then owned by the graph), and every
  // block an operand check saw is noted in `capture_refs` (checked again at
  // each replay).
  bool capturing = false;
  std::unordered_map<size_t, std::vector<void *>> capture_free;
  std::set<uintptr_t> capture_refs;
  std::set<uintptr_t> capture_writes;   // of those, the blocks some recorded call writes
  std::map<int, RecordedGraph> graphs;
  int next_graph = 1;
  std::vector<void *> retired_workspaces;  // outgrown while a graph might still name them
  // Filters that were searched for Inf / NaN: block base -> scans of ranges inside that block.
  // An entry holds the generation of the block it was made for, and leaves when the block is
  // written through this library (uploads, kernel results) or freed.
  struct FilterScan {
    uintptr_t ptr;
    size_t elems;
    uint64_t generation;
    bool nonfinite;
  };
  std::unordered_map<uintptr_t, std::vector<FilterScan>> filter_scans;
  int *scan_flag = nullptr;   // pinned host word the scan kernel's verdict is copied to
  int *scan_flag_dev = nullptr;
};


Runtime g;
std::mutex g_mutex;
thread_local char g_error[1024] = "";
char g_kernel[256] = "";
int g_repeat = 1;

// Size classes: eight per power of two, at least 256 bytes.
size_t class_size(size_t bytes) {
  if (bytes <= 256) return 256;
  size_t p = 256;
  while (p < bytes) p <<= 1;
  const size_t step = p >> 4;  // p/2 .. p in eight steps of p/16
  const size_t lo = p >> 1;
  size_t c = lo + ((bytes - lo + step - 1) / step) * step;
  return c < 256 ? 256 : c;
}

void give_back_locked(void *p, size_t cls) {
  g.free_lists[cls].push_back(p);
  g.pooled_bytes += cls;
}

void release_pool_locked() {
  for (auto &kv : g.free_lists) {
    for (void *p : kv.second) (void)hipFree(p);
    kv.second.clear();
  }
  g.pooled_bytes = 0;
}

}  // namespace

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof g_error, fmt, ap);
  va_end(ap);
  return code;
}

void note_kernel(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_kernel, sizeof g_kernel, fmt, ap);
  va_end(ap);
}

int launch_repeat() { return g_repeat; }

int g_init_count = 0;
const char *const kTuningNames[kTuneCount] = {
#define TFHIP_TUNING_NAME(id, name) name,
    TFHIP_TUNING_KNOBS(TFHIP_TUNING_NAME)
#undef TFHIP_TUNING_NAME
};
// Every knob starts unset, whatever their number.
struct TuningTable {
  int value[kTuneCount];
  TuningTable() {
    for (int &v : value) v = -1;
  }
};
TuningTable g_tuning;
int tuning(int key) { return g_tuning.value[key]; }

void read_tuning_from_environment() {
  for (int i = 0; i < kTuneCount; ++i) {
    char env_name[64] = "TFHIP_";
    size_t at = strlen(env_name);
    for (const char *c = kTuningNames[i]; *c && at + 1 < sizeof env_name; ++c) env_name[at++] = (char)toupper((unsigned char)*c);
    env_name[at] = 0;
    const char *e = getenv(env_name);
    g_tuning.value[i] = e ? atoi(e) : -1;
  }
}

bool initialised() { return g.ready; }
int init_count() { return g_init_count; }
int device_index() { return g.device; }
hipStream_t stream() { return g.stream; }
int num_cus() { return g.prop.multiProcessorCount; }

// Scratch for kernels that need device memory beyond their operands (split-K
// partial sums). One block that only grows; work on the single stream is
// ordered, so consecutive launches may share it.
// The fixed block belongs to the calling thread (the entry point that allocates
// nothing sets it for the length of its call): another thread's launches keep
// the library's own block.
thread_local void *g_fixed_ws = nullptr;
thread_local size_t g_fixed_ws_bytes = 0;
thread_local bool g_ws_fixed = false;
size_t g_workspace_allocations = 0;   // hipMalloc calls made by workspace() since tfhip_init
int g_last_splits = 0;                // K slices of the last GEMM launch

FixedWorkspace::FixedWorkspace(void *ptr, size_t bytes) {
  g_fixed_ws = ptr;
  g_fixed_ws_bytes = bytes;
  g_ws_fixed = true;
}
FixedWorkspace::~FixedWorkspace() {
  g_ws_fixed = false;
  g_fixed_ws = nullptr;
  g_fixed_ws_bytes = 0;
}
bool workspace_is_fixed() { return g_ws_fixed; }
size_t fixed_workspace_bytes() { return g_fixed_ws_bytes; }

void *workspace(size_t bytes) {
  if (g_ws_fixed) return bytes <= g_fixed_ws_bytes ? g_fixed_ws : nullptr;
  if (bytes <= g.workspace_bytes) return g.workspace;
  if (g.capturing || !g.graphs.empty()) {
    // a recorded graph may name the old block: it stays allocated until shutdown
    if (g.workspace) g.retired_workspaces.push_back(g.workspace);
  } else {
    (void)hipStreamSynchronize(g.stream);   // a launch in flight may still use the old block
    if (g.workspace) (void)hipFree(g.workspace);
  }
  g.workspace = nullptr;
  g.workspace_bytes = 0;
  const size_t want = (bytes + (size_t(1) << 24) - 1) & ~((size_t(1) << 24) - 1);
  if (hipMalloc(&g.workspace, want) != hipSuccess) {
    (void)hipGetLastError();
    g.workspace = nullptr;
    return nullptr;
  }
  g.workspace_bytes = want;
  ++g_workspace_allocations;
  return g.workspace;
}

void note_splits(int splits) { g_last_splits = splits; }

bool range_is_live(const void *p, size_t bytes) {
  std::lock_guard<std::mutex> lock(g_mutex);
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  auto it = g.live.upper_bound(a);
  if (it == g.live.begin()) return false;
  --it;
  const bool inside = a >= it->first && a + bytes <= it->first + it->second && a + bytes >= a;
  if (inside && g.capturing) g.capture_refs.insert(it->first);
  return inside;
}

bool capturing() { return g.capturing; }

__global__ void clear_word(int *word) { *word = 0; }

// 1 in *flag when any of the n values has an all-ones exponent (Inf or NaN)
__global__ __launch_bounds__(256) void find_nonfinite(const unsigned *__restrict__ bits, long long n, int *flag) {
  const long long stride = (long long)gridDim.x * 256;
  bool hit = false;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) hit |= (bits[i] & 0x7f800000u) == 0x7f800000u;
  if (hit) *flag = 1;   // (every writer writes the same value)
}

void forget_filter_scans(const void *p) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (g.filter_scans.empty() && !g.capturing) return;
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  auto it = g.live.upper_bound(a);
  if (it == g.live.begin()) return;
  --it;
  if (a >= it->first + it->second) return;
  g.filter_scans.erase(it->first);
  // a replay writes the block again, with whatever its inputs hold then
  if (g.capturing) g.capture_writes.insert(it->first);
}

int scan_filter(const float *w, int64_t elems, const char *who, bool *nonfinite) {
  *nonfinite = false;
  if (elems <= 0) return kOk;
  const uintptr_t a = reinterpret_cast<uintptr_t>(w);
  uintptr_t base = 0;
  uint64_t generation = 0;
  {
    std::lock_guard<std::mutex> lock(g_mutex);
    auto it = g.live.upper_bound(a);
    if (it == g.live.begin()) return fail(kOutOfRange, "%s: the filter is not inside a live device buffer", who);
    --it;
    if (a + (size_t)elems * 4 > it->first + it->second)
      return fail(kOutOfRange, "%s: the filter is not inside a live device buffer", who);
    base = it->first;
    generation = g.generation[base];
    auto found = g.filter_scans.find(base);
    if (found != g.filter_scans.end()) {
      for (const Runtime::FilterScan &f : found->second) {
        if (f.ptr == a && f.elems == (size_t)elems && f.generation == generation) {
          *nonfinite = f.nonfinite;
          return kOk;
        }
      }
    }
  }
  // not known yet: one small kernel and a wait for its verdict, once per filter
  if (g.capturing)
    return fail(kBadArgument,
                "%s: this filter has not been searched for Inf / NaN yet, which needs a wait for the stream; run the "
                "call once outside the recording",
                who);
  *g.scan_flag = 0;
  clear_word<<<dim3(1), dim3(1), 0, g.stream>>>(g.scan_flag_dev);
  long long blocks = (elems + 255) / 256;
  if (blocks > 1024) blocks = 1024;
  find_nonfinite<<<dim3((unsigned)blocks), dim3(256), 0, g.stream>>>(reinterpret_cast<const unsigned *>(w), elems,
                                                                     g.scan_flag_dev);
  TFHIP_CHECK_HIP(hipGetLastError());
  TFHIP_CHECK_HIP(hipMemcpyAsync(g.scan_flag, g.scan_flag_dev, sizeof(int), hipMemcpyDeviceToHost, g.stream));
  TFHIP_CHECK_HIP(hipStreamSynchronize(g.stream));
  *nonfinite = *g.scan_flag != 0;
  std::lock_guard<std::mutex> lock(g_mutex);
  // (the block may have gone while the lock was open: the entry would then never match)
  g.filter_scans[base].push_back({a, (size_t)elems, generation, *nonfinite});
  return kOk;
}

// Copies a small result straight into pinned host memory: a kernel starts within
// a few microseconds, the copy engine needs 10-15 for a transfer of any size.
__global__ __launch_bounds__(256) void copy_to_host(const float4 *__restrict__ src, float4 *__restrict__ dst, int n4) {
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n4; i += gridDim.x * 256) dst[i] = src[i];
}

}  // namespace tfhip

using namespace tfhip;

extern "C" {

const char *tfhip_last_error(void) { return g_error; }

int tfhip_init(int device) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (g.ready) {
    if (device == g.device) return kOk;
    return fail(kBadArgument, "tfhip_init: already initialised on device %d", g.device);
  }
  int count = 0;
  TFHIP_CHECK_HIP(hipGetDeviceCount(&count));
  TFHIP_CHECK_ARG(device >= 0 && device < count,
                  "tfhip_init: device %d not present (%d visible)", device, count);
  TFHIP_CHECK_HIP(hipSetDevice(device));
  TFHIP_CHECK_HIP(hipGetDeviceProperties(&g.prop, device));
  if (strncmp(g.prop.gcnArchName, "gfx950", 6) != 0) {
    return fail(kBadArgument,
                "tfhip_init: device %d is %s; this library carries gfx950 code only",
                device, g.prop.gcnArchName);
  }
  {
    const int rc = setup_static_scratch(device);   // this device's copy of the static scratch array
    if (rc != kOk) return rc;
  }
  TFHIP_CHECK_HIP(hipStreamCreateWithFlags(&g.stream, hipStreamNonBlocking));
  for (int i = 0; i < kStagingBuffers; ++i) {
    TFHIP_CHECK_HIP(hipHostMalloc(&g.staging[i], kStagingBytes, hipHostMallocDefault));
    TFHIP_CHECK_HIP(hipEventCreateWithFlags(&g.staging_done[i], hipEventDisableTiming));
    g.staging_busy[i] = false;
  }
  TFHIP_CHECK_HIP(hipHostMalloc(reinterpret_cast<void **>(&g.scan_flag), sizeof(int), hipHostMallocDefault));
  TFHIP_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&g.scan_flag_dev), sizeof(int)));
  g.device = device;
  ++g_init_count;
  read_tuning_from_environment();
  g.ready = true;
  return kOk;
}

int tfhip_shutdown(void) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g.ready) return kOk;
  if (g.capturing) {
    hipGraph_t abandoned = nullptr;
    (void)hipStreamEndCapture(g.stream, &abandoned);
    if (abandoned) (void)hipGraphDestroy(abandoned);
    (void)hipGetLastError();
    g.capturing = false;
  }
  (void)hipStreamSynchronize(g.stream);
  for (auto &kv : g.graphs) {
    if (kv.second.exec) (void)hipGraphExecDestroy(kv.second.exec);
    for (auto &b : kv.second.owned) (void)hipFree(b.first);
  }
  g.graphs.clear();
  for (auto &kv : g.capture_free) {
    for (void *p : kv.second) (void)hipFree(p);
  }
  g.capture_free.clear();
  g.capture_refs.clear();
  g.capture_writes.clear();
  for (void *p : g.retired_workspaces) (void)hipFree(p);
  g.retired_workspaces.clear();
  for (auto &kv : g.live) {
    if (g.owned[kv.first]) (void)hipFree(reinterpret_cast<void *>(kv.first));
  }
  g.live.clear();
  g.owned.clear();
  g.generation.clear();
  g.filter_scans.clear();
  if (g.scan_flag) (void)hipHostFree(g.scan_flag);
  if (g.scan_flag_dev) (void)hipFree(g.scan_flag_dev);
  g.scan_flag = nullptr;
  g.scan_flag_dev = nullptr;
  g.live_bytes = 0;
  release_pool_locked();
  for (int i = 0; i < kStagingBuffers; ++i) {
    if (g.staging[i]) (void)hipHostFree(g.staging[i]);
    if (g.staging_done[i]) (void)hipEventDestroy(g.staging_done[i]);
    g.staging[i] = nullptr;
    g.staging_done[i] = nullptr;
  }
  for (int i = 0; i < TFHIP_MAX_EVENTS; ++i) {
    if (g.events[i]) (void)hipEventDestroy(g.events[i]);
    g.events[i] = nullptr;
    g.event_recorded[i] = false;
  }
  if (g.workspace) (void)hipFree(g.workspace);
  g.workspace = nullptr;
  g.workspace_bytes = 0;
  g_workspace_allocations = 0;
  g_last_splits = 0;
  (void)hipStreamDestroy(g.stream);
  g.stream = nullptr;
  g.ready = false;
  return kOk;
}

int tfhip_device_info(char *name, size_t name_len, char *arch, size_t arch_len,
                      int *cus, int *clock_khz, size_t *hbm_bytes) {
  TFHIP_REQUIRE_INIT();
  if (name && name_len) snprintf(name, name_len, "%s", g.prop.name);
  if (arch && arch_len) snprintf(arch, arch_len, "%s", g.prop.gcnArchName);
  if (cus) *cus = g.prop.multiProcessorCount;
  if (clock_khz) *clock_khz = g.prop.clockRate;
  if (hbm_bytes) *hbm_bytes = g.prop.totalGlobalMem;
  return kOk;
}

int tfhip_alloc(size_t bytes, void **dptr) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(dptr != nullptr, "tfhip_alloc: dptr is NULL");
  const size_t cls = class_size(bytes);
  std::lock_guard<std::mutex> lock(g_mutex);
  void *p = nullptr;
  auto &fl = g.free_lists[cls];
  if (g.capturing && !g.capture_free[cls].empty()) {
    p = g.capture_free[cls].back();
    g.capture_free[cls].pop_back();
  } else if (!fl.empty()) {
    p = fl.back();
    fl.pop_back();
    g.pooled_bytes -= cls;
  } else {
    hipError_t e = hipMalloc(&p, cls);
    if (e == hipErrorOutOfMemory) {
      (void)hipGetLastError();
      if (!g.capturing) (void)hipStreamSynchronize(g.stream);   // (a recording stream cannot be waited for)
      release_pool_locked();
      e = hipMalloc(&p, cls);
    }
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return fail(kOutOfMemory, "tfhip_alloc: hipMalloc(%zu) failed: %s", cls,
                  hipGetErrorString(e));
    }
  }
  g.live[reinterpret_cast<uintptr_t>(p)] = cls;
  g.owned[reinterpret_cast<uintptr_t>(p)] = true;
  g.generation[reinterpret_cast<uintptr_t>(p)] = g.next_generation++;
  g.live_bytes += cls;
  *dptr = p;
  return kOk;
}

int tfhip_free(void *dptr) {
  TFHIP_REQUIRE_INIT();
  std::lock_guard<std::mutex> lock(g_mutex);
  const uintptr_t a = reinterpret_cast<uintptr_t>(dptr);
  auto it = g.live.find(a);
  if (it == g.live.end() || !g.owned[a]) {
    return fail(kBadArgument, "tfhip_free: %p is not a live block of this library", dptr);
  }
  // Work already enqueued on the single stream runs before any later kernel
  // that is handed this block again, so the block can be reused at once.
  const size_t cls = it->second;
  g.live.erase(it);
  g.owned.erase(a);
  g.generation.erase(a);
  g.filter_scans.erase(a);
  g.live_bytes -= cls;
  if (g.capturing) {
    g.capture_free[cls].push_back(dptr);   // the graph being recorded names it: the graph keeps it
  } else {
    give_back_locked(dptr, cls);
  }
  return kOk;
}

int tfhip_register_external(void *dptr, size_t bytes) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(dptr != nullptr && bytes > 0, "tfhip_register_external: empty range");
  std::lock_guard<std::mutex> lock(g_mutex);
  g.live[reinterpret_cast<uintptr_t>(dptr)] = bytes;
  g.owned[reinterpret_cast<uintptr_t>(dptr)] = false;
  g.generation[reinterpret_cast<uintptr_t>(dptr)] = g.next_generation++;
  return kOk;
}

int tfhip_unregister_external(void *dptr) {
  TFHIP_REQUIRE_INIT();
  std::lock_guard<std::mutex> lock(g_mutex);
  const uintptr_t a = reinterpret_cast<uintptr_t>(dptr);
  auto it = g.live.find(a);
  if (it == g.live.end() || g.owned[a]) {
    return fail(kBadArgument, "tfhip_unregister_external: %p was not registered", dptr);
  }
  g.live.erase(it);
  g.owned.erase(a);
  g.generation.erase(a);
  g.filter_scans.erase(a);
  return kOk;
}

int tfhip_memory_info(size_t *live, size_t *live_bytes, size_t *pooled_bytes) {
  TFHIP_REQUIRE_INIT();
  std::lock_guard<std::mutex> lock(g_mutex);
  size_t n = 0;
  for (auto &kv : g.owned) n += kv.second ? 1 : 0;
  if (live) *live = n;
  if (live_bytes) *live_bytes = g.live_bytes;
  if (pooled_bytes) *pooled_bytes = g.pooled_bytes;
  return kOk;
}

int tfhip_workspace_info(size_t *bytes, size_t *allocations, int *last_splits) {
  TFHIP_REQUIRE_INIT();
  if (bytes) *bytes = g.workspace_bytes;
  if (allocations) *allocations = g_workspace_allocations;
  if (last_splits) *last_splits = g_last_splits;
  return kOk;
}

int tfhip_filter_is_finite(const float *filter, int64_t elems, int *finite) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(finite != nullptr && elems >= 0, "tfhip_filter_is_finite: bad argument");
  bool nonfinite = false;
  const int rc = scan_filter(filter, elems, "tfhip_filter_is_finite", &nonfinite);
  if (rc != kOk) return rc;
  *finite = nonfinite ? 0 : 1;
  return kOk;
}

int tfhip_upload(void *dst, size_t dst_offset, const void *host, size_t bytes) {
  TFHIP_REQUIRE_INIT();
  TFHIP_REFUSE_WHILE_RECORDING();
  if (bytes == 0) return kOk;
  TFHIP_CHECK_ARG(host != nullptr, "tfhip_upload: host pointer is NULL");
  char *d = static_cast<char *>(dst) + dst_offset;
  TFHIP_CHECK_OUTPUT(d, bytes, 1, "dst");
  const char *h = static_cast<const char *>(host);
  size_t done = 0;
  while (done < bytes) {
    const size_t chunk = bytes - done < kStagingBytes ? bytes - done : kStagingBytes;
    const int s = g.next_staging;
    g.next_staging = (s + 1) % kStagingBuffers;
    if (g.staging_busy[s]) TFHIP_CHECK_HIP(hipEventSynchronize(g.staging_done[s]));
    memcpy(g.staging[s], h + done, chunk);
    TFHIP_CHECK_HIP(hipMemcpyAsync(d + done, g.staging[s], chunk, hipMemcpyHostToDevice, g.stream));
    TFHIP_CHECK_HIP(hipEventRecord(g.staging_done[s], g.stream));
    g.staging_busy[s] = true;
    done += chunk;
  }
  return kOk;
}

int tfhip_download(void *host, const void *src, size_t src_offset, size_t bytes) {
  TFHIP_REQUIRE_INIT();
  TFHIP_REFUSE_WHILE_RECORDING();
  if (bytes == 0) {
    TFHIP_CHECK_HIP(hipStreamSynchronize(g.stream));
    return kOk;
  }
  TFHIP_CHECK_ARG(host != nullptr, "tfhip_download: host pointer is NULL");
  const char *s = static_cast<const char *>(src) + src_offset;
  TFHIP_CHECK_RANGE(s, bytes, 1, "src");
  char *h = static_cast<char *>(host);
  size_t done = 0;
  while (done < bytes) {
    const size_t chunk = bytes - done < kStagingBytes ? bytes - done : kStagingBytes;
    const int b = g.next_staging;
    g.next_staging = (b + 1) % kStagingBuffers;
    if (g.staging_busy[b]) TFHIP_CHECK_HIP(hipEventSynchronize(g.staging_done[b]));
    g.staging_busy[b] = false;
    constexpr size_t kKernelCopyBytes = size_t(1) << 20;
    if (chunk <= kKernelCopyBytes && chunk % 16 == 0 && reinterpret_cast<uintptr_t>(s + done) % 16 == 0) {
      const int n4 = (int)(chunk / 16);
      const int blocks = (n4 + 255) / 256 < 64 ? (n4 + 255) / 256 : 64;
      copy_to_host<<<blocks, 256, 0, g.stream>>>(reinterpret_cast<const float4 *>(s + done),
                                                 static_cast<float4 *>(g.staging[b]), n4);
      TFHIP_CHECK_HIP(hipGetLastError());
    } else {
      TFHIP_CHECK_HIP(hipMemcpyAsync(g.staging[b], s + done, chunk, hipMemcpyDeviceToHost, g.stream));
    }
    TFHIP_CHECK_HIP(hipStreamSynchronize(g.stream));
    memcpy(h + done, g.staging[b], chunk);
    done += chunk;
  }
  return kOk;
}

int tfhip_set_tuning(const char *name, int value) {
  for (int i = 0; name && i < kTuneCount; ++i) {
    if (strcmp(name, kTuningNames[i]) == 0) {
      g_tuning.value[i] = value < 0 ? -1 : value;
      return kOk;
    }
  }
  return fail(kBadArgument, "tfhip_set_tuning: unknown knob '%s'", name ? name : "(null)");
}

int tfhip_set_launch_repeat(int n) {
  if (n < 1 || n > 100000) return fail(kBadArgument, "tfhip_set_launch_repeat: %d not in 1..100000", n);
  g_repeat = n;
  return kOk;
}

int tfhip_last_kernel(char *name, size_t name_len) {
  if (name && name_len) snprintf(name, name_len, "%s", g_kernel);
  return kOk;
}

int tfhip_sync(void) {
  TFHIP_REQUIRE_INIT();
  TFHIP_REFUSE_WHILE_RECORDING();
  TFHIP_CHECK_HIP(hipStreamSynchronize(g.stream));
  return kOk;
}

int tfhip_event_record(int slot) {
  TFHIP_REQUIRE_INIT();
  TFHIP_REFUSE_WHILE_RECORDING();
  TFHIP_CHECK_ARG(slot >= 0 && slot < TFHIP_MAX_EVENTS, "tfhip_event_record: slot %d out of range", slot);
  if (!g.events[slot]) TFHIP_CHECK_HIP(hipEventCreate(&g.events[slot]));
  TFHIP_CHECK_HIP(hipEventRecord(g.events[slot], g.stream));
  g.event_recorded[slot] = true;
  return kOk;
}

int tfhip_event_elapsed(int start_slot, int end_slot, float *ms) {
  TFHIP_REQUIRE_INIT();
  TFHIP_REFUSE_WHILE_RECORDING();
  TFHIP_CHECK_ARG(start_slot >= 0 && start_slot < TFHIP_MAX_EVENTS && end_slot >= 0 &&
                      end_slot < TFHIP_MAX_EVENTS && ms != nullptr,
                  "tfhip_event_elapsed: bad arguments");
  TFHIP_CHECK_ARG(g.event_recorded[start_slot] && g.event_recorded[end_slot],
                  "tfhip_event_elapsed: slot %d or %d was never recorded", start_slot, end_slot);
  TFHIP_CHECK_HIP(hipEventSynchronize(g.events[end_slot]));
  TFHIP_CHECK_HIP(hipEventElapsedTime(ms, g.events[start_slot], g.events[end_slot]));
  return kOk;
}

int tfhip_capture_begin(void) {
  TFHIP_REQUIRE_INIT();
  std::lock_guard<std::mutex> lock(g_mutex);
  TFHIP_CHECK_ARG(!g.capturing, "tfhip_capture_begin: a recording is already open");
  // Relaxed mode: an allocation that misses the pool may still call hipMalloc.
  TFHIP_CHECK_HIP(hipStreamBeginCapture(g.stream, hipStreamCaptureModeRelaxed));
  g.capturing = true;
  g.capture_refs.clear();
  g.capture_writes.clear();
  return kOk;
}

int tfhip_capture_end(int *graph_id, int *nodes) {
  TFHIP_REQUIRE_INIT();
  std::lock_guard<std::mutex> lock(g_mutex);
  TFHIP_CHECK_ARG(g.capturing, "tfhip_capture_end: no recording is open");
  g.capturing = false;
  hipGraph_t graph = nullptr;
  hipError_t e = hipStreamEndCapture(g.stream, &graph);
  RecordedGraph rec;
  if (e == hipSuccess) {
    (void)hipGraphGetNodes(graph, nullptr, &rec.nodes);
    if (graph_id != nullptr) e = hipGraphInstantiate(&rec.exec, graph, nullptr, nullptr, 0);
  }
  if (graph) (void)hipGraphDestroy(graph);
  if (e != hipSuccess || graph_id == nullptr) {
    // nothing will replay: the blocks set aside for the graph return to the pool
    (void)hipGetLastError();
    for (auto &kv : g.capture_free) {
      for (void *p : kv.second) give_back_locked(p, kv.first);
    }
    g.capture_free.clear();
    g.capture_refs.clear();
    g.capture_writes.clear();
    if (e != hipSuccess) return fail(kHipError, "tfhip_capture_end: %s", hipGetErrorString(e));
    if (nodes) *nodes = (int)rec.nodes;
    return kOk;
  }
  for (auto &kv : g.capture_free) {
    for (void *p : kv.second) {
      rec.owned.emplace_back(p, kv.first);
      g.capture_refs.erase(reinterpret_cast<uintptr_t>(p));
    }
  }
  g.capture_free.clear();
  for (uintptr_t base : g.capture_refs) {
    auto it = g.live.find(base);
    if (it != g.live.end()) {
      rec.refs.push_back({base, it->second, g.generation[base]});
      if (g.capture_writes.count(base)) rec.writes.push_back(base);
    }
  }
  g.capture_refs.clear();
  g.capture_writes.clear();
  const int id = g.next_graph++;
  if (nodes) *nodes = (int)rec.nodes;
  g.graphs[id] = std::move(rec);
  *graph_id = id;
  return kOk;
}

int tfhip_graph_launch(int graph_id) {
  TFHIP_REQUIRE_INIT();
  std::lock_guard<std::mutex> lock(g_mutex);
  TFHIP_CHECK_ARG(!g.capturing, "tfhip_graph_launch: a recording is open");
  auto it = g.graphs.find(graph_id);
  TFHIP_CHECK_ARG(it != g.graphs.end(), "tfhip_graph_launch: no graph %d", graph_id);
  for (auto &r : it->second.refs) {
    // the same address, size AND hand-out: a block that was freed and handed out again
    // at the same address belongs to someone else now
    auto b = g.live.find(r.base);
    auto gen = g.generation.find(r.base);
    if (b == g.live.end() || b->second != r.size || gen == g.generation.end() || gen->second != r.generation) {
      return fail(kOutOfRange,
                  "tfhip_graph_launch: graph %d names the device buffer at %p (%zu bytes), which has been freed since it was recorded",
                  graph_id, reinterpret_cast<void *>(r.base), r.size);
    }
  }
  // what the library remembered about the old contents of the blocks this replay writes
  for (uintptr_t base : it->second.writes) g.filter_scans.erase(base);
  for (int r = g_repeat; r > 0; --r) TFHIP_CHECK_HIP(hipGraphLaunch(it->second.exec, g.stream));
  return kOk;
}

int tfhip_graph_destroy(int graph_id) {
  TFHIP_REQUIRE_INIT();
  std::lock_guard<std::mutex> lock(g_mutex);
  auto it = g.graphs.find(graph_id);
  TFHIP_CHECK_ARG(it != g.graphs.end(), "tfhip_graph_destroy: no graph %d", graph_id);
  (void)hipStreamSynchronize(g.stream);   // no replay is in flight when the executable goes
  if (it->second.exec) (void)hipGraphExecDestroy(it->second.exec);
  for (auto &b : it->second.owned) give_back_locked(b.first, b.second);
  g.graphs.erase(it);
  return kOk;
}

}  // extern "C"
