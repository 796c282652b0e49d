// Internal declarations shared by the translation units of libtfjs_hip.so.
#pragma once

#include <initializer_list>
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/tfjs_hip.h"

namespace tfhip {

// Records the message returned by tfhip_last_error() and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

enum Status {
  kOk = 0,
  kNotInitialised = 1,
  kHipError = 2,
  kBadArgument = 3,
  kOutOfRange = 4,
  kOutOfMemory = 5
};

bool initialised();
int init_count();          // how many times tfhip_init has set a device up: per-device set-up keyed on it is redone after a shutdown
hipStream_t stream();
int num_cus();
int device_index();        // the device tfhip_init was given
// Device scratch of at least `bytes` (nullptr if it cannot be allocated); valid until the next call.
void *workspace(size_t bytes);
// While a FixedWorkspace object lives, workspace() hands the thread that made it
// the caller's block instead of the library's growing one and allocates nothing:
// a request beyond `bytes` returns nullptr, and workspace_is_fixed() tells a
// launcher to fit its request to fixed_workspace_bytes().
struct FixedWorkspace {
  FixedWorkspace(void *ptr, size_t bytes);
  ~FixedWorkspace();
};
bool workspace_is_fixed();
// Records the number of K slices a GEMM launch was cut into (tfhip_workspace_info reports the last).
void note_splits(int splits);
size_t fixed_workspace_bytes();
// Resolves the device address of gemm.hip's static scratch array for `device`
// (which must be current). Called by tfhip_init.
int setup_static_scratch(int device);

// True when [p, p + bytes) lies inside one live block (own or external).
bool range_is_live(const void *p, size_t bytes);
// No operand has more elements than this (2^40: four times the bytes of the largest memory this
// library runs on): element counts beyond it are refused before anything is multiplied by them.
constexpr long long kMaxElems = 1LL << 40;

// True when the product of the non-negative factors is below `limit`, decided
// without forming a product that could overflow 64 bits.
inline bool product_below(int64_t limit, std::initializer_list<int64_t> factors) {
  int64_t p = 1;
  for (const int64_t f : factors) {
    if (f < 0) return false;
    if (f == 0) return limit > 0;
    if (p > (limit - 1) / f) return false;
    p *= f;
  }
  return p < limit;
}
// Whether the `elems` floats at `w` hold an Inf or a NaN. The answer is remembered per (address,
// length, allocation generation of the block), so a filter costs one small kernel and one wait for
// the stream, once; a call for a filter not seen yet fails while a recording is open. `who` names
// the entry point in error messages.
int scan_filter(const float *w, int64_t elems, const char *who, bool *nonfinite);
// Drops what scan_filter remembers about the block that holds p (the block is being written).
void forget_filter_scans(const void *p);
// True when a filter window of `f` taps (dilation `dil`) can reach outside an axis of `in` positions:
// `out` windows, `stride` apart, the first one starting `pad` positions before the axis.
inline bool window_can_miss(int64_t in, int64_t out, int64_t stride, int64_t pad, int64_t f, int64_t dil) {
  return pad > 0 || (out - 1) * stride - pad + (f - 1) * dil >= in;
}
// For the fused kernels that pad with zeros and multiply them by the filter: kOk with *refuse = true when
// the `elems` values of the filter at `w` are not all finite (the reference skips taps outside the image,
// so an Inf or NaN filter value must not meet the padding: the caller runs the separate kernels, which
// route such a filter to their tap-skipping form).
constexpr const char *kNonfiniteFilterMessage =
    "a filter holds Inf or NaN and its windows reach outside the image: the fused kernel multiplies the padding's "
    "zeros by it where the reference skips the tap; run the separate convolutions (tfhip_filter_is_finite tells "
    "beforehand)";
inline int refuse_nonfinite_filter(const float *w, int64_t elems, const char *who, bool *refuse) {
  return scan_filter(w, elems, who, refuse);
}
// True between tfhip_capture_begin and tfhip_capture_end.
bool capturing();

#define TFHIP_REQUIRE_INIT()                                              \
  do {                                                                    \
    if (!::tfhip::initialised())                                          \
      return ::tfhip::fail(::tfhip::kNotInitialised,                      \
                           "%s: tfhip_init has not been called", __func__); \
  } while (0)

// Entry points that wait for the stream or copy through the host cannot be recorded.
#define TFHIP_REFUSE_WHILE_RECORDING()                                        \
  do {                                                                        \
    if (::tfhip::capturing())                                                 \
      return ::tfhip::fail(::tfhip::kBadArgument,                             \
                           "%s: not possible between tfhip_capture_begin and tfhip_capture_end", __func__); \
  } while (0)

#define TFHIP_CHECK_HIP(expr)                                               \
  do {                                                                      \
    hipError_t e_ = (expr);                                                 \
    if (e_ != hipSuccess)                                                   \
      return ::tfhip::fail(::tfhip::kHipError, "%s: %s failed: %s", __func__, \
                           #expr, hipGetErrorString(e_));                   \
  } while (0)

#define TFHIP_CHECK_ARG(cond, ...)                                \
  do {                                                            \
    if (!(cond)) return ::tfhip::fail(::tfhip::kBadArgument, __VA_ARGS__); \
  } while (0)

// Operand `name` of `elems` float-sized (`esize` bytes) elements must be live.
#define TFHIP_CHECK_RANGE(ptr, elems, esize, name)                             \
  do {                                                                         \
    if ((ptr) == nullptr || (long long)(elems) < 0 || (long long)(elems) > ::tfhip::kMaxElems || \
        !::tfhip::range_is_live((ptr), (size_t)(elems) * (esize)))             \
      return ::tfhip::fail(::tfhip::kOutOfRange,                               \
                           "%s: operand '%s' (%lld elements of %d bytes at %p) " \
                           "is not inside a live device buffer",               \
                           __func__, name, (long long)(elems), (int)(esize),   \
                           (const void *)(ptr));                               \
  } while (0)

// Operand `name` is about to be written: it must be live, and what the library remembered about its
// block's contents (filters searched for Inf / NaN) no longer holds.
#define TFHIP_CHECK_OUTPUT(ptr, elems, esize, name)       \
  do {                                                    \
    TFHIP_CHECK_RANGE(ptr, elems, esize, name);           \
    ::tfhip::forget_filter_scans(ptr);                    \
  } while (0)

// Checks the launch that was just enqueued.
#define TFHIP_CHECK_LAUNCH()  TFHIP_CHECK_HIP(hipGetLastError())

// Launch bookkeeping for measurement: the label of the kernel an entry point
// chose (as a profiler prints the symbol), and how many times each entry point
// enqueues its kernel (see tfhip_set_launch_repeat).
void note_kernel(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
int launch_repeat();

// Tuning overrides (tfhip_set_tuning, or TFHIP_<NAME> in the environment at
// tfhip_init): -1 when unset. One list names every knob: the enumerator, the
// name tfhip_set_tuning takes, and (in capitals behind TFHIP_) its environment variable.
#define TFHIP_TUNING_KNOBS(X)                                                                              \
  X(Tile, "tile") X(SplitK, "splitk") X(DwRows, "dw_rows") X(DwHalo, "dw_halo") X(NoSkinny, "no_skinny")    \
  X(SkinnyRegs, "skinny_regs") X(FusePwDw, "fuse_pw_dw")          \
  X(PwDwTile, "pw_dw_tile") X(TileSlice, "tile_slice") X(TileChunks, "tile_chunks")                         \
  X(FuseBlock, "fuse_block") X(KGroups, "k_groups") X(PwDwStream, "pw_dw_stream")                           \
  X(StreamRows, "stream_rows") X(StreamBlocks, "stream_blocks") X(SkinnyStage, "skinny_stage")              \
  X(BlockRows, "block_rows")
enum TuningKey {
#define TFHIP_TUNING_ENUM(id, name) kTune##id,
  TFHIP_TUNING_KNOBS(TFHIP_TUNING_ENUM)
#undef TFHIP_TUNING_ENUM
  kTuneCount
};
int tuning(int key);

// Enqueues `launch_expr` launch_repeat() times and checks the launch.
#define TFHIP_LAUNCH(launch_expr)                                  \
  do {                                                             \
    for (int r_ = ::tfhip::launch_repeat(); r_ > 0; --r_) {        \
      launch_expr;                                                 \
    }                                                              \
    TFHIP_CHECK_LAUNCH();                                          \
  } while (0)

// Largest element offset reached by a strided broadcast operand, plus one.
inline int64_t strided_extent(const int64_t *dims, const int64_t *strides, int rank) {
  int64_t last = 0;
  for (int i = 0; i < rank; ++i) {
    if (dims[i] <= 0) return 0;
    // (an extent beyond kMaxElems is no operand: say so without forming a product that could wrap)
    if (strides[i] < 0 || (dims[i] > 1 && strides[i] > kMaxElems / (dims[i] - 1))) return kMaxElems + 1;
    last += (dims[i] - 1) * strides[i];
    if (last > kMaxElems) return kMaxElems + 1;
  }
  return last + 1;
}

}  // namespace tfhip
