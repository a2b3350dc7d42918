// internal.h -- shared declarations of the hvdhip library (not installed).
#ifndef HVDHIP_INTERNAL_H
#define HVDHIP_INTERNAL_H

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdint>
#include <cstdio>
#include <string>
#include <tuple>
#include <type_traits>
#include <vector>

#include "hvdhip.h"

namespace hvdhip {

// Records a message for hvdhip_last_error() on the calling thread and returns code.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// Clears the calling thread's message; returns 0.
int ok();

// Evaluates a HIP call; on failure records "<call> failed: <text>" and returns
// the hipError_t value from the enclosing function.
#define HVDHIP_CHECK(call)                                                          \
  do {                                                                              \
    hipError_t hvdhip_e_ = (call);                                                  \
    if (hvdhip_e_ != hipSuccess) {                                                  \
      (void)hipGetLastError(); /* the code is returned; leave no stale error behind */ \
      return ::hvdhip::fail((int)hvdhip_e_, "%s failed: %s", #call,                 \
                            hipGetErrorString(hvdhip_e_));                          \
    }                                                                               \
  } while (0)

// Checks the status that launch() returned for the kernel `name`.  Only that value is looked at:
// the thread's last-error state belongs to the application and is neither read nor cleared.
#define HVDHIP_CHECK_LAUNCH(name, status)                                           \
  do {                                                                              \
    hipError_t hvdhip_e_ = (status);                                                \
    if (hvdhip_e_ != hipSuccess)                                                    \
      return ::hvdhip::fail((int)hvdhip_e_, "%s launch failed: %s", name,           \
                            hipGetErrorString(hvdhip_e_));                          \
  } while (0)

inline int64_t dtype_size(int dtype) {
  switch (dtype) {
  case HVDHIP_UINT8: case HVDHIP_INT8: case HVDHIP_BOOL: return 1;
  case HVDHIP_UINT16: case HVDHIP_INT16: case HVDHIP_FLOAT16: return 2;
  case HVDHIP_INT32: case HVDHIP_FLOAT32: return 4;
  case HVDHIP_INT64: case HVDHIP_FLOAT64: return 8;
  default: return -1;
  }
}

// The fp32 factor that an fp16 scale multiplies by under the current fp16 scale mode:
// (float)scale, or that value rounded to half (nearest even) and widened again.
float fp16_scale_factor(double scale);

// Threads per workgroup of every streaming kernel: four wave64 wavefronts.  (Workgroups of 64, 128,
// 512 and 1,024 lanes measured 0-9 % slower.)
constexpr int kWG = 256;
static_assert(kWG % 64 == 0 && kWG >= 64 && kWG <= 1024, "whole wave64 wavefronts");

// A launch may not exceed 2^32 - 1 threads in x.  Contiguous kernels cover larger buffers
// in slices of kMaxWorkgroups workgroups; a plan that needs more is refused.
constexpr uint64_t kMaxWorkgroups = 1ull << 23;

// Bytes of the wider side that one workgroup moves.  Measured on MI355X with
// buffers far larger than the 256 MB Infinity Cache: one 16-byte access per
// lane and workgroup (4 KiB) with non-temporal hints streams at about 80 % of
// the HBM peak, against about 70 % for 16-32 KiB per workgroup; the occupancy
// of many small workgroups hides latency better than unrolling inside one.
// The Adasum reduction pays a workgroup-wide tree per chunk and prefers 16 KiB.
// (A build with -DHVDHIP_TUNING reads HVDHIP_CHUNK_BYTES to override all of them; the shipped
// library reads nothing.)
enum class Family { kXfer, kXferNarrowing, kUnpack, kReduce, kAdasum };
constexpr uint32_t kXferChunkBytes = 4096;
constexpr uint32_t kXferNarrowingChunkBytes = 8192;  // fp32 -> fp16 pack: 32 bytes in, 16 out per lane
constexpr uint32_t kUnpackChunkBytes = 4096;  // every unpack, same-width or widening (a plan keeps a second table when this differs from its pack's)
constexpr uint32_t kReduceChunkBytes = 4096;
constexpr uint32_t kAdasumChunkBytes = 16384;
uint32_t chunk_bytes(Family f);

// Workgroups are handed to the eight XCDs of the device in turn (workgroup p runs on XCD p % 8),
// each XCD with an L2 and address-translation cache of its own.  Streaming is a little faster
// (1.5-2.5 % on the pack and unpack kernels, up to 5 % on the widening unpack) when one XCD walks
// runs of consecutive chunks instead of every eighth chunk, so tables and tile numbers are laid out
// accordingly: within each group of 8 * run chunks, XCD x gets chunks x * run .. x * run + run - 1.
// The ragged end (fewer than 8 * run chunks) keeps its natural order.  What counts is the length of
// a run in bytes.  Measured against natural order: 256 KiB per run is best for launches of 16-128
// MiB (+2-5 % on every kernel family; 128 KiB - 1 MiB are close, a single chunk and >= 4 MiB gain
// nothing) but costs 2-6 % at 512 MiB and more, where 1 MiB gains 1-3 % and 4 MiB loses 4-6 %; so
// launches that cover more than kXcdLongRunFrom bytes use the longer run.
constexpr uint32_t kXcds = 8;
constexpr uint32_t kXcdRunBytes = 256u << 10;
constexpr uint32_t kXcdLongRunBytes = 1u << 20;
constexpr uint64_t kXcdLongRunFrom = 128ull << 20;
// Run length in chunks for a launch of nchunks chunks of chunk_bytes each (at least one chunk).
// The Adasum kernels (two read streams of 16 KiB chunks) do best with the longer run at every size
// (2 x 16 MiB: 13.9 against 14.2 us, 2 x 64 MiB: 53.0 against 54.2 us): long_runs asks for it.
uint32_t xcd_run(uint64_t nchunks, uint32_t chunk_bytes, bool long_runs = false);
// Chunk (or tile) that the workgroup at table position `slot` handles.
__host__ __device__ inline uint64_t xcd_chunk(uint64_t slot, uint64_t nchunks, uint32_t run) {
  const uint64_t group = (uint64_t)kXcds * run;
  if (run == 0 || slot >= nchunks / group * group) return slot;
  const uint64_t w = slot % group;
  return slot - w + (w % kXcds) * run + w / kXcds;
}
// Table position of chunk `chunk`: the inverse of xcd_chunk.
__host__ __device__ inline uint64_t xcd_slot(uint64_t chunk, uint64_t nchunks, uint32_t run) {
  const uint64_t group = (uint64_t)kXcds * run;
  if (run == 0 || chunk >= nchunks / group * group) return chunk;
  const uint64_t w = chunk % group;
  return chunk - w + (w % run) * kXcds + w / run;
}

// The same mapping for kernels that number their tiles themselves, in shifts and masks and without a
// branch (nothing may stand between a workgroup's start and its first loads): the first `ordered`
// workgroups (a multiple of 8 << shift, 0 for natural order) are permuted in groups of 8 << shift.
struct XcdOrder {
  uint32_t shift;    // log2 of the run length in tiles
  uint32_t ordered;  // workgroups below this number are permuted
};
XcdOrder xcd_order(uint64_t nblocks, uint32_t tile_bytes);
__device__ __forceinline__ uint32_t xcd_tile(uint32_t block, XcdOrder o) {
  const uint32_t mask = (kXcds << o.shift) - 1;  // group of 8 * run tiles
  const uint32_t w = block & mask;
  const uint32_t permuted = block - w + ((w & (kXcds - 1)) << o.shift) + (w >> 3);
  return block < o.ordered ? permuted : block;
}

// Launches a streaming kernel: workgroups of kWG lanes, no dynamic LDS.  The arguments are
// converted to the kernel's own parameter types and handed over by address; the kernel is named
// by its host-side handle, never called through the pointer (a call through a pointer depends on
// the compiler turning the handle into the launch stub at that call, which a host build with
// -fsanitize=function does not do for a kernel that is not a template: its launches vanish
// without an error).  Returns the launch call's own status, for HVDHIP_CHECK_LAUNCH.
// completion: an event to be bound to the kernel's completion signal (the launch's stop event).
template <typename... KArgs, typename... Args>
inline hipError_t launch_with(hipEvent_t completion, void (*kernel)(KArgs...), uint32_t workgroups,
                              hipStream_t stream, Args... args) {
  static_assert(sizeof...(KArgs) == sizeof...(Args), "one argument per kernel parameter");
  std::tuple<KArgs...> values{KArgs(args)...};
  void* addresses[sizeof...(KArgs) ? sizeof...(KArgs) : 1];
  std::apply([&](auto&... v) { size_t i = 0; ((addresses[i++] = static_cast<void*>(&v)), ...); }, values);
  const void* handle = reinterpret_cast<const void*>(kernel);
  if (completion)
    return hipExtLaunchKernel(handle, dim3(workgroups), dim3(kWG), addresses, 0, stream, nullptr, completion, 0);
  return hipLaunchKernel(handle, dim3(workgroups), dim3(kWG), addresses, 0, stream);
}
template <typename... KArgs, typename... Args>
inline hipError_t launch(void (*kernel)(KArgs...), uint32_t workgroups, hipStream_t stream, Args... args) {
  return launch_with(nullptr, kernel, workgroups, stream, args...);
}

// Store policy per kernel family (the three kinds of store are described in vecmem.h).  Lines
// written through are installed in the 256 MB Infinity Cache on their way to HBM, so a kernel that
// runs next on the same stream and reads them (the collective or reduce-sum after a pack, the unpack
// after a reduce-sum) finds them there; non-temporal stores bypass it.  Installing costs the writer
// something (a stress-workload pack launched back to back with nothing reading its output: 18.0
// instead of 16.3 us) and saves the reader more (the unpack behind it: 12 instead of 16.4 us), so the
// kernels whose output the next kernel reads write through, and the ones whose output leaves the
// pipeline (unpack, batched copies, Adasum's scaled add, a whole-buffer scale) do not.
// (A build with -DHVDHIP_TUNING reads HVDHIP_WRITE_THROUGH=<mask>, bit = enumerator value, to
// override the built-in table; the shipped library reads nothing.)
enum class Stores {
  kPack = 0,        // same-width pack into the fusion buffer
  kUnpack = 1,      // same-width unpack out of it
  kDirect = 2,      // tensor to tensor (batched copies, allgather)
  kPackNarrowing = 3,   // fp32 -> fp16 pack
  kUnpackWidening = 4,  // fp16 -> fp32 unpack
  kContig = 5,      // whole-buffer scale
  kReduceFew = 6,   // reduce-sum of one or two peers
  kReduceMany = 7,  // reduce-sum of three to eight peers
  kAdasum = 8,      // scaled add
};
int store_policy(Stores family);  // a StorePolicy value

// Calls f(std::integral_constant<int, policy>) for the family's policy and returns what it returns.
template <typename F>
inline auto with_store_policy(Stores family, F&& f) {
  if (store_policy(family)) return f(std::integral_constant<int, 1>());
  return f(std::integral_constant<int, 0>());
}

// One contiguous run of elements to transfer (host side only).  `tensor` and
// `output` are absolute device addresses; `off` is a byte offset into the
// fusion buffer whose base address is given at launch.  `n` counts elements.
struct Seg {
  uint64_t tensor;
  uint64_t output;
  uint64_t off;
  uint64_t n;
};

// Where workgroup b finds its entry in a transfer table.  Four 32-byte entries share a 128-byte
// cache line, and workgroups b, b + 1, b + 2, b + 3 run on four different XCDs, each with an L2 of
// its own: read in workgroup order, every line is fetched from memory four times (128 bytes per
// workgroup for a 32-byte entry, +1.6 % read traffic on a 4 KiB chunk).  So within each group of
// 32 workgroups the four that share an XCD (b, b + 8, b + 16, b + 24: consecutive on that XCD)
// read the four entries of one line.  Tables are padded to a multiple of 32 entries with empty
// chunks (n = 0), and that many workgroups are launched, so the mapping needs no bounds check and
// no argument: nothing stands between a workgroup's start and the load of its entry but three
// scalar instructions.
constexpr uint32_t kLineGroup = 32;
inline uint64_t table_slots(uint64_t nchunks) { return (nchunks + kLineGroup - 1) / kLineGroup * kLineGroup; }
__host__ __device__ inline uint32_t line_slot(uint32_t b) { return (b & ~31u) | ((b & 7u) << 2) | ((b >> 3) & 3u); }

// One workgroup's share, self-contained so that a workgroup needs a single
// 32-byte scalar load before it can issue its data loads.  All three
// locations already point at the chunk's first element.
struct Chunk {
  uint64_t tensor;  // absolute address on the tensor side
  uint64_t output;  // absolute address on the output side
  uint64_t off;     // byte offset into the fusion buffer
  uint32_t n;       // elements in this chunk
  uint32_t pad;     // bytes to zero after the chunk in the fusion buffer (last chunk of a tensor)
};
static_assert(sizeof(Chunk) == 32, "Chunk is loaded as eight dwords");

// Device-resident chunk table of one plan.
struct DevTables {
  void* alloc = nullptr;
  Chunk* chunks = nullptr;
  uint32_t nchunks = 0;  // chunks with work in them
  uint32_t nlaunch = 0;  // entries in the table = workgroups to launch (transfer tables: padded to 32)
};

// Cuts every segment into chunks of at most chunk_units elements and uploads
// the table (allocates; synchronous).  tensor_es / buffer_es are the element
// sizes on the tensor/output side and on the fusion-buffer side.  Zero-length
// segments get no chunk.
int build_tables(const std::vector<Seg>& segs, uint32_t chunk_units, uint32_t tensor_es,
                 uint32_t buffer_es, DevTables* out);
// The two halves of build_tables for callers that stage the table themselves:
// the number of chunks the segments need (0xffffffffffffffff if over the
// limit), and the fill of a caller-provided array of table_slots(nchunks) entries: XCD order,
// each at the line_slot of its workgroup, the rest empty.
uint64_t count_chunks(const std::vector<Seg>& segs, uint32_t chunk_units);
void fill_chunks(const std::vector<Seg>& segs, uint32_t chunk_units, uint32_t tensor_es,
                 uint32_t buffer_es, Chunk* out, uint64_t nchunks);
// Makes `device` current for its lifetime when another one is, and puts the old one back.
// Plans and cached tables belong to the device that was current when they were made; their
// teardown must wait for and free on that device whatever the caller has selected since.
class DeviceGuard {
 public:
  explicit DeviceGuard(int device) {
    if (hipGetDevice(&prev_) == hipSuccess && prev_ != device && hipSetDevice(device) == hipSuccess) switched_ = true;
  }
  ~DeviceGuard() {
    if (switched_) (void)hipSetDevice(prev_);
  }
  DeviceGuard(const DeviceGuard&) = delete;
  DeviceGuard& operator=(const DeviceGuard&) = delete;

 private:
  int prev_ = 0;
  bool switched_ = false;
};

// Tells the copy-table caches that `stream` has been synchronised and is about to be destroyed.
void copy_cache_forget_stream(hipStream_t stream);
// Destroys the single-layer Adasum plans kept for `stream` (idle, about to be destroyed).
void adasum_forget_stream(hipStream_t stream);

// Uploads a ready-made chunk table; every entry is launched (nlaunch = nchunks = its size).
int upload_chunks(const std::vector<Chunk>& chunks, DevTables* out);
int free_tables(DevTables* t);

}  // namespace hvdhip

#endif  // HVDHIP_INTERNAL_H
