// Routing preprocessing: per-expert histogram, prefix-sum expert offsets and the
// stable sort of flat slot ids by expert id.  Replaces the argsort + histc +
// cumsum of the reference's get_token_indices (expert_permute.py:19-41) with a
// three-launch counting sort; all integer work, bit-exact by construction.
//
// The slot array is cut into chunks of CHUNK slots, one wavefront per chunk.
//   1. route_count : counts[c][e] = number of slots of chunk c routed to e
//   2. route_scan  : per expert, exclusive prefix over chunks + expert offset
//                    -> counts[c][e] becomes the first output position of
//                    (chunk c, expert e); writes group_indices
//   3. route_place : each wavefront walks its chunk in slot order, 64 slots a
//                    round; a lane's output position is the running offset of its
//                    expert plus the number of lower lanes with the same expert.
// Slots are placed in ascending slot order inside an expert, i.e. the stable sort.
#include "common.h"

#include <mutex>

namespace moe {
namespace {

constexpr int kWave = 64;
constexpr int kWavesPerBlock = 4;
constexpr int kChunk = 512;  // slots per wavefront
constexpr int kMaxExperts = 2048;

__device__ __forceinline__ int load_id(const void* ids, int idx_bytes, int64_t i) {
  int64_t v = load_index(ids, idx_bytes, i);
  return (v < 0 || v > 0x7fffffff) ? -1 : static_cast<int>(v);
}

__global__ __launch_bounds__(kWave* kWavesPerBlock) void route_count_kernel(
    const void* __restrict__ ids, int idx_bytes, int64_t R, int E, int32_t* __restrict__ counts) {
  extern __shared__ int32_t hist[];  // [kWavesPerBlock][E]
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int64_t chunk = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + wave;
  int32_t* my = hist + wave * E;
  for (int e = lane; e < E; e += kWave) my[e] = 0;
  __syncthreads();
  const int64_t begin = chunk * kChunk;
  for (int i = lane; i < kChunk; i += kWave) {
    int64_t s = begin + i;
    if (s < R) {
      int e = load_id(ids, idx_bytes, s);
      if (e >= 0 && e < E) atomicAdd(&my[e], 1);
    }
  }
  __syncthreads();
  if (begin < R) {
    for (int e = lane; e < E; e += kWave) counts[chunk * E + e] = my[e];
  }
}

// One block.  The chunk list of an expert is cut into P = blockDim / E parts (at most 64)
// that are summed in parallel, scanned per expert, and rewritten in parallel with their
// running offsets: a single thread per expert would walk R / 512 dependent loads (60 us at
// 100 000 slots and 64 experts).
__global__ __launch_bounds__(1024) void route_scan_kernel(int32_t* __restrict__ counts,
                                                          int64_t num_chunks, int E,
                                                          int32_t* __restrict__ group_indices,
                                                          int64_t* __restrict__ inclusive) {
  __shared__ int32_t partial[kMaxExperts];  // [P][E], P * E <= max(blockDim, E)
  __shared__ int32_t totals[kMaxExperts];
  __shared__ int32_t offsets[kMaxExperts + 1];
  const int nthreads = blockDim.x;
  int P = E >= nthreads ? 1 : nthreads / E;
  P = P > 64 ? 64 : P;
  const int64_t per = (num_chunks + P - 1) / P;
  const int items = E * P;
  for (int item = threadIdx.x; item < items; item += nthreads) {
    const int e = item % E, part = item / E;
    const int64_t c0 = part * per;
    const int64_t c1 = c0 + per < num_chunks ? c0 + per : num_chunks;
    int32_t sum = 0;
    for (int64_t c = c0; c < c1; ++c) sum += counts[c * E + e];
    partial[item] = sum;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += nthreads) {
    int32_t run = 0;
    for (int part = 0; part < P; ++part) {
      const int32_t v = partial[part * E + e];
      partial[part * E + e] = run;
      run += v;
    }
    totals[e] = run;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t run = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = run;
      run += totals[e];
    }
    offsets[E] = run;
  }
  __syncthreads();
  for (int e = threadIdx.x; e <= E; e += nthreads) {
    group_indices[e] = offsets[e];
    if (inclusive != nullptr && e > 0) inclusive[e - 1] = offsets[e];
  }
  // counts[c][e] becomes the first output position of (chunk c, expert e)
  for (int item = threadIdx.x; item < items; item += nthreads) {
    const int e = item % E, part = item / E;
    const int64_t c0 = part * per;
    const int64_t c1 = c0 + per < num_chunks ? c0 + per : num_chunks;
    int32_t run = offsets[e] + partial[item];
    for (int64_t c = c0; c < c1; ++c) {
      const int32_t v = counts[c * E + e];
      counts[c * E + e] = run;
      run += v;
    }
  }
}

__global__ __launch_bounds__(kWave* kWavesPerBlock) void route_place_kernel(
    const void* __restrict__ ids, int idx_bytes, int64_t R, int E,
    const int32_t* __restrict__ counts, int64_t* __restrict__ indices_out) {
  extern __shared__ int32_t next_pos[];  // [kWavesPerBlock][E]
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int64_t chunk = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + wave;
  const int64_t begin = chunk * kChunk;
  if (begin >= R) return;  // whole wavefront leaves; no block barrier below
  int32_t* my = next_pos + wave * E;
  for (int e = lane; e < E; e += kWave) my[e] = counts[chunk * E + e];
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");

  int bits = 0;
  while ((1 << bits) < E) ++bits;
  const uint64_t lower = (lane == 0) ? 0ull : (~0ull >> (kWave - lane));

  for (int i = 0; i < kChunk; i += kWave) {
    const int64_t s = begin + i + lane;
    int e = -1;
    if (s < R) {
      e = load_id(ids, idx_bytes, s);
      if (e >= E) e = -1;
    }
    const bool valid = e >= 0;
    // peers = lanes holding the same expert id, built from one ballot per id bit
    uint64_t peers = __ballot(valid);
    for (int b = 0; b < bits; ++b) {
      const bool bit = (e >> b) & 1;
      const uint64_t vote = __ballot(valid && bit);
      peers &= bit ? vote : ~vote;
    }
    if (valid) {
      const int rank = __popcll(peers & lower);
      const int32_t base = my[e];
      indices_out[base + rank] = s;
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      if (rank == 0) my[e] = base + __popcll(peers);
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  }
}

inline int64_t num_chunks_for(int64_t R) { return (R + kChunk - 1) / kChunk; }

}  // namespace
}  // namespace moe

extern "C" size_t moe_route_workspace_bytes(int64_t R, int E) {
  if (R < 0 || E <= 0) return 0;
  int64_t chunks = moe::num_chunks_for(R);
  if (chunks == 0) chunks = 1;
  return static_cast<size_t>(chunks) * static_cast<size_t>(E) * sizeof(int32_t);
}

namespace moe {
namespace {

// The three launches of the counting sort over a counts array of num_chunks * E words.
// Every word that is read has been written by route_count in the same call: nothing has to
// start at zero.
int route_preprocess_launch(const void* expert_ids, int idx_bytes, int64_t R, int E,
                            int64_t* indices_out, int32_t* group_indices_out,
                            int64_t* inclusive_out, int32_t* counts, hipStream_t stream) {
  const int64_t chunks = num_chunks_for(R);
  const unsigned blocks = static_cast<unsigned>((chunks + kWavesPerBlock - 1) / kWavesPerBlock);
  const size_t lds = static_cast<size_t>(kWavesPerBlock) * E * sizeof(int32_t);
  if (blocks > 0) {
    route_count_kernel<<<blocks, kWave * kWavesPerBlock, lds, stream>>>(expert_ids, idx_bytes, R, E,
                                                                       counts);
    if (int rc = check_launch("route_count")) return rc;
  }
  route_scan_kernel<<<1, 1024, 0, stream>>>(counts, chunks, E, group_indices_out, inclusive_out);
  if (int rc = check_launch("route_scan")) return rc;
  if (blocks > 0) {
    route_place_kernel<<<blocks, kWave * kWavesPerBlock, lds, stream>>>(expert_ids, idx_bytes, R, E,
                                                                       counts, indices_out);
    if (int rc = check_launch("route_place")) return rc;
  }
  return MOE_OK;
}

int check_route_args(const void* expert_ids, int idx_bytes, int64_t R, int E,
                     const int64_t* indices_out, const int32_t* group_indices_out) {
  MOE_REQUIRE(idx_bytes == 4 || idx_bytes == 8, "idx_bytes must be 4 or 8, got %d", idx_bytes);
  MOE_REQUIRE(R >= 0 && R <= 0x7fffffff, "R out of range: %lld", (long long)R);
  MOE_REQUIRE(E >= 1 && E <= kMaxExperts, "E must be in [1,%d], got %d", kMaxExperts, E);
  MOE_REQUIRE(group_indices_out != nullptr, "group_indices_out is null");
  MOE_REQUIRE(R == 0 || (expert_ids != nullptr && indices_out != nullptr),
              "expert_ids / indices_out is null");
  return MOE_OK;
}

// Scratch of moe_route_preprocess_noalloc: the counts array, resident in every device's copy of
// the library image until the process ends.  Host code never uses the array's name as an
// address: the device address is looked up once per device (scratch_of_current_device).
constexpr size_t kScratchWords = size_t(1) << 20;  // 4 MiB
static __device__ __align__(256) int32_t scratch[kScratchWords];

// One record per device: the buffer's address, and who used it last.  Eager calls from different
// streams would race on the buffer, so a call on another stream than the one before first makes
// its stream wait for an event recorded behind that call's launches: calls then run one after the
// other whatever streams they come from.  (Under graph capture nothing is recorded or waited for:
// the graph's replays are ordered by whoever launches them, see the header.)
struct ScratchOfDevice {
  int32_t* ptr = nullptr;
  hipEvent_t done = nullptr;     // behind the launches of the last eager call
  hipStream_t last = nullptr;    // the stream of that call
  bool used = false;
};
constexpr int kMaxScratchDevices = 64;
ScratchOfDevice g_scratch_of[kMaxScratchDevices];
std::mutex g_scratch_lock;

// The buffer of the current device for a call on `stream`, or nullptr (error set).  The first call
// on a device looks the address up (which may load the code object) and creates the event; that is
// not done while `stream` is being captured into a graph: such a call is refused, and the caller
// makes one call outside the capture first.  *capturing tells whether `stream` is being captured.
// The caller holds g_scratch_lock from here until release_scratch has returned, so that two host
// threads cannot both pass the wait for the call before them and then launch side by side.
int32_t* acquire_scratch(hipStream_t stream, ScratchOfDevice** rec, bool* capturing) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess || dev < 0 || dev >= kMaxScratchDevices) {
    fail(MOE_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(err));
    return nullptr;
  }
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  err = hipStreamIsCapturing(stream, &capture);
  if (err != hipSuccess) {
    fail(MOE_ERR_HIP, "hipStreamIsCapturing: %s", hipGetErrorString(err));
    return nullptr;
  }
  *capturing = capture != hipStreamCaptureStatusNone;
  ScratchOfDevice& d = g_scratch_of[dev];
  if (d.ptr == nullptr) {
    if (*capturing) {
      fail(MOE_ERR_HIP, "the first moe_route_preprocess_noalloc call on a device looks up its "
                        "resident buffer and cannot run under stream capture: make one call "
                        "(any size, R = 0 will do) before the capture begins");
      return nullptr;
    }
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess || p == nullptr) {
      fail(MOE_ERR_HIP, "hipGetSymbolAddress(routing scratch): %s", hipGetErrorString(err));
      return nullptr;
    }
    err = hipEventCreateWithFlags(&d.done, hipEventDisableTiming);
    if (err != hipSuccess) {
      fail(MOE_ERR_HIP, "hipEventCreateWithFlags: %s", hipGetErrorString(err));
      return nullptr;
    }
    d.ptr = static_cast<int32_t*>(p);
  }
  if (!*capturing && d.used && d.last != stream) {
    err = hipStreamWaitEvent(stream, d.done, 0);
    if (err != hipSuccess) {
      fail(MOE_ERR_HIP, "hipStreamWaitEvent: %s", hipGetErrorString(err));
      return nullptr;
    }
  }
  *rec = &d;
  return d.ptr;
}

// Behind the launches of an eager call.
int release_scratch(ScratchOfDevice* rec, hipStream_t stream) {
  const hipError_t err = hipEventRecord(rec->done, stream);
  if (err != hipSuccess) return fail(MOE_ERR_HIP, "hipEventRecord: %s", hipGetErrorString(err));
  rec->last = stream;
  rec->used = true;
  return MOE_OK;
}

}  // namespace
}  // namespace moe

extern "C" int moe_route_preprocess(const void* expert_ids, int idx_bytes, int64_t R, int E,
                                    int64_t* indices_out, int32_t* group_indices_out,
                                    int64_t* inclusive_out, void* workspace,
                                    size_t workspace_bytes, moe_stream_t stream_) {
  using namespace moe;
  clear_error();
  if (int rc = check_route_args(expert_ids, idx_bytes, R, E, indices_out, group_indices_out)) return rc;
  if (workspace == nullptr || workspace_bytes < moe_route_workspace_bytes(R, E))
    return fail(MOE_ERR_WORKSPACE, "routing workspace needs %zu bytes, got %zu",
                moe_route_workspace_bytes(R, E), workspace_bytes);
  return route_preprocess_launch(expert_ids, idx_bytes, R, E, indices_out, group_indices_out,
                                 inclusive_out, static_cast<int32_t*>(workspace),
                                 static_cast<hipStream_t>(stream_));
}

extern "C" size_t moe_route_noalloc_max_bytes(void) { return moe::kScratchWords * sizeof(int32_t); }

extern "C" int moe_route_preprocess_noalloc(const void* expert_ids, int idx_bytes, int64_t R, int E,
                                            int64_t* indices_out, int32_t* group_indices_out,
                                            int64_t* inclusive_out, moe_stream_t stream_) {
  using namespace moe;
  clear_error();
  if (int rc = check_route_args(expert_ids, idx_bytes, R, E, indices_out, group_indices_out)) return rc;
  const size_t need = moe_route_workspace_bytes(R, E);
  if (need > kScratchWords * sizeof(int32_t))
    return fail(MOE_ERR_WORKSPACE,
                "routing of %lld slots over %d experts needs %zu bytes of scratch; the resident "
                "buffer of moe_route_preprocess_noalloc has %zu (use moe_route_preprocess with a "
                "workspace)", (long long)R, E, need, kScratchWords * sizeof(int32_t));
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  ScratchOfDevice* rec = nullptr;
  bool capturing = false;
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  int32_t* const counts = acquire_scratch(stream, &rec, &capturing);
  if (counts == nullptr) return MOE_ERR_HIP;
  const int rc = route_preprocess_launch(expert_ids, idx_bytes, R, E, indices_out, group_indices_out,
                                         inclusive_out, counts, stream);
  if (rc != MOE_OK || capturing) return rc;
  return release_scratch(rec, stream);
}
