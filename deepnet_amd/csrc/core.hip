// Handle lifetime, device memory, transfers, views, row slices and transpose.
// Replaces cudamat/cudamat.cu:25-53, 87-123, 153-186, 217-434 and the copy
// kernels cudamat_kernels.cu:247-294.
#include "common.h"
#include <vector>
#include <unordered_map>
#include <stdio.h>
#include <string.h>

static int g_num_cus = 0;

int dn_num_cus() {
  if (g_num_cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
      g_num_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    else
      g_num_cus = 256;
  }
  return g_num_cus;
}

// ------------------------------------------------------------------ launch stream and graph capture
static hipStream_t g_stream = nullptr;     // nullptr: the NULL stream
static bool g_capturing = false;
static hipStream_t g_capture_stream = nullptr;

static int g_live_graphs = 0;
static void (*g_no_graphs_hook)() = nullptr;
void dn_set_no_graphs_hook(void (*f)()) { g_no_graphs_hook = f; }

// A product whose launch is held back so that the calls that follow it can ride in its
// epilogue (see "deferred epilogues" in elementwise.hip).  Everything that queues work, hands
// out a workspace, moves data or waits for the device comes through dn_flush() first.
static bool g_pending = false;
static void (*g_flush_hook)() = nullptr;
void dn_set_flush_hook(void (*f)()) { g_flush_hook = f; }
void dn_set_pending(bool on) { g_pending = on; }
// The conv library holds calls back in the same way (a MaxPool that a ResponseNorm may follow); it
// has its own flag and hook.  Whoever holds a call back launches what the other side holds first,
// so at most one of the two is set at any time.
static bool g_ext_pending = false;
static void (*g_ext_flush_hook)() = nullptr;
void dn_set_ext_flush_hook(void (*f)()) { g_ext_flush_hook = f; }
void dn_set_ext_pending(bool on) { g_ext_pending = on; }
void dn_flush_ext() {
  if (g_ext_pending) {
    g_ext_pending = false;
    if (g_ext_flush_hook) g_ext_flush_hook();
  }
}
void dn_flush() {
  if (g_pending) {
    g_pending = false;
    if (g_flush_hook) g_flush_hook();
  }
  dn_flush_ext();
}

hipStream_t dn_stream() {
  if (g_pending || g_ext_pending) dn_flush();
  return g_stream;
}
bool dn_capturing() { return g_capturing; }

// ------------------------------------------------------------------ scratch
// Grow-only device workspaces.  Slot 0: partials of two-stage reductions and
// split-K products, scalar results.  Slot 1: the patch matrix of the col2im
// form of convDown (it is live while a product that may use slot 0 runs).  Slot 2:
// batch-padded copies of conv operands (live across a whole conv call).  Slot 3: the same
// for operands padded to a multiple of 16 filters.
static void* g_scratch[4] = {nullptr, nullptr, nullptr, nullptr};
static size_t g_scratch_bytes[4] = {0, 0, 0, 0};
static bool g_scratch_recorded[4] = {false, false, false, false};
static std::vector<void*>& g_retired = *new std::vector<void*>;   // outgrown blocks that a recorded graph may still use

static void block_flush();

// hipMalloc for the library's own workspaces: when the device is out of memory, the blocks that
// free_device_memory keeps for reuse are given back first and the request is made again.
hipError_t dn_malloc(void** p, size_t bytes) {
  dn_flush();
  hipError_t e = hipMalloc(p, bytes);
  if (e != hipSuccess) {
    hipGetLastError();
    hipDeviceSynchronize();
    block_flush();
    e = hipMalloc(p, bytes);
    if (e != hipSuccess) { hipGetLastError(); *p = nullptr; }
  }
  return e;
}

void* dn_scratch(size_t bytes, int slot) {
  dn_flush();      // (a held-back product may take, and grow, a workspace of its own when it is launched)
  if (bytes > g_scratch_bytes[slot]) {
    if (g_capturing) return nullptr;   // growing means freeing and allocating: not while a graph is recorded

    if (g_scratch[slot]) {
      hipDeviceSynchronize();
      // A block that was handed out while a graph was being recorded stays allocated: the
      // graph's kernels carry its address (it is freed with the last graph of this library;
      // a library that only joins recordings keeps it for the life of the process).
      if (g_scratch_recorded[slot]) g_retired.push_back(g_scratch[slot]);
      else hipFree(g_scratch[slot]);
      g_scratch_recorded[slot] = false;
    }
    size_t want = bytes < (1u << 20) ? (1u << 20) : bytes;
    if (dn_malloc(&g_scratch[slot], want) != hipSuccess) {
      g_scratch[slot] = nullptr;
      g_scratch_bytes[slot] = 0;
      return nullptr;
    }
    g_scratch_bytes[slot] = want;
  }
  if (g_capturing) g_scratch_recorded[slot] = true;
  return g_scratch[slot];
}

// ------------------------------------------------------------------ matrix memory
// Matrices come from hipMalloc, one allocation each, as in the reference (cublasAlloc).
// hipFree waits for the device, which stalls code that makes a temporary per step
// (x = cm.dot(a, b); ...; del x: 19 us for two launches and a temporary, 10 us without the wait),
// so a freed block is kept for the next request of exactly its size instead: everything
// the library does is queued on one stream, a block's next owner can only touch it after
// the kernels of the previous one.  At most DN_CACHE_BYTES are kept (a block that would
// exceed them is freed at once); an allocation that fails frees them all and tries again.
#define DN_CACHE_BYTES ((size_t)4 << 30)
// (on the heap and never destroyed: matrices may still be freed while the process exits)
static std::unordered_map<void*, size_t>& g_block_bytes = *new std::unordered_map<void*, size_t>;   // blocks handed out by block_get
static std::unordered_map<size_t, std::vector<void*>>& g_block_cache = *new std::unordered_map<size_t, std::vector<void*>>;   // free blocks by size
static size_t g_cached_bytes = 0;

static void block_flush() {
  for (auto& kv : g_block_cache)
    for (void* p : kv.second) hipFree(p);
  g_block_cache.clear();
  g_cached_bytes = 0;
}

static void* block_get(size_t bytes) {
  void* p = nullptr;
  auto it = g_block_cache.find(bytes);
  if (it != g_block_cache.end() && !it->second.empty()) {
    p = it->second.back();
    it->second.pop_back();
    g_cached_bytes -= bytes;
  } else if (dn_malloc(&p, bytes) != hipSuccess) {
    return nullptr;
  }
  g_block_bytes[p] = bytes;
  return p;
}

// false when the runtime refuses to free the block
static bool block_put(void* p) {
  dn_flush();
  auto it = g_block_bytes.find(p);
  if (it == g_block_bytes.end()) return hipFree(p) == hipSuccess;      // not one of ours (a caller's own allocation)
  const size_t bytes = it->second;
  g_block_bytes.erase(it);
  if (g_cached_bytes + bytes > DN_CACHE_BYTES) return hipFree(p) == hipSuccess;
  g_block_cache[bytes].push_back(p);
  g_cached_bytes += bytes;
  return true;
}

// A block of 32-bit words that is zero whenever no kernel of the library is running (arrival
// counters that their kernels return to zero); allocated and cleared on first use.
static unsigned* g_zero_words = nullptr;
static int g_zero_words_n = 0;
static bool g_zero_words_recorded = false;

unsigned* dn_zero_words(int n) {
  dn_flush();
  if (n > g_zero_words_n) {
    if (g_capturing) return nullptr;
    if (g_zero_words) {
      hipDeviceSynchronize();
      if (g_zero_words_recorded) g_retired.push_back(g_zero_words);   // (as for the scratch blocks)
      else hipFree(g_zero_words);
      g_zero_words_recorded = false;
      g_zero_words = nullptr;
      g_zero_words_n = 0;
    }
    const int want = n < 16384 ? 16384 : n;
    if (dn_malloc((void**)&g_zero_words, (size_t)want * sizeof(unsigned)) != hipSuccess) { g_zero_words = nullptr; return nullptr; }
    if (hipMemset(g_zero_words, 0, (size_t)want * sizeof(unsigned)) != hipSuccess) return nullptr;
    g_zero_words_n = want;
  }
  if (g_capturing) g_zero_words_recorded = true;
  return g_zero_words;
}

// ------------------------------------------------------------------ kernels

// Column-major row-band copy: dst(r, c) = src(r + row0, c) for a band of `rows`
// rows; threads run down a column so both sides are read/written in 256-byte
// runs.  src_ld / dst_ld are the two leading dimensions.
__global__ void k_copy_rows(const float* src, float* dst, int rows, int cols, int src_ld, int dst_ld,
                            int src_row0, int dst_row0) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  for (int c = blockIdx.y; c < cols; c += gridDim.y)
    dst[(size_t)c * dst_ld + dst_row0 + r] = src[(size_t)c * src_ld + src_row0 + r];
}

// Out-of-place transpose through a 64x64 LDS tile (+1 column of padding so the
// transposed read walks distinct banks).  in is h x w column-major, out is w x h.
#define TR_TILE 64
__global__ void __launch_bounds__(256) k_transpose(const float* in, float* out, int h, int w) {
  __shared__ float tile[TR_TILE][TR_TILE + 1];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
  const int r0 = blockIdx.x * TR_TILE, c0 = blockIdx.y * TR_TILE;
#pragma unroll
  for (int j = ty; j < TR_TILE; j += 4) {
    const int r = r0 + tx, c = c0 + j;
    if (r < h && c < w) tile[j][tx] = in[(size_t)c * h + r];
  }
  __syncthreads();
#pragma unroll
  for (int j = ty; j < TR_TILE; j += 4) {
    const int c = c0 + tx, r = r0 + j;  // out(c, r) = in(r, c)
    if (r < h && c < w) out[(size_t)r * w + c] = tile[tx][j];
  }
}

// The same for 16-byte aligned matrices whose sides are multiples of 4: every lane moves
// 16 bytes per access on both sides (a quarter of the memory instructions; the transposes
// of the conv stage are latency-bound), the tile is turned around in LDS one float at a
// time.  Lane t: 4 consecutive rows 4*(t%16).. of column t/16 + 16*u on the way in,
// 4 consecutive columns of row t/16 + 16*u of the tile on the way out.
__global__ void __launch_bounds__(256) k_transpose4(const float* in, float* out, int h, int w) {
  __shared__ float tile[TR_TILE][TR_TILE + 1];   // [column][row]
  const int q = (threadIdx.x & 15) * 4, p = threadIdx.x >> 4;
  const int r0 = blockIdx.x * TR_TILE, c0 = blockIdx.y * TR_TILE;
  float4 v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int r = r0 + q, c = c0 + p + 16 * u;
    v[u] = (r < h && c < w) ? *reinterpret_cast<const float4*>(in + (size_t)c * h + r) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    float* t = &tile[p + 16 * u][q];
    t[0] = v[u].x; t[1] = v[u].y; t[2] = v[u].z; t[3] = v[u].w;
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int r = r0 + p + 16 * u, c = c0 + q;     // out(c, r) = in(r, c), contiguous along c
    if (r < h && c < w) {
      const int lr = p + 16 * u;
      *reinterpret_cast<float4*>(out + (size_t)r * w + c) =
          make_float4(tile[q][lr], tile[q + 1][lr], tile[q + 2][lr], tile[q + 3][lr]);
    }
  }
}

// ------------------------------------------------------------------ C ABI

extern "C" {

const char* get_last_cuda_error(void) { return hipGetErrorString(hipGetLastError()); }

int cublas_init(void) {
  // Nothing to create: the contraction kernels are part of this library.  Touch
  // the device so a missing GPU is reported here rather than at the first op.
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) return CUBLAS_ERROR;
  // the fixed workspace of the entry points that allocate nothing, for the current device
  if (dn_noalloc_setup() == CUDA_ERROR) return CUBLAS_ERROR;
  return 0;
}

int cublas_shutdown(void) {
  dn_flush();
  hipDeviceSynchronize();
  block_flush();
  return 0;
}

int cuda_set_device(int deviceId) {
  dn_flush();
  int before = -1;
  hipGetDevice(&before);
  if (hipSetDevice(deviceId) != hipSuccess) return CUDA_ERROR;
  g_num_cus = 0;
  if (before != deviceId && before >= 0) {
    // the workspaces live in the memory of the device that was current when they were made
    hipSetDevice(before);
    hipDeviceSynchronize();
    block_flush();
    for (int slot = 0; slot < 4; ++slot) {
      if (g_scratch[slot]) hipFree(g_scratch[slot]);
      g_scratch[slot] = nullptr;
      g_scratch_bytes[slot] = 0;
      g_scratch_recorded[slot] = false;
    }
    if (g_zero_words) hipFree(g_zero_words);
    g_zero_words = nullptr;
    g_zero_words_n = 0;
    g_zero_words_recorded = false;
    hipSetDevice(deviceId);
  }
  return 0;
}

void cuda_sync_threads(void) {
  dn_flush();
  if (!g_capturing) hipDeviceSynchronize();
}

// ---- HIP graphs (no counterpart in the reference): record a fixed sequence of library calls
// once and replay it with one launch, for steps whose cost is the launching itself.
// Small results (a loss, a vector of counts: up to 64 KiB) reach the host through a pinned
// block that one workgroup fills: its lanes store the data, meet at a barrier, and one lane
// then makes the stores visible to the host (a release fence at system scope) and writes
// this call's tag; the host polls the tag and copies the data out.  One launch and no wait
// on the stream: 7.5 us where the runtime's copy call takes 12.
#define DN_STAGE_FLOATS 16384
#define DN_STAGE_POLLS (1 << 16)
struct DnStage {
  unsigned long long tag;          // written last by the kernel
  char pad[248];
  float data[DN_STAGE_FLOATS];
};
static DnStage* g_stage_host = nullptr;
static DnStage* g_stage_dev = nullptr;
static unsigned long long g_stage_tag = 0;

__global__ void __launch_bounds__(1024) k_stage_out(const float* src, DnStage* stage, int n, unsigned long long tag) {
  for (int i = threadIdx.x; i < n; i += 1024) stage->data[i] = src[i];
  __syncthreads();
  if (threadIdx.x == 0) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
    __hip_atomic_store(&stage->tag, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

static bool stage_out(const float* src, float* host, int n) {
  if (!g_stage_host) {
    void* h = nullptr;
    void* d = nullptr;
    if (hipHostMalloc(&h, sizeof(DnStage), hipHostMallocCoherent | hipHostMallocMapped) != hipSuccess) { hipGetLastError(); return false; }
    if (hipHostGetDevicePointer(&d, h, 0) != hipSuccess) { hipGetLastError(); hipHostFree(h); return false; }
    g_stage_host = (DnStage*)h;
    g_stage_dev = (DnStage*)d;
    g_stage_host->tag = 0;
  }
  const unsigned long long tag = ++g_stage_tag;
  hipLaunchKernelGGL(k_stage_out, dim3(1), dim3(1024), 0, dn_stream(), src, g_stage_dev, n, tag);
  if (hipGetLastError() != hipSuccess) return false;
  bool seen = false;
  for (int i = 0; i < DN_STAGE_POLLS && !seen; ++i) seen = __atomic_load_n(&g_stage_host->tag, __ATOMIC_ACQUIRE) == tag;
  if (!seen) {
    if (hipStreamSynchronize(g_stream) != hipSuccess) return false;
    if (__atomic_load_n(&g_stage_host->tag, __ATOMIC_ACQUIRE) != tag) return false;
  }
  memcpy(host, g_stage_host->data, (size_t)n * sizeof(float));
  return true;
}

// graph_capture_begin() switches the library to a capturing stream: every call until
// graph_capture_end() is recorded instead of run (with the pointers and scalars it was given).
// What cannot be recorded fails with its usual error code: calls that wait for the device
// (copy_to_host, vdot, euclid_norm) and workspaces that would have to grow (run the sequence
// once before recording it).  The random generator's state lives on the device, so every
// replay draws fresh numbers.  graph_launch() queues a replay on the NULL stream, in order with
// everything else the library does.
void* graph_capture_begin(void) {
  if (g_capturing) return nullptr;
  dn_flush();
  if (!g_capture_stream && hipStreamCreateWithFlags(&g_capture_stream, hipStreamNonBlocking) != hipSuccess) {
    g_capture_stream = nullptr;
    hipGetLastError();
    return nullptr;
  }
  if (hipDeviceSynchronize() != hipSuccess) return nullptr;        // recorded work starts from a quiet device
  if (hipStreamBeginCapture(g_capture_stream, hipStreamCaptureModeThreadLocal) != hipSuccess) {
    hipGetLastError();
    return nullptr;
  }
  g_stream = g_capture_stream;
  g_capturing = true;
  return (void*)g_capture_stream;
}

// Ends the recording; returns an executable graph (NULL on failure) for graph_launch / graph_free.
void* graph_capture_end(void) {
  if (!g_capturing) return nullptr;
  dn_flush();      // (a held-back product belongs to the recording)
  hipGraph_t graph = nullptr;
  const hipError_t e = hipStreamEndCapture(g_capture_stream, &graph);
  g_stream = nullptr;
  g_capturing = false;
  if (e != hipSuccess || !graph) { hipGetLastError(); return nullptr; }
  hipGraphExec_t exec = nullptr;
  const hipError_t e2 = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  hipGraphDestroy(graph);
  if (e2 != hipSuccess) { hipGetLastError(); return nullptr; }
  ++g_live_graphs;
  return (void*)exec;
}

int graph_launch(void* exec) {
  if (!exec || g_capturing) return ERROR_GENERIC;
  dn_flush();
  return hipGraphLaunch((hipGraphExec_t)exec, nullptr) == hipSuccess ? 0 : CUDA_ERROR;
}

int graph_free(void* exec) {
  if (!exec) return 0;
  dn_flush();
  hipDeviceSynchronize();
  const hipError_t e = hipGraphExecDestroy((hipGraphExec_t)exec);
  if (g_live_graphs > 0 && --g_live_graphs == 0) {
    for (void* p : g_retired) hipFree(p);
    g_retired.clear();
    for (bool& r : g_scratch_recorded) r = false;
    g_zero_words_recorded = false;
    if (g_no_graphs_hook) g_no_graphs_hook();
  }
  return e == hipSuccess ? 0 : CUDA_ERROR;
}

// Queue on a stream of the caller's (capturing != 0: the caller is capturing it); NULL, 0 afterwards.
int graph_set_stream(void* stream, int capturing) {
  dn_flush();
  g_stream = (hipStream_t)stream;
  g_capturing = capturing != 0;
  return 0;
}

int get_leading_dimension(cudamat* mat) { return mat->is_trans ? mat->size[1] : mat->size[0]; }
int get_nonleading_dimension(cudamat* mat) { return mat->is_trans ? mat->size[0] : mat->size[1]; }
void set_transpose(cudamat* mat, int is_trans) { mat->is_trans = is_trans; }

int allocate_device_memory(cudamat* mat) {
  if (g_capturing) return ERROR_UNSUPPORTED;      // (allocations and transfers are not recorded into a graph)
  const long long len = dn_len(mat);
  // A 0-element matrix still gets a distinct, valid pointer.
  const size_t bytes = (size_t)(len > 0 ? len : 1) * sizeof(float);
  void* p = block_get(bytes);
  if (!p) return CUBLAS_ERROR;
  mat->data_device = (float*)p;
  mat->on_device = 1;
  return 0;
}

int copy_to_host(cudamat* mat) {
  if (!mat->on_device) return ERROR_NOT_ON_DEVICE;
  dn_flush();
  if (g_capturing) return ERROR_UNSUPPORTED;
  const long long len = dn_len(mat);
  if (len > 0 && len <= DN_STAGE_FLOATS && stage_out(mat->data_device, mat->data_host, (int)len)) return 0;
  if (len > 0 &&
      hipMemcpy(mat->data_host, mat->data_device, (size_t)len * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess)
    return CUBLAS_ERROR;
  return 0;
}

int copy_to_device(cudamat* mat) {
  if (g_capturing) return ERROR_UNSUPPORTED;
  dn_flush();
  if (!mat->on_device) {
    int err = allocate_device_memory(mat);
    if (err) return err;
  }
  const long long len = dn_len(mat);
  if (len > 0 &&
      hipMemcpy(mat->data_device, mat->data_host, (size_t)len * sizeof(float), hipMemcpyHostToDevice) != hipSuccess)
    return CUBLAS_ERROR;
  return 0;
}

}  // extern "C"

// Device-to-device copy as a kernel of the library (16-byte groups when both sides allow them,
// non-temporal for large matrices): 64 MiB in 23 us where the runtime's copy takes 26, and a
// kernel node instead of a copy node when a graph is being recorded.
template <bool VEC, bool STREAM>
__global__ void __launch_bounds__(256) k_copy(const float* src, float* dst, long long n) {
  const long long tid = (long long)blockIdx.x * 256 + threadIdx.x;
  if (VEC) {
    const long long n4 = n >> 2;
    if (tid < n4) dn_st4<STREAM>(dst + 4 * tid, dn_ld4<STREAM>(src + 4 * tid));
    else if (tid - n4 < (n & 3)) dst[4 * n4 + (tid - n4)] = src[4 * n4 + (tid - n4)];
  } else if (tid < n) {
    dst[tid] = src[tid];
  }
}

extern "C" {

int copy_on_device(cudamat* mat1, cudamat* mat2) {
  if (mat1->size[0] != mat2->size[0] || mat1->size[1] != mat2->size[1]) return ERROR_INCOMPATIBLE_DIMENSIONS;
  const long long len = dn_len(mat1);
  if (len <= 0 || mat1->data_device == mat2->data_device) return 0;
  const float* src = mat1->data_device;
  float* dst = mat2->data_device;
  if (dn_aligned16(src) && dn_aligned16(dst)) {
    const unsigned blocks = (unsigned)(((len >> 2) + (len & 3) + 255) / 256);
    if (len >= DN_STREAM_MIN_ELEMS) hipLaunchKernelGGL((k_copy<true, true>), dim3(blocks), dim3(256), 0, dn_stream(), src, dst, len);
    else hipLaunchKernelGGL((k_copy<true, false>), dim3(blocks), dim3(256), 0, dn_stream(), src, dst, len);
  } else {
    hipLaunchKernelGGL((k_copy<false, false>), dim3((unsigned)((len + 255) / 256)), dim3(256), 0, dn_stream(), src, dst, len);
  }
  return dn_launch_status() ? CUBLAS_ERROR : 0;
}

int free_device_memory(cudamat* mat) {
  if (g_capturing) return ERROR_UNSUPPORTED;
  if (mat->owns_data && mat->on_device) {
    const bool ok = block_put(mat->data_device);
    mat->on_device = 0;
    if (!ok) return CUBLAS_ERROR;
  }
  return 0;
}

int set_shape(cudamat* mat, unsigned int m, unsigned int n) {
  mat->size[0] = m;
  mat->size[1] = n;
  return 0;
}

int reshape(cudamat* mat, unsigned int m, unsigned int n) {
  if ((unsigned int)(mat->size[0] * mat->size[1]) != m * n) return ERROR_INCOMPATIBLE_DIMENSIONS;
  mat->size[0] = m;
  mat->size[1] = n;
  return 0;
}

int get_slice(cudamat* source, cudamat* target, unsigned int first_col, unsigned int last_col) {
  if (source->is_trans) return ERROR_TRANSPOSED;
  if (!source->on_device) return ERROR_NOT_ON_DEVICE;
  if (last_col > (unsigned int)source->size[1] || first_col >= last_col) return ERROR_INCOMPATIBLE_DIMENSIONS;
  const int num_rows = source->size[0];
  target->data_host = 0;
  target->data_device = source->data_device + (size_t)first_col * num_rows;
  target->on_device = 1;
  target->on_host = 0;
  target->size[0] = source->size[0];
  target->size[1] = last_col - first_col;
  target->is_trans = 0;
  target->owns_data = 0;
  return 0;
}

int get_vector_slice(cudamat* source, cudamat* target, unsigned int first_ind, unsigned int last_ind) {
  if (source->size[0] > 1 && source->size[1] > 1) return ERROR_GENERIC;
  if (source->is_trans) return ERROR_TRANSPOSED;
  if (!source->on_device) return ERROR_NOT_ON_DEVICE;
  if (first_ind >= last_ind) return ERROR_INCOMPATIBLE_DIMENSIONS;
  const int num_rows = source->size[0];
  // The reference offsets by first_ind * num_rows for both orientations
  // (cudamat.cu:369-372); for a column vector that walks first_ind whole
  // columns, i.e. past the data for any first_ind > 0.  Offset by elements.
  (void)num_rows;
  target->data_host = 0;
  target->data_device = source->data_device + first_ind;
  target->on_device = 1;
  target->on_host = 0;
  target->is_trans = 0;
  target->owns_data = 0;
  if (source->size[0] > 1) {
    if (last_ind > (unsigned int)source->size[0]) return ERROR_INCOMPATIBLE_DIMENSIONS;
    target->size[0] = last_ind - first_ind;
    target->size[1] = 1;
  } else {
    if (last_ind > (unsigned int)source->size[1]) return ERROR_INCOMPATIBLE_DIMENSIONS;
    target->size[0] = 1;
    target->size[1] = last_ind - first_ind;
  }
  return 0;
}

void init_from_array(cudamat* mat, float* data, int m, int n) {
  mat->data_host = data;
  mat->size[0] = m;
  mat->size[1] = n;
  mat->on_device = 0;
  mat->on_host = 1;
  mat->is_trans = 0;
  mat->owns_data = 1;
}

void set_on_device(cudamat* mat) { mat->on_device = 1; }

int init_empty(cudamat* mat, int m, int n) {
  mat->size[0] = m;
  mat->size[1] = n;
  mat->on_device = 0;
  mat->on_host = 0;
  mat->is_trans = 0;
  mat->owns_data = 1;
  return allocate_device_memory(mat);
}

int get_row_slice(cudamat* source, cudamat* target, unsigned int start, unsigned int end) {
  const int height = source->size[0], width = source->size[1];
  if ((end - start) != (unsigned int)target->size[0] || source->size[1] != target->size[1] || start >= end ||
      end > (unsigned int)height)
    return ERROR_INCOMPATIBLE_DIMENSIONS;
  const int rows = end - start;
  if (width == 0) return 0;
  dim3 grid((rows + 255) / 256, width < 4096 ? width : 4096);
  hipLaunchKernelGGL(k_copy_rows, grid, dim3(256), 0, dn_stream(), source->data_device, target->data_device, rows, width,
                     height, rows, (int)start, 0);
  return dn_launch_status();
}

int set_row_slice(cudamat* source, cudamat* target, unsigned int start, unsigned int end) {
  const int height = target->size[0], width = target->size[1];
  if ((end - start) != (unsigned int)source->size[0] || source->size[1] != target->size[1] || start >= end ||
      end > (unsigned int)height)
    return ERROR_INCOMPATIBLE_DIMENSIONS;
  const int rows = end - start;
  if (width == 0) return 0;
  dim3 grid((rows + 255) / 256, width < 4096 ? width : 4096);
  hipLaunchKernelGGL(k_copy_rows, grid, dim3(256), 0, dn_stream(), source->data_device, target->data_device, rows, width, rows,
                     height, 0, (int)start);
  return dn_launch_status();
}

int copy_transpose(cudamat* source, cudamat* target) {
  const int height = source->size[0], width = source->size[1];
  if (source->size[0] != target->size[1] || source->size[1] != target->size[0]) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (height == 0 || width == 0) return 0;
  dim3 grid((height + TR_TILE - 1) / TR_TILE, (width + TR_TILE - 1) / TR_TILE);
  if (height % 4 == 0 && width % 4 == 0 && dn_aligned16(source->data_device) && dn_aligned16(target->data_device))
    hipLaunchKernelGGL(k_transpose4, grid, dim3(256), 0, dn_stream(), source->data_device, target->data_device, height, width);
  else
    hipLaunchKernelGGL(k_transpose, grid, dim3(256), 0, dn_stream(), source->data_device, target->data_device, height, width);
  return dn_launch_status();
}

}  // extern "C"
