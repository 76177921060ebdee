// Edge-list preprocessing for the fused scatter (gfx950): range checks of the edge
// indices and a stable sort of edge ids by destination, giving CSR row pointers.
//
// The reference adds messages with scatter_add_ (e3nn/nn/models/v2106/points_convolution.py:13-17);
// grouping the edges of one destination lets one wavefront sum them in registers and
// write each output row exactly once.  The sort is integer-only and stable, so the
// permutation (and therefore the summation order) is unique for a given edge list.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <mutex>

#include <rocprim/rocprim.hpp>

#include "e3x_internal.h"

namespace {

constexpr int kBlock = 256;

__device__ int d_flag[4];  // range-check result of e3x_index_check (one copy per device)
std::mutex g_flag_mutex;   // one check at a time: concurrent callers would share the flag

// Sort buffers of e3x_csr_build_static.  Every device the library runs on holds its own copy of this array at its
// own address for the life of the process; host code must use the address hipGetSymbolAddress reports for the
// current device (static_scratch() below), never the array's name.
constexpr size_t kStaticScratchBytes = 64u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;
// one call at a time per device: the callers of a device share its array, and a call ends with the stream synchronised
// (the range-check read-back), so holding the lock from the first launch to that point makes host threads take turns
std::mutex g_scratch_busy[kMaxDevices];

// device address of `scratch` on the current device, looked up once per device
int static_scratch(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return e3x::fail(E3X_ERR_HIP, "e3x_csr_build_static: no current HIP device");
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p)
      return e3x::fail(E3X_ERR_HIP, "e3x_csr_build_static: hipGetSymbolAddress failed");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return E3X_OK;
}

template <typename IdxT>
__global__ __launch_bounds__(kBlock) void keys_kernel(const IdxT* __restrict__ dst, long long E, long long N,
                                                      unsigned* __restrict__ keys, int* __restrict__ ids,
                                                      int* __restrict__ flags) {
  bool bad = false;
  for (long long e = (long long)blockIdx.x * kBlock + threadIdx.x; e < E; e += (long long)gridDim.x * kBlock) {
    const long long d = (long long)dst[e];
    if (d < 0 || d >= N) bad = true;
    keys[e] = (unsigned)d;
    ids[e] = (int)e;
  }
  if (bad) atomicOr(&flags[0], 1);
}

template <typename IdxT>
__global__ __launch_bounds__(kBlock) void range_kernel(const IdxT* __restrict__ idx, long long E, long long N,
                                                       int* __restrict__ flags) {
  bool bad = false;
  for (long long e = (long long)blockIdx.x * kBlock + threadIdx.x; e < E; e += (long long)gridDim.x * kBlock) {
    const long long d = (long long)idx[e];
    if (d < -N || d >= N) bad = true;
  }
  if (bad) atomicOr(&flags[0], 1);
}

// src_rows[k] = source row of the edge at position k of the destination-sorted list, negative values wrapped
template <typename IdxT>
__global__ __launch_bounds__(kBlock) void src_rows_kernel(const IdxT* __restrict__ src, const int* __restrict__ perm,
                                                          long long E, long long n_src, int* __restrict__ src_rows) {
  for (long long k = (long long)blockIdx.x * kBlock + threadIdx.x; k < E; k += (long long)gridDim.x * kBlock) {
    long long s = (long long)src[perm ? perm[k] : k];
    if (s < 0) s += n_src;
    src_rows[k] = (int)s;
  }
}

// rowptr[n] = first position k with sorted_key[k] >= n   (n = 0..N)
__global__ __launch_bounds__(kBlock) void rowptr_kernel(const unsigned* __restrict__ sorted, long long E,
                                                        long long N, int* __restrict__ rowptr) {
  for (long long n = (long long)blockIdx.x * kBlock + threadIdx.x; n <= N; n += (long long)gridDim.x * kBlock) {
    long long lo = 0, hi = E;
    while (lo < hi) {
      const long long mid = (lo + hi) >> 1;
      if ((long long)sorted[mid] < n) lo = mid + 1; else hi = mid;
    }
    rowptr[n] = (int)lo;
  }
}

// key[n] = smallest source row among the in-edges of output row n (all ones for a row without edges), second[n] the
// smallest one above it, ids[n] = n
template <typename IdxT>
__global__ __launch_bounds__(kBlock) void rowkey_kernel(const IdxT* __restrict__ src, const int* __restrict__ rowptr,
                                                        const int* __restrict__ perm, long long N, long long n_src,
                                                        unsigned* __restrict__ keys, unsigned* __restrict__ second,
                                                        int* __restrict__ ids) {
  for (long long n = (long long)blockIdx.x * kBlock + threadIdx.x; n < N; n += (long long)gridDim.x * kBlock) {
    unsigned k1 = 0xffffffffu, k2 = 0xffffffffu;
    for (int k = rowptr[n]; k < rowptr[n + 1]; ++k) {
      long long s = (long long)src[perm ? perm[k] : k];
      if (s < 0) s += n_src;  // gather semantics: negative indices wrap
      const unsigned v = (unsigned)s;
      if (v < k1) {
        k2 = k1;
        k1 = v;
      } else if (v > k1 && v < k2) {
        k2 = v;
      }
    }
    keys[n] = k1;
    second[n] = k2;
    ids[n] = (int)n;
  }
}

// counts the neighbours in the order that agree in BOTH smallest sources: chance alone makes rows share one
// (a small id is the minimum of many rows), two in common mean overlapping source sets
__global__ __launch_bounds__(kBlock) void order_score_kernel(const int* __restrict__ order, const unsigned* __restrict__ keys,
                                                             const unsigned* __restrict__ second, long long N,
                                                             int* __restrict__ score) {
  int hits = 0;
  for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i + 1 < N; i += (long long)gridDim.x * kBlock) {
    const int a = order[i], b = order[i + 1];
    if (keys[a] != 0xffffffffu && keys[a] == keys[b] && second[a] != 0xffffffffu && second[a] == second[b]) ++hits;
  }
  if (hits) atomicAdd(score, hits);
}

// One more level of the row key for graphs whose sources and destinations are the same node set:
// level[n] <- key[level[n]] (the smallest source of the row's current key node), and its value for the rows in
// their current order
__global__ __launch_bounds__(kBlock) void level_key_kernel(const int* __restrict__ order, const unsigned* __restrict__ keys,
                                                           unsigned* __restrict__ level, unsigned* __restrict__ by_position,
                                                           long long N, int first) {
  for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < N; i += (long long)gridDim.x * kBlock) {
    const int n = order[i];
    const unsigned prev = first ? keys[n] : level[n];  // each row appears once in `order`: no other thread touches level[n]
    const unsigned next = prev < (unsigned)N ? keys[prev] : 0xffffffffu;
    level[n] = next;
    by_position[i] = next;
  }
}

__global__ __launch_bounds__(kBlock) void fill_zero_kernel(int* p, int n) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i < n) p[i] = 0;
}

// one 16-byte element per thread and a grid that covers the buffer once
__global__ __launch_bounds__(kBlock) void copy16_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                        size_t n16) {
  const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n16) dst[i] = src[i];
}

// One wavefront per row: reads the row's in16 16-byte pieces (consecutive rows are stored one after the other) with
// non-temporal loads, eight 1 KB instructions in flight, folds them with XOR and writes out16 pieces of the fold.
typedef unsigned stream_u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(kBlock) void stream_rows_kernel(const stream_u32x4* __restrict__ in, long long in16,
                                                             long long n_rows, stream_u32x4* __restrict__ out, int out16) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * (kBlock / 64) + threadIdx.x / 64;
  if (row >= n_rows) return;
  const stream_u32x4* p = in + row * in16;
  stream_u32x4 acc = {0u, 0u, 0u, 0u};
  for (long long i = lane; i < in16; i += 64 * 8) {
    stream_u32x4 v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k)
      v[k] = i + 64 * k < in16 ? __builtin_nontemporal_load(p + i + 64 * k) : stream_u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int k = 0; k < 8; ++k) acc ^= v[k];
  }
  for (int q = lane; q < out16; q += 64) out[row * out16 + q] = acc;
}

__global__ __launch_bounds__(kBlock) void fill_zero_bytes_kernel(unsigned char* p, size_t n) {
  // 16-byte stores over the aligned middle, byte stores at the ragged ends
  const size_t head = (16 - ((uintptr_t)p & 15)) & 15;
  const size_t h = head < n ? head : n;
  const size_t n16 = (n - h) / 16;
  const size_t tid = (size_t)blockIdx.x * kBlock + threadIdx.x, stride = (size_t)gridDim.x * kBlock;
  uint4* mid = reinterpret_cast<uint4*>(p + h);
  for (size_t i = tid; i < n16; i += stride) mid[i] = make_uint4(0, 0, 0, 0);
  if (tid < h) p[tid] = 0;
  const size_t tail0 = h + n16 * 16;
  if (tid < n - tail0) p[tail0 + tid] = 0;
}

unsigned grid_for(long long n, int per_block) {
  long long b = (n + per_block - 1) / per_block;
  if (b < 1) b = 1;
  if (b > 256 * 16) b = 256 * 16;
  return (unsigned)b;
}

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

int key_bits(long long N) {
  int b = 1;
  while ((1LL << b) < N) ++b;
  return b;
}

size_t sort_temp_bytes(long long E, long long N) {
  size_t temp = 0;
  (void)rocprim::radix_sort_pairs(nullptr, temp, (unsigned*)nullptr, (unsigned*)nullptr, (int*)nullptr, (int*)nullptr,
                            (size_t)E, 0, key_bits(N), (hipStream_t)0);
  return temp;
}

}  // namespace

int e3x::fill_zero_bytes(void* p, size_t n_bytes, void* stream) {
  if (n_bytes == 0) return E3X_OK;
  hipLaunchKernelGGL(fill_zero_bytes_kernel, dim3(grid_for((long long)(n_bytes / 16 + 1), kBlock)), dim3(kBlock), 0,
                     (hipStream_t)stream, (unsigned char*)p, n_bytes);
  return hipGetLastError() == hipSuccess ? E3X_OK : e3x::fail(E3X_ERR_HIP, "zero-fill launch failed");
}

extern "C" size_t e3x_csr_workspace_bytes(int64_t E, int64_t num_nodes) {
  if (E < 0 || num_nodes < 0) return 0;
  const size_t e4 = align_up((size_t)E * 4, 256);
  // flags | keys_in | keys_out | ids_in | rocPRIM temp
  return 256 + 3 * e4 + align_up(sort_temp_bytes(E > 0 ? E : 1, num_nodes > 1 ? num_nodes : 2), 256);
}

extern "C" int e3x_csr_build_static(const void* dst, int idx_bits, int64_t E, int64_t num_nodes, int32_t* rowptr,
                                    int32_t* perm, void* stream) {
  if (E < 0 || num_nodes < 0 || E >= (1LL << 31) || num_nodes >= (1LL << 31))
    return e3x::fail(E3X_ERR_INVALID, "e3x_csr_build_static: E and num_nodes must fit in int32");
  const size_t need = e3x_csr_workspace_bytes(E, num_nodes);
  if (need > kStaticScratchBytes) {
    char msg[200];
    snprintf(msg, sizeof msg,
             "e3x_csr_build_static: %lld edges need %zu bytes of sort buffers, the static buffer holds %zu "
             "(use e3x_csr_build with a workspace)", (long long)E, need, kStaticScratchBytes);
    return e3x::fail(E3X_ERR_INVALID, msg);
  }
  if (E == 0) return e3x_csr_build(dst, idx_bits, E, num_nodes, rowptr, perm, nullptr, kStaticScratchBytes, stream);  // touches no scratch
  void* ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc != E3X_OK) return rc;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return e3x::fail(E3X_ERR_HIP, "e3x_csr_build_static: no current HIP device");
  std::lock_guard<std::mutex> busy(g_scratch_busy[dev]);
  return e3x_csr_build(dst, idx_bits, E, num_nodes, rowptr, perm, ws, kStaticScratchBytes, stream);
}

extern "C" size_t e3x_csr_static_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int e3x_csr_build(const void* dst, int idx_bits, int64_t E, int64_t num_nodes, int32_t* rowptr,
                             int32_t* perm, void* workspace, size_t workspace_bytes, void* stream) {
  if (E < 0 || num_nodes < 0 || E >= (1LL << 31) || num_nodes >= (1LL << 31))
    return e3x::fail(E3X_ERR_INVALID, "e3x_csr_build: E and num_nodes must fit in int32");
  if (idx_bits != 32 && idx_bits != 64) return e3x::fail(E3X_ERR_INVALID, "e3x_csr_build: idx_bits must be 32 or 64");
  if (!rowptr || (E > 0 && (!dst || !perm || !workspace)))
    return e3x::fail(E3X_ERR_INVALID, "e3x_csr_build: null pointer");
  if (workspace_bytes < e3x_csr_workspace_bytes(E, num_nodes))
    return e3x::fail(E3X_ERR_INVALID, "e3x_csr_build: workspace smaller than e3x_csr_workspace_bytes()");
  hipStream_t st = (hipStream_t)stream;
  if (E == 0) {
    hipLaunchKernelGGL(fill_zero_kernel, dim3(grid_for(num_nodes + 1, kBlock)), dim3(kBlock), 0, st, rowptr,
                       (int)(num_nodes + 1));
    return hipGetLastError() == hipSuccess ? E3X_OK : e3x::fail(E3X_ERR_HIP, "e3x_csr_build: launch failed");
  }
  const size_t e4 = align_up((size_t)E * 4, 256);
  char* ws = (char*)workspace;
  int* flags = (int*)ws;
  unsigned* keys_in = (unsigned*)(ws + 256);
  unsigned* keys_out = (unsigned*)(ws + 256 + e4);
  int* ids_in = (int*)(ws + 256 + 2 * e4);
  void* temp = ws + 256 + 3 * e4;
  size_t temp_bytes = sort_temp_bytes(E, num_nodes > 1 ? num_nodes : 2);

  hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(kBlock), 0, st, flags, 2);
  if (idx_bits == 64)
    hipLaunchKernelGGL((keys_kernel<long long>), dim3(grid_for(E, kBlock)), dim3(kBlock), 0, st,
                       (const long long*)dst, (long long)E, (long long)num_nodes, keys_in, ids_in, flags);
  else
    hipLaunchKernelGGL((keys_kernel<int>), dim3(grid_for(E, kBlock)), dim3(kBlock), 0, st, (const int*)dst,
                       (long long)E, (long long)num_nodes, keys_in, ids_in, flags);
  // stable LSD radix sort of (dst, edge id) over the significant key bits only
  hipError_t err = rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_out, ids_in, perm, (size_t)E, 0,
                                             key_bits(num_nodes > 1 ? num_nodes : 2), st);
  if (err != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_csr_build: radix sort failed");
  hipLaunchKernelGGL(rowptr_kernel, dim3(grid_for(num_nodes + 1, kBlock)), dim3(kBlock), 0, st, keys_out, (long long)E,
                     (long long)num_nodes, rowptr);
  int h_flags[2] = {0, 0};
  if (hipMemcpyAsync(h_flags, flags, sizeof(h_flags), hipMemcpyDeviceToHost, st) != hipSuccess ||
      hipStreamSynchronize(st) != hipSuccess)
    return e3x::fail(E3X_ERR_HIP, "e3x_csr_build: reading back the range flags failed");
  if (h_flags[0]) return e3x::fail(E3X_ERR_INDEX, "index out of range in scatter destination");
  return E3X_OK;
}

extern "C" size_t e3x_row_order_workspace_bytes(int64_t num_nodes) {
  if (num_nodes < 0) return 0;
  const size_t n4 = align_up((size_t)(num_nodes > 0 ? num_nodes : 1) * 4, 256);
  size_t temp = 0;
  (void)rocprim::radix_sort_pairs(nullptr, temp, (unsigned*)nullptr, (unsigned*)nullptr, (int*)nullptr, (int*)nullptr,
                                  (size_t)(num_nodes > 0 ? num_nodes : 1), 0, 32, (hipStream_t)0);
  return 256 + 6 * n4 + align_up(temp, 256);  // score | keys_in | keys_out | ids_in | second | level | level keys | rocPRIM temp
}

extern "C" int e3x_row_order_build(const void* src, int idx_bits, const int32_t* rowptr, const int32_t* perm, int64_t E,
                                   int64_t num_nodes, int64_t num_src_nodes, int32_t* row_order, int32_t* shared_pairs,
                                   void* workspace, size_t workspace_bytes, void* stream) {
  if (E < 0 || num_nodes < 0 || num_src_nodes < 0 || num_nodes >= (1LL << 31) || num_src_nodes >= (1LL << 31))
    return e3x::fail(E3X_ERR_INVALID, "e3x_row_order_build: sizes must fit in int32");
  if (idx_bits != 32 && idx_bits != 64) return e3x::fail(E3X_ERR_INVALID, "e3x_row_order_build: idx_bits must be 32 or 64");
  if (shared_pairs) *shared_pairs = 0;
  if (num_nodes == 0) return E3X_OK;
  if (!rowptr || !row_order || !workspace || (E > 0 && !src)) return e3x::fail(E3X_ERR_INVALID, "e3x_row_order_build: null pointer");
  if (workspace_bytes < e3x_row_order_workspace_bytes(num_nodes))
    return e3x::fail(E3X_ERR_INVALID, "e3x_row_order_build: workspace smaller than e3x_row_order_workspace_bytes()");
  hipStream_t st = (hipStream_t)stream;
  const size_t n4 = align_up((size_t)num_nodes * 4, 256);
  char* ws = (char*)workspace;
  int* score = (int*)ws;
  unsigned* keys_in = (unsigned*)(ws + 256);
  unsigned* keys_out = (unsigned*)(ws + 256 + n4);
  int* ids_in = (int*)(ws + 256 + 2 * n4);
  unsigned* second = (unsigned*)(ws + 256 + 3 * n4);
  unsigned* level = (unsigned*)(ws + 256 + 4 * n4);
  unsigned* level_keys = (unsigned*)(ws + 256 + 5 * n4);
  void* temp = ws + 256 + 6 * n4;
  size_t temp_bytes = workspace_bytes - 256 - 6 * n4;
  hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(kBlock), 0, st, score, 1);
  if (idx_bits == 64)
    hipLaunchKernelGGL((rowkey_kernel<long long>), dim3(grid_for(num_nodes, kBlock)), dim3(kBlock), 0, st, (const long long*)src,
                       rowptr, perm, (long long)num_nodes, (long long)num_src_nodes, keys_in, second, ids_in);
  else
    hipLaunchKernelGGL((rowkey_kernel<int>), dim3(grid_for(num_nodes, kBlock)), dim3(kBlock), 0, st, (const int*)src, rowptr,
                       perm, (long long)num_nodes, (long long)num_src_nodes, keys_in, second, ids_in);
  if (hipGetLastError() != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_row_order_build: launch failed");
  // stable: rows with the same key keep their numbering
  hipError_t err = rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_out, ids_in, row_order, (size_t)num_nodes, 0, 32, st);
  if (err != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_row_order_build: radix sort failed");
  // Sources and destinations numbered alike (one node set): two more levels, key of the key.  Rows are then grouped
  // by (smallest source of the smallest source of their smallest source, ..., smallest source), which puts groups of
  // rows with neighbouring key nodes next to each other as well.  Two stable sorts, the most significant level last.
  if (num_src_nodes == num_nodes && num_nodes > 1) {
    int* cur = row_order;
    int* other = ids_in;
    for (int lev = 0; lev < 2; ++lev) {
      hipLaunchKernelGGL(level_key_kernel, dim3(grid_for(num_nodes, kBlock)), dim3(kBlock), 0, st, cur, keys_in, level, level_keys,
                         (long long)num_nodes, lev == 0 ? 1 : 0);
      if (hipGetLastError() != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_row_order_build: launch failed");
      err = rocprim::radix_sort_pairs(temp, temp_bytes, level_keys, keys_out, cur, other, (size_t)num_nodes, 0, 32, st);
      if (err != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_row_order_build: radix sort failed");
      std::swap(cur, other);
    }
    // two sorts: the result is back in row_order
  }
  if (shared_pairs) {
    hipLaunchKernelGGL(order_score_kernel, dim3(grid_for(num_nodes, kBlock)), dim3(kBlock), 0, st, row_order, keys_in, second,
                       (long long)num_nodes, score);
    if (hipMemcpyAsync(shared_pairs, score, sizeof(int), hipMemcpyDeviceToHost, st) != hipSuccess ||
        hipStreamSynchronize(st) != hipSuccess)
      return e3x::fail(E3X_ERR_HIP, "e3x_row_order_build: reading back the score failed");
  }
  return E3X_OK;
}

extern "C" int e3x_src_rows_build(const void* src, int idx_bits, const int32_t* perm, int64_t E, int64_t num_src_nodes,
                                   int32_t* src_rows, void* stream) {
  if (idx_bits != 32 && idx_bits != 64) return e3x::fail(E3X_ERR_INVALID, "e3x_src_rows_build: idx_bits must be 32 or 64");
  if (E < 0 || num_src_nodes < 0 || num_src_nodes >= (1LL << 31))
    return e3x::fail(E3X_ERR_INVALID, "e3x_src_rows_build: sizes must be in [0, 2^31)");
  if (E == 0) return E3X_OK;
  if (!src || !src_rows) return e3x::fail(E3X_ERR_INVALID, "e3x_src_rows_build: null pointer");
  hipStream_t st = (hipStream_t)stream;
  if (idx_bits == 64)
    hipLaunchKernelGGL((src_rows_kernel<long long>), dim3(grid_for(E, kBlock)), dim3(kBlock), 0, st,
                       (const long long*)src, perm, (long long)E, (long long)num_src_nodes, src_rows);
  else
    hipLaunchKernelGGL((src_rows_kernel<int>), dim3(grid_for(E, kBlock)), dim3(kBlock), 0, st, (const int*)src, perm,
                       (long long)E, (long long)num_src_nodes, src_rows);
  return hipGetLastError() == hipSuccess ? E3X_OK : e3x::fail(E3X_ERR_HIP, "e3x_src_rows_build: launch failed");
}

extern "C" int e3x_index_check(const void* idx, int idx_bits, int64_t E, int64_t num_nodes, void* stream) {
  if (idx_bits != 32 && idx_bits != 64) return e3x::fail(E3X_ERR_INVALID, "e3x_index_check: idx_bits must be 32 or 64");
  if (E == 0) return E3X_OK;
  if (!idx) return e3x::fail(E3X_ERR_INVALID, "e3x_index_check: null pointer");
  hipStream_t st = (hipStream_t)stream;
  // zero, launch and read-back form one critical section (it ends with a stream synchronisation anyway)
  std::lock_guard<std::mutex> lock(g_flag_mutex);
  int* flag = nullptr;
  if (hipGetSymbolAddress((void**)&flag, HIP_SYMBOL(d_flag)) != hipSuccess)
    return e3x::fail(E3X_ERR_HIP, "e3x_index_check: hipGetSymbolAddress failed");
  hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(kBlock), 0, st, flag, 1);
  if (idx_bits == 64)
    hipLaunchKernelGGL((range_kernel<long long>), dim3(grid_for(E, kBlock)), dim3(kBlock), 0, st,
                       (const long long*)idx, (long long)E, (long long)num_nodes, flag);
  else
    hipLaunchKernelGGL((range_kernel<int>), dim3(grid_for(E, kBlock)), dim3(kBlock), 0, st, (const int*)idx,
                       (long long)E, (long long)num_nodes, flag);
  int h = 0;
  if (hipMemcpyAsync(&h, flag, sizeof(int), hipMemcpyDeviceToHost, st) != hipSuccess ||
      hipStreamSynchronize(st) != hipSuccess)
    return e3x::fail(E3X_ERR_HIP, "e3x_index_check: reading back the range flag failed");
  if (h) return e3x::fail(E3X_ERR_INDEX, "index out of range in gather source");
  return E3X_OK;
}

extern "C" int e3x_copy_bytes(const void* src, void* dst, size_t n_bytes, void* stream) {
  if (n_bytes % 16 || ((uintptr_t)src % 16) || ((uintptr_t)dst % 16))
    return e3x::fail(E3X_ERR_INVALID, "e3x_copy_bytes: size and pointers must be multiples of 16");
  if (n_bytes == 0) return E3X_OK;
  const size_t blocks = (n_bytes / 16 + kBlock - 1) / kBlock;
  if (blocks > 0x7fffffffULL) return e3x::fail(E3X_ERR_INVALID, "e3x_copy_bytes: buffer too large for one launch");
  hipLaunchKernelGGL(copy16_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, (hipStream_t)stream, (const uint4*)src,
                     (uint4*)dst, n_bytes / 16);
  return hipGetLastError() == hipSuccess ? E3X_OK : e3x::fail(E3X_ERR_HIP, "e3x_copy_bytes: launch failed");
}

extern "C" int e3x_stream_rows(const void* in, size_t in_bytes_per_row, int64_t n_rows, void* out, size_t out_bytes_per_row,
                               void* stream) {
  if (in_bytes_per_row % 16 || out_bytes_per_row % 16 || ((uintptr_t)in % 16) || ((uintptr_t)out % 16) || n_rows < 0 ||
      out_bytes_per_row > (1u << 20))
    return e3x::fail(E3X_ERR_INVALID, "e3x_stream_rows: sizes and pointers must be multiples of 16, rows of output at most 1 MiB");
  if (n_rows == 0) return E3X_OK;
  if (!in || (out_bytes_per_row && !out)) return e3x::fail(E3X_ERR_INVALID, "e3x_stream_rows: null pointer");
  const int64_t blocks = (n_rows + kBlock / 64 - 1) / (kBlock / 64);
  if (blocks > 0x7fffffffLL) return e3x::fail(E3X_ERR_INVALID, "e3x_stream_rows: too many rows for one launch");
  hipLaunchKernelGGL(stream_rows_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, (hipStream_t)stream,
                     (const stream_u32x4*)in, (long long)(in_bytes_per_row / 16), (long long)n_rows, (stream_u32x4*)out,
                     (int)(out_bytes_per_row / 16));
  return hipGetLastError() == hipSuccess ? E3X_OK : e3x::fail(E3X_ERR_HIP, "e3x_stream_rows: launch failed");
}
