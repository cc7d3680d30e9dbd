// Keys and values of a step's tokens, copied from the rows of a fused projection into their
// cache slots.  Keys and values may differ in size per head; nothing is normed or rotated.
// Values can be stored transposed inside their page, [page, element of all heads, slot in page]
// (page_size > 0), for attention kernels that feed runs of neighbouring keys to a matrix unit.
#include "common.h"

template <typename T>
__global__ void kv_store_kernel(T* __restrict__ k_cache, T* __restrict__ v_cache, const T* __restrict__ proj,
                                long long ld, int k_off, int v_off, const int* __restrict__ slot_map, int k_row,
                                int v_row, int page_size) {
  const int t = blockIdx.x;
  const size_t slot = static_cast<size_t>(slot_map[t]);
  const T* pr = proj + static_cast<size_t>(t) * ld;
  T* kd = k_cache + slot * k_row;
  T* vd = v_cache + slot * v_row;
  for (int i = threadIdx.x; i < k_row; i += blockDim.x) kd[i] = pr[k_off + i];
  if (page_size > 0) {
    T* page = v_cache + (slot / page_size) * page_size * v_row + slot % page_size;
    for (int i = threadIdx.x; i < v_row; i += blockDim.x) page[static_cast<size_t>(i) * page_size] = pr[v_off + i];
  } else {
    for (int i = threadIdx.x; i < v_row; i += blockDim.x) vd[i] = pr[v_off + i];
  }
}

// proj: [tokens, ld]; k_cache: [slots, k_row]; v_cache: [slots, v_row], all of dtype; k_row and
// v_row are the elements of all key/value heads of one token; page_size > 0: v_cache is
// [pages, v_row, page_size] instead.  The host guarantees that every
// slot_map[t] is a slot of the caches.
extern "C" int pylon_kv_store(void* k_cache, void* v_cache, const void* proj, int dtype, long long ld, int k_off,
                              int v_off, const int* slot_map, int tokens, int k_row, int v_row, int page_size,
                              hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(dtype), "kv_store: unknown dtype");
  PYLON_REQUIRE(tokens >= 0 && k_row > 0 && v_row > 0 && k_off >= 0 && v_off >= 0, "kv_store: bad sizes");
  PYLON_REQUIRE(ld >= k_off + k_row && ld >= v_off + v_row, "kv_store: the projection's rows are too short");
  if (tokens == 0) return 0;
  dim3 grid(tokens), block(256);
  if (dtype == PYLON_F32)
    hipLaunchKernelGGL(kv_store_kernel<float>, grid, block, 0, stream, (float*)k_cache, (float*)v_cache,
                       (const float*)proj, ld, k_off, v_off, slot_map, k_row, v_row, page_size);
  else
    hipLaunchKernelGGL(kv_store_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)k_cache, (bf16_t*)v_cache,
                       (const bf16_t*)proj, ld, k_off, v_off, slot_map, k_row, v_row, page_size);
  PYLON_LAUNCHED("kv_store");
}
