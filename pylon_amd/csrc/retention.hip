// Retention: linear attention with one fixed decay per head, no softmax and no denominator.
// Per request and head a state S [dim, vdim] of floats is carried from token to token:
//
//   S_t = decay * S_{t-1} + k_t v_t^T,     o_t = S_t^T q_t,
//   out_t = o_t / sqrt(mean(o_t^2) + eps) * silu(g_t)
//
// q and k are first rotated by the token's position (the first rot_dims elements of a head,
// element i paired with i + rot_dims/2, angle = position * inv_freq[i]); k is then multiplied
// by k_scale.  Everything but the loads of the projection and the store of the result is float.
//
// This file holds the recurrent form: one workgroup per (row of the step, head) walks the
// row's tokens in order with S in registers, column j of S in the threads j, j + vdim, ...,
// each of which keeps every IP-th row.  The order of every sum is fixed by the head's sizes,
// so a request's results do not depend on how it was cut into steps or what shared a step.
#include "common.h"

template <typename T, int NI, int THREADS>
__global__ __launch_bounds__(THREADS) void retention_recurrent_kernel(T* __restrict__ out, const T* __restrict__ proj, long long ld,
                                           int q_off, int k_off, int v_off, int g_off, float* state,
                                           const float* __restrict__ decay, const float* __restrict__ inv_freq,
                                           int rot_dims, const int* __restrict__ positions,
                                           const int* __restrict__ row_start, const int* __restrict__ row_slots,
                                           int heads, int dim, int vdim, int ip_count, float eps, float k_scale) {
  extern __shared__ float lds[];
  float* qs = lds;                 // [dim]
  float* ks = qs + dim;            // [dim]
  float* part = ks + dim;          // [ip_count * vdim]
  float* red = part + ip_count * vdim;  // [16]
  const int row = blockIdx.x, head = blockIdx.y;
  const int tid = threadIdx.x;
  const int j = tid % vdim, ip = tid / vdim;  // column of S, and which rows of it
  const bool owner = ip < ip_count;           // the workgroup is padded to whole wavefronts
  const int begin = row_start[row], end = row_start[row + 1];
  float* st = state + ((static_cast<size_t>(row_slots[row]) * heads + head) * dim) * vdim;
  const float lam = decay[head];
  float s[NI];
#pragma unroll
  for (int n = 0; n < NI; ++n) {
    const int i = ip + n * ip_count;
    s[n] = (owner && i < dim) ? st[static_cast<size_t>(i) * vdim + j] : 0.f;
  }
  const int half = rot_dims / 2;
  for (int t = begin; t < end; ++t) {
    const T* pr = proj + static_cast<size_t>(t) * ld;
    const float pos = static_cast<float>(positions[t]);
    for (int e = tid; e < 2 * dim; e += blockDim.x) {
      const bool is_k = e >= dim;
      const int d = is_k ? e - dim : e;
      const T* src = pr + (is_k ? k_off : q_off) + head * dim;
      float v = to_float(src[d]);
      if (d < rot_dims) {
        const int pair = d < half ? d : d - half;
        const float angle = pos * inv_freq[pair];
        float sn, cs;
        sincosf(angle, &sn, &cs);
        const float other = to_float(src[d < half ? d + half : d - half]);
        v = d < half ? v * cs - other * sn : v * cs + other * sn;
      }
      if (is_k) ks[d] = v * k_scale;
      else qs[d] = v;
    }
    __syncthreads();
    const float vj = to_float(pr[v_off + head * vdim + j]);
    float acc = 0.f;
    if (owner) {
#pragma unroll
      for (int n = 0; n < NI; ++n) {
        const int i = ip + n * ip_count;
        if (i < dim) {
          s[n] = fmaf(lam, s[n], ks[i] * vj);
          acc = fmaf(s[n], qs[i], acc);
        }
      }
      part[ip * vdim + j] = acc;
    }
    __syncthreads();
    float o = 0.f, sq = 0.f;
    if (ip == 0) {
      for (int p = 0; p < ip_count; ++p) o += part[p * vdim + j];
      sq = o * o;
    }
    const float total = block_sum(sq, red);  // two barriers inside: qs, ks and part are free again after it
    if (ip == 0) {
      const float inv = 1.0f / sqrtf(total / static_cast<float>(vdim) + eps);
      const float g = to_float(pr[g_off + head * vdim + j]);
      out[(static_cast<size_t>(t) * heads + head) * vdim + j] = from_float<T>((o * inv) * (g / (1.0f + expf(-g))));
    }
  }
#pragma unroll
  for (int n = 0; n < NI; ++n) {
    const int i = ip + n * ip_count;
    if (owner && i < dim) st[static_cast<size_t>(i) * vdim + j] = s[n];
  }
}

// proj: [tokens, ld] of dtype, one row per token holding q (heads * dim elements from q_off),
// k (from k_off), v (heads * vdim from v_off) and the gate g (heads * vdim from g_off).
// out: [tokens, heads * vdim] of dtype.  state: float [slots, heads, dim, vdim].
// decay: float [heads]; inv_freq: float [rot_dims / 2] (null when rot_dims is 0).
// The host guarantees row_slots < slots, one position per token and row_start[rows] <= tokens.
extern "C" int pylon_retention_recurrent(void* out, const void* proj, int dtype, long long ld, int q_off, int k_off,
                                         int v_off, int g_off, float* state, const float* decay,
                                         const float* inv_freq, int rot_dims, const int* positions,
                                         const int* row_start, const int* row_slots, int rows, int heads, int dim,
                                         int vdim, float eps, float k_scale, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(dtype), "retention: unknown dtype");
  PYLON_REQUIRE(rows >= 0 && heads > 0 && dim > 0 && vdim > 0, "retention: bad sizes");
  PYLON_REQUIRE(vdim <= 256 && dim <= 1024, "retention: heads of up to 1024 key and 256 value elements, got %d and %d",
                dim, vdim);
  PYLON_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dim, "retention: rot_dims %d does not fit a head of %d",
                rot_dims, dim);
  PYLON_REQUIRE(rot_dims == 0 || inv_freq != nullptr, "retention: a rotation needs its frequencies");
  if (rows == 0) return 0;
  int ip_count = 256 / vdim;
  if (ip_count > dim) ip_count = dim;
  if ((dim + ip_count - 1) / ip_count > 64) {  // a large head: more threads, fewer rows of S each
    ip_count = 1024 / vdim;
    if (ip_count > dim) ip_count = dim;
  }
  const int per = (dim + ip_count - 1) / ip_count;
  PYLON_REQUIRE(per <= 64, "retention: a head of %d x %d does not fit a workgroup's registers", dim, vdim);
  dim3 grid(rows, heads), block((vdim * ip_count + PYLON_WAVE - 1) / PYLON_WAVE * PYLON_WAVE);
  const size_t lds = sizeof(float) * (2 * dim + ip_count * vdim + 16);
#define GO(T, NI)                                                                                              \
  if (block.x <= 256)                                                                                          \
    hipLaunchKernelGGL((retention_recurrent_kernel<T, NI, 256>), grid, block, lds, stream, (T*)out, (const T*)proj, ld, \
                       q_off, k_off, v_off, g_off, state, decay, inv_freq, rot_dims, positions, row_start,      \
                       row_slots, heads, dim, vdim, ip_count, eps, k_scale);                                    \
  else                                                                                                         \
    hipLaunchKernelGGL((retention_recurrent_kernel<T, NI, 1024>), grid, block, lds, stream, (T*)out, (const T*)proj, ld, \
                     q_off, k_off, v_off, g_off, state, decay, inv_freq, rot_dims, positions, row_start,        \
                     row_slots, heads, dim, vdim, ip_count, eps, k_scale)
#define PICK(T)                 \
  do {                          \
    if (per <= 4) GO(T, 4);     \
    else if (per <= 16) GO(T, 16); \
    else GO(T, 64);             \
  } while (0)
  if (dtype == PYLON_F32) PICK(float);
  else PICK(bf16_t);
#undef PICK
#undef GO
  PYLON_LAUNCHED("retention_recurrent");
}
