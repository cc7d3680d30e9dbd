// Kernels of latent attention, in which only a small latent per token is cached and every head's
// keys and values are linear maps of it.  With q'_h = W_uk[h]^T q_h the score q_h . (W_uk[h] c)
// equals q'_h . c, and sum_j p_j W_uv[h] c_j equals W_uv[h] (sum_j p_j c_j): attention runs over
// the cached latents themselves (one key/value head, keys = values = c), between two small
// products per head.
//
// latent_prepare: from the fused down projection's float sums [tokens, q_rank + kv_rank + gates]
//   the normed query latent, the normed key/value latent into its cache slot, and sigmoid of the
//   gate logits.  Norms (root mean square, eps inside the root, times a weight) in float.
// head_project: out[t, h, :] = gate[t, h] * x[t, h, :] @ m[h] with m [heads, n_in, n_out]; a
//   workgroup keeps the inputs of a few tokens in LDS and walks 64 columns of m[h] once for all of
//   them, its four waves a quarter of n_in each; sums in float in one fixed order, whatever the batch.
// gate_heads: x[t, h, :] *= gate[t, h] in place.
#include "common.h"

#define LP_THREADS 256

template <typename T>
__global__ void __launch_bounds__(LP_THREADS)
latent_prepare_kernel(T* __restrict__ q_latent, T* __restrict__ c_cache, float* __restrict__ gate_out,
                      const float* __restrict__ down, long long row_stride, const float* __restrict__ q_weight,
                      const float* __restrict__ c_weight, float eps, const int* __restrict__ slot_map, int q_rank,
                      int kv_rank, int n_gate, int store) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const float* row = down + static_cast<size_t>(t) * row_stride;
  float sq = 0.f;
  for (int i = tid; i < q_rank; i += LP_THREADS) sq = fmaf(row[i], row[i], sq);
  const float inv_q = 1.0f / sqrtf(block_sum(sq, scratch) / static_cast<float>(q_rank > 0 ? q_rank : 1) + eps);
  for (int i = tid; i < q_rank; i += LP_THREADS)
    q_latent[static_cast<size_t>(t) * q_rank + i] = from_float<T>(row[i] * inv_q * q_weight[i]);
  if (store) {
    const float* c = row + q_rank;
    float sc = 0.f;
    for (int i = tid; i < kv_rank; i += LP_THREADS) sc = fmaf(c[i], c[i], sc);
    const float inv_c = 1.0f / sqrtf(block_sum(sc, scratch) / static_cast<float>(kv_rank) + eps);
    T* dst = c_cache + static_cast<size_t>(slot_map[t]) * kv_rank;
    for (int i = tid; i < kv_rank; i += LP_THREADS) dst[i] = from_float<T>(c[i] * inv_c * c_weight[i]);
  }
  const float* g = row + q_rank + kv_rank;
  for (int i = tid; i < n_gate; i += LP_THREADS)
    gate_out[static_cast<size_t>(t) * n_gate + i] = 1.0f / (1.0f + expf(-g[i]));
}

extern "C" int pylon_latent_prepare(void* q_latent, void* c_cache, float* gate_out, const float* down,
                                    long long row_stride, int dtype, const float* q_weight, const float* c_weight,
                                    float eps, const int* slot_map, int tokens, int q_rank, int kv_rank, int n_gate,
                                    int store, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(dtype), "latent_prepare: unknown dtype");
  PYLON_REQUIRE(tokens >= 0 && q_rank > 0 && kv_rank > 0 && n_gate >= 0, "latent_prepare: sizes must be positive");
  PYLON_REQUIRE(row_stride >= static_cast<long long>(q_rank) + kv_rank + n_gate,
                "latent_prepare: rows hold fewer numbers than the latents and gates take");
  PYLON_REQUIRE(q_weight != nullptr && c_weight != nullptr, "latent_prepare: both norms have weights");
  PYLON_REQUIRE(!store || (c_cache != nullptr && slot_map != nullptr), "latent_prepare: storing needs cache and slots");
  PYLON_REQUIRE(n_gate == 0 || gate_out != nullptr, "latent_prepare: gates need a place");
  if (tokens == 0) return 0;
  if (dtype == PYLON_F32)
    hipLaunchKernelGGL((latent_prepare_kernel<float>), dim3(tokens), dim3(LP_THREADS), 0, stream, (float*)q_latent,
                       (float*)c_cache, gate_out, down, row_stride, q_weight, c_weight, eps, slot_map, q_rank,
                       kv_rank, n_gate, store);
  else
    hipLaunchKernelGGL((latent_prepare_kernel<bf16_t>), dim3(tokens), dim3(LP_THREADS), 0, stream,
                       (bf16_t*)q_latent, (bf16_t*)c_cache, gate_out, down, row_stride, q_weight, c_weight, eps,
                       slot_map, q_rank, kv_rank, n_gate, store);
  PYLON_LAUNCHED("latent_prepare");
}

#define HP_THREADS 256
#define HP_TOKENS 8
#define HP_COLS 64   // outputs of a workgroup
#define HP_SLICES 4  // the waves of a workgroup cut n_in between them

template <typename TX, typename TM>
__global__ void __launch_bounds__(HP_THREADS)
head_project_kernel(TX* __restrict__ out, const TX* __restrict__ x, long long x_stride, const TM* __restrict__ m,
                    const float* __restrict__ gate, int tokens, int heads, int n_in, int n_out) {
  extern __shared__ float xs[];  // [HP_TOKENS, n_in], then the slices' partial sums [HP_SLICES, HP_TOKENS, HP_COLS]
  float* partial = xs + HP_TOKENS * n_in;
  const int t0 = blockIdx.x * HP_TOKENS, h = blockIdx.y, tid = threadIdx.x;
  for (int i = tid; i < HP_TOKENS * n_in; i += HP_THREADS) {
    const int tt = i / n_in, k = i - tt * n_in;
    xs[i] = (t0 + tt < tokens) ? to_float(x[static_cast<size_t>(t0 + tt) * x_stride + static_cast<size_t>(h) * n_in + k])
                               : 0.f;
  }
  __syncthreads();
  const int slice = tid / HP_COLS, col = tid % HP_COLS;
  const int o = blockIdx.z * HP_COLS + col;
  const int per = (n_in + HP_SLICES - 1) / HP_SLICES;
  const int k0 = slice * per, k1 = k0 + per < n_in ? k0 + per : n_in;
  float acc[HP_TOKENS];
#pragma unroll
  for (int tt = 0; tt < HP_TOKENS; ++tt) acc[tt] = 0.f;
  if (o < n_out) {
    const TM* mh = m + static_cast<size_t>(h) * n_in * n_out + o;
#pragma unroll 8
    for (int k = k0; k < k1; ++k) {  // unrolled: eight loads of m in flight
      const float w = to_float(mh[static_cast<size_t>(k) * n_out]);
#pragma unroll
      for (int tt = 0; tt < HP_TOKENS; ++tt) acc[tt] = fmaf(xs[tt * n_in + k], w, acc[tt]);
    }
  }
#pragma unroll
  for (int tt = 0; tt < HP_TOKENS; ++tt) partial[(slice * HP_TOKENS + tt) * HP_COLS + col] = acc[tt];
  __syncthreads();
  // the slices' sums are added in their order, whatever the batch
  for (int i = tid; i < HP_TOKENS * HP_COLS; i += HP_THREADS) {
    const int tt = i / HP_COLS, c = i % HP_COLS;
    const int oc = blockIdx.z * HP_COLS + c;
    if (t0 + tt >= tokens || oc >= n_out) continue;
    float sum = partial[tt * HP_COLS + c];
#pragma unroll
    for (int sl = 1; sl < HP_SLICES; ++sl) sum += partial[(sl * HP_TOKENS + tt) * HP_COLS + c];
    const float g = gate != nullptr ? gate[static_cast<size_t>(t0 + tt) * heads + h] : 1.f;
    out[(static_cast<size_t>(t0 + tt) * heads + h) * n_out + oc] = from_float<TX>(sum * g);
  }
}

// The same product for bfloat16 matrices whose rows are whole 16-byte pieces: a lane reads eight
// neighbouring columns of a row of m[h] at once, sixteen lanes a 256-byte row segment, the sixteen
// groups of lanes of a workgroup every sixteenth row; their sums meet by two shuffles inside a wave
// and through LDS between the four waves, always in the same order.
#define HW_COLS 128

__global__ void __launch_bounds__(HP_THREADS)
head_project_wide_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ x, long long x_stride,
                         const bf16_t* __restrict__ m, const float* __restrict__ gate, int tokens, int heads, int n_in,
                         int n_out) {
  extern __shared__ float xs[];  // [HP_TOKENS, n_in], then the waves' partial sums [4, HP_TOKENS, HW_COLS]
  float* partial = xs + HP_TOKENS * n_in;
  const int t0 = blockIdx.x * HP_TOKENS, h = blockIdx.y, c0 = blockIdx.z * HW_COLS, tid = threadIdx.x;
  for (int i = tid; i < HP_TOKENS * n_in; i += HP_THREADS) {
    const int tt = i / n_in, k = i - tt * n_in;
    xs[i] = (t0 + tt < tokens) ? to_float(x[static_cast<size_t>(t0 + tt) * x_stride + static_cast<size_t>(h) * n_in + k])
                               : 0.f;
  }
  __syncthreads();
  const int lane = tid & (PYLON_WAVE - 1), wave = tid / PYLON_WAVE;
  const int cg = lane & 15, kg = wave * 4 + (lane >> 4);
  float acc[HP_TOKENS][8];
#pragma unroll
  for (int tt = 0; tt < HP_TOKENS; ++tt)
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[tt][c] = 0.f;
  const int col = c0 + 8 * cg;
  if (col < n_out) {  // n_out is a multiple of 8: the lane's eight columns are all inside
    const bf16_t* mh = m + static_cast<size_t>(h) * n_in * n_out + col;
#pragma unroll 4
    for (int k = kg; k < n_in; k += 16) {
      const uint4 raw = *reinterpret_cast<const uint4*>(mh + static_cast<size_t>(k) * n_out);
      const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
      float wv[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        wv[2 * j] = __uint_as_float(words[j] << 16);
        wv[2 * j + 1] = __uint_as_float(words[j] & 0xffff0000u);
      }
#pragma unroll
      for (int tt = 0; tt < HP_TOKENS; ++tt) {
        const float xv = xs[tt * n_in + k];
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[tt][c] = fmaf(xv, wv[c], acc[tt][c]);
      }
    }
  }
#pragma unroll
  for (int tt = 0; tt < HP_TOKENS; ++tt)
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      float v = acc[tt][c];
      v += __shfl_xor(v, 16, PYLON_WAVE);
      v += __shfl_xor(v, 32, PYLON_WAVE);
      if (lane < 16) partial[(wave * HP_TOKENS + tt) * HW_COLS + 8 * cg + c] = v;
    }
  __syncthreads();
  for (int i = tid; i < HP_TOKENS * HW_COLS; i += HP_THREADS) {
    const int tt = i / HW_COLS, c = i % HW_COLS;
    if (t0 + tt >= tokens || c0 + c >= n_out) continue;
    float sum = partial[tt * HW_COLS + c];
#pragma unroll
    for (int wv = 1; wv < 4; ++wv) sum += partial[(wv * HP_TOKENS + tt) * HW_COLS + c];
    const float g = gate != nullptr ? gate[static_cast<size_t>(t0 + tt) * heads + h] : 1.f;
    out[(static_cast<size_t>(t0 + tt) * heads + h) * n_out + c0 + c] = from_float<bf16_t>(sum * g);
  }
}

// x: [tokens, heads, n_in], rows x_stride elements apart; m: [heads, n_in, n_out]; gate: null or
// float [tokens, heads]; out: [tokens, heads, n_out] of x's type.  m may be float while x is bfloat16.
extern "C" int pylon_head_project(void* out, const void* x, int x_dtype, long long x_stride, const void* m,
                                  int m_dtype, const float* gate, int tokens, int heads, int n_in, int n_out,
                                  hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(x_dtype) && pylon_valid_dtype(m_dtype), "head_project: unknown dtype");
  PYLON_REQUIRE(tokens >= 0 && heads > 0 && n_in > 0 && n_out > 0, "head_project: sizes must be positive");
  PYLON_REQUIRE(heads <= 65535, "head_project: too many heads for one launch");
  PYLON_REQUIRE(x_stride >= static_cast<long long>(heads) * n_in, "head_project: rows of x overlap");
  const size_t lds = sizeof(float) * (HP_TOKENS * n_in + HP_SLICES * HP_TOKENS * HP_COLS);
  PYLON_REQUIRE(lds <= 64 * 1024, "head_project: %d inputs per head do not fit LDS", n_in);
  PYLON_REQUIRE(!(x_dtype == PYLON_F32 && m_dtype == PYLON_BF16), "head_project: float inputs take a float matrix");
  if (tokens == 0) return 0;
  if (x_dtype == PYLON_BF16 && m_dtype == PYLON_BF16 && n_out % 8 == 0 && reinterpret_cast<uintptr_t>(m) % 16 == 0) {
    const size_t wide_lds = sizeof(float) * (HP_TOKENS * n_in + 4 * HP_TOKENS * HW_COLS);
    const int zw = (n_out + HW_COLS - 1) / HW_COLS;
    if (wide_lds <= 64 * 1024 && zw <= 65535) {
      hipLaunchKernelGGL(head_project_wide_kernel, dim3((tokens + HP_TOKENS - 1) / HP_TOKENS, heads, zw),
                         dim3(HP_THREADS), wide_lds, stream, (bf16_t*)out, (const bf16_t*)x, x_stride,
                         (const bf16_t*)m, gate, tokens, heads, n_in, n_out);
      PYLON_LAUNCHED("head_project");
    }
  }
  const int zs = (n_out + HP_COLS - 1) / HP_COLS;
  PYLON_REQUIRE(zs <= 65535, "head_project: too many outputs per head for one launch");
  dim3 grid((tokens + HP_TOKENS - 1) / HP_TOKENS, heads, zs), block(HP_THREADS);
#define GO(TX, TM)                                                                                              \
  hipLaunchKernelGGL((head_project_kernel<TX, TM>), grid, block, lds, stream, (TX*)out, (const TX*)x, x_stride, \
                     (const TM*)m, gate, tokens, heads, n_in, n_out)
  if (x_dtype == PYLON_F32) GO(float, float);
  else if (m_dtype == PYLON_F32) GO(bf16_t, float);
  else GO(bf16_t, bf16_t);
#undef GO
  PYLON_LAUNCHED("head_project");
}

template <typename T>
__global__ void gate_heads_kernel(T* __restrict__ x, const float* __restrict__ gate, long long total, int n_out) {
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < total) x[i] = from_float<T>(to_float(x[i]) * gate[i / n_out]);
}

// x: [tokens * heads, n_out] contiguous, multiplied in place by gate[tokens * heads].
extern "C" int pylon_gate_heads(void* x, int dtype, const float* gate, long long rows, int n_out,
                                hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(dtype), "gate_heads: unknown dtype");
  PYLON_REQUIRE(rows >= 0 && n_out > 0 && gate != nullptr, "gate_heads: bad sizes");
  const long long total = rows * n_out;
  if (total == 0) return 0;
  PYLON_REQUIRE((total + 255) / 256 < (1ll << 31), "gate_heads: too many elements for one launch");
  dim3 grid((unsigned)((total + 255) / 256)), block(256);
  if (dtype == PYLON_F32)
    hipLaunchKernelGGL((gate_heads_kernel<float>), grid, block, 0, stream, (float*)x, gate, total, n_out);
  else
    hipLaunchKernelGGL((gate_heads_kernel<bf16_t>), grid, block, 0, stream, (bf16_t*)x, gate, total, n_out);
  PYLON_LAUNCHED("gate_heads");
}
