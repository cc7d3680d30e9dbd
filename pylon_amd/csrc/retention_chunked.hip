// Retention of bfloat16 prompt portions on the matrix cores, in chunks of 32 tokens.  For the
// tokens 0..n-1 of a chunk, with S the state before it and L the head's decay:
//
//   o_i = L^(i+1) S^T q_i + sum_{j <= i} L^(i-j) (q_i . k_j) v_j
//   S'  = L^n S + sum_j L^(n-1-j) k_j v_j^T
//
// (q and k rotated by their positions, k scaled), then out_i = o_i / rms(o_i) * silu(g_i) as in
// the recurrent form; a chunk's tokens are neighbours in their request, so a token's angle is the
// chunk's first angle plus its steps, and the rotation of token i comes from one sine and cosine
// per frequency and chunk and a table of the steps'.  One workgroup of four waves per (row of the step, head) walks the row's
// chunks in order.  The state stays in float accumulators for the whole walk, every wave
// owning the columns (value elements) of its tiles; everything else of a chunk is staged in LDS.
// All products run as 16x16x32 bfloat16 instructions with float accumulation, and every float
// operand (the rotated q and k, the state, the decayed scores, the decayed keys) enters them as
// two bfloat16 terms, x = hi + lo, products of two such operands as hi*hi + hi*lo + lo*hi: what
// the design keeps in 32 bits is carried with sixteen bits of mantissa or more; v is the
// projection's bfloat16 as it is.  Outputs are computed transposed (rows: value elements,
// columns: tokens), so that a token's norm is a sum within its column's lanes.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

#define RC_CHUNK 32
#define RC_TSTR (RC_CHUNK + 8)  // row of a [element][token] array in LDS, 16-byte aligned

// Upper halves of two floats side by side (a bfloat16 pair, truncated), and of what is left.
__device__ __forceinline__ void rc_split(float a, float b, uint32_t& hi, uint32_t& lo) {
  const uint32_t ua = __float_as_uint(a), ub = __float_as_uint(b);
  hi = __builtin_amdgcn_perm(ub, ua, 0x07060302u);
  const float ra = a - __uint_as_float(ua & 0xffff0000u), rb = b - __uint_as_float(ub & 0xffff0000u);
  lo = __builtin_amdgcn_perm(__float_as_uint(rb), __float_as_uint(ra), 0x07060302u);
}
__device__ __forceinline__ void rc_split1(float a, uint16_t& hi, uint16_t& lo) {
  const uint32_t ua = __float_as_uint(a);
  hi = static_cast<uint16_t>(ua >> 16);
  lo = static_cast<uint16_t>(__float_as_uint(a - __uint_as_float(ua & 0xffff0000u)) >> 16);
}

#define RC_MFMA(a, b, c) __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0)

// KS: slabs of 32 key elements (dim = 32 KS); NVW: tiles of 16 value elements per wave (vdim <= 64 NVW).
// MODE 0: a workgroup walks all chunks of its (row, head) in order.  MODE 1 and 2 take one chunk a
// workgroup (blockIdx.z), for requests too few to fill the chip with one workgroup a head: MODE 1 leaves
// what the chunk alone adds to the state, U_c = sum_j L^(n-1-j) k_j v_j^T, in `chunk_state`; a scan kernel
// turns that into the state before every chunk; MODE 2 computes the chunk's outputs from it.
template <int KS, int NVW, int MODE>
__global__ __launch_bounds__(256) void retention_chunked_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ proj, long long ld, int q_off, int k_off, int v_off, int g_off,
    float* state, const float* __restrict__ decay, const float* __restrict__ inv_freq, int rot_dims,
    const int* __restrict__ positions, const int* __restrict__ row_start, const int* __restrict__ row_slots,
    int heads, int vdim, float eps, float k_scale, float* __restrict__ chunk_state, int max_chunks) {
  constexpr int dim = 32 * KS, ND = 2 * KS;
  constexpr int QSTR = dim + 8;  // row of a [token][element] array in LDS
  extern __shared__ uint16_t rc_lds[];
  uint16_t* q_hi = rc_lds;                      // [32][QSTR]
  uint16_t* q_lo = q_hi + RC_CHUNK * QSTR;
  uint16_t* k_hi = q_lo + RC_CHUNK * QSTR;
  uint16_t* k_lo = k_hi + RC_CHUNK * QSTR;
  uint16_t* kw_hi = k_lo + RC_CHUNK * QSTR;     // [dim][RC_TSTR]: decayed keys, transposed
  uint16_t* kw_lo = kw_hi + dim * RC_TSTR;
  uint16_t* v_t = kw_lo + dim * RC_TSTR;        // [vdim16][RC_TSTR]: values, transposed
  const int vdim16 = (vdim + 15) & ~15;
  float* red = reinterpret_cast<float*>(v_t + vdim16 * RC_TSTR);  // [4][32]
  float* step_c = red + 128;                    // [32][half]: cos and sin of i * frequency, i = 0..31
  float* step_s = step_c + RC_CHUNK * (rot_dims / 2);
  float* base_all = step_s + RC_CHUNK * (rot_dims / 2);  // [2][cos, sin][half]: of a chunk's first position, in turns

  const int row = blockIdx.x, head = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int row_begin = row_start[row], row_end = row_start[row + 1];
  // the tokens this workgroup takes: the whole row, or one chunk of it
  const int begin = MODE == 0 ? row_begin : row_begin + static_cast<int>(blockIdx.z) * RC_CHUNK;
  const int end = MODE == 0 ? row_end : (begin + RC_CHUNK < row_end ? begin + RC_CHUNK : row_end);
  if (begin >= end) return;
  float* st = MODE != 0 ? chunk_state + (((static_cast<size_t>(row) * heads + head) * max_chunks + blockIdx.z) * dim) * vdim :
              state + ((static_cast<size_t>(row_slots[row]) * heads + head) * dim) * vdim;
  const float lam = decay[head];
  const float log2lam = lam > 0.f ? log2f(lam) : -1e30f;  // a decay of zero: every power but the zeroth is zero
  const int half = rot_dims / 2;
  const int n_vt = vdim16 / 16;

  // A chunk's tokens are neighbours: the angle of token i is that of the chunk's first token plus
  // i steps, so a chunk needs one sine and cosine per frequency and the table of the steps'.
  for (int idx = tid; idx < RC_CHUNK * half; idx += 256) {
    const int i = idx / half, pr = idx - i * half;
    sincosf(static_cast<float>(i) * inv_freq[pr], &step_s[idx], &step_c[idx]);
  }
  const bool wide = rot_dims % 16 == 0 && vdim % 8 == 0 && ld % 8 == 0 && q_off % 8 == 0 && k_off % 8 == 0 &&
                    v_off % 8 == 0;  // 16-byte loads of the projection
  const int pos_begin = begin < end ? positions[begin] : 0;
  if (tid < half) sincosf(static_cast<float>(pos_begin) * inv_freq[tid], &base_all[half + tid], &base_all[tid]);
  // With 16-byte loads a chunk travels global -> registers -> LDS, and the registers of the next
  // chunk are filled while this one is computed.
  constexpr int QKI = (KS + 3) / 4;
  u32x4 qk_raw[QKI][4], v_raw[NVW];
  auto fetch = [&](int c0, int n_tok) {
#pragma unroll
    for (int it = 0; it < QKI; ++it) {
      const int idx = tid + it * 256;
      const int tok = idx % RC_CHUNK, pr0 = (idx / RC_CHUNK) * 8;  // neighbours in a wave take neighbouring tokens
      const bool rotated = pr0 < half;
      const int d0 = rotated ? pr0 : rot_dims + 2 * (pr0 - half);
      const int d1 = rotated ? d0 + half : d0 + 8;
#pragma unroll
      for (int a = 0; a < 4; ++a) qk_raw[it][a] = u32x4{0u, 0u, 0u, 0u};
      if (idx < RC_CHUNK * (dim / 16) && tok < n_tok) {
        const bf16_t* pr_row = proj + static_cast<size_t>(c0 + tok) * ld + head * dim;
        qk_raw[it][0] = *reinterpret_cast<const u32x4*>(pr_row + q_off + d0);
        qk_raw[it][1] = *reinterpret_cast<const u32x4*>(pr_row + q_off + d1);
        qk_raw[it][2] = *reinterpret_cast<const u32x4*>(pr_row + k_off + d0);
        qk_raw[it][3] = *reinterpret_cast<const u32x4*>(pr_row + k_off + d1);
      }
    }
#pragma unroll
    for (int it = 0; it < NVW; ++it) {
      const int idx = tid + it * 256;
      const int tok = idx % RC_CHUNK, e0 = (idx / RC_CHUNK) * 8;
      v_raw[it] = u32x4{0u, 0u, 0u, 0u};
      if (idx < RC_CHUNK * (vdim16 / 8) && tok < n_tok && e0 < vdim)
        v_raw[it] = *reinterpret_cast<const u32x4*>(proj + static_cast<size_t>(c0 + tok) * ld + v_off + head * vdim + e0);
    }
  };
  if (wide && begin < end) fetch(begin, end - begin < RC_CHUNK ? end - begin : RC_CHUNK);

  // S[d tile][own value tile]: column = value element, rows = key elements 4 grp + i
  floatx4 s[ND][NVW];
#pragma unroll
  for (int n = 0; n < NVW; ++n) {
    const int e = (wave + 4 * n) * 16 + col;
#pragma unroll
    for (int dt = 0; dt < ND; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        s[dt][n][i] = (MODE != 1 && e < vdim) ? st[static_cast<size_t>(dt * 16 + 4 * grp + i) * vdim + e] : 0.f;
  }

  for (int c0 = begin; c0 < end; c0 += RC_CHUNK) {
    const int n_tok = end - c0 < RC_CHUNK ? end - c0 : RC_CHUNK;
    // ---- stage the chunk: rotated q and k as two terms, decayed keys transposed, values transposed
    const int turn = ((c0 - begin) / RC_CHUNK) & 1;
    const float* base_c = base_all + turn * rot_dims;
    const float* base_s = base_c + half;
    __syncthreads();  // the tables of this chunk's angles are written
    if (wide) {
      // a thread takes eight pairs of one token: elements d0..d0+7 with d0+half.. (rotated), or
      // sixteen neighbours (not rotated)
#pragma unroll
      for (int it = 0; it < QKI; ++it) {
        const int idx = tid + it * 256;
        if (idx >= RC_CHUNK * (dim / 16)) break;
        const int tok = idx % RC_CHUNK, pr0 = (idx / RC_CHUNK) * 8;  // neighbours in a wave take neighbouring tokens
        const bool rotated = pr0 < half;
        const int d0 = rotated ? pr0 : rot_dims + 2 * (pr0 - half);
        const int d1 = rotated ? d0 + half : d0 + 8;
        const u32x4* raw = qk_raw[it];
        float x[4][8];
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
          for (int e = 0; e < 8; ++e)
            x[a][e] = __uint_as_float((e & 1) ? (raw[a][e >> 1] & 0xffff0000u) : (raw[a][e >> 1] << 16));
        if (rotated) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float bc = base_c[pr0 + e], bs = base_s[pr0 + e];
            const float rc = step_c[tok * half + pr0 + e], rs = step_s[tok * half + pr0 + e];
            const float cs = bc * rc - bs * rs, sn = bs * rc + bc * rs;
            const float qa = x[0][e] * cs - x[1][e] * sn, qb = x[1][e] * cs + x[0][e] * sn;
            const float ka = x[2][e] * cs - x[3][e] * sn, kb = x[3][e] * cs + x[2][e] * sn;
            x[0][e] = qa; x[1][e] = qb; x[2][e] = ka; x[3][e] = kb;
          }
        }
        const float w = tok < n_tok ? exp2f(static_cast<float>(n_tok - 1 - tok) * log2lam) : 0.f;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          const int d = (a & 1) ? d1 : d0;
          u32x4 hi, lo;
#pragma unroll
          for (int e = 0; e < 8; e += 2) {
            const float sc = a >= 2 ? k_scale : 1.0f;
            uint32_t h, l;
            rc_split(x[a][e] * sc, x[a][e + 1] * sc, h, l);
            hi[e >> 1] = h;
            lo[e >> 1] = l;
          }
          uint16_t* dst_hi = (a >= 2 ? k_hi : q_hi) + tok * QSTR + d;
          uint16_t* dst_lo = (a >= 2 ? k_lo : q_lo) + tok * QSTR + d;
          *reinterpret_cast<u32x4*>(dst_hi) = hi;
          *reinterpret_cast<u32x4*>(dst_lo) = lo;
          if (a >= 2) {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              rc_split1(x[a][e] * k_scale * w, kw_hi[(d + e) * RC_TSTR + tok], kw_lo[(d + e) * RC_TSTR + tok]);
          }
        }
      }
#pragma unroll
      for (int it = 0; it < NVW; ++it) {
        const int idx = tid + it * 256;
        if (idx >= RC_CHUNK * (vdim16 / 8)) break;
        const int tok = idx % RC_CHUNK, e0 = (idx / RC_CHUNK) * 8;
        const u32x4 raw = v_raw[it];
#pragma unroll
        for (int e = 0; e < 8; ++e)
          v_t[(e0 + e) * RC_TSTR + tok] = static_cast<uint16_t>((e & 1) ? (raw[e >> 1] >> 16) : (raw[e >> 1] & 0xffffu));
      }
    } else {
    for (int idx = tid; idx < RC_CHUNK * (dim / 2); idx += 256) {
      const int tok = idx / (dim / 2), pr = idx - tok * (dim / 2);
      int d0, d1;
      if (pr < half) { d0 = pr; d1 = pr + half; } else { d0 = rot_dims + 2 * (pr - half); d1 = d0 + 1; }
      float q0 = 0.f, q1 = 0.f, k0 = 0.f, k1 = 0.f;
      if (tok < n_tok) {
        const bf16_t* pr_row = proj + static_cast<size_t>(c0 + tok) * ld;
        const bf16_t* qr = pr_row + q_off + head * dim;
        const bf16_t* kr = pr_row + k_off + head * dim;
        q0 = to_float(qr[d0]); q1 = to_float(qr[d1]);
        k0 = to_float(kr[d0]); k1 = to_float(kr[d1]);
        if (pr < half) {
          const float bc = base_c[pr], bs = base_s[pr], rc = step_c[tok * half + pr], rs = step_s[tok * half + pr];
          const float cs = bc * rc - bs * rs, sn = bs * rc + bc * rs;
          const float a = q0 * cs - q1 * sn, b = q1 * cs + q0 * sn;
          q0 = a; q1 = b;
          const float e = k0 * cs - k1 * sn, f = k1 * cs + k0 * sn;
          k0 = e; k1 = f;
        }
        k0 *= k_scale; k1 *= k_scale;
      }
      rc_split1(q0, q_hi[tok * QSTR + d0], q_lo[tok * QSTR + d0]);
      rc_split1(q1, q_hi[tok * QSTR + d1], q_lo[tok * QSTR + d1]);
      rc_split1(k0, k_hi[tok * QSTR + d0], k_lo[tok * QSTR + d0]);
      rc_split1(k1, k_hi[tok * QSTR + d1], k_lo[tok * QSTR + d1]);
      // the key's weight in the state after the chunk: L^(n - 1 - j)
      const float w = tok < n_tok ? exp2f(static_cast<float>(n_tok - 1 - tok) * log2lam) : 0.f;
      rc_split1(k0 * w, kw_hi[d0 * RC_TSTR + tok], kw_lo[d0 * RC_TSTR + tok]);
      rc_split1(k1 * w, kw_hi[d1 * RC_TSTR + tok], kw_lo[d1 * RC_TSTR + tok]);
    }
    for (int idx = tid; idx < RC_CHUNK * vdim16; idx += 256) {
      const int tok = idx / vdim16, e = idx - tok * vdim16;
      uint16_t bits = 0;
      if (tok < n_tok && e < vdim) bits = proj[static_cast<size_t>(c0 + tok) * ld + v_off + head * vdim + e].bits;
      v_t[e * RC_TSTR + tok] = bits;
    }
    }
    __syncthreads();
    if (c0 + RC_CHUNK < end) {
      if (wide) fetch(c0 + RC_CHUNK, end - c0 - RC_CHUNK < RC_CHUNK ? end - c0 - RC_CHUNK : RC_CHUNK);
      // the next chunk's first angle (a row's tokens are neighbours: its position is this one's plus 32)
      float* next = base_all + (turn ^ 1) * rot_dims;
      if (tid < half)
        sincosf(static_cast<float>(pos_begin + (c0 - begin) + RC_CHUNK) * inv_freq[tid], &next[half + tid], &next[tid]);
    }

    floatx4 o[NVW][2];
    if (MODE != 1) {
    // ---- decayed scores, transposed: rows = tokens j, columns = tokens i; p[ti] holds for token
    // i = 16 ti + col the tokens j = 4 grp + i' (first four) and 16 + 4 grp + i' (last four)
    u32x4 p_hi[2], p_lo[2];
#pragma unroll
    for (int ti = 0; ti < 2; ++ti) {
      float pv[8];
#pragma unroll
      for (int tj = 0; tj < 2; ++tj) {
        floatx4 acc = {0.f, 0.f, 0.f, 0.f};
        if (tj <= ti) {
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            const int off = ks * 32 + grp * 8;
            const u32x4 kh = *reinterpret_cast<const u32x4*>(k_hi + (tj * 16 + col) * QSTR + off);
            const u32x4 kl = *reinterpret_cast<const u32x4*>(k_lo + (tj * 16 + col) * QSTR + off);
            const u32x4 qh = *reinterpret_cast<const u32x4*>(q_hi + (ti * 16 + col) * QSTR + off);
            const u32x4 ql = *reinterpret_cast<const u32x4*>(q_lo + (ti * 16 + col) * QSTR + off);
            acc = RC_MFMA(kh, qh, acc);
            acc = RC_MFMA(kh, ql, acc);
            acc = RC_MFMA(kl, qh, acc);
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int dist = (ti * 16 + col) - (tj * 16 + 4 * grp + i);
          pv[tj * 4 + i] = dist >= 0 ? acc[i] * exp2f(static_cast<float>(dist) * log2lam) : 0.f;
        }
      }
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        uint32_t h, l;
        rc_split(pv[e], pv[e + 1], h, l);
        p_hi[ti][e >> 1] = h;
        p_lo[ti][e >> 1] = l;
      }
    }

    // ---- outputs, transposed: rows = value elements of the wave's tiles, columns = tokens
#pragma unroll
    for (int n = 0; n < NVW; ++n) {
      const int dt_e = wave + 4 * n;
      o[n][0] = floatx4{0.f, 0.f, 0.f, 0.f};
      o[n][1] = floatx4{0.f, 0.f, 0.f, 0.f};
      if (dt_e >= n_vt) continue;
      // what the state before the chunk gives: S^T q, the key elements of a slab in the order the
      // accumulators hold them (4 grp + i, then 16 + 4 grp + i)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        u32x4 sh, sl;
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          uint32_t h, l;
          rc_split(s[2 * ks + (e >> 2)][n][e & 3], s[2 * ks + (e >> 2)][n][(e & 3) + 1], h, l);
          sh[e >> 1] = h;
          sl[e >> 1] = l;
        }
#pragma unroll
        for (int ti = 0; ti < 2; ++ti) {
          const uint16_t* qh_row = q_hi + (ti * 16 + col) * QSTR + ks * 32 + 4 * grp;
          const uint16_t* ql_row = q_lo + (ti * 16 + col) * QSTR + ks * 32 + 4 * grp;
          const u32x2 a0 = *reinterpret_cast<const u32x2*>(qh_row), a1 = *reinterpret_cast<const u32x2*>(qh_row + 16);
          const u32x2 b0 = *reinterpret_cast<const u32x2*>(ql_row), b1 = *reinterpret_cast<const u32x2*>(ql_row + 16);
          const u32x4 qh = {a0[0], a0[1], a1[0], a1[1]}, ql = {b0[0], b0[1], b1[0], b1[1]};
          o[n][ti] = RC_MFMA(sh, qh, o[n][ti]);
          o[n][ti] = RC_MFMA(sh, ql, o[n][ti]);
          o[n][ti] = RC_MFMA(sl, qh, o[n][ti]);
        }
      }
#pragma unroll
      for (int ti = 0; ti < 2; ++ti) {
        const float w = exp2f(static_cast<float>(ti * 16 + col + 1) * log2lam);  // L^(i + 1)
        o[n][ti][0] *= w; o[n][ti][1] *= w; o[n][ti][2] *= w; o[n][ti][3] *= w;
      }
      // what the chunk's own tokens give
      const uint16_t* v_row = v_t + (dt_e * 16 + col) * RC_TSTR + 4 * grp;
      const u32x2 v0 = *reinterpret_cast<const u32x2*>(v_row), v1 = *reinterpret_cast<const u32x2*>(v_row + 16);
      const u32x4 vv = {v0[0], v0[1], v1[0], v1[1]};
#pragma unroll
      for (int ti = 0; ti < 2; ++ti) {
        o[n][ti] = RC_MFMA(vv, p_hi[ti], o[n][ti]);
        o[n][ti] = RC_MFMA(vv, p_lo[ti], o[n][ti]);
      }
    }

    }
    if (MODE != 2) {
    // ---- the state after the chunk: S = L^n S + Kw^T V
    const float shrink = exp2f(static_cast<float>(n_tok) * log2lam);
#pragma unroll
    for (int n = 0; n < NVW; ++n) {
      const int dt_e = wave + 4 * n;
      if (dt_e >= n_vt) continue;
      const u32x4 vb = *reinterpret_cast<const u32x4*>(v_t + (dt_e * 16 + col) * RC_TSTR + 8 * grp);
#pragma unroll
      for (int dt = 0; dt < ND; ++dt) {
        const u32x4 kh = *reinterpret_cast<const u32x4*>(kw_hi + (dt * 16 + col) * RC_TSTR + 8 * grp);
        const u32x4 kl = *reinterpret_cast<const u32x4*>(kw_lo + (dt * 16 + col) * RC_TSTR + 8 * grp);
        floatx4 acc = s[dt][n];
        acc[0] *= shrink; acc[1] *= shrink; acc[2] *= shrink; acc[3] *= shrink;
        acc = RC_MFMA(kh, vb, acc);
        s[dt][n] = RC_MFMA(kl, vb, acc);
      }
    }

    }
    if (MODE != 1) {
    // ---- every token's norm over all value elements, the gate, the store
    float sq[2] = {0.f, 0.f};
#pragma unroll
    for (int n = 0; n < NVW; ++n)
#pragma unroll
      for (int ti = 0; ti < 2; ++ti)
#pragma unroll
        for (int i = 0; i < 4; ++i) sq[ti] += o[n][ti][i] * o[n][ti][i];
#pragma unroll
    for (int ti = 0; ti < 2; ++ti) {
      sq[ti] += __shfl_xor(sq[ti], 16, 64);
      sq[ti] += __shfl_xor(sq[ti], 32, 64);
      if (grp == 0) red[wave * 32 + ti * 16 + col] = sq[ti];
    }
    __syncthreads();  // also: every wave is done with the chunk's arrays
#pragma unroll
    for (int ti = 0; ti < 2; ++ti) {
      const int tok = ti * 16 + col;
      const float total = red[tok] + red[32 + tok] + red[64 + tok] + red[96 + tok];
      const float inv = 1.0f / sqrtf(total / static_cast<float>(vdim) + eps);
      if (tok >= n_tok) continue;
      const bf16_t* g_row = proj + static_cast<size_t>(c0 + tok) * ld + g_off + head * vdim;
      bf16_t* o_row = out + (static_cast<size_t>(c0 + tok) * heads + head) * vdim;
      if (wide && g_off % 8 == 0) {
        // four neighbouring value elements a lane: 8-byte loads of the gate, all sent for first
        u32x2 graw[NVW];
#pragma unroll
        for (int n = 0; n < NVW; ++n) {
          const int e0 = (wave + 4 * n) * 16 + 4 * grp;
          graw[n] = u32x2{0u, 0u};
          if (e0 < vdim) graw[n] = *reinterpret_cast<const u32x2*>(g_row + e0);
        }
#pragma unroll
        for (int n = 0; n < NVW; ++n) {
          const int e0 = (wave + 4 * n) * 16 + 4 * grp;
          if (e0 >= vdim) continue;
          float y[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float g = __uint_as_float((i & 1) ? (graw[n][i >> 1] & 0xffff0000u) : (graw[n][i >> 1] << 16));
            y[i] = (o[n][ti][i] * inv) * (g / (1.0f + expf(-g)));
          }
          u32x2 packed;
          packed[0] = static_cast<uint32_t>(float_to_bf16_bits(y[0])) | (static_cast<uint32_t>(float_to_bf16_bits(y[1])) << 16);
          packed[1] = static_cast<uint32_t>(float_to_bf16_bits(y[2])) | (static_cast<uint32_t>(float_to_bf16_bits(y[3])) << 16);
          *reinterpret_cast<u32x2*>(o_row + e0) = packed;
        }
        continue;
      }
#pragma unroll
      for (int n = 0; n < NVW; ++n) {
        const int e0 = (wave + 4 * n) * 16 + 4 * grp;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (e0 + i < vdim) {
            const float g = to_float(g_row[e0 + i]);
            o_row[e0 + i].bits = float_to_bf16_bits((o[n][ti][i] * inv) * (g / (1.0f + expf(-g))));
          }
        }
      }
    }
    }
    __syncthreads();  // red is read before the next chunk's waves write it again
  }

#pragma unroll
  for (int n = 0; n < NVW; ++n) {
    const int e = (wave + 4 * n) * 16 + col;
#pragma unroll
    for (int dt = 0; dt < ND; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (MODE != 2 && e < vdim) st[static_cast<size_t>(dt * 16 + 4 * grp + i) * vdim + e] = s[dt][n][i];
  }
}

// The state before every chunk from what every chunk adds: chunk_state[.., c] holds U_c on entry and
// S_c (the state before chunk c) on exit, S_(c+1) = L^n S_c + U_c; the request's state slot receives
// the state after the last chunk.  One thread an element of the state; a chunk's loads do not wait
// for the chunk before.
__global__ void retention_scan_kernel(float* __restrict__ chunk_state, float* __restrict__ state,
                                      const float* __restrict__ decay, const int* __restrict__ row_start,
                                      const int* __restrict__ row_slots, int heads, int per_head, int max_chunks) {
  const int row = blockIdx.x / heads, head = blockIdx.x - row * heads;
  const int x = blockIdx.y * blockDim.x + threadIdx.x;
  if (x >= per_head) return;
  const int count = row_start[row + 1] - row_start[row];
  const int n_chunks = (count + RC_CHUNK - 1) / RC_CHUNK;
  float* cs = chunk_state + (static_cast<size_t>(row) * heads + head) * max_chunks * per_head + x;
  float* st = state + (static_cast<size_t>(row_slots[row]) * heads + head) * per_head + x;
  const float log2lam = decay[head] > 0.f ? log2f(decay[head]) : -1e30f;
  float sv = *st;
  for (int c0 = 0; c0 < n_chunks; c0 += 8) {
    float u[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) u[i] = (c0 + i < n_chunks) ? cs[static_cast<size_t>(c0 + i) * per_head] : 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (c0 + i >= n_chunks) break;
      const int left = count - (c0 + i) * RC_CHUNK;
      const float shrink = exp2f(static_cast<float>(left < RC_CHUNK ? left : RC_CHUNK) * log2lam);
      cs[static_cast<size_t>(c0 + i) * per_head] = sv;
      sv = fmaf(shrink, sv, u[i]);
    }
  }
  *st = sv;
}

// Arguments as for the recurrent form (bfloat16 only): proj [tokens, ld] with q, k, v and the gate
// at their offsets; out [tokens, heads * vdim]; state float [slots, heads, dim, vdim].  dim a
// multiple of 32 up to 256, vdim up to 256, rot_dims even and at most dim.
extern "C" int pylon_retention_chunked(void* out, const void* proj, long long ld, int q_off, int k_off, int v_off,
                                       int g_off, float* state, const float* decay, const float* inv_freq,
                                       int rot_dims, const int* positions, const int* row_start, const int* row_slots,
                                       int rows, int heads, int dim, int vdim, float eps, float k_scale,
                                       int max_count, float* chunk_state, long long chunk_floats,
                                       hipStream_t stream) {
  PYLON_REQUIRE(rows >= 0 && heads > 0, "retention_chunked: bad sizes");
  PYLON_REQUIRE(dim >= 32 && dim % 32 == 0 && dim <= 256, "retention_chunked: keys of a multiple of 32 up to 256 elements, got %d", dim);
  PYLON_REQUIRE(vdim >= 1 && vdim <= 256, "retention_chunked: values of up to 256 elements, got %d", vdim);
  PYLON_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dim && (dim - rot_dims) % 2 == 0,
                "retention_chunked: rot_dims %d does not fit a head of %d", rot_dims, dim);
  PYLON_REQUIRE(rot_dims == 0 || inv_freq != nullptr, "retention_chunked: a rotation needs its frequencies");
  if (rows == 0) return 0;
  const int vdim16 = (vdim + 15) & ~15;
  const int nvw = (vdim16 / 16 + 3) / 4;
  const size_t lds = 2 * (4 * static_cast<size_t>(RC_CHUNK) * (dim + 8) + 2 * static_cast<size_t>(dim) * RC_TSTR +
                          static_cast<size_t>(vdim16) * RC_TSTR) + sizeof(float) * (128 + (RC_CHUNK + 2) * rot_dims);
  // chunk_state given: one workgroup a chunk, in three launches (contributions, scan, outputs)
  const int max_chunks = (max_count + RC_CHUNK - 1) / RC_CHUNK;
  PYLON_REQUIRE(chunk_state == nullptr ||
                    (max_count >= 1 && chunk_floats >= static_cast<long long>(rows) * heads * max_chunks * dim * vdim),
                "retention_chunked: the chunks' states need rows x heads x chunks x dim x vdim floats");
  const int mode = chunk_state != nullptr ? 1 : 0;
  dim3 grid(rows, heads, mode ? max_chunks : 1), block(256);
#define LAUNCH(KS, NVW, MODE) \
  do { \
    if (lds > 48 * 1024) \
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&retention_chunked_kernel<KS, NVW, MODE>), \
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)); \
    hipLaunchKernelGGL((retention_chunked_kernel<KS, NVW, MODE>), grid, block, lds, stream, (bf16_t*)out, \
                       (const bf16_t*)proj, ld, q_off, k_off, v_off, g_off, state, decay, inv_freq, rot_dims, \
                       positions, row_start, row_slots, heads, vdim, eps, k_scale, chunk_state, max_chunks); \
  } while (0)
#define GO(KS, NVW) \
  do { \
    if (mode == 0) { \
      LAUNCH(KS, NVW, 0); \
    } else { \
      LAUNCH(KS, NVW, 1); \
      hipLaunchKernelGGL(retention_scan_kernel, dim3(rows * heads, (dim * vdim + 255) / 256), dim3(256), 0, stream, \
                         chunk_state, state, decay, row_start, row_slots, heads, dim * vdim, max_chunks); \
      LAUNCH(KS, NVW, 2); \
    } \
  } while (0)
#define PICK(KS)                    \
  do {                              \
    if (nvw <= 1) GO(KS, 1);        \
    else if (nvw <= 2) GO(KS, 2);   \
    else GO(KS, 4);                 \
  } while (0)
  switch (dim / 32) {
    case 1: PICK(1); break;
    case 2: PICK(2); break;
    case 3: PICK(3); break;
    case 4: PICK(4); break;
    case 5: PICK(5); break;
    case 6: PICK(6); break;
    case 7: PICK(7); break;
    default: PICK(8); break;
  }
#undef PICK
#undef GO
#undef LAUNCH
  PYLON_LAUNCHED("retention_chunked");
}
