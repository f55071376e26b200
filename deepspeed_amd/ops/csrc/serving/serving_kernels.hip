// Ragged-batch row kernels for MI355X (gfx950): single-gain RMS norm, norm +
// short causal convolution with carried state, residual add with row
// statistics, feed-forward activations, routers and the routed-expert
// combine. Attention and recurrent mixers live in libraries of their own.
//
// Plain C ABI (raw device pointers + a hipStream_t) so the library builds in
// seconds with hipcc alone and is loaded through ctypes. dtype codes:
// 0 = float, 1 = bfloat16. Everything the models define as 32-bit (norm
// statistics, rotations, scores, softmax, the weighted sums, router and
// gates) is computed in float here whatever the storage type.

#include "serving_common.h"

namespace {

// ---------------------------------------------------------------- norm
// out[r] = x[idx ? idx[r] : r] * rsqrt(mean(x^2) + eps) * gain
template <typename TI, typename TO>
__global__ __launch_bounds__(NT) void scalar_rms_norm_k(
    const TI* __restrict__ x, const int64_t* __restrict__ idx,
    const float* __restrict__ gain, TO* __restrict__ out, int C, float eps) {
  __shared__ float red[NT / 64];
  const int64_t r = blockIdx.x;
  const TI* row = x + (idx ? idx[r] : r) * (int64_t)C;
  float ss = 0.f;
  for (int c = threadIdx.x; c < C; c += NT) {
    float v = ld(row + c);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float k = rsqrtf(ss / (float)C + eps) * gain[0];
  for (int c = threadIdx.x; c < C; c += NT) st(out + r * C + c, ld(row + c) * k);
}


// ------------------------------------------------- layer norm on rows
// v = (in - mean) / sqrt(var + eps) * w + b over one row (var = mean squared
// deviation, fp32). ADD: x[r] += v and `out` (optional) receives the new x
// rounded to TO; otherwise out[r] = v. `idx` (optional) gathers input rows.
template <typename TI, typename TO, bool ADD>
__global__ __launch_bounds__(NT) void layer_norm_k(
    const TI* __restrict__ in, const int64_t* __restrict__ idx,
    const float* __restrict__ w, const float* __restrict__ b, float* __restrict__ x,
    TO* __restrict__ out, int C, float eps) {
  __shared__ float red[NT / 64];
  const int64_t r = blockIdx.x;
  const TI* row = in + (idx ? idx[r] : r) * (int64_t)C;
  float sum = 0.f;
  for (int c = threadIdx.x; c < C; c += NT) sum += ld(row + c);
  const float mean = block_sum(sum, red) / (float)C;
  float ss = 0.f;
  for (int c = threadIdx.x; c < C; c += NT) {
    const float d = ld(row + c) - mean;
    ss += d * d;
  }
  const float inv = rsqrtf(block_sum(ss, red) / (float)C + eps);
  for (int c = threadIdx.x; c < C; c += NT) {
    float v = (ld(row + c) - mean) * inv * w[c] + b[c];
    if (ADD) {
      v += x[r * C + c];
      x[r * C + c] = v;
      if (out) st(out + r * C + c, v);
    } else {
      st(out + r * C + c, v);
    }
  }
}

// The same with eight columns per thread and the row kept in registers over
// the three passes (C a multiple of 8, at most 8 * NT * LN_G).
constexpr int LN_G = 4;
template <typename TI, typename TO, bool ADD>
__global__ __launch_bounds__(NT) void layer_norm_vec_k(
    const TI* __restrict__ in, const int64_t* __restrict__ idx,
    const float* __restrict__ w, const float* __restrict__ b, float* __restrict__ x,
    TO* __restrict__ out, int C, float eps) {
  __shared__ float red[NT / 64];
  const int64_t r = blockIdx.x;
  const TI* row = in + (idx ? idx[r] : r) * (int64_t)C;
  float v[LN_G][8];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < LN_G; ++i) {
    const int c = (threadIdx.x + i * NT) * 8;
    if (c < C) {
      load8(row + c, v[i]);
#pragma unroll
      for (int e = 0; e < 8; ++e) sum += v[i][e];
    }
  }
  const float mean = block_sum(sum, red) / (float)C;
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < LN_G; ++i) {
    const int c = (threadIdx.x + i * NT) * 8;
    if (c < C) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        v[i][e] -= mean;
        ss += v[i][e] * v[i][e];
      }
    }
  }
  const float inv = rsqrtf(block_sum(ss, red) / (float)C + eps);
#pragma unroll
  for (int i = 0; i < LN_G; ++i) {
    const int c = (threadIdx.x + i * NT) * 8;
    if (c < C) {
      float wv[8], bv[8];
      load8(w + c, wv);
      load8(b + c, bv);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[i][e] = v[i][e] * inv * wv[e] + bv[e];
      if (ADD) {
        float xv[8];
        load8(x + r * C + c, xv);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] += xv[e];
        store8(x + r * C + c, v[i]);
        if (out) store8(out + r * C + c, v[i]);
      } else {
        store8(out + r * C + c, v[i]);
      }
    }
  }
}

// out[r] = table[ids[r]] * scale (+ table2[ids2[r]]) (fp32)
template <typename T>
__global__ __launch_bounds__(NT) void embed_rows_k(
    const T* __restrict__ table, const int64_t* __restrict__ ids, const T* __restrict__ table2,
    const int64_t* __restrict__ ids2, float* __restrict__ out, int C, float scale) {
  const int64_t r = blockIdx.x;
  const T* row = table + ids[r] * (int64_t)C;
  const T* row2 = table2 ? table2 + ids2[r] * (int64_t)C : nullptr;
  for (int c = threadIdx.x; c < C; c += NT) {
    float v = ld(row + c) * scale;
    if (row2) v += ld(row2 + c);
    out[r * C + c] = v;
  }
}

// Row of a hashed pair table for every token of a ragged step:
// (previous * mul_prev + current * mul_cur) mod buckets, and row `buckets` for
// a sequence's first token. The previous token of a step's first token is the
// slot's carried one. pair_hash_tail_k then stores each sequence's last token
// (a launch of its own: every read of the old value has finished).
__global__ void pair_hash_rows_k(const int64_t* __restrict__ ids, const int* __restrict__ cu,
                                 const int* __restrict__ seq_slot, const int* __restrict__ tok_seq,
                                 const int* __restrict__ tok_pos, const int64_t* __restrict__ prev,
                                 int64_t* __restrict__ rows, int Ttok, int64_t mul_prev,
                                 int64_t mul_cur, int64_t buckets) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= Ttok) return;
  if (tok_pos[t] == 0) {
    rows[t] = buckets;
    return;
  }
  const int s = tok_seq[t];
  const int64_t before = t > cu[s] ? ids[t - 1] : prev[seq_slot[s]];
  rows[t] = (before * mul_prev + ids[t] * mul_cur) % buckets;
}
__global__ void pair_hash_tail_k(const int64_t* __restrict__ ids, const int* __restrict__ cu,
                                 const int* __restrict__ seq_slot, int64_t* __restrict__ prev,
                                 int nseq) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s < nseq && cu[s + 1] > cu[s]) prev[seq_slot[s]] = ids[cu[s + 1] - 1];
}

// ------------------------------------------------- norm + causal conv
constexpr int MAXTAPS = 32;

// One block per token. h = round_T(norm(x)); out = h_t + sum_k w[c][taps-1-k]
// * h_(t-k). Earlier inputs come from this step's rows when the sequence
// brought them, from the slot's tail otherwise, and are zero before position 0.
template <typename T>
__global__ __launch_bounds__(NT) void norm_conv_k(
    const float* __restrict__ x, const float* __restrict__ gain,
    const T* __restrict__ w, const T* __restrict__ state,
    int64_t state_slot_stride, const int* __restrict__ cu,
    const int* __restrict__ seq_slot, const int* __restrict__ tok_seq,
    const int* __restrict__ tok_pos, T* __restrict__ out, int C, int taps,
    float eps) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x;
  const int s = tok_seq[t];
  const int j = t - cu[s];
  const int pos = tok_pos[t];
  const int tail = taps - 1;
  const T* sl = state + (int64_t)seq_slot[s] * state_slot_stride;
  float scale[MAXTAPS];  // per distance k: norm factor of an in-step row
  const float g = gain[0];
  for (int k = 0; k < taps; ++k) {
    scale[k] = 0.f;
    if (k <= j) {  // block-uniform
      const float* row = x + (int64_t)(t - k) * C;
      float ss = 0.f;
      for (int c = threadIdx.x; c < C; c += NT) ss += row[c] * row[c];
      ss = block_sum(ss, red);
      scale[k] = rsqrtf(ss / (float)C + eps) * g;
    }
  }
  for (int c = threadIdx.x; c < C; c += NT) {
    float h0 = rnd<T>(x[(int64_t)t * C + c] * scale[0]);
    float acc = ld(w + (int64_t)c * taps + tail) * h0;
    for (int k = 1; k < taps; ++k) {
      float hk;
      if (pos - k < 0) break;
      if (k <= j)
        hk = rnd<T>(x[(int64_t)(t - k) * C + c] * scale[k]);
      else
        hk = ld(sl + (int64_t)(tail + j - k) * C + c);
      acc += ld(w + (int64_t)c * taps + tail - k) * hk;
    }
    st(out + (int64_t)t * C + c, h0 + acc);
  }
}

// Tiled form for the usual short filters: a block owns CONV_TOKS consecutive
// tokens, computes each row's norm factor once (one wave per row) and then
// slides a register window over the tokens per channel, so a row of the
// stream is read twice instead of once per tap.
constexpr int CONV_TOKS = 8;

template <int VEC>
__device__ __forceinline__ void ld_vec(const float* p, float (&v)[VEC]) {
  if (VEC == 4) {
    const float4 q = *reinterpret_cast<const float4*>(p);
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[VEC - 1] = q.w;
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = p[i];
  }
}
template <int VEC>
__device__ __forceinline__ void st_vec(float* p, const float (&v)[VEC]) {
  if (VEC == 4) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[VEC - 1]);
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) p[i] = v[i];
  }
}
template <int VEC>
__device__ __forceinline__ void st_vec(bf16* p, const float (&v)[VEC]) {
  if (VEC == 4) {
    uint2 q;
    q.x = (unsigned short)f2bf_bits(v[0]) | ((unsigned)(unsigned short)f2bf_bits(v[1]) << 16);
    q.y = (unsigned short)f2bf_bits(v[2]) | ((unsigned)(unsigned short)f2bf_bits(v[VEC - 1]) << 16);
    *reinterpret_cast<uint2*>(p) = q;
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) p[i] = __float2bfloat16(v[i]);
  }
}

template <typename T, int TAPS, int VEC>
__global__ __launch_bounds__(NT) void norm_conv_tile_k(
    const float* __restrict__ x, const float* __restrict__ gain,
    const T* __restrict__ w, const T* __restrict__ state,
    int64_t state_slot_stride, const int* __restrict__ cu,
    const int* __restrict__ seq_slot, const int* __restrict__ tok_seq,
    const int* __restrict__ tok_pos, T* __restrict__ out,
    const float* __restrict__ sumsq,  // optional: sum of x^2 per row
    int Ttok, int C, float eps) {
  constexpr int TAIL = TAPS - 1;
  constexpr int NR = CONV_TOKS + TAIL;
  __shared__ float rinv[NR];
  __shared__ int meta[CONV_TOKS][3];  // offset in its sequence's step, position, slot
  const int t0 = blockIdx.x * CONV_TOKS;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const float g = gain[0];
  if (threadIdx.x < CONV_TOKS && t0 + threadIdx.x < Ttok) {
    const int t = t0 + threadIdx.x, s = tok_seq[t];
    meta[threadIdx.x][0] = t - cu[s];
    meta[threadIdx.x][1] = tok_pos[t];
    meta[threadIdx.x][2] = seq_slot[s];
  }
  if (sumsq) {  // the producer of x already summed its squares
    if (threadIdx.x < NR) {
      const int tt = t0 - TAIL + threadIdx.x;
      const float ss = (tt >= 0 && tt < Ttok) ? sumsq[tt] : 0.f;
      rinv[threadIdx.x] = rsqrtf(ss / (float)C + eps) * g;
    }
  } else
  for (int ri = wid; ri < NR; ri += NT / 64) {
    const int tt = t0 - TAIL + ri;
    float ss = 0.f;
    if (tt >= 0 && tt < Ttok) {
      const float* row = x + (int64_t)tt * C;
      for (int c = lane * VEC; c < C; c += 64 * VEC) {
        float v[VEC];
        ld_vec<VEC>(row + c, v);
#pragma unroll
        for (int i = 0; i < VEC; ++i) ss += v[i] * v[i];
      }
    }
    ss = wave_sum(ss);
    if (lane == 0) rinv[ri] = rsqrtf(ss / (float)C + eps) * g;
  }
  __syncthreads();
  for (int c = threadIdx.x * VEC; c < C; c += NT * VEC) {
    float wv[VEC][TAPS];
#pragma unroll
    for (int v = 0; v < VEC; ++v)
#pragma unroll
      for (int k = 0; k < TAPS; ++k) wv[v][k] = ld(w + (int64_t)(c + v) * TAPS + k);
    float win[TAIL > 0 ? TAIL : 1][VEC];  // win[k-1]: input k tokens back (flat order)
#pragma unroll
    for (int k = 1; k <= TAIL; ++k) {
      const int tt = t0 - k;
      float xv[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) xv[v] = 0.f;
      if (tt >= 0) ld_vec<VEC>(x + (int64_t)tt * C + c, xv);
#pragma unroll
      for (int v = 0; v < VEC; ++v) win[k - 1][v] = rnd<T>(xv[v] * rinv[TAIL - k]);
    }
    float xs[CONV_TOKS][VEC];
#pragma unroll
    for (int i = 0; i < CONV_TOKS; ++i) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) xs[i][v] = 0.f;
      if (t0 + i < Ttok) ld_vec<VEC>(x + (int64_t)(t0 + i) * C + c, xs[i]);
    }
#pragma unroll
    for (int i = 0; i < CONV_TOKS; ++i) {
      const int t = t0 + i;
      if (t < Ttok) {
        const int j = meta[i][0], pos = meta[i][1];
        const T* sl = state + (int64_t)meta[i][2] * state_slot_stride;
        float h0[VEC], res[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          h0[v] = rnd<T>(xs[i][v] * rinv[TAIL + i]);
          res[v] = wv[v][TAIL] * h0[v];
        }
#pragma unroll
        for (int k = 1; k <= TAIL; ++k) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            float hk;
            if (k <= j)
              hk = win[k - 1][v];
            else if (pos - k < 0)
              hk = 0.f;
            else
              hk = ld(sl + (int64_t)(TAIL + j - k) * C + c + v);
            res[v] += wv[v][TAIL - k] * hk;
          }
        }
#pragma unroll
        for (int v = 0; v < VEC; ++v) res[v] += h0[v];
        st_vec<VEC>(out + (int64_t)t * C + c, res);
#pragma unroll
        for (int k = TAIL; k >= 2; --k)
#pragma unroll
          for (int v = 0; v < VEC; ++v) win[k - 1][v] = win[k - 2][v];
        if (TAIL > 0) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) win[0][v] = h0[v];
        }
      }
    }
  }
}

// x += delta (fp32 stream, delta in the compute type) and the sum of squares
// of every updated row, which the next norm needs: the norm's reduction rides
// on the pass that has to touch the stream anyway.
template <typename T, int VEC>
__global__ __launch_bounds__(NT) void residual_add_stats_k(
    float* __restrict__ x, const T* __restrict__ delta, float* __restrict__ sumsq, int C) {
  __shared__ float red[NT / 64];
  const int64_t r = blockIdx.x;
  float* row = x + r * C;
  const T* drow = delta + r * C;
  float ss = 0.f;
  for (int c = threadIdx.x * VEC; c < C; c += NT * VEC) {
    float v[VEC];
    ld_vec<VEC>(row + c, v);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      v[i] += ld(drow + c + i);
      ss += v[i] * v[i];
    }
    st_vec<VEC>(row + c, v);
  }
  ss = block_sum(ss, red);
  if (threadIdx.x == 0) sumsq[r] = ss;
}

// One block per sequence: the tail becomes the last taps-1 normed inputs.
template <typename T>
__global__ __launch_bounds__(NT) void conv_tail_k(
    const float* __restrict__ x, const float* __restrict__ gain,
    T* __restrict__ state, int64_t state_slot_stride,
    const int* __restrict__ cu, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, const float* __restrict__ sumsq, int C, int taps,
    float eps) {
  __shared__ float red[NT / 64];
  const int s = blockIdx.x;
  const int tail = taps - 1;
  const int start = seq_start[s];
  const int count = cu[s + 1] - cu[s];
  T* sl = state + (int64_t)seq_slot[s] * state_slot_stride;
  float scale[MAXTAPS];
  const float g = gain[0];
  for (int i = 0; i < tail; ++i) {
    scale[i] = 0.f;
    const int p = start + count - tail + i;  // absolute position kept at i
    if (p >= start) {
      float ss;
      if (sumsq) {
        ss = sumsq[cu[s] + p - start];
      } else {
        const float* row = x + (int64_t)(cu[s] + p - start) * C;
        ss = 0.f;
        for (int c = threadIdx.x; c < C; c += NT) ss += row[c] * row[c];
        ss = block_sum(ss, red);
      }
      scale[i] = rsqrtf(ss / (float)C + eps) * g;
    }
  }
  for (int c = threadIdx.x; c < C; c += NT) {
    float v[MAXTAPS];
    for (int i = 0; i < tail; ++i) {
      const int p = start + count - tail + i;
      if (p < 0)
        v[i] = 0.f;
      else if (p >= start)
        v[i] = x[(int64_t)(cu[s] + p - start) * C + c] * scale[i];
      else
        v[i] = ld(sl + (int64_t)(i + count) * C + c);
    }
    for (int i = 0; i < tail; ++i) st(sl + (int64_t)i * C + c, v[i]);
  }
}

// ---------------------------------------------------------- activations
__device__ __forceinline__ float softplusf(float x) {
  return x > 20.f ? x : log1pf(expf(x));
}

template <typename T>
__global__ void xielu_k(const T* __restrict__ z, const float* __restrict__ pq,
                        T* __restrict__ out, int64_t n) {
  const float a = softplusf(pq[0]);
  const float b = 0.5f + softplusf(pq[1]);
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const float v = ld(z + i);
    const float r = v > 0.f ? a * v * v + 0.5f * v : b * (expm1f(v) - v) + 0.5f * v;
    st(out + i, r);
  }
}

// gu [rows, 2F] (gate | up) -> out [rows, F]
template <typename T>
__global__ void clamped_swiglu_k(const T* __restrict__ gu, T* __restrict__ out,
                                 int64_t rows, int F, float limit) {
  const int64_t n = rows * F;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / F;
    const int c = i - r * F;
    const float g = fminf(ld(gu + r * 2 * F + c), limit);
    const float u = fminf(fmaxf(ld(gu + r * 2 * F + F + c), -limit), limit);
    st(out + i, g / (1.f + expf(-1.702f * g)) * (u + 1.f));
  }
}

// the same, eight columns per thread (F a multiple of 8)
template <typename T>
__global__ void clamped_swiglu8_k(const T* __restrict__ gu, T* __restrict__ out, int64_t rows,
                                  int F, float limit) {
  const int F8 = F >> 3;
  const int64_t n = rows * F8;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / F8;
    const int c = (int)(i - r * F8) << 3;
    float g[8], u[8];
    load8(gu + r * 2 * F + c, g);
    load8(gu + r * 2 * F + F + c, u);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float gc = fminf(g[e], limit);
      const float uc = fminf(fmaxf(u[e], -limit), limit);
      g[e] = gc / (1.f + expf(-1.702f * gc)) * (uc + 1.f);
    }
    store8(out + r * F + c, g);
  }
}

// gu [rows, 2F] (gate | up) -> act(gate) * up; ACT 0 = silu, 1 = tanh-form gelu
template <typename T, int ACT>
__global__ void glu_k(const T* __restrict__ gu, T* __restrict__ out, int64_t rows, int F) {
  const int64_t n = rows * F;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / F;
    const int c = i - r * F;
    const float g = ld(gu + r * 2 * F + c);
    const float u = ld(gu + r * 2 * F + F + c);
    float a;
    if (ACT == 0)
      a = g / (1.f + expf(-g));
    else
      a = 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    st(out + i, a * u);
  }
}

// the same, eight columns per thread (F a multiple of 8)
template <typename T, int ACT>
__global__ void glu8_k(const T* __restrict__ gu, T* __restrict__ out, int64_t rows, int F) {
  const int F8 = F >> 3;
  const int64_t n = rows * F8;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / F8;
    const int c = (int)(i - r * F8) << 3;
    float g[8], u[8];
    load8(gu + r * 2 * F + c, g);
    load8(gu + r * 2 * F + F + c, u);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float a = ACT == 0 ? g[e] / (1.f + expf(-g[e]))
                               : 0.5f * g[e] * (1.f + tanhf(0.7978845608028654f *
                                                            (g[e] + 0.044715f * g[e] * g[e] * g[e])));
      g[e] = a * u[e];
    }
    store8(out + r * F + c, g);
  }
}

// Per token: scores s = sigmoid(z), or softmax(z) over all E with SOFTMAX;
// choice c = s + corr. Experts form `groups` equal runs; a group's score is the
// sum of its two largest c (its one when a run holds one expert), or its
// largest alone with `group_max`; only experts of the `keep` best groups
// compete (the others count as minus infinity: c may be negative). The `top`
// largest allowed c are chosen; weights are their s, with `renorm` divided by
// their sum (+ 1e-20), times `scale`.
constexpr int MAXGROUPS = 64;
template <bool SOFTMAX>
__global__ void grouped_topk_k(const float* __restrict__ z, const float* __restrict__ corr,
                               int64_t* __restrict__ idx, float* __restrict__ w, int Ttok, int E,
                               int top, int groups, int keep, int group_max, int renorm,
                               float scale) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= Ttok) return;
  const float* r = z + (int64_t)t * E;
  const int per = E / groups;
  float zmax = 0.f, zinv = 1.f;
  if (SOFTMAX) {
    zmax = -INFINITY;
    for (int e = 0; e < E; ++e) zmax = fmaxf(zmax, r[e]);
    float sum = 0.f;
    for (int e = 0; e < E; ++e) sum += expf(r[e] - zmax);
    zinv = 1.f / sum;
  }
  auto score = [&](int e) -> float {
    return SOFTMAX ? expf(r[e] - zmax) * zinv : 1.f / (1.f + expf(-r[e]));
  };
  unsigned long long allowed = ~0ull;
  if (groups > 1) {
    float gs[MAXGROUPS];
    for (int g = 0; g < groups; ++g) {
      float a = -INFINITY, b2 = -INFINITY;  // largest, second largest
      for (int e = g * per; e < (g + 1) * per; ++e) {
        const float c = score(e) + corr[e];
        if (c > a) {
          b2 = a;
          a = c;
        } else if (c > b2) {
          b2 = c;
        }
      }
      gs[g] = (per > 1 && !group_max) ? a + b2 : a;
    }
    allowed = 0ull;
    for (int k = 0; k < keep; ++k) {
      int bi = -1;
      float bv = -INFINITY;
      for (int g = 0; g < groups; ++g)
        if (!((allowed >> g) & 1ull) && (bi < 0 || gs[g] > bv)) {
          bi = g;
          bv = gs[g];
        }
      allowed |= 1ull << bi;
    }
  }
  float total = 0.f;
  // experts already chosen: a bit each in a register while they fit, else
  // read back from the output row
  unsigned long long chosen = 0ull;
  for (int k = 0; k < top; ++k) {
    int bi = -1;
    float bv = -INFINITY, bs = 0.f;
    for (int e = 0; e < E; ++e) {
      if (!((allowed >> (e / per)) & 1ull)) continue;
      bool taken = false;
      if (E <= 64)
        taken = (chosen >> e) & 1ull;
      else
        for (int q = 0; q < k; ++q) taken |= idx[(int64_t)t * top + q] == e;
      if (taken) continue;
      const float sg = score(e);
      const float c = sg + corr[e];
      if (bi < 0 || c > bv) {
        bi = e;
        bv = c;
        bs = sg;
      }
    }
    idx[(int64_t)t * top + k] = bi;
    w[(int64_t)t * top + k] = bs;
    total += bs;
    if (E <= 64 && bi >= 0) chosen |= 1ull << bi;
  }
  const float f = renorm ? scale / (total + 1e-20f) : scale;
  if (renorm || scale != 1.f)
    for (int k = 0; k < top; ++k) w[(int64_t)t * top + k] *= f;
}

// out[t] = sum_k w[t,k] * y[inv[t,k]] (+ sigmoid(sg[t]) * shared[t]); several
// picks may name one row of y (identity outputs), a row index outside y's
// nrows rows is skipped rather than read
template <typename T>
__global__ void moe_combine_k(const T* __restrict__ y, const int64_t* __restrict__ inv,
                              const float* __restrict__ w, const T* __restrict__ shared,
                              const T* __restrict__ sg, T* __restrict__ out,
                              int top, int C, int64_t nrows) {
  const int64_t t = blockIdx.x;
  const float g = shared ? 1.f / (1.f + expf(-ld(sg + t))) : 0.f;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float a = 0.f;
    for (int k = 0; k < top; ++k) {
      const int64_t r = inv[t * top + k];
      if (r >= 0 && r < nrows) a += w[t * top + k] * ld(y + r * C + c);
    }
    if (shared) a += g * ld(shared + t * C + c);
    st(out + t * C + c, a);
  }
}

// per token: the `top` largest of E logits, softmax over them
__global__ void topk_softmax_k(const float* __restrict__ z, int64_t* __restrict__ idx,
                               float* __restrict__ w, int Ttok, int E, int top) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= Ttok) return;
  const float* r = z + (int64_t)t * E;
  float best = 0.f, sum = 0.f;
  for (int k = 0; k < top; ++k) {
    int bi = -1;
    float bv = -INFINITY;
    for (int e = 0; e < E; ++e) {
      bool taken = false;
      for (int q = 0; q < k; ++q) taken |= idx[(int64_t)t * top + q] == e;
      if (!taken && (bi < 0 || r[e] > bv)) {
        bi = e;
        bv = r[e];
      }
    }
    idx[(int64_t)t * top + k] = bi;
    if (k == 0) best = bv;
    const float p = expf(bv - best);
    w[(int64_t)t * top + k] = p;
    sum += p;
  }
  for (int k = 0; k < top; ++k) w[(int64_t)t * top + k] /= sum;
}


// ------------------------------------------------ weighted RMS norm of rows
// out[r] = x[idx ? idx[r] : r] / sqrt(mean(x^2) + eps) * (w or 1 + w); input
// rows may be a column slice (row stride ld_in). The VEC form keeps the row in
// registers (C a multiple of 8, at most 8*NT*LN_G).
template <typename TI, typename TO, bool VEC>
__global__ __launch_bounds__(NT) void rms_norm_rows_k(
    const TI* __restrict__ in, int ld_in, const int64_t* __restrict__ idx,
    const float* __restrict__ w, TO* __restrict__ out, int C, float eps, float w_add) {
  __shared__ float red[NT / 64];
  const int64_t r = blockIdx.x;
  const TI* row = in + (idx ? idx[r] : r) * (int64_t)ld_in;
  TO* o = out + r * (int64_t)C;
  if (VEC) {
    float v[LN_G][8];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < LN_G; ++i) {
      const int c = (threadIdx.x + i * NT) * 8;
      if (c < C) {
        load8(row + c, v[i]);
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += v[i][e] * v[i][e];
      }
    }
    const float inv = rsqrtf(block_sum(ss, red) / (float)C + eps);
#pragma unroll
    for (int i = 0; i < LN_G; ++i) {
      const int c = (threadIdx.x + i * NT) * 8;
      if (c < C) {
        float wv[8];
        load8(w + c, wv);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] *= inv * (wv[e] + w_add);
        store8(o + c, v[i]);
      }
    }
  } else {
    float ss = 0.f;
    for (int c = threadIdx.x; c < C; c += NT) {
      const float v = ld(row + c);
      ss += v * v;
    }
    const float inv = rsqrtf(block_sum(ss, red) / (float)C + eps);
    for (int c = threadIdx.x; c < C; c += NT) st(o + c, ld(row + c) * inv * (w[c] + w_add));
  }
}

// ---------------------------------------------- sigmoid-gated residual add
// x[r] += sigmoid(g1[r]) * y1[r] (+ sigmoid(g2[r]) * y2[r]) on the float
// stream; with a norm weight the same pass emits the RMS norm of the new row.
// The gates are column slices of a wider projection (row stride ld_g).
__device__ __forceinline__ float sigm(float x) { return 1.f / (1.f + expf(-x)); }

template <typename T, typename TO, bool VEC>
__global__ __launch_bounds__(NT) void gated_add_k(
    float* __restrict__ x, const T* __restrict__ g1, const T* __restrict__ g2, int ld_g,
    const T* __restrict__ y1, const T* __restrict__ y2, const float* __restrict__ w,
    TO* __restrict__ h, int C, float eps, float w_add) {
  __shared__ float red[NT / 64];
  const int64_t r = blockIdx.x;
  float* xr = x + r * C;
  const T* a1 = g1 + r * ld_g;
  const T* a2 = g2 ? g2 + r * ld_g : nullptr;
  const T* b1 = y1 + r * C;
  const T* b2 = y2 ? y2 + r * C : nullptr;
  if (VEC) {
    float v[LN_G][8];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < LN_G; ++i) {
      const int c = (threadIdx.x + i * NT) * 8;
      if (c < C) {
        float g[8], y[8];
        load8(xr + c, v[i]);
        load8(a1 + c, g);
        load8(b1 + c, y);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float d = sigm(g[e]) * y[e];
          g[e] = d;
        }
        if (a2) {
          float g2v[8], y2v[8];
          load8(a2 + c, g2v);
          load8(b2 + c, y2v);
#pragma unroll
          for (int e = 0; e < 8; ++e) g[e] += sigm(g2v[e]) * y2v[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          v[i][e] += g[e];
          ss += v[i][e] * v[i][e];
        }
        store8(xr + c, v[i]);
      }
    }
    if (!w) return;
    const float inv = rsqrtf(block_sum(ss, red) / (float)C + eps);
#pragma unroll
    for (int i = 0; i < LN_G; ++i) {
      const int c = (threadIdx.x + i * NT) * 8;
      if (c < C) {
        float wv[8];
        load8(w + c, wv);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] *= inv * (wv[e] + w_add);
        store8(h + r * C + c, v[i]);
      }
    }
  } else {
    float ss = 0.f;
    for (int c = threadIdx.x; c < C; c += NT) {
      float d = sigm(ld(a1 + c)) * ld(b1 + c);
      if (a2) d += sigm(ld(a2 + c)) * ld(b2 + c);
      const float v = xr[c] + d;
      xr[c] = v;
      ss += v * v;
    }
    if (!w) return;
    const float inv = rsqrtf(block_sum(ss, red) / (float)C + eps);
    for (int c = threadIdx.x; c < C; c += NT) st(h + r * C + c, xr[c] * inv * (w[c] + w_add));
  }
}

// ------------------------------------- scaled residual add, paired norms
// x[r] += s1 * y1[r] (+ s2 * y2[r]) (+ extra[r]) on the float stream, s1/s2 one
// factor per column (y1 may be null: nothing is added, the row is only normed).
// With w1 (and w2) the same pass emits the RMS norm of the new row under each
// weight: two sublayers that read the same row through norms of their own
// share one read and one statistic.
template <typename T, typename TO, bool VEC>
__global__ __launch_bounds__(NT) void scaled_add_k(
    float* __restrict__ x, const float* __restrict__ s1, const T* __restrict__ y1,
    const float* __restrict__ s2, const T* __restrict__ y2, const float* __restrict__ extra,
    const float* __restrict__ w1, const float* __restrict__ w2, TO* __restrict__ h1,
    TO* __restrict__ h2, int C, float eps) {
  __shared__ float red[NT / 64];
  const int64_t r = blockIdx.x;
  float* xr = x + r * C;
  const T* b1 = y1 ? y1 + r * C : nullptr;
  const T* b2 = y2 ? y2 + r * C : nullptr;
  const float* ex = extra ? extra + r * C : nullptr;
  if (VEC) {
    float v[LN_G][8];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < LN_G; ++i) {
      const int c = (threadIdx.x + i * NT) * 8;
      if (c < C) {
        load8(xr + c, v[i]);
        if (b1) {
          float d[8], y[8], sc[8];
          load8(b1 + c, y);
          load8(s1 + c, sc);
#pragma unroll
          for (int e = 0; e < 8; ++e) d[e] = sc[e] * y[e];
          if (b2) {
            load8(b2 + c, y);
            load8(s2 + c, sc);
#pragma unroll
            for (int e = 0; e < 8; ++e) d[e] += sc[e] * y[e];
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) v[i][e] += d[e];
        }
        if (ex) {
          float y[8];
          load8(ex + c, y);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[i][e] += y[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += v[i][e] * v[i][e];
        if (b1 || ex) store8(xr + c, v[i]);
      }
    }
    if (!w1) return;
    const float inv = rsqrtf(block_sum(ss, red) / (float)C + eps);
#pragma unroll
    for (int i = 0; i < LN_G; ++i) {
      const int c = (threadIdx.x + i * NT) * 8;
      if (c < C) {
        float wv[8], o[8];
        load8(w1 + c, wv);
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = v[i][e] * inv * wv[e];
        store8(h1 + r * C + c, o);
        if (w2) {
          load8(w2 + c, wv);
#pragma unroll
          for (int e = 0; e < 8; ++e) o[e] = v[i][e] * inv * wv[e];
          store8(h2 + r * C + c, o);
        }
      }
    }
  } else {
    float ss = 0.f;
    for (int c = threadIdx.x; c < C; c += NT) {
      float v = xr[c];
      if (b1) {
        float d = s1[c] * ld(b1 + c);
        if (b2) d += s2[c] * ld(b2 + c);
        v += d;
      }
      if (ex) v += ex[c];
      if (b1 || ex) xr[c] = v;
      ss += v * v;
    }
    if (!w1) return;
    const float inv = rsqrtf(block_sum(ss, red) / (float)C + eps);
    for (int c = threadIdx.x; c < C; c += NT) {
      const float v = xr[c] * inv;
      st(h1 + r * C + c, v * w1[c]);
      if (w2) st(h2 + r * C + c, v * w2[c]);
    }
  }
}

// -------------------------------------------------- plain row activations
// ACT: 0 = exact GELU (erf), 1 = tanh GELU, 2 = SiLU; z is a column slice
// with row stride ld_z, out is contiguous.
template <int ACT>
__device__ __forceinline__ float row_act(float z) {
  if (ACT == 0) return 0.5f * z * (1.f + erff(z * 0.70710678118654752f));
  if (ACT == 1) return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  return z / (1.f + expf(-z));
}

template <typename T, int ACT, bool VEC>
__global__ void act_rows_k(const T* __restrict__ z, int ld_z, T* __restrict__ out,
                           int64_t rows, int F) {
  if (VEC) {
    const int F8 = F / 8;
    const int64_t n = rows * F8;
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
         i += (int64_t)gridDim.x * blockDim.x) {
      const int64_t r = i / F8;
      const int c = (int)(i - r * F8) * 8;
      float v[8];
      load8(z + r * ld_z + c, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = row_act<ACT>(v[e]);
      store8(out + r * F + c, v);
    }
  } else {
    const int64_t n = rows * F;
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
         i += (int64_t)gridDim.x * blockDim.x) {
      const int64_t r = i / F;
      const int c = (int)(i - r * F);
      st(out + i, row_act<ACT>(ld(z + r * ld_z + c)));
    }
  }
}

}  // namespace

extern "C" {

int dsv_scalar_rms_norm(const void* x, int in_dt, const int64_t* idx, const float* gain,
                        void* out, int out_dt, int rows, int C, float eps, hipStream_t s) {
  if (rows <= 0) return 0;
  if (in_dt == 0 && out_dt == 0)
    scalar_rms_norm_k<float, float><<<rows, NT, 0, s>>>((const float*)x, idx, gain, (float*)out, C, eps);
  else if (in_dt == 0)
    scalar_rms_norm_k<float, bf16><<<rows, NT, 0, s>>>((const float*)x, idx, gain, (bf16*)out, C, eps);
  else if (out_dt == 0)
    scalar_rms_norm_k<bf16, float><<<rows, NT, 0, s>>>((const bf16*)x, idx, gain, (float*)out, C, eps);
  else
    scalar_rms_norm_k<bf16, bf16><<<rows, NT, 0, s>>>((const bf16*)x, idx, gain, (bf16*)out, C, eps);
  return (int)hipGetLastError();
}

int dsv_norm_conv(const float* x, const float* gain, const void* w, void* state,
                  int64_t state_slot_stride, const int* cu, const int* seq_slot,
                  const int* seq_start, const int* tok_seq, const int* tok_pos, void* out,
                  const float* sumsq, int dt, int Ttok, int nseq, int C, int taps, float eps,
                  hipStream_t s) {
  if (taps > MAXTAPS) return -1;
  if (Ttok <= 0) return 0;
  const int tiles = (Ttok + CONV_TOKS - 1) / CONV_TOKS;
#define TILE(N)                                                                              \
  case N:                                                                                    \
    if (C % 4 == 0)                                                                          \
      BY_DTYPE(dt, (norm_conv_tile_k<T, N, 4><<<tiles, NT, 0, s>>>(                          \
                       x, gain, (const T*)w, (const T*)state, state_slot_stride, cu,         \
                       seq_slot, tok_seq, tok_pos, (T*)out, sumsq, Ttok, C, eps)));          \
    else                                                                                     \
      BY_DTYPE(dt, (norm_conv_tile_k<T, N, 1><<<tiles, NT, 0, s>>>(                          \
                       x, gain, (const T*)w, (const T*)state, state_slot_stride, cu,         \
                       seq_slot, tok_seq, tok_pos, (T*)out, sumsq, Ttok, C, eps)));          \
    break
  switch (taps) {
    TILE(1);
    TILE(2);
    TILE(3);
    TILE(4);
    TILE(5);
    TILE(6);
    TILE(7);
    TILE(8);
    default:
      BY_DTYPE(dt, (norm_conv_k<T><<<Ttok, NT, 0, s>>>(x, gain, (const T*)w, (const T*)state,
                                                        state_slot_stride, cu, seq_slot,
                                                        tok_seq, tok_pos, (T*)out, C, taps,
                                                        eps)));
  }
#undef TILE
  if (taps > 1)
    BY_DTYPE(dt, (conv_tail_k<T><<<nseq, NT, 0, s>>>(x, gain, (T*)state, state_slot_stride, cu,
                                                      seq_slot, seq_start, sumsq, C, taps, eps)));
  return (int)hipGetLastError();
}

int dsv_residual_add_stats(float* x, const void* delta, float* sumsq, int dt, int rows, int C,
                           hipStream_t s) {
  if (rows <= 0) return 0;
  if (C % 4 == 0)
    BY_DTYPE(dt, (residual_add_stats_k<T, 4><<<rows, NT, 0, s>>>(x, (const T*)delta, sumsq, C)));
  else
    BY_DTYPE(dt, (residual_add_stats_k<T, 1><<<rows, NT, 0, s>>>(x, (const T*)delta, sumsq, C)));
  return (int)hipGetLastError();
}

// in_dt/out_dt: 0 float, 1 bf16. add != 0: x += norm(in) and `out` (may be null)
// gets the rounded new x; add == 0: out = norm(in[idx]).
int dsv_layer_norm(const void* in, int in_dt, const int64_t* idx, const float* w, const float* b,
                   float* x, void* out, int out_dt, int add, int rows, int C, float eps,
                   hipStream_t s) {
  if (rows <= 0) return 0;
  if (add && !x) return -1;
  if (!add && !out) return -1;
#define LN(TI, TO, ADD)                                                                     \
  do {                                                                                      \
    if (C % 8 == 0 && C <= 8 * NT * LN_G)                                                   \
      layer_norm_vec_k<TI, TO, ADD><<<rows, NT, 0, s>>>((const TI*)in, idx, w, b, x,         \
                                                        (TO*)out, C, eps);                  \
    else                                                                                    \
      layer_norm_k<TI, TO, ADD><<<rows, NT, 0, s>>>((const TI*)in, idx, w, b, x, (TO*)out,   \
                                                    C, eps);                                \
  } while (0)
  if (add) {
    if (in_dt == 0 && out_dt == 0) LN(float, float, true);
    else if (in_dt == 0) LN(float, bf16, true);
    else if (out_dt == 0) LN(bf16, float, true);
    else LN(bf16, bf16, true);
  } else {
    if (in_dt == 0 && out_dt == 0) LN(float, float, false);
    else if (in_dt == 0) LN(float, bf16, false);
    else if (out_dt == 0) LN(bf16, float, false);
    else LN(bf16, bf16, false);
  }
#undef LN
  return (int)hipGetLastError();
}

int dsv_embed_rows(const void* table, int dt, const int64_t* ids, const void* table2,
                   const int64_t* ids2, float* out, int rows, int C, float scale, hipStream_t s) {
  if (rows <= 0) return 0;
  if ((table2 == nullptr) != (ids2 == nullptr)) return -1;
  BY_DTYPE(dt, (embed_rows_k<T><<<rows, NT, 0, s>>>((const T*)table, ids, (const T*)table2, ids2,
                                                    out, C, scale)));
  return (int)hipGetLastError();
}

int dsv_pair_hash_rows(const int64_t* ids, const int* cu, const int* seq_slot, const int* tok_seq,
                       const int* tok_pos, int64_t* prev, int64_t* rows, int Ttok, int nseq,
                       int64_t mul_prev, int64_t mul_cur, int64_t buckets, hipStream_t s) {
  if (buckets < 1 || mul_prev < 0 || mul_cur < 0) return -1;
  if (Ttok <= 0) return 0;
  pair_hash_rows_k<<<(Ttok + 255) / 256, 256, 0, s>>>(ids, cu, seq_slot, tok_seq, tok_pos, prev,
                                                      rows, Ttok, mul_prev, mul_cur, buckets);
  pair_hash_tail_k<<<(nseq + 63) / 64, 64, 0, s>>>(ids, cu, seq_slot, prev, nseq);
  return (int)hipGetLastError();
}

int dsv_glu(const void* gu, void* out, int dt, int64_t rows, int F, int act, hipStream_t s) {
  if (rows * F <= 0) return 0;
  if (act != 0 && act != 1) return -1;
  if (F % 8 == 0) {
    const int64_t n = rows * (F / 8);
    const int g = (int)((n + 255) / 256 < 1 ? 1 : ((n + 255) / 256 > 65535 * 4 ? 65535 * 4 : (n + 255) / 256));
    if (act == 0)
      BY_DTYPE(dt, (glu8_k<T, 0><<<g, 256, 0, s>>>((const T*)gu, (T*)out, rows, F)));
    else
      BY_DTYPE(dt, (glu8_k<T, 1><<<g, 256, 0, s>>>((const T*)gu, (T*)out, rows, F)));
    return (int)hipGetLastError();
  }
  if (act == 0)
    BY_DTYPE(dt, (glu_k<T, 0><<<nblocks(rows * F, 256), 256, 0, s>>>((const T*)gu, (T*)out, rows, F)));
  else if (act == 1)
    BY_DTYPE(dt, (glu_k<T, 1><<<nblocks(rows * F, 256), 256, 0, s>>>((const T*)gu, (T*)out, rows, F)));
  else
    return -1;
  return (int)hipGetLastError();
}

// kind: 0 = sigmoid scores, 1 = softmax over all experts
int dsv_grouped_topk(const float* z, const float* corr, int64_t* idx, float* w, int Ttok, int E,
                     int top, int groups, int keep, int kind, int group_max, int renorm,
                     float scale, hipStream_t s) {
  if (groups < 1 || groups > MAXGROUPS || E % groups || keep < 1 || keep > groups) return -1;
  if (top < 1 || top > keep * (E / groups)) return -2;
  if (kind != 0 && kind != 1) return -3;
  if (Ttok <= 0) return 0;
  if (kind == 1)
    grouped_topk_k<true><<<(Ttok + 63) / 64, 64, 0, s>>>(z, corr, idx, w, Ttok, E, top, groups,
                                                         keep, group_max, renorm, scale);
  else
    grouped_topk_k<false><<<(Ttok + 63) / 64, 64, 0, s>>>(z, corr, idx, w, Ttok, E, top, groups,
                                                          keep, group_max, renorm, scale);
  return (int)hipGetLastError();
}

int dsv_grouped_sigmoid_topk(const float* z, const float* corr, int64_t* idx, float* w, int Ttok,
                             int E, int top, int groups, int keep, hipStream_t s) {
  return dsv_grouped_topk(z, corr, idx, w, Ttok, E, top, groups, keep, 0, 0, 0, 1.f, s);
}

int dsv_xielu(const void* z, const float* pq, void* out, int dt, int64_t n, hipStream_t s) {
  if (n <= 0) return 0;
  BY_DTYPE(dt, (xielu_k<T><<<nblocks(n, 256), 256, 0, s>>>((const T*)z, pq, (T*)out, n)));
  return (int)hipGetLastError();
}

int dsv_clamped_swiglu(const void* gu, void* out, int dt, int64_t rows, int F, float limit,
                       hipStream_t s) {
  if (rows * F <= 0) return 0;
  if (F % 8 == 0) {
    BY_DTYPE(dt, (clamped_swiglu8_k<T><<<nblocks(rows * (F / 8), 256), 256, 0, s>>>(
                     (const T*)gu, (T*)out, rows, F, limit)));
    return (int)hipGetLastError();
  }
  BY_DTYPE(dt, (clamped_swiglu_k<T><<<nblocks(rows * F, 256), 256, 0, s>>>((const T*)gu, (T*)out, rows, F, limit)));
  return (int)hipGetLastError();
}

int dsv_moe_combine(const void* y, int64_t nrows, const int64_t* inv, const float* w,
                    const void* shared, const void* sg, void* out, int dt, int Ttok, int top,
                    int C, hipStream_t s) {
  if (Ttok <= 0) return 0;
  BY_DTYPE(dt, (moe_combine_k<T><<<Ttok, 256, 0, s>>>((const T*)y, inv, w, (const T*)shared,
                                                     (const T*)sg, (T*)out, top, C, nrows)));
  return (int)hipGetLastError();
}

int dsv_topk_softmax(const float* z, int64_t* idx, float* w, int Ttok, int E, int top,
                     hipStream_t s) {
  if (Ttok <= 0) return 0;
  topk_softmax_k<<<(Ttok + 63) / 64, 64, 0, s>>>(z, idx, w, Ttok, E, top);
  return (int)hipGetLastError();
}

int dsv_rms_norm_rows(const void* x, int in_dt, int ld_in, const int64_t* idx, const float* w,
                      void* out, int out_dt, int rows, int C, float eps, int one_plus,
                      hipStream_t s) {
  if (rows <= 0) return 0;
  if (ld_in < C) return -1;
  const float wa = one_plus ? 1.f : 0.f;
  const bool vec = C % 8 == 0 && C <= 8 * NT * LN_G && ld_in % 8 == 0 &&
                   (uintptr_t)x % 32 == 0;
#define RN(TI, TO)                                                                              \
  do {                                                                                          \
    if (vec)                                                                                    \
      rms_norm_rows_k<TI, TO, true><<<rows, NT, 0, s>>>((const TI*)x, ld_in, idx, w, (TO*)out,  \
                                                        C, eps, wa);                            \
    else                                                                                        \
      rms_norm_rows_k<TI, TO, false><<<rows, NT, 0, s>>>((const TI*)x, ld_in, idx, w, (TO*)out, \
                                                         C, eps, wa);                           \
  } while (0)
  if (in_dt == 0 && out_dt == 0) RN(float, float);
  else if (in_dt == 0) RN(float, bf16);
  else if (out_dt == 0) RN(bf16, float);
  else RN(bf16, bf16);
#undef RN
  return (int)hipGetLastError();
}

// g1/g2: gate pre-activations with row stride ld_g (g2, y2 may be null
// together); w null: no norm output. dt: type of the gates and results.
int dsv_gated_add(float* x, const void* g1, const void* g2, int ld_g, const void* y1,
                  const void* y2, const float* w, void* h, int dt, int out_dt, int rows, int C,
                  float eps, int one_plus, hipStream_t s) {
  if (rows <= 0) return 0;
  if ((g2 == nullptr) != (y2 == nullptr) || (w && !h)) return -1;
  const float wa = one_plus ? 1.f : 0.f;
  const bool vec = C % 8 == 0 && ld_g % 8 == 0 && C <= 8 * NT * LN_G &&
                   ((uintptr_t)g1 % 16 == 0) && (!g2 || (uintptr_t)g2 % 16 == 0);
#define GA(T, TO)                                                                               \
  do {                                                                                          \
    if (vec)                                                                                    \
      gated_add_k<T, TO, true><<<rows, NT, 0, s>>>(x, (const T*)g1, (const T*)g2, ld_g,         \
                                                   (const T*)y1, (const T*)y2, w, (TO*)h, C,    \
                                                   eps, wa);                                    \
    else                                                                                        \
      gated_add_k<T, TO, false><<<rows, NT, 0, s>>>(x, (const T*)g1, (const T*)g2, ld_g,        \
                                                    (const T*)y1, (const T*)y2, w, (TO*)h, C,   \
                                                    eps, wa);                                   \
  } while (0)
  if (dt == 0 && out_dt == 0) GA(float, float);
  else if (dt == 0) GA(float, bf16);
  else if (out_dt == 0) GA(bf16, float);
  else GA(bf16, bf16);
#undef GA
  return (int)hipGetLastError();
}

// y1/y2 (dtype dt) may be null: y2 alone never. extra: float rows added as
// they are. w1 null: no norm output; w2 needs w1. h1/h2 have dtype out_dt.
int dsv_scaled_add(float* x, const float* s1, const void* y1, const float* s2, const void* y2,
                   const float* extra, const float* w1, const float* w2, void* h1, void* h2,
                   int dt, int out_dt, int rows, int C, float eps, hipStream_t s) {
  if (rows <= 0) return 0;
  if ((y1 && !s1) || (y2 && (!y1 || !s2)) || (w1 && !h1) || (w2 && (!w1 || !h2))) return -1;
  const bool vec = C % 8 == 0 && C <= 8 * NT * LN_G;
#define SA(T, TO)                                                                              \
  do {                                                                                         \
    if (vec)                                                                                   \
      scaled_add_k<T, TO, true><<<rows, NT, 0, s>>>(x, s1, (const T*)y1, s2, (const T*)y2,     \
                                                    extra, w1, w2, (TO*)h1, (TO*)h2, C, eps);  \
    else                                                                                       \
      scaled_add_k<T, TO, false><<<rows, NT, 0, s>>>(x, s1, (const T*)y1, s2, (const T*)y2,    \
                                                     extra, w1, w2, (TO*)h1, (TO*)h2, C, eps); \
  } while (0)
  if (dt == 0 && out_dt == 0) SA(float, float);
  else if (dt == 0) SA(float, bf16);
  else if (out_dt == 0) SA(bf16, float);
  else SA(bf16, bf16);
#undef SA
  return (int)hipGetLastError();
}

int dsv_act_rows(const void* z, int ld_z, void* out, int dt, int64_t rows, int F, int act,
                 hipStream_t s) {
  if (rows * F <= 0) return 0;
  if (act < 0 || act > 2) return -1;
  const bool vec = F % 8 == 0 && ld_z % 8 == 0 && (uintptr_t)z % 16 == 0;
  const int64_t n = vec ? rows * (F / 8) : rows * F;
  const int g = (int)((n + 255) / 256 > 262140 ? 262140 : (n + 255) / 256);
#define AR(ACT)                                                                                 \
  do {                                                                                          \
    if (vec)                                                                                    \
      BY_DTYPE(dt, (act_rows_k<T, ACT, true><<<g, 256, 0, s>>>((const T*)z, ld_z, (T*)out,      \
                                                               rows, F)));                      \
    else                                                                                        \
      BY_DTYPE(dt, (act_rows_k<T, ACT, false><<<g, 256, 0, s>>>((const T*)z, ld_z, (T*)out,     \
                                                                rows, F)));                     \
  } while (0)
  if (act == 0) AR(0);
  else if (act == 1) AR(1);
  else AR(2);
#undef AR
  return (int)hipGetLastError();
}

}  // extern "C"
