// Sequence mixers over ragged batches for MI355X (gfx950): multi-head
// attention over paged K/V rows with a sliding window that keeps the first
// tokens, and linear recurrences with a matrix state per head (plain and
// delta-rule form) with their prologues and epilogue.
//
// Plain C ABI (raw device pointers + a hipStream_t) so the library builds in
// seconds with hipcc alone and is loaded through ctypes. dtype codes:
// 0 = float, 1 = bfloat16. Norm statistics, rotations, scores, softmax, the
// weighted sums, decays, gates and the recurrent state are float whatever
// the storage type.

#include "serving_common.h"

namespace {

__device__ __forceinline__ float sigmoidf_(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float siluf_(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float softplusf_(float x) {
  return x > 20.f ? x : log1pf(expf(x));
}

// ------------------------------------------------------ attention prologue
// proj row = [ q (H x dim) | k (G x dim) | v (G x vdim) ] (q alone without
// own_kv). RMS norm over the WHOLE q projection and over the whole k
// projection, rotation of adjacent pairs in the first rot_dims coordinates of
// each head, rows [k ; v] into the pool.
template <typename T>
__global__ __launch_bounds__(NT) void attn_prep_k(
    const T* __restrict__ proj, int ld_proj, const float* __restrict__ wq,
    const float* __restrict__ wk, const int* __restrict__ tok_pos,
    const int* __restrict__ tok_row, const float* __restrict__ cosT,
    const float* __restrict__ sinT, T* __restrict__ pool, T* __restrict__ q_out, int H, int G,
    int dim, int vdim, int rot_dims, int own_kv, float eps) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x;
  const T* p = proj + (int64_t)t * ld_proj;
  const int nq = H * dim, nk = G * dim, nv = G * vdim;
  const int half = rot_dims >> 1;
  const float* cs = cosT + (int64_t)tok_pos[t] * half;
  const float* sn = sinT + (int64_t)tok_pos[t] * half;
  float ss = 0.f;
  for (int i = threadIdx.x; i < nq; i += NT) {
    const float v = ld(p + i);
    ss += v * v;
  }
  const float rq = rsqrtf(block_sum(ss, red) / (float)nq + eps);
  for (int i = threadIdx.x; i < nq; i += NT) {
    const int c = i % dim;
    float v = ld(p + i) * rq * wq[i];
    if (c < rot_dims) {
      const int j = i - c + (c ^ 1);
      const float o = ld(p + j) * rq * wq[j];
      const float co = cs[c >> 1], si = sn[c >> 1];
      v = (c & 1) ? v * co + o * si : v * co - o * si;
    }
    st(q_out + (int64_t)t * nq + i, v);
  }
  if (!own_kv) return;
  T* row = pool + (int64_t)tok_row[t] * (nk + nv);
  const T* pk = p + nq;
  ss = 0.f;
  for (int i = threadIdx.x; i < nk; i += NT) {
    const float v = ld(pk + i);
    ss += v * v;
  }
  const float rk = rsqrtf(block_sum(ss, red) / (float)nk + eps);
  for (int i = threadIdx.x; i < nk; i += NT) {
    const int c = i % dim;
    float v = ld(pk + i) * rk * wk[i];
    if (c < rot_dims) {
      const int j = i - c + (c ^ 1);
      const float o = ld(pk + j) * rk * wk[j];
      const float co = cs[c >> 1], si = sn[c >> 1];
      v = (c & 1) ? v * co + o * si : v * co - o * si;
    }
    st(row + i, v);
  }
  for (int i = threadIdx.x; i < nv; i += NT) row[nk + i] = pk[nk + i];
}

// The same with eight values per thread and the projection kept in registers
// between the two passes (sizes that are multiples of 8, rows of up to
// 8 * NT * PREP_G values).
constexpr int PREP_G = 4;

template <typename T>
__device__ __forceinline__ void norm_rotate_row(
    const T* __restrict__ in, int n, const float* __restrict__ w, int dim, int rot_dims,
    const float* __restrict__ cs, const float* __restrict__ sn, T* __restrict__ out, float eps,
    float* red) {
  float x[PREP_G][8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < PREP_G; ++i) {
    const int at = (threadIdx.x + i * NT) * 8;
    if (at < n) {
      load8(in + at, x[i]);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += x[i][e] * x[i][e];
    }
  }
  const float r = rsqrtf(block_sum(ss, red) / (float)n + eps);
#pragma unroll
  for (int i = 0; i < PREP_G; ++i) {
    const int at = (threadIdx.x + i * NT) * 8;
    if (at < n) {
      float wv[8];
      load8(w + at, wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[i][e] *= r * wv[e];
      const int c0 = at % dim;
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        if (c0 + e < rot_dims) {
          const float co = cs[(c0 + e) >> 1], si = sn[(c0 + e) >> 1];
          const float a = x[i][e], b = x[i][e + 1];
          x[i][e] = a * co - b * si;
          x[i][e + 1] = b * co + a * si;
        }
      }
      store8(out + at, x[i]);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void attn_prep_vec_k(
    const T* __restrict__ proj, int ld_proj, const float* __restrict__ wq,
    const float* __restrict__ wk, const int* __restrict__ tok_pos,
    const int* __restrict__ tok_row, const float* __restrict__ cosT,
    const float* __restrict__ sinT, T* __restrict__ pool, T* __restrict__ q_out, int H, int G,
    int dim, int vdim, int rot_dims, int own_kv, float eps) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x;
  const T* p = proj + (int64_t)t * ld_proj;
  const int nq = H * dim, nk = G * dim, nv = G * vdim;
  const int half = rot_dims >> 1;
  const float* cs = cosT + (int64_t)tok_pos[t] * half;
  const float* sn = sinT + (int64_t)tok_pos[t] * half;
  norm_rotate_row(p, nq, wq, dim, rot_dims, cs, sn, q_out + (int64_t)t * nq, eps, red);
  if (!own_kv) return;
  T* row = pool + (int64_t)tok_row[t] * (nk + nv);
  norm_rotate_row(p + nq, nk, wk, dim, rot_dims, cs, sn, row, eps, red);
  for (int at = threadIdx.x * 8; at < nv; at += NT * 8) {
    float x[8];
    load8(p + nq + nk + at, x);
    store8(row + nk + at, x);
  }
}

// ------------------------------------------------------ windowed attention
// Exact kernel: one block per (token, key/value head, key split); the query
// heads of that key/value head go in groups of WHG. The keys a token sees are
// [0, n_keep) and [lo, pos]: lo = max(0, pos - window + 1) (0 without a
// window), n_keep = min(keep_first, lo). They are walked as one virtual range
// in chunks of KC, staged through LDS; scores, online softmax and the
// weighted sum are float. With nsplit > 1 the block writes (max, sum,
// unnormalised sum) and window_attn_merge_k finishes.
constexpr int WHG = 8;
constexpr int WVPT = 2;  // value columns per thread: vdim <= WVPT * NT

template <typename T>
__global__ __launch_bounds__(NT) void window_attn_k(
    const T* __restrict__ q,     // [Ttok, H, dim]
    const T* __restrict__ pool,  // rows of G*dim keys then G*vdim values
    const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
    const int* __restrict__ table, int maxb, int bs,
    T* __restrict__ out,       // [Ttok, H, vdim]
    float* __restrict__ part,  // [Ttok, nsplit, H, vdim + 2] when nsplit > 1
    int ld_out, int H, int G, int dim, int vdim, int KC, int nsplit, float scale, int window,
    int keep_first, int chunk, float softcap, float out_scale) {
  extern __shared__ float smem[];
  const int DS = dim | 1;
  float* qs = smem;              // [WHG][dim]
  float* sc = qs + WHG * dim;    // [WHG][KC]
  float* alpha = sc + WHG * KC;  // [WHG]
  float* mrun = alpha + WHG;
  float* lrun = mrun + WHG;
  T* ks = reinterpret_cast<T*>(lrun + WHG);  // [KC][DS]
  T* vs = ks + KC * DS;                      // [KC][vdim]
  const int t = blockIdx.x, g = blockIdx.y, split = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int rep = H / G;
  const int row_w = G * (dim + vdim);
  const int pos = tok_pos[t];
  const int lo = window > 0 ? max(0, pos - window + 1) : (chunk > 0 ? pos - pos % chunk : 0);
  const int n_keep = min(keep_first, lo);
  const int nkeys = n_keep + pos - lo + 1;
  const int* tab = table + (int64_t)tok_seq[t] * maxb;
  const int nchunk = (nkeys + KC - 1) / KC;
  const int cps = (nchunk + nsplit - 1) / nsplit;
  const int c_lo = split * cps, c_hi = min(nchunk, c_lo + cps);

  for (int h0 = 0; h0 < rep; h0 += WHG) {
    const int nh = min(WHG, rep - h0);
    const int hbase = g * rep + h0;
    __syncthreads();
    for (int i = tid; i < nh * dim; i += NT)
      qs[i] = ld(q + ((int64_t)t * H + hbase) * dim + i);
    if (tid < WHG) {
      mrun[tid] = -INFINITY;
      lrun[tid] = 0.f;
    }
    float acc[WHG][WVPT];
#pragma unroll
    for (int h = 0; h < WHG; ++h)
#pragma unroll
      for (int i = 0; i < WVPT; ++i) acc[h][i] = 0.f;
    for (int ch = c_lo; ch < c_hi; ++ch) {
      const int k0 = ch * KC;
      const int nk = min(KC, nkeys - k0);
      __syncthreads();
      for (int i = tid; i < nk * dim; i += NT) {
        const int kk = i / dim, c = i - kk * dim;
        const int u = k0 + kk;
        const int p = u < n_keep ? u : lo + (u - n_keep);
        const int64_t r = (int64_t)tab[p / bs] * bs + p % bs;
        ks[kk * DS + c] = pool[r * row_w + g * dim + c];
      }
      for (int i = tid; i < nk * vdim; i += NT) {
        const int kk = i / vdim, c = i - kk * vdim;
        const int u = k0 + kk;
        const int p = u < n_keep ? u : lo + (u - n_keep);
        const int64_t r = (int64_t)tab[p / bs] * bs + p % bs;
        vs[kk * vdim + c] = pool[r * row_w + G * dim + g * vdim + c];
      }
      __syncthreads();
      for (int i = tid; i < nh * KC; i += NT) {
        const int h = i / KC, kk = i - h * KC;
        float d = -INFINITY;
        if (kk < nk) {
          d = 0.f;
          const float* qh = qs + h * dim;
          const T* kr = ks + kk * DS;
          for (int c = 0; c < dim; ++c) d += qh[c] * ld(kr + c);
          d *= scale;
          if (softcap > 0.f) d = softcap * tanhf(d / softcap);
        }
        sc[i] = d;
      }
      __syncthreads();
      for (int h = wid; h < nh; h += NT / 64) {
        float mx = -INFINITY;
        for (int kk = lane; kk < nk; kk += 64) mx = fmaxf(mx, sc[h * KC + kk]);
        mx = wave_max(mx);
        const float m_old = mrun[h];
        const float m_new = fmaxf(m_old, mx);
        float psum = 0.f;
        for (int kk = lane; kk < nk; kk += 64) {
          const float pw = expf(sc[h * KC + kk] - m_new);
          sc[h * KC + kk] = pw;
          psum += pw;
        }
        psum = wave_sum(psum);
        if (lane == 0) {
          const float a = expf(m_old - m_new);  // 0 on the first chunk
          alpha[h] = a;
          mrun[h] = m_new;
          lrun[h] = lrun[h] * a + psum;
        }
      }
      __syncthreads();
#pragma unroll
      for (int h = 0; h < WHG; ++h) {
        if (h < nh) {
          const float a = alpha[h];
#pragma unroll
          for (int i = 0; i < WVPT; ++i) acc[h][i] *= a;
        }
      }
      for (int kk = 0; kk < nk; ++kk) {
        float c[WVPT];
#pragma unroll
        for (int i = 0; i < WVPT; ++i) {
          const int col = tid + i * NT;
          c[i] = col < vdim ? ld(vs + kk * vdim + col) : 0.f;
        }
#pragma unroll
        for (int h = 0; h < WHG; ++h) {
          if (h < nh) {
            const float pw = sc[h * KC + kk];
#pragma unroll
            for (int i = 0; i < WVPT; ++i) acc[h][i] += pw * c[i];
          }
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < WHG; ++h) {
      if (h < nh) {
        if (nsplit == 1) {
          const float inv = out_scale / lrun[h];
#pragma unroll
          for (int i = 0; i < WVPT; ++i) {
            const int col = tid + i * NT;
            if (col < vdim)
              st(out + (int64_t)t * ld_out + (hbase + h) * vdim + col, acc[h][i] * inv);
          }
        } else {
          float* pp = part + (((int64_t)t * nsplit + split) * H + hbase + h) * (vdim + 2);
          if (tid == 0) {
            pp[0] = mrun[h];
            pp[1] = lrun[h];
          }
#pragma unroll
          for (int i = 0; i < WVPT; ++i) {
            const int col = tid + i * NT;
            if (col < vdim) pp[2 + col] = acc[h][i];
          }
        }
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void window_attn_merge_k(
    const float* __restrict__ part, T* __restrict__ out, int ld_out, int H, int vdim,
    int nsplit, float out_scale) {
  const int t = blockIdx.x, h = blockIdx.y;
  float m = -INFINITY;
  for (int s = 0; s < nsplit; ++s) {
    const float* pp = part + (((int64_t)t * nsplit + s) * H + h) * (vdim + 2);
    if (pp[1] > 0.f) m = fmaxf(m, pp[0]);
  }
  float l = 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float* pp = part + (((int64_t)t * nsplit + s) * H + h) * (vdim + 2);
    if (pp[1] > 0.f) l += pp[1] * expf(pp[0] - m);
  }
  for (int c = threadIdx.x; c < vdim; c += NT) {
    float a = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const float* pp = part + (((int64_t)t * nsplit + s) * H + h) * (vdim + 2);
      if (pp[1] > 0.f) a += pp[2 + c] * expf(pp[0] - m);
    }
    st(out + (int64_t)t * ld_out + h * vdim + c, a / l * out_scale);
  }
}

// ------------------------------------------- windowed attention, MFMA tiles
// bf16 path for steps that bring portions of prompts. For one sequence and one
// key/value head g the rows are (token, query head of g) pairs, token-major:
// row m belongs to token m / rep and head g*rep + m % rep, so the heads that
// share keys sit in one [count*rep, dim] x [dim, keys] product. A workgroup of
// 4 waves owns 128 rows (32 per wave) and walks the key steps (32 keys each)
// that any of its rows can see: the steps that hold kept first tokens, then
// the steps from the earliest window start to the last row's own position.
//   S^T[key, row] = mfma(A = K tile from LDS, B = Q fragments in registers)
//   mask (causal, window, kept tokens), online softmax per row (fp32)
//   O^T[d, row]  += mfma(A = V^T tile from LDS, B = P fragments)
// The weights stay 32-bit through the second product: P goes in as a bf16
// head plus a bf16 remainder (two MFMAs), which carries 16 bits of mantissa.
// mfma_f32_32x32x16_bf16 layouts: A row = lane&31, k = reg + 8*(lane>>5);
// B col = lane&31, k = reg + 8*(lane>>5); C/D col = lane&31,
// row = (reg&3) + 8*(reg>>2) + 4*(lane>>5).
typedef short bf16x8s __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int TB_ROWS = 128;
constexpr int TB_KEYS = 32;
constexpr int VT_STRIDE = TB_KEYS + 8;
constexpr float LAZY_MAX = 8.f;
constexpr bool P_TWO = true;  // weights as bf16 head + remainder in the second product

// round-to-nearest-even through the native conversion (one packed
// instruction per two values on gfx950)
__device__ __forceinline__ short f2bf_native(float f) {
  const __bf16 b = static_cast<__bf16>(f);
  return __builtin_bit_cast(short, b);
}
__device__ __forceinline__ float bf_bits2f(short b) {
  union { unsigned u; float f; } c;
  c.u = ((unsigned)(unsigned short)b) << 16;
  return c.f;
}

// two workgroups per CU for the classes whose registers allow it: one hides
// the other's barriers and softmax behind its products
template <int DKT_MAX, int DVB, bool PREFETCH>
__global__ __launch_bounds__(256, (DKT_MAX <= 8 ? 2 : 1)) void window_attn_mfma_k(
    const short* __restrict__ q,     // [Ttok, H, dim]
    const short* __restrict__ pool,  // rows of G*dim keys then G*vdim values
    const int* __restrict__ work,    // [nwork][3] = (sequence, key/value head, first row)
    const int* __restrict__ cu, const int* __restrict__ seq_start,
    const int* __restrict__ table, int maxb, int bs, bf16* __restrict__ out, int ld_out,
    float* __restrict__ part,  // [Ttok, nsplit, H, vdim + 2] when nsplit > 1
    int H, int G, int dim, int vdim, int nsplit, float scale, int window, int keep_first,
    int chunk, float softcap, float out_scale) {
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  constexpr int CPT = (2 * DKT_MAX + 4 * DVB + 7) / 8;  // 16-byte chunks per thread and tile
  const int dimP = (dim + 15) & ~15;
  const int DKT = dimP >> 4;
  const int KSS = dimP + 8;
  const int cpk = dimP >> 3;        // key chunks per row
  const int cpv = (vdim + 7) >> 3;  // value chunks per row
  const int dvb = (vdim + 31) >> 5;
  // one tile = K [TB_KEYS][KSS] then V^T [DVB*32][VT_STRIDE]; with PREFETCH two
  // tiles alternate, so a step needs one barrier and the next tile's LDS
  // writes overlap this tile's products
  const int tile_sz = TB_KEYS * KSS + DVB * 32 * VT_STRIDE;
  short* tiles = reinterpret_cast<short*>(smem_raw);
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int hl = lane >> 5, l31 = lane & 31;
  const int s = work[3 * blockIdx.x], g = work[3 * blockIdx.x + 1];
  const int m0 = work[3 * blockIdx.x + 2];
  const int split = blockIdx.y;
  const int rep = H / G;
  const int row_w = G * (dim + vdim);
  const int count = cu[s + 1] - cu[s], start = seq_start[s];
  const int rows = count * rep;
  const int m_raw = m0 + wid * 32 + l31;
  const int m = min(m_raw, rows - 1);
  const int j = m / rep, h = g * rep + (m - j * rep);
  const int t = cu[s] + j;
  const int qpos = start + j;
  const int j_lo = m0 / rep;
  const int kmax = start + min(m0 + TB_ROWS - 1, rows - 1) / rep;  // inclusive
  // first key a position sees (kept first tokens aside); it never decreases
  // along a sequence, so a tile's earliest start is its first row's
  auto lo_of = [&](int p) -> int {
    return window > 0 ? max(0, p - window + 1) : (chunk > 0 ? p - p % chunk : 0);
  };
  const int lo_q = lo_of(qpos);
  const int lo_min = lo_of(start + j_lo);
  const int first_step = lo_min / TB_KEYS;
  const int keep_steps = keep_first > 0 ? min((keep_first - 1) / TB_KEYS + 1, first_step) : 0;
  const int nsteps = keep_steps + kmax / TB_KEYS - first_step + 1;
  const int* tab = table + (int64_t)s * maxb;
  const int per = (nsteps + nsplit - 1) / nsplit;
  const int v_lo = split * per, v_hi = min(nsteps, v_lo + per);
  float* pp = nullptr;
  if (nsplit > 1) pp = part + (((int64_t)t * nsplit + split) * H + h) * (vdim + 2);
  if (v_lo >= v_hi) {  // block-uniform: nothing to see in this split
    if (m_raw < rows && hl == 0) {
      pp[0] = -INFINITY;
      pp[1] = 0.f;
    }
    return;
  }
  auto key0_of = [&](int v) -> int {
    return (v < keep_steps ? v : first_step + v - keep_steps) * TB_KEYS;
  };

  const bool vec_ok = (dim & 7) == 0 && (vdim & 7) == 0;
  bf16x8s qf[DKT_MAX];
#pragma unroll
  for (int i = 0; i < DKT_MAX; ++i) {
    if (i < DKT) {
      const int d0 = 16 * i + 8 * hl;
      const short* src = q + ((int64_t)t * H + h) * dim + d0;
      if (vec_ok && d0 + 8 <= dim) {
        qf[i] = *reinterpret_cast<const bf16x8s*>(src);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[i][e] = d0 + e < dim ? src[e] : (short)0;
      }
    }
  }
  f32x16 oacc[DVB];
#pragma unroll
  for (int db = 0; db < DVB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
  float mrun = -INFINITY, lrun = 0.f;

  // Staging: chunk c of a tile is (8 values from 8*(c>>5), key c&31):
  // neighbouring lanes take neighbouring keys, so the transposed writes of a
  // value chunk fall into one LDS row. Every chunk of a thread belongs to the
  // same key (256 is a multiple of 32), so the thread resolves ONE pool row
  // per tile through the block table, a step ahead of the loads.
  auto row_of = [&](int k0) -> int64_t {
    const int p = k0 + (tid & 31);
    return p <= kmax ? (int64_t)tab[p / bs] * bs + p % bs : (int64_t)-1;
  };
  auto fetch_one = [&](int i, int64_t row) -> bf16x8s {
    const int c = tid + i * 256;
    bf16x8s v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = 0;
    if (c < TB_KEYS * (cpk + cpv) && row >= 0) {
      const int ch = c >> 5;
      const bool is_k = ch < cpk;
      const int d0 = is_k ? ch * 8 : (ch - cpk) * 8;
      const int lim = is_k ? dim : vdim;
      const short* src = pool + row * row_w + (is_k ? g * dim : G * dim + g * vdim) + d0;
      if (vec_ok && d0 + 8 <= lim) {
        v = *reinterpret_cast<const bf16x8s*>(src);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (d0 + e < lim) v[e] = src[e];
      }
    }
    return v;
  };
  auto stash_one = [&](int i, const bf16x8s& v, short* Ks) {
    short* Vt = Ks + TB_KEYS * KSS;
    const int c = tid + i * 256;
    if (c < TB_KEYS * (cpk + cpv)) {
      const int ch = c >> 5, key = c & 31;
      if (ch < cpk) {
        *reinterpret_cast<bf16x8s*>(Ks + key * KSS + ch * 8) = v;
      } else {
        const int d0 = (ch - cpk) * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) Vt[(d0 + e) * VT_STRIDE + key] = v[e];
      }
    }
  };
  bf16x8s pre[PREFETCH ? CPT : 1];
  auto fetch = [&](int64_t row) {
#pragma unroll
    for (int i = 0; i < CPT; ++i)
      if (PREFETCH) pre[i] = fetch_one(i, row);
  };
  auto stash = [&](int64_t row, short* Ks) {
    if (PREFETCH) {
#pragma unroll
      for (int i = 0; i < CPT; ++i) stash_one(i, pre[i], Ks);
    } else {
#pragma unroll 1
      for (int i = 0; i < CPT; i += 4) {
        bf16x8s v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = fetch_one(i + u, row);
#pragma unroll
        for (int u = 0; u < 4; ++u) stash_one(i + u, v[u], Ks);
      }
    }
  };

  // the wave's rows span these query positions (for skipping the mask on
  // tiles that every row sees whole)
  const int w_first = min(m0 + wid * 32, rows - 1), w_last = min(m0 + wid * 32 + 31, rows - 1);
  const int qpos_lo = start + w_first / rep, qpos_hi = start + w_last / rep;
  const int lo_hi = lo_of(qpos_hi);
  const float cap_inv = softcap > 0.f ? 1.f / softcap : 0.f;

  int64_t row_next = row_of(key0_of(v_lo));
  if (PREFETCH) {
    fetch(row_next);
    stash(row_next, tiles);
    if (v_lo + 1 < v_hi) fetch(row_of(key0_of(v_lo + 1)));
    row_next = v_lo + 2 < v_hi ? row_of(key0_of(v_lo + 2)) : (int64_t)-1;
    __syncthreads();
  }
  for (int v = v_lo; v < v_hi; ++v) {
    const int k0 = key0_of(v);
    short* Ks = tiles;
    if (PREFETCH) {
      const int cur = (v - v_lo) & 1;
      Ks = tiles + cur * tile_sz;
      if (v + 1 < v_hi) stash(0, tiles + (cur ^ 1) * tile_sz);  // tile v + 1
      if (v + 2 < v_hi) fetch(row_next);
      row_next = v + 3 < v_hi ? row_of(key0_of(v + 3)) : (int64_t)-1;
    } else {
      __syncthreads();
      stash(row_next, tiles);  // fetches tile v itself
      __syncthreads();
      row_next = v + 1 < v_hi ? row_of(key0_of(v + 1)) : (int64_t)-1;
    }
    const short* Vt = Ks + TB_KEYS * KSS;
    f32x16 st;
#pragma unroll
    for (int r = 0; r < 16; ++r) st[r] = 0.f;
#pragma unroll
    for (int i = 0; i < DKT_MAX; ++i) {
      if (i < DKT) {
        const bf16x8s kf =
            *reinterpret_cast<const bf16x8s*>(Ks + l31 * KSS + 16 * i + 8 * hl);
        st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[i], st, 0, 0, 0);
      }
    }
    float mx = -INFINITY;
    if (softcap > 0.f) {  // uniform: s <- softcap * tanh(s / softcap)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float e2 = __expf(2.f * st[r] * scale * cap_inv);
        st[r] = softcap * (1.f - 2.f / (e2 + 1.f));
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) st[r] *= scale;
    }
    if (k0 + TB_KEYS - 1 <= qpos_lo &&
        (k0 >= lo_hi || k0 + TB_KEYS - 1 < keep_first)) {  // wave-uniform
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, st[r]);
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = k0 + (r & 3) + 8 * (r >> 2) + 4 * hl;
        const bool see = key <= qpos && (key >= lo_q || key < keep_first);
        const float sv = see ? st[r] : -INFINITY;
        st[r] = sv;
        mx = fmaxf(mx, sv);
      }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    // The running maximum follows the scores lazily: it moves only when a
    // score exceeds it by more than LAZY_MAX (weights stay below e^LAZY_MAX,
    // harmless in fp32), so most steps need no rescaling of the sums. A row
    // that has seen no key yet keeps weight zero without producing inf - inf.
    const float m_new = (mx > mrun + LAZY_MAX) ? mx : mrun;
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __expf(mrun - m_use);
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float pw = __expf(st[r] - m_use);
      st[r] = pw;
      psum += pw;
    }
    psum += __shfl_xor(psum, 32, 64);
    lrun = lrun * alpha + psum;
    if (__any(m_new != mrun)) {
#pragma unroll
      for (int db = 0; db < DVB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
    }
    mrun = m_new;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      // B fragment of P: keys 16*ks + 8*hl + 0..7 of this lane's row; half of
      // them sit in the partner lane (lane ^ 32)
      bf16x8s ph, pl;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float a0 = st[i + 8 * ks], a1 = st[i + 8 * ks + 4];
        const float recv = __shfl_xor(hl ? a0 : a1, 32, 64);
        const float x0 = hl ? recv : a0, x1 = hl ? a1 : recv;
        ph[i] = f2bf_native(x0);
        ph[i + 4] = f2bf_native(x1);
        pl[i] = f2bf_native(x0 - bf_bits2f(ph[i]));
        pl[i + 4] = f2bf_native(x1 - bf_bits2f(ph[i + 4]));
      }
#pragma unroll
      for (int db = 0; db < DVB; ++db) {
        if (db < dvb) {
          const bf16x8s vf = *reinterpret_cast<const bf16x8s*>(
              Vt + (32 * db + l31) * VT_STRIDE + 16 * ks + 8 * hl);
          oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, ph, oacc[db], 0, 0, 0);
          if (P_TWO) oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pl, oacc[db], 0, 0, 0);
        }
      }
    }
    if (PREFETCH) __syncthreads();
  }
  if (m_raw < rows) {
    if (nsplit > 1) {
      if (hl == 0) {
        pp[0] = mrun;
        pp[1] = lrun;
      }
#pragma unroll
      for (int db = 0; db < DVB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int d = 32 * db + (r & 3) + 8 * (r >> 2) + 4 * hl;
          if (d < vdim) pp[2 + d] = oacc[db][r];
        }
    } else {
      const float inv = out_scale / lrun;
      bf16* o = out + (int64_t)t * ld_out + h * vdim;
#pragma unroll
      for (int db = 0; db < DVB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int d = 32 * db + (r & 3) + 8 * (r >> 2) + 4 * hl;
          if (d < vdim) o[d] = __float2bfloat16(oacc[db][r] * inv);
        }
    }
  }
}

template <int DKT_MAX, int DVB, bool PREFETCH>
int launch_window_attn_mfma(const void* q, const void* pool, const int* work, int nwork,
                            const int* cu, const int* seq_start, const int* table, int maxb,
                            int bs, void* out, int ld_out, float* part, int Ttok, int H, int G,
                            int dim, int vdim, int nsplit, float scale, int window,
                            int keep_first, int chunk, float softcap, float out_scale,
                            hipStream_t s) {
  const int dimP = (dim + 15) & ~15;
  const size_t lds = ((size_t)TB_KEYS * (dimP + 8) * 2 + (size_t)DVB * 32 * VT_STRIDE * 2) *
                     (PREFETCH ? 2 : 1);
  auto kern = window_attn_mfma_k<DKT_MAX, DVB, PREFETCH>;
  kern<<<dim3(nwork, nsplit), 256, lds, s>>>((const short*)q, (const short*)pool, work, cu,
                                             seq_start, table, maxb, bs, (bf16*)out, ld_out,
                                             part, H, G, dim, vdim, nsplit, scale, window,
                                             keep_first, chunk, softcap, out_scale);
  if (nsplit > 1)
    window_attn_merge_k<bf16><<<dim3(Ttok, H), NT, 0, s>>>(part, (bf16*)out, ld_out, H, vdim,
                                                           nsplit, out_scale);
  return (int)hipGetLastError();
}

// -------------------------------------------------- delta-rule prologue
// proj row = [ q (G x dim) | k (G x dim) | v (H x vdim) | ... ]; the H columns
// of b start at beta_col and those of a at a_col (a_col < 0: the decay is not
// made here, e.g. one per key channel that comes from a product of its own).
// One block per token: causal convolution + SiLU over the q|k|v channels
// (earlier inputs from this step's rows, from the slot's tail, or zero before
// position 0), q and k to unit length per head (q also times dim^-1/2),
// beta = sigmoid(b), decay = exp(-exp(A_log) * softplus(a + dt_bias)).
constexpr int MAXTAPS_SEQ = 32;

template <typename T>
__global__ __launch_bounds__(NT) void delta_prep_k(
    const T* __restrict__ proj, int ld_proj, const T* __restrict__ w,
    const T* __restrict__ state, int64_t state_slot_stride, const int* __restrict__ cu,
    const int* __restrict__ seq_slot, const int* __restrict__ tok_seq,
    const int* __restrict__ tok_pos, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, float* __restrict__ q_out, float* __restrict__ k_out,
    float* __restrict__ v_out, float* __restrict__ beta, float* __restrict__ decay, int G, int H,
    int dim, int vdim, int taps, int beta_col, int a_col) {
  extern __shared__ float ys[];  // [2*G*dim] conv outputs of q and k
  const int t = blockIdx.x;
  const int s = tok_seq[t];
  const int j = t - cu[s];
  const int pos = tok_pos[t];
  const int tail = taps - 1;
  const int nqk = G * dim, nv = H * vdim;
  const int C = 2 * nqk + nv;
  const T* sl = state + (int64_t)seq_slot[s] * state_slot_stride;
  const T* p = proj + (int64_t)t * ld_proj;
  for (int c = threadIdx.x; c < C; c += NT) {
    float acc = ld(w + (int64_t)c * taps + tail) * ld(p + c);
    for (int k = 1; k < taps; ++k) {
      if (pos - k < 0) break;
      const float hk = k <= j ? ld(p - (int64_t)k * ld_proj + c)
                              : ld(sl + (int64_t)(tail + j - k) * C + c);
      acc += ld(w + (int64_t)c * taps + tail - k) * hk;
    }
    const float y = siluf_(acc);
    if (c < 2 * nqk)
      ys[c] = y;
    else
      v_out[(int64_t)t * nv + c - 2 * nqk] = y;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const float qscale = rsqrtf((float)dim);
  for (int hd = wid; hd < 2 * G; hd += NT / 64) {
    const float* y = ys + hd * dim;
    float ss = 0.f;
    for (int c = lane; c < dim; c += 64) ss += y[c] * y[c];
    ss = wave_sum(ss);
    const float inv = rsqrtf(ss + 1e-6f) * (hd < G ? qscale : 1.f);
    float* o = hd < G ? q_out + ((int64_t)t * G + hd) * dim
                      : k_out + ((int64_t)t * G + hd - G) * dim;
    for (int c = lane; c < dim; c += 64) o[c] = y[c] * inv;
  }
  for (int h = threadIdx.x; h < H; h += NT) {
    beta[(int64_t)t * H + h] = sigmoidf_(ld(p + beta_col + h));
    if (a_col >= 0) {
      const float dt = softplusf_(ld(p + a_col + h) + dt_bias[h]);
      decay[(int64_t)t * H + h] = expf(-expf(a_log[h]) * dt);
    }
  }
}

// The same with eight channels per thread (sizes in multiples of 8).
template <typename T, int TAPS>
__global__ __launch_bounds__(NT) void delta_prep_vec_k(
    const T* __restrict__ proj, int ld_proj, const T* __restrict__ w,
    const T* __restrict__ state, int64_t state_slot_stride, const int* __restrict__ cu,
    const int* __restrict__ seq_slot, const int* __restrict__ tok_seq,
    const int* __restrict__ tok_pos, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, float* __restrict__ q_out, float* __restrict__ k_out,
    float* __restrict__ v_out, float* __restrict__ beta, float* __restrict__ decay, int G, int H,
    int dim, int vdim, int beta_col, int a_col) {
  extern __shared__ float ys[];  // [2*G*dim] conv outputs of q and k
  constexpr int TAIL = TAPS - 1;
  const int t = blockIdx.x;
  const int s = tok_seq[t];
  const int j = t - cu[s];
  const int pos = tok_pos[t];
  const int nqk = G * dim, nv = H * vdim;
  const int C = 2 * nqk + nv;
  const T* sl = state + (int64_t)seq_slot[s] * state_slot_stride;
  const T* p = proj + (int64_t)t * ld_proj;
  for (int c = threadIdx.x * 8; c < C; c += NT * 8) {
    float wv[8 * TAPS];  // channel-major: wv[e * TAPS + tap]
#pragma unroll
    for (int i = 0; i < TAPS; ++i) {
      float tmp[8];
      load8(w + (int64_t)c * TAPS + 8 * i, tmp);
#pragma unroll
      for (int e = 0; e < 8; ++e) wv[8 * i + e] = tmp[e];
    }
    float acc[8], x[8];
    load8(p + c, x);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = wv[e * TAPS + TAIL] * x[e];
#pragma unroll
    for (int k = 1; k <= TAIL; ++k) {
      if (pos - k >= 0) {  // block-uniform
        if (k <= j)
          load8(p - (int64_t)k * ld_proj + c, x);
        else
          load8(sl + (int64_t)(TAIL + j - k) * C + c, x);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += wv[e * TAPS + TAIL - k] * x[e];
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = siluf_(acc[e]);
    if (c < 2 * nqk)
      store8(ys + c, acc);
    else
      store8(v_out + (int64_t)t * nv + c - 2 * nqk, acc);
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const float qscale = rsqrtf((float)dim);
  for (int hd = wid; hd < 2 * G; hd += NT / 64) {
    const float* y = ys + hd * dim;
    float ss = 0.f;
    for (int c = lane; c < dim; c += 64) ss += y[c] * y[c];
    ss = wave_sum(ss);
    const float inv = rsqrtf(ss + 1e-6f) * (hd < G ? qscale : 1.f);
    float* o = hd < G ? q_out + ((int64_t)t * G + hd) * dim
                      : k_out + ((int64_t)t * G + hd - G) * dim;
    for (int c = lane; c < dim; c += 64) o[c] = y[c] * inv;
  }
  for (int h = threadIdx.x; h < H; h += NT) {
    beta[(int64_t)t * H + h] = sigmoidf_(ld(p + beta_col + h));
    if (a_col >= 0) {
      const float dt = softplusf_(ld(p + a_col + h) + dt_bias[h]);
      decay[(int64_t)t * H + h] = expf(-expf(a_log[h]) * dt);
    }
  }
}

// One block per sequence: the tail becomes the sequence's last taps-1 inputs
// (from this step's rows, or shifted out of the old tail for short steps).
template <typename T>
__global__ __launch_bounds__(NT) void conv_tail_shift_k(
    const T* __restrict__ x, int ld_x, T* __restrict__ state, int64_t state_slot_stride,
    const int* __restrict__ cu, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, int C, int taps) {
  const int s = blockIdx.x;
  const int tail = taps - 1;
  const int start = seq_start[s];
  const int count = cu[s + 1] - cu[s];
  T* sl = state + (int64_t)seq_slot[s] * state_slot_stride;
  for (int c = threadIdx.x; c < C; c += NT) {
    for (int i = 0; i < tail; ++i) {  // ascending: reads stay ahead of writes
      const int p = start + count - tail + i;  // position kept at i
      T v;
      if (p >= start)
        v = x[(int64_t)(cu[s] + p - start) * ld_x + c];
      else if (p >= 0)
        v = sl[(int64_t)(i + count) * C + c];
      else
        st(&v, 0.f);
      sl[(int64_t)i * C + c] = v;
    }
  }
}

// sigmoid(z + bias)^inv_tau = exp(inv_tau * log_sigmoid(z + bias))
template <typename T>
__global__ void sigmoid_pow_k(const T* __restrict__ z, const float* __restrict__ bias,
                              float* __restrict__ out, int64_t n, int C, float inv_tau) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const float x = ld(z + i) + bias[i % C];
    const float ls = fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
    out[i] = expf(inv_tau * ls);
  }
}

// exp(-exp(a_log[h]) * softplus(z + bias)) per head h and key channel: z is
// [rows, H*dim] with row stride ld_z, bias [H*dim], out [rows, H, dim] float.
template <typename T>
__global__ void softplus_decay_k(const T* __restrict__ z, int ld_z, const float* __restrict__ bias,
                                 const float* __restrict__ a_log, float* __restrict__ out,
                                 int64_t rows, int H, int dim) {
  const int C = H * dim;
  const int64_t n = rows * C;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / C;
    const int c = (int)(i - r * C);
    const float dt = softplusf_(ld(z + r * ld_z + c) + bias[c]);
    out[i] = expf(-expf(a_log[c / dim]) * dt);
  }
}

// the same, eight neighbouring channels per thread (dim and ld_z multiples of
// 8, z aligned for load8): a group of 8 lies inside one head
template <typename T>
__global__ void softplus_decay8_k(const T* __restrict__ z, int ld_z,
                                  const float* __restrict__ bias, const float* __restrict__ a_log,
                                  float* __restrict__ out, int64_t rows, int H, int dim) {
  const int C8 = (H * dim) >> 3;
  const int64_t n = rows * C8;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / C8;
    const int c = (int)(i - r * C8) << 3;
    float v[8], b[8];
    load8(z + r * ld_z + c, v);
    load8(bias + c, b);
    const float rate = -expf(a_log[c / dim]);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = expf(rate * softplusf_(v[e] + b[e]));
    store8(out + r * (int64_t)(C8 << 3) + c, v);
  }
}

// ------------------------------------------------------ linear recurrence
// S [dim, vdim] per (slot, head), float. The columns of S are independent in
// both forms, so the work is split by column: SCAN_R lanes share a column,
// each holding ROWS consecutive rows of it in registers (dim <= SCAN_R * ROWS,
// rows beyond dim stay zero); a block of NT threads owns NT / SCAN_R columns of
// one head of one sequence and walks the sequence's tokens in order (few rows
// per lane and many lanes: the chain from token to token is short, and two
// or more waves per SIMD fill each other's issue gaps):
//   S *= decay; d = S^T k; u = DELTA ? beta * (v - d) : v; S += k u; o = S^T q.
// Sums over rows go lane-local first, then across the SCAN_R lanes by DPP
// swaps in a fixed order, so a result does not depend on where a sequence was
// cut. The operands of CT tokens at a time are staged through LDS (widened to
// float, q scaled), double-buffered: the next chunk's global loads are in
// flight while the current chunk is computed, so the token-to-token chain
// sees LDS latency only.
constexpr int SCAN_R = 16;
constexpr int SCAN_COLS = NT / SCAN_R;

template <int CTRL>
__device__ __forceinline__ float dpp_swap(float x) {
  return __int_as_float(
      __builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}
// sum over the 16 lanes (one DPP row) that share a column; every lane gets
// the same bits
__device__ __forceinline__ float group_sum(float x) {
  x += dpp_swap<0xB1>(x);   // quad_perm [1,0,3,2]
  x += dpp_swap<0x4E>(x);   // quad_perm [2,3,0,1]
  x += dpp_swap<0x141>(x);  // row_half_mirror: the other quad of the 8
  x += dpp_swap<0x140>(x);  // row_mirror: the other half of the row
  return x;
}

// four neighbouring values p[e..e+3] widened to float, zero beyond n
__device__ __forceinline__ bool vec4_ok(const float* p, int ld, int n) {
  return (reinterpret_cast<uintptr_t>(p) & 15) == 0 && (ld & 3) == 0 && (n & 3) == 0;
}
__device__ __forceinline__ bool vec4_ok(const bf16* p, int ld, int n) {
  return (reinterpret_cast<uintptr_t>(p) & 7) == 0 && (ld & 3) == 0 && (n & 3) == 0;
}
__device__ __forceinline__ float4 load4(const float* p, int e, int n, bool vec) {
  if (vec && e + 4 <= n) return *reinterpret_cast<const float4*>(p + e);
  float4 x;
  x.x = e < n ? p[e] : 0.f;
  x.y = e + 1 < n ? p[e + 1] : 0.f;
  x.z = e + 2 < n ? p[e + 2] : 0.f;
  x.w = e + 3 < n ? p[e + 3] : 0.f;
  return x;
}
__device__ __forceinline__ float4 load4(const bf16* p, int e, int n, bool vec) {
  float4 x;
  if (vec && e + 4 <= n) {
    const uint2 w = *reinterpret_cast<const uint2*>(p + e);
    x.x = __uint_as_float(w.x << 16);
    x.y = __uint_as_float(w.x & 0xffff0000u);
    x.z = __uint_as_float(w.y << 16);
    x.w = __uint_as_float(w.y & 0xffff0000u);
    return x;
  }
  x.x = e < n ? ld(p + e) : 0.f;
  x.y = e + 1 < n ? ld(p + e + 1) : 0.f;
  x.z = e + 2 < n ? ld(p + e + 2) : 0.f;
  x.w = e + 3 < n ? ld(p + e + 3) : 0.f;
  return x;
}

template <typename T, int ROWS, bool DELTA, bool CHANNEL_DECAY>
__global__ __launch_bounds__(NT) void linear_scan_k(
    const T* __restrict__ q, int ld_q, const T* __restrict__ k, int ld_k,
    const T* __restrict__ v, int ld_v, const float* __restrict__ decay,
    const float* __restrict__ beta, float* __restrict__ state, const int* __restrict__ cu,
    const int* __restrict__ seq_slot, float* __restrict__ out, int G, int H, int dim, int vdim,
    float q_scale) {
  constexpr int CT = ROWS <= 4 ? 16 : 8;  // tokens per staged chunk
  constexpr int RS = ROWS + 4;            // stride of a lane's rows: 16-byte reads, spread banks
  constexpr int KQ = SCAN_R * RS;
  constexpr int DP = SCAN_R * ROWS;       // padded key size
  __shared__ __attribute__((aligned(16))) float sK[2][CT][KQ];
  __shared__ __attribute__((aligned(16))) float sQ[2][CT][KQ];
  __shared__ __attribute__((aligned(16))) float sD[2][CT][CHANNEL_DECAY ? KQ : 4];
  __shared__ float sV[2][CT][SCAN_COLS];
  __shared__ float sB[2][CT][2];  // beta, per-head decay
  const int s = blockIdx.x, h = blockIdx.y;
  const int r = threadIdx.x % SCAN_R;
  const int cl = threadIdx.x / SCAN_R;
  const int col0 = blockIdx.z * SCAN_COLS;
  const int col = col0 + cl;
  const bool live = col < vdim;
  const int cc = live ? col : vdim - 1;  // idle lanes shadow the last column
  const int g = h / (H / G);
  const int r0 = r * ROWS;
  float* Sg = state + (((int64_t)seq_slot[s] * H + h) * dim) * vdim + cc;
  float S[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) S[i] = r0 + i < dim ? Sg[(int64_t)(r0 + i) * vdim] : 0.f;
  const int t0 = cu[s], n = cu[s + 1] - t0;
  const int nchunks = (n + CT - 1) / CT;

  // Staging: a thread moves groups of four neighbouring values (one 8- or
  // 16-byte load when the operand allows it, one 16-byte LDS store); all sizes
  // are powers of two, so the index arithmetic is shifts and masks.
  constexpr int V4 = DP / 4;                         // groups of four per token
  constexpr int VPT = (CT * V4 + NT - 1) / NT;       // per thread and operand
  constexpr int SM = SCAN_COLS + 2;                  // v columns, beta, decay
  constexpr int SPT = (CT * SM + NT - 1) / NT;
  const bool vec_k = vec4_ok(k, ld_k, dim), vec_q = vec4_ok(q, ld_q, dim);
  float4 pk[VPT], pq[VPT], pd[CHANNEL_DECAY ? VPT : 1];
  float ps[SPT];
  auto fetch = [&](int c) {
    const int nt = min(CT, n - c * CT);
    const int tc = t0 + c * CT;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int f = threadIdx.x + i * NT;
      const int tk = f / V4, e = (f % V4) * 4;
      const bool in = tk < nt;
      pk[i] = in ? load4(k + (int64_t)(tc + tk) * ld_k + g * dim, e, dim, vec_k)
                 : make_float4(0.f, 0.f, 0.f, 0.f);
      pq[i] = in ? load4(q + (int64_t)(tc + tk) * ld_q + g * dim, e, dim, vec_q)
                 : make_float4(0.f, 0.f, 0.f, 0.f);
      if (CHANNEL_DECAY)
        pd[i] = in ? load4(decay + ((int64_t)(tc + tk) * H + h) * dim, e, dim, (dim & 3) == 0)
                   : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int i = 0; i < SPT; ++i) {
      const int f = threadIdx.x + i * NT;
      const int tk = f / SM, e = f - tk * SM;
      float x = 0.f;
      if (tk < nt) {
        const int t = tc + tk;
        if (e < SCAN_COLS)
          x = col0 + e < vdim ? ld(v + (int64_t)t * ld_v + h * vdim + col0 + e) : 0.f;
        else if (e == SCAN_COLS)
          x = DELTA ? beta[(int64_t)t * H + h] : 1.f;
        else
          x = CHANNEL_DECAY ? 1.f : decay[(int64_t)t * H + h];
      }
      ps[i] = x;
    }
  };
  auto stash = [&](int b) {
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int f = threadIdx.x + i * NT;
      const int tk = f / V4, e = (f % V4) * 4;
      if (tk < CT) {
        const int at = (e / ROWS) * RS + e % ROWS;
        float4 x = pq[i];
        x.x *= q_scale; x.y *= q_scale; x.z *= q_scale; x.w *= q_scale;
        *reinterpret_cast<float4*>(&sK[b][tk][at]) = pk[i];
        *reinterpret_cast<float4*>(&sQ[b][tk][at]) = x;
        if (CHANNEL_DECAY) *reinterpret_cast<float4*>(&sD[b][tk][at]) = pd[i];
      }
    }
#pragma unroll
    for (int i = 0; i < SPT; ++i) {
      const int f = threadIdx.x + i * NT;
      const int tk = f / SM, e = f - tk * SM;
      if (tk < CT) {
        if (e < SCAN_COLS)
          sV[b][tk][e] = ps[i];
        else
          sB[b][tk][e - SCAN_COLS] = ps[i];
      }
    }
  };

  if (nchunks > 0) {
    fetch(0);
    stash(0);
  }
  __syncthreads();
  for (int c = 0; c < nchunks; ++c) {
    const int b = c & 1;
    if (c + 1 < nchunks) fetch(c + 1);
    const int nt = min(CT, n - c * CT);
    // the operands at the head of a token's chain (k, decay) are read from
    // LDS one token ahead; sums run as four interleaved partial sums so that
    // a single wave per SIMD still has independent work in flight
    float kn[ROWS], dn[CHANNEL_DECAY ? ROWS : 1];
    auto head = [&](int tk) {
      const float4* kp = reinterpret_cast<const float4*>(&sK[b][tk][r * RS]);
#pragma unroll
      for (int i = 0; i < ROWS / 4; ++i) {
        const float4 x = kp[i];
        kn[4 * i] = x.x; kn[4 * i + 1] = x.y; kn[4 * i + 2] = x.z; kn[4 * i + 3] = x.w;
      }
      if (CHANNEL_DECAY) {
        const float4* dp = reinterpret_cast<const float4*>(&sD[b][tk][r * RS]);
#pragma unroll
        for (int i = 0; i < ROWS / 4; ++i) {
          const float4 x = dp[i];
          dn[4 * i] = x.x; dn[4 * i + 1] = x.y; dn[4 * i + 2] = x.z; dn[(4 * i + 3) % (CHANNEL_DECAY ? ROWS : 1)] = x.w;
        }
      }
    };
    head(0);
    for (int tk = 0; tk < nt; ++tk) {
      const float4* qp = reinterpret_cast<const float4*>(&sQ[b][tk][r * RS]);
      const float vc = sV[b][tk][cl];
      const float bc = sB[b][tk][0], dh = sB[b][tk][1];
      float kc[ROWS];
#pragma unroll
      for (int i = 0; i < ROWS; ++i) kc[i] = kn[i];
      if (CHANNEL_DECAY) {
#pragma unroll
        for (int i = 0; i < ROWS; ++i) S[i] *= dn[i % (CHANNEL_DECAY ? ROWS : 1)];
      } else {
#pragma unroll
        for (int i = 0; i < ROWS; ++i) S[i] *= dh;
      }
      if (tk + 1 < nt) head(tk + 1);
      float u = vc;
      if (DELTA) {
        float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll
        for (int i = 0; i < ROWS; i += 4) {
          d0 += S[i] * kc[i];
          d1 += S[i + 1] * kc[i + 1];
          d2 += S[i + 2] * kc[i + 2];
          d3 += S[i + 3] * kc[i + 3];
        }
        u = bc * (vc - group_sum((d0 + d1) + (d2 + d3)));
      }
      float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
      for (int i = 0; i < ROWS / 4; ++i) {
        const float4 x = qp[i];
        S[4 * i] += kc[4 * i] * u;         o0 += S[4 * i] * x.x;
        S[4 * i + 1] += kc[4 * i + 1] * u; o1 += S[4 * i + 1] * x.y;
        S[4 * i + 2] += kc[4 * i + 2] * u; o2 += S[4 * i + 2] * x.z;
        S[4 * i + 3] += kc[4 * i + 3] * u; o3 += S[4 * i + 3] * x.w;
      }
      const float o = group_sum((o0 + o1) + (o2 + o3));
      if (live && r == 0) out[((int64_t)(t0 + c * CT + tk) * H + h) * vdim + col] = o;
    }
    if (c + 1 < nchunks) stash(b ^ 1);
    __syncthreads();
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i)
      if (r0 + i < dim) Sg[(int64_t)(r0 + i) * vdim] = S[i];
  }
}

// out[t, h*vdim + c] = o / sqrt(mean_c(o^2) + eps) * w[c] * act(gate),
// act = SiLU, or the plain sigmoid with SIGMOID
template <typename T, bool SIGMOID>
__global__ __launch_bounds__(NT) void head_norm_gate_k(
    const float* __restrict__ o, const float* __restrict__ w, const T* __restrict__ gate,
    int ld_gate, T* __restrict__ out, int H, int vdim, float eps) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  for (int h = wid; h < H; h += NT / 64) {
    const float* oh = o + ((int64_t)t * H + h) * vdim;
    float ss = 0.f;
    for (int c = lane; c < vdim; c += 64) ss += oh[c] * oh[c];
    const float inv = rsqrtf(wave_sum(ss) / (float)vdim + eps);
    for (int c = lane; c < vdim; c += 64) {
      const float gv = ld(gate + (int64_t)t * ld_gate + h * vdim + c);
      st(out + ((int64_t)t * H + h) * vdim + c,
         oh[c] * inv * w[c] * (SIGMOID ? sigmoidf_(gv) : siluf_(gv)));
    }
  }
}

// ------------------------------------- attention prologue, per-head options
// proj row (stride ld_proj) = [ q (H x dim) | k (G x dim) | v (G x vdim) ].
// NORM: 0 none, 2 per head over dim with one weight of size dim shared by the
// heads. Rotation of the first rot_dims coordinates of each head, pairing
// (2i, 2i+1) (HALF false) or (i, i + rot_dims/2) (HALF true). v_eps >= 0:
// every value head is divided by its root mean square. One wave per head.
template <typename T, bool HALF>
__global__ __launch_bounds__(NT) void attn_prep_heads_k(
    const T* __restrict__ proj, int ld_proj, const float* __restrict__ wq,
    const float* __restrict__ wk, const int* __restrict__ tok_pos,
    const int* __restrict__ tok_row, const float* __restrict__ cosT,
    const float* __restrict__ sinT, T* __restrict__ pool, T* __restrict__ q_out, int H, int G,
    int dim, int vdim, int rot_dims, int own_kv, int norm, float eps, float v_eps) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const T* p = proj + (int64_t)t * ld_proj;
  const int nq = H * dim, nk = G * dim, nv = G * vdim;
  const int half = rot_dims >> 1;
  const float* cs = cosT + (int64_t)tok_pos[t] * half;
  const float* sn = sinT + (int64_t)tok_pos[t] * half;
  T* row = own_kv ? pool + (int64_t)tok_row[t] * (nk + nv) : nullptr;
  const int jobs = own_kv ? H + 2 * G : H;
  for (int job = wid; job < jobs; job += NT / 64) {
    if (job < H + G) {  // a query or key head
      const bool is_q = job < H;
      const T* in = is_q ? p + job * dim : p + nq + (job - H) * dim;
      T* out = is_q ? q_out + (int64_t)t * nq + job * dim : row + (job - H) * dim;
      const float* w = is_q ? wq : wk;
      float inv = 1.f;
      if (norm == 2) {
        float ss = 0.f;
        for (int c = lane; c < dim; c += 64) {
          const float v = ld(in + c);
          ss += v * v;
        }
        inv = rsqrtf(wave_sum(ss) / (float)dim + eps);
      }
      for (int c = lane; c < dim; c += 64) {
        float v = ld(in + c) * inv * (norm == 2 ? w[c] : 1.f);
        if (c < rot_dims) {
          const int j = HALF ? (c < half ? c + half : c - half) : (c ^ 1);
          const float o = ld(in + j) * inv * (norm == 2 ? w[j] : 1.f);
          const int f = HALF ? (c < half ? c : c - half) : (c >> 1);
          const bool second = HALF ? c >= half : (c & 1);
          const float co = cs[f], si = sn[f];
          v = second ? v * co + o * si : v * co - o * si;
        }
        st(out + c, v);
      }
    } else {  // a value head
      const int g = job - H - G;
      const T* in = p + nq + nk + g * vdim;
      T* out = row + nk + g * vdim;
      float inv = 1.f;
      if (v_eps >= 0.f) {
        float ss = 0.f;
        for (int c = lane; c < vdim; c += 64) {
          const float v = ld(in + c);
          ss += v * v;
        }
        inv = rsqrtf(wave_sum(ss) / (float)vdim + v_eps);
      }
      for (int c = lane; c < vdim; c += 64) st(out + c, ld(in + c) * inv);
    }
  }
}

// ------------------------------------ short convolution + bias + SiLU, rows
// x is a column slice (row stride ld_x) of C channels; earlier inputs come
// from this step's rows, from the slot's tail, or are zero before position 0.
template <typename T, typename TO>
__global__ __launch_bounds__(NT) void conv_silu_k(
    const T* __restrict__ x, int ld_x, const T* __restrict__ w, const float* __restrict__ bias,
    const T* __restrict__ state, int64_t state_slot_stride, const int* __restrict__ cu,
    const int* __restrict__ seq_slot, const int* __restrict__ tok_seq,
    const int* __restrict__ tok_pos, TO* __restrict__ out, int C, int taps) {
  const int t = blockIdx.x;
  const int s = tok_seq[t];
  const int j = t - cu[s];
  const int pos = tok_pos[t];
  const int tail = taps - 1;
  const T* sl = state + (int64_t)seq_slot[s] * state_slot_stride;
  const T* p = x + (int64_t)t * ld_x;
  for (int c = threadIdx.x; c < C; c += NT) {
    float acc = ld(w + (int64_t)c * taps + tail) * ld(p + c);
    for (int k = 1; k < taps; ++k) {
      if (pos - k < 0) break;
      const float hk = k <= j ? ld(p - (int64_t)k * ld_x + c)
                              : ld(sl + (int64_t)(tail + j - k) * C + c);
      acc += ld(w + (int64_t)c * taps + tail - k) * hk;
    }
    if (bias) acc += bias[c];
    st(out + (int64_t)t * C + c, siluf_(acc));
  }
}

// ------------------------------------------- scalar-decay state-space prologue
// proj row = [ z (H*P) | x (H*P) | B (G*N) | C (G*N) | dt (H) ]. One block per
// token: convolution + bias + SiLU over the x|B|C channels,
// dt = softplus(dt + dt_bias), decay = exp(-exp(A_log) * dt); outputs float:
// x, v = dt * x, B, C, decay.
template <typename T>
__global__ __launch_bounds__(NT) void ssd_prep_k(
    const T* __restrict__ proj, int ld_proj, const T* __restrict__ w,
    const float* __restrict__ bias, const T* __restrict__ state, int64_t state_slot_stride,
    const int* __restrict__ cu, const int* __restrict__ seq_slot,
    const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    float* __restrict__ x_out, float* __restrict__ v_out, float* __restrict__ b_out,
    float* __restrict__ c_out, float* __restrict__ decay, int H, int P, int G, int N, int taps) {
  extern __shared__ float dts[];  // [H]
  const int t = blockIdx.x;
  const int s = tok_seq[t];
  const int j = t - cu[s];
  const int pos = tok_pos[t];
  const int tail = taps - 1;
  const int inner = H * P, gn = G * N;
  const int C = inner + 2 * gn;
  const T* sl = state + (int64_t)seq_slot[s] * state_slot_stride;
  const T* p = proj + (int64_t)t * ld_proj + inner;  // the convolved columns
  for (int h = threadIdx.x; h < H; h += NT) {
    const float dt = softplusf_(ld(p + C + h) + dt_bias[h]);
    dts[h] = dt;
    decay[(int64_t)t * H + h] = expf(-expf(a_log[h]) * dt);
  }
  __syncthreads();
  for (int c = threadIdx.x; c < C; c += NT) {
    float acc = ld(w + (int64_t)c * taps + tail) * ld(p + c);
    for (int k = 1; k < taps; ++k) {
      if (pos - k < 0) break;
      const float hk = k <= j ? ld(p - (int64_t)k * ld_proj + c)
                              : ld(sl + (int64_t)(tail + j - k) * C + c);
      acc += ld(w + (int64_t)c * taps + tail - k) * hk;
    }
    const float y = siluf_(acc + bias[c]);
    if (c < inner) {
      x_out[(int64_t)t * inner + c] = y;
      v_out[(int64_t)t * inner + c] = dts[c / P] * y;
    } else if (c < inner + gn) {
      b_out[(int64_t)t * gn + c - inner] = y;
    } else {
      c_out[(int64_t)t * gn + c - inner - gn] = y;
    }
  }
}

// y = (o + skip_h * x) * silu(gate); out = y / sqrt(mean_part(y^2) + eps) * w.
// One block per (token, part of the row).
template <typename T>
__global__ __launch_bounds__(NT) void gate_group_norm_k(
    const float* __restrict__ o, const float* __restrict__ x, const float* __restrict__ skip,
    const T* __restrict__ gate, int ld_gate, const float* __restrict__ w, T* __restrict__ out,
    int n, int vdim, int parts, float eps) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x, part = blockIdx.y;
  const int len = n / parts, c0 = part * len;
  const float* orow = o + (int64_t)t * n;
  const float* xrow = x + (int64_t)t * n;
  const T* grow = gate + (int64_t)t * ld_gate;
  float ss = 0.f;
  for (int c = c0 + threadIdx.x; c < c0 + len; c += NT) {
    const float y = (orow[c] + skip[c / vdim] * xrow[c]) * siluf_(ld(grow + c));
    ss += y * y;
  }
  const float inv = rsqrtf(block_sum(ss, red) / (float)len + eps);
  for (int c = c0 + threadIdx.x; c < c0 + len; c += NT) {
    const float y = (orow[c] + skip[c / vdim] * xrow[c]) * siluf_(ld(grow + c));
    st(out + (int64_t)t * n + c, y * inv * w[c]);
  }
}

// The same with eight columns per thread and the part kept in registers
// between the two passes (part length a multiple of 8, at most 8 * NT * GGN).
constexpr int GGN = 4;
template <typename T>
__global__ __launch_bounds__(NT) void gate_group_norm_vec_k(
    const float* __restrict__ o, const float* __restrict__ x, const float* __restrict__ skip,
    const T* __restrict__ gate, int ld_gate, const float* __restrict__ w, T* __restrict__ out,
    int n, int vdim, int parts, float eps) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x, part = blockIdx.y;
  const int len = n / parts, c0 = part * len;
  const float* orow = o + (int64_t)t * n;
  const float* xrow = x + (int64_t)t * n;
  const T* grow = gate + (int64_t)t * ld_gate;
  float y[GGN][8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < GGN; ++i) {
    const int c = c0 + (threadIdx.x + i * NT) * 8;
    if (c < c0 + len) {
      float xv[8], gv[8];
      load8(orow + c, y[i]);
      load8(xrow + c, xv);
      load8(grow + c, gv);
      const float sk = skip[c / vdim];  // vdim is a multiple of 8: one head per group
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        y[i][e] = (y[i][e] + sk * xv[e]) * siluf_(gv[e]);
        ss += y[i][e] * y[i][e];
      }
    }
  }
  const float inv = rsqrtf(block_sum(ss, red) / (float)len + eps);
#pragma unroll
  for (int i = 0; i < GGN; ++i) {
    const int c = c0 + (threadIdx.x + i * NT) * 8;
    if (c < c0 + len) {
      float wv[8];
      load8(w + c, wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) y[i][e] *= inv * wv[e];
      store8(out + (int64_t)t * n + c, y[i]);
    }
  }
}

// Eight neighbouring channels of the short convolution (+ bias) + SiLU at one
// token: p points at the token's row of the convolved columns, sl at the
// slot's tail. C, ld and the slot stride are multiples of 8.
template <typename T, int TAPS>
__device__ __forceinline__ void conv8_silu(const T* __restrict__ p, int ld,
                                           const T* __restrict__ w,
                                           const float* __restrict__ bias,
                                           const T* __restrict__ sl, int C, int c, int j,
                                           int pos, float (&acc)[8]) {
  constexpr int TAIL = TAPS - 1;
  float wv[8 * TAPS];  // channel-major: wv[e * TAPS + tap]
#pragma unroll
  for (int i = 0; i < TAPS; ++i) {
    float tmp[8];
    load8(w + (int64_t)c * TAPS + 8 * i, tmp);
#pragma unroll
    for (int e = 0; e < 8; ++e) wv[8 * i + e] = tmp[e];
  }
  float x[8];
  load8(p + c, x);
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = wv[e * TAPS + TAIL] * x[e];
#pragma unroll
  for (int k = 1; k <= TAIL; ++k) {
    if (pos - k >= 0) {  // block-uniform
      if (k <= j)
        load8(p - (int64_t)k * ld + c, x);
      else
        load8(sl + (int64_t)(TAIL + j - k) * C + c, x);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += wv[e * TAPS + TAIL - k] * x[e];
    }
  }
  if (bias) {
    float bv[8];
    load8(bias + c, bv);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += bv[e];
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = siluf_(acc[e]);
}

template <typename T, typename TO, int TAPS>
__global__ __launch_bounds__(NT) void conv_silu_vec_k(
    const T* __restrict__ x, int ld_x, const T* __restrict__ w, const float* __restrict__ bias,
    const T* __restrict__ state, int64_t state_slot_stride, const int* __restrict__ cu,
    const int* __restrict__ seq_slot, const int* __restrict__ tok_seq,
    const int* __restrict__ tok_pos, TO* __restrict__ out, int C) {
  const int t = blockIdx.x;
  const int s = tok_seq[t];
  const int j = t - cu[s];
  const int pos = tok_pos[t];
  const T* sl = state + (int64_t)seq_slot[s] * state_slot_stride;
  const T* p = x + (int64_t)t * ld_x;
  for (int c = (blockIdx.y * NT + threadIdx.x) * 8; c < C; c += gridDim.y * NT * 8) {
    float acc[8];
    conv8_silu<T, TAPS>(p, ld_x, w, bias, sl, C, c, j, pos, acc);
    store8(out + (int64_t)t * C + c, acc);
  }
}

template <typename T, int TAPS>
__global__ __launch_bounds__(NT) void ssd_prep_vec_k(
    const T* __restrict__ proj, int ld_proj, const T* __restrict__ w,
    const float* __restrict__ bias, const T* __restrict__ state, int64_t state_slot_stride,
    const int* __restrict__ cu, const int* __restrict__ seq_slot,
    const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    float* __restrict__ x_out, float* __restrict__ v_out, float* __restrict__ b_out,
    float* __restrict__ c_out, float* __restrict__ decay, int H, int P, int G, int N) {
  const int t = blockIdx.x;
  const int s = tok_seq[t];
  const int j = t - cu[s];
  const int pos = tok_pos[t];
  const int inner = H * P, gn = G * N;
  const int C = inner + 2 * gn;
  const T* sl = state + (int64_t)seq_slot[s] * state_slot_stride;
  const T* p = proj + (int64_t)t * ld_proj + inner;  // the convolved columns
  if (blockIdx.y == 0)
    for (int h = threadIdx.x; h < H; h += NT)
      decay[(int64_t)t * H + h] = expf(-expf(a_log[h]) * softplusf_(ld(p + C + h) + dt_bias[h]));
  for (int c = (blockIdx.y * NT + threadIdx.x) * 8; c < C; c += gridDim.y * NT * 8) {
    float y[8];
    conv8_silu<T, TAPS>(p, ld_proj, w, bias, sl, C, c, j, pos, y);
    if (c < inner) {
      const int h = c / P;  // P is a multiple of 8: one head per group
      const float dt = softplusf_(ld(p + C + h) + dt_bias[h]);
      store8(x_out + (int64_t)t * inner + c, y);
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] *= dt;
      store8(v_out + (int64_t)t * inner + c, y);
    } else if (c < inner + gn) {
      store8(b_out + (int64_t)t * gn + c - inner, y);
    } else {
      store8(c_out + (int64_t)t * gn + c - inner - gn, y);
    }
  }
}

// The per-head prologue with eight values per lane: a head is shared by LG
// lanes (a power of two, 8 * LG >= dim and vdim); all sizes multiples of 8.
template <typename T, bool HALF, int LG>
__global__ __launch_bounds__(NT) void attn_prep_heads_vec_k(
    const T* __restrict__ proj, int ld_proj, const float* __restrict__ wq,
    const float* __restrict__ wk, const int* __restrict__ tok_pos,
    const int* __restrict__ tok_row, const float* __restrict__ cosT,
    const float* __restrict__ sinT, T* __restrict__ pool, T* __restrict__ q_out, int H, int G,
    int dim, int vdim, int rot_dims, int own_kv, int norm, float eps, float v_eps) {
  const int t = blockIdx.x;
  const int l = threadIdx.x % LG, grp = threadIdx.x / LG;
  const T* p = proj + (int64_t)t * ld_proj;
  const int nq = H * dim, nk = G * dim, nv = G * vdim;
  const int half = rot_dims >> 1;
  const float* cs = cosT + (int64_t)tok_pos[t] * half;
  const float* sn = sinT + (int64_t)tok_pos[t] * half;
  T* row = own_kv ? pool + (int64_t)tok_row[t] * (nk + nv) : nullptr;
  const int jobs = own_kv ? H + 2 * G : H;
  const int c0 = l * 8;
  // every lane of a wave walks the same number of rounds: the group sums
  // below use whole-wave shuffles
  for (int j0 = 0; j0 < jobs; j0 += NT / LG) {
    const int job = j0 + grp;
    const bool have = job < jobs;
    const bool is_v = have && job >= H + G;
    const bool is_q = have && job < H;
    const int n = is_v ? vdim : dim;
    const T* in = p;
    T* out = q_out;
    if (is_q) {
      in = p + job * dim;
      out = q_out + (int64_t)t * nq + job * dim;
    } else if (have && !is_v) {
      in = p + nq + (job - H) * dim;
      out = row + (job - H) * dim;
    } else if (is_v) {
      in = p + nq + nk + (job - H - G) * vdim;
      out = row + nk + (job - H - G) * vdim;
    }
    const bool act = have && c0 < n;
    float x[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = 0.f;
    if (act) load8(in + c0, x);
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
#pragma unroll
    for (int o = 1; o < LG; o <<= 1) ss += __shfl_xor(ss, o, 64);
    if (!act) continue;
    if (is_v) {
      if (v_eps >= 0.f) {
        const float inv = rsqrtf(ss / (float)vdim + v_eps);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] *= inv;
      }
      store8(out + c0, x);
      continue;
    }
    const float* w = is_q ? wq : wk;
    const float inv = norm == 2 ? rsqrtf(ss / (float)dim + eps) : 1.f;
    if (norm == 2) {
      float wv[8];
      load8(w + c0, wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] *= inv * wv[e];
    }
    if (c0 < rot_dims) {
      if (HALF) {  // the partner group sits half the rotated width away
        const bool second = c0 >= half;
        const int pc = second ? c0 - half : c0 + half;
        const int f0 = second ? c0 - half : c0;
        float o[8];
        load8(in + pc, o);
        if (norm == 2) {
          float wv[8];
          load8(w + pc, wv);
#pragma unroll
          for (int e = 0; e < 8; ++e) o[e] *= inv * wv[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float co = cs[f0 + e], si = sn[f0 + e];
          x[e] = second ? x[e] * co + o[e] * si : x[e] * co - o[e] * si;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          if (c0 + e < rot_dims) {
            const float co = cs[(c0 + e) >> 1], si = sn[(c0 + e) >> 1];
            const float a = x[e], b = x[e + 1];
            x[e] = a * co - b * si;
            x[e + 1] = b * co + a * si;
          }
        }
      }
    }
    store8(out + c0, x);
  }
}

// --------------------------------------------------------- selective scan
// One state vector S[c, 0..N) per channel, float. The 16 lanes of a DPP row
// share a channel, each holding NS consecutive states in registers
// (N <= 16 * NS); a block owns NT / 16 channels of one sequence and walks its
// tokens in order:
//   dt = softplus(dt_pre + dt_bias); S[n] = exp(dt * A[n]) * S[n] + dt * x * B[n];
//   y = sum_n S[n] * C[n] + D * x; out = y * silu(z) * out_scale.
// The operands of SCT tokens at a time are staged through LDS, double-buffered
// (the next chunk's global loads are in flight while this chunk is computed);
// the staging thread also evaluates softplus and silu, once per channel and
// token. The sum runs lane-local in a fixed order, then over the 16 lanes in
// a fixed DPP tree, so a result does not depend on where a sequence was cut.
// A is kept times log2(e): the decay is one multiply and one exp2.
constexpr int SCH = NT / 16;  // channels per block
constexpr int SCT = 16;       // tokens per staged chunk

template <typename T, int NS>
__global__ __launch_bounds__(NT) void selective_scan_k(
    const T* __restrict__ x, int ld_x, const float* __restrict__ dt_pre,
    const float* __restrict__ dt_bias, const float* __restrict__ a_log,
    const T* __restrict__ Bm, const T* __restrict__ Cm, int ld_bc,
    const float* __restrict__ skip, const T* __restrict__ z, int ld_z,
    float* __restrict__ state, const int* __restrict__ cu, const int* __restrict__ seq_slot,
    T* __restrict__ out, int ld_out, int ch, int N, float out_scale) {
  constexpr int NP = 16 * NS;  // padded state size
  __shared__ float sDt[2][SCT][SCH];
  __shared__ float sX[2][SCT][SCH];
  __shared__ float sG[2][SCT][SCH];
  __shared__ __attribute__((aligned(16))) float sB[2][SCT][NP];
  __shared__ __attribute__((aligned(16))) float sC[2][SCT][NP];
  __shared__ float sO[SCT][SCH];
  const int s = blockIdx.x;
  const int r = threadIdx.x & 15;
  const int cl = threadIdx.x >> 4;
  const int c0 = blockIdx.y * SCH;
  const int c_raw = c0 + cl;
  const bool live = c_raw < ch;
  const int c = live ? c_raw : ch - 1;  // idle lanes shadow the last channel
  const int n0 = r * NS;
  float* Sg = state + ((int64_t)seq_slot[s] * ch + c) * N;
  float S[NS], A[NS];
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    const bool in = n0 + i < N;
    S[i] = in ? Sg[n0 + i] : 0.f;
    A[i] = in ? -expf(a_log[(int64_t)c * N + n0 + i]) * 1.4426950408889634f : 0.f;
  }
  const float dsk = skip[c];
  const int t0 = cu[s], n = cu[s + 1] - t0;
  const int nchunks = (n + SCT - 1) / SCT;

  // staging: element f of a chunk's [SCT][SCH] block is (token f / SCH,
  // channel f % SCH); of its [SCT][NP] block (token f / NP, state f % NP)
  constexpr int EPT = SCT * SCH / NT;              // = 1
  constexpr int BPT = (SCT * NP + NT - 1) / NT;    // = NS
  float pdt[EPT], px[EPT], pz[EPT], pb[BPT], pc[BPT];
  auto fetch = [&](int k) {
    const int nt = min(SCT, n - k * SCT);
    const int tc = t0 + k * SCT;
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
      const int f = threadIdx.x + i * NT;
      const int tk = f / SCH, e = c0 + f % SCH;
      const bool in = tk < nt && e < ch;
      pdt[i] = in ? dt_pre[(int64_t)(tc + tk) * ch + e] + dt_bias[e] : 0.f;
      px[i] = in ? ld(x + (int64_t)(tc + tk) * ld_x + e) : 0.f;
      pz[i] = in ? ld(z + (int64_t)(tc + tk) * ld_z + e) : 0.f;
    }
#pragma unroll
    for (int i = 0; i < BPT; ++i) {
      const int f = threadIdx.x + i * NT;
      const int tk = f / NP, e = f % NP;
      const bool in = tk < nt && e < N;
      pb[i] = in ? ld(Bm + (int64_t)(tc + tk) * ld_bc + e) : 0.f;
      pc[i] = in ? ld(Cm + (int64_t)(tc + tk) * ld_bc + e) : 0.f;
    }
  };
  auto stash = [&](int b) {
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
      const int f = threadIdx.x + i * NT;
      const int tk = f / SCH, e = f % SCH;
      sDt[b][tk][e] = softplusf_(pdt[i]);
      sX[b][tk][e] = px[i];
      sG[b][tk][e] = siluf_(pz[i]) * out_scale;
    }
#pragma unroll
    for (int i = 0; i < BPT; ++i) {
      const int f = threadIdx.x + i * NT;
      const int tk = f / NP, e = f % NP;
      if (tk < SCT) {
        sB[b][tk][e] = pb[i];
        sC[b][tk][e] = pc[i];
      }
    }
  };
  if (nchunks > 0) {
    fetch(0);
    stash(0);
  }
  __syncthreads();
  for (int k = 0; k < nchunks; ++k) {
    const int b = k & 1;
    if (k + 1 < nchunks) fetch(k + 1);
    const int nt = min(SCT, n - k * SCT);
    for (int tk = 0; tk < nt; ++tk) {
      const float dt = sDt[b][tk][cl], xv = sX[b][tk][cl];
      const float dx = dt * xv;
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        S[i] = __builtin_amdgcn_exp2f(dt * A[i]) * S[i] + dx * sB[b][tk][n0 + i];
        acc += S[i] * sC[b][tk][n0 + i];
      }
      acc = group_sum(acc);
      if (r == 0) sO[tk][cl] = (acc + dsk * xv) * sG[b][tk][cl];
    }
    __syncthreads();  // sO complete; every lane is done with buffer b
    {  // the chunk's results, channel-contiguous
      const int f = threadIdx.x;
      const int tk = f / SCH, e = c0 + f % SCH;
      if (tk < nt && e < ch) st(out + (int64_t)(t0 + k * SCT + tk) * ld_out + e, sO[tk][f % SCH]);
    }
    if (k + 1 < nchunks) stash(b ^ 1);
    __syncthreads();
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < NS; ++i)
      if (n0 + i < N) Sg[n0 + i] = S[i];
  }
}

}  // namespace

extern "C" {

int dsv_attn_prep(const void* proj, int ld_proj, const float* wq, const float* wk,
                  const int* tok_pos, const int* tok_row, const float* cosT, const float* sinT,
                  void* pool, void* q_out, int dt, int Ttok, int H, int G, int dim, int vdim,
                  int rot_dims, int own_kv, float eps, hipStream_t s) {
  if (rot_dims < 0 || (rot_dims & 1) || rot_dims > dim || H % G) return -1;
  if (Ttok <= 0) return 0;
  const int row_max = 8 * NT * PREP_G;
  if (dim % 8 == 0 && vdim % 8 == 0 && ld_proj % 8 == 0 && H * dim <= row_max &&
      G * dim <= row_max) {
    BY_DTYPE(dt, (attn_prep_vec_k<T><<<Ttok, NT, 0, s>>>(
                     (const T*)proj, ld_proj, wq, wk, tok_pos, tok_row, cosT, sinT, (T*)pool,
                     (T*)q_out, H, G, dim, vdim, rot_dims, own_kv, eps)));
    return (int)hipGetLastError();
  }
  BY_DTYPE(dt, (attn_prep_k<T><<<Ttok, NT, 0, s>>>((const T*)proj, ld_proj, wq, wk, tok_pos,
                                                   tok_row, cosT, sinT, (T*)pool, (T*)q_out, H,
                                                   G, dim, vdim, rot_dims, own_kv, eps)));
  return (int)hipGetLastError();
}

// LDS bytes of the exact attention kernel for a chunk of KC keys
int64_t dsv_window_attn_lds(int dt, int dim, int vdim, int KC) {
  return (int64_t)(WHG * dim + WHG * KC + 3 * WHG) * 4 +
         (int64_t)KC * ((dim | 1) + vdim) * (dt == 0 ? 4 : 2);
}

int dsv_window_attn(const void* q, const void* pool, const int* tok_seq, const int* tok_pos,
                    const int* table, int maxb, int bs, void* out, int ld_out, float* part,
                    int dt, int Ttok, int H, int G, int dim, int vdim, int KC, int nsplit,
                    float scale, int window, int keep_first, int chunk, float softcap,
                    float out_scale, hipStream_t s) {
  if (vdim > WVPT * NT || H % G || nsplit < 1 || (nsplit > 1 && !part)) return -1;
  if ((window > 0 && chunk > 0) || ld_out < H * vdim) return -3;
  if (Ttok <= 0) return 0;
  const int64_t lds = dsv_window_attn_lds(dt, dim, vdim, KC);
  if (lds > 64 * 1024) return -2;
  dim3 grid(Ttok, G, nsplit);
  BY_DTYPE(dt, (window_attn_k<T><<<grid, NT, lds, s>>>(
                   (const T*)q, (const T*)pool, tok_seq, tok_pos, table, maxb, bs, (T*)out, part,
                   ld_out, H, G, dim, vdim, KC, nsplit, scale, window, keep_first, chunk, softcap,
                   nsplit > 1 ? 1.f : out_scale)));
  if (nsplit > 1) {
    dim3 g2(Ttok, H);
    BY_DTYPE(dt, (window_attn_merge_k<T><<<g2, NT, 0, s>>>(part, (T*)out, ld_out, H, vdim,
                                                           nsplit, out_scale)));
  }
  return (int)hipGetLastError();
}

// 1 when the MFMA tile kernel covers these head sizes (bf16 only)
int dsv_window_attn_mfma_ok(int dim, int vdim) {
  return dim >= 1 && dim <= 256 && vdim >= 1 && vdim <= 256;
}

int dsv_window_attn_mfma_rows() { return TB_ROWS; }

// work: [nwork][3] = (sequence, key/value head, first row of a tile of the
// sequence's count * (H/G) rows for that head)
int dsv_window_attn_mfma(const void* q, const void* pool, const int* work, int nwork,
                         const int* cu, const int* seq_start, const int* table, int maxb, int bs,
                         void* out, int ld_out, float* part, int Ttok, int H, int G, int dim,
                         int vdim, int nsplit, float scale, int window, int keep_first,
                         int chunk, float softcap, float out_scale, hipStream_t s) {
  if (!dsv_window_attn_mfma_ok(dim, vdim) || H % G) return -1;
  if ((window > 0 && chunk > 0) || ld_out < H * vdim) return -4;
  if (nsplit < 1 || (nsplit > 1 && !part)) return -3;
  if (nwork <= 0) return 0;
#define GO(DKT, DVB, PF)                                                                        \
  return launch_window_attn_mfma<DKT, DVB, PF>(q, pool, work, nwork, cu, seq_start, table, maxb, \
                                               bs, out, ld_out, part, Ttok, H, G, dim, vdim,     \
                                               nsplit, scale, window, keep_first, chunk,         \
                                               softcap, out_scale, s)
  if (dim <= 64 && vdim <= 64) GO(4, 2, true);
  if (dim <= 128 && vdim <= 128) GO(8, 4, true);
  GO(16, 8, false);
#undef GO
}

int dsv_delta_prep(const void* proj, int ld_proj, const void* w, void* state,
                   int64_t state_slot_stride, const int* cu, const int* seq_slot,
                   const int* seq_start, const int* tok_seq, const int* tok_pos,
                   const float* a_log, const float* dt_bias, float* q_out, float* k_out,
                   float* v_out, float* beta, float* decay, int dt, int Ttok, int nseq, int G,
                   int H, int dim, int vdim, int taps, int beta_col, int a_col, hipStream_t s) {
  if (taps < 1 || taps > MAXTAPS_SEQ || H % G) return -1;
  if (beta_col < 0 || beta_col + H > ld_proj || a_col + H > ld_proj) return -3;
  if (a_col >= 0 && !decay) return -3;
  if (Ttok <= 0) return 0;
  const int64_t lds = (int64_t)2 * G * dim * 4;
  if (lds > 64 * 1024) return -2;
  const int C = 2 * G * dim + H * vdim;
  // the state's rows are C wide, so C % 8 keeps every 8-channel group aligned
  const bool vec = dim % 8 == 0 && vdim % 8 == 0 && ld_proj % 8 == 0 &&
                   state_slot_stride % 8 == 0 && (taps == 2 || taps == 4);
#define PREP_VEC(TAPS)                                                                         \
  BY_DTYPE(dt, (delta_prep_vec_k<T, TAPS><<<Ttok, NT, lds, s>>>(                                \
                   (const T*)proj, ld_proj, (const T*)w, (const T*)state, state_slot_stride,   \
                   cu, seq_slot, tok_seq, tok_pos, a_log, dt_bias, q_out, k_out, v_out, beta,  \
                   decay, G, H, dim, vdim, beta_col, a_col)))
  if (vec && taps == 4)
    PREP_VEC(4);
  else if (vec && taps == 2)
    PREP_VEC(2);
  else
#undef PREP_VEC
  BY_DTYPE(dt, (delta_prep_k<T><<<Ttok, NT, lds, s>>>(
                   (const T*)proj, ld_proj, (const T*)w, (const T*)state, state_slot_stride, cu,
                   seq_slot, tok_seq, tok_pos, a_log, dt_bias, q_out, k_out, v_out, beta, decay,
                   G, H, dim, vdim, taps, beta_col, a_col)));
  if (taps > 1)
    BY_DTYPE(dt, (conv_tail_shift_k<T><<<nseq, NT, 0, s>>>((const T*)proj, ld_proj, (T*)state,
                                                           state_slot_stride, cu, seq_slot,
                                                           seq_start, C, taps)));
  return (int)hipGetLastError();
}

int dsv_sigmoid_pow(const void* z, const float* bias, float* out, int dt, int64_t n, int C,
                    float inv_tau, hipStream_t s) {
  if (n <= 0) return 0;
  BY_DTYPE(dt, (sigmoid_pow_k<T><<<nblocks(n, 256), 256, 0, s>>>((const T*)z, bias, out, n, C,
                                                                 inv_tau)));
  return (int)hipGetLastError();
}

// largest head size of keys the scan covers
int dsv_linear_scan_max_dim() { return SCAN_R * 16; }

// q/k/v: dtype dt with row strides in elements; decay [T, H] (channel_decay 0)
// or [T, H, dim]; beta [T, H] or null (plain form).
int dsv_linear_scan(const void* q, int ld_q, const void* k, int ld_k, const void* v, int ld_v,
                    const float* decay, int channel_decay, const float* beta, float* state,
                    const int* cu, const int* seq_slot, float* out, int dt, int nseq, int G, int H,
                    int dim, int vdim, float q_scale, hipStream_t s) {
  if (dim > dsv_linear_scan_max_dim() || dim < 1 || H % G) return -1;
  if (nseq <= 0) return 0;
  dim3 grid(nseq, H, (vdim + SCAN_COLS - 1) / SCAN_COLS);
#define SCAN(ROWS, DELTA, CD)                                                                   \
  BY_DTYPE(dt, (linear_scan_k<T, ROWS, DELTA, CD><<<grid, NT, 0, s>>>(                           \
                   (const T*)q, ld_q, (const T*)k, ld_k, (const T*)v, ld_v, decay, beta, state,  \
                   cu, seq_slot, out, G, H, dim, vdim, q_scale)))
#define SCAN_BY_ROWS(DELTA, CD)                   \
  do {                                            \
    if (dim <= SCAN_R * 4) SCAN(4, DELTA, CD);    \
    else if (dim <= SCAN_R * 8) SCAN(8, DELTA, CD);   \
    else SCAN(16, DELTA, CD);                     \
  } while (0)
  if (beta && channel_decay) SCAN_BY_ROWS(true, true);
  else if (beta) SCAN_BY_ROWS(true, false);
  else if (channel_decay) SCAN_BY_ROWS(false, true);
  else SCAN_BY_ROWS(false, false);
#undef SCAN_BY_ROWS
#undef SCAN
  return (int)hipGetLastError();
}

// act: 0 = SiLU of the gate, 1 = sigmoid
int dsv_head_norm_gate(const float* o, const float* w, const void* gate, int ld_gate, void* out,
                       int dt, int Ttok, int H, int vdim, float eps, int act, hipStream_t s) {
  if (Ttok <= 0) return 0;
  if (act == 1)
    BY_DTYPE(dt, (head_norm_gate_k<T, true><<<Ttok, NT, 0, s>>>(o, w, (const T*)gate, ld_gate,
                                                                (T*)out, H, vdim, eps)));
  else if (act == 0)
    BY_DTYPE(dt, (head_norm_gate_k<T, false><<<Ttok, NT, 0, s>>>(o, w, (const T*)gate, ld_gate,
                                                                 (T*)out, H, vdim, eps)));
  else
    return -1;
  return (int)hipGetLastError();
}

int dsv_softplus_decay(const void* z, int ld_z, const float* bias, const float* a_log, float* out,
                       int dt, int64_t rows, int H, int dim, hipStream_t s) {
  if (rows * H * dim <= 0) return 0;
  const size_t align = dt == 0 ? 32 : 16;
  if (dim % 8 == 0 && ld_z % 8 == 0 && (uintptr_t)z % align == 0 && (uintptr_t)bias % 32 == 0) {
    BY_DTYPE(dt, (softplus_decay8_k<T><<<nblocks(rows * (H * dim / 8), 256), 256, 0, s>>>(
                     (const T*)z, ld_z, bias, a_log, out, rows, H, dim)));
    return (int)hipGetLastError();
  }
  BY_DTYPE(dt, (softplus_decay_k<T><<<nblocks(rows * H * dim, 256), 256, 0, s>>>(
                   (const T*)z, ld_z, bias, a_log, out, rows, H, dim)));
  return (int)hipGetLastError();
}

// norm: 0 none, 2 per head (weights of size dim); half: rotary pairing
// (i, i + rot_dims/2) instead of (2i, 2i+1); v_eps < 0: values pass unchanged.
int dsv_attn_prep_heads(const void* proj, int ld_proj, const float* wq, const float* wk,
                        const int* tok_pos, const int* tok_row, const float* cosT,
                        const float* sinT, void* pool, void* q_out, int dt, int Ttok, int H,
                        int G, int dim, int vdim, int rot_dims, int own_kv, int norm, int half,
                        float eps, float v_eps, hipStream_t s) {
  if (rot_dims < 0 || (rot_dims & 1) || rot_dims > dim || H % G) return -1;
  if ((norm != 0 && norm != 2) || (norm == 2 && (!wq || (own_kv && !wk)))) return -2;
  if (rot_dims > 0 && (!cosT || !sinT)) return -3;
  if (Ttok <= 0) return 0;
  const int big = dim > vdim ? dim : vdim;
  // vector form: whole groups of 8 everywhere; with the half pairing a group's
  // partner is a whole group too
  const bool vec = dim % 8 == 0 && vdim % 8 == 0 && ld_proj % 8 == 0 && big <= 512 &&
                   (half ? rot_dims % 16 == 0 : true) && (uintptr_t)proj % 16 == 0;
#define PREPH(HALF, LG)                                                                        \
  BY_DTYPE(dt, (attn_prep_heads_vec_k<T, HALF, LG><<<Ttok, NT, 0, s>>>(                         \
                   (const T*)proj, ld_proj, wq, wk, tok_pos, tok_row, cosT, sinT, (T*)pool,    \
                   (T*)q_out, H, G, dim, vdim, rot_dims, own_kv, norm, eps, v_eps)))
#define PREPH_BY_LG(HALF)                        \
  do {                                           \
    if (big <= 32) PREPH(HALF, 4);               \
    else if (big <= 64) PREPH(HALF, 8);          \
    else if (big <= 128) PREPH(HALF, 16);        \
    else if (big <= 256) PREPH(HALF, 32);        \
    else PREPH(HALF, 64);                        \
  } while (0)
  if (vec) {
    if (half) PREPH_BY_LG(true);
    else PREPH_BY_LG(false);
    return (int)hipGetLastError();
  }
#undef PREPH_BY_LG
#undef PREPH
  if (half)
    BY_DTYPE(dt, (attn_prep_heads_k<T, true><<<Ttok, NT, 0, s>>>(
                     (const T*)proj, ld_proj, wq, wk, tok_pos, tok_row, cosT, sinT, (T*)pool,
                     (T*)q_out, H, G, dim, vdim, rot_dims, own_kv, norm, eps, v_eps)));
  else
    BY_DTYPE(dt, (attn_prep_heads_k<T, false><<<Ttok, NT, 0, s>>>(
                     (const T*)proj, ld_proj, wq, wk, tok_pos, tok_row, cosT, sinT, (T*)pool,
                     (T*)q_out, H, G, dim, vdim, rot_dims, own_kv, norm, eps, v_eps)));
  return (int)hipGetLastError();
}

// out_dt: 0 float, otherwise the input's type
int dsv_conv_silu(const void* x, int ld_x, const void* w, const float* bias, void* state,
                  int64_t state_slot_stride, const int* cu, const int* seq_slot,
                  const int* seq_start, const int* tok_seq, const int* tok_pos, void* out,
                  int dt, int out_dt, int Ttok, int nseq, int C, int taps, hipStream_t s) {
  if (taps < 1 || taps > MAXTAPS_SEQ || ld_x < C) return -1;
  if (Ttok <= 0) return 0;
  const bool vec = C % 8 == 0 && ld_x % 8 == 0 && state_slot_stride % 8 == 0 &&
                   (uintptr_t)x % 16 == 0 && taps >= 2 && taps <= 4;
  const dim3 grid(Ttok, Ttok < 512 ? (C / 8 + NT - 1) / NT : 1);
#define CONVV(TAPS)                                                                             \
  do {                                                                                          \
    if (out_dt == 0)                                                                            \
      BY_DTYPE(dt, (conv_silu_vec_k<T, float, TAPS><<<grid, NT, 0, s>>>(                         \
                       (const T*)x, ld_x, (const T*)w, bias, (const T*)state,                   \
                       state_slot_stride, cu, seq_slot, tok_seq, tok_pos, (float*)out, C)));    \
    else                                                                                        \
      BY_DTYPE(dt, (conv_silu_vec_k<T, T, TAPS><<<grid, NT, 0, s>>>(                             \
                       (const T*)x, ld_x, (const T*)w, bias, (const T*)state,                   \
                       state_slot_stride, cu, seq_slot, tok_seq, tok_pos, (T*)out, C)));        \
  } while (0)
  if (vec && taps == 4) CONVV(4);
  else if (vec && taps == 3) CONVV(3);
  else if (vec && taps == 2) CONVV(2);
  else if (out_dt == 0)
#undef CONVV
    BY_DTYPE(dt, (conv_silu_k<T, float><<<Ttok, NT, 0, s>>>(
                     (const T*)x, ld_x, (const T*)w, bias, (const T*)state, state_slot_stride,
                     cu, seq_slot, tok_seq, tok_pos, (float*)out, C, taps)));
  else
    BY_DTYPE(dt, (conv_silu_k<T, T><<<Ttok, NT, 0, s>>>(
                     (const T*)x, ld_x, (const T*)w, bias, (const T*)state, state_slot_stride,
                     cu, seq_slot, tok_seq, tok_pos, (T*)out, C, taps)));
  if (taps > 1)
    BY_DTYPE(dt, (conv_tail_shift_k<T><<<nseq, NT, 0, s>>>((const T*)x, ld_x, (T*)state,
                                                           state_slot_stride, cu, seq_slot,
                                                           seq_start, C, taps)));
  return (int)hipGetLastError();
}

int dsv_ssd_prep(const void* proj, int ld_proj, const void* w, const float* bias, void* state,
                 int64_t state_slot_stride, const int* cu, const int* seq_slot,
                 const int* seq_start, const int* tok_seq, const int* tok_pos,
                 const float* a_log, const float* dt_bias, float* x_out, float* v_out,
                 float* b_out, float* c_out, float* decay, int dt, int Ttok, int nseq, int H,
                 int P, int G, int N, int taps, hipStream_t s) {
  if (taps < 1 || taps > MAXTAPS_SEQ || H % G || H > 16384) return -1;
  if (ld_proj < 2 * H * P + 2 * G * N + H) return -2;
  if (Ttok <= 0) return 0;
  const int inner = H * P, C = inner + 2 * G * N;
  const bool vec = P % 8 == 0 && (G * N) % 8 == 0 && ld_proj % 8 == 0 &&
                   state_slot_stride % 8 == 0 && (uintptr_t)proj % 16 == 0 && taps >= 2 &&
                   taps <= 4;
  const dim3 grid(Ttok, Ttok < 512 ? (C / 8 + NT - 1) / NT : 1);
#define SSDV(TAPS)                                                                             \
  BY_DTYPE(dt, (ssd_prep_vec_k<T, TAPS><<<grid, NT, 0, s>>>(                                    \
                   (const T*)proj, ld_proj, (const T*)w, bias, (const T*)state,                \
                   state_slot_stride, cu, seq_slot, tok_seq, tok_pos, a_log, dt_bias, x_out,   \
                   v_out, b_out, c_out, decay, H, P, G, N)))
  if (vec && taps == 4) SSDV(4);
  else if (vec && taps == 3) SSDV(3);
  else if (vec && taps == 2) SSDV(2);
  else
#undef SSDV
  BY_DTYPE(dt, (ssd_prep_k<T><<<Ttok, NT, H * sizeof(float), s>>>(
                   (const T*)proj, ld_proj, (const T*)w, bias, (const T*)state,
                   state_slot_stride, cu, seq_slot, tok_seq, tok_pos, a_log, dt_bias, x_out,
                   v_out, b_out, c_out, decay, H, P, G, N, taps)));
  if (taps > 1)
    BY_DTYPE(dt, (conv_tail_shift_k<T><<<nseq, NT, 0, s>>>(
                     (const T*)proj + inner, ld_proj, (T*)state, state_slot_stride, cu, seq_slot,
                     seq_start, C, taps)));
  return (int)hipGetLastError();
}

int dsv_gate_group_norm(const float* o, const float* x, const float* skip, const void* gate,
                        int ld_gate, const float* w, void* out, int dt, int Ttok, int H, int vdim,
                        int parts, float eps, hipStream_t s) {
  const int n = H * vdim;
  if (parts < 1 || n % parts || ld_gate < n) return -1;
  if (Ttok <= 0) return 0;
  const int len = n / parts;
  if (len % 8 == 0 && vdim % 8 == 0 && ld_gate % 8 == 0 && len <= 8 * NT * GGN &&
      (uintptr_t)gate % 16 == 0)
    BY_DTYPE(dt, (gate_group_norm_vec_k<T><<<dim3(Ttok, parts), NT, 0, s>>>(
                     o, x, skip, (const T*)gate, ld_gate, w, (T*)out, n, vdim, parts, eps)));
  else
    BY_DTYPE(dt, (gate_group_norm_k<T><<<dim3(Ttok, parts), NT, 0, s>>>(
                     o, x, skip, (const T*)gate, ld_gate, w, (T*)out, n, vdim, parts, eps)));
  return (int)hipGetLastError();
}

// largest state size of the selective scan
int dsv_selective_scan_max_state() { return 256; }

int dsv_selective_scan(const void* x, int ld_x, const float* dt_pre, const float* dt_bias,
                       const float* a_log, const void* Bm, const void* Cm, int ld_bc,
                       const float* skip, const void* z, int ld_z, float* state, const int* cu,
                       const int* seq_slot, void* out, int ld_out, int dt, int nseq, int ch,
                       int N, float out_scale, hipStream_t s) {
  if (N < 1 || N > dsv_selective_scan_max_state() || ch < 1) return -1;
  if (ld_x < ch || ld_z < ch || ld_out < ch || ld_bc < N) return -2;
  if (nseq <= 0) return 0;
#define SSCAN(NS)                                                                              \
  do {                                                                                         \
    dim3 grid(nseq, (ch + SCH - 1) / SCH);                                                     \
    BY_DTYPE(dt, (selective_scan_k<T, NS><<<grid, NT, 0, s>>>(                                  \
                     (const T*)x, ld_x, dt_pre, dt_bias, a_log, (const T*)Bm, (const T*)Cm,    \
                     ld_bc, skip, (const T*)z, ld_z, state, cu, seq_slot, (T*)out, ld_out, ch, \
                     N, out_scale)));                                                          \
  } while (0)
  if (N <= 16) SSCAN(1);
  else if (N <= 32) SSCAN(2);
  else if (N <= 64) SSCAN(4);
  else if (N <= 128) SSCAN(8);
  else SSCAN(16);
#undef SSCAN
  return (int)hipGetLastError();
}

}  // extern "C"
