// Latent (compressed-KV) attention over a paged row pool for MI355X (gfx950):
// prologue (latent norm, rotations, gate, cache write), exact and MFMA-tile
// attention with key splits, and the gated head merge.
//
// Plain C ABI (raw device pointers + a hipStream_t) so the library builds in
// seconds with hipcc alone and is loaded through ctypes. dtype codes:
// 0 = float, 1 = bfloat16. Everything the models define as 32-bit (norm
// statistics, rotations, scores, softmax, the weighted sums, router and
// gates) is computed in float here whatever the storage type.

#include "serving_common.h"

namespace {

// ------------------------------------------------------ latent prologue
// Three row sources (each a column slice with a row stride of its own, so they
// may be parts of one projection or come from different products):
//   q    = [ H x (dim + rot) ]      kv = [ latent (rank) | k_rot (rot) ]
//   gate = [ H ] logits, or null (no gate output)
// HALF pairs coordinate i with i + rot_dims/2 among the first rot_dims of a
// rotated part; otherwise neighbours (2i, 2i+1) form a pair.
template <typename T>
__global__ __launch_bounds__(NT) void latent_prep_k(
    const T* __restrict__ q_src, int ld_q, const T* __restrict__ kv_src, int ld_kv,
    const T* __restrict__ gate_src, int ld_g, const float* __restrict__ norm_w,
    const int* __restrict__ tok_pos, const int* __restrict__ tok_row,
    const float* __restrict__ cosT, const float* __restrict__ sinT,
    T* __restrict__ pool, T* __restrict__ q_nope, T* __restrict__ q_rot,
    float* __restrict__ gate, int Ttok, int H, int dim, int rot, int rank,
    int rot_dims, float eps, int half_layout) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x;
  const T* pq = q_src + (int64_t)t * ld_q;
  const T* pkv = kv_src + (int64_t)t * ld_kv;
  const int half = rot_dims >> 1;
  const float* cs = rot_dims ? cosT + (int64_t)tok_pos[t] * half : nullptr;
  const float* sn = rot_dims ? sinT + (int64_t)tok_pos[t] * half : nullptr;
  T* row = pool + (int64_t)tok_row[t] * (rank + rot);
  float ss = 0.f;
  for (int c = threadIdx.x; c < rank; c += NT) {
    float v = ld(pkv + c);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float k = rsqrtf(ss / (float)rank + eps);
  for (int c = threadIdx.x; c < rank; c += NT)
    st(row + c, ld(pkv + c) * k * norm_w[c]);
  // one coordinate of a rotated part: its partner, its pair and its side
  auto turn = [&](const T* src, int c) -> float {
    float v = ld(src + c);
    if (c < rot_dims) {
      int partner, pair;
      bool second;
      if (half_layout) {
        second = c >= half;
        partner = second ? c - half : c + half;
        pair = second ? c - half : c;
      } else {
        second = c & 1;
        partner = c ^ 1;
        pair = c >> 1;
      }
      const float o = ld(src + partner);
      const float co = cs[pair], si = sn[pair];
      v = second ? v * co + o * si : v * co - o * si;
    }
    return v;
  };
  // shared rotated key part
  for (int c = threadIdx.x; c < rot; c += NT) st(row + rank + c, turn(pkv + rank, c));
  // queries: rotated part [T, H, rot]; unrotated part regrouped [H, T, dim]
  for (int i = threadIdx.x; i < H * rot; i += NT) {
    const int h = i / rot, c = i - h * rot;
    st(q_rot + ((int64_t)t * H + h) * rot + c, turn(pq + h * (dim + rot) + dim, c));
  }
  for (int i = threadIdx.x; i < H * dim; i += NT) {
    const int h = i / dim, c = i - h * dim;
    q_nope[((int64_t)h * Ttok + t) * dim + c] = pq[h * (dim + rot) + c];
  }
  if (gate_src)
    for (int h = threadIdx.x; h < H; h += NT)
      gate[(int64_t)t * H + h] = 1.f / (1.f + expf(-ld(gate_src + (int64_t)t * ld_g + h)));
}

// ------------------------------------------------------ latent attention
// Generic exact kernel: one block per (token, key split), heads in groups of
// HG. Keys are staged through LDS in chunks (odd row stride: conflict-free
// column reads); scores, online softmax and the weighted sum of latents are
// float. With nsplit > 1 the block writes (max, sum, unnormalised sum) and
// latent_attn_merge_k finishes.
constexpr int HG = 8;
constexpr int RPT = 4;  // latent columns per thread: rank <= RPT * NT

template <typename T>
__global__ __launch_bounds__(NT) void latent_attn_k(
    const T* __restrict__ q_lat,  // [H, Ttok, rank]
    const T* __restrict__ q_rot,  // [Ttok, H, rot]
    const T* __restrict__ pool,   // rows of rank+rot
    const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
    const int* __restrict__ table, int maxb, int bs,
    T* __restrict__ out,          // [H, Ttok, rank]
    float* __restrict__ part,     // [Ttok, nsplit, H, rank + 2] when nsplit > 1
    int Ttok, int H, int rank, int rot, int KC, int nsplit, float scale, int window,
    const float* __restrict__ sink) {
  extern __shared__ float smem[];
  const int D = rank + rot;
  const int DS = D | 1;
  float* qs = smem;                       // [HG][D]
  float* sc = qs + HG * D;                // [HG][KC]
  float* alpha = sc + HG * KC;            // [HG] rescale of this chunk
  float* mrun = alpha + HG;               // [HG] running max
  float* lrun = mrun + HG;                // [HG] running sum
  T* ks = reinterpret_cast<T*>(lrun + HG);   // [KC][DS]
  const int t = blockIdx.x, split = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int s = tok_seq[t];
  // visible keys klo .. tok_pos[t]; chunks count from klo
  const int klo = window > 0 ? max(0, tok_pos[t] + 1 - window) : 0;
  const int nkeys = tok_pos[t] + 1 - klo;
  const int* tab = table + (int64_t)s * maxb;
  // key range of this split, in whole chunks
  const int nchunk = (nkeys + KC - 1) / KC;
  const int cps = (nchunk + nsplit - 1) / nsplit;
  const int c_lo = split * cps, c_hi = min(nchunk, c_lo + cps);

  for (int h0 = 0; h0 < H; h0 += HG) {
    const int nh = min(HG, H - h0);
    __syncthreads();
    for (int i = tid; i < nh * D; i += NT) {
      const int h = i / D, c = i - h * D;
      qs[i] = c < rank ? ld(q_lat + ((int64_t)(h0 + h) * Ttok + t) * rank + c)
                       : ld(q_rot + ((int64_t)t * H + h0 + h) * rot + c - rank);
    }
    if (tid < HG) {
      mrun[tid] = -INFINITY;
      lrun[tid] = 0.f;
    }
    float acc[HG][RPT];
#pragma unroll
    for (int h = 0; h < HG; ++h)
#pragma unroll
      for (int i = 0; i < RPT; ++i) acc[h][i] = 0.f;
    for (int ch = c_lo; ch < c_hi; ++ch) {
      const int k0 = ch * KC;
      const int nk = min(KC, nkeys - k0);
      __syncthreads();
      for (int i = tid; i < nk * D; i += NT) {
        const int kk = i / D, c = i - kk * D;
        const int p = klo + k0 + kk;
        const int64_t r = (int64_t)tab[p / bs] * bs + p % bs;
        ks[kk * DS + c] = pool[r * D + c];
      }
      __syncthreads();
      for (int i = tid; i < nh * KC; i += NT) {
        const int h = i / KC, kk = i - h * KC;
        float d = -INFINITY;
        if (kk < nk) {
          d = 0.f;
          const float* q = qs + h * D;
          const T* kr = ks + kk * DS;
          for (int c = 0; c < D; ++c) d += q[c] * ld(kr + c);
          d *= scale;
        }
        sc[i] = d;
      }
      __syncthreads();
      // online softmax: wave w owns heads w, w + 4, ...; scores become weights
      for (int h = wid; h < nh; h += NT / 64) {
        float mx = -INFINITY;
        for (int kk = lane; kk < nk; kk += 64) mx = fmaxf(mx, sc[h * KC + kk]);
        mx = wave_max(mx);
        const float m_old = mrun[h];
        const float m_new = fmaxf(m_old, mx);
        float psum = 0.f;
        for (int kk = lane; kk < nk; kk += 64) {
          const float p = expf(sc[h * KC + kk] - m_new);
          sc[h * KC + kk] = p;
          psum += p;
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
      for (int h = 0; h < HG; ++h) {
        if (h < nh) {
          const float a = alpha[h];
#pragma unroll
          for (int i = 0; i < RPT; ++i) acc[h][i] *= a;
        }
      }
      // weighted sum of latents: thread owns columns tid + i*NT
      for (int kk = 0; kk < nk; ++kk) {
        float c[RPT];
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
          const int col = tid + i * NT;
          c[i] = col < rank ? ld(ks + kk * DS + col) : 0.f;
        }
#pragma unroll
        for (int h = 0; h < HG; ++h) {
          if (h < nh) {
            const float p = sc[h * KC + kk];
#pragma unroll
            for (int i = 0; i < RPT; ++i) acc[h][i] += p * c[i];
          }
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < HG; ++h) {
      if (h < nh) {
        if (nsplit == 1) {
          float inv = 1.f / lrun[h];
          if (sink) {  // one more term of the denominator, no value
            const float sk = sink[h0 + h];
            const float m2 = fmaxf(mrun[h], sk);
            const float f = expf(mrun[h] - m2);
            inv = f / (lrun[h] * f + expf(sk - m2));
          }
#pragma unroll
          for (int i = 0; i < RPT; ++i) {
            const int col = tid + i * NT;
            if (col < rank)
              st(out + ((int64_t)(h0 + h) * Ttok + t) * rank + col, acc[h][i] * inv);
          }
        } else {
          float* pp = part + (((int64_t)t * nsplit + split) * H + h0 + h) * (rank + 2);
          if (tid == 0) {
            pp[0] = mrun[h];
            pp[1] = lrun[h];
          }
#pragma unroll
          for (int i = 0; i < RPT; ++i) {
            const int col = tid + i * NT;
            if (col < rank) pp[2 + col] = acc[h][i];
          }
        }
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void latent_attn_merge_k(
    const float* __restrict__ part, T* __restrict__ out, int Ttok, int H,
    int rank, int nsplit, const float* __restrict__ sink) {
  const int t = blockIdx.x, h = blockIdx.y;
  float m = sink ? sink[h] : -INFINITY;
  for (int s = 0; s < nsplit; ++s)
    m = fmaxf(m, part[(((int64_t)t * nsplit + s) * H + h) * (rank + 2)]);
  float l = sink ? expf(sink[h] - m) : 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float* pp = part + (((int64_t)t * nsplit + s) * H + h) * (rank + 2);
    if (pp[1] > 0.f) l += pp[1] * expf(pp[0] - m);
  }
  for (int c = threadIdx.x; c < rank; c += NT) {
    float a = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const float* pp = part + (((int64_t)t * nsplit + s) * H + h) * (rank + 2);
      if (pp[1] > 0.f) a += pp[2 + c] * expf(pp[0] - m);
    }
    st(out + ((int64_t)h * Ttok + t) * rank + c, a / l);
  }
}

// ------------------------------------------- latent attention, MFMA tiles
// bf16 prefill path. The rows of one sequence's step are (token, head) pairs,
// token-major: row m belongs to token m / H and sees keys 0..start + m / H, so
// all heads of a token share its key range and the whole step is one
// [count*H, Dk] x [Dk, keys] product per sequence. A workgroup of 4 waves owns
// 128 rows (32 per wave) and walks the keys 32 at a time:
//   S^T[key, row] = mfma(A = K tile from LDS, B = Q fragments in registers)
//   online softmax per row (one row per lane pair, fp32)
//   O^T[d, row]  += mfma(A = V^T tile from LDS, B = P fragments)
// mfma_f32_32x32x16_bf16 layouts: A row = lane&31, k = reg + 8*(lane>>5);
// B col = lane&31, k = reg + 8*(lane>>5); C/D col = lane&31,
// row = (reg&3) + 8*(reg>>2) + 4*(lane>>5).
typedef short bf16x8s __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int TB_ROWS = 128;  // rows per workgroup
constexpr int TB_KEYS = 32;   // keys per step
constexpr int VT_STRIDE = TB_KEYS + 8;
constexpr float LAZY_MAX = 8.f;

// SPLIT = 2 (wide latents): two waves share a row block so that the operands
// fit the register file. Each keeps half of the query's dimensions and half of
// the output columns; the two partial score tiles are summed through LDS. The
// workgroup then owns 64 rows.
template <int DVB, int DKT_MAX, int SPLIT, bool PREFETCH>
__global__ __launch_bounds__(256) void latent_attn_mfma_k(
    const short* __restrict__ q_lat,  // [H, Ttok, rank]
    const short* __restrict__ q_rot,  // [Ttok, H, rot]
    const short* __restrict__ pool, const int* __restrict__ work,
    const int* __restrict__ cu, const int* __restrict__ seq_start,
    const int* __restrict__ table, int maxb, int bs, bf16* __restrict__ out,
    float* __restrict__ part,  // [Ttok, nsplit, H, rank + 2] when nsplit > 1
    int Ttok, int H, int rank, int rot, int nsplit, float scale, int window,
    const float* __restrict__ sink) {
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  constexpr int DVW = DVB / SPLIT;     // output blocks of this wave
  constexpr int ROWS = TB_ROWS / SPLIT;
  constexpr int CPT = (DKT_MAX + 3) / 4;  // staged 16-byte chunks per thread
  constexpr int QKT = DKT_MAX / SPLIT;    // query fragments of this wave
  const int Dk = rank + rot;
  const int DkP = (Dk + 15) & ~15;
  const int DKT = DkP >> 4;
  const int KSS = DkP + 8;
  short* Ks = reinterpret_cast<short*>(smem_raw);  // [TB_KEYS][KSS]
  short* Vt = Ks + TB_KEYS * KSS;                  // [DVB*32][VT_STRIDE]
  float* xch = reinterpret_cast<float*>(Vt + DVB * 32 * VT_STRIDE);  // [4][16][64]
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int hl = lane >> 5, l31 = lane & 31;
  const int s = work[2 * blockIdx.x], m0 = work[2 * blockIdx.x + 1];
  const int split = blockIdx.y;
  const int count = cu[s + 1] - cu[s], start = seq_start[s];
  const int rows = count * H;
  const int part_id = wid % SPLIT;
  const int m_raw = m0 + (wid / SPLIT) * 32 + l31;
  const int m = min(m_raw, rows - 1);
  const int j = m / H, h = m - j * H;
  const int t = cu[s] + j;
  const int qpos = start + j;
  const int kmax = start + min(m0 + ROWS - 1, rows - 1) / H;  // inclusive
  const int* tab = table + (int64_t)s * maxb;
  // first key this row sees, and the tile's earliest (its first row's)
  const int klo = window > 0 ? max(0, qpos - window + 1) : 0;
  const int kmin = window > 0 ? max(0, start + m0 / H - window + 1) : 0;
  // this split's key steps
  const int step0 = kmin / TB_KEYS;
  const int nsteps = kmax / TB_KEYS + 1 - step0;
  const int per = (nsteps + nsplit - 1) / nsplit;
  const int s_lo = step0 + split * per, s_hi = min(step0 + nsteps, s_lo + per);
  float* pp = nullptr;
  if (nsplit > 1)
    pp = part + (((int64_t)t * nsplit + split) * H + h) * (rank + 2);
  if (s_lo >= s_hi) {  // block-uniform: nothing to see in this split
    if (m_raw < rows && part_id == 0 && hl == 0) {
      pp[0] = -INFINITY;
      pp[1] = 0.f;
    }
    return;
  }

  // this wave's share of the key dimension: fragments kt_lo .. kt_lo + QKT - 1
  const int kt_lo = part_id * QKT;
  const bool q_vec = (rank & 7) == 0 && (rot & 7) == 0;
  bf16x8s qf[QKT];
#pragma unroll
  for (int i = 0; i < QKT; ++i) {
    const int kt = kt_lo + i;
    if (kt < DKT) {
      const int d0 = 16 * kt + 8 * hl;
      if (q_vec && d0 + 8 <= rank) {
        qf[i] = *reinterpret_cast<const bf16x8s*>(q_lat + ((int64_t)h * Ttok + t) * rank + d0);
      } else if (q_vec && d0 >= rank && d0 + 8 <= Dk) {
        qf[i] = *reinterpret_cast<const bf16x8s*>(q_rot + ((int64_t)t * H + h) * rot + d0 - rank);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int d = d0 + e;
          short v = 0;
          if (d < rank)
            v = q_lat[((int64_t)h * Ttok + t) * rank + d];
          else if (d < Dk)
            v = q_rot[((int64_t)t * H + h) * rot + d - rank];
          qf[i][e] = v;
        }
      }
    }
  }
  f32x16 oacc[DVW];
#pragma unroll
  for (int db = 0; db < DVW; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
  float mrun = -INFINITY, lrun = 0.f;
  const int cpk = DkP >> 3;  // 8-element chunks per key
  const bool vec_ok = (Dk & 7) == 0;

  // Staging: chunk c of a tile is (dims 8*(c>>5).., key c&31): neighbouring
  // lanes take neighbouring keys, so the transposed writes fall into one row.
  // Every chunk of a thread belongs to the same key (256 is a multiple of 32),
  // so the thread resolves ONE pool row per tile through the block table, and
  // does so a step ahead: the data loads never wait for a table load.
  auto row_of = [&](int k0) -> int64_t {
    const int p = k0 + (tid & 31);
    return p <= kmax ? (int64_t)tab[p / bs] * bs + p % bs : (int64_t)-1;
  };
  auto fetch_one = [&](int i, int64_t row) -> bf16x8s {
    const int c = tid + i * 256;
    bf16x8s v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = 0;
    if (c < TB_KEYS * cpk && row >= 0) {
      const int ch = c >> 5;
      const short* src = pool + row * Dk + ch * 8;
      if (vec_ok && ch * 8 + 8 <= Dk) {
        v = *reinterpret_cast<const bf16x8s*>(src);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (ch * 8 + e < Dk) v[e] = src[e];
      }
    }
    return v;
  };
  auto stash_one = [&](int i, const bf16x8s& v) {
    const int c = tid + i * 256;
    if (c < TB_KEYS * cpk) {
      const int ch = c >> 5, key = c & 31;
      *reinterpret_cast<bf16x8s*>(Ks + key * KSS + ch * 8) = v;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int d = ch * 8 + e;
        if (d < DVB * 32) Vt[d * VT_STRIDE + key] = d < rank ? v[e] : (short)0;
      }
    }
  };
  bf16x8s pre[PREFETCH ? CPT : 1];
  auto fetch = [&](int64_t row) {
#pragma unroll
    for (int i = 0; i < CPT; ++i)
      if (PREFETCH) pre[i] = fetch_one(i, row);
  };
  auto stash = [&](int64_t row) {
    if (PREFETCH) {
#pragma unroll
      for (int i = 0; i < CPT; ++i) stash_one(i, pre[i]);
    } else {
      // the tile's loads all in flight, consumed before the products start
      // (registers that live only here, unlike a prefetch across the step)
#pragma unroll 1
      for (int i = 0; i < CPT; i += 10) {
        bf16x8s v[10];
#pragma unroll
        for (int u = 0; u < 10; ++u) v[u] = fetch_one(i + u, row);
#pragma unroll
        for (int u = 0; u < 10; ++u) stash_one(i + u, v[u]);
      }
    }
  };

  // PREFETCH keeps the next tile's loads in flight during the products; the
  // widest class has no registers to spare for that. row_next is the pool
  // row of this thread's key in the tile that is fetched next.
  int64_t row_next = row_of(s_lo * TB_KEYS);
  if (PREFETCH) {
    fetch(row_next);
    row_next = row_of((s_lo + 1) * TB_KEYS);
  }
  for (int step = s_lo; step < s_hi; ++step) {
    const int k0 = step * TB_KEYS;
    __syncthreads();
    stash(row_next);          // without PREFETCH: fetches tile `step` itself
    __syncthreads();
    if (PREFETCH) {
      if (step + 1 < s_hi) fetch(row_next);
      row_next = row_of(k0 + 2 * TB_KEYS);
    } else {
      row_next = row_of(k0 + TB_KEYS);
    }
    f32x16 st;
#pragma unroll
    for (int r = 0; r < 16; ++r) st[r] = 0.f;
#pragma unroll
    for (int i = 0; i < QKT; ++i) {
      const int kt = kt_lo + i;
      if (kt < DKT) {
        const bf16x8s kf =
            *reinterpret_cast<const bf16x8s*>(Ks + l31 * KSS + 16 * kt + 8 * hl);
        st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[i], st, 0, 0, 0);
      }
    }
    if (SPLIT == 2) {  // add the partner wave's half of the dot products
#pragma unroll
      for (int r = 0; r < 16; ++r) xch[(wid * 16 + r) * 64 + lane] = st[r];
      __syncthreads();
#pragma unroll
      for (int r = 0; r < 16; ++r) st[r] += xch[((wid ^ 1) * 16 + r) * 64 + lane];
    }
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = k0 + (r & 3) + 8 * (r >> 2) + 4 * hl;
      const float v = (key <= qpos && key >= klo) ? st[r] * scale : -INFINITY;
      st[r] = v;
      mx = fmaxf(mx, v);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    // The running maximum follows the scores lazily: it moves only when a
    // score exceeds it by more than LAZY_MAX (weights stay below e^LAZY_MAX,
    // harmless in fp32), so most steps need no rescaling of the sums at all.
    // A row that has seen no key yet (a later split of an early token) keeps
    // weight zero without producing inf - inf.
    const float m_new = (mx > mrun + LAZY_MAX) ? mx : mrun;
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __expf(mrun - m_use);
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float p = __expf(st[r] - m_use);
      st[r] = p;
      psum += p;
    }
    psum += __shfl_xor(psum, 32, 64);
    lrun = lrun * alpha + psum;
    if (__any(m_new != mrun)) {
#pragma unroll
      for (int db = 0; db < DVW; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
    }
    mrun = m_new;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      // B fragment of P: keys 16*ks + 8*hl + 0..7 of this lane's row; half of
      // them sit in the partner lane (lane ^ 32)
      bf16x8s pf;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float a0 = st[i + 8 * ks], a1 = st[i + 8 * ks + 4];
        const float recv = __shfl_xor(hl ? a0 : a1, 32, 64);
        pf[i] = f2bf_bits(hl ? recv : a0);
        pf[i + 4] = f2bf_bits(hl ? a1 : recv);
      }
#pragma unroll
      for (int db = 0; db < DVW; ++db) {
        const bf16x8s vf = *reinterpret_cast<const bf16x8s*>(
            Vt + (32 * (part_id * DVW + db) + l31) * VT_STRIDE + 16 * ks + 8 * hl);
        oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf, oacc[db], 0, 0, 0);
      }
    }
  }
  if (m_raw < rows) {
    if (nsplit > 1) {
      if (part_id == 0 && hl == 0) {
        pp[0] = mrun;
        pp[1] = lrun;
      }
#pragma unroll
      for (int db = 0; db < DVW; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int d = 32 * (part_id * DVW + db) + (r & 3) + 8 * (r >> 2) + 4 * hl;
          if (d < rank) pp[2 + d] = oacc[db][r];
        }
    } else {
      float inv = 1.f / lrun;
      if (sink) {  // one more term of the denominator, no value
        const float sk = sink[h];
        const float m2 = fmaxf(mrun, sk);
        const float f = __expf(mrun - m2);
        inv = f / (lrun * f + __expf(sk - m2));
      }
      bf16* o = out + ((int64_t)h * Ttok + t) * rank;
#pragma unroll
      for (int db = 0; db < DVW; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int d = 32 * (part_id * DVW + db) + (r & 3) + 8 * (r >> 2) + 4 * hl;
          if (d < rank) o[d] = __float2bfloat16(oacc[db][r] * inv);
        }
    }
  }
}

template <int DVB, int DKT_MAX, int SPLIT, bool PREFETCH>
int launch_latent_attn_mfma(const void* q_lat, const void* q_rot, const void* pool,
                            const int* work, int nwork, const int* cu, const int* seq_start,
                            const int* table, int maxb, int bs, void* out, float* part,
                            int Ttok, int H, int rank, int rot, int nsplit, float scale,
                            int window, const float* sink, hipStream_t s) {
  const int DkP = (rank + rot + 15) & ~15;
  const size_t lds = (size_t)TB_KEYS * (DkP + 8) * 2 + (size_t)DVB * 32 * VT_STRIDE * 2 +
                     (SPLIT == 2 ? 4 * 16 * 64 * 4 : 0);
  auto kern = latent_attn_mfma_k<DVB, DKT_MAX, SPLIT, PREFETCH>;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  kern<<<dim3(nwork, nsplit), 256, lds, s>>>((const short*)q_lat, (const short*)q_rot,
                                             (const short*)pool, work, cu, seq_start, table, maxb,
                                             bs, (bf16*)out, part, Ttok, H, rank, rot, nsplit,
                                             scale, window, sink);
  if (nsplit > 1)
    latent_attn_merge_k<bf16><<<dim3(Ttok, H), NT, 0, s>>>(part, (bf16*)out, Ttok, H, rank, nsplit,
                                                           sink);
  return (int)hipGetLastError();
}

// out[t, h*v + c] = o[h, t, c] * gate[t, h] (gate null: heads merged as they are)
template <typename T>
__global__ void gate_merge_k(const T* __restrict__ o, const float* __restrict__ gate,
                             T* __restrict__ out, int Ttok, int H, int v) {
  const int64_t n = (int64_t)Ttok * H * v;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int c = i % v;
    const int h = (i / v) % H;
    const int64_t t = i / ((int64_t)v * H);
    st(out + i, ld(o + ((int64_t)h * Ttok + t) * v + c) * (gate ? gate[t * H + h] : 1.f));
  }
}

// the same, eight neighbouring columns of a head per thread (v a multiple of 8)
template <typename T>
__global__ void gate_merge8_k(const T* __restrict__ o, const float* __restrict__ gate,
                              T* __restrict__ out, int Ttok, int H, int v) {
  const int v8 = v >> 3, per_tok = H * v8;
  const int64_t n = (int64_t)Ttok * per_tok;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / per_tok;
    const int j = (int)(i - t * per_tok);
    const int h = j / v8, c = (j - h * v8) << 3;
    float x[8];
    load8(o + ((int64_t)h * Ttok + t) * v + c, x);
    if (gate) {
      const float g = gate[t * H + h];
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] *= g;
    }
    store8(out + (t * H + h) * (int64_t)v + c, x);
  }
}

}  // namespace

extern "C" {

int dsv_latent_prep(const void* q_src, int ld_q, const void* kv_src, int ld_kv,
                    const void* gate_src, int ld_g, const float* norm_w, const int* tok_pos,
                    const int* tok_row, const float* cosT, const float* sinT, void* pool,
                    void* q_nope, void* q_rot, float* gate, int dt, int Ttok, int H, int dim,
                    int rot, int rank, int rot_dims, float eps, int half_layout, hipStream_t s) {
  if (Ttok <= 0) return 0;
  if (rot_dims < 0 || rot_dims > rot || (rot_dims & 1)) return -1;
  if (rot_dims && (!cosT || !sinT)) return -2;
  if (gate_src && !gate) return -3;
  BY_DTYPE(dt, (latent_prep_k<T><<<Ttok, NT, 0, s>>>(
                   (const T*)q_src, ld_q, (const T*)kv_src, ld_kv, (const T*)gate_src, ld_g,
                   norm_w, tok_pos, tok_row, cosT, sinT, (T*)pool, (T*)q_nope, (T*)q_rot, gate,
                   Ttok, H, dim, rot, rank, rot_dims, eps, half_layout)));
  return (int)hipGetLastError();
}

// LDS bytes the generic attention kernel needs for a chunk of KC keys
int64_t dsv_latent_attn_lds(int dt, int rank, int rot, int KC) {
  const int D = rank + rot;
  return (int64_t)(HG * D + HG * KC + 3 * HG) * 4 + (int64_t)KC * (D | 1) * (dt == 0 ? 4 : 2);
}

int dsv_latent_attn(const void* q_lat, const void* q_rot, const void* pool, const int* tok_seq,
                    const int* tok_pos, const int* table, int maxb, int bs, void* out,
                    float* part, int dt, int Ttok, int H, int rank, int rot, int KC,
                    int nsplit, float scale, int window, const float* sink, hipStream_t s) {
  if (rank > RPT * NT || window < 0) return -1;
  if (Ttok <= 0) return 0;
  const int64_t lds = dsv_latent_attn_lds(dt, rank, rot, KC);
  if (lds > 64 * 1024) return -2;
  dim3 grid(Ttok, nsplit);
  BY_DTYPE(dt, (latent_attn_k<T><<<grid, NT, lds, s>>>(
                   (const T*)q_lat, (const T*)q_rot, (const T*)pool, tok_seq, tok_pos, table,
                   maxb, bs, (T*)out, part, Ttok, H, rank, rot, KC, nsplit, scale, window,
                   sink)));
  if (nsplit > 1) {
    dim3 g2(Ttok, H);
    BY_DTYPE(dt, (latent_attn_merge_k<T><<<g2, NT, 0, s>>>(part, (T*)out, Ttok, H, rank, nsplit,
                                                           sink)));
  }
  return (int)hipGetLastError();
}

// 1 when the MFMA tile kernel covers these sizes (bf16 only)
int dsv_latent_attn_mfma_ok(int rank, int rot) {
  return rank >= 1 && rank <= 512 && rank + rot <= 640;
}

// rows of a sequence's count*H that one workgroup takes
int dsv_latent_attn_mfma_rows(int rank, int rot) {
  return (rank <= 256 && rank + rot <= 320) ? TB_ROWS : TB_ROWS / 2;
}

// work: [nwork][2] = (sequence, first row of a tile of its count*H rows)
int dsv_latent_attn_mfma(const void* q_lat, const void* q_rot, const void* pool, const int* work,
                         int nwork, const int* cu, const int* seq_start, const int* table,
                         int maxb, int bs, void* out, float* part, int Ttok, int H, int rank,
                         int rot, int nsplit, float scale, int window, const float* sink,
                         hipStream_t s) {
  if (!dsv_latent_attn_mfma_ok(rank, rot) || window < 0) return -1;
  if (nsplit < 1 || (nsplit > 1 && !part)) return -3;
  if (nwork <= 0) return 0;
  const int dk = rank + rot;
#define GO(DVB, DKT, SPLIT, PF) \
  return launch_latent_attn_mfma<DVB, DKT, SPLIT, PF>(q_lat, q_rot, pool, work, nwork, cu, seq_start, \
                                           table, maxb, bs, out, part, Ttok, H, rank, rot, \
                                           nsplit, scale, window, sink, s)
  if (rank <= 64 && dk <= 128) GO(2, 8, 1, true);
  if (rank <= 128 && dk <= 192) GO(4, 12, 1, true);
  if (rank <= 256 && dk <= 320) GO(8, 20, 1, true);
  GO(16, 40, 2, false);
#undef GO
}

int dsv_gate_merge(const void* o, const float* gate, void* out, int dt, int Ttok, int H, int v,
                   hipStream_t s) {
  const int64_t n = (int64_t)Ttok * H * v;
  if (n <= 0) return 0;
  if (v % 8 == 0 && (uintptr_t)o % 32 == 0 && (uintptr_t)out % 32 == 0) {
    BY_DTYPE(dt, (gate_merge8_k<T><<<nblocks(n / 8, 256), 256, 0, s>>>((const T*)o, gate, (T*)out,
                                                                       Ttok, H, v)));
    return (int)hipGetLastError();
  }
  BY_DTYPE(dt, (gate_merge_k<T><<<nblocks(n, 256), 256, 0, s>>>((const T*)o, gate, (T*)out, Ttok, H, v)));
  return (int)hipGetLastError();
}

}  // extern "C"
