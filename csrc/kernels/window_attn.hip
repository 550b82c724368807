// Grouped-query attention over a sliding window of a paged key/value cache, optionally with pooled
// blocks: every block of P tokens that lies wholly before the window is seen through one row, the mean
// of its cached keys and the mean of its cached values. Caches (activation dtype):
//   kc [pages][G][page][D], vc [pages][G][page][V]       token rows
//   kp [pages][G][NP][D],   vp [pages][G][NP][V]         pooled rows, NP = ceil(page / P): block b's row
//                                                        lives in the page of its last position e = b P + P - 1,
//                                                        at index (e mod page) / P
// window_write  one workgroup per token: query / key RMS norm (per head or over the whole projection,
//               fp32 statistics), interleaved-pair rotation of the leading rot_dims entries of every head
//               (angle = position * inv_freq in fp32, full-range sin / cos), values optionally turned over
//               all of V, the paged stores, and the prepared query rows.
// window_pool   workgroups of 256 elements per token whose position completes a block: fp32 mean of the block's P
//               cached rows, in position order, into the pooled row. It runs after window_write of the
//               same step, so a block completed inside a prompt portion reads rows of that portion too.
// window_attn   one workgroup per (token, key/value head, chunk of its query heads): the keys a query
//               sees are numbered pooled rows first, then window tokens; tiles of 16 of them are staged in
//               LDS as fp32; scores, running max / sum and the weighted value sum are fp32 FMA. A sink
//               starts the running max at its logit and the running sum at 1. With turned values the
//               normalised output is turned back by the query's position before it is stored.
// window_attn, bf16 caches with head sizes in multiples of 8 up to 256: MFMA kernel. Rows are (token,
//               query head of one key/value head) pairs of one sequence, 16 per workgroup, whose four
//               waves take every fourth key tile and merge through LDS; keys in tiles of 32: first the pooled rows (two groups of 16, each lane
//               addressing its own pooled row), then token tiles aligned to two whole pages.
//                 S = Q K^T   v_mfma 16x16x32, Q fragments stationary, K fragments 16 B of a cached row
//                 online softmax in fp32 (exp2 of log2(e)-scaled scores, per-lane partial row sums)
//                 O += P V    P goes C-layout -> A-layout through a 16 x 32 bf16 tile in LDS; the B operand
//                             needs eight consecutive KEYS of one value column per lane: for token tiles
//                             window_write keeps a second, transposed copy of the values
//                             ([page][G][column][16 keys]) so that is one 16-B load; for the (few) pooled
//                             tiles the eight values are gathered from the pooled rows.
//               Window, causal and pooled-block visibility are per-row masks on whole tiles, and tiles sit
//               at fixed absolute key positions, so a row's sums do not depend on which rows share its wave.
// Distance term (no pooled blocks then): a score may carry a bias that depends on the head and the distance
//               n = i - j alone, -r1[h] ln(1 + r2[h] n) or a table entry tab[h][min(n, last)]; the MFMA kernels
//               compute it in log2 units beside the mask (the table of a workgroup's heads staged in LDS when
//               it fits). An output gate multiplies the normalised result by sigmoid(gate) in the epilogue.
// Softcap c > 0 (not with a distance term): the scaled score s becomes c tanh(s / c) (CAP instantiations of the MFMA
//               kernels). The value caches may have fewer heads (GV) than the key cache: key head g reads value head
//               g / (G / GV), which is how two score maps of one head share their values.
// Every row of every kernel depends only on its own sequence's cache rows, in an order fixed by the
// position, so results do not depend on how a prompt is cut or what else is in the batch.
#include "common.h"
#include "seq_launchers.h"

namespace vgate {
namespace {

__device__ __forceinline__ float ldx(const void* p, int64_t i, int f32) {
  return f32 ? reinterpret_cast<const float*>(p)[i] : bf2f(reinterpret_cast<const bf16_t*>(p)[i]);
}
__device__ __forceinline__ void stx(void* p, int64_t i, int f32, float v) {
  if (f32) reinterpret_cast<float*>(p)[i] = v;
  else reinterpret_cast<bf16_t*>(p)[i] = f2bf(v);
}

__device__ __forceinline__ int seq_of_token(const int32_t* query_start, int S, int t) {
  int lo = 0, hi = S - 1;  // query_start[s] <= t < query_start[s + 1]
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (query_start[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

__global__ __launch_bounds__(256) void window_write_kernel(WindowArgs a, const void* __restrict__ q, int64_t ldq,
                                                            const void* __restrict__ k, int64_t ldk,
                                                            const void* __restrict__ v, int64_t ldv,
                                                            const float* __restrict__ qw, const float* __restrict__ kw,
                                                            float eps, int norm_all, void* __restrict__ q_out,
                                                            bf16_t* __restrict__ vt, const float* __restrict__ q_head_scale,
                                                            float q_temp_coef, int q_temp_every, int rot_half) {
  extern __shared__ float lds[];
  const int H = a.H, G = a.G, D = a.D, V = a.V, GV = a.GV;
  float* xs = lds;                    // [(H + G) * D] q heads then k heads
  float* inv = xs + (H + G) * D;      // [H + G]
  const int t = blockIdx.x;
  const int slot = a.slots[t];
  if (slot < 0) return;  // padding row (uniform per block)
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
  for (int e = tid; e < H * D; e += 256) xs[e] = ldx(q, (int64_t)t * ldq + e, a.f32);
  for (int e = tid; e < G * D; e += 256) xs[H * D + e] = ldx(k, (int64_t)t * ldk + e, a.f32);
  __syncthreads();
  for (int h = wv; h < H + G; h += 4) {  // sum of squares per head
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) ss = fmaf(xs[h * D + d], xs[h * D + d], ss);
    ss = wave_reduce_sum(ss);
    if (lane == 0) inv[h] = ss;
  }
  __syncthreads();
  if (qw != nullptr) {
    float mine = 0.f;
    if (norm_all) {
      float sq = 0.f, sk = 0.f;
      for (int h = 0; h < H; ++h) sq += inv[h];
      for (int h = 0; h < G; ++h) sk += inv[H + h];
      if (tid < H + G) mine = 1.f / sqrtf((tid < H ? sq / (float)(H * D) : sk / (float)(G * D)) + eps);
    } else if (tid < H + G) {
      mine = 1.f / sqrtf(inv[tid] / (float)D + eps);
    }
    __syncthreads();
    if (tid < H + G) inv[tid] = mine;
    __syncthreads();
  }
  const float pos = (float)a.positions[t];
  // query temperature of the position: 1 + coef ln(floor((p + 1) / every) + 1)
  const float qgrow = q_temp_coef != 0.f ? 1.f + q_temp_coef * logf((float)((a.positions[t] + 1) / q_temp_every) + 1.f) : 1.f;
  const int page = a.page;
  const int64_t pg = slot / page, off = slot % page;
  for (int e = tid; e < (H + G) * D; e += 256) {
    const int h = e / D, i = e % D;
    const bool isq = h < H;
    const float* w = isq ? qw : kw;
    const int wo = norm_all ? (isq ? h : h - H) * D : 0;
    const float sc = w != nullptr ? inv[h] : 1.f;
    float o;
    if (i < a.rot_dims) {  // the pair (i0, i1) = (2j, 2j + 1), or (j, j + rot_dims / 2) with rot_half
      const int hr = a.rot_dims >> 1;
      const int j = rot_half ? (i < hr ? i : i - hr) : (i >> 1);
      const int i0 = rot_half ? j : (i & ~1), i1 = rot_half ? j + hr : (i | 1);
      const float x0 = xs[h * D + i0] * sc * (w ? w[wo + i0] : 1.f), x1 = xs[h * D + i1] * sc * (w ? w[wo + i1] : 1.f);
      const float ang = pos * a.inv_freq[j];
      const float cs = cosf(ang), sn = sinf(ang);
      o = (i == i1) ? (x1 * cs + x0 * sn) : (x0 * cs - x1 * sn);
    } else {
      o = xs[h * D + i] * sc * (w ? w[wo + i] : 1.f);
    }
    if (isq) stx(q_out, (int64_t)t * H * D + e, a.f32, o * (q_head_scale != nullptr ? q_head_scale[h] * qgrow : qgrow));
    else stx(a.kc, ((pg * G + (h - H)) * page + off) * D + i, a.f32, o);
  }
  const int vrot = a.v_freq != nullptr ? 2 * (V / 2) : 0;
  for (int e = tid; e < GV * V; e += 256) {
    const int g = e / V, i = e % V;
    float o;
    if (i < vrot) {
      const float x0 = ldx(v, (int64_t)t * ldv + g * V + (i & ~1), a.f32), x1 = ldx(v, (int64_t)t * ldv + g * V + (i | 1), a.f32);
      const float ang = pos * a.v_freq[i >> 1];
      const float cs = cosf(ang), sn = sinf(ang);
      o = (i & 1) ? (x1 * cs + x0 * sn) : (x0 * cs - x1 * sn);
    } else {
      o = ldx(v, (int64_t)t * ldv + e, a.f32);
    }
    stx(a.vc, ((pg * GV + g) * page + off) * V + i, a.f32, o);
    if (vt != nullptr) vt[((pg * GV + g) * V + i) * page + off] = f2bf(o);  // [page][GV][column][key in page]
  }
}

template <typename T>
__device__ __forceinline__ float ld_as_float(const T* p, int64_t i);
template <>
__device__ __forceinline__ float ld_as_float<float>(const float* p, int64_t i) { return p[i]; }
template <>
__device__ __forceinline__ float ld_as_float<bf16_t>(const bf16_t* p, int64_t i) { return bf2f(p[i]); }

template <typename T>
__global__ __launch_bounds__(256) void window_pool_kernel(WindowArgs a) {
  __shared__ int32_t pages[64];  // the pages of the block's rows, a stretch of up to 64 at a time
  const int t = blockIdx.x;
  if (t >= a.query_start[a.S]) return;
  const int e = a.positions[t], P = a.pool;
  if ((e + 1) % P != 0) return;  // uniform per block
  const int s = seq_of_token(a.query_start, a.S, t);
  const int32_t* bt = a.block_tables + (int64_t)s * a.max_blocks;
  const int G = a.G, D = a.D, V = a.V, page = a.page;
  const int64_t dpg = bt[e / page];
  const int drow = (e % page) / P;
  const int j0 = e + 1 - P, pg_first = j0 / page, npg = e / page - pg_first + 1;
  const int nx = G * (D + V);
  // every thread sums one element over the block's rows in position order; the page ids come from LDS, so a
  // row's loads do not wait for a block-table load and sixteen rows are in flight (the rows were written by
  // the launch before, mostly on other XCDs: each batch costs a trip past the L2)
  {  // blockIdx.y: which 256 elements
    const int x = blockIdx.y * blockDim.x + threadIdx.x;
    const bool on = x < nx;
    const bool isk = x < G * D;
    const int y = isk ? x : x - G * D;
    const int w = isk ? D : V;
    const int g = on ? y / w : 0, i = on ? y % w : 0;
    const T* src = reinterpret_cast<const T*>(isk ? a.kc : a.vc);
    float sum = 0.f;
    for (int pb = 0; pb < npg; pb += 64) {
      __syncthreads();
      if ((int)threadIdx.x < min(64, npg - pb)) pages[threadIdx.x] = bt[pg_first + pb + threadIdx.x];
      __syncthreads();
      const int ja = max(j0, (pg_first + pb) * page), jb = min(e, (pg_first + min(npg, pb + 64)) * page - 1);
      if (on) {
        for (int j = ja; j <= jb; j += 16) {  // sixteen rows' loads in flight, added in position order
          float v[16];
#pragma unroll
          for (int u = 0; u < 16; ++u) {
            const int jj = min(j + u, jb);
            v[u] = ld_as_float<T>(src, (((int64_t)pages[jj / page - pg_first - pb] * G + g) * page + jj % page) * w + i);
          }
#pragma unroll
          for (int u = 0; u < 16; ++u)
            if (j + u <= jb) sum += v[u];
        }
      }
    }
    if (on) stx(isk ? a.kp : a.vp, ((dpg * G + g) * a.npool + drow) * w + i, a.f32, sum / (float)P);
  }
}

constexpr int KT = 16;      // keys per tile
constexpr int MAXACC = 8;   // outputs per thread: heads-per-block * V <= 256 * MAXACC

__global__ __launch_bounds__(256) void window_attn_kernel(WindowArgs a, const void* __restrict__ q, int HC, float scale,
                                                           void* __restrict__ out) {
  extern __shared__ float lds[];
  const int D = a.D, V = a.V, DP = D + 1, VP = V + 1, G = a.G, page = a.page;
  float* qs = lds;                  // [HC][DP]
  float* ks = qs + HC * DP;         // [KT][DP]
  float* vs = ks + KT * DP;         // [KT][VP]
  float* sc = vs + KT * VP;         // [HC][KT] scores, then weights
  float* mrun = sc + HC * KT;       // [HC]
  float* lrun = mrun + HC;          // [HC]
  float* alpha = lrun + HC;         // [HC]
  float* os = alpha + HC;           // [HC][V] normalised outputs (for the turn back)
  const int t = blockIdx.x;
  if (t >= a.query_start[a.S]) return;
  const int s = seq_of_token(a.query_start, a.S, t);
  const int pos = a.context_lens[s] - (a.query_start[s + 1] - t);  // position of token t
  const int g = blockIdx.y;
  const int gv = g / (G / a.GV);           // the value head of key head g
  const int rep = a.H / G;
  const int r0 = blockIdx.z * HC;          // first query head of the group handled here
  const int nh = min(HC, rep - r0);
  const int h0 = g * rep + r0;
  const int tid = threadIdx.x;
  const int lo = max(0, pos - a.window + 1);
  const int nb = a.pool > 0 ? max(0, pos - a.window + 1) / a.pool : 0;  // pooled blocks wholly before the window
  const int nkeys = nb + (pos - lo + 1);
  for (int e = tid; e < nh * D; e += 256) qs[(e / D) * DP + e % D] = ldx(q, ((int64_t)t * a.H + h0) * D + e, a.f32);
  if (tid < HC) {
    const bool sk = a.sink != nullptr && tid < nh;
    mrun[tid] = sk ? a.sink[h0 + tid] : -INFINITY;
    lrun[tid] = sk ? 1.f : 0.f;
    alpha[tid] = 1.f;
  }
  float acc[MAXACC];
#pragma unroll
  for (int i = 0; i < MAXACC; ++i) acc[i] = 0.f;
  const int32_t* bt = a.block_tables + (int64_t)s * a.max_blocks;
  for (int j0 = 0; j0 < nkeys; j0 += KT) {
    __syncthreads();  // previous tile fully consumed (and q / running stats written)
    for (int e = tid; e < KT * (D + V); e += 256) {
      const int jj = e / (D + V), c = e % (D + V);
      const int kj = j0 + jj;
      float val = 0.f;
      if (kj < nkeys) {
        const bool isk = c < D;
        const int ci = isk ? c : c - D, w = isk ? D : V;
        if (kj < nb) {   // pooled row of block kj
          const int e1 = kj * a.pool + a.pool - 1;
          const int64_t row = ((int64_t)bt[e1 / page] * G + g) * a.npool + (e1 % page) / a.pool;
          val = ldx(isk ? a.kp : a.vp, row * w + ci, a.f32);
        } else {
          const int j = lo + kj - nb;
          const int64_t row = isk ? ((int64_t)bt[j / page] * G + g) * page + j % page
                                  : ((int64_t)bt[j / page] * a.GV + gv) * page + j % page;
          val = ldx(isk ? a.kc : a.vc, row * w + ci, a.f32);
        }
      }
      if (c < D) ks[jj * DP + c] = val; else vs[jj * VP + c - D] = val;
    }
    __syncthreads();
    {  // scores: two threads per (head, key), each half of the dot product
      const int wi = tid >> 1, half = tid & 1;
      float d = 0.f;
      const bool on = wi < nh * KT;
      const int h = on ? wi / KT : 0, jj = on ? wi % KT : 0;
      if (on) {
        const int c0 = half ? (D >> 1) : 0, c1 = half ? D : (D >> 1);
        const float* qp = qs + h * DP;
        const float* kp = ks + jj * DP;
        for (int c = c0; c < c1; ++c) d = fmaf(qp[c], kp[c], d);
      }
      d += __shfl_xor(d, 1, 64);
      float bias = 0.f;
      if (a.bias_kind != 0 && on && j0 + jj >= nb && j0 + jj < nkeys) {  // (token keys: kj - nb keys after lo)
        const int n = pos - (lo + j0 + jj - nb);
        bias = a.bias_kind == 1 ? -a.bias_a[h0 + h] * logf(1.f + a.bias_b[h0 + h] * (float)n)
                                : a.bias_a[(int64_t)(h0 + h) * a.bias_n + min(n, a.bias_n - 1)];
      }
      float sv = d * scale;
      if (a.softcap > 0.f) sv = a.softcap * tanhf(sv / a.softcap);
      if (on && half == 0) sc[h * KT + jj] = (j0 + jj < nkeys) ? sv + bias : -INFINITY;
    }
    __syncthreads();
    if (tid < nh) {
      const float m0 = mrun[tid];
      float m1 = m0;
      for (int jj = 0; jj < KT; ++jj) m1 = fmaxf(m1, sc[tid * KT + jj]);
      const float al = expf(m0 - m1);  // m0 = -inf on the first tile: 0
      float l = 0.f;  // the tile's own sum first: the running sum takes one rounding per tile, not per key
      for (int jj = 0; jj < KT; ++jj) {
        const float pj = expf(sc[tid * KT + jj] - m1);
        sc[tid * KT + jj] = pj;
        l += pj;
      }
      mrun[tid] = m1; lrun[tid] = fmaf(lrun[tid], al, l); alpha[tid] = al;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MAXACC; ++i) {
      const int o = tid + i * 256;
      if (o < nh * V) {
        const int h = o / V, c = o % V;
        float x = 0.f;
        const float* pp = sc + h * KT;
#pragma unroll
        for (int jj = 0; jj < KT; ++jj) x = fmaf(pp[jj], vs[jj * VP + c], x);
        acc[i] = fmaf(acc[i], alpha[h], x);
      }
    }
  }
  __syncthreads();
  auto gated = [&](int o, float y) {  // o: (head - h0) * V + column
    return a.gate != nullptr ? y / (1.f + expf(-ldx(a.gate, (int64_t)t * a.ldg + (int64_t)h0 * V + o, a.f32))) : y;
  };
  if (a.v_freq == nullptr) {
#pragma unroll
    for (int i = 0; i < MAXACC; ++i) {
      const int o = tid + i * 256;
      if (o < nh * V) stx(out, ((int64_t)t * a.H + h0) * V + o, a.f32, gated(o, acc[i] / lrun[o / V]));
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < MAXACC; ++i) {
    const int o = tid + i * 256;
    if (o < nh * V) os[o] = acc[i] / lrun[o / V];
  }
  __syncthreads();
  const int vrot = 2 * (V / 2);
  const float fp = -(float)pos;
  for (int o = tid; o < nh * V; o += 256) {
    const int h = o / V, i = o % V;
    float y = os[o];
    if (i < vrot) {
      const float x0 = os[h * V + (i & ~1)], x1 = os[h * V + (i | 1)];
      const float ang = fp * a.v_freq[i >> 1];
      const float cs = cosf(ang), sn = sinf(ang);
      y = (i & 1) ? (x1 * cs + x0 * sn) : (x0 * cs - x1 * sn);
    }
    stx(out, ((int64_t)t * a.H + h0) * V + o, a.f32, gated(o, y));
  }
}


// ---------------------------------------------------------------------------------- MFMA (bf16)
__device__ __forceinline__ bf16x8 frag16(const bf16_t* rowp, int k, int K, bool valid) {
  uint4 v = make_uint4(0, 0, 0, 0);
  if (valid && k < K) {
    const bf16_t* q = rowp + k;
    if (k + 8 <= K && (reinterpret_cast<uintptr_t>(q) & 15) == 0) {
      v = ld16(q);
    } else {
      uint32_t w[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = (k + 2 * j < K) ? q[2 * j] : 0;
        const uint32_t hi = (k + 2 * j + 1 < K) ? q[2 * j + 1] : 0;
        w[j] = lo | (hi << 16);
      }
      v = make_uint4(w[0], w[1], w[2], w[3]);
    }
  }
  return as_bf16x8(v);
}

// reductions over the 16 lanes that share l >> 4: rotations by 8, 4, 2, 1 inside the DPP row (VALU, no LDS)
template <int CTRL>
__device__ __forceinline__ float row_rot(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float group16_max(float v) {
  v = fmaxf(v, row_rot<0x128>(v)); v = fmaxf(v, row_rot<0x124>(v));
  v = fmaxf(v, row_rot<0x122>(v)); v = fmaxf(v, row_rot<0x121>(v));
  return v;
}
__device__ __forceinline__ float group16_sum(float v) {
  v += row_rot<0x128>(v); v += row_rot<0x124>(v); v += row_rot<0x122>(v); v += row_rot<0x121>(v);
  return v;
}

// Distance term of the MFMA kernels, in log2 units. Per C-layout row of a lane: bw / bx are (r1, r2) of the
// row's head for the logarithmic penalty; bo is the row's offset into the table of the workgroup's heads.
constexpr float LOG2E = 1.4426950408889634f;
__device__ __forceinline__ void bias_stage(const WindowArgs& a, float* btab, int g, int rep, int tid, int nthreads) {
  if (a.bias_kind == 2 && a.bias_lds)
    for (int e = tid; e < rep * a.bias_n; e += nthreads) btab[e] = a.bias_a[(int64_t)g * rep * a.bias_n + e] * LOG2E;
}
__device__ __forceinline__ void bias_row(const WindowArgs& a, int g, int rep, int r, bool ok, float& bw, float& bx, int& bo) {
  const int hr = ok ? r % rep : 0;
  bw = bx = 0.f;
  bo = hr * a.bias_n;
  if (a.bias_kind == 1) { bw = a.bias_a[g * rep + hr]; bx = a.bias_b[g * rep + hr]; }
}
__device__ __forceinline__ float bias_of(const WindowArgs& a, const float* btab, int g, int rep, float bw, float bx, int bo,
                                         int n) {
  n = max(n, 0);  // (a key the row does not see: masked by the caller)
  if (a.bias_kind == 1) return -bw * __log2f(fmaf(bx, (float)n, 1.f));
  const int idx = bo + min(n, a.bias_n - 1);
  return a.bias_lds ? btab[idx] : a.bias_a[(int64_t)g * rep * a.bias_n + idx] * LOG2E;
}
// the terms of a lane's 4 x 2 scores of one tile (keys c0 and c0 + 16), asked for together, before the softmax's
// arithmetic, and whether the key is visible or not (a negative distance reads entry 0). all_far (wave-uniform):
// every key of the tile is at least the table's last distance away from every row of the wave.
__device__ __forceinline__ void bias_tile(const WindowArgs& a, const float* btab, int g, int rep, const float* bw,
                                          const float* bx, const int* bo, const float* bfar, const int* hi, int c0,
                                          bool all_far, float* bt0, float* bt1) {
  if (a.bias_kind == 2 && all_far) {
#pragma unroll
    for (int i = 0; i < 4; ++i) bt0[i] = bt1[i] = bfar[i];
    return;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    bt0[i] = bias_of(a, btab, g, rep, bw[i], bx[i], bo[i], hi[i] - c0);
    bt1[i] = bias_of(a, btab, g, rep, bw[i], bx[i], bo[i], hi[i] - c0 - 16);
  }
}
__device__ __forceinline__ float gate_of(const bf16_t* grow, int col) { return 1.f / (1.f + __expf(-bf2f(grow[col]))); }

// NCT: 16-column tiles of the value (V <= 16 NCT); NQF: 32-wide fragments of a query row (D <= 32 NQF).
// D % 8 == 0 (host-checked): every key fragment is one unconditional 16-B load; a fragment past the row's
// end or the value's last column is read from a clamped address: its partner (zero Q fragment) or its
// output column (never stored) makes the value irrelevant, and cached values are always finite.
constexpr int LG = 4;
// NW: waves of a workgroup, which share out the key tiles of its 16 rows
// the score of one key in log2 units: the scaled score, softcapped (CAP) or with its distance term (BIAS) added
template <bool CAP>
__device__ __forceinline__ float score_log2(const WindowArgs& a, float s, float scale_log2e, float bias) {
  if (!CAP) return fmaf(s, scale_log2e, bias);
  // cap tanh(x / cap) log2e with x / cap = s scale / cap; tanh(y) = 1 - 2 / (e^(2y) + 1), exact at both ends
  const float e = exp2f(s * scale_log2e * a.cap_in);   // cap_in = 2 / cap
  return a.cap_out * (1.f - 2.f / (e + 1.f));          // cap_out = cap log2e
}

template <int NCT, int NQF, int NW, int BIAS, bool CAP>
__global__ __launch_bounds__(64 * NW) void window_attn_mfma_kernel(WindowArgs a, const bf16_t* __restrict__ q,
                                                                float scale_log2e, const bf16_t* __restrict__ vt,
                                                                int num_pages, bf16_t* __restrict__ out) {
  extern __shared__ float btab[];  // BIAS: the distance table of this workgroup's heads (when it is staged)
  __shared__ __attribute__((aligned(16))) bf16_t pl[NW][16][40];
  __shared__ float mrg_m[NW][16], mrg_l[NW][16];
  __shared__ float mrg_o[16][16 * NCT];  // the merged weighted values of the 16 rows
  const int D = a.D, V = a.V, G = a.G, H = a.H, rep = H / G, g = blockIdx.y, P = a.pool;
  const int GV = a.GV, gv = g / (G / GV);  // value heads; the value head of key head g
  int s = -1, tile = 0, base = 0;
  for (int i = 0; i < a.S; ++i) {  // (sequence, 16-row tile) of this workgroup
    const int nt = ((a.query_start[i + 1] - a.query_start[i]) * rep + 15) / 16;
    if ((int)blockIdx.x < base + nt) { s = i; tile = blockIdx.x - base; break; }
    base += nt;
  }
  if (s < 0) return;
  const int wv = threadIdx.x >> 6, l = threadIdx.x & 63, lr = l & 15, lg = l >> 4;
  const int t0 = a.query_start[s], ntok = a.query_start[s + 1] - t0;
  const int pos0 = a.context_lens[s] - ntok;
  const int nrows = ntok * rep;
  // a workgroup owns 16 rows; its four waves take every fourth key tile of them and merge their partial
  // (max, sum, weighted values) through LDS: four times the waves to hide the cache's latency behind
  const int row0 = tile * 16;
  if (row0 >= nrows) return;  // (workgroup-uniform)
  if (BIAS) {
    bias_stage(a, btab, g, rep, threadIdx.x, 64 * NW);
    __syncthreads();
  }
  const bf16_t* kc = reinterpret_cast<const bf16_t*>(a.kc);
  const bf16_t* kp = reinterpret_cast<const bf16_t*>(a.kp);
  const bf16_t* vp = reinterpret_cast<const bf16_t*>(a.vp);
  const int nqf = (D + 31) >> 5, nct = (V + 15) >> 4;
  bf16x8 qf[NQF];  // stationary Q fragments: A operand, lane holds Q[row lr][32 kk + 8 lg ..]
  {
    const int r = row0 + lr;
    const bool ok = r < nrows;
    const bf16_t* qrow = q + ((int64_t)(t0 + (ok ? r / rep : 0)) * H + g * rep + (ok ? r % rep : 0)) * D;
#pragma unroll
    for (int kk = 0; kk < NQF; ++kk) qf[kk] = frag16(qrow, 32 * kk + 8 * lg, D, ok && kk < nqf);
  }
  // C-layout rows of this lane: row0 + 4 lg + i; what each sees: tokens [lo, hi], pooled blocks [0, nbv)
  int hi[4], lo[4], nbv[4];
  float m[4], lsum[4];
  float bw[BIAS ? 4 : 1], bx[BIAS ? 4 : 1], bfar[BIAS ? 4 : 1];
  int bo[BIAS ? 4 : 1];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + 4 * lg + i;
    const bool ok = r < nrows;
    const int p = pos0 + (ok ? r / rep : 0);
    hi[i] = ok ? p : -1;
    lo[i] = p - a.window + 1;
    nbv[i] = (ok && P > 0) ? max(0, lo[i]) / P : 0;
    if (BIAS) {
      bias_row(a, g, rep, r, ok, bw[i], bx[i], bo[i]);
      bfar[i] = a.bias_kind == 2 ? bias_of(a, btab, g, rep, 0.f, 0.f, bo[i], a.bias_n - 1) : 0.f;
    }
    const bool sk = ok && a.sink != nullptr && wv == 0 && blockIdx.z == 0;  // the sink counts once
    m[i] = sk ? a.sink[g * rep + r % rep] * 1.4426950408889634f : -INFINITY;
    lsum[i] = (sk && lr == 0) ? 1.f : 0.f;
  }
  const int last = min(row0 + 15, nrows - 1);
  const int pmin = pos0 + row0 / rep, pmax = pos0 + last / rep;  // wave-uniform
  const int klo = max(0, pmin - a.window + 1);
  const int nbmax = P > 0 ? max(0, pmax - a.window + 1) / P : 0;
  const int ntp = (nbmax + 31) >> 5, jt0 = klo >> 5;
  const int ntiles = ntp + (pmax >> 5) - jt0 + 1;
  f32x4 O[NCT];
#pragma unroll
  for (int ct = 0; ct < NCT; ++ct) O[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int32_t* bt = a.block_tables + (int64_t)s * a.max_blocks;
  // a.parts > 1 (decoded tokens of long contexts): blockIdx.z is one of several workgroups that share the key tiles
  // of these 16 rows; each leaves its merged (max, sum, weighted values) in scratch for window_attn_merge_kernel
  const int nparts = a.parts > 1 ? a.parts : 1;
  for (int ti = blockIdx.z * NW + wv; ti < ntiles; ti += NW * nparts) {
    const bool pooled = ti < ntp;  // wave-uniform
    int kbase, pg0 = 0, pg1 = 0;
    const bf16_t* k0p;
    const bf16_t* k1p;
    if (pooled) {
      kbase = 32 * ti;
      const int e0 = min(kbase + lr, nbmax - 1) * P + P - 1, e1 = min(kbase + 16 + lr, nbmax - 1) * P + P - 1;
      const int q0 = min(max(bt[e0 >> 4], 0), num_pages - 1), q1 = min(max(bt[e1 >> 4], 0), num_pages - 1);
      k0p = kp + (((int64_t)q0 * G + g) * a.npool + (e0 & 15) / P) * D;
      k1p = kp + (((int64_t)q1 * G + g) * a.npool + (e1 & 15) / P) * D;
    } else {
      kbase = 32 * (jt0 + ti - ntp);
      pg0 = bt[kbase >> 4];
      pg1 = (kbase + 16 <= pmax) ? bt[(kbase >> 4) + 1] : pg0;
      pg0 = min(max(pg0, 0), num_pages - 1);
      pg1 = min(max(pg1, 0), num_pages - 1);
      k0p = kc + (((int64_t)pg0 * G + g) * 16 + lr) * D;
      k1p = kc + (((int64_t)pg1 * G + g) * 16 + lr) * D;
    }
    f32x4 s0 = f32x4{0.f, 0.f, 0.f, 0.f}, s1 = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k0 = 0; k0 < NQF; k0 += LG) {
      if (k0 < nqf) {  // wave-uniform
        uint4 b0[LG], b1[LG];
#pragma unroll
        for (int u = 0; u < LG; ++u) {
          const int off = min(32 * (k0 + u) + 8 * lg, D - 8);
          b0[u] = ld16(k0p + off);
          b1[u] = ld16(k1p + off);
        }
#pragma unroll
        for (int u = 0; u < LG; ++u)
          if (k0 + u < NQF) {
            s0 = mfma16(qf[k0 + u], as_bf16x8(b0[u]), s0);
            s1 = mfma16(qf[k0 + u], as_bf16x8(b1[u]), s1);
          }
      }
    }
    float al[4];
    const int c0 = kbase + lr, c1 = kbase + 16 + lr;
    float bt0[BIAS ? 4 : 1], bt1[BIAS ? 4 : 1];
    if (BIAS) bias_tile(a, btab, g, rep, bw, bx, bo, bfar, hi, c0, kbase + 31 <= pmin - (a.bias_n - 1), bt0, bt1);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool vis0 = pooled ? c0 < nbv[i] : (c0 >= lo[i] && c0 <= hi[i]);
      const bool vis1 = pooled ? c1 < nbv[i] : (c1 >= lo[i] && c1 <= hi[i]);
      const float v0 = vis0 ? score_log2<CAP>(a, s0[i], scale_log2e, BIAS ? bt0[i] : 0.f) : -INFINITY;
      const float v1 = vis1 ? score_log2<CAP>(a, s1[i], scale_log2e, BIAS ? bt1[i] : 0.f) : -INFINITY;
      const float mnew = fmaxf(m[i], group16_max(fmaxf(v0, v1)));
      const float ms = (mnew == -INFINITY) ? 0.f : mnew;  // a row that has seen no key yet
      al[i] = exp2f(m[i] - ms);
      const float p0 = exp2f(v0 - ms), p1 = exp2f(v1 - ms);
      lsum[i] = lsum[i] * al[i] + p0 + p1;
      m[i] = mnew;
      pl[wv][4 * lg + i][lr] = f2bf(p0);
      pl[wv][4 * lg + i][16 + lr] = f2bf(p1);
    }
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
      for (int i = 0; i < 4; ++i) O[ct][i] *= al[i];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wave's P tile is written (LDS is in order per wave)
    const bf16x8 pf = as_bf16x8(*reinterpret_cast<const uint4*>(&pl[wv][lr][8 * lg]));
    if (!pooled) {
      const int pgs = (lg >> 1) ? pg1 : pg0;
      const bf16_t* tp = vt + ((int64_t)pgs * GV + gv) * V * 16 + 8 * (lg & 1);
#pragma unroll
      for (int cb = 0; cb < NCT; cb += 2 * LG) {
        if (cb < nct) {  // wave-uniform
          uint4 b[2 * LG];
#pragma unroll
          for (int u = 0; u < 2 * LG; ++u) b[u] = ld16(tp + (int64_t)min(16 * (cb + u) + lr, V - 1) * 16);
#pragma unroll
          for (int u = 0; u < 2 * LG; ++u)
            if (cb + u < NCT) O[cb + u] = mfma16(pf, as_bf16x8(b[u]), O[cb + u]);
        }
      }
    } else {
      // eight pooled rows per lane (keys kbase + 8 lg ..), one value column of each 16-column tile
      int64_t ro[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int e1 = min(kbase + 8 * lg + e, nbmax - 1) * P + P - 1;
        const int pq = min(max(bt[e1 >> 4], 0), num_pages - 1);
        ro[e] = (((int64_t)pq * G + g) * a.npool + (e1 & 15) / P) * V;
      }
#pragma unroll
      for (int ct = 0; ct < NCT; ++ct) {
        if (ct < nct) {  // wave-uniform
          const int col = min(16 * ct + lr, V - 1);
          uint32_t w[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) w[j] = (uint32_t)vp[ro[2 * j] + col] | ((uint32_t)vp[ro[2 * j + 1] + col] << 16);
          O[ct] = mfma16(pf, as_bf16x8(make_uint4(w[0], w[1], w[2], w[3])), O[ct]);
        }
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // P tile read before the next tile overwrites it
  }
  {  // merge the waves' partials of every row
    float f[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float tot = group16_sum(lsum[i]);
      if (lr == 0) { mrg_m[wv][4 * lg + i] = m[i]; mrg_l[wv][4 * lg + i] = tot; }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 4 * lg + i;
      float M = mrg_m[0][r];
#pragma unroll
      for (int w = 1; w < NW; ++w) M = fmaxf(M, mrg_m[w][r]);
      const float Ms = (M == -INFINITY) ? 0.f : M;  // (rows past the sequence's last)
      float L = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) L += mrg_l[w][r] * exp2f(mrg_m[w][r] - Ms);  // a wave that saw no key: l = 0, exp2(-inf) = 0
      f[i] = exp2f(m[i] - Ms);
      lsum[i] = L;                // the merged row sum (the same in every lane of the row)
      m[i] = M;
    }
    for (int w = 0; w < NW; ++w) {  // waves add their scaled partials in turn
      if (wv == w) {
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float* dst = &mrg_o[4 * lg + i][16 * ct + lr];
            const float v = O[ct][i] * f[i];
            *dst = (w == 0) ? v : *dst + v;
          }
      }
      __syncthreads();
    }
  }
  // eight waves (decoded tokens) share the epilogue out: wave w finishes the column tiles ct = w, w + NW, ..;
  // with four (prompt portions) wave 0 finishes all of them: the shared form costs four registers there, which
  // is the step from four waves per SIMD to three (measured 167 us against 109 us)
  if (a.parts > 1) {  // (workgroup-uniform) hand the partial result on: the merge kernel finishes the rows
    const int64_t slot = ((int64_t)blockIdx.z * G + g) * gridDim.x + blockIdx.x;
    float* po = a.part_o + slot * (16 * 16 * NCT);
    for (int e = threadIdx.x; e < 16 * 16 * NCT; e += 64 * NW) po[e] = (&mrg_o[0][0])[e];
    if (wv == 0 && lr == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a.part_ml[(slot * 16 + 4 * lg + i) * 2] = m[i];
        a.part_ml[(slot * 16 + 4 * lg + i) * 2 + 1] = lsum[i];
      }
    }
    return;
  }
  constexpr bool SHARE = NW > 4;
  if (!SHARE && wv != 0) return;
  const int vrot = a.v_freq != nullptr ? 2 * (V / 2) : 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float inv = 1.f / lsum[i];
    const int r = row0 + 4 * lg + i;
    const bool ok = r < nrows;
    const float fp = -(float)(pos0 + (ok ? r / rep : 0));
    bf16_t* orow = out + ((int64_t)(t0 + (ok ? r / rep : 0)) * H + g * rep + (ok ? r % rep : 0)) * V;
    const bf16_t* grow = a.gate == nullptr ? nullptr : reinterpret_cast<const bf16_t*>(a.gate) +
        (int64_t)(t0 + (ok ? r / rep : 0)) * a.ldg + (int64_t)(g * rep + (ok ? r % rep : 0)) * V;
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) {
      if (SHARE && ct % NW != wv) continue;  // wave-uniform
      const int col = 16 * ct + lr;
      float y = mrg_o[4 * lg + i][col] * inv;
      if (vrot > 0) {  // turn the pair (even column, the next one) back by the row's position: the partner is lane l ^ 1
        const float other = __shfl_xor(y, 1, 64);
        if (col < vrot) {
          const float ang = fp * a.v_freq[col >> 1];
          const float cs = cosf(ang), sn = sinf(ang);
          y = (col & 1) ? (y * cs + other * sn) : (y * cs - other * sn);
        }
      }
      if (ok && ct < nct && col < V) orow[col] = f2bf(grow != nullptr ? y * gate_of(grow, col) : y);
    }
  }
}

// The rows of one 16-row tile from the partial results of a.parts workgroups: M = max of the parts' maxima (log2
// units), sums and weighted values rescaled by 2^(M_p - M) and added in part order, then the epilogue of the kernel
// above (normalise, turn back, gate, store). vs: the row stride of the parts' weighted values.
__global__ __launch_bounds__(256) void window_attn_merge_kernel(WindowArgs a, int vs, bf16_t* __restrict__ out) {
  const int V = a.V, G = a.G, H = a.H, rep = H / G, g = blockIdx.y;
  int s = -1, tile = 0, base = 0;
  for (int i = 0; i < a.S; ++i) {
    const int nt = ((a.query_start[i + 1] - a.query_start[i]) * rep + 15) / 16;
    if ((int)blockIdx.x < base + nt) { s = i; tile = blockIdx.x - base; break; }
    base += nt;
  }
  if (s < 0) return;
  const int t0 = a.query_start[s], ntok = a.query_start[s + 1] - t0;
  const int pos0 = a.context_lens[s] - ntok, nrows = ntok * rep;
  const int vrot = a.v_freq != nullptr ? 2 * (V / 2) : 0;
  // blockIdx.z: which four rows of the tile
  for (int e = threadIdx.x; e < 4 * V; e += blockDim.x) {
    const int rr = 4 * blockIdx.z + e / V, col = e % V, r = tile * 16 + rr;
    if (r >= nrows) continue;
    constexpr int MAXP = 8;  // (window_attn_parts() gives at most eight)
    float pm[MAXP], pl[MAXP], po[MAXP], M = -INFINITY;
#pragma unroll
    for (int p = 0; p < MAXP; ++p) {  // all parts' loads asked for together
      const int64_t slot = ((int64_t)min(p, a.parts - 1) * G + g) * gridDim.x + blockIdx.x;
      pm[p] = p < a.parts ? a.part_ml[(slot * 16 + rr) * 2] : -INFINITY;
      pl[p] = a.part_ml[(slot * 16 + rr) * 2 + 1];
      po[p] = a.part_o[slot * (16 * vs) + rr * vs + col];
      M = fmaxf(M, pm[p]);
    }
    float L = 0.f, y = 0.f, yo = 0.f;  // yo: the pair's other column (turned values)
    const int colo = col ^ 1;
#pragma unroll
    for (int p = 0; p < MAXP; ++p) {
      const float f = exp2f(pm[p] - M);  // a part that saw no key (or is none): max -inf, factor 0
      L = fmaf(pl[p], f, L);
      y = fmaf(po[p], f, y);
      if (col < vrot && p < a.parts) {
        const int64_t slot = ((int64_t)p * G + g) * gridDim.x + blockIdx.x;
        yo = fmaf(a.part_o[slot * (16 * vs) + rr * vs + colo], f, yo);
      }
    }
    const float inv = 1.f / L;
    y *= inv;
    if (col < vrot) {
      const float ang = -(float)(pos0 + r / rep) * a.v_freq[col >> 1];
      const float cs = cosf(ang), sn = sinf(ang);
      yo *= inv;
      y = (col & 1) ? (y * cs + yo * sn) : (y * cs - yo * sn);
    }
    const int64_t t = t0 + r / rep, h = g * rep + r % rep;
    if (a.gate != nullptr) y *= gate_of(reinterpret_cast<const bf16_t*>(a.gate) + t * a.ldg + h * V, col);
    out[(t * H + h) * V + col] = f2bf(y);
  }
}

// Prompt portions: 64 rows per workgroup (16 per wave). The waves walk the same key tiles; a token tile's keys
// and transposed values are brought into LDS once per workgroup (two buffers: tile t + 1 is asked for before
// tile t is computed, written after it, one barrier per tile), and every wave takes its fragments from there.
// Pooled tiles come first and are read straight from the pooled caches by each wave, as in the kernel above.
template <int NCT, int NQF, int BIAS, bool CAP>
__global__ __launch_bounds__(256) void window_attn_tiled_kernel(WindowArgs a, const bf16_t* __restrict__ q,
                                                                 float scale_log2e, const bf16_t* __restrict__ vt,
                                                                 int num_pages, bf16_t* __restrict__ out) {
  extern __shared__ float btab[];  // BIAS: the distance table of this workgroup's heads (when it is staged)
  constexpr int DP = 32 * NQF + 8;  // padded row of a staged key (bf16): rows 16 B apart in the banks
  constexpr int VP = 40;            // padded row of a staged value column: 32 keys + 8
  constexpr int NKC = (32 * 4 * NQF + 255) / 256, NVC = (4 * 16 * NCT + 255) / 256;  // 16-B pieces per thread
  __shared__ __attribute__((aligned(16))) bf16_t kl[2][32][DP];
  __shared__ __attribute__((aligned(16))) bf16_t vl[2][16 * NCT][VP];
  __shared__ __attribute__((aligned(16))) bf16_t pl[4][16][40];
  const int D = a.D, V = a.V, G = a.G, H = a.H, rep = H / G, g = blockIdx.y, P = a.pool;
  const int GV = a.GV, gv = g / (G / GV);  // value heads; the value head of key head g
  int s = -1, tile = 0, base = 0;
  for (int i = 0; i < a.S; ++i) {  // (sequence, 64-row tile) of this workgroup
    const int nt = ((a.query_start[i + 1] - a.query_start[i]) * rep + 63) / 64;
    if ((int)blockIdx.x < base + nt) { s = i; tile = blockIdx.x - base; break; }
    base += nt;
  }
  if (s < 0) return;
  const int tid = threadIdx.x, wv = tid >> 6, l = tid & 63, lr = l & 15, lg = l >> 4;
  const int t0 = a.query_start[s], ntok = a.query_start[s + 1] - t0;
  const int pos0 = a.context_lens[s] - ntok;
  const int nrows = ntok * rep;
  const int rowb = tile * 64;        // first row of the workgroup
  if (rowb >= nrows) return;
  const int row0 = rowb + wv * 16;   // first row of the wave
  const bool active = row0 < nrows;  // wave-uniform; an idle wave still stages tiles and meets the barriers
  const bf16_t* kc = reinterpret_cast<const bf16_t*>(a.kc);
  const bf16_t* kp = reinterpret_cast<const bf16_t*>(a.kp);
  const bf16_t* vp = reinterpret_cast<const bf16_t*>(a.vp);
  const int nqf = (D + 31) >> 5, nct = (V + 15) >> 4, d8 = D >> 3;
  for (int e = tid; e < 2 * 32 * DP / 8; e += 256) reinterpret_cast<uint4*>(&kl[0][0][0])[e] = make_uint4(0, 0, 0, 0);
  for (int e = tid; e < 2 * 16 * NCT * VP / 8; e += 256) reinterpret_cast<uint4*>(&vl[0][0][0])[e] = make_uint4(0, 0, 0, 0);
  if (BIAS) {
    bias_stage(a, btab, g, rep, tid, 256);
    __syncthreads();  // the rows' set-up below reads the staged table
  }
  bf16x8 qf[NQF];
  {
    const int r = row0 + lr;
    const bool ok = r < nrows;
    const bf16_t* qrow = q + ((int64_t)(t0 + (ok ? r / rep : 0)) * H + g * rep + (ok ? r % rep : 0)) * D;
#pragma unroll
    for (int kk = 0; kk < NQF; ++kk) qf[kk] = frag16(qrow, 32 * kk + 8 * lg, D, ok && kk < nqf);
  }
  int hi[4], lo[4], nbv[4];
  float m[4], lsum[4];
  float bw[BIAS ? 4 : 1], bx[BIAS ? 4 : 1], bfar[BIAS ? 4 : 1];
  int bo[BIAS ? 4 : 1];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + 4 * lg + i;
    const bool ok = r < nrows;
    const int p = pos0 + (ok ? r / rep : 0);
    hi[i] = ok ? p : -1;
    lo[i] = p - a.window + 1;
    nbv[i] = (ok && P > 0) ? max(0, lo[i]) / P : 0;
    if (BIAS) {
      bias_row(a, g, rep, r, ok, bw[i], bx[i], bo[i]);
      bfar[i] = a.bias_kind == 2 ? bias_of(a, btab, g, rep, 0.f, 0.f, bo[i], a.bias_n - 1) : 0.f;
    }
    const bool sk = ok && a.sink != nullptr;
    m[i] = sk ? a.sink[g * rep + r % rep] * 1.4426950408889634f : -INFINITY;
    lsum[i] = (sk && lr == 0) ? 1.f : 0.f;
  }
  // workgroup-uniform key ranges
  const int lastb = min(rowb + 63, nrows - 1);
  const int pminb = pos0 + rowb / rep, pmaxb = pos0 + lastb / rep;
  const int jt0 = max(0, pminb - a.window + 1) >> 5, jt1 = pmaxb >> 5;
  // wave-uniform: what this wave's rows can see at all
  const int lastw = min(row0 + 15, nrows - 1);
  const int pminw = pos0 + row0 / rep, pmaxw = pos0 + lastw / rep;
  const int klow = max(0, pminw - a.window + 1);
  const int nbmax = (active && P > 0) ? max(0, pmaxw - a.window + 1) / P : 0;
  f32x4 O[NCT];
#pragma unroll
  for (int ct = 0; ct < NCT; ++ct) O[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int32_t* bt = a.block_tables + (int64_t)s * a.max_blocks;

  // one tile's scores -> weights -> P in LDS; returns nothing, updates m, lsum, O scale
  auto softmax_tile = [&](const f32x4& s0, const f32x4& s1, int kbase, bool pooled) {
    float al[4];
    const int c0 = kbase + lr, c1 = kbase + 16 + lr;
    float bt0[BIAS ? 4 : 1], bt1[BIAS ? 4 : 1];
    if (BIAS) bias_tile(a, btab, g, rep, bw, bx, bo, bfar, hi, c0, kbase + 31 <= pminw - (a.bias_n - 1), bt0, bt1);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool vis0 = pooled ? c0 < nbv[i] : (c0 >= lo[i] && c0 <= hi[i]);
      const bool vis1 = pooled ? c1 < nbv[i] : (c1 >= lo[i] && c1 <= hi[i]);
      const float v0 = vis0 ? score_log2<CAP>(a, s0[i], scale_log2e, BIAS ? bt0[i] : 0.f) : -INFINITY;
      const float v1 = vis1 ? score_log2<CAP>(a, s1[i], scale_log2e, BIAS ? bt1[i] : 0.f) : -INFINITY;
      const float mnew = fmaxf(m[i], group16_max(fmaxf(v0, v1)));
      const float ms = (mnew == -INFINITY) ? 0.f : mnew;
      al[i] = exp2f(m[i] - ms);
      const float p0 = exp2f(v0 - ms), p1 = exp2f(v1 - ms);
      lsum[i] = lsum[i] * al[i] + p0 + p1;
      m[i] = mnew;
      pl[wv][4 * lg + i][lr] = f2bf(p0);
      pl[wv][4 * lg + i][16 + lr] = f2bf(p1);
    }
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
      for (int i = 0; i < 4; ++i) O[ct][i] *= al[i];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wave's P tile is written (LDS is in order per wave)
  };

  // pooled tiles: each wave for itself, straight from the pooled caches
  for (int ti = 0; ti < ((nbmax + 31) >> 5); ++ti) {
    const int kbase = 32 * ti;
    const int e0 = min(kbase + lr, nbmax - 1) * P + P - 1, e1 = min(kbase + 16 + lr, nbmax - 1) * P + P - 1;
    const int q0 = min(max(bt[e0 >> 4], 0), num_pages - 1), q1 = min(max(bt[e1 >> 4], 0), num_pages - 1);
    const bf16_t* k0p = kp + (((int64_t)q0 * G + g) * a.npool + (e0 & 15) / P) * D;
    const bf16_t* k1p = kp + (((int64_t)q1 * G + g) * a.npool + (e1 & 15) / P) * D;
    f32x4 s0 = f32x4{0.f, 0.f, 0.f, 0.f}, s1 = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < NQF; ++kk)
      if (kk < nqf) {
        const int off = min(32 * kk + 8 * lg, D - 8);
        s0 = mfma16(qf[kk], as_bf16x8(ld16(k0p + off)), s0);
        s1 = mfma16(qf[kk], as_bf16x8(ld16(k1p + off)), s1);
      }
    softmax_tile(s0, s1, kbase, true);
    const bf16x8 pf = as_bf16x8(*reinterpret_cast<const uint4*>(&pl[wv][lr][8 * lg]));
    int64_t ro[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int e1b = min(kbase + 8 * lg + e, nbmax - 1) * P + P - 1;
      const int pq = min(max(bt[e1b >> 4], 0), num_pages - 1);
      ro[e] = (((int64_t)pq * G + g) * a.npool + (e1b & 15) / P) * V;
    }
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct)
      if (ct < nct) {
        const int col = min(16 * ct + lr, V - 1);
        uint32_t w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) w[j] = (uint32_t)vp[ro[2 * j] + col] | ((uint32_t)vp[ro[2 * j + 1] + col] << 16);
        O[ct] = mfma16(pf, as_bf16x8(make_uint4(w[0], w[1], w[2], w[3])), O[ct]);
      }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // P tile read before the next tile overwrites it
  }

  // token tiles through LDS (asking for tile t + 2 as well, through a second register set, was measured: 164
  // registers, 139 us against 85 us)
  uint4 kr[NKC], vr[NVC];
  auto fetch = [&](int jt) {
    const int kbase = 32 * jt;
    int pg0 = bt[kbase >> 4];
    int pg1 = (kbase + 16 <= pmaxb) ? bt[(kbase >> 4) + 1] : pg0;
    pg0 = min(max(pg0, 0), num_pages - 1);
    pg1 = min(max(pg1, 0), num_pages - 1);
#pragma unroll
    for (int u = 0; u < NKC; ++u) {
      const int c = tid + 256 * u;
      const int key = c / d8, off = (c % d8) * 8;
      const int pg = key < 16 ? pg0 : pg1;
      kr[u] = c < 32 * d8 ? ld16(kc + (((int64_t)pg * G + g) * 16 + (key & 15)) * D + off) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < NVC; ++u) {
      const int c = tid + 256 * u;
      const int col = c >> 2, half = (c >> 1) & 1, sub = c & 1;
      const int pg = half ? pg1 : pg0;
      vr[u] = col < V ? ld16(vt + (((int64_t)pg * GV + gv) * V + col) * 16 + 8 * sub) : make_uint4(0, 0, 0, 0);
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int u = 0; u < NKC; ++u) {
      const int c = tid + 256 * u;
      if (c < 32 * d8) *reinterpret_cast<uint4*>(&kl[buf][c / d8][(c % d8) * 8]) = kr[u];
    }
#pragma unroll
    for (int u = 0; u < NVC; ++u) {
      const int c = tid + 256 * u;
      const int col = c >> 2;
      if (col < V) *reinterpret_cast<uint4*>(&vl[buf][col][16 * ((c >> 1) & 1) + 8 * (c & 1)]) = vr[u];
    }
  };
  __syncthreads();  // the zero fill is done before the first tile is staged
  fetch(jt0);
  int buf = 0;
  // a buffer is rewritten two tiles later, after the barrier of the tile in between, which every wave
  // reaches only when it has finished reading it
  for (int jt = jt0; jt <= jt1; ++jt) {
    stage(buf);
    __syncthreads();
    if (jt < jt1) fetch(jt + 1);
    const int kbase = 32 * jt;
    if (active && kbase + 31 >= klow && kbase <= pmaxw) {  // wave-uniform: some row of the wave may see the tile
      f32x4 s0 = f32x4{0.f, 0.f, 0.f, 0.f}, s1 = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < NQF; ++kk)
        if (kk < nqf) {
          s0 = mfma16(qf[kk], as_bf16x8(*reinterpret_cast<const uint4*>(&kl[buf][lr][32 * kk + 8 * lg])), s0);
          s1 = mfma16(qf[kk], as_bf16x8(*reinterpret_cast<const uint4*>(&kl[buf][16 + lr][32 * kk + 8 * lg])), s1);
        }
      softmax_tile(s0, s1, kbase, false);
      const bf16x8 pf = as_bf16x8(*reinterpret_cast<const uint4*>(&pl[wv][lr][8 * lg]));
#pragma unroll
      for (int ct = 0; ct < NCT; ++ct)
        if (ct < nct)
          O[ct] = mfma16(pf, as_bf16x8(*reinterpret_cast<const uint4*>(&vl[buf][16 * ct + lr][8 * lg])), O[ct]);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // P tile read before the next tile overwrites it
    }
    buf ^= 1;
  }
  if (!active) return;
  const int vrot = a.v_freq != nullptr ? 2 * (V / 2) : 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float inv = 1.f / group16_sum(lsum[i]);
    const int r = row0 + 4 * lg + i;
    const bool ok = r < nrows;
    const float fp = -(float)(pos0 + (ok ? r / rep : 0));
    bf16_t* orow = out + ((int64_t)(t0 + (ok ? r / rep : 0)) * H + g * rep + (ok ? r % rep : 0)) * V;
    const bf16_t* grow = a.gate == nullptr ? nullptr : reinterpret_cast<const bf16_t*>(a.gate) +
        (int64_t)(t0 + (ok ? r / rep : 0)) * a.ldg + (int64_t)(g * rep + (ok ? r % rep : 0)) * V;
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) {
      const int col = 16 * ct + lr;
      float y = O[ct][i] * inv;
      if (vrot > 0) {
        const float other = __shfl_xor(y, 1, 64);
        if (col < vrot) {
          const float ang = fp * a.v_freq[col >> 1];
          const float cs = cosf(ang), sn = sinf(ang);
          y = (col & 1) ? (y * cs + other * sn) : (y * cs - other * sn);
        }
      }
      if (ok && ct < nct && col < V) orow[col] = f2bf(grow != nullptr ? y * gate_of(grow, col) : y);
    }
  }
}

template <int NCT, int NQF, int BIAS, bool CAP>
void launch_window_mfma(const WindowArgs& a, const void* q, float scale, const void* vt, int num_pages, void* out,
                        hipStream_t st) {
  const int rep = a.H / a.G;
  const size_t dyn = (BIAS && a.bias_kind == 2 && a.bias_lds) ? (size_t)rep * a.bias_n * sizeof(float) : 0;
  const int blocks = (a.T * rep + 15) / 16 + a.S;
  const bf16_t* qp = reinterpret_cast<const bf16_t*>(q);
  const bf16_t* vp = reinterpret_cast<const bf16_t*>(vt);
  bf16_t* op = reinterpret_cast<bf16_t*>(out);
  const float sl = scale * 1.4426950408889634f;
  // few rows per sequence (decoded tokens): few workgroups, so eight waves each stream the keys of 16 rows;
  // prompt portions: 64 rows per workgroup over key / value tiles staged in LDS (or, by a.prefill_kernel == 1,
  // 16 rows per workgroup with the key tiles shared out over four waves)
  if ((int64_t)a.T * rep <= 16 * (int64_t)a.S) {
    const int parts = a.parts > 1 ? a.parts : 1;
    hipLaunchKernelGGL((window_attn_mfma_kernel<NCT, NQF, 8, BIAS, CAP>), dim3(blocks, a.G, parts), dim3(512), dyn, st, a, qp, sl, vp,
                       num_pages, op);
    if (parts > 1) hipLaunchKernelGGL(window_attn_merge_kernel, dim3(blocks, a.G, 4), dim3(256), 0, st, a, 16 * NCT, op);
  }
  else if (a.prefill_kernel == 1 || NCT > 8)
    hipLaunchKernelGGL((window_attn_mfma_kernel<NCT, NQF, 4, BIAS, CAP>), dim3(blocks, a.G), dim3(256), dyn, st, a, qp, sl, vp, num_pages, op);
  else
    hipLaunchKernelGGL((window_attn_tiled_kernel<NCT, NQF, BIAS, CAP>), dim3((a.T * rep + 63) / 64 + a.S, a.G), dim3(256), dyn, st, a, qp, sl,
                       vp, num_pages, op);
}

}  // namespace
int window_attn_nct(int D, int V);
namespace {

template <int BIAS, bool CAP>
void launch_window_mfma_sized(const WindowArgs& a, const void* q, float scale, const void* vt, int num_pages, void* out,
                              hipStream_t st) {
  const int nct = window_attn_nct(a.D, a.V);  // (the scratch of a split launch is sized by the same rule)
  if (nct == 4) launch_window_mfma<4, 2, BIAS, CAP>(a, q, scale, vt, num_pages, out, st);
  else if (nct == 8) launch_window_mfma<8, 4, BIAS, CAP>(a, q, scale, vt, num_pages, out, st);
  else launch_window_mfma<16, 8, BIAS, CAP>(a, q, scale, vt, num_pages, out, st);
}

int heads_per_block(const WindowArgs& a) {
  const int rep = a.H / a.G;
  int HC = rep < 8 ? rep : 8;
  auto lds = [&](int hc) { return window_attn_lds_bytes(a, hc); };
  while (HC > 1 && (HC * a.V > 256 * MAXACC || lds(HC) > 60 * 1024)) --HC;
  return HC;
}

}  // namespace

// Decoded tokens on the MFMA kernel: how many workgroups share the key tiles of a 16-row tile (1: no split) so that
// the launch has about two workgroups of eight waves per CU, and the scratch floats their partial results take.
int window_attn_parts(int T, int S, int H, int G, int D, int V, int f32, int page) {
  const int rep = H / G;
  if (f32 || page != 16 || D % 8 != 0 || D < 8 || D > 256 || V > 256 || (int64_t)T * rep > 16 * (int64_t)S) return 1;
  const int wg = ((T * rep + 15) / 16 + S) * G;
  const int parts = 512 / (wg > 0 ? wg : 1);
  return parts < 2 ? 1 : (parts > 8 ? 8 : parts);
}
int window_attn_nct(int D, int V) { return (D <= 64 && V <= 64) ? 4 : ((D <= 128 && V <= 128) ? 8 : 16); }
size_t window_attn_part_floats(int T, int S, int H, int G, int D, int V, int parts) {
  const int rep = H / G;
  const size_t slots = (size_t)parts * G * ((T * rep + 15) / 16 + S);
  return parts > 1 ? slots * 16 * (16 * window_attn_nct(D, V) + 2) : 0;
}

size_t window_attn_lds_bytes(const WindowArgs& a, int HC) {
  return ((size_t)HC * (a.D + 1) + (size_t)KT * (a.D + 1) + (size_t)KT * (a.V + 1) + HC * KT + 3 * HC + (size_t)HC * a.V) *
         sizeof(float);
}

bool window_attn_fits(const WindowArgs& a) {
  return a.V <= 256 * MAXACC && window_attn_lds_bytes(a, 1) <= 60 * 1024 &&
         (size_t)((a.H + a.G) * (a.D + 1)) * sizeof(float) <= 60 * 1024;
}

void launch_window_write(const WindowArgs& a, const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v,
                         int64_t ldv, const float* qw, const float* kw, float eps, int norm_all, void* q_out, void* vt,
                         const float* q_head_scale, float q_temp_coef, int q_temp_every, int rot_half, hipStream_t st) {
  if (a.T <= 0) return;
  const size_t lds = (size_t)((a.H + a.G) * a.D + a.H + a.G) * sizeof(float);
  hipLaunchKernelGGL(window_write_kernel, dim3(a.T), dim3(256), lds, st, a, q, ldq, k, ldk, v, ldv, qw, kw, eps, norm_all,
                     q_out, reinterpret_cast<bf16_t*>(vt), q_head_scale, q_temp_coef, q_temp_every, rot_half);
}

void launch_window_pool(const WindowArgs& a, hipStream_t st) {
  if (a.T <= 0 || a.pool <= 0 || a.S <= 0) return;
  const dim3 grid(a.T, (a.G * (a.D + a.V) + 255) / 256);
  if (a.f32) hipLaunchKernelGGL(window_pool_kernel<float>, grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL(window_pool_kernel<bf16_t>, grid, dim3(256), 0, st, a);
}

void launch_window_attn(const WindowArgs& a0, const void* q, float scale, void* out, const void* vt, int num_pages,
                        hipStream_t st) {
  if (a0.T <= 0 || a0.S <= 0) return;
  WindowArgs a = a0;
  if (a.softcap > 0.f) { a.cap_in = 2.f / a.softcap; a.cap_out = a.softcap * 1.4426950408889634f; }
  if (!a.f32 && vt != nullptr && a.page == 16 && a.D % 8 == 0 && a.D >= 8 && a.D <= 256 && a.V <= 256) {
    if (a.bias_kind != 0) launch_window_mfma_sized<1, false>(a, q, scale, vt, num_pages, out, st);
    else if (a.softcap > 0.f) launch_window_mfma_sized<0, true>(a, q, scale, vt, num_pages, out, st);
    else launch_window_mfma_sized<0, false>(a, q, scale, vt, num_pages, out, st);
    return;
  }
  const int HC = heads_per_block(a);
  const int rep = a.H / a.G;
  hipLaunchKernelGGL(window_attn_kernel, dim3(a.T, a.G, (rep + HC - 1) / HC), dim3(256), window_attn_lds_bytes(a, HC), st,
                     a, q, HC, scale, out);
}

}  // namespace vgate
