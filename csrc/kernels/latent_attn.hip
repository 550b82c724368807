// Latent attention over a paged cache that holds, per token, one normed latent vector (rank) and one
// rotated key part (rot) shared by all heads. The per-head key and value up-projections are absorbed
// into the query and the output (q' = W_uk^T q, out = W_uv (sum_j p_j c_j)), so prompt portions and
// single decoded tokens run the same kernel on the cached rows alone:
//   score(t, h, j) = scale * (q'[t][h] . c_j + rope(q_rot[t][h]) . k_rot_j),   0 <= position(t) - j < window
//   ol[t][h]       = sum_j softmax_j(score) c_j
// A sink (one logit per head) only enters the softmax denominator: the running max starts at it, the sum at 1.
// Key tiles sit at absolute positions whatever the window's start, so a row's sums keep their order.
// latent_write: RMS norm of the latent (fp32 statistics) + interleaved-pair rotation of the shared key
// part + the paged store, one launch. Angles are position * inv_freq in fp32 with full-range sin / cos.
// latent_attn, fp32 caches (and shapes the MFMA kernel does not take): one workgroup per (token, group
// of heads); key tiles of 16 rows staged in LDS as fp32, scores, running max / sum and the weighted
// latent sum all in fp32 FMA.
// latent_attn, bf16 caches: MFMA kernel. Query rows are (token, head) pairs of one sequence, 16 per wave
// (4 independent waves per workgroup), keys in tiles of 32 = two pages:
//   S = Q K^T    v_mfma 16x16x32, Q fragments stationary in registers, K fragments (16 B of one cached
//                row per lane) straight from the cache
//   online softmax in fp32 (exp2 of log2(e)-scaled scores, per-lane partial row sums)
//   O += P C     P goes C-layout -> A-layout through a 16 x 32 bf16 tile in LDS; the B operand needs
//                eight consecutive KEYS of one latent column per lane, which the cache's second,
//                transposed copy of the latent part ([page][column][16 keys], written by latent_write)
//                delivers as one 16-B load: no transposition in the kernel
// Waves of a workgroup never meet at a barrier (each loops to its own causal limit), except for a
// sequence whose rows fit one wave (a decoded token): there the four waves take every fourth key tile
// of the same rows and merge their partial (max, sum, weighted latent) through LDS, so a lone token's
// keys are streamed by four waves instead of one. With parts > 1 (steps of decoded tokens: few workgroups), blockIdx.y
// of up to eight workgroups share such a sequence's key tiles (tile t goes to workgroup (t / 4) mod parts, wave
// t mod 4); each leaves its merged (max, sum, weighted latent) in an fp32 scratch and latent_attn_merge_kernel
// rescales and adds them in part order. The number of parts depends on the step's shape alone.
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

__global__ __launch_bounds__(256) void latent_write_kernel(LatentArgs a, const void* __restrict__ kv, int64_t ldkv,
                                                            const float* __restrict__ w, float eps,
                                                            bf16_t* __restrict__ cache_t, int page) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  const int slot = a.slots[t];
  if (slot < 0) return;  // uniform per block
  const int64_t src = (int64_t)t * ldkv;
  const int64_t dst = (int64_t)slot * (a.rank + a.rot);
  float ss = 0.f;
  for (int c = threadIdx.x; c < a.rank; c += blockDim.x) {
    const float v = ldx(kv, src + c, a.f32);
    ss = fmaf(v, v, ss);
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)a.rank + eps);
  for (int c = threadIdx.x; c < a.rank; c += blockDim.x) {
    const float v = ldx(kv, src + c, a.f32) * inv * w[c];
    stx(a.cache, dst + c, a.f32, v);
    if (cache_t != nullptr)  // [page][column][key in page]
      cache_t[((int64_t)(slot / page) * a.rank + c) * page + slot % page] = f2bf(v);
  }
  const float pos = (float)a.positions[t];
  for (int i = threadIdx.x; i < a.rot; i += blockDim.x) {
    float o;
    if (i < a.rot_dims) {
      const float ang = pos * a.inv_freq[i >> 1];
      const float cs = cosf(ang), sn = sinf(ang);
      const float u = ldx(kv, src + a.rank + (i & ~1), a.f32), v = ldx(kv, src + a.rank + (i | 1), a.f32);
      o = (i & 1) ? (v * cs + u * sn) : (u * cs - v * sn);
    } else {
      o = ldx(kv, src + a.rank + i, a.f32);
    }
    stx(a.cache, dst + a.rank + i, a.f32, o);
  }
}

__global__ __launch_bounds__(256) void latent_qrope_kernel(LatentArgs a, const void* __restrict__ q, int H, int dim,
                                                            void* __restrict__ qa) {
  const int t = blockIdx.x;
  const float pos = (float)a.positions[t];
  for (int e = threadIdx.x; e < H * a.rot; e += blockDim.x) {
    const int h = e / a.rot, i = e % a.rot;
    const int64_t src = ((int64_t)t * H + h) * (dim + a.rot) + dim;
    float o;
    if (i < a.rot_dims) {
      const float ang = pos * a.inv_freq[i >> 1];
      const float cs = cosf(ang), sn = sinf(ang);
      const float u = ldx(q, src + (i & ~1), a.f32), v = ldx(q, src + (i | 1), a.f32);
      o = (i & 1) ? (v * cs + u * sn) : (u * cs - v * sn);
    } else {
      o = ldx(q, src + i, a.f32);
    }
    stx(qa, ((int64_t)t * H + h) * (a.rank + a.rot) + a.rank + i, a.f32, o);
  }
}

constexpr int KT = 16;      // keys per tile
constexpr int MAXACC = 16;  // latent outputs per thread: heads-per-block * rank <= 256 * MAXACC

__global__ __launch_bounds__(256) void latent_attn_kernel(LatentArgs a, const void* __restrict__ qa, int H, int HC,
                                                           float scale, const int32_t* __restrict__ block_tables,
                                                           int max_blocks, int page,
                                                           const int32_t* __restrict__ context_lens,
                                                           const int32_t* __restrict__ query_start, int S,
                                                           void* __restrict__ ol, int window,
                                                           const float* __restrict__ sink) {
  extern __shared__ float lds[];
  const int E = a.rank + a.rot, EP = E + 1;
  float* qs = lds;                  // [HC][EP]
  float* ks = qs + HC * EP;         // [KT][EP]
  float* sc = ks + KT * EP;         // [HC][KT] scores, then weights
  float* mrun = sc + HC * KT;       // [HC]
  float* lrun = mrun + HC;          // [HC]
  float* alpha = lrun + HC;         // [HC]
  const int t = blockIdx.x;
  if (t >= query_start[S]) return;
  int lo = 0, hi = S - 1;           // the sequence of token t: query_start[s] <= t < query_start[s + 1]
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (query_start[mid] <= t) lo = mid; else hi = mid - 1;
  }
  const int s = lo;
  const int nkeys = context_lens[s] - (query_start[s + 1] - t) + 1;
  const int first = max(0, nkeys - window);  // the oldest key the token sees
  const int h0 = blockIdx.y * HC;
  const int nh = min(HC, H - h0);
  const int tid = threadIdx.x;
  for (int e = tid; e < nh * E; e += 256) {
    const int h = e / E, c = e % E;
    qs[h * EP + c] = ldx(qa, ((int64_t)t * H + h0 + h) * E + c, a.f32);
  }
  if (tid < HC) {
    const bool sk = sink != nullptr && tid < nh;
    mrun[tid] = sk ? sink[h0 + tid] : -INFINITY;
    lrun[tid] = sk ? 1.f : 0.f;
    alpha[tid] = 1.f;
  }
  float acc[MAXACC];
#pragma unroll
  for (int i = 0; i < MAXACC; ++i) acc[i] = 0.f;
  const int32_t* bt = block_tables + (int64_t)s * max_blocks;
  for (int j0 = (first / KT) * KT; j0 < nkeys; j0 += KT) {
    __syncthreads();  // previous tile fully consumed (and q / running stats written)
    for (int e = tid; e < KT * E; e += 256) {
      const int jj = e / E, c = e % E;
      const int kj = j0 + jj;
      float v = 0.f;
      if (kj < nkeys && kj >= first) {
        const int64_t row = (int64_t)bt[kj / page] * page + kj % page;
        v = ldx(a.cache, row * E + c, a.f32);
      }
      ks[jj * EP + c] = v;
    }
    __syncthreads();
    {  // scores: two threads per (head, key), each half of the dot product
      const int wi = tid >> 1, half = tid & 1;
      float d = 0.f;
      const bool on = wi < nh * KT;
      const int h = on ? wi / KT : 0, jj = on ? wi % KT : 0;
      if (on) {
        const int c0 = half ? (E >> 1) : 0, c1 = half ? E : (E >> 1);
        const float* qp = qs + h * EP;
        const float* kp = ks + jj * EP;
        for (int c = c0; c < c1; ++c) d = fmaf(qp[c], kp[c], d);
      }
      d += __shfl_xor(d, 1, 64);
      if (on && half == 0) sc[h * KT + jj] = (j0 + jj < nkeys && j0 + jj >= first) ? d * scale : -INFINITY;
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
      if (o < nh * a.rank) {
        const int h = o / a.rank, c = o % a.rank;
        float v = 0.f;
        const float* pp = sc + h * KT;
#pragma unroll
        for (int jj = 0; jj < KT; ++jj) v = fmaf(pp[jj], ks[jj * EP + c], v);
        acc[i] = fmaf(acc[i], alpha[h], v);
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < MAXACC; ++i) {
    const int o = tid + i * 256;
    if (o < nh * a.rank) {
      const int h = o / a.rank, c = o % a.rank;
      stx(ol, ((int64_t)t * H + h0 + h) * a.rank + c, a.f32, acc[i] / lrun[h]);
    }
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

// NCT: 16-column tiles of the latent (rank <= 16 NCT); NQF: 32-wide fragments of a query row (E <= 32 NQF).
// E % 8 == 0 (host-checked): every cache fragment is one unconditional 16-B load. Loads are issued in
// groups (LG fragments, then their MFMAs) so a lone wave has several in flight; a fragment past the row's
// end or the latent's last column is read from a clamped address: its partner (zero Q fragment) or its
// output column (never stored) makes the value irrelevant, and cached values are always finite.
constexpr int LG = 4;
template <int NCT, int NQF>
__global__ __launch_bounds__(256) void latent_attn_mfma_kernel(LatentArgs a, const bf16_t* __restrict__ qa, int H,
                                                                float scale_log2e,
                                                                const int32_t* __restrict__ block_tables,
                                                                int max_blocks, int num_pages,
                                                                const int32_t* __restrict__ context_lens,
                                                                const int32_t* __restrict__ query_start, int S,
                                                                const bf16_t* __restrict__ cache_t,
                                                                bf16_t* __restrict__ ol, int window,
                                                                const float* __restrict__ sink, int parts,
                                                                float* __restrict__ part_o, float* __restrict__ part_ml) {
  __shared__ __attribute__((aligned(16))) bf16_t pl[4][16][40];
  __shared__ float mrg_m[4][16], mrg_l[4][16];
  __shared__ float mrg_o[16][16 * NCT];  // split mode: the merged weighted latent of the 16 rows
  const int E = a.rank + a.rot, KR = a.rank;
  int s = -1, tile = 0, base = 0;
  for (int i = 0; i < S; ++i) {  // (sequence, 64-row tile) of this workgroup
    const int nt = ((query_start[i + 1] - query_start[i]) * H + 63) / 64;
    if ((int)blockIdx.x < base + nt) { s = i; tile = blockIdx.x - base; break; }
    base += nt;
  }
  if (s < 0) return;
  const int wv = threadIdx.x >> 6, l = threadIdx.x & 63, lr = l & 15, lg = l >> 4;
  const int t0 = query_start[s], ntok = query_start[s + 1] - t0;
  const int pos0 = context_lens[s] - ntok;
  const int nrows = ntok * H;
  const bool split = nrows <= 16;  // workgroup-uniform: one row tile, keys shared out over the four waves
  const int part = blockIdx.y;     // (only sequences in split mode are shared out over several workgroups)
  if (!split && part > 0) return;
  const int np = split ? parts : 1;
  const int row0 = split ? 0 : tile * 64 + wv * 16;
  if (row0 >= nrows) return;
  const bf16_t* cache = reinterpret_cast<const bf16_t*>(a.cache);
  const int nqf = (E + 31) >> 5, nct = (KR + 15) >> 4;
  // stationary Q fragments: A operand, lane holds Q[row lr][32 kk + 8 lg ..]
  bf16x8 qf[NQF];
  {
    const int r = row0 + lr;
    const bool ok = r < nrows;
    const bf16_t* qrow = qa + ((int64_t)(t0 + (ok ? r / H : 0)) * H + (ok ? r % H : 0)) * E;
#pragma unroll
    for (int kk = 0; kk < NQF; ++kk) qf[kk] = frag16(qrow, 32 * kk + 8 * lg, E, ok && kk < nqf);
  }
  // C-layout rows of this lane: row0 + 4 lg + i; keys visible to each
  int limit[4], lowest[4];
  float m[4], lsum[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + 4 * lg + i;
    const bool ok = r < nrows;
    limit[i] = ok ? pos0 + r / H + 1 : 0;   // keys [lowest, limit); a row past the last sees none
    lowest[i] = max(0, limit[i] - window);
    const bool sk = ok && sink != nullptr && (!split || (wv == 0 && part == 0));  // the sink counts once
    m[i] = sk ? sink[r % H] * 1.4426950408889634f : -INFINITY;
    lsum[i] = (sk && lr == 0) ? 1.f : 0.f;
  }
  const int last = min(row0 + 15, nrows - 1);
  const int kmax = pos0 + last / H + 1;  // wave-uniform
  const int kmin = max(0, pos0 + row0 / H + 1 - window) & ~31;  // first tile any row of the wave sees
  f32x4 O[NCT];
#pragma unroll
  for (int ct = 0; ct < NCT; ++ct) O[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int32_t* bt = block_tables + (int64_t)s * max_blocks;
  for (int j0 = kmin + (split ? 32 * (wv + 4 * part) : 0); j0 < kmax; j0 += split ? 128 * np : 32) {
    int pg0 = bt[j0 >> 4];
    int pg1 = (j0 + 16 < kmax) ? bt[(j0 >> 4) + 1] : pg0;
    pg0 = min(max(pg0, 0), num_pages - 1);
    pg1 = min(max(pg1, 0), num_pages - 1);
    f32x4 s0 = f32x4{0.f, 0.f, 0.f, 0.f}, s1 = f32x4{0.f, 0.f, 0.f, 0.f};
    const bf16_t* k0p = cache + ((int64_t)pg0 * 16 + lr) * E;
    const bf16_t* k1p = cache + ((int64_t)pg1 * 16 + lr) * E;
#pragma unroll
    for (int k0 = 0; k0 < NQF; k0 += LG) {
      if (k0 < nqf) {  // wave-uniform
        uint4 b0[LG], b1[LG];
#pragma unroll
        for (int u = 0; u < LG; ++u) {
          const int off = min(32 * (k0 + u) + 8 * lg, E - 8);
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
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float v0 = (j0 + lr < limit[i] && j0 + lr >= lowest[i]) ? s0[i] * scale_log2e : -INFINITY;
      const float v1 = (j0 + 16 + lr < limit[i] && j0 + 16 + lr >= lowest[i]) ? s1[i] * scale_log2e : -INFINITY;
      const float mnew = fmaxf(m[i], group16_max(fmaxf(v0, v1)));
      const float ms = (mnew == -INFINITY) ? 0.f : mnew;  // a row that has seen no key yet (split mode)
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
    const int pgs = (lg >> 1) ? pg1 : pg0;
    const bf16_t* tp = cache_t + (int64_t)pgs * KR * 16 + 8 * (lg & 1);
#pragma unroll
    for (int c0 = 0; c0 < NCT; c0 += 2 * LG) {
      if (c0 < nct) {  // wave-uniform
        uint4 b[2 * LG];
#pragma unroll
        for (int u = 0; u < 2 * LG; ++u) b[u] = ld16(tp + (int64_t)min(16 * (c0 + u) + lr, KR - 1) * 16);
#pragma unroll
        for (int u = 0; u < 2 * LG; ++u)
          if (c0 + u < NCT) O[c0 + u] = mfma16(pf, as_bf16x8(b[u]), O[c0 + u]);
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // P tile read before the next tile overwrites it
  }
  if (split) {
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
      for (int w = 1; w < 4; ++w) M = fmaxf(M, mrg_m[w][r]);
      const float Ms = (M == -INFINITY) ? 0.f : M;  // (rows past the sequence's last)
      float L = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) L += mrg_l[w][r] * exp2f(mrg_m[w][r] - Ms);  // a wave that saw no key: l = 0, exp2(-inf) = 0
      f[i] = exp2f(m[i] - Ms);
      lsum[i] = L;                // the merged row sum (the same in every lane of the row)
      m[i] = M;
    }
    for (int w = 0; w < 4; ++w) {  // waves add their scaled partials in turn
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
    if (np > 1) {  // (workgroup-uniform) hand the partial result on: the merge kernel finishes the rows
      const int64_t slot = (int64_t)part * gridDim.x + blockIdx.x;
      float* po = part_o + slot * (16 * 16 * NCT);
      for (int e = threadIdx.x; e < 16 * 16 * NCT; e += 256) po[e] = (&mrg_o[0][0])[e];
      if (wv == 0 && lr == 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          part_ml[(slot * 16 + 4 * lg + i) * 2] = m[i];
          part_ml[(slot * 16 + 4 * lg + i) * 2 + 1] = lsum[i];
        }
      }
      return;
    }
    if (wv != 0) return;
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
      for (int i = 0; i < 4; ++i) O[ct][i] = mrg_o[4 * lg + i][16 * ct + lr];
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float tot = split ? lsum[i] : group16_sum(lsum[i]);
    const float inv = 1.f / tot;
    const int r = row0 + 4 * lg + i;
    if (r < nrows) {
      bf16_t* orow = ol + ((int64_t)(t0 + r / H) * H + r % H) * KR;
#pragma unroll
      for (int ct = 0; ct < NCT; ++ct) {
        const int col = 16 * ct + lr;
        if (ct < nct && col < KR) orow[col] = f2bf(O[ct][i] * inv);
      }
    }
  }
}

// The rows of a split sequence from the partial results of `parts` workgroups: M = max of the parts' maxima (log2
// units), sums and weighted latents rescaled by 2^(M_p - M) and added in part order, then normalised and stored.
// vs: the row stride of the parts' weighted latents.
__global__ __launch_bounds__(256) void latent_attn_merge_kernel(int rank, int H, const int32_t* __restrict__ query_start,
                                                                 int S, int parts, int vs, const float* __restrict__ part_o,
                                                                 const float* __restrict__ part_ml,
                                                                 bf16_t* __restrict__ ol) {
  int s = -1, base = 0;
  for (int i = 0; i < S; ++i) {  // the sequence of this workgroup, numbered as in the attention kernel
    const int nt = ((query_start[i + 1] - query_start[i]) * H + 63) / 64;
    if ((int)blockIdx.x < base + nt) { s = i; break; }
    base += nt;
  }
  if (s < 0) return;
  const int t0 = query_start[s], nrows = (query_start[s + 1] - t0) * H;
  if (nrows > 16) return;  // (not shared out: the attention kernel has stored its rows)
  constexpr int MAXP = 8;
  // blockIdx.y: which four rows of the tile
  for (int e = threadIdx.x; e < 4 * rank; e += blockDim.x) {
    const int r = 4 * blockIdx.y + e / rank, col = e % rank;
    if (r >= nrows) continue;
    float pm[MAXP], plv[MAXP], po[MAXP], M = -INFINITY;
#pragma unroll
    for (int p = 0; p < MAXP; ++p) {  // all parts' loads asked for together
      const int64_t slot = (int64_t)min(p, parts - 1) * gridDim.x + blockIdx.x;
      pm[p] = p < parts ? part_ml[(slot * 16 + r) * 2] : -INFINITY;
      plv[p] = part_ml[(slot * 16 + r) * 2 + 1];
      po[p] = part_o[slot * (16 * vs) + r * vs + col];
      M = fmaxf(M, pm[p]);
    }
    float L = 0.f, y = 0.f;
#pragma unroll
    for (int p = 0; p < MAXP; ++p) {
      const float f = exp2f(pm[p] - M);  // a part that saw no key (or is none): max -inf, factor 0
      L = fmaf(plv[p], f, L);
      y = fmaf(po[p], f, y);
    }
    ol[((int64_t)(t0 + r / H) * H + r % H) * rank + col] = f2bf(y / L);
  }
}

template <int NCT, int NQF>
void launch_mfma(const LatentArgs& a, const void* qa, int H, float scale, const int32_t* block_tables, int max_blocks,
                 int num_pages, const int32_t* context_lens, const int32_t* query_start, int S, const void* cache_t,
                 void* ol, int window, const float* sink, int parts, float* scratch, hipStream_t st) {
  const int blocks = (a.T * H + 63) / 64 + S;
  float* part_o = scratch;
  float* part_ml = parts > 1 ? scratch + (size_t)parts * blocks * 16 * 16 * NCT : nullptr;
  hipLaunchKernelGGL((latent_attn_mfma_kernel<NCT, NQF>), dim3(blocks, parts), dim3(256), 0, st, a,
                     reinterpret_cast<const bf16_t*>(qa), H, scale * 1.4426950408889634f, block_tables, max_blocks,
                     num_pages, context_lens, query_start, S, reinterpret_cast<const bf16_t*>(cache_t),
                     reinterpret_cast<bf16_t*>(ol), window, sink, parts, part_o, part_ml);
  if (parts > 1)
    hipLaunchKernelGGL(latent_attn_merge_kernel, dim3(blocks, 4), dim3(256), 0, st, a.rank, H, query_start, S, parts, 16 * NCT,
                       part_o, part_ml, reinterpret_cast<bf16_t*>(ol));
}

// 16-column tiles / 32-wide query fragments of the instantiation that takes a latent of this size
void mfma_shape(int rank, int E, int& nct, int& nqf) {
  if (rank <= 128 && E <= 128) { nct = 8; nqf = 4; }
  else if (rank <= 128 && E <= 192) { nct = 8; nqf = 6; }
  else if (rank <= 256 && E <= 256) { nct = 16; nqf = 8; }
  else if (rank <= 256 && E <= 384) { nct = 16; nqf = 12; }
  else if (E <= 512) { nct = 32; nqf = 16; }
  else { nct = 32; nqf = 20; }
}
bool mfma_takes(int rank, int rot, int f32, int page) {
  const int E = rank + rot;
  return !f32 && page == 16 && rank <= 512 && E <= 640 && E % 8 == 0 && E >= 8;
}

}  // namespace

void launch_latent_write(const LatentArgs& a, const void* kv, int64_t ldkv, const float* w, float eps, void* cache_t,
                         int page, hipStream_t st) {
  if (a.T <= 0) return;
  hipLaunchKernelGGL(latent_write_kernel, dim3(a.T), dim3(256), 0, st, a, kv, ldkv, w, eps,
                     reinterpret_cast<bf16_t*>(cache_t), page);
}

void launch_latent_qrope(const LatentArgs& a, const void* q, int H, int dim, void* qa, hipStream_t st) {
  if (a.T <= 0) return;
  hipLaunchKernelGGL(latent_qrope_kernel, dim3(a.T), dim3(256), 0, st, a, q, H, dim, qa);
}

void launch_latent_attn(const LatentArgs& a, const void* qa, int H, float scale, const int32_t* block_tables,
                        int max_blocks, int page, const int32_t* context_lens, const int32_t* query_start, int S,
                        void* ol, const void* cache_t, int num_pages, int window, const float* sink, int parts,
                        float* scratch, hipStream_t st) {
  if (a.T <= 0 || S <= 0) return;
  const int E = a.rank + a.rot;
  if (cache_t != nullptr && mfma_takes(a.rank, a.rot, a.f32, page)) {
    int nct, nqf;
    mfma_shape(a.rank, E, nct, nqf);
    if (parts < 1 || scratch == nullptr) parts = 1;
#define VG_LAT(NCT, NQF) if (nct == NCT && nqf == NQF) launch_mfma<NCT, NQF>(a, qa, H, scale, block_tables, max_blocks, \
    num_pages, context_lens, query_start, S, cache_t, ol, window, sink, parts, scratch, st)
    VG_LAT(8, 4); VG_LAT(8, 6); VG_LAT(16, 8); VG_LAT(16, 12); VG_LAT(32, 16); VG_LAT(32, 20);
#undef VG_LAT
    return;
  }
  int HC = H < 8 ? H : 8;
  while (HC > 1 && (HC * a.rank > 256 * MAXACC || (size_t)(HC + KT) * (E + 1) * 4 > 56 * 1024)) --HC;
  const size_t lds = ((size_t)(HC + KT) * (E + 1) + HC * KT + 3 * HC) * sizeof(float);
  hipLaunchKernelGGL(latent_attn_kernel, dim3(a.T, (H + HC - 1) / HC), dim3(256), lds, st, a, qa, H, HC, scale,
                     block_tables, max_blocks, page, context_lens, query_start, S, ol, window, sink);
}

// Decoded tokens on the MFMA kernel: how many workgroups share a sequence's key tiles (1: no split), chosen from the
// step's shape so that the launch has about two workgroups per CU, and the scratch floats their partial results take.
int latent_attn_parts(int T, int S, int H, int rank, int rot, int f32, int page) {
  if (!mfma_takes(rank, rot, f32, page) || (int64_t)T * H > 16 * (int64_t)S) return 1;
  const int wg = (T * H + 63) / 64 + S;
  const int parts = 512 / (wg > 0 ? wg : 1);
  return parts < 2 ? 1 : (parts > 8 ? 8 : parts);
}
size_t latent_attn_part_floats(int T, int S, int H, int rank, int rot, int parts) {
  if (parts <= 1) return 0;
  int nct, nqf;
  mfma_shape(rank, rank + rot, nct, nqf);
  return (size_t)parts * ((T * H + 63) / 64 + S) * 16 * (16 * nct + 2);
}

}  // namespace vgate
