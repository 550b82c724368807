// Row-wise kernels of layered hybrid models over an fp32 residual stream: embedding gather into
// fp32, RMS norm with a scalar or vector weight (fp32 statistics, bf16 or fp32 rows in and out,
// optional row gather), a tanh norm without statistics, the gated residual update of a parallel layer,
// the read / write of a sublayer over several learned-weight copies of the stream, and mixture-of-experts
// routing (sigmoid or softmax scores with an optional selection-only correction, top-k, counting sort by
// expert, weighted combine with an optional shared-expert row). Every kernel reads its sizes from arguments and its per-step metadata from device
// memory, so the launches are graph-capturable.
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
__device__ __forceinline__ float sigm(float x) { return 1.f / (1.f + expf(-x)); }

__global__ __launch_bounds__(256) void norm_rows_kernel(const void* __restrict__ x, int64_t ldx_, int x_f32,
                                                         const int32_t* __restrict__ rows,
                                                         const float* __restrict__ w, int w_scalar, float eps,
                                                         void* __restrict__ y, int64_t ldy, int y_f32, int n) {
  __shared__ float red[16];
  const int m = blockIdx.x;
  const int64_t src = rows ? rows[m] : m;
  const int64_t xo = src * ldx_;
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const float v = ldx(x, xo + c, x_f32);
    ss = fmaf(v, v, ss);
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)n + eps);
  const float ws = w_scalar ? w[0] : 1.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const float v = ldx(x, xo + c, x_f32) * inv * (w_scalar ? ws : w[c]);
    stx(y, (int64_t)m * ldy + c, y_f32, v);
  }
}

__global__ __launch_bounds__(256) void embed_rows_kernel(const int32_t* __restrict__ ids,
                                                          const int32_t* __restrict__ prev,
                                                          const void* __restrict__ table, int t_f32,
                                                          float* __restrict__ x, int W, int vocab) {
  const int t = blockIdx.x;
  int tok = ids[t];
  if (tok < 0 && prev != nullptr) tok = prev[-tok - 1];
  const bool ok = tok >= 0 && tok < vocab;
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    x[(int64_t)t * W + c] = ok ? ldx(table, (int64_t)tok * W + c, t_f32) : 0.f;
}

__global__ __launch_bounds__(256) void gated_residual_kernel(float* __restrict__ x, const void* __restrict__ y1,
                                                              const void* __restrict__ g1, int64_t ldg1,
                                                              const float* __restrict__ b1,
                                                              const void* __restrict__ y2,
                                                              const void* __restrict__ g2, int64_t ldg2,
                                                              const float* __restrict__ b2, int f32, int W) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const int64_t i = (int64_t)t * W + c;
    float v = ldx(y1, i, f32);
    if (g1 != nullptr) v *= sigm(ldx(g1, (int64_t)t * ldg1 + c, f32) + (b1 ? b1[c] : 0.f));
    if (y2 != nullptr) {
      float u = ldx(y2, i, f32);
      if (g2 != nullptr) u *= sigm(ldx(g2, (int64_t)t * ldg2 + c, f32) + (b2 ? b2[c] : 0.f));
      v += u;
    }
    x[i] += v;
  }
}

__global__ __launch_bounds__(256) void cast_rows_kernel(const float* __restrict__ x, bf16_t* __restrict__ y, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) y[i] = f2bf(x[i]);
}

// out[t][j] = act(gu[t][j]) * gu[t][n + j] for a stacked [gate; up] projection (bf16), 8 columns per thread
__global__ __launch_bounds__(256) void glu_rows_kernel(const bf16_t* __restrict__ gu, int64_t ldg, bf16_t* __restrict__ out,
                                                        int64_t ldo, int n, int act, float limit, float alpha,
                                                        int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int per = n / 8;
  const int64_t t = i / per;
  const int j = (int)(i % per) * 8;
  float g[8], u[8];
  unpack8(ld16(gu + t * ldg + j), g);
  unpack8(ld16(gu + t * ldg + n + j), u);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float x = g[e];
    if (act == 2) {  // clamped: min(g, L) * sigmoid(alpha min(g, L)) * (clamp(u, -L, L) + 1)
      x = fminf(x, limit);
      g[e] = x * sigm(alpha * x) * (fminf(fmaxf(u[e], -limit), limit) + 1.f);
      continue;
    }
    const float a = act == 4 ? 0.5f * x * (1.f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x))) : x * sigm(x);
    g[e] = a * u[e];
  }
  *reinterpret_cast<uint4*>(out + t * ldo + j) = pack8(g);
}

// one workgroup per token; every element is read and written by the same thread, so out may be x and
// mix may be x
__global__ __launch_bounds__(256) void post_norm_add_kernel(PostNormArgs a) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  const int64_t ro = (int64_t)t * a.W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < a.W; c += blockDim.x) {
    float u = a.s1 * ldx(a.y1, ro + c, a.y_f32);
    if (a.y2 != nullptr) u = fmaf(a.s2, ldx(a.y2, ro + c, a.y_f32), u);
    ss = fmaf(u, u, ss);
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)a.W + a.eps);
  for (int c = threadIdx.x; c < a.W; c += blockDim.x) {
    float u = a.s1 * ldx(a.y1, ro + c, a.y_f32);
    if (a.y2 != nullptr) u = fmaf(a.s2, ldx(a.y2, ro + c, a.y_f32), u);
    float r = a.x[ro + c] + u * inv * a.w[c];
    a.out[ro + c] = r;
    if (a.hist != nullptr) {   // depth average, planes ascending; the last plane is the row just made
      float m = 0.f;
      for (int j = 0; j + 1 < a.planes; ++j) m = fmaf(a.coef[j], a.hist[(int64_t)j * a.hist_ps + ro + c], m);
      r = fmaf(a.coef[a.planes - 1], r, m);
      a.mix[ro + c] = r;
    }
    if (a.act_out != nullptr) reinterpret_cast<bf16_t*>(a.act_out)[ro + c] = f2bf(r);
  }
}

__global__ __launch_bounds__(256) void tanh_norm_rows_kernel(const float* __restrict__ x, int64_t ldx_,
                                                              const int32_t* __restrict__ rows,
                                                              const float* __restrict__ alpha, const float* __restrict__ w,
                                                              const float* __restrict__ b, void* __restrict__ y,
                                                              int64_t ldy, int y_f32, int n) {
  const int m = blockIdx.x;
  const int64_t src = rows ? rows[m] : m;
  const float al = alpha[0];
  for (int c = threadIdx.x; c < n; c += blockDim.x)
    stx(y, (int64_t)m * ldy + c, y_f32, fmaf(tanhf(al * x[src * ldx_ + c]), w[c], b[c]));
}

// one thread per (token, column): the S <= MS copies of the element are read, mixed and written by the same thread
template <int MS>
__global__ __launch_bounds__(256) void hyper_mix_kernel(HyperArgs a) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)a.T * a.W) return;
  const int c = (int)(i % a.W);
  const int S = a.S;
  float x[MS];
#pragma unroll
  for (int s = 0; s < MS; ++s) x[s] = s < S ? a.xs[s * a.plane + i] : 0.f;
  if (a.y != nullptr) {
    const float yv = ldx(a.y, i, a.y_f32);
    float nx[MS];
#pragma unroll
    for (int t = 0; t < MS; ++t) {
      float v = 0.f;
      if (t < S) {
#pragma unroll
        for (int s = 0; s < MS; ++s)
          if (s < S) v = fmaf(a.mix[s * S + t], x[s], v);
        v = fmaf(a.out_w[t], yv, v);
        a.xs[t * a.plane + i] = v;
      }
      nx[t] = v;
    }
#pragma unroll
    for (int s = 0; s < MS; ++s) x[s] = nx[s];
  }
  if (a.read_w != nullptr) {
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < MS; ++s)
      if (s < S) u = fmaf(a.read_w[s], x[s], u);
    stx(a.h_out, i, a.h_f32, fmaf(tanhf(a.alpha[0] * u), a.w[c], a.b[c]));
  }
  if (a.sum_out != nullptr) {
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < MS; ++s)
      if (s < S) u += x[s];
    a.sum_out[i] = u;
  }
}

// one wave per token, lane l holding the scores of experts l, l + 64, .. (E <= 64 RPL): `top` (<= 64) rounds of
// a wave-wide arg-max over the corrected scores (lowest index wins a tie)
constexpr int RPL = 8;
__global__ __launch_bounds__(256) void moe_route_wave_kernel(const float* __restrict__ z, const float* __restrict__ corr,
                                                             int T, int E, int top, float norm_eps, int softmax, float scale,
                                                             int32_t* __restrict__ idx, float* __restrict__ wts) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= T) return;  // (wave-uniform)
  const float* zr = z + (int64_t)t * E;
  float s[RPL], v[RPL];
  float zmax = -INFINITY;
#pragma unroll
  for (int j = 0; j < RPL; ++j) {
    const int e = lane + 64 * j;
    s[j] = e < E ? zr[e] : -INFINITY;
    zmax = fmaxf(zmax, s[j]);
  }
  float den = 1.f;
  if (softmax) {  // scores over all experts: exp(z - max) / sum
    zmax = wave_reduce_max(zmax);
    float part = 0.f;
#pragma unroll
    for (int j = 0; j < RPL; ++j) part += lane + 64 * j < E ? expf(s[j] - zmax) : 0.f;
    den = wave_reduce_sum(part);
  }
#pragma unroll
  for (int j = 0; j < RPL; ++j) {
    const int e = lane + 64 * j;
    s[j] = softmax ? expf(s[j] - zmax) / den : sigm(s[j]);
    v[j] = e < E ? s[j] + (corr ? corr[e] : 0.f) : -INFINITY;
  }
  float sum = 0.f, mine = 0.f;
  for (int c = 0; c < top; ++c) {
    float bv = -INFINITY, bs = 0.f;
    int bi = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < RPL; ++j)   // (ascending index inside a lane: strict > keeps the lowest)
      if (lane + 64 * j < E && (bi == 0x7fffffff || v[j] > bv)) { bv = v[j]; bi = lane + 64 * j; bs = s[j]; }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64), os = __shfl_xor(bs, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; bs = os; }
    }
#pragma unroll
    for (int j = 0; j < RPL; ++j)
      if (lane + 64 * j == bi) v[j] = -INFINITY, s[j] = 0.f;   // taken (only its owner's copy matters)
    if (lane == 0) idx[(int64_t)t * top + c] = bi;
    if (lane == c) mine = bs;
    sum += bs;
  }
  if (lane < top) wts[(int64_t)t * top + lane] = mine * (1.f / (sum + norm_eps)) * scale;
}

// one thread per token: `top` rounds of arg-max over the corrected scores (lowest index wins a tie)
__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ z, const float* __restrict__ corr,
                                                        int T, int E, int top, float norm_eps, int softmax, float scale,
                                                        int32_t* __restrict__ idx, float* __restrict__ wts) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const float* zr = z + (int64_t)t * E;
  float zmax = -INFINITY, den = 1.f;
  if (softmax) {  // scores over all experts: exp(z - max) / sum
    for (int e = 0; e < E; ++e) zmax = fmaxf(zmax, zr[e]);
    den = 0.f;
    for (int e = 0; e < E; ++e) den += expf(zr[e] - zmax);
  }
  float sum = 0.f;
  for (int c = 0; c < top; ++c) {
    int best = -1;
    float bv = -INFINITY, bs = 0.f;
    for (int e = 0; e < E; ++e) {
      bool taken = false;
      for (int d = 0; d < c; ++d) taken |= idx[(int64_t)t * top + d] == e;
      if (taken) continue;
      const float s = softmax ? expf(zr[e] - zmax) / den : sigm(zr[e]);
      const float v = s + (corr ? corr[e] : 0.f);
      if (best < 0 || v > bv) { best = e; bv = v; bs = s; }
    }
    idx[(int64_t)t * top + c] = best;
    wts[(int64_t)t * top + c] = bs;
    sum += bs;
  }
  const float inv = 1.f / (sum + norm_eps);
  for (int c = 0; c < top; ++c) wts[(int64_t)t * top + c] = wts[(int64_t)t * top + c] * inv * scale;
}

// single workgroup: histogram, exclusive scan, placement (token order inside a group is arbitrary:
// every row of a grouped GEMM is computed independently of its neighbours)
__global__ __launch_bounds__(1024) void moe_sort_kernel(const int32_t* __restrict__ idx, int n, int E,
                                                         int top, int32_t* __restrict__ rows,
                                                         int32_t* __restrict__ pos, int32_t* __restrict__ off) {
  extern __shared__ int32_t cnt[];  // [E] counts, then [E] cursors
  int32_t* cur = cnt + E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) atomicAdd(&cnt[idx[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int a = 0;
    for (int e = 0; e < E; ++e) {
      off[e] = a; cur[e] = a;
      a += cnt[e];
    }
    off[E] = a;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int p = atomicAdd(&cur[idx[i]], 1);
    rows[p] = i / top;
    pos[i] = p;
  }
}

// x[t] += mult * y[t] (fp32 sum); with w: h[t] = x[t] / sqrt(mean(x[t]^2) + eps) * w from the new row. One workgroup
// per token; the row stays in registers between the add and the norm (W <= 256 * RN_MAX), else it is read again.
constexpr int RN_MAX = 16;
__global__ __launch_bounds__(256) void residual_norm_kernel(float* __restrict__ x, const void* __restrict__ y, int y_f32,
                                                             float mult, const float* __restrict__ w, float eps,
                                                             void* __restrict__ h, int h_f32, int W) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  float* xr = x + (int64_t)t * W;
  float keep[RN_MAX];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < RN_MAX; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < W) {
      const float v = fmaf(mult, ldx(y, (int64_t)t * W + c, y_f32), xr[c]);
      xr[c] = v;
      keep[i] = v;
      ss = fmaf(v, v, ss);
    }
  }
  for (int c = threadIdx.x + 256 * RN_MAX; c < W; c += 256) {
    const float v = fmaf(mult, ldx(y, (int64_t)t * W + c, y_f32), xr[c]);
    xr[c] = v;
    ss = fmaf(v, v, ss);
  }
  if (w == nullptr) return;  // (uniform)
  ss = block_reduce_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)W + eps);
#pragma unroll
  for (int i = 0; i < RN_MAX; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < W) stx(h, (int64_t)t * W + c, h_f32, keep[i] * inv * w[c]);
  }
  for (int c = threadIdx.x + 256 * RN_MAX; c < W; c += 256) stx(h, (int64_t)t * W + c, h_f32, xr[c] * inv * w[c]);
}

// out[t] = [a[t], b[t]] in out's dtype
__global__ __launch_bounds__(256) void pair_rows_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                         void* __restrict__ out, int out_f32, int W, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / (2 * W);
  const int c = (int)(i % (2 * W));
  stx(out, i, out_f32, c < W ? a[t * W + c] : b[t * W + c - W]);
}

// out[s][t] = h[t] + (h'[t] - h[t]) * mu[s], h' = the row before (the slot's kept row for a portion's first token,
// zeros at position 0). blockIdx.x: token. The slot's row is rewritten by shift_keep_kernel in a launch of its own,
// after every read of it.
__global__ __launch_bounds__(256) void shift_mix_kernel(const void* __restrict__ h, int h_f32, const float* __restrict__ last,
                                                         const float* __restrict__ mu, int n,
                                                         const int32_t* __restrict__ state_slots,
                                                         const int32_t* __restrict__ context_lens,
                                                         const int32_t* __restrict__ query_start, int S,
                                                         void* __restrict__ out, int64_t plane, int W) {
  const int t = blockIdx.x;
  if (t >= query_start[S]) return;
  int lo = 0, hi = S - 1;  // query_start[s] <= t < query_start[s + 1]
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (query_start[mid] <= t) lo = mid; else hi = mid - 1;
  }
  const int s = lo, slot = state_slots[s];
  if (slot < 0) return;
  const int t0 = query_start[s];
  const bool first = t == t0;
  const bool zero = first && context_lens[s] - (query_start[s + 1] - t0) <= 0;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float x = ldx(h, (int64_t)t * W + c, h_f32);
    const float p = zero ? 0.f : (first ? last[(int64_t)slot * W + c] : ldx(h, (int64_t)(t - 1) * W + c, h_f32));
    const float d = p - x;
    for (int k = 0; k < n; ++k) stx(out, (int64_t)k * plane + (int64_t)t * W + c, h_f32, fmaf(d, mu[(int64_t)k * W + c], x));
  }
}
__global__ __launch_bounds__(256) void shift_keep_kernel(const void* __restrict__ h, int h_f32, float* __restrict__ last,
                                                          const int32_t* __restrict__ state_slots,
                                                          const int32_t* __restrict__ query_start, int W) {
  const int s = blockIdx.x, slot = state_slots[s];
  const int t0 = query_start[s], t1 = query_start[s + 1];
  if (slot < 0 || t1 <= t0) return;
  for (int c = threadIdx.x; c < W; c += blockDim.x) last[(int64_t)slot * W + c] = ldx(h, (int64_t)(t1 - 1) * W + c, h_f32);
}

// a [T][G][2][rep][V] (two maps' results per head) -> out [T][H][V]: o = a1 - lam a2, o / sqrt(mean(o^2) + eps) * scale,
// times sigmoid(gate). One wave per (token, head).
__global__ __launch_bounds__(256) void map_pair_combine_kernel(const void* __restrict__ a, int f32, float lam, float scale,
                                                                float eps, const void* __restrict__ gate, int64_t ldg,
                                                                void* __restrict__ out, int H, int G, int V, int T) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= T * H) return;
  const int t = row / H, hd = row % H, rep = H / G, g = hd / rep, r = hd % rep;
  const int64_t a1 = (((int64_t)t * G + g) * 2 * rep + r) * V, a2 = a1 + (int64_t)rep * V;
  float ss = 0.f;
  for (int c = lane; c < V; c += 64) {
    const float o = ldx(a, a1 + c, f32) - lam * ldx(a, a2 + c, f32);
    ss = fmaf(o, o, ss);
  }
  ss = wave_reduce_sum(ss);
  const float inv = scale / sqrtf(ss / (float)V + eps);
  for (int c = lane; c < V; c += 64) {
    float o = (ldx(a, a1 + c, f32) - lam * ldx(a, a2 + c, f32)) * inv;
    if (gate != nullptr) o *= sigm(ldx(gate, (int64_t)t * ldg + (int64_t)hd * V + c, f32));
    stx(out, ((int64_t)t * H + hd) * V + c, f32, o);
  }
}

__global__ __launch_bounds__(256) void moe_combine_kernel(const void* __restrict__ y, const int32_t* __restrict__ pos,
                                                           const float* __restrict__ wts, int W, int top, int y_f32,
                                                           const void* __restrict__ add, void* __restrict__ out,
                                                           int out_f32) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float a = 0.f;
    for (int k = 0; k < top; ++k)
      a = fmaf(wts[(int64_t)t * top + k], ldx(y, (int64_t)pos[(int64_t)t * top + k] * W + c, y_f32), a);
    if (add != nullptr) a += ldx(add, (int64_t)t * W + c, out_f32);
    stx(out, (int64_t)t * W + c, out_f32, a);
  }
}

}  // namespace

void launch_cast_rows(const float* x, void* y, int T, int n, hipStream_t st) {
  const int64_t tot = (int64_t)T * n;
  if (tot <= 0) return;
  hipLaunchKernelGGL(cast_rows_kernel, dim3((unsigned)((tot + 255) / 256)), dim3(256), 0, st, x,
                     reinterpret_cast<bf16_t*>(y), tot);
}

void launch_glu_rows(const void* gu, int64_t ldg, void* out, int64_t ldo, int T, int n, int act, float limit, float alpha,
                     hipStream_t st) {
  const int64_t total = (int64_t)T * (n / 8);
  if (total <= 0) return;
  hipLaunchKernelGGL(glu_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                     reinterpret_cast<const bf16_t*>(gu), ldg, reinterpret_cast<bf16_t*>(out), ldo, n, act, limit, alpha, total);
}

void launch_residual_norm(float* x, const void* y, int y_f32, float mult, const float* w, float eps, void* h, int h_f32,
                          int T, int W, hipStream_t st) {
  if (T <= 0 || W <= 0) return;
  hipLaunchKernelGGL(residual_norm_kernel, dim3(T), dim3(256), 0, st, x, y, y_f32, mult, w, eps, h, h_f32, W);
}

void launch_pair_rows(const float* a, const float* b, void* out, int out_f32, int T, int W, hipStream_t st) {
  const int64_t total = (int64_t)T * 2 * W;
  if (total <= 0) return;
  hipLaunchKernelGGL(pair_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, a, b, out, out_f32, W, total);
}

void launch_shift_mix(const void* h, int h_f32, float* last, const float* mu, int n, const int32_t* state_slots,
                      const int32_t* context_lens, const int32_t* query_start, int S, void* out, int64_t plane, int T, int W,
                      hipStream_t st) {
  if (T <= 0 || S <= 0 || W <= 0) return;
  hipLaunchKernelGGL(shift_mix_kernel, dim3(T), dim3(256), 0, st, h, h_f32, last, mu, n, state_slots, context_lens,
                     query_start, S, out, plane, W);
  hipLaunchKernelGGL(shift_keep_kernel, dim3(S), dim3(256), 0, st, h, h_f32, last, state_slots, query_start, W);
}

void launch_map_pair_combine(const void* a, int f32, float lam, float scale, float eps, const void* gate, int64_t ldg,
                             void* out, int H, int G, int V, int T, hipStream_t st) {
  if (T <= 0 || H <= 0) return;
  hipLaunchKernelGGL(map_pair_combine_kernel, dim3((T * H + 3) / 4), dim3(256), 0, st, a, f32, lam, scale, eps, gate, ldg,
                     out, H, G, V, T);
}

void launch_post_norm_add(const PostNormArgs& a, hipStream_t st) {
  if (a.T <= 0 || a.W <= 0) return;
  hipLaunchKernelGGL(post_norm_add_kernel, dim3(a.T), dim3(256), 0, st, a);
}

void launch_norm_rows(const void* x, int64_t ldx_, int x_f32, const int32_t* rows, const float* w, int w_scalar,
                      float eps, void* y, int64_t ldy, int y_f32, int M, int n, hipStream_t st) {
  if (M <= 0) return;
  hipLaunchKernelGGL(norm_rows_kernel, dim3(M), dim3(256), 0, st, x, ldx_, x_f32, rows, w, w_scalar, eps, y, ldy,
                     y_f32, n);
}

void launch_embed_rows(const int32_t* ids, const int32_t* prev, const void* table, int t_f32, float* x, int T, int W,
                       int vocab, hipStream_t st) {
  if (T <= 0) return;
  hipLaunchKernelGGL(embed_rows_kernel, dim3(T), dim3(256), 0, st, ids, prev, table, t_f32, x, W, vocab);
}

void launch_gated_residual(float* x, const void* y1, const void* g1, int64_t ldg1, const float* b1, const void* y2,
                           const void* g2, int64_t ldg2, const float* b2, int f32, int T, int W, hipStream_t st) {
  if (T <= 0) return;
  hipLaunchKernelGGL(gated_residual_kernel, dim3(T), dim3(256), 0, st, x, y1, g1, ldg1, b1, y2, g2, ldg2, b2, f32, W);
}

void launch_moe_route(const float* z, const float* corr, int T, int E, int top, float norm_eps, int softmax, float scale,
                      int32_t* idx, float* wts, hipStream_t st) {
  if (T <= 0) return;
  if (E <= 64 * RPL && top <= 64) {
    hipLaunchKernelGGL(moe_route_wave_kernel, dim3((T + 3) / 4), dim3(256), 0, st, z, corr, T, E, top, norm_eps, softmax,
                       scale, idx, wts);
    return;
  }
  hipLaunchKernelGGL(moe_route_kernel, dim3((T + 63) / 64), dim3(64), 0, st, z, corr, T, E, top, norm_eps, softmax, scale,
                     idx, wts);
}

void launch_tanh_norm_rows(const float* x, int64_t ldx_, const int32_t* rows, const float* alpha, const float* w,
                           const float* b, void* y, int64_t ldy, int y_f32, int M, int n, hipStream_t st) {
  if (M <= 0) return;
  hipLaunchKernelGGL(tanh_norm_rows_kernel, dim3(M), dim3(256), 0, st, x, ldx_, rows, alpha, w, b, y, ldy, y_f32, n);
}

void launch_hyper_mix(const HyperArgs& a, hipStream_t st) {
  const int64_t tot = (int64_t)a.T * a.W;
  if (tot <= 0 || a.S <= 0) return;
  const dim3 grid((unsigned)((tot + 255) / 256));
  if (a.S <= 2) hipLaunchKernelGGL(hyper_mix_kernel<2>, grid, dim3(256), 0, st, a);
  else if (a.S <= 4) hipLaunchKernelGGL(hyper_mix_kernel<4>, grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL(hyper_mix_kernel<kMaxStreams>, grid, dim3(256), 0, st, a);
}

void launch_moe_sort(const int32_t* idx, int T, int E, int top, int32_t* rows, int32_t* pos, int32_t* off,
                     hipStream_t st) {
  if (T <= 0) return;
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 2 * E * sizeof(int32_t), st, idx, T * top, E, top, rows,
                     pos, off);
}

void launch_moe_combine(const void* y, const int32_t* pos, const float* wts, int T, int W, int top, int y_f32,
                        const void* add, void* out, int out_f32, hipStream_t st) {
  if (T <= 0) return;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(256), 0, st, y, pos, wts, W, top, y_f32, add, out, out_f32);
}

}  // namespace vgate
