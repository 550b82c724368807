// Linear attention with decay: one fp32 state matrix S [key][value] per (sequence, head) kept in a state
// slot between steps,
//   S <- diag(a_t) S + k_t v_t^T,   o_t = S^T (q_scale q_t)
// with a_t either a constant per head or sigmoid(z_t)^(1 / tau) per key channel (z fp32), optionally
// silu on q, k and v, optionally rotary positions on the leading rot_dims entries of every q / k head
// (entry i paired with i + rot_dims / 2, or 2i with 2i + 1; angle = position * inv_freq in fp32) and a key
// scale after them, then an RMS norm of o (per head, or over the concatenated heads; with or without a
// weight) and an output gate silu(g) or sigmoid(g). Key and value sizes may differ.
// Variants: the decay exp(-exp(z_t)); with a bonus u [H][D] the state is read BEFORE its update and the current
// token's own outer product enters the output through u,
//   o_t = (S_(t-1) + diag(u) k_t v_t^T)^T (q_scale q_t),   then   S_t = diag(a_t) S_(t-1) + k_t v_t^T
// (PRE instantiations of the scan: the prepared vector's fourth entry is u k); a per-head norm whose weight has one
// entry per output channel. Three launches:
//   prep   (token, head) parallel: the fp32 per-channel triples {a, k_scale k, q_scale q} and the values.
//   scan   the recurrence. Column v of S depends on no other column, so a head's value columns are split
//          into slices of 8 NC and every (sequence, head, slice) is one wave: lane = (key group of eight,
//          columns c + 8 n for n < NC), ceil(D / 8) x NC state entries in registers; per token one FMA pair
//          per entry and three lane exchanges per column for o; one LDS read of a key channel's {a, k, q}
//          serves the lane's NC columns (NC = 4 when there are enough waves without the finer split, else 1). Tokens are staged through LDS, the next batch loaded into registers
//          while the current one computes. A sequence's tokens of the step run in order from the slot's
//          state; a portion that starts at position 0 starts from zero, so a reused slot needs no clearing.
//   finish token parallel: norm, norm weight, output gate, store in the activation dtype.
// Long steps (a prompt portion of hundreds of tokens) run the scan over chunks of CH tokens in parallel:
//   local   every chunk from a zero state: its local state L_c and the product A_c of its decays
//   carry   per sequence, chunk after chunk: I_0 = slot state, I_(c+1) = diag(A_c) I_c + L_c (the same
//           recurrence taken CH tokens at a time, all fp32); the slot receives the last one
//   output  every chunk again from its true initial state I_c, now writing o
// Twice the arithmetic, but a lone sequence's dependent chain is CH tokens long instead of the whole portion.
#include "common.h"
#include "seq_launchers.h"

namespace vgate {
namespace {

__device__ __forceinline__ float ldx(const void* p, int64_t i, int f32) {
  return f32 ? reinterpret_cast<const float*>(p)[i] : bf2f(reinterpret_cast<const bf16_t*>(p)[i]);
}
__device__ __forceinline__ float sigm(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x * sigm(x); }
// log(sigmoid(z)) without overflow on either side
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float xor8(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));
}

// one workgroup per token: vec[t][h][d] = {a, k, q}, vals[t][h][c] = v
__global__ __launch_bounds__(256) void linear_prep_kernel(LinearAttnArgs p, float4* __restrict__ vec,
                                                           float* __restrict__ vals) {
  const int t = blockIdx.x;
  if (t >= p.query_start[p.S]) return;  // padding rows of a graph bucket
  const int HD = p.H * p.D, HV = p.H * p.V;
  const float inv_tau = 1.f / p.tau;
  const float pos = p.rot_dims > 0 ? (float)p.positions[t] : 0.f;
  const int half = p.rot_dims >> 1;
  for (int e = threadIdx.x; e < HD; e += blockDim.x) {
    float q = ldx(p.q, (int64_t)t * p.ldq + e, p.f32), k = ldx(p.k, (int64_t)t * p.ldk + e, p.f32);
    if (p.in_silu) { q = silu_f(q); k = silu_f(k); }
    const int d = e % p.D;
    if (d < p.rot_dims) {  // the pair's other entry, then (u, v) -> (u c - v s, v c + u s)
      const bool first = p.rot_half ? d < half : !(d & 1);
      const int eo = p.rot_half ? (first ? e + half : e - half) : (e ^ 1);
      float qo = ldx(p.q, (int64_t)t * p.ldq + eo, p.f32), ko = ldx(p.k, (int64_t)t * p.ldk + eo, p.f32);
      if (p.in_silu) { qo = silu_f(qo); ko = silu_f(ko); }
      const float ang = pos * p.inv_freq[p.rot_half ? (first ? d : d - half) : (d >> 1)];
      const float cs = cosf(ang), sn = sinf(ang);
      q = first ? q * cs - qo * sn : q * cs + qo * sn;
      k = first ? k * cs - ko * sn : k * cs + ko * sn;
    }
    float a;
    if (p.z == nullptr) a = p.head_decay[e / p.D];
    else if (p.decay_exp) a = expf(-expf(p.z[(int64_t)t * p.ldz + e]));
    else a = expf(log_sigmoid(p.z[(int64_t)t * p.ldz + e]) * inv_tau);
    k *= p.k_scale;
    vec[(int64_t)t * HD + e] = make_float4(a, k, q * p.q_scale, p.bonus != nullptr ? p.bonus[e] * k : 0.f);
  }
  for (int e = threadIdx.x; e < HV; e += blockDim.x) {
    const float v = ldx(p.v, (int64_t)t * p.ldv + e, p.f32);
    vals[(int64_t)t * HV + e] = p.in_silu ? silu_f(v) : v;
  }
}

// lane = 8 * q + c: key group q of 8 (keys [q dq, (q + 1) dq) with dq = ceil(D / 8) <= DQ), value column c0 + c
// MODE 0: a sequence's whole portion from its slot. MODE 1 / 2: one chunk of CH tokens per blockIdx.x (chunks
// of all sequences numbered in order), 1 = from zero, writes the chunk's local state and decay product;
// 2 = from cstate[chunk], writes the outputs.
enum { SCAN_WHOLE = 0, SCAN_LOCAL = 1, SCAN_OUTPUT = 2 };

__device__ __forceinline__ bool locate_chunk(const LinearAttnArgs& p, int CH, int bx, int& s, int& t0, int& t1) {
  int base = 0;
  for (int i = 0; i < p.S; ++i) {
    const int a = p.query_start[i], b = p.query_start[i + 1];
    const int nc = (p.state_slots[i] < 0 || b <= a) ? 0 : (b - a + CH - 1) / CH;
    if (bx < base + nc) {
      s = i; t0 = a + (bx - base) * CH; t1 = min(b, t0 + CH);
      return true;
    }
    base += nc;
  }
  return false;
}

template <int DQ, int TC, int NC, int MODE, bool PRE>
__global__ __launch_bounds__(64) void linear_scan_kernel(LinearAttnArgs p, const float4* __restrict__ vec,
                                                          const float* __restrict__ vals, float* __restrict__ oraw,
                                                          int CH, float* __restrict__ cstate, float* __restrict__ cdecay) {
  constexpr int QV = DQ + 1;              // padded group stride: the groups' broadcast reads hit different banks
  constexpr int NE = (8 * DQ + 63) / 64;  // channels a lane stages per token
  constexpr int CW = 8 * NC;              // value columns of a wave: lane column + 8 n, n < NC
  constexpr int NVL = (TC * CW + 63) / 64;
  __shared__ float4 lv[2][TC][8 * QV];
  __shared__ float lvv[2][TC][CW];
  const int h = blockIdx.y, c0 = blockIdx.z * CW;
  int s = blockIdx.x, t0, t1;
  if (MODE == SCAN_WHOLE) {
    t0 = p.query_start[s]; t1 = p.query_start[s + 1];
    if (p.state_slots[s] < 0 || t1 <= t0) return;
  } else if (!locate_chunk(p, CH, blockIdx.x, s, t0, t1)) {
    return;
  }
  const int D = p.D, V = p.V, lane = threadIdx.x;
  const int q = lane >> 3, cl = lane & 7;
  const int dq = (D + 7) >> 3;
  const int k0 = q * dq;
  // where this block's state starts from and goes to
  float* sp = MODE == SCAN_WHOLE ? p.state + ((int64_t)p.state_slots[s] * p.H + h) * D * V
                                 : cstate + ((int64_t)blockIdx.x * p.H + h) * D * V;
  const bool from_zero = MODE == SCAN_LOCAL ||
                         (MODE == SCAN_WHOLE && p.context_lens[s] - (t1 - t0) <= 0);
  float S[DQ][NC], A[MODE == SCAN_LOCAL ? DQ : 1];
#pragma unroll
  for (int j = 0; j < DQ; ++j) {
#pragma unroll
    for (int n = 0; n < NC; ++n) {
      const int c = c0 + cl + 8 * n;
      S[j][n] = (c < V && j < dq && k0 + j < D && !from_zero) ? sp[(int64_t)(k0 + j) * V + c] : 0.f;
    }
    if (MODE == SCAN_LOCAL) A[j] = 1.f;
  }
  float4 pv[TC][NE];
  float pvv[NVL];
  auto fetch = [&](int tb) {
#pragma unroll
    for (int i = 0; i < TC; ++i)
#pragma unroll
      for (int e = 0; e < NE; ++e) {
        const int d = lane + 64 * e, t = tb + i;
        const bool ok = d < D && t < t1;
        pv[i][e] = ok ? vec[((int64_t)t * p.H + h) * D + d] : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
    for (int r = 0; r < NVL; ++r) {  // TC x CW values, lane -> (token, column)
      const int e = lane + 64 * r;
      const int t = tb + e / CW, cc = c0 + e % CW;
      pvv[r] = (e < TC * CW && t < t1 && cc < V) ? vals[((int64_t)t * p.H + h) * V + cc] : 0.f;
    }
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TC; ++i)
#pragma unroll
      for (int e = 0; e < NE; ++e) {
        const int d = lane + 64 * e;
        if (d < D) lv[buf][i][(d / dq) * QV + (d % dq)] = pv[i][e];
      }
#pragma unroll
    for (int r = 0; r < NVL; ++r) {
      const int e = lane + 64 * r;
      if (e < TC * CW) lvv[buf][e / CW][e % CW] = pvv[r];
    }
  };
  // entries of channels past D are zeroed once and never written: the token loops run DQ iterations with
  // no bounds test (a = k = q = 0 leaves S and o alone)
  for (int e = lane; e < 2 * TC * 8 * QV; e += 64) (&lv[0][0][0])[e] = make_float4(0.f, 0.f, 0.f, 0.f);
  __syncthreads();
  fetch(t0);
  put(0);
  __syncthreads();
  int buf = 0;
  for (int tb = t0; tb < t1; tb += TC) {
    const bool more = tb + TC < t1;
    if (more) fetch(tb + TC);
    const int nt = min(TC, t1 - tb);
#pragma unroll
    for (int i = 0; i < TC; ++i) {
      if (i >= nt) break;
      const float4* tv = &lv[buf][i][q * QV];
      float vv[NC], o[NC];
#pragma unroll
      for (int n = 0; n < NC; ++n) { vv[n] = lvv[buf][i][cl + 8 * n]; o[n] = 0.f; }
#pragma unroll
      for (int j = 0; j < DQ; ++j) {
        const float4 x = tv[j];  // {a, k, q, u k}: one LDS read serves the lane's NC columns
#pragma unroll
        for (int n = 0; n < NC; ++n) {
          if (PRE && MODE != SCAN_LOCAL) o[n] = fmaf(x.z, fmaf(x.w, vv[n], S[j][n]), o[n]);  // the state before its update
          S[j][n] = fmaf(x.y, vv[n], x.x * S[j][n]);
          if (!PRE && MODE != SCAN_LOCAL) o[n] = fmaf(x.z, S[j][n], o[n]);
        }
        if (MODE == SCAN_LOCAL) A[j] *= x.x;
      }
      if (MODE != SCAN_LOCAL) {
#pragma unroll
        for (int n = 0; n < NC; ++n) {
          float r = o[n];
          r += xor8(r);
          r += xor16(r);
          r += xor32(r);
          const int c = c0 + cl + 8 * n;
          if (c < V && q == 0) oraw[((int64_t)(tb + i) * p.H + h) * V + c] = r;
        }
      }
    }
    if (more) {
      put(buf ^ 1);
      __syncthreads();
      buf ^= 1;
    }
  }
  if (MODE == SCAN_OUTPUT) return;
#pragma unroll
  for (int j = 0; j < DQ; ++j)
#pragma unroll
    for (int n = 0; n < NC; ++n) {
      const int c = c0 + cl + 8 * n;
      if (c < V && j < dq && k0 + j < D) sp[(int64_t)(k0 + j) * V + c] = S[j][n];
    }
  if (MODE == SCAN_LOCAL && blockIdx.z == 0 && cl == 0) {
#pragma unroll
    for (int j = 0; j < DQ; ++j)
      if (j < dq && k0 + j < D) cdecay[((int64_t)blockIdx.x * p.H + h) * D + k0 + j] = A[MODE == SCAN_LOCAL ? j : 0];
  }
}

// one thread per (sequence, head, state entry): I_0 = slot state (zero at position 0),
// I_(c+1) = diag(A_c) I_c + L_c; cstate[c] becomes I_c, the slot the state after the last chunk
__global__ __launch_bounds__(256) void linear_carry_kernel(LinearAttnArgs p, int CH, float* __restrict__ cstate,
                                                            const float* __restrict__ cdecay) {
  const int s = blockIdx.x, h = blockIdx.y;
  const int slot = p.state_slots[s];
  const int t0 = p.query_start[s], t1 = p.query_start[s + 1];
  if (slot < 0 || t1 <= t0) return;
  int base = 0;
  for (int i = 0; i < s; ++i) {
    const int a = p.query_start[i], b = p.query_start[i + 1];
    base += (p.state_slots[i] < 0 || b <= a) ? 0 : (b - a + CH - 1) / CH;
  }
  const int nc = (t1 - t0 + CH - 1) / CH;
  const int D = p.D, V = p.V;
  const bool from_zero = p.context_lens[s] - (t1 - t0) <= 0;
  float* sp = p.state + ((int64_t)slot * p.H + h) * D * V;
  for (int e = blockIdx.z * blockDim.x + threadIdx.x; e < D * V; e += gridDim.z * blockDim.x) {
    const int k = e / V;
    float cur = from_zero ? 0.f : sp[e];
    for (int c = 0; c < nc; ++c) {
      float* cs = cstate + ((int64_t)(base + c) * p.H + h) * D * V + e;
      const float loc = *cs;
      *cs = cur;
      cur = fmaf(cdecay[((int64_t)(base + c) * p.H + h) * D + k], cur, loc);
    }
    sp[e] = cur;
  }
}

// one workgroup per token; waves take heads in turn
__global__ __launch_bounds__(256) void linear_finish_kernel(LinearAttnArgs p, const float* __restrict__ oraw) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  if (t >= p.query_start[p.S]) return;
  const int H = p.H, V = p.V, HV = H * V;
  const float* o = oraw + (int64_t)t * HV;
  auto emit = [&](int e, float y) {
    const float g = ldx(p.g, (int64_t)t * p.ldg + e, p.f32);
    y *= p.gate_silu ? silu_f(g) : sigm(g);
    const int64_t oi = (int64_t)t * p.ldo + e;
    if (p.f32) reinterpret_cast<float*>(p.out)[oi] = y;
    else reinterpret_cast<bf16_t*>(p.out)[oi] = f2bf(y);
  };
  if (p.norm_all) {
    float ss = 0.f;
    for (int e = threadIdx.x; e < HV; e += blockDim.x) ss = fmaf(o[e], o[e], ss);
    ss = block_reduce_sum(ss, red);
    const float inv = 1.f / sqrtf(ss / (float)HV + p.eps);
    for (int e = threadIdx.x; e < HV; e += blockDim.x) emit(e, o[e] * inv * (p.nw != nullptr ? p.nw[e] : 1.f));
    return;
  }
  const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int h = wv; h < H; h += 4) {
    float ss = 0.f;
    for (int c = lane; c < V; c += 64) ss = fmaf(o[h * V + c], o[h * V + c], ss);
    ss = wave_reduce_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)V + p.eps);
    for (int c = lane; c < V; c += 64)
      emit(h * V + c, o[h * V + c] * inv * (p.nw != nullptr ? p.nw[p.norm_full ? h * V + c : c] : 1.f));
  }
}

template <int DQ, int TC, int NC, bool PRE>
void launch_scan_pre(const LinearAttnArgs& a, int T, const float4* vec, const float* vals, float* oraw, int CH, float* cstate,
                 float* cdecay, hipStream_t st) {
  const int cols = (a.V + 8 * NC - 1) / (8 * NC);
  if (CH <= 0) {
    hipLaunchKernelGGL((linear_scan_kernel<DQ, TC, NC, SCAN_WHOLE, PRE>), dim3(a.S, a.H, cols), dim3(64), 0, st, a, vec, vals,
                       oraw, 0, nullptr, nullptr);
    return;
  }
  const int chunks = linear_attn_chunks(T, a.S, CH);
  hipLaunchKernelGGL((linear_scan_kernel<DQ, TC, NC, SCAN_LOCAL, false>), dim3(chunks, a.H, cols), dim3(64), 0, st, a, vec, vals,
                     oraw, CH, cstate, cdecay);
  const int ez = min(64, (a.D * a.V + 255) / 256);
  hipLaunchKernelGGL(linear_carry_kernel, dim3(a.S, a.H, ez), dim3(256), 0, st, a, CH, cstate, cdecay);
  hipLaunchKernelGGL((linear_scan_kernel<DQ, TC, NC, SCAN_OUTPUT, PRE>), dim3(chunks, a.H, cols), dim3(64), 0, st, a, vec, vals,
                     oraw, CH, cstate, cdecay);
}

template <int DQ, int TC, int NC>
void launch_scan(const LinearAttnArgs& a, int T, const float4* vec, const float* vals, float* oraw, int CH, float* cstate,
                 float* cdecay, hipStream_t st) {
  if (a.bonus != nullptr) launch_scan_pre<DQ, TC, NC, true>(a, T, vec, vals, oraw, CH, cstate, cdecay, st);
  else launch_scan_pre<DQ, TC, NC, false>(a, T, vec, vals, oraw, CH, cstate, cdecay, st);
}

}  // namespace

int linear_attn_chunk_size(int T, int S) {
  // steps of a few tokens per sequence (decoding, short portions): one pass per sequence; long ones: chunks
  return T >= 256 && T >= 64 * S ? 64 : 0;
}
int linear_attn_chunks(int T, int S, int CH) { return CH > 0 ? T / CH + S : 0; }
size_t linear_attn_scratch_floats(int T, int S, int H, int D, int V) {
  const int CH = linear_attn_chunk_size(T, S);
  return (size_t)T * H * (4 * D + 2 * V) + (size_t)linear_attn_chunks(T, S, CH) * H * D * (V + 1);
}

// scratch: linear_attn_scratch_floats(): {a, k, q, -} per key channel, the values, the raw outputs, and for
// chunked steps every chunk's state and decay product
void launch_linear_attn(const LinearAttnArgs& a, int T, float* scratch, hipStream_t st) {
  if (a.S <= 0 || a.H <= 0 || T <= 0) return;
  const int64_t nk = (int64_t)T * a.H * a.D, nv = (int64_t)T * a.H * a.V;
  float4* vec = reinterpret_cast<float4*>(scratch);
  float* vals = scratch + 4 * nk;
  float* oraw = vals + nv;
  const int CH = linear_attn_chunk_size(T, a.S);
  float* cstate = oraw + nv;
  float* cdecay = cstate + (size_t)linear_attn_chunks(T, a.S, CH) * a.H * a.D * a.V;
  hipLaunchKernelGGL(linear_prep_kernel, dim3(T), dim3(256), 0, st, a, vec, vals);
  // columns per lane: few columns -> more waves (a small batch of decoded tokens needs them to fill the chip);
  // wide values -> every LDS read of a key channel's {a, k, q} serves four columns
  const bool wide = a.cols_per_lane > 0 ? a.cols_per_lane > 1
                                        : a.V >= 32 && (int64_t)a.S * a.H * ((a.V + 31) / 32) * (CH > 0 ? T / CH + 1 : 1) >= 512;
  if (a.D <= 32) { if (wide) launch_scan<4, 8, 4>(a, T, vec, vals, oraw, CH, cstate, cdecay, st); else launch_scan<4, 8, 1>(a, T, vec, vals, oraw, CH, cstate, cdecay, st); }
  else if (a.D <= 64) { if (wide) launch_scan<8, 8, 4>(a, T, vec, vals, oraw, CH, cstate, cdecay, st); else launch_scan<8, 8, 1>(a, T, vec, vals, oraw, CH, cstate, cdecay, st); }
  else if (a.D <= 128) { if (wide) launch_scan<16, 4, 4>(a, T, vec, vals, oraw, CH, cstate, cdecay, st); else launch_scan<16, 4, 1>(a, T, vec, vals, oraw, CH, cstate, cdecay, st); }
  else { if (wide) launch_scan<32, 4, 2>(a, T, vec, vals, oraw, CH, cstate, cdecay, st); else launch_scan<32, 4, 1>(a, T, vec, vals, oraw, CH, cstate, cdecay, st); }
  hipLaunchKernelGGL(linear_finish_kernel, dim3(T), dim3(256), 0, st, a, oraw);
}

}  // namespace vgate
