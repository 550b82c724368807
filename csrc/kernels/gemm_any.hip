// Row-major GEMM of any shape: out = epi(A W^T) with W stored [N][K] as checkpoints hold it.
//
// It serves what the fragment-packed GEMMs (gemm.hip, gemm_prefill.hip) do not take: fp32 models (true
// fp32 FMA, no reduced-precision matrix mode), sizes that are not multiples of the MFMA tile, one
// product per head (batch = blockIdx.z with strides on A, W and out), one product per expert over a
// device-side row grouping (group_off; tiles are located on the device, so the grid is fixed and
// the launch is graph-capturable), A-row gathers, and gated pairs (two weight matrices, one
// activation in the epilogue).
//   bf16: 64 x 64 block tile, 4 waves of 2 x 2 v_mfma_f32_16x16x32_bf16 tiles, operands read as 16-B
//         fragments straight from global memory (both operands are k-contiguous rows), fp32 accumulate.
//         Large aligned products (hundreds of rows, wide outputs: the expert GEMMs of a prompt portion):
//         128 x 128 block tile (a weight pair: 128 x 64 of each matrix), 4 waves of 4 x 4 MFMA tiles, k-steps of
//         32 staged through two LDS buffers, the next step's loads in flight during the current step's MFMAs.
//   fp32: 64 x 64 x 16 LDS-tiled FMA kernel, 4 x 4 outputs per thread, k ascending.
#include <cstdlib>

#include "common.h"
#include "seq_launchers.h"

namespace vgate {
namespace {

constexpr int BM = 64, BN = 64;

__device__ __forceinline__ bool locate_tile(const AnyGemmArgs& p, int by, int& grp, int& r0, int& rend, int bm = BM) {
  if (p.group_off == nullptr) {
    grp = 0; r0 = by * bm; rend = p.M;
    return r0 < p.M;
  }
  int base = 0;
  for (int g = 0; g < p.groups; ++g) {
    const int a = p.group_off[g], b = p.group_off[g + 1];
    const int nt = (b - a + bm - 1) / bm;
    if (by < base + nt) {
      grp = g; r0 = a + (by - base) * bm; rend = b;
      return true;
    }
    base += nt;
  }
  return false;
}

__device__ __forceinline__ float sigmoidf_(float x) { return 1.f / (1.f + expf(-x)); }

__device__ __forceinline__ float epi_val(const AnyGemmArgs& p, float g, float u) {
  if (p.act == 1) return g * sigmoidf_(g) * u;
  if (p.act == 2) {
    const float gg = fminf(g, p.limit);
    const float uu = fminf(fmaxf(u, -p.limit), p.limit);
    return gg * sigmoidf_(p.alpha * gg) * (uu + 1.f);
  }
  if (p.act == 3) return tanhf(g);
  if (p.act == 4) return 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))) * u;
  return g;
}

__device__ __forceinline__ void store_out(const AnyGemmArgs& p, int64_t b, int m, int n, float v) {
  if (p.gate != nullptr) {
    const int64_t gi = (int64_t)m * p.ldg + b * p.g_bs + n;
    const float gl = p.gate_f32 ? reinterpret_cast<const float*>(p.gate)[gi]
                                : bf2f(reinterpret_cast<const bf16_t*>(p.gate)[gi]);
    v *= sigmoidf_(gl);
  }
  const int64_t oi = (int64_t)m * p.ldo + b * p.o_bs + n;
  if (p.out_f32) reinterpret_cast<float*>(p.out)[oi] = v;
  else reinterpret_cast<bf16_t*>(p.out)[oi] = f2bf(v);
}

__device__ __forceinline__ bf16x8 load_frag(const bf16_t* rowp, int k, int K, bool valid) {
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

// AL: K, the row strides and the batch strides are multiples of 8 elements and the bases 16-B aligned
// (host-checked): every fragment is one unconditional 16-B load (rows / columns past the edge read a
// clamped, valid row and are dropped at the store; k past K selects zero), two k-steps are loaded before
// their MFMAs, so the loads of a wave overlap.
// NJ: 16-column tiles per wave (2: 64-column block tile; 4: 128-column block tile for wide outputs, which
// loads 1.5x fewer fragment bytes per MFMA)
// A tile with at most 32 rows (an expert's few rows of a decode step) on the aligned 64-column form: the two
// waves that would split the rows split the k range instead (k-steps of 64 in turn, so each weight fragment is
// loaded by one wave only and a wave's dependent chain of loads is half as long) and add up through LDS.
template <int DUAL, bool AL, int NJ>
__global__ __launch_bounds__(256) void gemm_any_mfma_kernel(AnyGemmArgs p) {
  constexpr bool KS = AL && NJ == 2;
  __shared__ f32x4 red[KS ? 2 : 1][KS ? (DUAL ? 8 : 4) : 1][KS ? 64 : 1];
  int grp, r0, rend;
  if (!locate_tile(p, blockIdx.y, grp, r0, rend)) return;
  const bool ks = KS && rend - r0 <= 32;  // (workgroup-uniform)
  const int64_t b = blockIdx.z;
  const int64_t wsel = (p.group_off != nullptr) ? grp : b;
  const int n0 = blockIdx.x * (32 * NJ);
  const int l = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int wm = wv & 1, wn = wv >> 1;
  const int lr = l & 15, lk = 8 * (l >> 4);
  const int mrow = ks ? 0 : wm * 32;  // first row of this wave
  const bf16_t* A = reinterpret_cast<const bf16_t*>(p.a) + b * p.a_bs;
  const bf16_t* W = reinterpret_cast<const bf16_t*>(p.w) + wsel * p.w_bs;
  const bf16_t* W2 = DUAL ? reinterpret_cast<const bf16_t*>(p.w2) + wsel * p.w_bs : nullptr;
  const bf16_t* arow[2];
  bool aval[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m = r0 + mrow + i * 16 + lr;
    aval[i] = m < rend;
    const int src = aval[i] ? (p.a_rows ? p.a_rows[m] : m) : 0;
    arow[i] = A + (int64_t)src * p.lda;
  }
  const bf16_t* wrow[NJ];
  const bf16_t* w2row[NJ];
  bool wval[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int n = n0 + wn * 16 * NJ + j * 16 + lr;
    wval[j] = n < p.N;
    wrow[j] = W + (int64_t)(wval[j] ? n : 0) * p.ldw;
    w2row[j] = DUAL ? W2 + (int64_t)(wval[j] ? n : 0) * p.ldw : nullptr;
  }
  f32x4 acc[2][NJ], acc2[2][NJ];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      acc2[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  if (AL) {
    const uint4 zero = make_uint4(0, 0, 0, 0);
    const int K = p.K;
    for (int k0 = ks ? 64 * wm : 0; k0 < K; k0 += ks ? 128 : 64) {
      uint4 av[2][2], wv_[2][NJ], uv[2][NJ];
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        const int k = k0 + 32 * st + lk;
        const int kc = min(k, K - 8);
#pragma unroll
        for (int i = 0; i < 2; ++i) av[st][i] = ld16(arow[i] + kc);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          wv_[st][j] = ld16(wrow[j] + kc);
          if (DUAL) uv[st][j] = ld16(w2row[j] + kc);
        }
      }
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        const bool in = k0 + 32 * st + lk < K;
        if (!in) {
#pragma unroll
          for (int i = 0; i < 2; ++i) av[st][i] = zero;  // a zero A fragment zeroes the product
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < NJ; ++j) {
            acc[i][j] = mfma16(as_bf16x8(av[st][i]), as_bf16x8(wv_[st][j]), acc[i][j]);
            if (DUAL) acc2[i][j] = mfma16(as_bf16x8(av[st][i]), as_bf16x8(uv[st][j]), acc2[i][j]);
          }
      }
    }
  } else
  for (int k0 = 0; k0 < p.K; k0 += 32) {
    const int k = k0 + lk;
    bf16x8 af[2], bfr[NJ], b2[NJ];
#pragma unroll
    for (int i = 0; i < 2; ++i) af[i] = load_frag(arow[i], k, p.K, aval[i]);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      bfr[j] = load_frag(wrow[j], k, p.K, wval[j]);
      if (DUAL) b2[j] = load_frag(w2row[j], k, p.K, wval[j]);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        acc[i][j] = mfma16(af[i], bfr[j], acc[i][j]);
        if (DUAL) acc2[i][j] = mfma16(af[i], b2[j], acc2[i][j]);
      }
  }
  if (KS && ks) {  // the k halves of a wave pair: wm 1 hands its sums to wm 0
    if (wm == 1) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          red[KS ? wn : 0][KS ? 2 * i + j : 0][KS ? l : 0] = acc[i][j];
          if (DUAL) red[KS ? wn : 0][KS ? 4 + 2 * i + j : 0][KS ? l : 0] = acc2[i][j];
        }
    }
    __syncthreads();
    if (wm == 1) return;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        acc[i][j] += red[KS ? wn : 0][KS ? 2 * i + j : 0][KS ? l : 0];
        if (DUAL) acc2[i][j] += red[KS ? wn : 0][KS ? 4 + 2 * i + j : 0][KS ? l : 0];
      }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int n = n0 + wn * 16 * NJ + j * 16 + lr;
      if (n >= p.N) continue;
      const float bias = p.bias ? p.bias[n] : 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int m = r0 + mrow + i * 16 + 4 * (l >> 4) + e;
        if (m >= rend) continue;
        store_out(p, b, m, n, epi_val(p, acc[i][j][e] + bias, DUAL ? acc2[i][j][e] : 0.f));
      }
    }
}

// LDS-tiled form. Host-checked: K, the row strides and the batch strides are multiples of 8 elements, the bases
// 16-B aligned, K >= 8. Block tile 128 rows x 128 weight rows (DUAL: rows 0..63 of the tile are W's, 64..127 the
// same columns of W2, so a lane holds gate and up of one output); wave (wm, wn) owns rows 64 wm .. and 4 x 4 MFMA
// tiles. A k-step's 128 x 32 A and weight tiles are two 16-B pieces per thread each; rows past the group's end
// read the tile's first row and columns past N the last one (both dropped at the store), k past K reads a
// clamped address and zeroes the A piece.
constexpr int LM = 128, LKS = 32, LPAD = LKS + 8;
template <int DUAL>
__global__ __launch_bounds__(256) void gemm_any_lds_kernel(AnyGemmArgs p) {
  constexpr int WN = DUAL ? 64 : 128;  // columns of each weight matrix per block
  __shared__ __attribute__((aligned(16))) bf16_t As[2][LM][LPAD];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[2][128][LPAD];
  int grp, r0, rend;
  if (!locate_tile(p, blockIdx.y, grp, r0, rend, LM)) return;
  const int64_t b = blockIdx.z;
  const int64_t wsel = (p.group_off != nullptr) ? grp : b;
  const int n0 = blockIdx.x * WN;
  const int tid = threadIdx.x, l = tid & 63, wv = tid >> 6;
  const int wm = wv & 1, wn = wv >> 1, lr = l & 15, lg = l >> 4;
  const bf16_t* A = reinterpret_cast<const bf16_t*>(p.a) + b * p.a_bs;
  const bf16_t* W = reinterpret_cast<const bf16_t*>(p.w) + wsel * p.w_bs;
  const bf16_t* W2 = DUAL ? reinterpret_cast<const bf16_t*>(p.w2) + wsel * p.w_bs : nullptr;
  const int K = p.K;
  const int kq = (tid & 3) * 8;  // this thread's quarter of a k-step
  const bf16_t* asrc[2];
  const bf16_t* wsrc[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int row = (tid >> 2) + 64 * u;
    const int m = r0 + row < rend ? r0 + row : r0;
    asrc[u] = A + (int64_t)(p.a_rows ? p.a_rows[m] : m) * p.lda;
    const int n = min(n0 + (DUAL ? (row & 63) : row), p.N - 1);
    wsrc[u] = ((DUAL && row >= 64) ? W2 : W) + (int64_t)n * p.ldw;
  }
  f32x4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  uint4 ar[2], wr[2];
  auto fetch = [&](int k0) {
    const int k = k0 + kq, kk = min(k, K - 8);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      ar[u] = ld16(asrc[u] + kk);
      wr[u] = ld16(wsrc[u] + kk);
      if (k >= K) ar[u] = make_uint4(0, 0, 0, 0);  // a zero A piece zeroes the product
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int row = (tid >> 2) + 64 * u;
      *reinterpret_cast<uint4*>(&As[buf][row][kq]) = ar[u];
      *reinterpret_cast<uint4*>(&Ws[buf][row][kq]) = wr[u];
    }
  };
  fetch(0);
  stage(0);
  __syncthreads();
  int buf = 0;
  // a buffer is rewritten one step later, after the barrier that every wave reaches only when it has read it
  for (int k0 = 0; k0 < K; k0 += LKS) {
    const bool more = k0 + LKS < K;
    if (more) fetch(k0 + LKS);
    bf16x8 af[4], wf[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) af[i] = as_bf16x8(*reinterpret_cast<const uint4*>(&As[buf][wm * 64 + i * 16 + lr][8 * lg]));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int wrow = DUAL ? (j >> 1) * 64 + wn * 32 + (j & 1) * 16 + lr : wn * 64 + j * 16 + lr;
      wf[j] = as_bf16x8(*reinterpret_cast<const uint4*>(&Ws[buf][wrow][8 * lg]));
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = mfma16(af[i], wf[j], acc[i][j]);
    if (more) stage(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < (DUAL ? 2 : 4); ++j) {
      const int n = n0 + (DUAL ? wn * 32 : wn * 64) + j * 16 + lr;
      if (n >= p.N) continue;
      const float bias = p.bias ? p.bias[n] : 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int m = r0 + wm * 64 + i * 16 + 4 * lg + e;
        if (m >= rend) continue;
        store_out(p, b, m, n, epi_val(p, acc[i][j][e] + bias, DUAL ? acc[i][j + 2][e] : 0.f));
      }
    }
}

template <typename T>
__device__ __forceinline__ float ldf(const T* q);
template <>
__device__ __forceinline__ float ldf<float>(const float* q) { return *q; }
template <>
__device__ __forceinline__ float ldf<bf16_t>(const bf16_t* q) { return bf2f(*q); }

constexpr int BK = 16;

template <typename T, int DUAL>
__global__ __launch_bounds__(256) void gemm_any_fma_kernel(AnyGemmArgs p) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  __shared__ float Us[DUAL ? BK : 1][BN + 4];
  int grp, r0, rend;
  if (!locate_tile(p, blockIdx.y, grp, r0, rend)) return;
  const int64_t b = blockIdx.z;
  const int64_t wsel = (p.group_off != nullptr) ? grp : b;
  const int n0 = blockIdx.x * BN;
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const T* A = reinterpret_cast<const T*>(p.a) + b * p.a_bs;
  const T* W = reinterpret_cast<const T*>(p.w) + wsel * p.w_bs;
  const T* W2 = DUAL ? reinterpret_cast<const T*>(p.w2) + wsel * p.w_bs : nullptr;
  // loader: row tid >> 2 of the tile, 4 consecutive k from (tid & 3) * 4
  const int lrow = tid >> 2, lk = (tid & 3) * 4;
  const int am = r0 + lrow;
  const bool aok = am < rend;
  const T* ap = A + (int64_t)(aok ? (p.a_rows ? p.a_rows[am] : am) : 0) * p.lda;
  const int wn_ = n0 + lrow;
  const bool wok = wn_ < p.N;
  const T* wp = W + (int64_t)(wok ? wn_ : 0) * p.ldw;
  const T* up = DUAL ? W2 + (int64_t)(wok ? wn_ : 0) * p.ldw : nullptr;
  float acc[4][4], acc2[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) { acc[i][j] = 0.f; acc2[i][j] = 0.f; }
  for (int k0 = 0; k0 < p.K; k0 += BK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      const bool kin = k < p.K;
      As[lk + e][lrow] = (aok && kin) ? ldf<T>(ap + k) : 0.f;
      Ws[lk + e][lrow] = (wok && kin) ? ldf<T>(wp + k) : 0.f;
      if (DUAL) Us[lk + e][lrow] = (wok && kin) ? ldf<T>(up + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float av[4], wv[4], uv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        wv[j] = Ws[k][tx * 4 + j];
        uv[j] = DUAL ? Us[k][tx * 4 + j] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
          if (DUAL) acc2[i][j] = fmaf(av[i], uv[j], acc2[i][j]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = r0 + ty * 4 + i;
    if (m >= rend) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= p.N) continue;
      const float bias = p.bias ? p.bias[n] : 0.f;
      store_out(p, b, m, n, epi_val(p, acc[i][j] + bias, DUAL ? acc2[i][j] : 0.f));
    }
  }
}

// "1": large products through the LDS-tiled kernel (default); "0": the direct-fragment kernels only
bool lds_tiles() {
  static const bool v = [] {
    const char* e = getenv("VGATE_GEMM_ANY_LDS");
    return e == nullptr || e[0] != '0';
  }();
  return v;
}

bool simple_only() {
  static const bool v = [] {
    const char* e = getenv("VGATE_GEMM_ANY_FMA");
    return e != nullptr && e[0] == '1';
  }();
  return v;
}

}  // namespace

void launch_gemm_any(const AnyGemmArgs& g, hipStream_t st) {
  if (g.M <= 0 || g.N <= 0 || g.batch <= 0) return;
  const int mt = (g.M + BM - 1) / BM + (g.group_off ? g.groups : 0);
  const dim3 grid((g.N + BN - 1) / BN, mt, g.batch), block(256);
  const bool dual = g.w2 != nullptr;
  if (g.in_f32) {
    if (dual) hipLaunchKernelGGL((gemm_any_fma_kernel<float, 1>), grid, block, 0, st, g);
    else hipLaunchKernelGGL((gemm_any_fma_kernel<float, 0>), grid, block, 0, st, g);
  } else if (simple_only()) {
    if (dual) hipLaunchKernelGGL((gemm_any_fma_kernel<bf16_t, 1>), grid, block, 0, st, g);
    else hipLaunchKernelGGL((gemm_any_fma_kernel<bf16_t, 0>), grid, block, 0, st, g);
  } else {
    auto a16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    const bool al = g.K >= 8 && g.K % 8 == 0 && g.lda % 8 == 0 && g.ldw % 8 == 0 && g.a_bs % 8 == 0 &&
                    g.w_bs % 8 == 0 && a16(g.a) && a16(g.w) && (!dual || a16(g.w2));
    const bool wide = al && g.N >= 512 && g.M >= 256;  // enough 64 x 128 tiles to fill the chip
    const dim3 gridw((g.N + 127) / 128, mt, g.batch);
    if (wide && g.M >= 1024 && lds_tiles()) {  // enough 128-row tiles
      const int mt128 = (g.M + LM - 1) / LM + (g.group_off ? g.groups : 0);
      if (dual) hipLaunchKernelGGL((gemm_any_lds_kernel<1>), dim3((g.N + 63) / 64, mt128, g.batch), block, 0, st, g);
      else hipLaunchKernelGGL((gemm_any_lds_kernel<0>), dim3((g.N + 127) / 128, mt128, g.batch), block, 0, st, g);
    } else if (dual && wide) hipLaunchKernelGGL((gemm_any_mfma_kernel<1, true, 4>), gridw, block, 0, st, g);
    else if (wide) hipLaunchKernelGGL((gemm_any_mfma_kernel<0, true, 4>), gridw, block, 0, st, g);
    else if (dual && al) hipLaunchKernelGGL((gemm_any_mfma_kernel<1, true, 2>), grid, block, 0, st, g);
    else if (dual) hipLaunchKernelGGL((gemm_any_mfma_kernel<1, false, 2>), grid, block, 0, st, g);
    else if (al) hipLaunchKernelGGL((gemm_any_mfma_kernel<0, true, 2>), grid, block, 0, st, g);
    else hipLaunchKernelGGL((gemm_any_mfma_kernel<0, false, 2>), grid, block, 0, st, g);
  }
}

}  // namespace vgate
