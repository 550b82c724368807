// Host-side launcher declarations for the kernels of layered hybrid models: row-major GEMMs of any
// shape (batched per head, grouped per expert, gated-linear-unit pairs), row norms with a scalar or a
// vector weight over an fp32 residual stream, latent (compressed key/value) attention over a paged
// cache, sliding-window attention with pooled blocks and sinks over paged key / value caches, the
// generalized delta rule and decayed linear attention over per-sequence state slots, the post-norm
// residual update with depth averaging, and mixture-of-experts routing.
// Activations are bf16 or fp32 (`f32` flags); the residual stream, scores, norms and states are fp32.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vgate {

// out[b][m][n] = epi(sum_k A[b][row(m)][k] * W[g][n][k]); A, W both bf16 or both fp32 (in_f32).
struct AnyGemmArgs {
  const void* a = nullptr; int64_t lda = 0, a_bs = 0;
  const int32_t* a_rows = nullptr;      // optional gather of A rows (device)
  const void* w = nullptr; const void* w2 = nullptr;  // w2: the "up" matrix of a gated pair (same layout)
  int64_t ldw = 0, w_bs = 0;            // w_bs: stride between batches / groups
  const float* bias = nullptr;          // [N] added to the accumulator (single-matrix form)
  const void* gate = nullptr; int64_t ldg = 0, g_bs = 0;  // out *= sigmoid(gate[m][n]) (activation dtype)
  void* out = nullptr; int64_t ldo = 0, o_bs = 0;
  int M = 0, N = 0, K = 0, batch = 1;
  const int32_t* group_off = nullptr;   // [groups + 1] row ranges (device): rows of group g use W + g * w_bs
  int groups = 0;
  int act = 0;                          // 0 none; 1 silu(g) * u; 2 clamped: g' = min(g, L), u' = clamp(u, -L, L),
  float limit = 0.f;                    //   g' * sigmoid(alpha g') * (u' + 1); 3 tanh (single matrix);
                                        //   4 gelu_tanh(g) * u
  float alpha = 1.702f;
  int in_f32 = 0, out_f32 = 0, gate_f32 = 0;
};
void launch_gemm_any(const AnyGemmArgs& g, hipStream_t st);

// y[m][:] = x[row(m)][:] * rsqrt(mean(x^2) + eps) * w   (w: one number if w_scalar, else [n])
void launch_norm_rows(const void* x, int64_t ldx, int x_f32, const int32_t* rows, const float* w, int w_scalar,
                      float eps, void* y, int64_t ldy, int y_f32, int M, int n, hipStream_t st);
// x[t][:] = table[id(t)][:] as fp32; ids < 0 name the previous step's sample prev[-id - 1]
void launch_embed_rows(const int32_t* ids, const int32_t* prev, const void* table, int t_f32, float* x, int T, int W,
                       int vocab, hipStream_t st);
// x += y1 * sigmoid(g1 + b1) [+ y2 * sigmoid(g2 + b2)]; null g: plain add
void launch_gated_residual(float* x, const void* y1, const void* g1, int64_t ldg1, const float* b1, const void* y2,
                           const void* g2, int64_t ldg2, const float* b2, int f32, int T, int W, hipStream_t st);

// y = x rounded to the activation dtype (bf16), rows of n
void launch_cast_rows(const float* x, void* y, int T, int n, hipStream_t st);
// out[t][j] = act(gu[t][j]) * gu[t][n + j], j < n (bf16 rows, n % 8 == 0, 16-B aligned); act 1 silu, 4 gelu_tanh,
// 2 clamped: g' = min(g, limit), g' * sigmoid(alpha g') * (clamp(u, -limit, limit) + 1)
void launch_glu_rows(const void* gu, int64_t ldg, void* out, int64_t ldo, int T, int n, int act, float limit, float alpha,
                     hipStream_t st);
// x[t] += mult * y[t] in fp32 (x [T][W]); with w [W]: h[t] = x[t] * rsqrt(mean(x[t]^2) + eps) * w from the new row
void launch_residual_norm(float* x, const void* y, int y_f32, float mult, const float* w, float eps, void* h, int h_f32,
                          int T, int W, hipStream_t st);
// out[t] = [a[t], b[t]] (fp32 rows of W side by side) in out's dtype
void launch_pair_rows(const float* a, const float* b, void* out, int out_f32, int T, int W, hipStream_t st);
// out[k][t] = h[t] + (h'[t] - h[t]) * mu[k] for k < n blend vectors mu [n][W] (plane: stride between out's k planes),
// h' the row of the token before: h[t - 1] inside a sequence's portion, last[slot] for its first token, zeros at
// position 0; afterwards last[slot] = the portion's last row (a second launch)
void launch_shift_mix(const void* h, int h_f32, float* last, const float* mu, int n, const int32_t* state_slots,
                      const int32_t* context_lens, const int32_t* query_start, int S, void* out, int64_t plane, int T, int W,
                      hipStream_t st);
// a [T][G][2][H / G][V]: two maps' attention results per head; out [T][H][V] = (a1 - lam a2) * rsqrt(mean(.^2) + eps) *
// scale * sigmoid(gate[t][h][:]) (gate null: none)
void launch_map_pair_combine(const void* a, int f32, float lam, float scale, float eps, const void* gate, int64_t ldg,
                             void* out, int H, int G, int V, int T, hipStream_t st);
// out = x + u * rsqrt(mean(u^2) + eps) * w, u = s1 y1 [+ s2 y2] (fp32; out may alias x). With hist
// ([planes][T][W] fp32, plane stride hist_ps, whose last used plane is out): mix = sum_j coef[j] hist[j].
// act_out (bf16): a copy of mix, or of out without hist.
struct PostNormArgs {
  const float* x = nullptr; const void* y1 = nullptr; const void* y2 = nullptr; int y_f32 = 0;
  float s1 = 1.f, s2 = 1.f, eps = 0.f;
  const float* w = nullptr;
  float* out = nullptr;
  const float* hist = nullptr; int64_t hist_ps = 0; int planes = 0; const float* coef = nullptr;
  float* mix = nullptr;
  void* act_out = nullptr;
  int T = 0, W = 0;
};
void launch_post_norm_add(const PostNormArgs& a, hipStream_t st);

struct LatentArgs {
  int rank = 0, rot = 0, rot_dims = 0;  // latent size, rotated key size, leading rotated dims (<= rot, even)
  const float* inv_freq = nullptr;      // [rot_dims / 2]
  const int32_t* positions = nullptr;   // [T]
  const int32_t* slots = nullptr;       // [T] cache row of each token (-1: padding)
  void* cache = nullptr;                // [pages * page][rank + rot]
  int f32 = 0;
  int T = 0;
};
// cache[slot] = [rmsnorm(kv[:rank]) * w, rope(kv[rank:])]
// (cache_t: optional second, transposed bf16 copy of the latent part, [page][column][key in page])
void launch_latent_write(const LatentArgs& a, const void* kv, int64_t ldkv, const float* w, float eps, void* cache_t,
                         int page, hipStream_t st);
// qa[t][h][rank:] = rope(q[t][h][dim:]) for q laid out [T][H][dim + rot], qa [T][H][rank + rot]
void launch_latent_qrope(const LatentArgs& a, const void* q, int H, int dim, void* qa, hipStream_t st);
// ol[t][h][:rank] = softmax_j(scale * qa[t][h] . cache[j]) . cache[j][:rank] over the keys j with
// 0 <= position(t) - j < window; sink [H] (null: none): exp(sink[h]) is added to the softmax denominator
void launch_latent_attn(const LatentArgs& a, const void* qa, int H, float scale, const int32_t* block_tables,
                        int max_blocks, int page, const int32_t* context_lens, const int32_t* query_start, int S,
                        void* ol, const void* cache_t, int num_pages, int window, const float* sink, int parts,
                        float* scratch, hipStream_t st);
// decoded tokens on the bf16 MFMA kernel: how many workgroups share a sequence's key tiles (1: no split), and the fp32
// scratch elements launch_latent_attn then needs (parts and scratch must be these for the step's shape)
int latent_attn_parts(int T, int S, int H, int rank, int rot, int f32, int page);
size_t latent_attn_part_floats(int T, int S, int H, int rank, int rot, int parts);

struct DeltaArgs {
  const void* r = nullptr; const void* k = nullptr; const void* v = nullptr; const void* g = nullptr;
  const void* a = nullptr; int64_t ld = 0;      // rows of the fused projection (activation dtype), one stride
  const void* wl = nullptr; int64_t ldw = 0;    // decay pre-activation rows
  const float* w0 = nullptr; const float* ab = nullptr; const float* nw = nullptr;  // [H * D]
  float decay_c = 0.f, unit_eps = 0.f, eps = 0.f;
  float* state = nullptr;                       // [slots][H][D][D] (key-major)
  const int32_t* state_slots = nullptr;         // [S] (-1: padding)
  const int32_t* context_lens = nullptr; const int32_t* query_start = nullptr;
  void* out = nullptr; int64_t ldo = 0;
  int S = 0, H = 0, D = 0, f32 = 0;
};
// T rows; scratch: T * H * D * 6 floats (the prepared per-channel vectors and the raw outputs)
void launch_delta_rule(const DeltaArgs& a, int T, float* scratch, hipStream_t st);

// Sliding-window attention over paged key / value caches with optional pooled blocks (window_attn.hip).
struct WindowArgs {
  int H = 0, G = 0, D = 0, V = 0;       // query heads, key/value heads, key size, value size
  int GV = 0;                           // value heads (divides G): key head g reads value head g / (G / GV)
  float softcap = 0.f;                  // c > 0: the scaled score s becomes c tanh(s / c) (not with a distance term)
  float cap_in = 0.f, cap_out = 0.f;    // (set by launch_window_attn: 2 / c and c log2 e)
  int page = 0, npool = 0;              // tokens per page; pooled rows per page (0: no pooled caches)
  int rot_dims = 0, window = 0, pool = 0;
  int f32 = 0, T = 0, S = 0, max_blocks = 0;
  int prefill_kernel = 0;               // MFMA path, prompt portions: 0 LDS-staged tiles (64 rows), 1 split tiles (16 rows)
  const float* inv_freq = nullptr;      // [rot_dims / 2]
  const float* v_freq = nullptr;        // [V / 2]: values are turned by their position (null: not)
  const float* sink = nullptr;          // [H] logits that only enter the softmax denominator (null: none)
  // distance term of a token's score, n = query position - key position (0: none; not with pooled blocks):
  // 1: -bias_a[h] * ln(1 + bias_b[h] * n); 2: bias_a[h][min(n, bias_n - 1)]
  int bias_kind = 0, bias_n = 0, bias_lds = 0;   // bias_lds: the MFMA kernels stage a workgroup's heads' table in LDS
  const float* bias_a = nullptr; const float* bias_b = nullptr;
  const void* gate = nullptr; int64_t ldg = 0;   // [T][H * V] rows (activation dtype): out *= sigmoid(gate); null: none
  // decoded tokens, MFMA kernel: parts > 1 workgroups share a 16-row tile's keys and leave partial results in
  // part_o [parts][G][tiles][16][16 NCT] / part_ml [parts][G][tiles][16][2] for a merge launch
  int parts = 1; float* part_o = nullptr; float* part_ml = nullptr;
  const int32_t* positions = nullptr;   // [T]
  const int32_t* slots = nullptr;       // [T] page * tokens-per-page + offset of each token (-1: padding)
  const int32_t* block_tables = nullptr; const int32_t* context_lens = nullptr; const int32_t* query_start = nullptr;
  void* kc = nullptr; void* vc = nullptr;  // [pages][G][page][D], [pages][GV][page][V]
  void* kp = nullptr; void* vp = nullptr;  // [pages][G][npool][D | V]
};
size_t window_attn_lds_bytes(const WindowArgs& a, int heads_per_block);
// how many workgroups share a decoded token's key tiles (1: no split; only the bf16 MFMA kernel splits), and the
// fp32 scratch elements window_attn then needs
int window_attn_parts(int T, int S, int H, int G, int D, int V, int f32, int page);
int window_attn_nct(int D, int V);   // 16-column value tiles of the MFMA kernel instantiation for these head sizes
size_t window_attn_part_floats(int T, int S, int H, int G, int D, int V, int parts);
bool window_attn_fits(const WindowArgs& a);   // sizes the kernels' LDS and register budgets take
// q / k norm (qw, kw null: none; norm_all: one norm over the whole projection) + rotation + paged stores; q_out [T][H * D];
// the query of head h at position p is multiplied by q_head_scale[h] (null: 1) * (1 + q_temp_coef ln(floor((p + 1) / q_temp_every) + 1));
// vt: optional second, transposed bf16 copy of the values [pages][GV][V][page]; rot_half: entry i is paired with
// entry i + rot_dims / 2 instead of 2i with 2i + 1
void launch_window_write(const WindowArgs& a, const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v,
                         int64_t ldv, const float* qw, const float* kw, float eps, int norm_all, void* q_out, void* vt,
                         const float* q_head_scale, float q_temp_coef, int q_temp_every, int rot_half, hipStream_t st);
// pooled rows of the blocks this step's tokens complete
void launch_window_pool(const WindowArgs& a, hipStream_t st);
// out[t][h][:V] = softmax over (pooled blocks before the window, window tokens [, sink]) of scale q . key, times values
// (vt: optional transposed bf16 copy of the values [pages][G][V][page] that window_write keeps; with it bf16
// caches of head sizes in multiples of 8 up to 256 run the MFMA kernel)
void launch_window_attn(const WindowArgs& a, const void* q, float scale, void* out, const void* vt, int num_pages,
                        hipStream_t st);

// Linear attention with decay over per-sequence state slots (linear_attn.hip).
struct LinearAttnArgs {
  const void* q = nullptr; const void* k = nullptr; const void* v = nullptr; const void* g = nullptr;
  int64_t ldq = 0, ldk = 0, ldv = 0, ldg = 0;   // activation dtype rows: q, k [H * D]; v, g [H * V]
  const float* z = nullptr; int64_t ldz = 0;    // decay logits per key channel (null: head_decay)
  const float* head_decay = nullptr;            // [H]
  float tau = 1.f, q_scale = 1.f, k_scale = 1.f, eps = 0.f;
  int in_silu = 0, norm_all = 0, gate_silu = 0;
  // rotary positions on the leading rot_dims (even) entries of every q / k head: rot_half pairs entry i with
  // i + rot_dims / 2, otherwise 2i with 2i + 1; angle = positions[t] * inv_freq[pair]
  int rot_dims = 0, rot_half = 1;
  const float* inv_freq = nullptr;              // [rot_dims / 2]
  const int32_t* positions = nullptr;           // [T] (read when rot_dims > 0)
  const float* nw = nullptr;                    // [V], or [H * V] with norm_all; null: no weight
  float* state = nullptr;                       // [slots][H][D][V]
  const int32_t* state_slots = nullptr; const int32_t* context_lens = nullptr; const int32_t* query_start = nullptr;
  void* out = nullptr; int64_t ldo = 0;
  int S = 0, H = 0, D = 0, V = 0, f32 = 0;
  int cols_per_lane = 0;                        // value columns per lane of the scan: 0 = by the launch's size, 1, or > 1 (wide)
  int decay_exp = 0;                            // a = exp(-exp(z)) instead of sigmoid(z)^(1 / tau)
  const float* bonus = nullptr;                 // [H * D]: read the state before its update, o_t = (S + diag(bonus) k v^T)^T q
  int norm_full = 0;                            // per-head norm with a weight [H * V] (one entry per output channel)
};
// tokens per chunk a step of T rows over S sequences is scanned in (0: every sequence in one pass), the
// chunks such a step has at most, and the scratch floats it needs
int linear_attn_chunk_size(int T, int S);
int linear_attn_chunks(int T, int S, int CH);
size_t linear_attn_scratch_floats(int T, int S, int H, int D, int V);
// T rows; scratch: linear_attn_scratch_floats() floats, 16-B aligned
void launch_linear_attn(const LinearAttnArgs& a, int T, float* scratch, hipStream_t st);

// idx, wts [T][top]: the `top` largest of s + corr with s = sigmoid(z) or, with `softmax`, softmax(z) over all E;
// wts = s of the chosen / (their sum + norm_eps) * scale
void launch_moe_route(const float* z, const float* corr, int T, int E, int top, float norm_eps, int softmax, float scale,
                      int32_t* idx, float* wts, hipStream_t st);
// counting sort of the T * top (token, choice) pairs by expert: rows[p] = token, pos[t * top + c] = p,
// off[E + 1] = group boundaries
void launch_moe_sort(const int32_t* idx, int T, int E, int top, int32_t* rows, int32_t* pos, int32_t* off,
                     hipStream_t st);
// out[t] = sum_c wts[t][c] * y[pos[t][c]] [+ add[t]] (add: out's dtype)
void launch_moe_combine(const void* y, const int32_t* pos, const float* wts, int T, int W, int top, int y_f32,
                        const void* add, void* out, int out_f32, hipStream_t st);

// y[m][:] = tanh(alpha[0] * x[row(m)][:]) * w + b   (x fp32; a norm without statistics)
void launch_tanh_norm_rows(const float* x, int64_t ldx, const int32_t* rows, const float* alpha, const float* w,
                           const float* b, void* y, int64_t ldy, int y_f32, int M, int n, hipStream_t st);

// Several fp32 copies of the residual stream, xs [S][T][W] (plane stride `plane`), that a sublayer reads through
// learned weights and writes back to. One launch does a sublayer's write and the next one's read:
//   y given:      xs[t] <- sum_s mix[s][t] xs[s] + out_w[t] * y      (all copies at once from the old ones)
//   read_w given: h_out = tanh(alpha[0] * sum_s read_w[s] xs[s]) * w + b   (from the new copies)
//   sum_out given: the sum of the new copies
constexpr int kMaxStreams = 16;
struct HyperArgs {
  float* xs = nullptr; int64_t plane = 0;
  const void* y = nullptr; int y_f32 = 0;
  const float* mix = nullptr; const float* out_w = nullptr;
  const float* read_w = nullptr; const float* alpha = nullptr; const float* w = nullptr; const float* b = nullptr;
  void* h_out = nullptr; int h_f32 = 0;
  float* sum_out = nullptr;
  int S = 0, T = 0, W = 0;
};
void launch_hyper_mix(const HyperArgs& a, hipStream_t st);

}  // namespace vgate
