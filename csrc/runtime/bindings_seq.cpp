// Torch bindings of the hybrid-model kernels (csrc/kernels/seq_launchers.h): shapes, dtypes and strides
// are checked here, on the host, before anything is launched; every op runs on torch's current HIP
// stream and allocates nothing, so a forward pass built from them is graph-capturable.
#include <torch/extension.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/DeviceGuard.h>

#include "../kernels/seq_launchers.h"

namespace {

using torch::Tensor;
using OptT = c10::optional<Tensor>;

hipStream_t cur_stream() { return at::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

bool has(const OptT& t) { return t.has_value() && t->defined(); }

int act_f32(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
  TORCH_CHECK(t.scalar_type() == torch::kFloat32 || t.scalar_type() == torch::kBFloat16, name, ": bf16 or fp32");
  TORCH_CHECK(t.dim() == 0 || t.stride(-1) == 1, name, " must be contiguous in its last dim");
  return t.scalar_type() == torch::kFloat32 ? 1 : 0;
}

const float* f32p(const OptT& t, const char* name, int64_t n = -1) {
  if (!has(t)) return nullptr;
  TORCH_CHECK(t->is_cuda() && t->scalar_type() == torch::kFloat32 && t->is_contiguous(), name, ": contiguous fp32 GPU tensor");
  if (n >= 0) TORCH_CHECK(t->numel() == n, name, " has ", t->numel(), " elements, expected ", n);
  return t->data_ptr<float>();
}

const int32_t* i32p(const Tensor& t, const char* name, int64_t min_n) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kInt32 && t.is_contiguous(), name, ": contiguous int32 GPU tensor");
  TORCH_CHECK(t.numel() >= min_n, name, " has ", t.numel(), " elements, needs ", min_n);
  return t.data_ptr<int32_t>();
}

// a [M, K] or [B, M, K]; w (and w2) [N, K] or [B | G, N, K]; out [M, N] or [B, M, N]
void gemm_any(const Tensor& a, const Tensor& w, Tensor& out, const OptT& w2, const OptT& bias, const OptT& gate,
              const OptT& a_rows, const OptT& group_off, int64_t act, double limit, double alpha) {
  vgate::AnyGemmArgs g;
  g.in_f32 = act_f32(a, "a");
  TORCH_CHECK(act_f32(w, "w") == g.in_f32, "gemm_any: a and w must share a dtype");
  g.out_f32 = act_f32(out, "out");
  const bool b3 = a.dim() == 3;
  TORCH_CHECK((a.dim() == 2 || b3) && out.dim() == a.dim(), "gemm_any: a / out 2-D or 3-D");
  const bool grouped = has(group_off);
  const int64_t B = b3 ? a.size(0) : 1;
  g.batch = (int)B;
  g.M = (int)out.size(-2); g.N = (int)out.size(-1); g.K = (int)a.size(-1);
  g.a = a.data_ptr(); g.lda = a.stride(-2); g.a_bs = b3 ? a.stride(0) : 0;
  g.out = out.data_ptr(); g.ldo = out.stride(-2); g.o_bs = b3 ? out.stride(0) : 0;
  if (b3) TORCH_CHECK(out.size(0) == B, "gemm_any: batch of out");
  TORCH_CHECK(w.size(-1) == g.K && w.size(-2) == g.N, "gemm_any: w must be [.., N=", g.N, ", K=", g.K, "]");
  TORCH_CHECK(g.lda >= g.K && g.ldo >= g.N, "gemm_any: row strides");
  g.w = w.data_ptr(); g.ldw = w.stride(-2);
  if (w.dim() == 3) {
    g.w_bs = w.stride(0);
    TORCH_CHECK(grouped || w.size(0) == B, "gemm_any: batch of w");
  } else {
    TORCH_CHECK(w.dim() == 2 && !grouped, "gemm_any: w 2-D (3-D when batched / grouped)");
    g.w_bs = 0;
  }
  if (has(w2)) {
    TORCH_CHECK(act_f32(*w2, "w2") == g.in_f32 && w2->sizes() == w.sizes() && w2->strides() == w.strides(),
                "gemm_any: w2 must match w");
    g.w2 = w2->data_ptr();
    TORCH_CHECK(act == 1 || act == 2 || act == 4, "gemm_any: a weight pair needs act 1, 2 or 4");
  } else {
    TORCH_CHECK(act == 0 || act == 3, "gemm_any: act 1 / 2 / 4 need a weight pair");
  }
  g.bias = f32p(bias, "bias", g.N);
  TORCH_CHECK(!(g.bias && B > 1), "gemm_any: bias only without batch");
  if (has(gate)) {
    g.gate_f32 = act_f32(*gate, "gate");
    TORCH_CHECK(gate->dim() == out.dim() && gate->size(-1) == g.N && gate->size(-2) >= g.M, "gemm_any: gate shape");
    g.gate = gate->data_ptr(); g.ldg = gate->stride(-2); g.g_bs = b3 ? gate->stride(0) : 0;
  }
  const int64_t rows_in = a.size(-2);
  if (has(a_rows)) {
    g.a_rows = i32p(*a_rows, "a_rows", g.M);  // values < rows of a: produced by moe_sort from token ids
  } else {
    TORCH_CHECK(rows_in >= g.M, "gemm_any: a has ", rows_in, " rows < M=", g.M);
  }
  if (grouped) {
    TORCH_CHECK(!b3 && w.dim() == 3, "gemm_any: grouped form takes 2-D a / out and 3-D w");
    g.groups = (int)w.size(0);
    g.group_off = i32p(*group_off, "group_off", g.groups + 1);
  }
  g.act = (int)act; g.limit = (float)limit; g.alpha = (float)alpha;
  TORCH_CHECK(B <= 65535, "gemm_any: batch too large");
  c10::DeviceGuard guard(a.device());
  vgate::launch_gemm_any(g, cur_stream());
}

void norm_rows(const Tensor& x, const Tensor& w, double eps, Tensor& y, const OptT& rows, bool scalar) {
  const int xf = act_f32(x, "x"), yf = act_f32(y, "y");
  TORCH_CHECK(x.dim() == 2 && y.dim() == 2 && x.size(1) == y.size(1), "norm_rows: [M, n] rows");
  const int64_t n = x.size(1), M = y.size(0);
  const float* wp = f32p(w, "w", scalar ? 1 : n);
  const int32_t* rp = nullptr;
  if (has(rows)) rp = i32p(*rows, "rows", M);
  else TORCH_CHECK(x.size(0) >= M, "norm_rows: x rows");
  c10::DeviceGuard guard(x.device());
  vgate::launch_norm_rows(x.data_ptr(), x.stride(0), xf, rp, wp, scalar ? 1 : 0, (float)eps, y.data_ptr(), y.stride(0),
                          yf, (int)M, (int)n, cur_stream());
}

void embed_rows(const Tensor& ids, const Tensor& table, Tensor& x, const OptT& prev) {
  const int tf = act_f32(table, "table");
  TORCH_CHECK(table.dim() == 2 && table.is_contiguous(), "embed_rows: table [vocab, W]");
  TORCH_CHECK(x.is_cuda() && x.scalar_type() == torch::kFloat32 && x.is_contiguous() && x.dim() == 2 &&
              x.size(1) == table.size(1), "embed_rows: x fp32 [T, W]");
  const int T = (int)x.size(0);
  const int32_t* ip = i32p(ids, "ids", T);
  const int32_t* pp = has(prev) ? i32p(*prev, "prev", 1) : nullptr;
  c10::DeviceGuard guard(x.device());
  vgate::launch_embed_rows(ip, pp, table.data_ptr(), tf, x.data_ptr<float>(), T, (int)x.size(1), (int)table.size(0),
                           cur_stream());
}

void gated_residual(Tensor& x, const Tensor& y1, const OptT& g1, const OptT& b1, const OptT& y2, const OptT& g2,
                    const OptT& b2) {
  TORCH_CHECK(x.is_cuda() && x.scalar_type() == torch::kFloat32 && x.is_contiguous() && x.dim() == 2,
              "gated_residual: x fp32 [T, W]");
  const int T = (int)x.size(0), W = (int)x.size(1);
  const int f = act_f32(y1, "y1");
  auto chk = [&](const Tensor& t, const char* name, bool dense) {
    TORCH_CHECK(act_f32(t, name) == f && t.dim() == 2 && t.size(0) >= T && t.size(1) == W, name, ": [T, W] of y1's dtype");
    if (dense) TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
  };
  chk(y1, "y1", true);
  if (has(y2)) chk(*y2, "y2", true);
  if (has(g1)) chk(*g1, "g1", false);
  if (has(g2)) chk(*g2, "g2", false);
  TORCH_CHECK(!has(g2) || has(y2), "gated_residual: g2 without y2");
  c10::DeviceGuard guard(x.device());
  vgate::launch_gated_residual(x.data_ptr<float>(), y1.data_ptr(), has(g1) ? g1->data_ptr() : nullptr,
                               has(g1) ? g1->stride(0) : 0, f32p(b1, "b1", W), has(y2) ? y2->data_ptr() : nullptr,
                               has(g2) ? g2->data_ptr() : nullptr, has(g2) ? g2->stride(0) : 0, f32p(b2, "b2", W), f,
                               T, W, cur_stream());
}

vgate::LatentArgs latent_common(const Tensor& positions, const Tensor& inv_freq, int64_t rot_dims, int64_t rank,
                                int64_t rot, int64_t T) {
  vgate::LatentArgs a;
  a.rank = (int)rank; a.rot = (int)rot; a.rot_dims = (int)rot_dims; a.T = (int)T;
  TORCH_CHECK(rank > 0 && rot >= 0 && rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0, "latent: rank / rot sizes");
  OptT f(inv_freq);
  a.inv_freq = f32p(f, "inv_freq", rot_dims / 2);
  a.positions = i32p(positions, "positions", T);
  return a;
}

void latent_write(const Tensor& kv, const Tensor& w, double eps, const Tensor& positions, const Tensor& slots,
                  const Tensor& inv_freq, int64_t rot_dims, Tensor& cache, int64_t rank, const OptT& cache_t) {
  const int f = act_f32(kv, "kv");
  TORCH_CHECK(kv.dim() == 2 && cache.dim() == 3 && cache.is_contiguous() && act_f32(cache, "cache") == f,
              "latent_write: kv [T, rank + rot], cache [pages, page, rank + rot] of one dtype");
  const int64_t rot = kv.size(1) - rank;
  TORCH_CHECK(cache.size(2) == kv.size(1), "latent_write: cache row width");
  auto a = latent_common(positions, inv_freq, rot_dims, rank, rot, kv.size(0));
  a.slots = i32p(slots, "slots", kv.size(0));  // values < pages * page: written by the step's block tables
  a.cache = cache.data_ptr(); a.f32 = f;
  OptT wo(w);
  void* ct = nullptr;
  if (has(cache_t)) {
    TORCH_CHECK(cache_t->is_cuda() && cache_t->scalar_type() == torch::kBFloat16 && cache_t->is_contiguous() &&
                cache_t->numel() == cache.size(0) * cache.size(1) * rank, "latent_write: cache_t bf16 [pages, rank, page]");
    ct = cache_t->data_ptr();
  }
  c10::DeviceGuard guard(kv.device());
  vgate::launch_latent_write(a, kv.data_ptr(), kv.stride(0), f32p(wo, "w", rank), (float)eps, ct, (int)cache.size(1),
                             cur_stream());
}

void latent_qrope(const Tensor& q, const Tensor& positions, const Tensor& inv_freq, int64_t rot_dims, Tensor& qa,
                  int64_t H, int64_t dim, int64_t rank, int64_t rot) {
  const int f = act_f32(q, "q");
  TORCH_CHECK(q.dim() == 2 && q.is_contiguous() && q.size(1) == H * (dim + rot), "latent_qrope: q [T, H * (dim + rot)]");
  TORCH_CHECK(act_f32(qa, "qa") == f && qa.is_contiguous() && qa.numel() == q.size(0) * H * (rank + rot),
              "latent_qrope: qa [T, H, rank + rot]");
  auto a = latent_common(positions, inv_freq, rot_dims, rank, rot, q.size(0));
  a.f32 = f;
  c10::DeviceGuard guard(q.device());
  vgate::launch_latent_qrope(a, q.data_ptr(), (int)H, (int)dim, qa.data_ptr(), cur_stream());
}

void latent_attn(const Tensor& qa, const Tensor& cache, const Tensor& block_tables, const Tensor& context_lens,
                 const Tensor& query_start, Tensor& ol, double scale, int64_t H, int64_t rank, int64_t rot,
                 const OptT& cache_t, int64_t window, const OptT& sink, int64_t parts, const OptT& part_scratch) {
  const int f = act_f32(qa, "qa");
  TORCH_CHECK(window >= 1 && window <= (1 << 30), "latent_attn: window 1 .. 2^30");
  const int64_t E = rank + rot;
  TORCH_CHECK(qa.is_contiguous() && qa.numel() % (H * E) == 0, "latent_attn: qa [T, H, rank + rot]");
  const int64_t T = qa.numel() / (H * E);
  TORCH_CHECK(act_f32(ol, "ol") == f && ol.is_contiguous() && ol.numel() == T * H * rank, "latent_attn: ol [T, H, rank]");
  TORCH_CHECK(cache.dim() == 3 && cache.is_contiguous() && act_f32(cache, "cache") == f && cache.size(2) == E,
              "latent_attn: cache [pages, page, rank + rot]");
  TORCH_CHECK(rank <= 4096 && 17 * (E + 1) * 4 <= 56 * 1024, "latent_attn: latent size out of range");
  TORCH_CHECK(block_tables.dim() == 2, "latent_attn: block_tables [S, max_blocks]");
  const int64_t S = block_tables.size(0);
  vgate::LatentArgs a;
  a.rank = (int)rank; a.rot = (int)rot; a.T = (int)T; a.f32 = f; a.cache = cache.data_ptr();
  const int32_t* bt = i32p(block_tables, "block_tables", 1);
  const int32_t* cl = i32p(context_lens, "context_lens", S);
  const int32_t* qs = i32p(query_start, "query_start", S + 1);
  const void* ct = nullptr;
  if (has(cache_t)) {
    TORCH_CHECK(cache_t->is_cuda() && cache_t->scalar_type() == torch::kBFloat16 && cache_t->is_contiguous() &&
                cache_t->numel() == cache.size(0) * cache.size(1) * rank, "latent_attn: cache_t bf16 [pages, rank, page]");
    ct = cache_t->data_ptr();
  }
  float* sp = nullptr;
  if (parts > 1) {  // only what latent_attn_parts() allows for this launch, with its scratch
    TORCH_CHECK(ct != nullptr && parts == vgate::latent_attn_parts((int)T, (int)S, (int)H, (int)rank, (int)rot, f, (int)cache.size(1)),
                "latent_attn: parts must be latent_attn_split()'s for this step");
    const size_t need = vgate::latent_attn_part_floats((int)T, (int)S, (int)H, (int)rank, (int)rot, (int)parts);
    TORCH_CHECK(has(part_scratch) && part_scratch->is_cuda() && part_scratch->scalar_type() == torch::kFloat32 &&
                part_scratch->is_contiguous() && (size_t)part_scratch->numel() >= need, "latent_attn: part_scratch fp32 with ",
                need, " elements");
    sp = part_scratch->data_ptr<float>();
  }
  c10::DeviceGuard guard(qa.device());
  vgate::launch_latent_attn(a, qa.data_ptr(), (int)H, (float)scale, bt, (int)block_tables.size(1), (int)cache.size(1),
                            cl, qs, (int)S, ol.data_ptr(), ct, (int)cache.size(0), (int)window, f32p(sink, "sink", H),
                            (int)parts, sp, cur_stream());
}

void delta_rule(const Tensor& r, const Tensor& k, const Tensor& v, const Tensor& g, const Tensor& a, const Tensor& wl,
                const Tensor& w0, const Tensor& ab, const Tensor& nw, Tensor& state, const Tensor& state_slots,
                const Tensor& context_lens, const Tensor& query_start, Tensor& out, double decay_c, double unit_eps,
                double eps, Tensor& scratch) {
  vgate::DeltaArgs p;
  p.f32 = act_f32(r, "r");
  TORCH_CHECK(state.is_cuda() && state.scalar_type() == torch::kFloat32 && state.is_contiguous() && state.dim() == 4 &&
              state.size(2) == state.size(3), "delta_rule: state fp32 [slots, H, D, D]");
  p.H = (int)state.size(1); p.D = (int)state.size(2);
  TORCH_CHECK(p.D >= 1 && p.D <= 128, "delta_rule: head size 1..128");
  const int64_t HD = (int64_t)p.H * p.D;
  const int64_t T = r.size(0);
  for (const Tensor* t : {&r, &k, &v, &g, &a, &wl}) {
    TORCH_CHECK(act_f32(*t, "delta_rule input") == p.f32 && t->dim() == 2 && t->size(0) == T && t->size(1) == HD,
                "delta_rule: inputs [T, H * D] of one dtype");
  }
  for (const Tensor* t : {&k, &v, &g, &a}) TORCH_CHECK(t->stride(0) == r.stride(0), "delta_rule: one row stride");
  TORCH_CHECK(act_f32(out, "out") == p.f32 && out.dim() == 2 && out.size(0) == T && out.size(1) == HD, "delta_rule: out");
  p.r = r.data_ptr(); p.k = k.data_ptr(); p.v = v.data_ptr(); p.g = g.data_ptr(); p.a = a.data_ptr(); p.ld = r.stride(0);
  p.wl = wl.data_ptr(); p.ldw = wl.stride(0);
  OptT o0(w0), o1(ab), o2(nw);
  p.w0 = f32p(o0, "w0", HD); p.ab = f32p(o1, "ab", HD); p.nw = f32p(o2, "nw", HD);
  p.decay_c = (float)decay_c; p.unit_eps = (float)unit_eps; p.eps = (float)eps;
  p.state = state.data_ptr<float>();
  p.S = (int)state_slots.numel();
  p.state_slots = i32p(state_slots, "state_slots", p.S);  // values < slots (or -1): set by the slot manager
  p.context_lens = i32p(context_lens, "context_lens", p.S);
  p.query_start = i32p(query_start, "query_start", p.S + 1);  // values <= T: set by the step metadata
  p.out = out.data_ptr(); p.ldo = out.stride(0);
  TORCH_CHECK(scratch.is_cuda() && scratch.scalar_type() == torch::kFloat32 && scratch.is_contiguous() &&
              scratch.numel() >= 6 * T * HD, "delta_rule: scratch fp32 with T * H * D * 6 elements");
  TORCH_CHECK((reinterpret_cast<uintptr_t>(scratch.data_ptr()) & 15) == 0, "delta_rule: scratch must be 16-B aligned");
  c10::DeviceGuard guard(r.device());
  vgate::launch_delta_rule(p, (int)T, scratch.data_ptr<float>(), cur_stream());
}


void cast_rows(const Tensor& x, Tensor& y) {
  TORCH_CHECK(x.is_cuda() && x.scalar_type() == torch::kFloat32 && x.is_contiguous() && x.dim() == 2, "cast_rows: x fp32 [T, n]");
  TORCH_CHECK(y.is_cuda() && y.scalar_type() == torch::kBFloat16 && y.is_contiguous() && y.dim() == 2 &&
              y.size(1) == x.size(1) && y.size(0) <= x.size(0), "cast_rows: y bf16 [<= T, n]");
  c10::DeviceGuard guard(x.device());
  vgate::launch_cast_rows(x.data_ptr<float>(), y.data_ptr(), (int)y.size(0), (int)y.size(1), cur_stream());
}

void glu_rows(const Tensor& gu, Tensor& out, int64_t act, double limit, double alpha) {
  TORCH_CHECK(gu.is_cuda() && gu.scalar_type() == torch::kBFloat16 && gu.dim() == 2 && gu.stride(1) == 1, "glu_rows: gu bf16 [T, 2 n]");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == torch::kBFloat16 && out.dim() == 2 && out.stride(1) == 1 &&
              out.size(0) <= gu.size(0) && gu.size(1) == 2 * out.size(1), "glu_rows: out bf16 [<= T, n]");
  const int64_t n = out.size(1);
  TORCH_CHECK(n % 8 == 0 && gu.stride(0) % 8 == 0 && out.stride(0) % 8 == 0 &&
              (reinterpret_cast<uintptr_t>(gu.data_ptr()) & 15) == 0 && (reinterpret_cast<uintptr_t>(out.data_ptr()) & 15) == 0,
              "glu_rows: rows of whole 16-B pieces");
  TORCH_CHECK(act == 1 || act == 2 || act == 4, "glu_rows: act 1 (silu), 2 (clamped) or 4 (gelu_tanh)");
  c10::DeviceGuard guard(gu.device());
  vgate::launch_glu_rows(gu.data_ptr(), gu.stride(0), out.data_ptr(), out.stride(0), (int)out.size(0), (int)n, (int)act,
                         (float)limit, (float)alpha, cur_stream());
}

void residual_norm(Tensor& x, const Tensor& y, double mult, const OptT& w, double eps, const OptT& h_out) {
  TORCH_CHECK(x.is_cuda() && x.scalar_type() == torch::kFloat32 && x.is_contiguous() && x.dim() == 2, "residual_norm: x fp32 [T, W]");
  const int yf = act_f32(y, "y");
  const int64_t T = y.size(0), W = x.size(1);
  TORCH_CHECK(y.dim() == 2 && y.is_contiguous() && y.size(1) == W && T <= x.size(0), "residual_norm: y [<= T, W]");
  const float* wp = f32p(w, "w", W);
  void* hp = nullptr;
  int hf = 0;
  TORCH_CHECK(has(w) == has(h_out), "residual_norm: the norm weight and its output come together");
  if (has(h_out)) {
    hf = act_f32(*h_out, "h_out");
    TORCH_CHECK(h_out->dim() == 2 && h_out->is_contiguous() && h_out->size(1) == W && h_out->size(0) >= T, "residual_norm: h_out [T, W]");
    hp = h_out->data_ptr();
  }
  c10::DeviceGuard guard(x.device());
  vgate::launch_residual_norm(x.data_ptr<float>(), y.data_ptr(), yf, (float)mult, wp, (float)eps, hp, hf, (int)T, (int)W,
                              cur_stream());
}

void pair_rows(const Tensor& a, const Tensor& b, Tensor& out) {
  const int of = act_f32(out, "out");
  TORCH_CHECK(out.dim() == 2 && out.is_contiguous() && out.size(1) % 2 == 0, "pair_rows: out [T, 2 W]");
  const int64_t T = out.size(0), W = out.size(1) / 2;
  for (const Tensor* t : {&a, &b})
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == torch::kFloat32 && t->is_contiguous() && t->dim() == 2 && t->size(0) >= T &&
                t->size(1) == W, "pair_rows: fp32 [>= T, W] inputs");
  c10::DeviceGuard guard(out.device());
  vgate::launch_pair_rows(a.data_ptr<float>(), b.data_ptr<float>(), out.data_ptr(), of, (int)T, (int)W, cur_stream());
}

void shift_mix(const Tensor& h, Tensor& last, const Tensor& mu, const Tensor& state_slots, const Tensor& context_lens,
               const Tensor& query_start, Tensor& out) {
  const int hf = act_f32(h, "h");
  TORCH_CHECK(h.dim() == 2 && h.is_contiguous(), "shift_mix: h [T, W]");
  const int64_t T = h.size(0), W = h.size(1);
  TORCH_CHECK(last.is_cuda() && last.scalar_type() == torch::kFloat32 && last.is_contiguous() && last.dim() == 2 &&
              last.size(1) == W, "shift_mix: last fp32 [slots, W]");
  TORCH_CHECK(mu.dim() == 2 && mu.size(1) == W, "shift_mix: mu [n, W]");
  OptT mo(mu);
  const float* mp = f32p(mo, "mu", -1);
  const int64_t n = mu.size(0);
  TORCH_CHECK(act_f32(out, "out") == hf && out.dim() == 3 && out.is_contiguous() && out.size(0) == n && out.size(1) == T &&
              out.size(2) == W, "shift_mix: out [n, T, W] of h's dtype");
  const int64_t S = state_slots.numel();
  const int32_t* sp = i32p(state_slots, "state_slots", S);  // values < slots (or -1): set by the slot manager
  const int32_t* cl = i32p(context_lens, "context_lens", S);
  const int32_t* qs = i32p(query_start, "query_start", S + 1);
  c10::DeviceGuard guard(h.device());
  vgate::launch_shift_mix(h.data_ptr(), hf, last.data_ptr<float>(), mp, (int)n, sp, cl, qs, (int)S, out.data_ptr(),
                          T * W, (int)T, (int)W, cur_stream());
}

void map_pair_combine(const Tensor& a, double lam, double out_scale, double eps, const OptT& gate, Tensor& out, int64_t H,
                      int64_t G, int64_t V) {
  const int f = act_f32(a, "a");
  TORCH_CHECK(G >= 1 && H % G == 0 && V >= 1, "map_pair_combine: heads a multiple of key/value heads");
  TORCH_CHECK(out.dim() == 2 && out.is_contiguous() && act_f32(out, "out") == f && out.size(1) == H * V, "map_pair_combine: out [T, H V]");
  const int64_t T = out.size(0);
  TORCH_CHECK(a.dim() == 2 && a.is_contiguous() && a.size(0) >= T && a.size(1) == 2 * H * V, "map_pair_combine: a [T, 2 H V]");
  const void* gp = nullptr;
  int64_t ldg = 0;
  if (has(gate)) {
    TORCH_CHECK(act_f32(*gate, "gate") == f && gate->dim() == 2 && gate->size(0) >= T && gate->size(1) == H * V,
                "map_pair_combine: gate [T, H V] of a's dtype");
    gp = gate->data_ptr(); ldg = gate->stride(0);
  }
  c10::DeviceGuard guard(a.device());
  vgate::launch_map_pair_combine(a.data_ptr(), f, (float)lam, (float)out_scale, (float)eps, gp, ldg, out.data_ptr(), (int)H,
                                 (int)G, (int)V, (int)T, cur_stream());
}

void post_norm_add(const Tensor& x, const Tensor& y1, const Tensor& w, double eps, Tensor& out, double s1, const OptT& y2,
                   double s2, const OptT& act_out, const OptT& hist, int64_t planes, const OptT& coef, const OptT& mix) {
  auto f32_2d = [](const Tensor& t, const char* name) {
    TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kFloat32 && t.is_contiguous() && t.dim() == 2, name, ": fp32 [T, W]");
  };
  f32_2d(x, "x"); f32_2d(out, "out");
  vgate::PostNormArgs a;
  a.T = (int)out.size(0); a.W = (int)out.size(1);
  TORCH_CHECK(x.size(0) >= a.T && x.size(1) == a.W, "post_norm_add: x rows / width");
  a.y_f32 = act_f32(y1, "y1");
  TORCH_CHECK(y1.dim() == 2 && y1.is_contiguous() && y1.size(0) >= a.T && y1.size(1) == a.W, "post_norm_add: y1 [T, W]");
  if (has(y2)) {
    TORCH_CHECK(act_f32(*y2, "y2") == a.y_f32 && y2->dim() == 2 && y2->is_contiguous() && y2->size(0) >= a.T &&
                y2->size(1) == a.W, "post_norm_add: y2 like y1");
    a.y2 = y2->data_ptr();
  }
  OptT wo(w);
  a.x = x.data_ptr<float>(); a.y1 = y1.data_ptr(); a.w = f32p(wo, "w", a.W); a.out = out.data_ptr<float>();
  a.s1 = (float)s1; a.s2 = (float)s2; a.eps = (float)eps;
  if (has(hist)) {
    TORCH_CHECK(hist->is_cuda() && hist->scalar_type() == torch::kFloat32 && hist->dim() == 3 && hist->is_contiguous() &&
                hist->size(2) == a.W && hist->size(1) >= a.T, "post_norm_add: hist fp32 [n, T, W]");
    TORCH_CHECK(planes >= 1 && planes <= hist->size(0), "post_norm_add: planes");
    TORCH_CHECK(out.data_ptr<float>() == hist->data_ptr<float>() + (planes - 1) * hist->stride(0),
                "post_norm_add: out must be hist's plane planes - 1");
    TORCH_CHECK(has(mix) && has(coef), "post_norm_add: hist needs coef and mix");
    f32_2d(*mix, "mix");
    TORCH_CHECK(mix->size(0) >= a.T && mix->size(1) == a.W, "post_norm_add: mix rows / width");
    a.hist = hist->data_ptr<float>(); a.hist_ps = hist->stride(0); a.planes = (int)planes;
    a.coef = f32p(coef, "coef", planes); a.mix = mix->data_ptr<float>();
  }
  if (has(act_out)) {
    TORCH_CHECK(act_out->is_cuda() && act_out->scalar_type() == torch::kBFloat16 && act_out->is_contiguous() &&
                act_out->dim() == 2 && act_out->size(0) >= a.T && act_out->size(1) == a.W, "post_norm_add: act_out bf16 [T, W]");
    a.act_out = act_out->data_ptr();
  }
  c10::DeviceGuard guard(x.device());
  vgate::launch_post_norm_add(a, cur_stream());
}

// caches kc [pages, G, page, D], vc [pages, G, page, V], pooled kp / vp [pages, G, npool, D | V]
vgate::WindowArgs window_common(const Tensor& kc, const Tensor& vc, const OptT& kp, const OptT& vp, int64_t H, int64_t pool) {
  vgate::WindowArgs a;
  a.f32 = act_f32(kc, "kc");
  TORCH_CHECK(kc.dim() == 4 && vc.dim() == 4 && kc.is_contiguous() && vc.is_contiguous() && act_f32(vc, "vc") == a.f32 &&
              kc.size(0) == vc.size(0) && vc.size(1) >= 1 && kc.size(1) % vc.size(1) == 0 && kc.size(2) == vc.size(2),
              "window: kc [pages, G, page, D], vc [pages, GV, page, V] of one dtype, GV dividing G");
  a.G = (int)kc.size(1); a.page = (int)kc.size(2); a.D = (int)kc.size(3); a.V = (int)vc.size(3); a.H = (int)H;
  a.GV = (int)vc.size(1);
  TORCH_CHECK(pool == 0 || a.GV == a.G, "window: pooled blocks need one value head per key head");
  TORCH_CHECK(a.G >= 1 && H >= a.G && H % a.G == 0 && H + a.G <= 256, "window: heads a multiple of kv heads, at most 256 together");
  a.kc = kc.data_ptr(); a.vc = vc.data_ptr();
  a.pool = (int)pool;
  TORCH_CHECK(pool >= 0, "window: pool");
  if (pool > 0) {
    TORCH_CHECK(has(kp) && has(vp), "window: pooled caches missing");
    const int64_t np = (a.page + pool - 1) / pool;
    for (const Tensor* t : {&*kp, &*vp})
      TORCH_CHECK(t->dim() == 4 && t->is_contiguous() && act_f32(*t, "pooled cache") == a.f32 && t->size(0) == kc.size(0) &&
                  t->size(1) == a.G && t->size(2) == np, "window: pooled caches [pages, G, ceil(page / pool), D | V]");
    TORCH_CHECK(kp->size(3) == a.D && vp->size(3) == a.V, "window: pooled row widths");
    a.npool = (int)np; a.kp = kp->data_ptr(); a.vp = vp->data_ptr();
  }
  TORCH_CHECK(vgate::window_attn_fits(a), "window: head sizes out of the kernels' range");
  return a;
}

// the transposed bf16 value copy [pages, G, V, page] of a bf16 value cache [pages, G, page, V]
void* window_vt(const OptT& vt, const Tensor& vc) {
  if (!has(vt)) return nullptr;
  TORCH_CHECK(vc.scalar_type() == torch::kBFloat16 && vt->is_cuda() && vt->scalar_type() == torch::kBFloat16 &&
              vt->is_contiguous() && vt->dim() == 4 && vt->size(0) == vc.size(0) && vt->size(1) == vc.size(1) &&
              vt->size(2) == vc.size(3) && vt->size(3) == vc.size(2), "window: vt bf16 [pages, G, V, page] beside a bf16 vc");
  return vt->data_ptr();
}

void window_write(const Tensor& q, const Tensor& k, const Tensor& v, const OptT& qw, const OptT& kw, double eps,
                  bool norm_all, const Tensor& positions, const Tensor& slots, const Tensor& inv_freq, int64_t rot_dims,
                  const OptT& v_freq, Tensor& kc, Tensor& vc, Tensor& q_out, int64_t H, int64_t G, const OptT& vt,
                  const OptT& q_head_scale, double q_temp_coef, int64_t q_temp_every, bool rot_half) {
  auto a = window_common(kc, vc, c10::nullopt, c10::nullopt, H, 0);
  TORCH_CHECK(q_temp_every >= 1, "window_write: q_temp_every >= 1");
  TORCH_CHECK(G == a.G, "window_write: kv heads");
  const int64_t T = q.size(0);
  TORCH_CHECK(act_f32(q, "q") == a.f32 && act_f32(k, "k") == a.f32 && act_f32(v, "v") == a.f32 && q.dim() == 2 &&
              k.dim() == 2 && v.dim() == 2 && k.size(0) == T && v.size(0) == T && q.size(1) == H * a.D &&
              k.size(1) == G * a.D && v.size(1) == (int64_t)a.GV * a.V,
              "window_write: q [T, H D], k [T, G D], v [T, GV V] of the caches' dtype");
  TORCH_CHECK(act_f32(q_out, "q_out") == a.f32 && q_out.is_contiguous() && q_out.dim() == 2 && q_out.size(0) == T &&
              q_out.size(1) == H * a.D, "window_write: q_out [T, H D]");
  TORCH_CHECK(rot_dims >= 0 && rot_dims <= a.D && rot_dims % 2 == 0, "window_write: rot_dims");
  a.rot_dims = (int)rot_dims; a.T = (int)T;
  OptT fo(inv_freq);
  a.inv_freq = f32p(fo, "inv_freq", -1);
  TORCH_CHECK(inv_freq.numel() >= rot_dims / 2, "window_write: inv_freq");
  a.v_freq = f32p(v_freq, "v_freq", a.V / 2);
  a.positions = i32p(positions, "positions", T);
  a.slots = i32p(slots, "slots", T);  // values < pages * page: written from the step's block tables
  TORCH_CHECK(has(qw) == has(kw), "window_write: q / k norm weights come together");
  const float* qwp = f32p(qw, "qw", norm_all ? H * a.D : a.D);
  const float* kwp = f32p(kw, "kw", norm_all ? G * a.D : a.D);
  void* vtp = window_vt(vt, vc);
  c10::DeviceGuard guard(q.device());
  vgate::launch_window_write(a, q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), qwp, kwp,
                             (float)eps, norm_all ? 1 : 0, q_out.data_ptr(), vtp, f32p(q_head_scale, "q_head_scale", H),
                             (float)q_temp_coef, (int)q_temp_every, rot_half ? 1 : 0, cur_stream());
}

void window_seq_meta(vgate::WindowArgs& a, const Tensor& block_tables, const Tensor& query_start) {
  TORCH_CHECK(block_tables.dim() == 2, "window: block_tables [S, max_blocks]");
  a.S = (int)block_tables.size(0); a.max_blocks = (int)block_tables.size(1);
  a.block_tables = i32p(block_tables, "block_tables", 1);
  a.query_start = i32p(query_start, "query_start", a.S + 1);  // values <= T: set by the step metadata
}

void window_pool(const Tensor& kc, const Tensor& vc, const OptT& kp, const OptT& vp, const Tensor& positions,
                 const Tensor& block_tables, const Tensor& query_start, int64_t pool) {
  TORCH_CHECK(pool >= 1, "window_pool: pool >= 1");
  auto a = window_common(kc, vc, kp, vp, kc.size(1), pool);
  window_seq_meta(a, block_tables, query_start);
  a.T = (int)positions.numel();
  a.positions = i32p(positions, "positions", a.T);
  c10::DeviceGuard guard(kc.device());
  vgate::launch_window_pool(a, cur_stream());
}

void window_attn(const Tensor& q, const Tensor& kc, const Tensor& vc, const OptT& kp, const OptT& vp,
                 const Tensor& block_tables, const Tensor& context_lens, const Tensor& query_start, Tensor& out,
                 double scale, int64_t H, int64_t window, int64_t pool, const OptT& sink, const OptT& v_freq, const OptT& vt,
                 int64_t prefill_kernel, int64_t bias_kind, const OptT& bias_a, const OptT& bias_b, const OptT& gate,
                 int64_t parts, const OptT& part_scratch, double softcap) {
  auto a = window_common(kc, vc, kp, vp, H, pool);
  TORCH_CHECK(softcap >= 0.0 && (softcap == 0.0 || bias_kind == 0), "window_attn: softcap >= 0, not with a distance term");
  a.softcap = (float)softcap;
  window_seq_meta(a, block_tables, query_start);
  a.context_lens = i32p(context_lens, "context_lens", a.S);
  const int64_t T = q.size(0);
  TORCH_CHECK(act_f32(q, "q") == a.f32 && q.dim() == 2 && q.is_contiguous() && q.size(1) == H * a.D, "window_attn: q [T, H D]");
  TORCH_CHECK(act_f32(out, "out") == a.f32 && out.dim() == 2 && out.is_contiguous() && out.size(0) == T &&
              out.size(1) == H * a.V, "window_attn: out [T, H V]");
  TORCH_CHECK(window >= 1 && window <= (1 << 30), "window_attn: window 1 .. 2^30");
  a.T = (int)T; a.window = (int)window;
  TORCH_CHECK(bias_kind >= 0 && bias_kind <= 2, "window_attn: bias_kind 0 (none), 1 (log) or 2 (table)");
  a.bias_kind = (int)bias_kind;
  if (bias_kind != 0) {
    TORCH_CHECK(pool == 0, "window_attn: a distance term and pooled blocks do not combine");
    TORCH_CHECK(has(bias_a), "window_attn: bias_a missing");
    if (bias_kind == 1) {
      a.bias_a = f32p(bias_a, "bias_a", H);
      TORCH_CHECK(has(bias_b), "window_attn: bias_b missing");
      a.bias_b = f32p(bias_b, "bias_b", H);
    } else {
      TORCH_CHECK(bias_a->dim() == 2 && bias_a->size(0) == H && bias_a->size(1) >= 1 && bias_a->size(1) < (1 << 24),
                  "window_attn: distance table [H, distances]");
      a.bias_a = f32p(bias_a, "bias_a", -1);
      a.bias_n = (int)bias_a->size(1);
      a.bias_lds = (int64_t)(H / a.G) * a.bias_n * 4 <= 16 * 1024;   // beside the kernels' own tiles
    }
  }
  if (has(gate)) {
    TORCH_CHECK(act_f32(*gate, "gate") == a.f32 && gate->dim() == 2 && gate->size(0) >= T && gate->size(1) == H * a.V,
                "window_attn: gate [T, H V] of q's dtype");
    a.gate = gate->data_ptr(); a.ldg = gate->stride(0);
  }
  a.sink = f32p(sink, "sink", H);
  a.v_freq = f32p(v_freq, "v_freq", a.V / 2);
  const void* vtp = window_vt(vt, vc);
  if (parts > 1) {  // only what window_attn_parts() allows for this launch, with its scratch
    TORCH_CHECK(vtp != nullptr && parts == vgate::window_attn_parts((int)T, a.S, a.H, a.G, a.D, a.V, a.f32, a.page),
                "window_attn: parts must be window_attn_split()'s for this step");
    const size_t need = vgate::window_attn_part_floats((int)T, a.S, a.H, a.G, a.D, a.V, (int)parts);
    TORCH_CHECK(has(part_scratch) && part_scratch->is_cuda() && part_scratch->scalar_type() == torch::kFloat32 &&
                part_scratch->is_contiguous() && (size_t)part_scratch->numel() >= need, "window_attn: part_scratch fp32 with ",
                need, " elements");
    const int nct = vgate::window_attn_nct(a.D, a.V);
    const size_t slots = need / (16 * (16 * nct + 2));
    a.parts = (int)parts;
    a.part_o = part_scratch->data_ptr<float>();
    a.part_ml = a.part_o + slots * 16 * 16 * nct;
  }
  TORCH_CHECK(prefill_kernel == 0 || prefill_kernel == 1, "window_attn: prefill_kernel 0 or 1");
  a.prefill_kernel = (int)prefill_kernel;
  c10::DeviceGuard guard(q.device());
  vgate::launch_window_attn(a, q.data_ptr(), (float)scale, out.data_ptr(), vtp, (int)kc.size(0), cur_stream());
}

void linear_attn(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& g, const OptT& z, const OptT& head_decay,
                 double tau, double q_scale, bool in_silu, const OptT& nw, bool norm_all, bool gate_silu, Tensor& state,
                 const Tensor& state_slots, const Tensor& context_lens, const Tensor& query_start, Tensor& out, double eps,
                 Tensor& scratch, int64_t cols_per_lane, double k_scale, const OptT& positions, const OptT& inv_freq,
                 int64_t rot_dims, bool rot_half, bool decay_exp, const OptT& bonus, bool norm_full) {
  vgate::LinearAttnArgs p;
  TORCH_CHECK(cols_per_lane >= 0 && cols_per_lane <= 4, "linear_attn: cols_per_lane 0 (auto), 1 or 4");
  p.cols_per_lane = (int)cols_per_lane;
  p.f32 = act_f32(q, "q");
  TORCH_CHECK(state.is_cuda() && state.scalar_type() == torch::kFloat32 && state.is_contiguous() && state.dim() == 4,
              "linear_attn: state fp32 [slots, H, D, V]");
  p.H = (int)state.size(1); p.D = (int)state.size(2); p.V = (int)state.size(3);
  TORCH_CHECK(p.D >= 1 && p.D <= 256 && p.V >= 1, "linear_attn: key size 1..256");
  const int64_t T = q.size(0), HD = (int64_t)p.H * p.D, HV = (int64_t)p.H * p.V;
  auto rows = [&](const Tensor& t, int64_t n, const char* name) {
    TORCH_CHECK(act_f32(t, name) == p.f32 && t.dim() == 2 && t.size(0) == T && t.size(1) == n, "linear_attn: ", name, " [T, ", n, "]");
  };
  rows(q, HD, "q"); rows(k, HD, "k"); rows(v, HV, "v"); rows(g, HV, "g"); rows(out, HV, "out");
  p.q = q.data_ptr(); p.k = k.data_ptr(); p.v = v.data_ptr(); p.g = g.data_ptr();
  p.ldq = q.stride(0); p.ldk = k.stride(0); p.ldv = v.stride(0); p.ldg = g.stride(0);
  p.out = out.data_ptr(); p.ldo = out.stride(0);
  TORCH_CHECK(has(z) != has(head_decay), "linear_attn: either decay logits or one decay per head");
  if (has(z)) {
    TORCH_CHECK(z->is_cuda() && z->scalar_type() == torch::kFloat32 && z->dim() == 2 && z->stride(1) == 1 && z->size(0) == T &&
                z->size(1) == HD, "linear_attn: z fp32 [T, H D]");
    p.z = z->data_ptr<float>(); p.ldz = z->stride(0);
    TORCH_CHECK(tau > 0, "linear_attn: tau > 0");
  }
  p.head_decay = f32p(head_decay, "head_decay", p.H);
  TORCH_CHECK(!(norm_all && norm_full), "linear_attn: norm_full is a per-head norm");
  p.nw = f32p(nw, "nw", (norm_all || norm_full) ? HV : p.V);
  p.norm_full = norm_full ? 1 : 0;
  p.decay_exp = decay_exp ? 1 : 0;
  TORCH_CHECK(!decay_exp || has(z), "linear_attn: decay_exp needs decay logits");
  p.bonus = f32p(bonus, "bonus", HD);
  p.tau = (float)tau; p.q_scale = (float)q_scale; p.k_scale = (float)k_scale; p.eps = (float)eps;
  TORCH_CHECK(rot_dims >= 0 && rot_dims <= p.D && rot_dims % 2 == 0, "linear_attn: rot_dims even, <= key size");
  p.rot_dims = (int)rot_dims; p.rot_half = rot_half ? 1 : 0;
  if (rot_dims > 0) {
    TORCH_CHECK(has(positions) && has(inv_freq) && inv_freq->numel() >= rot_dims / 2, "linear_attn: positions / inv_freq");
    p.positions = i32p(*positions, "positions", T);
    p.inv_freq = f32p(inv_freq, "inv_freq", -1);
  }
  p.in_silu = in_silu; p.norm_all = norm_all; p.gate_silu = gate_silu;
  p.state = state.data_ptr<float>();
  p.S = (int)state_slots.numel();
  p.state_slots = i32p(state_slots, "state_slots", p.S);  // values < slots (or -1): set by the slot manager
  p.context_lens = i32p(context_lens, "context_lens", p.S);
  p.query_start = i32p(query_start, "query_start", p.S + 1);
  TORCH_CHECK(scratch.is_cuda() && scratch.scalar_type() == torch::kFloat32 && scratch.is_contiguous() &&
              (size_t)scratch.numel() >= vgate::linear_attn_scratch_floats((int)T, p.S, p.H, p.D, p.V),
              "linear_attn: scratch fp32 with linear_attn_scratch(T, S, H, D, V) elements");
  TORCH_CHECK((reinterpret_cast<uintptr_t>(scratch.data_ptr()) & 15) == 0, "linear_attn: scratch must be 16-B aligned");
  c10::DeviceGuard guard(q.device());
  vgate::launch_linear_attn(p, (int)T, scratch.data_ptr<float>(), cur_stream());
}

void moe_route(const Tensor& z, const OptT& corr, int64_t top, double norm_eps, Tensor& idx, Tensor& wts, bool softmax,
               double scale) {
  TORCH_CHECK(z.is_cuda() && z.scalar_type() == torch::kFloat32 && z.is_contiguous() && z.dim() == 2, "moe_route: z fp32 [T, E]");
  const int64_t T = z.size(0), E = z.size(1);
  TORCH_CHECK(top >= 1 && top <= E, "moe_route: top");
  TORCH_CHECK(idx.is_cuda() && idx.scalar_type() == torch::kInt32 && idx.is_contiguous() && idx.numel() == T * top, "moe_route: idx");
  TORCH_CHECK(wts.is_cuda() && wts.scalar_type() == torch::kFloat32 && wts.is_contiguous() && wts.numel() == T * top, "moe_route: wts");
  c10::DeviceGuard guard(z.device());
  vgate::launch_moe_route(z.data_ptr<float>(), f32p(corr, "corr", E), (int)T, (int)E, (int)top, (float)norm_eps,
                          softmax ? 1 : 0, (float)scale, idx.data_ptr<int32_t>(), wts.data_ptr<float>(), cur_stream());
}

void moe_sort(const Tensor& idx, int64_t E, Tensor& rows, Tensor& pos, Tensor& off) {
  TORCH_CHECK(idx.dim() == 2, "moe_sort: idx [T, top]");
  const int64_t T = idx.size(0), top = idx.size(1);
  TORCH_CHECK(E >= 1 && E <= 4096, "moe_sort: experts 1..4096");
  const int32_t* ip = i32p(idx, "idx", T * top);
  TORCH_CHECK(rows.numel() == T * top && pos.numel() == T * top && off.numel() == E + 1, "moe_sort: outputs");
  i32p(rows, "rows", 0); i32p(pos, "pos", 0); i32p(off, "off", 0);
  c10::DeviceGuard guard(idx.device());
  vgate::launch_moe_sort(ip, (int)T, (int)E, (int)top, rows.data_ptr<int32_t>(), pos.data_ptr<int32_t>(),
                         off.data_ptr<int32_t>(), cur_stream());
}

void moe_combine(const Tensor& y, const Tensor& pos, const Tensor& wts, Tensor& out, const OptT& add) {
  const int f = act_f32(y, "y"), of = act_f32(out, "out");
  TORCH_CHECK(out.dim() == 2 && out.is_contiguous() && y.is_contiguous() && y.dim() == 2 &&
              y.size(1) == out.size(1), "moe_combine: y [T * top, W], out [T, W]");
  const void* addp = nullptr;
  if (has(add)) {
    TORCH_CHECK(act_f32(*add, "add") == of && add->dim() == 2 && add->is_contiguous() && add->size(0) >= out.size(0) &&
                add->size(1) == out.size(1), "moe_combine: add [T, W] of out's dtype");
    addp = add->data_ptr();
  }
  const int64_t T = out.size(0), W = out.size(1);
  TORCH_CHECK(T > 0 && y.size(0) % T == 0, "moe_combine: rows of y");
  const int64_t top = y.size(0) / T;
  const int32_t* pp = i32p(pos, "pos", T * top);
  OptT wo(wts);
  c10::DeviceGuard guard(y.device());
  vgate::launch_moe_combine(y.data_ptr(), pp, f32p(wo, "wts", T * top), (int)T, (int)W, (int)top, f, addp, out.data_ptr(),
                            of, cur_stream());
}

void tanh_norm_rows(const Tensor& x, const Tensor& alpha, const Tensor& w, const Tensor& b, Tensor& y, const OptT& rows) {
  TORCH_CHECK(x.is_cuda() && x.scalar_type() == torch::kFloat32 && x.dim() == 2 && x.stride(1) == 1, "tanh_norm_rows: x fp32 [M, n]");
  const int yf = act_f32(y, "y");
  TORCH_CHECK(y.dim() == 2 && y.size(1) == x.size(1), "tanh_norm_rows: y [M, n]");
  const int64_t n = x.size(1), M = y.size(0);
  OptT ao(alpha), wo(w), bo(b);
  const int32_t* rp = nullptr;
  if (has(rows)) rp = i32p(*rows, "rows", M);   // values < rows of x: row numbers of the step's batch
  else TORCH_CHECK(x.size(0) >= M, "tanh_norm_rows: x rows");
  c10::DeviceGuard guard(x.device());
  vgate::launch_tanh_norm_rows(x.data_ptr<float>(), x.stride(0), rp, f32p(ao, "alpha", 1), f32p(wo, "w", n), f32p(bo, "b", n),
                               y.data_ptr(), y.stride(0), yf, (int)M, (int)n, cur_stream());
}

void hyper_mix(Tensor& xs, const OptT& y, const OptT& mix, const OptT& out_w, const OptT& read_w, const OptT& alpha,
               const OptT& w, const OptT& b, const OptT& h_out, const OptT& sum_out) {
  vgate::HyperArgs a;
  TORCH_CHECK(xs.is_cuda() && xs.scalar_type() == torch::kFloat32 && xs.dim() == 3 && xs.is_contiguous(), "hyper_mix: xs fp32 [S, T, W]");
  a.S = (int)xs.size(0); a.T = (int)xs.size(1); a.W = (int)xs.size(2);
  TORCH_CHECK(a.S >= 1 && a.S <= vgate::kMaxStreams, "hyper_mix: 1 .. ", vgate::kMaxStreams, " copies");
  a.xs = xs.data_ptr<float>(); a.plane = xs.stride(0);
  auto rows = [&](const Tensor& t, const char* name) {
    TORCH_CHECK(t.dim() == 2 && t.is_contiguous() && t.size(0) == a.T && t.size(1) == a.W, "hyper_mix: ", name, " [T, W]");
  };
  if (has(y)) {
    a.y_f32 = act_f32(*y, "y");
    rows(*y, "y");
    a.y = y->data_ptr();
    TORCH_CHECK(has(mix) && has(out_w), "hyper_mix: mix / out_w come with y");
    a.mix = f32p(mix, "mix", (int64_t)a.S * a.S);
    a.out_w = f32p(out_w, "out_w", a.S);
  }
  if (has(read_w)) {
    TORCH_CHECK(has(alpha) && has(w) && has(b) && has(h_out), "hyper_mix: alpha / w / b / h_out come with read_w");
    a.read_w = f32p(read_w, "read_w", a.S);
    a.alpha = f32p(alpha, "alpha", 1); a.w = f32p(w, "w", a.W); a.b = f32p(b, "b", a.W);
    Tensor h = *h_out;
    a.h_f32 = act_f32(h, "h_out");
    rows(h, "h_out");
    a.h_out = h.data_ptr();
  }
  if (has(sum_out)) {
    TORCH_CHECK(sum_out->is_cuda() && sum_out->scalar_type() == torch::kFloat32, "hyper_mix: sum_out fp32");
    rows(*sum_out, "sum_out");
    a.sum_out = sum_out->data_ptr<float>();
  }
  c10::DeviceGuard guard(xs.device());
  vgate::launch_hyper_mix(a, cur_stream());
}

}  // namespace

void bind_seq(pybind11::module& m) {
  namespace py = pybind11;
  m.def("gemm_any", &gemm_any, "row-major GEMM of any shape (batched / grouped / gated pair), bf16 MFMA or fp32 FMA",
        py::arg("a"), py::arg("w"), py::arg("out"), py::arg("w2") = py::none(), py::arg("bias") = py::none(),
        py::arg("gate") = py::none(), py::arg("a_rows") = py::none(), py::arg("group_off") = py::none(),
        py::arg("act") = 0, py::arg("limit") = 0.0, py::arg("alpha") = 1.702);
  m.def("norm_rows", &norm_rows, "RMS norm of rows, scalar or vector weight, fp32 statistics", py::arg("x"), py::arg("w"),
        py::arg("eps"), py::arg("y"), py::arg("rows") = py::none(), py::arg("scalar") = false);
  m.def("embed_rows", &embed_rows, "embedding gather into the fp32 residual stream", py::arg("ids"), py::arg("table"),
        py::arg("x"), py::arg("prev") = py::none());
  m.def("gated_residual", &gated_residual, "x += y1 * sigmoid(g1 + b1) + y2 * sigmoid(g2 + b2)", py::arg("x"),
        py::arg("y1"), py::arg("g1") = py::none(), py::arg("b1") = py::none(), py::arg("y2") = py::none(),
        py::arg("g2") = py::none(), py::arg("b2") = py::none());
  m.def("latent_write", &latent_write, "latent norm + shared-key rotation + paged cache store", py::arg("kv"), py::arg("w"),
        py::arg("eps"), py::arg("positions"), py::arg("slots"), py::arg("inv_freq"), py::arg("rot_dims"), py::arg("cache"),
        py::arg("rank"), py::arg("cache_t") = py::none());
  m.def("latent_qrope", &latent_qrope, "rotate the rotated query part into the absorbed query buffer");
  m.def("latent_attn", &latent_attn, "causal attention over the paged latent cache (absorbed projections)", py::arg("qa"),
        py::arg("cache"), py::arg("block_tables"), py::arg("context_lens"), py::arg("query_start"), py::arg("ol"),
        py::arg("scale"), py::arg("H"), py::arg("rank"), py::arg("rot"), py::arg("cache_t") = py::none(),
        py::arg("window") = (int64_t)1 << 30, py::arg("sink") = py::none(), py::arg("parts") = 1,
        py::arg("part_scratch") = py::none());
  m.def("latent_attn_split", [](int64_t T, int64_t S, int64_t H, int64_t rank, int64_t rot, bool f32, int64_t page) {
    const int parts = vgate::latent_attn_parts((int)T, (int)S, (int)H, (int)rank, (int)rot, f32 ? 1 : 0, (int)page);
    return std::make_pair((int64_t)parts, (int64_t)vgate::latent_attn_part_floats((int)T, (int)S, (int)H, (int)rank, (int)rot, parts));
  }, "workgroups that share a decoded token's key tiles in latent_attn, and the fp32 scratch elements they need");
  m.def("delta_rule", &delta_rule, "generalized delta rule recurrence over state slots + head norm + gate");
  m.def("cast_rows", &cast_rows, "fp32 rows rounded to bf16");
  m.def("glu_rows", &glu_rows, "out = act(gate) * up over a stacked [gate; up] projection", py::arg("gu"), py::arg("out"),
        py::arg("act"), py::arg("limit") = 0.0, py::arg("alpha") = 1.702);
  m.def("residual_norm", &residual_norm, "x += mult * y in fp32, and the RMS norm of the new rows for the next sublayer",
        py::arg("x"), py::arg("y"), py::arg("mult"), py::arg("w") = py::none(), py::arg("eps") = 0.0,
        py::arg("h_out") = py::none());
  m.def("pair_rows", &pair_rows, "two fp32 row sets side by side in the activation dtype");
  m.def("shift_mix", &shift_mix, "blends of every token's row with the row of the token before it; keeps the last row");
  m.def("map_pair_combine", &map_pair_combine, "two attention maps per head: a1 - lam a2, head RMS norm, scale, gate");
  m.def("post_norm_add", &post_norm_add, "out = x + rmsnorm(s1 y1 + s2 y2) * w, optional depth average and bf16 copy",
        py::arg("x"), py::arg("y1"), py::arg("w"), py::arg("eps"), py::arg("out"), py::arg("s1") = 1.0,
        py::arg("y2") = py::none(), py::arg("s2") = 1.0, py::arg("act_out") = py::none(), py::arg("hist") = py::none(),
        py::arg("planes") = 0, py::arg("coef") = py::none(), py::arg("mix") = py::none());
  m.def("window_write", &window_write, "q / k norm + rotation + paged key / value stores of window attention", py::arg("q"),
        py::arg("k"), py::arg("v"), py::arg("qw"), py::arg("kw"), py::arg("eps"), py::arg("norm_all"), py::arg("positions"),
        py::arg("slots"), py::arg("inv_freq"), py::arg("rot_dims"), py::arg("v_freq"), py::arg("kc"), py::arg("vc"),
        py::arg("q_out"), py::arg("H"), py::arg("G"), py::arg("vt") = py::none(), py::arg("q_head_scale") = py::none(),
        py::arg("q_temp_coef") = 0.0, py::arg("q_temp_every") = 1, py::arg("rot_half") = false);
  m.def("window_pool", &window_pool, "mean key / value rows of the blocks a step completes");
  m.def("window_attn", &window_attn, "sliding-window attention with pooled blocks and an optional sink", py::arg("q"),
        py::arg("kc"), py::arg("vc"), py::arg("kp"), py::arg("vp"), py::arg("block_tables"), py::arg("context_lens"),
        py::arg("query_start"), py::arg("out"), py::arg("scale"), py::arg("H"), py::arg("window"), py::arg("pool"),
        py::arg("sink"), py::arg("v_freq"), py::arg("vt") = py::none(), py::arg("prefill_kernel") = 0,
        py::arg("bias_kind") = 0, py::arg("bias_a") = py::none(), py::arg("bias_b") = py::none(), py::arg("gate") = py::none(),
        py::arg("parts") = 1, py::arg("part_scratch") = py::none(), py::arg("softcap") = 0.0);
  m.def("window_attn_split", [](int64_t T, int64_t S, int64_t H, int64_t G, int64_t D, int64_t V, bool f32, int64_t page) {
    const int parts = vgate::window_attn_parts((int)T, (int)S, (int)H, (int)G, (int)D, (int)V, f32 ? 1 : 0, (int)page);
    return std::make_pair((int64_t)parts, (int64_t)vgate::window_attn_part_floats((int)T, (int)S, (int)H, (int)G, (int)D, (int)V, parts));
  }, "workgroups that share a decoded token's key tiles in window_attn, and the fp32 scratch elements they need");
  m.def("linear_attn_scratch", [](int64_t T, int64_t S, int64_t H, int64_t D, int64_t V) {
    return (int64_t)vgate::linear_attn_scratch_floats((int)T, (int)S, (int)H, (int)D, (int)V);
  }, "fp32 elements of scratch a linear_attn call over T rows and S sequences needs");
  m.def("linear_attn", &linear_attn, "decayed linear attention recurrence over state slots + norm + gate", py::arg("q"),
        py::arg("k"), py::arg("v"), py::arg("g"), py::arg("z"), py::arg("head_decay"), py::arg("tau"), py::arg("q_scale"),
        py::arg("in_silu"), py::arg("nw"), py::arg("norm_all"), py::arg("gate_silu"), py::arg("state"), py::arg("state_slots"),
        py::arg("context_lens"), py::arg("query_start"), py::arg("out"), py::arg("eps"), py::arg("scratch"),
        py::arg("cols_per_lane") = 0, py::arg("k_scale") = 1.0, py::arg("positions") = py::none(),
        py::arg("inv_freq") = py::none(), py::arg("rot_dims") = 0, py::arg("rot_half") = true,
        py::arg("decay_exp") = false, py::arg("bonus") = py::none(), py::arg("norm_full") = false);
  m.def("moe_route", &moe_route, "sigmoid or softmax router: corrected top-k choice, normalised uncorrected weights, scaled",
        py::arg("z"), py::arg("corr"), py::arg("top"), py::arg("norm_eps"), py::arg("idx"), py::arg("wts"),
        py::arg("softmax") = false, py::arg("scale") = 1.0);
  m.def("tanh_norm_rows", &tanh_norm_rows, "tanh(alpha x) * w + b over (gathered) rows");
  m.def("hyper_mix", &hyper_mix, "write of a sublayer to the stream's copies + the next sublayer's normed read + their sum");
  m.def("moe_sort", &moe_sort, "counting sort of (token, choice) pairs by expert");
  m.def("moe_combine", &moe_combine, "weighted sum of a token's expert rows (+ a shared row)", py::arg("y"), py::arg("pos"),
        py::arg("wts"), py::arg("out"), py::arg("add") = py::none());
}
