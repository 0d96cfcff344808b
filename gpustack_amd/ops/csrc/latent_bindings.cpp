// Torch bindings for the fp32-residual op family (resid32.hip,
// latent_attn.hip). Every shape a kernel or its grid assumes is checked
// here on the host before the launch.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

void embed_pair_hash_launch(float*, void*, const long*, const long*, const void*, const void*, int, int, long, long, long, long, int, hipStream_t);
void rms_scale_add_launch(float*, const void*, const float*, const float*, void*, int, int, float, int, hipStream_t);
void rms_norm_f32_launch(void*, const float*, const float*, int, int, float, int, hipStream_t);
void latent_norm_store_launch(void*, const void*, long, int, const float*, const long*, int, int, int, int, long, float, int, hipStream_t);
void act_inplace_launch(void*, long, int, int, hipStream_t);
void softcap_launch(float*, long, float, hipStream_t);
void route_grouped_topk_launch(int*, float*, const float*, int, int, int, int, int, int, float, hipStream_t);
void moe_combine_launch(float*, const void*, const int*, const float*, const void*, const float*, int, int, int, int, int, int, hipStream_t);
void argmax_f32_launch(long*, const float*, int, int, hipStream_t);
void latent_attention_launch(void*, const void*, const void*, const int*, const int*, const int*, int, float, int, int, int, int, int, int, int, int, int, int, int, long, long, long, long, int, float*, float*, hipStream_t);
int latent_attn_max_rank();
void grouped_up_act_launch(void*, const void*, const void*, const int*, const int*, const int*, int, int, int, int, int, int, hipStream_t);
void grouped_down_launch(void*, const void*, const void*, const int*, const int*, int, int, int, int, hipStream_t);
int latent_attn_uses_mfma(int, int, int, int);

#define HIP_CHECK_LAST()                                                     \
  do {                                                                       \
    hipError_t e_ = hipGetLastError();                                       \
    TORCH_CHECK(e_ == hipSuccess, "HIP kernel launch failed: ",              \
                hipGetErrorString(e_));                                      \
  } while (0)

namespace {

using at::Tensor;
using OptTensor = c10::optional<Tensor>;

hipStream_t cur_stream(const Tensor& t) {
  return c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

void chk(const Tensor& t, const char* name, at::ScalarType ty) {
  TORCH_CHECK(t.is_cuda(), name, " must be on GPU");
  TORCH_CHECK(t.scalar_type() == ty, name, " has the wrong dtype");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

// bf16 -> 1, fp32 -> 0
int act_kind(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be on GPU");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
  if (t.scalar_type() == at::kBFloat16) return 1;
  TORCH_CHECK(t.scalar_type() == at::kFloat, name, " must be bf16 or fp32");
  return 0;
}

void embed_pair_hash(Tensor x, OptTensor h, Tensor tokens, Tensor prev,
                     Tensor embed, OptTensor pair, long buckets,
                     long mul_prev, long mul_cur) {
  chk(x, "x", at::kFloat);
  chk(tokens, "tokens", at::kLong);
  chk(prev, "prev", at::kLong);
  const int bf = act_kind(embed, "embed");
  TORCH_CHECK(x.dim() == 2 && embed.dim() == 2);
  const int T = x.size(0), W = x.size(1);
  TORCH_CHECK(tokens.numel() == T && prev.numel() == T && embed.size(1) == W);
  void* hp = nullptr;
  if (h.has_value()) {
    TORCH_CHECK(bf == 1, "a GEMM-dtype copy is only emitted for bf16 engines");
    chk(*h, "h", at::kBFloat16);
    TORCH_CHECK(h->numel() == x.numel());
    hp = h->data_ptr();
  }
  const void* pp = nullptr;
  if (pair.has_value()) {
    TORCH_CHECK(act_kind(*pair, "pair_table") == bf && pair->dim() == 2);
    TORCH_CHECK(buckets > 0 && pair->size(0) == buckets + 1 && pair->size(1) == W,
                "pair table must hold buckets + 1 rows of the model width");
    pp = pair->data_ptr();
  }
  // token ids are clamped to the table inside the kernel (no host sync)
  embed_pair_hash_launch(x.data_ptr<float>(), hp, tokens.data_ptr<long>(),
                         prev.data_ptr<long>(), embed.data_ptr(), pp, T, W,
                         embed.size(0), buckets, mul_prev, mul_cur, bf,
                         cur_stream(x));
  HIP_CHECK_LAST();
}

void rms_scale_add(Tensor x, Tensor a, Tensor w, OptTensor s, double eps,
                   OptTensor h) {
  chk(x, "x", at::kFloat);
  chk(w, "weight", at::kFloat);
  const int a_bf = act_kind(a, "a");
  TORCH_CHECK(x.dim() == 2 && a.sizes() == x.sizes());
  const int T = x.size(0), W = x.size(1);
  TORCH_CHECK(w.numel() == W);
  const float* sp = nullptr;
  if (s.has_value()) {
    chk(*s, "scale", at::kFloat);
    TORCH_CHECK(s->numel() == W);
    sp = s->data_ptr<float>();
  }
  void* hp = nullptr;
  if (h.has_value()) {
    chk(*h, "h", at::kBFloat16);
    TORCH_CHECK(h->numel() == x.numel());
    hp = h->data_ptr();
  }
  rms_scale_add_launch(x.data_ptr<float>(), a.data_ptr(), w.data_ptr<float>(),
                       sp, hp, T, W, (float)eps, a_bf, cur_stream(x));
  HIP_CHECK_LAST();
}

void rms_norm_f32(Tensor out, Tensor x, Tensor w, double eps) {
  chk(x, "x", at::kFloat);
  chk(w, "weight", at::kFloat);
  const int out_bf = act_kind(out, "out");
  TORCH_CHECK(x.dim() == 2 && out.sizes() == x.sizes() && w.numel() == x.size(1));
  rms_norm_f32_launch(out.data_ptr(), x.data_ptr<float>(), w.data_ptr<float>(),
                      (int)x.size(0), (int)x.size(1), (float)eps, out_bf,
                      cur_stream(x));
  HIP_CHECK_LAST();
}

void latent_norm_store(Tensor cache, Tensor src, long col0, Tensor w,
                       Tensor slots, double eps) {
  const int bf = act_kind(cache, "cache");
  TORCH_CHECK(src.is_cuda() && src.dim() == 2 && src.stride(1) == 1);
  TORCH_CHECK(src.scalar_type() == cache.scalar_type(),
              "latent source and pool must share a dtype");
  chk(w, "weight", at::kFloat);
  chk(slots, "slots", at::kLong);
  TORCH_CHECK(cache.dim() == 4 && (cache.size(1) == 1 || cache.size(1) == 2),
              "pool must be [nblocks, 1|2, BS, R]");
  const int R = cache.size(3);
  const int T = src.size(0);
  TORCH_CHECK(col0 >= 0 && col0 + R <= src.size(1) && w.numel() == R);
  TORCH_CHECK(slots.numel() == T);
  // slots outside [0, nblocks*BS) are skipped inside the kernel
  latent_norm_store_launch(cache.data_ptr(), src.data_ptr(), src.stride(0),
                           (int)col0, w.data_ptr<float>(),
                           slots.data_ptr<long>(), T, R, (int)cache.size(2),
                           (int)cache.size(1), cache.size(0) * cache.size(2),
                           (float)eps, bf, cur_stream(src));
  HIP_CHECK_LAST();
}

void latent_attention(Tensor ctx, Tensor q_lat, Tensor cache,
                      Tensor block_tables, Tensor tiles, Tensor pos32,
                      double scale, bool exact, long nsplit) {
  chk(block_tables, "block_tables", at::kInt);
  chk(tiles, "tiles", at::kInt);
  chk(pos32, "pos32", at::kInt);
  const int bf = act_kind(cache, "cache");
  // q~ and ctx: [T, H, R] views with a contiguous last axis (any row and
  // head strides), both fp32 or both bf16
  TORCH_CHECK(q_lat.is_cuda() && ctx.is_cuda() && q_lat.dim() == 3 &&
              ctx.sizes() == q_lat.sizes());
  TORCH_CHECK(q_lat.stride(2) == 1 && ctx.stride(2) == 1,
              "q_lat / ctx need a contiguous latent axis");
  TORCH_CHECK(q_lat.scalar_type() == ctx.scalar_type() &&
              (q_lat.scalar_type() == at::kFloat ||
               q_lat.scalar_type() == at::kBFloat16),
              "q_lat / ctx must both be fp32 or both bf16");
  const int io_bf = q_lat.scalar_type() == at::kBFloat16 ? 1 : 0;
  TORCH_CHECK(cache.dim() == 4 && (cache.size(1) == 1 || cache.size(1) == 2),
              "pool must be [nblocks, 1|2, BS, R]");
  const int T = q_lat.size(0), H = q_lat.size(1), R = q_lat.size(2);
  const int BS = cache.size(2);
  TORCH_CHECK(cache.size(3) == R, "pool width must equal the latent width");
  TORCH_CHECK(R >= 1 && R <= latent_attn_max_rank(), "latent width unsupported");
  TORCH_CHECK(block_tables.dim() == 2 && tiles.dim() == 2 && tiles.size(1) == 6);
  TORCH_CHECK(pos32.numel() == T && block_tables.size(1) >= 1);
  const bool mfma = !exact && latent_attn_uses_mfma(bf, (int)cache.size(1), BS, R);
  TORCH_CHECK(mfma || !io_bf, "bf16 q_lat / ctx need the MFMA path");
  if (!mfma) nsplit = 1;
  TORCH_CHECK(nsplit >= 1 && nsplit <= 64);
  const int ntiles = tiles.size(0);
  Tensor ws_acc, ws_ml;
  float *wa = nullptr, *wm = nullptr;
  if (nsplit > 1 && ntiles > 0) {
    auto opt = at::TensorOptions().dtype(at::kFloat).device(q_lat.device());
    ws_acc = at::empty({(long)ntiles * nsplit * 16 * R}, opt);
    ws_ml = at::empty({(long)ntiles * nsplit * 16 * 2}, opt);
    wa = ws_acc.data_ptr<float>();
    wm = ws_ml.data_ptr<float>();
  }
  // Shapes are checked here; the VALUES inside tiles, positions and block
  // tables are bounded inside the kernels (tiles that do not fit are
  // skipped, positions and block ids are clamped), so no launch can read
  // or write outside its operands and no host sync is needed.
  latent_attention_launch(ctx.data_ptr(), q_lat.data_ptr(), cache.data_ptr(),
                          block_tables.data_ptr<int>(), tiles.data_ptr<int>(),
                          pos32.data_ptr<int>(), ntiles, (float)scale, T, H, R,
                          BS, (int)block_tables.size(0),
                          (int)block_tables.size(1), (int)cache.size(0),
                          (int)cache.size(1), bf, exact ? 1 : 0, io_bf,
                          q_lat.stride(0), q_lat.stride(1), ctx.stride(0),
                          ctx.stride(1), (int)nsplit, wa, wm,
                          cur_stream(q_lat));
  HIP_CHECK_LAST();
}

bool latent_attention_uses_mfma(Tensor cache) {
  return latent_attn_uses_mfma(cache.scalar_type() == at::kBFloat16 ? 1 : 0,
                               (int)cache.size(1), (int)cache.size(2),
                               (int)cache.size(3)) != 0;
}

void act_inplace(Tensor x, long mode) {
  const int bf = act_kind(x, "x");
  TORCH_CHECK(mode >= 0 && mode <= 3);
  act_inplace_launch(x.data_ptr(), x.numel(), (int)mode, bf, cur_stream(x));
  HIP_CHECK_LAST();
}

void softcap(Tensor x, double cap) {
  chk(x, "logits", at::kFloat);
  TORCH_CHECK(cap > 0);
  softcap_launch(x.data_ptr<float>(), x.numel(), (float)cap, cur_stream(x));
  HIP_CHECK_LAST();
}

void route_grouped_topk(Tensor experts, Tensor weights, Tensor logits,
                        long E, long G, long keep, double scale) {
  chk(experts, "experts", at::kInt);
  chk(weights, "weights", at::kFloat);
  chk(logits, "logits", at::kFloat);
  TORCH_CHECK(logits.dim() == 2 && experts.dim() == 2 &&
              weights.sizes() == experts.sizes());
  const int T = logits.size(0), top = experts.size(1);
  TORCH_CHECK(experts.size(0) == T && E >= 1 && E <= logits.size(1));
  TORCH_CHECK(G >= 1 && E % G == 0 && keep >= 1 && keep <= G);
  TORCH_CHECK(top >= 1 && top <= keep * (E / G),
              "top must fit into the experts of the kept groups");
  TORCH_CHECK((E + G) * 4 <= 60 * 1024, "too many experts for one LDS tile");
  route_grouped_topk_launch(experts.data_ptr<int>(), weights.data_ptr<float>(),
                            logits.data_ptr<float>(), (int)logits.size(1), T,
                            (int)E, (int)G, (int)keep, top, (float)scale,
                            cur_stream(logits));
  HIP_CHECK_LAST();
}

void moe_combine(Tensor out, Tensor y, Tensor inv, Tensor weights,
                 OptTensor shared, OptTensor gate, long gate_col) {
  chk(out, "out", at::kFloat);
  chk(inv, "inv", at::kInt);
  chk(weights, "weights", at::kFloat);
  const int bf = act_kind(y, "y");
  TORCH_CHECK(out.dim() == 2 && y.dim() == 2 && inv.dim() == 2);
  const int T = out.size(0), W = out.size(1), top = inv.size(1);
  TORCH_CHECK(inv.size(0) == T && weights.sizes() == inv.sizes());
  TORCH_CHECK(y.size(1) == W && y.size(0) == (long)T * top);
  // inv values are clamped to y's rows inside the kernel
  const void* sp = nullptr;
  const float* gp = nullptr;
  int ldg = 0;
  if (shared.has_value()) {
    TORCH_CHECK(act_kind(*shared, "shared") == bf && shared->sizes() == out.sizes());
    sp = shared->data_ptr();
    if (gate.has_value()) {
      chk(*gate, "gate_logits", at::kFloat);
      TORCH_CHECK(gate->dim() == 2 && gate->size(0) == T && gate_col >= 0 &&
                  gate_col < gate->size(1));
      gp = gate->data_ptr<float>();
      ldg = gate->size(1);
    }
  }
  moe_combine_launch(out.data_ptr<float>(), y.data_ptr(), inv.data_ptr<int>(),
                     weights.data_ptr<float>(), sp, gp, ldg, (int)gate_col, T,
                     W, top, bf, cur_stream(out));
  HIP_CHECK_LAST();
}

// u[TK, F] = act(x[s_tok] . up[e]^T) over the expert-sorted rows
void grouped_up_act(Tensor u, Tensor x, Tensor up, Tensor s_tok, Tensor offs,
                    Tensor counts, long act_mode) {
  chk(u, "u", at::kBFloat16); chk(x, "x", at::kBFloat16);
  chk(up, "up", at::kBFloat16);
  chk(s_tok, "s_tok", at::kInt); chk(offs, "offs", at::kInt);
  chk(counts, "counts", at::kInt);
  TORCH_CHECK(u.dim() == 2 && x.dim() == 2 && up.dim() == 3);
  const int TK = u.size(0), F = u.size(1), T = x.size(0), W = x.size(1);
  const int E = up.size(0);
  TORCH_CHECK(up.size(1) == F && up.size(2) == W);
  TORCH_CHECK(s_tok.numel() == TK && offs.numel() == E && counts.numel() == E);
  TORCH_CHECK(W % 32 == 0 && F % 64 == 0 && T >= 1,
              "grouped_up_act needs width % 32 == 0 and ff % 64 == 0");
  TORCH_CHECK(act_mode >= 0 && act_mode <= 3);
  grouped_up_act_launch(u.data_ptr(), x.data_ptr(), up.data_ptr(),
                        s_tok.data_ptr<int>(), offs.data_ptr<int>(),
                        counts.data_ptr<int>(), E, W, F, TK, T, (int)act_mode,
                        cur_stream(x));
  HIP_CHECK_LAST();
}

// y[TK, W] = u . down[e]^T over the expert-sorted rows
void grouped_down(Tensor y, Tensor u, Tensor down, Tensor offs, Tensor counts) {
  chk(y, "y", at::kBFloat16); chk(u, "u", at::kBFloat16);
  chk(down, "down", at::kBFloat16);
  chk(offs, "offs", at::kInt); chk(counts, "counts", at::kInt);
  TORCH_CHECK(y.dim() == 2 && u.dim() == 2 && down.dim() == 3);
  const int TK = u.size(0), F = u.size(1), W = y.size(1), E = down.size(0);
  TORCH_CHECK(y.size(0) == TK && down.size(1) == W && down.size(2) == F);
  TORCH_CHECK(offs.numel() == E && counts.numel() == E);
  TORCH_CHECK(F % 32 == 0 && W % 64 == 0,
              "grouped_down needs ff % 32 == 0 and width % 64 == 0");
  grouped_down_launch(y.data_ptr(), u.data_ptr(), down.data_ptr(),
                      offs.data_ptr<int>(), counts.data_ptr<int>(), E, F, W,
                      TK, cur_stream(u));
  HIP_CHECK_LAST();
}

void argmax_f32(Tensor out, Tensor logits) {
  chk(out, "out", at::kLong);
  chk(logits, "logits", at::kFloat);
  TORCH_CHECK(logits.dim() == 2 && out.numel() == logits.size(0));
  argmax_f32_launch(out.data_ptr<long>(), logits.data_ptr<float>(),
                    (int)logits.size(0), (int)logits.size(1),
                    cur_stream(logits));
  HIP_CHECK_LAST();
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_pair_hash", &embed_pair_hash);
  m.def("rms_scale_add", &rms_scale_add);
  m.def("rms_norm_f32", &rms_norm_f32);
  m.def("latent_norm_store", &latent_norm_store);
  m.def("latent_attention", &latent_attention);
  m.def("latent_attention_uses_mfma", &latent_attention_uses_mfma);
  m.def("act_inplace", &act_inplace);
  m.def("softcap", &softcap);
  m.def("route_grouped_topk", &route_grouped_topk);
  m.def("moe_combine", &moe_combine);
  m.def("argmax_f32", &argmax_f32);
  m.def("grouped_up_act", &grouped_up_act);
  m.def("grouped_down", &grouped_down);
}
