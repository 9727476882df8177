// TORCH_LIBRARY registration of the kernels in seq_mix.hip, latent_attention.hip and glu_moe.hip
// (symmetry_amd/_C_latent.so, namespace symmetry_amd_latent).
//
// Out-parameter style like the main kernel library: the caller pre-allocates, nothing is allocated here, every
// launch goes to torch's current HIP stream (hipGraph-capturable), and every shape / dtype / range the kernels
// and their grids assume is checked on the host before the launch.  Activation tensors are all bf16 or all
// fp32; which one is read off the first activation argument.
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include "latent_launchers.h"

namespace {

using at::Tensor;
using OptTensor = std::optional<Tensor>;

hipStream_t cur_stream(const Tensor& t) { return c10::hip::getCurrentHIPStream(t.get_device()).stream(); }

void gpu(const Tensor& t, const char* name, bool contiguous = true) {
  TORCH_CHECK(t.device().type() == c10::DeviceType::CUDA, name, " must be a GPU tensor");
  TORCH_CHECK(!contiguous || t.is_contiguous(), name, " must be contiguous");
}

void dtype(const Tensor& t, at::ScalarType dt, const char* name) {
  gpu(t, name);
  TORCH_CHECK(t.scalar_type() == dt, name, " has dtype ", t.scalar_type(), ", expected ", dt);
}

// activation dtype: returns 1 for fp32, 0 for bf16
int act(const Tensor& t, const char* name, bool contiguous = true) {
  gpu(t, name, contiguous);
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16, name, " must be bf16 or fp32");
  return t.scalar_type() == at::kFloat;
}

void same_act(const Tensor& t, int f32, const char* name, bool contiguous = true) {
  TORCH_CHECK(act(t, name, contiguous) == f32, name, ": activation dtypes differ");
}

template <typename T>
T* ptr(const Tensor& t) {
  return reinterpret_cast<T*>(t.data_ptr());
}

template <typename T>
T* optptr(const OptTensor& t) {
  return t.has_value() ? reinterpret_cast<T*>(t->data_ptr()) : nullptr;
}

void embed_rows(const Tensor& ids, const OptTensor& src, const OptTensor& prev, const Tensor& table, Tensor& x,
                Tensor& hist0) {
  const int f32 = act(table, "table");
  dtype(ids, at::kInt, "ids");
  dtype(x, at::kFloat, "x");
  dtype(hist0, at::kFloat, "hist0");
  const int64_t T = ids.numel(), d = table.size(1);
  TORCH_CHECK(table.dim() == 2 && x.numel() == T * d && hist0.numel() == T * d, "embed_rows: shapes");
  if (src.has_value()) {
    TORCH_CHECK(prev.has_value(), "embed_rows: src without prev");
    dtype(*src, at::kInt, "src");
    dtype(*prev, at::kInt, "prev");
    TORCH_CHECK(src->numel() >= T, "embed_rows: src too short");
  }
  launch_embed_rows(ptr<int>(ids), optptr<int>(src), optptr<int>(prev), table.data_ptr(), ptr<float>(x),
                    ptr<float>(hist0), (int)T, (int)d, f32, cur_stream(x));
}

void token_shift(const Tensor& x, const Tensor& mu, const Tensor& prev_row, const Tensor& state, Tensor& h) {
  const int f32 = act(h, "h");
  same_act(mu, f32, "mu");
  dtype(x, at::kFloat, "x");
  dtype(prev_row, at::kInt, "prev_row");
  gpu(state, "state", false);
  TORCH_CHECK(state.scalar_type() == at::kFloat && state.dim() == 2 && state.stride(1) == 1, "token_shift: state [slots, d] fp32");
  const int64_t T = x.size(0), d = x.size(1);
  TORCH_CHECK(x.dim() == 2 && h.numel() == T * d && mu.numel() == d && state.size(1) == d && prev_row.numel() >= T,
              "token_shift: shapes");
  launch_token_shift(ptr<float>(x), mu.data_ptr(), ptr<int>(prev_row), ptr<float>(state), state.stride(0),
                     h.data_ptr(), (int)T, (int)d, f32, cur_stream(x));
}

void add_layer_norm(const Tensor& delta, const Tensor& w, double eps, Tensor& x, const OptTensor& save,
                    const OptTensor& state, const OptTensor& hist, const OptTensor& coef, int64_t hist_idx,
                    const OptTensor& out_act) {
  const int f32 = act(w, "w");
  const int dl32 = act(delta, "delta");
  TORCH_CHECK(dl32 == f32 || dl32 == 1, "add_layer_norm: delta dtype");
  dtype(x, at::kFloat, "x");
  const int64_t T = x.size(0), d = x.size(1);
  TORCH_CHECK(x.dim() == 2 && delta.numel() == T * d && w.numel() == d, "add_layer_norm: shapes");
  long long sstride = 0, hstride = 0;
  if (save.has_value()) {
    TORCH_CHECK(state.has_value(), "add_layer_norm: save without state");
    dtype(*save, at::kInt, "save");
    gpu(*state, "state", false);
    TORCH_CHECK(state->scalar_type() == at::kFloat && state->dim() == 2 && state->stride(1) == 1 && state->size(1) == d &&
                    save->numel() >= T, "add_layer_norm: state [slots, d] fp32");
    sstride = state->stride(0);
  }
  if (hist.has_value()) {
    TORCH_CHECK(coef.has_value(), "add_layer_norm: hist without coef");
    dtype(*hist, at::kFloat, "hist");
    dtype(*coef, at::kFloat, "coef");
    TORCH_CHECK(hist->dim() == 3 && hist->size(1) == T && hist->size(2) == d && hist_idx >= 1 &&
                    hist_idx < hist->size(0) && coef->numel() == hist_idx + 1, "add_layer_norm: history shapes");
    hstride = T * d;
  }
  if (out_act.has_value()) {
    same_act(*out_act, f32, "out_act");
    TORCH_CHECK(out_act->numel() == T * d, "add_layer_norm: out_act shape");
  }
  launch_add_layer_norm(delta.data_ptr(), dl32, w.data_ptr(), (float)eps, ptr<float>(x), optptr<int>(save),
                        save.has_value() ? ptr<float>(*state) : nullptr, sstride, optptr<float>(hist), hstride,
                        optptr<float>(coef), (int)hist_idx, out_act.has_value() ? out_act->data_ptr() : nullptr,
                        (int)T, (int)d, f32, cur_stream(x));
}

void layer_norm(const Tensor& x, const OptTensor& rows, const Tensor& w, double eps, Tensor& out) {
  const int f32 = act(out, "out");
  same_act(w, f32, "w");
  dtype(x, at::kFloat, "x");
  const int64_t n = out.size(0), d = x.size(1);
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.size(1) == d && w.numel() == d, "layer_norm: shapes");
  if (rows.has_value()) {
    dtype(*rows, at::kLong, "rows");
    TORCH_CHECK(rows->numel() >= n, "layer_norm: rows too short");
  } else {
    TORCH_CHECK(x.size(0) >= n, "layer_norm: x too short");
  }
  launch_layer_norm(ptr<float>(x), optptr<long long>(rows), w.data_ptr(), (float)eps, out.data_ptr(), (int)n, (int)d,
                    f32, cur_stream(x));
}

void latent_prep(const Tensor& z, int64_t q_rank, int64_t kv_rank, int64_t rot, const Tensor& wq, const OptTensor& wkv,
                 double eps, const Tensor& positions, const Tensor& slots, const Tensor& rope, Tensor& cq,
                 const OptTensor& cache, int64_t half_dims) {
  const int f32 = act(z, "z", false);
  same_act(wq, f32, "wq");
  same_act(cq, f32, "cq");
  dtype(positions, at::kInt, "positions");
  dtype(slots, at::kInt, "slots");
  dtype(rope, at::kFloat, "rope");
  const int64_t T = z.size(0);
  LatentPrepArgs a{};
  a.z = z.data_ptr();
  TORCH_CHECK(z.dim() == 2 && (z.size(1) == 1 || z.stride(1) == 1), "latent_prep: z [T, n] with unit inner stride");
  a.nz = (int)(T > 1 ? z.stride(0) : z.size(1));
  const int64_t zcols = z.size(1);
  TORCH_CHECK(half_dims >= 0 && half_dims % 2 == 0 && half_dims <= rot, "latent_prep: half_dims");
  a.half_dims = (int)half_dims;
  a.q_rank = (int)q_rank;
  a.kv_rank = (int)kv_rank;
  a.rot = (int)rot;
  TORCH_CHECK(z.dim() == 2 && wq.numel() == q_rank && cq.numel() == T * q_rank && positions.numel() >= T &&
                  slots.numel() >= T && rot % 2 == 0, "latent_prep: shapes");
  if (kv_rank > 0) {
    TORCH_CHECK(wkv.has_value() && cache.has_value(), "latent_prep: kv part needs wkv and cache");
    same_act(*wkv, f32, "wkv");
    same_act(*cache, f32, "cache");
    TORCH_CHECK(zcols == q_rank + kv_rank + rot && wkv->numel() == kv_rank && cache->size(-1) == kv_rank + rot &&
                    rope.dim() == 3 && rope.size(1) == rot / 2 && rope.size(2) == 2, "latent_prep: kv shapes");
    a.wkv = wkv->data_ptr();
    a.cache = cache->data_ptr();
  } else {
    TORCH_CHECK(zcols == q_rank, "latent_prep: z width");
  }
  a.wq = wq.data_ptr();
  a.eps = (float)eps;
  a.positions = ptr<int>(positions);
  a.slots = ptr<int>(slots);
  a.rope = ptr<float>(rope);
  a.cq = cq.data_ptr();
  launch_latent_prep(a, (int)T, f32, cur_stream(z));
}

void rope_pairs(const Tensor& src, Tensor& dst, const Tensor& positions, const Tensor& rope, int64_t half_dims) {
  const int f32 = act(src, "src", false);
  same_act(dst, f32, "dst", false);
  dtype(positions, at::kInt, "positions");
  dtype(rope, at::kFloat, "rope");
  TORCH_CHECK(src.dim() == 3 && dst.dim() == 3 && src.sizes() == dst.sizes() && src.stride(2) == 1 && dst.stride(2) == 1,
              "rope_pairs: [T, H, rot] views with unit inner stride");
  const int64_t T = src.size(0), H = src.size(1), rot = src.size(2);
  TORCH_CHECK(rot % 2 == 0 && rope.dim() == 3 && rope.size(1) == rot / 2 && rope.size(2) == 2 && positions.numel() >= T &&
                  half_dims >= 0 && half_dims % 2 == 0 && half_dims <= rot, "rope_pairs: table / positions / half_dims");
  launch_rope_pairs(src.data_ptr(), src.stride(0), src.stride(1), dst.data_ptr(), dst.stride(0), dst.stride(1),
                    ptr<int>(positions), ptr<float>(rope), (int)T, (int)H, (int)rot, (int)half_dims, f32, cur_stream(src));
}

int64_t latent_attn(const Tensor& q, const Tensor& cache, const Tensor& block_tables, const Tensor& row_seq,
                    const Tensor& positions, double scale, int64_t kv_rank, Tensor& out, const OptTensor& part_o,
                    const OptTensor& part_ml, const OptTensor& tiles, const OptTensor& cu_q, int64_t impl, int64_t window) {
  const int f32 = act(q, "q");
  same_act(cache, f32, "cache");
  same_act(out, f32, "out");
  dtype(block_tables, at::kInt, "block_tables");
  dtype(row_seq, at::kInt, "row_seq");
  dtype(positions, at::kInt, "positions");
  TORCH_CHECK(q.dim() == 3 && cache.dim() == 3 && block_tables.dim() == 2, "latent_attn: q [T,H,Dk], cache [NB,BS,Dk]");
  LatentAttnArgs a{};
  a.T = (int)q.size(0);
  a.H = (int)q.size(1);
  a.Dk = (int)q.size(2);
  a.kv_rank = (int)kv_rank;
  a.BS = (int)cache.size(1);
  a.max_blocks = (int)block_tables.size(1);
  a.bs_shift = -1;
  for (int sh = 0; sh < 20; ++sh)
    if ((1 << sh) == a.BS) a.bs_shift = sh;
  TORCH_CHECK(cache.size(2) == a.Dk && kv_rank > 0 && kv_rank <= a.Dk && kv_rank <= 512 && a.Dk <= 8192 &&
                  out.numel() == (int64_t)a.T * a.H * kv_rank && row_seq.numel() >= a.T && positions.numel() >= a.T &&
                  a.H <= 65535 && window >= 0, "latent_attn: shapes");
  a.window = (int)std::min<int64_t>(window, 1 << 30);
  a.parts = 1;
  a.part_tokens = 32;
  if (part_o.has_value()) {
    // partials [T, H, parts, kv_rank] + [T, H, parts, 2]: the caller's `parts` partitions cover the block-table span
    TORCH_CHECK(part_ml.has_value(), "latent_attn: part_o without part_ml");
    dtype(*part_o, at::kFloat, "part_o");
    dtype(*part_ml, at::kFloat, "part_ml");
    TORCH_CHECK(part_o->dim() == 4 && part_o->size(0) == a.T && part_o->size(1) == a.H && part_o->size(3) == kv_rank &&
                    part_ml->numel() == (int64_t)a.T * a.H * part_o->size(2) * 2, "latent_attn: partial buffer shapes");
    a.parts = (int)part_o->size(2);
    // (with a window a row's partitions start at its first visible key and cover at most the window)
    const int64_t span = a.window > 0 ? std::min<int64_t>((int64_t)a.max_blocks * a.BS, a.window) : (int64_t)a.max_blocks * a.BS;
    a.part_tokens = (int)(((span + a.parts - 1) / a.parts + 31) / 32 * 32);
    TORCH_CHECK(a.parts >= 1 && a.parts <= 1024 && (int64_t)a.parts * a.part_tokens >= span, "latent_attn: partitions");
    a.part_o = ptr<float>(*part_o);
    a.part_ml = ptr<float>(*part_ml);
  }
  a.q = q.data_ptr();
  a.cache = cache.data_ptr();
  a.block_tables = ptr<int>(block_tables);
  a.row_seq = ptr<int>(row_seq);
  a.positions = ptr<int>(positions);
  a.out = out.data_ptr();
  a.scale = (float)scale;
  if (tiles.has_value()) {
    TORCH_CHECK(cu_q.has_value() && !part_o.has_value(), "latent_attn: tiles need cu_q and take no split-KV partials");
    dtype(*tiles, at::kInt, "tiles");
    dtype(*cu_q, at::kInt, "cu_q");
    TORCH_CHECK(tiles->dim() == 2 && tiles->size(1) == 2 && cu_q->numel() == block_tables.size(0) + 1,
                "latent_attn: tiles [n, 2], cu_q [seqs + 1]");
    a.tiles = ptr<int>(*tiles);
    a.cu_q = ptr<int>(*cu_q);
    a.ntiles = (int)tiles->size(0);
  }
  TORCH_CHECK(q.data_ptr() != nullptr && (reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 == 0) &&
                  (reinterpret_cast<uintptr_t>(cache.data_ptr()) % 16 == 0) &&
                  (reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0), "latent_attn: 16-byte aligned tensors");
  return launch_latent_attn(a, f32, (int)impl, cur_stream(q));
}

void clamped_glu(const Tensor& gu, double limit, double alpha, Tensor& out) {
  const int f32 = act(gu, "gu");
  same_act(out, f32, "out");
  TORCH_CHECK(gu.dim() == 2 && out.dim() == 2 && gu.size(0) == out.size(0) && gu.size(1) == 2 * out.size(1),
              "clamped_glu: gu [R, 2F], out [R, F]");
  launch_clamped_glu(gu.data_ptr(), out.data_ptr(), (int)out.size(0), (int)out.size(1), (float)limit, (float)alpha, f32,
                     cur_stream(gu));
}

void sigmoid_topk(const Tensor& x, const Tensor& Wr, int64_t k, Tensor& ids, Tensor& w) {
  const int f32 = act(x, "x");
  same_act(Wr, f32, "Wr");
  dtype(ids, at::kInt, "ids");
  dtype(w, at::kFloat, "w");
  const int64_t T = x.size(0), d = x.size(1), E = Wr.size(0);
  TORCH_CHECK(x.dim() == 2 && Wr.dim() == 2 && Wr.size(1) == d && k >= 1 && k <= E && E <= 1024 && d <= 12288 &&
                  ids.numel() >= T * k && w.numel() >= T * k, "sigmoid_topk: shapes");
  launch_sigmoid_topk(x.data_ptr(), Wr.data_ptr(), (int)T, (int)d, (int)E, (int)k, ptr<int>(ids), ptr<float>(w), f32,
                      cur_stream(x));
}

void expert_offsets(const Tensor& ids, int64_t R, int64_t E, Tensor& offsets, Tensor& cursor) {
  dtype(ids, at::kInt, "ids");
  dtype(offsets, at::kInt, "offsets");
  dtype(cursor, at::kInt, "cursor");
  TORCH_CHECK(ids.numel() >= R && E <= 1024 && offsets.numel() >= E + 1 && cursor.numel() >= E, "expert_offsets: shapes");
  launch_expert_offsets(ptr<int>(ids), (int)R, (int)E, ptr<int>(offsets), ptr<int>(cursor), cur_stream(ids));
}

void scatter_scaled(const Tensor& x, const Tensor& ids, const Tensor& w, int64_t k, const Tensor& offsets, Tensor& cursor,
                    Tensor& xs, Tensor& dst) {
  const int f32 = act(x, "x");
  same_act(xs, f32, "xs");
  dtype(ids, at::kInt, "ids");
  dtype(w, at::kFloat, "w");
  dtype(offsets, at::kInt, "offsets");
  dtype(cursor, at::kInt, "cursor");
  dtype(dst, at::kInt, "dst");
  const int64_t T = x.size(0), d = x.size(1), R = T * k;
  TORCH_CHECK(x.dim() == 2 && xs.numel() == R * d && ids.numel() >= R && w.numel() >= R && dst.numel() >= R,
              "scatter_scaled: shapes");
  launch_scatter_scaled(x.data_ptr(), ptr<int>(ids), ptr<float>(w), (int)k, (int)R, (int)d, ptr<int>(offsets),
                        ptr<int>(cursor), xs.data_ptr(), ptr<int>(dst), f32, cur_stream(x));
}

void grouped_linear(const Tensor& xs, const Tensor& W, const Tensor& offsets, Tensor& y) {
  const int f32 = act(xs, "xs");
  same_act(W, f32, "W");
  same_act(y, f32, "y");
  dtype(offsets, at::kInt, "offsets");
  TORCH_CHECK(xs.dim() == 2 && W.dim() == 3 && y.dim() == 2, "grouped_linear: xs [R,K], W [E,N,K], y [R,N]");
  const int64_t R = xs.size(0), K = xs.size(1), E = W.size(0), N = W.size(1);
  TORCH_CHECK(W.size(2) == K && y.size(0) == R && y.size(1) == N && offsets.numel() >= E + 1 &&
                  (R + 63) / 64 + E <= 65535, "grouped_linear: shapes");
  launch_grouped_linear(xs.data_ptr(), W.data_ptr(), ptr<int>(offsets), (int)E, (int)R, (int)N, (int)K, y.data_ptr(), f32,
                        cur_stream(xs));
}

void gather_sum(const Tensor& y, const Tensor& dst, int64_t k, const OptTensor& extra, Tensor& out) {
  const int f32 = act(y, "y");
  dtype(dst, at::kInt, "dst");
  dtype(out, at::kFloat, "out");
  const int64_t T = out.size(0), d = out.size(1);
  TORCH_CHECK(out.dim() == 2 && y.dim() == 2 && y.size(1) == d && y.size(0) >= T * k && dst.numel() >= T * k,
              "gather_sum: shapes");
  if (extra.has_value()) {
    same_act(*extra, f32, "extra");
    TORCH_CHECK(extra->numel() == T * d, "gather_sum: extra shape");
  }
  launch_gather_sum(y.data_ptr(), ptr<int>(dst), (int)k, extra.has_value() ? extra->data_ptr() : nullptr, ptr<float>(out),
                    (int)T, (int)d, f32, cur_stream(y));
}

}  // namespace

TORCH_LIBRARY(symmetry_amd_latent, m) {
  m.def("embed_rows(Tensor ids, Tensor? src, Tensor? prev, Tensor table, Tensor(a!) x, Tensor(b!) hist0) -> ()", &embed_rows);
  m.def("token_shift(Tensor x, Tensor mu, Tensor prev_row, Tensor state, Tensor(a!) h) -> ()", &token_shift);
  m.def(
      "add_layer_norm(Tensor delta, Tensor w, float eps, Tensor(a!) x, Tensor? save, Tensor(b!)? state, Tensor(c!)? hist, "
      "Tensor? coef, int hist_idx, Tensor(d!)? out_act) -> ()",
      &add_layer_norm);
  m.def("layer_norm(Tensor x, Tensor? rows, Tensor w, float eps, Tensor(a!) out) -> ()", &layer_norm);
  m.def(
      "latent_prep(Tensor z, int q_rank, int kv_rank, int rot, Tensor wq, Tensor? wkv, float eps, Tensor positions, "
      "Tensor slots, Tensor rope, Tensor(a!) cq, Tensor(b!)? cache, int half_dims) -> ()",
      &latent_prep);
  m.def("rope_pairs(Tensor src, Tensor(a!) dst, Tensor positions, Tensor rope, int half_dims) -> ()", &rope_pairs);
  m.def(
      "latent_attn(Tensor q, Tensor cache, Tensor block_tables, Tensor row_seq, Tensor positions, float scale, "
      "int kv_rank, Tensor(a!) out, Tensor(b!)? part_o, Tensor(c!)? part_ml, Tensor? tiles, Tensor? cu_q, int impl, "
      "int window) -> int",
      &latent_attn);
  m.def("clamped_glu(Tensor gu, float limit, float alpha, Tensor(a!) out) -> ()", &clamped_glu);
  m.def("sigmoid_topk(Tensor x, Tensor Wr, int k, Tensor(a!) ids, Tensor(b!) w) -> ()", &sigmoid_topk);
  m.def("expert_offsets(Tensor ids, int R, int E, Tensor(a!) offsets, Tensor(b!) cursor) -> ()", &expert_offsets);
  m.def(
      "scatter_scaled(Tensor x, Tensor ids, Tensor w, int k, Tensor offsets, Tensor(a!) cursor, Tensor(b!) xs, "
      "Tensor(c!) dst) -> ()",
      &scatter_scaled);
  m.def("grouped_linear(Tensor xs, Tensor W, Tensor offsets, Tensor(a!) y) -> ()", &grouped_linear);
  m.def("gather_sum(Tensor y, Tensor dst, int k, Tensor? extra, Tensor(a!) out) -> ()", &gather_sum);
}
