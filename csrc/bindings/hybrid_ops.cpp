// TORCH_LIBRARY registration of the kernels in hybrid_rows.hip, stream_rows.hip, window_attention.hip and decay_scan.hip, plus the
// expert-segment kernels of glu_moe.hip that the routed feed-forward shares (symmetry_amd/_C_hybrid.so, namespace
// symmetry_amd_hybrid).
//
// Out-parameter style like the other kernel libraries: the caller pre-allocates, nothing is allocated here, every
// launch goes to torch's current HIP stream (hipGraph-capturable), and every shape / dtype / range the kernels and
// their grids assume is checked on the host before the launch.  Activation tensors are all bf16 or all fp32; which
// one is read off the first activation argument.  "view" arguments may be column ranges of a wider matrix (unit inner
// stride, any row stride).
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include "hybrid_launchers.h"
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

// a [rows, cols] column range: unit inner stride; returns the row stride
int64_t view2(const Tensor& t, int f32, int64_t rows, int64_t cols, const char* name) {
  same_act(t, f32, name, false);
  TORCH_CHECK(t.dim() == 2 && t.size(0) == rows && t.size(1) == cols, name, ": expected [", rows, ", ", cols, "], got ",
              t.sizes());
  TORCH_CHECK(cols == 1 || t.stride(1) == 1, name, ": inner stride must be 1");
  return rows > 1 ? t.stride(0) : cols;
}

template <typename T>
T* ptr(const Tensor& t) {
  return reinterpret_cast<T*>(t.data_ptr());
}

template <typename T>
T* optptr(const OptTensor& t) {
  return t.has_value() ? reinterpret_cast<T*>(t->data_ptr()) : nullptr;
}

void embed_norm(const Tensor& ids, const OptTensor& src, const OptTensor& prev, const Tensor& table, const Tensor& w,
                double eps, double offset, Tensor& x) {
  const int f32 = act(table, "table");
  dtype(ids, at::kInt, "ids");
  dtype(x, at::kFloat, "x");
  dtype(w, at::kFloat, "w");
  const int64_t T = ids.numel(), d = table.size(1);
  TORCH_CHECK(table.dim() == 2 && x.numel() == T * d && w.numel() == d, "embed_norm: shapes");
  if (src.has_value()) {
    TORCH_CHECK(prev.has_value(), "embed_norm: src without prev");
    dtype(*src, at::kInt, "src");
    dtype(*prev, at::kInt, "prev");
    TORCH_CHECK(src->numel() >= T, "embed_norm: src too short");
  }
  launch_embed_norm(ptr<int>(ids), optptr<int>(src), optptr<int>(prev), table.data_ptr(), ptr<float>(w), (float)eps,
                    (float)offset, ptr<float>(x), (int)T, (int)d, f32, cur_stream(x));
}

void rms_norm_rows(const Tensor& x, const OptTensor& rows, const Tensor& w, double eps, double offset, Tensor& out) {
  const int f32 = act(out, "out");
  dtype(x, at::kFloat, "x");
  dtype(w, at::kFloat, "w");
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2, "rms_norm_rows: x [T, d], out [n, d]");
  const int64_t n = out.size(0), d = x.size(1);
  TORCH_CHECK(out.size(1) == d && w.numel() == d, "rms_norm_rows: widths");
  if (rows.has_value()) {
    dtype(*rows, at::kLong, "rows");
    TORCH_CHECK(rows->numel() >= n, "rms_norm_rows: rows too short");
  } else {
    TORCH_CHECK(x.size(0) >= n, "rms_norm_rows: x too short");
  }
  launch_rms_norm_rows(ptr<float>(x), optptr<long long>(rows), ptr<float>(w), (float)eps, (float)offset, out.data_ptr(),
                       (int)n, (int)d, f32, cur_stream(x));
}

void residual_mix_norm(Tensor& x, const Tensor& a, double sa, const OptTensor& bias_a, const OptTensor& b, double sb,
                       const OptTensor& c, double sc, const OptTensor& w, double eps, double offset, OptTensor out) {
  dtype(x, at::kFloat, "x");
  TORCH_CHECK(x.dim() == 2, "residual_mix_norm: x [T, d]");
  const int64_t T = x.size(0), d = x.size(1);
  ResidualMixArgs r{};
  r.x = ptr<float>(x);
  r.a_f32 = act(a, "a");
  TORCH_CHECK(a.numel() == T * d, "residual_mix_norm: a shape");
  r.a = a.data_ptr();
  r.sa = (float)sa;
  if (bias_a.has_value()) {
    dtype(*bias_a, at::kFloat, "bias_a");
    TORCH_CHECK(bias_a->numel() == d, "residual_mix_norm: bias shape");
    r.bias_a = ptr<float>(*bias_a);
  }
  if (b.has_value()) {
    r.b_f32 = act(*b, "b");
    TORCH_CHECK(b->numel() == T * d, "residual_mix_norm: b shape");
    r.b = b->data_ptr();
    r.sb = (float)sb;
  }
  if (c.has_value()) {
    r.c_f32 = act(*c, "c");
    TORCH_CHECK(c->numel() == T * d, "residual_mix_norm: c shape");
    r.c = c->data_ptr();
    r.sc = (float)sc;
  }
  int f32 = 0;
  if (out.has_value()) {
    f32 = act(*out, "out");
    TORCH_CHECK(w.has_value(), "residual_mix_norm: out without w");
    dtype(*w, at::kFloat, "w");
    TORCH_CHECK(out->numel() == T * d && w->numel() == d, "residual_mix_norm: out / w shape");
    r.out = out->data_ptr();
    r.w = ptr<float>(*w);
  }
  r.eps = (float)eps;
  r.offset = (float)offset;
  r.T = (int)T;
  r.d = (int)d;
  launch_residual_mix_norm(r, f32, cur_stream(x));
}

void qkv_rope_cache(const Tensor& z, const OptTensor& bias, int64_t H, int64_t G, int64_t dk, int64_t dv,
                    const Tensor& positions, const Tensor& slots, const OptTensor& rope, Tensor& q_out, Tensor& k_cache,
                    Tensor& v_cache, int64_t half_dims) {
  const int f32 = act(z, "z", false);
  TORCH_CHECK(z.dim() == 2, "qkv_rope_cache: z [T, n]");
  const int64_t T = z.size(0), n = H * dk + G * dk + G * dv;
  QkvRopeArgs a{};
  a.ldz = view2(z, f32, T, z.size(1), "z");
  TORCH_CHECK(z.size(1) >= n, "qkv_rope_cache: z narrower than q | k | v");
  same_act(q_out, f32, "q_out");
  same_act(k_cache, f32, "k_cache");
  same_act(v_cache, f32, "v_cache");
  dtype(positions, at::kInt, "positions");
  dtype(slots, at::kInt, "slots");
  if (bias.has_value()) {
    dtype(*bias, at::kFloat, "bias");
    TORCH_CHECK(bias->numel() >= n, "qkv_rope_cache: bias shorter than q | k | v");
  }
  if (rope.has_value()) {
    dtype(*rope, at::kFloat, "rope");
    TORCH_CHECK(rope->dim() == 3 && rope->size(2) == 2 && 2 * rope->size(1) <= dk,
                "qkv_rope_cache: rope [max_pos, pairs, 2]");
    TORCH_CHECK(half_dims == 0 || half_dims == 2 * rope->size(1), "qkv_rope_cache: half_dims = 2 * pairs of the table");
  }
  TORCH_CHECK(q_out.numel() == T * H * dk && positions.numel() >= T && slots.numel() >= T &&
                  k_cache.dim() == 4 && v_cache.dim() == 4 && k_cache.size(2) == G && k_cache.size(3) == dk &&
                  v_cache.size(2) == G && v_cache.size(3) == dv && H % G == 0,
              "qkv_rope_cache: shapes");
  a.z = z.data_ptr();
  a.bias = optptr<float>(bias);
  a.H = (int)H, a.G = (int)G, a.dk = (int)dk, a.dv = (int)dv, a.pairs = rope.has_value() ? (int)rope->size(1) : 0;
  a.half = half_dims > 0;
  a.positions = ptr<int>(positions);
  a.slots = ptr<int>(slots);
  a.rope = optptr<float>(rope);
  a.q_out = q_out.data_ptr();
  a.k_cache = k_cache.data_ptr();
  a.v_cache = v_cache.data_ptr();
  launch_qkv_rope_cache(a, (int)T, f32, cur_stream(z));
}

int64_t window_attn(const Tensor& q, const Tensor& k_cache, const Tensor& v_cache, const Tensor& block_tables,
                    const Tensor& row_seq, const Tensor& positions, int64_t window, double scale, const OptTensor& gate,
                    Tensor& out, const OptTensor& tiles, const OptTensor& cu_q, int64_t impl, const OptTensor& bias,
                    int64_t keep_first, const OptTensor& sink) {
  const int f32 = act(q, "q");
  same_act(k_cache, f32, "k_cache");
  same_act(v_cache, f32, "v_cache");
  same_act(out, f32, "out");
  dtype(block_tables, at::kInt, "block_tables");
  dtype(row_seq, at::kInt, "row_seq");
  dtype(positions, at::kInt, "positions");
  TORCH_CHECK(q.dim() == 3 && k_cache.dim() == 4 && v_cache.dim() == 4 && block_tables.dim() == 2, "window_attn: ranks");
  WindowAttnArgs a{};
  a.T = (int)q.size(0), a.H = (int)q.size(1), a.dk = (int)q.size(2);
  a.BS = (int)k_cache.size(1), a.G = (int)k_cache.size(2), a.dv = (int)v_cache.size(3);
  a.max_blocks = (int)block_tables.size(1);
  TORCH_CHECK(k_cache.size(3) == a.dk && v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == a.BS &&
                  v_cache.size(2) == a.G && a.G > 0 && a.H % a.G == 0 && a.dv <= 512 && a.dk <= 4096 && window >= 1 &&
                  out.numel() == (int64_t)a.T * a.H * a.dv && row_seq.numel() >= a.T && positions.numel() >= a.T &&
                  a.T <= 65535 && k_cache.size(0) * k_cache.size(1) < (1LL << 31),
              "window_attn: shapes");
  if (gate.has_value()) {
    a.ldg = view2(*gate, f32, a.T, a.H, "gate");
    a.gate = gate->data_ptr();
  }
  if (bias.has_value()) {
    dtype(*bias, at::kFloat, "bias");
    TORCH_CHECK(bias->dim() == 2 && bias->size(0) == 2 && bias->size(1) == a.H, "window_attn: bias [2, H]");
    a.bias = ptr<float>(*bias);
  }
  if (sink.has_value()) {
    dtype(*sink, at::kFloat, "sink");
    TORCH_CHECK(sink->numel() == a.H, "window_attn: sink [H]");
    a.sink = ptr<float>(*sink);
  }
  TORCH_CHECK(keep_first >= 0 && keep_first < (1LL << 30), "window_attn: keep_first");
  a.keep_first = (int)keep_first;
  if (tiles.has_value() && cu_q.has_value()) {
    dtype(*tiles, at::kInt, "tiles");
    dtype(*cu_q, at::kInt, "cu_q");
    a.tiles = ptr<int>(*tiles);
    a.cu_q = ptr<int>(*cu_q);
    a.ntiles = (int)tiles->size(0);
  }
  a.q = q.data_ptr();
  a.k_cache = k_cache.data_ptr();
  a.v_cache = v_cache.data_ptr();
  a.block_tables = ptr<int>(block_tables);
  a.row_seq = ptr<int>(row_seq);
  a.positions = ptr<int>(positions);
  a.out = out.data_ptr();
  a.window = (int)window;
  a.scale = (float)scale;
  return launch_window_attn(a, f32, (int)impl, cur_stream(q));
}

void decay_scan(int64_t mode, const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& dz, const Tensor& dbias,
                const OptTensor& rate, double tau, const OptTensor& skip, double q_scale, int64_t H, int64_t N, int64_t P,
                int64_t hpg, Tensor& state, const OptTensor& cu_q, const Tensor& prev_row, const Tensor& save_slot,
                int64_t runs, Tensor& out, const OptTensor& mout) {
  const int f32 = act(v, "v", false);
  dtype(out, at::kFloat, "out");
  dtype(dbias, at::kFloat, "dbias");
  dtype(prev_row, at::kInt, "prev_row");
  dtype(save_slot, at::kInt, "save_slot");
  gpu(state, "state");
  TORCH_CHECK(mode >= 0 && mode <= 2, "decay_scan: mode");
  const int64_t PS = mode == 2 ? P + 1 : P;      // columns of the state and of out
  TORCH_CHECK(state.scalar_type() == at::kFloat && state.dim() == 4 && state.size(1) == H &&
                  state.size(2) == (mode == 2 ? N + 1 : N) && state.size(3) == PS,
              "decay_scan: state [slots, H, N, P] fp32 (log gates: [slots, H, N + 1, P + 1])");
  TORCH_CHECK(H > 0 && hpg > 0 && H % hpg == 0 && N >= 1 && N <= 256 && P >= 1 && runs <= 65535, "decay_scan: sizes");
  const int64_t T = v.size(0), groups = H / hpg;
  DecayScanArgs a{};
  a.ldq = view2(q, f32, T, groups * N, "q");
  a.ldk = view2(k, f32, T, groups * N, "k");
  a.ldv = view2(v, f32, T, H * P, "v");
  a.ldd = view2(dz, mode == 2 ? 1 : f32, T, mode == 0 ? H * N : (mode == 1 ? H : 2 * H), "dz");
  TORCH_CHECK(dbias.numel() == (mode == 0 ? H * N : (mode == 1 ? H : 2 * H)) && out.numel() == T * H * PS &&
                  prev_row.numel() >= T && save_slot.numel() >= T, "decay_scan: shapes");
  if (mode == 2) {
    TORCH_CHECK(mout.has_value() && !skip.has_value(), "decay_scan: the log-gate mode writes its maxima and has no skip");
    dtype(*mout, at::kFloat, "mout");
    TORCH_CHECK(mout->numel() == T * H, "decay_scan: mout [T, H]");
    a.mout = ptr<float>(*mout);
  }
  if (mode == 1) {
    TORCH_CHECK(rate.has_value(), "decay_scan: the step-size mode needs the per-head rates");
    dtype(*rate, at::kFloat, "rate");
    TORCH_CHECK(rate->numel() == H, "decay_scan: rate [H]");
    a.rate = ptr<float>(*rate);
  } else {
    TORCH_CHECK(tau > 0, "decay_scan: tau");
  }
  if (skip.has_value()) {
    dtype(*skip, at::kFloat, "skip");
    TORCH_CHECK(skip->numel() == H, "decay_scan: skip [H]");
    a.skip = ptr<float>(*skip);
  }
  if (cu_q.has_value()) {
    dtype(*cu_q, at::kInt, "cu_q");
    TORCH_CHECK(cu_q->numel() >= runs + 1, "decay_scan: cu_q too short");
    a.cu_q = ptr<int>(*cu_q);
  } else {
    TORCH_CHECK(runs <= T, "decay_scan: more runs than rows");
  }
  a.mode = (int)mode;
  a.q = q.data_ptr(), a.k = k.data_ptr(), a.v = v.data_ptr(), a.dz = dz.data_ptr();
  a.dbias = ptr<float>(dbias);
  a.tau = (float)tau;
  a.q_scale = (float)q_scale;
  a.H = (int)H, a.N = (int)N, a.P = (int)PS, a.vcols = (int)P, a.hpg = (int)hpg;
  a.state = ptr<float>(state);
  a.state_stride = state.stride(0);
  a.prev_row = ptr<int>(prev_row);
  a.save_slot = ptr<int>(save_slot);
  a.runs = (int)runs, a.T = (int)T;
  a.out = ptr<float>(out);
  launch_decay_scan(a, f32, cur_stream(v));
}

void gated_group_norm(const Tensor& y, const Tensor& gate, const Tensor& w, double eps, int64_t group, bool gate_first,
                      Tensor& out) {
  const int f32 = act(out, "out");
  dtype(y, at::kFloat, "y");
  dtype(w, at::kFloat, "w");
  TORCH_CHECK(y.dim() == 2, "gated_group_norm: y [T, C]");
  const int64_t T = y.size(0), C = y.size(1);
  const int64_t ldg = view2(gate, f32, T, C, "gate");
  TORCH_CHECK(group > 0 && C % group == 0 && w.numel() > 0 && C % w.numel() == 0 && out.numel() == T * C &&
                  C / group <= 65535, "gated_group_norm: shapes");
  launch_gated_group_norm(ptr<float>(y), gate.data_ptr(), ldg, ptr<float>(w), (int)w.numel(), (float)eps, (int)group,
                          gate_first ? 1 : 0, out.data_ptr(), (int)T, (int)C, f32, cur_stream(y));
}

ConvArgs conv_args(const Tensor& xin, const OptTensor& w, const OptTensor& b, Tensor& state, const OptTensor& cu_q,
                   const OptTensor& row_seq, const Tensor& prev_row, const OptTensor& save_slot, int64_t runs, int f32) {
  TORCH_CHECK(xin.dim() == 2 && state.dim() == 3, "conv: xin [T, C], state [slots, taps - 1, C]");
  const int64_t T = xin.size(0), C = xin.size(1);
  ConvArgs a{};
  a.ldx = view2(xin, f32, T, C, "xin");
  same_act(state, f32, "state");
  TORCH_CHECK(state.size(2) == C && state.size(1) + 1 <= 16, "conv: state shape (at most 16 taps)");
  a.taps = (int)state.size(1) + 1;
  dtype(prev_row, at::kInt, "prev_row");
  TORCH_CHECK(prev_row.numel() >= T, "conv: prev_row too short");
  if (w.has_value()) {
    same_act(*w, f32, "w");
    TORCH_CHECK(w->dim() == 2 && w->size(0) == C && w->size(1) == a.taps, "conv: w [C, taps]");
    a.w = w->data_ptr();
  }
  if (b.has_value()) {
    dtype(*b, at::kFloat, "b");
    TORCH_CHECK(b->numel() == C, "conv: b [C]");
    a.b = ptr<float>(*b);
  }
  if (cu_q.has_value()) {
    dtype(*cu_q, at::kInt, "cu_q");
    TORCH_CHECK(cu_q->numel() >= runs + 1, "conv: cu_q too short");
    a.cu_q = ptr<int>(*cu_q);
    if (row_seq.has_value()) {
      dtype(*row_seq, at::kInt, "row_seq");
      TORCH_CHECK(row_seq->numel() >= T, "conv: row_seq too short");
      a.row_seq = ptr<int>(*row_seq);
    }
  } else {
    TORCH_CHECK(runs <= T, "conv: more runs than rows");
  }
  if (save_slot.has_value()) {
    dtype(*save_slot, at::kInt, "save_slot");
    TORCH_CHECK(save_slot->numel() >= T, "conv: save_slot too short");
    a.save_slot = ptr<int>(*save_slot);
  }
  a.prev_row = ptr<int>(prev_row);
  a.xin = xin.data_ptr();
  a.state = state.data_ptr();
  a.state_stride = state.stride(0);
  a.T = (int)T, a.C = (int)C, a.runs = (int)runs;
  TORCH_CHECK(T <= 65535 * 64 && runs <= 65535 * 64, "conv: too many rows");
  return a;
}

void causal_conv_silu(const Tensor& xin, const Tensor& w, const Tensor& b, Tensor& state, const OptTensor& cu_q,
                      const OptTensor& row_seq, const Tensor& prev_row, int64_t runs, Tensor& out) {
  const int f32 = act(out, "out");
  ConvArgs a = conv_args(xin, w, b, state, cu_q, row_seq, prev_row, std::nullopt, runs, f32);
  TORCH_CHECK(!cu_q.has_value() || row_seq.has_value(), "causal_conv_silu: cu_q without row_seq");
  TORCH_CHECK(out.numel() == (int64_t)a.T * a.C, "causal_conv_silu: out shape");
  a.out = out.data_ptr();
  launch_causal_conv_silu(a, f32, cur_stream(out));
}

void conv_state_update(const Tensor& xin, Tensor& state, const OptTensor& cu_q, const Tensor& prev_row,
                       const Tensor& save_slot, int64_t runs) {
  const int f32 = act(xin, "xin", false);
  ConvArgs a = conv_args(xin, std::nullopt, std::nullopt, state, cu_q, std::nullopt, prev_row, save_slot, runs, f32);
  launch_conv_state_update(a, f32, cur_stream(xin));
}

void relu_sq(const Tensor& a, Tensor& out) {
  const int f32 = act(out, "out");
  TORCH_CHECK(out.dim() == 2, "relu_sq: out [R, F]");
  const int64_t lda = view2(a, f32, out.size(0), out.size(1), "a");
  launch_relu_sq(a.data_ptr(), lda, out.data_ptr(), (int)out.size(0), (int)out.size(1), f32, cur_stream(out));
}

void silu_mul(const Tensor& gate, const Tensor& up, Tensor& out) {
  const int f32 = act(out, "out");
  TORCH_CHECK(out.dim() == 2, "silu_mul: out [R, F]");
  const int64_t ldg = view2(gate, f32, out.size(0), out.size(1), "gate");
  const int64_t ldu = view2(up, f32, out.size(0), out.size(1), "up");
  launch_silu_mul(gate.data_ptr(), ldg, up.data_ptr(), ldu, out.data_ptr(), (int)out.size(0), (int)out.size(1), f32,
                  cur_stream(out));
}

void softmax_topk(const Tensor& x, const Tensor& Wr, const OptTensor& corr, int64_t k, Tensor& ids, Tensor& w,
                  int64_t groups, int64_t keep, bool renorm) {
  const int f32 = act(x, "x");
  same_act(Wr, f32, "Wr");
  if (corr.has_value()) dtype(*corr, at::kFloat, "corr");
  dtype(ids, at::kInt, "ids");
  dtype(w, at::kFloat, "w");
  TORCH_CHECK(x.dim() == 2 && Wr.dim() == 2, "softmax_topk: x [T, d], Wr [En, d]");
  const int64_t T = x.size(0), d = x.size(1), En = Wr.size(0);
  TORCH_CHECK(Wr.size(1) == d && (!corr.has_value() || corr->numel() == En) && k >= 1 && k <= En && En <= 4096 &&
                  ids.numel() >= T * k && w.numel() >= T * k, "softmax_topk: shapes");
  TORCH_CHECK(groups >= 1 && groups <= 64 && En % groups == 0 && keep >= 1 && keep <= groups && k <= keep * (En / groups),
              "softmax_topk: groups (at most 64, equal sizes) / keep / k");
  launch_softmax_topk(x.data_ptr(), Wr.data_ptr(), optptr<float>(corr), (int)T, (int)d, (int)En, (int)k, (int)groups,
                      (int)keep, renorm ? 1 : 0, ptr<int>(ids), ptr<float>(w), f32, cur_stream(x));
}

void moe_mix(const Tensor& y, const Tensor& dst, const Tensor& ids, const Tensor& w, int64_t k, int64_t E, const Tensor& h,
             const OptTensor& shared, const OptTensor& sgate, Tensor& out) {
  const int f32 = act(y, "y");
  same_act(h, f32, "h");
  dtype(dst, at::kInt, "dst");
  dtype(ids, at::kInt, "ids");
  dtype(w, at::kFloat, "w");
  dtype(out, at::kFloat, "out");
  TORCH_CHECK(out.dim() == 2 && y.dim() == 2, "moe_mix: out [T, d], y [R, d]");
  const int64_t T = out.size(0), d = out.size(1);
  TORCH_CHECK(y.size(1) == d && y.size(0) >= T * k && h.numel() == T * d && dst.numel() >= T * k && ids.numel() >= T * k &&
                  w.numel() >= T * k, "moe_mix: shapes");
  int64_t ldsg = 0;
  if (shared.has_value()) {
    same_act(*shared, f32, "shared");
    TORCH_CHECK(shared->numel() == T * d && sgate.has_value(), "moe_mix: shared [T, d] with its gate");
    ldsg = view2(*sgate, f32, T, 1, "sgate");
    if (T > 1) ldsg = sgate->stride(0);
  }
  launch_moe_mix(y.data_ptr(), ptr<int>(dst), ptr<int>(ids), ptr<float>(w), (int)k, (int)E, h.data_ptr(),
                 shared.has_value() ? shared->data_ptr() : nullptr, sgate.has_value() ? sgate->data_ptr() : nullptr, ldsg,
                 ptr<float>(out), (int)T, (int)d, f32, cur_stream(out));
}

// ---- expert segments (kernels of glu_moe.hip) -----------------------------------------------------------------
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

// ---- post-norm stream, input convolutions, normed grouped heads ---------------------------------------------------
void embed_scale(const Tensor& ids, const OptTensor& src, const OptTensor& prev, const Tensor& table, double scale,
                 Tensor& x) {
  const int f32 = act(table, "table");
  dtype(ids, at::kInt, "ids");
  dtype(x, at::kFloat, "x");
  const int64_t T = ids.numel(), d = table.size(1);
  TORCH_CHECK(table.dim() == 2 && x.numel() == T * d, "embed_scale: shapes");
  if (src.has_value()) {
    TORCH_CHECK(prev.has_value(), "embed_scale: src without prev");
    dtype(*src, at::kInt, "src");
    dtype(*prev, at::kInt, "prev");
    TORCH_CHECK(src->numel() >= T, "embed_scale: src too short");
  }
  launch_embed_scale(ptr<int>(ids), optptr<int>(src), optptr<int>(prev), table.data_ptr(), (float)scale, ptr<float>(x),
                     (int)T, (int)d, f32, cur_stream(x));
}

void residual_conv(const Tensor& x, const Tensor& w, Tensor& state, const OptTensor& cu_q, const OptTensor& row_seq,
                   const Tensor& prev_row, const OptTensor& save_slot, int64_t runs, Tensor& out) {
  const int f32 = act(out, "out");
  dtype(x, at::kFloat, "x");
  dtype(w, at::kFloat, "w");
  dtype(state, at::kFloat, "state");
  // (the taps are tap-major here, [taps, C]: conv_args checks the channel-major form of causal_conv_silu)
  ConvArgs a = conv_args(x, std::nullopt, std::nullopt, state, cu_q, row_seq, prev_row, save_slot, runs, 1);
  TORCH_CHECK(w.dim() == 2 && w.size(0) == a.taps && w.size(1) == a.C, "residual_conv: w [taps, C]");
  a.w = w.data_ptr();
  TORCH_CHECK(!cu_q.has_value() || row_seq.has_value(), "residual_conv: cu_q without row_seq");
  TORCH_CHECK(!(cu_q.has_value() && save_slot.has_value()), "residual_conv: the taps move on in this launch only where "
              "every row is a run of its own");
  TORCH_CHECK(out.numel() == (int64_t)a.T * a.C, "residual_conv: out shape");
  a.out = out.data_ptr();
  launch_residual_conv(a, f32, cur_stream(out));
}

void post_rms_norm(Tensor& x, double alpha, const Tensor& delta, const Tensor& w, double eps, const OptTensor& conv_w,
                   OptTensor conv_state, const OptTensor& prev_row, const OptTensor& save_slot, OptTensor h) {
  const int f32 = act(delta, "delta");
  dtype(x, at::kFloat, "x");
  dtype(w, at::kFloat, "w");
  TORCH_CHECK(x.dim() == 2 && delta.numel() == x.numel() && w.numel() == x.size(1), "post_rms_norm: x [T, d], delta [T, d]");
  const int64_t T = x.size(0), d = x.size(1);
  NormConvArgs cv{};
  if (h.has_value()) {
    TORCH_CHECK(conv_w.has_value() && conv_state.has_value() && prev_row.has_value() && save_slot.has_value(),
                "post_rms_norm: the convolution needs its taps, state, prev_row and save_slot");
    same_act(*h, f32, "h");
    dtype(*conv_w, at::kFloat, "conv_w");
    dtype(*conv_state, at::kFloat, "conv_state");
    dtype(*prev_row, at::kInt, "prev_row");
    dtype(*save_slot, at::kInt, "save_slot");
    TORCH_CHECK(conv_w->dim() == 2 && conv_w->size(1) == d && conv_state->dim() == 3 && conv_state->size(2) == d &&
                    conv_state->size(1) + 1 == conv_w->size(0) && conv_w->size(0) <= 16 && h->numel() == T * d &&
                    prev_row->numel() >= T && save_slot->numel() >= T, "post_rms_norm: convolution shapes");
    cv.w = ptr<float>(*conv_w);
    cv.state = ptr<float>(*conv_state);
    cv.state_stride = conv_state->stride(0);
    cv.prev_row = ptr<int>(*prev_row);
    cv.save_slot = ptr<int>(*save_slot);
    cv.h = h->data_ptr();
    cv.taps = (int)conv_w->size(0);
  }
  launch_post_rms_norm(ptr<float>(x), (float)alpha, delta.data_ptr(), ptr<float>(w), (float)eps, (int)T, (int)d, cv, f32,
                       cur_stream(x));
}

void qk_norm_cache(const Tensor& z, int64_t H, int64_t G, int64_t dk, int64_t dv, const Tensor& wq, const Tensor& wk,
                   const OptTensor& q_mult, double eps, const Tensor& slots, Tensor& q_out, Tensor& k_cache,
                   Tensor& v_cache) {
  const int f32 = act(z, "z", false);
  TORCH_CHECK(z.dim() == 2, "qk_norm_cache: z [T, n]");
  const int64_t T = z.size(0), n = H * dk + G * dk + G * dv;
  QkNormArgs a{};
  a.ldz = view2(z, f32, T, z.size(1), "z");
  TORCH_CHECK(z.size(1) >= n, "qk_norm_cache: z narrower than q | k | v");
  same_act(q_out, f32, "q_out");
  same_act(k_cache, f32, "k_cache");
  same_act(v_cache, f32, "v_cache");
  dtype(wq, at::kFloat, "wq");
  dtype(wk, at::kFloat, "wk");
  dtype(slots, at::kInt, "slots");
  TORCH_CHECK(wq.numel() == dk && wk.numel() == dk && q_out.numel() == T * H * dk && slots.numel() >= T &&
                  k_cache.dim() == 4 && v_cache.dim() == 4 && k_cache.size(2) == G && k_cache.size(3) == dk &&
                  v_cache.size(2) == G && v_cache.size(3) == dv && G > 0 && H % G == 0 && T <= 65535 * 64 && H + G <= 65535,
              "qk_norm_cache: shapes");
  if (q_mult.has_value()) {
    dtype(*q_mult, at::kFloat, "q_mult");
    TORCH_CHECK(q_mult->numel() == H, "qk_norm_cache: q_mult [H]");
    a.q_mult = ptr<float>(*q_mult);
  }
  a.z = z.data_ptr();
  a.H = (int)H, a.G = (int)G, a.dk = (int)dk, a.dv = (int)dv;
  a.wq = ptr<float>(wq), a.wk = ptr<float>(wk);
  a.eps = (float)eps;
  a.slots = ptr<int>(slots);
  a.q_out = q_out.data_ptr();
  a.k_cache = k_cache.data_ptr();
  a.v_cache = v_cache.data_ptr();
  launch_qk_norm_cache(a, (int)T, f32, cur_stream(z));
}

void gelu_tanh_mul(const Tensor& gate, const Tensor& up, Tensor& out) {
  const int f32 = act(out, "out");
  TORCH_CHECK(out.dim() == 2, "gelu_tanh_mul: out [R, F]");
  const int64_t ldg = view2(gate, f32, out.size(0), out.size(1), "gate");
  const int64_t ldu = view2(up, f32, out.size(0), out.size(1), "up");
  launch_gelu_tanh_mul(gate.data_ptr(), ldg, up.data_ptr(), ldu, out.data_ptr(), (int)out.size(0), (int)out.size(1), f32,
                       cur_stream(out));
}

void sigmoid_mul(const Tensor& a, const Tensor& gate, Tensor& out) {
  const int f32 = act(out, "out");
  TORCH_CHECK(out.dim() == 2, "sigmoid_mul: out [R, F]");
  const int64_t lda = view2(a, f32, out.size(0), out.size(1), "a");
  const int64_t ldg = view2(gate, f32, out.size(0), out.size(1), "gate");
  launch_sigmoid_mul(a.data_ptr(), lda, gate.data_ptr(), ldg, out.data_ptr(), (int)out.size(0), (int)out.size(1), f32,
                     cur_stream(out));
}


// ---- several residual streams, hashed token pairs, convolved projections, the matrix memory's read-out ------------
void embed_pair_hash(const Tensor& ids, const OptTensor& src, const OptTensor& prev, const Tensor& table,
                     const OptTensor& pair_table, int64_t buckets, int64_t mul_prev, int64_t mul_cur, const Tensor& prev_row,
                     Tensor& tok_state, const OptTensor& save_slot, Tensor& x) {
  const int f32 = act(table, "table");
  dtype(ids, at::kInt, "ids");
  dtype(x, at::kFloat, "x");
  dtype(prev_row, at::kInt, "prev_row");
  dtype(tok_state, at::kInt, "tok_state");
  TORCH_CHECK(x.dim() == 3 && table.dim() == 2 && x.size(2) == table.size(1), "embed_pair_hash: x [T, S, d], table [V, d]");
  const int64_t T = x.size(0), S = x.size(1), d = x.size(2);
  TORCH_CHECK(ids.numel() >= T && prev_row.numel() >= T && S >= 1 && S <= 8, "embed_pair_hash: shapes (at most 8 streams)");
  PairHashArgs a{};
  if (src.has_value()) {
    TORCH_CHECK(prev.has_value(), "embed_pair_hash: src without prev");
    dtype(*src, at::kInt, "src");
    dtype(*prev, at::kInt, "prev");
    TORCH_CHECK(src->numel() >= T, "embed_pair_hash: src too short");
    a.src = ptr<int>(*src), a.prev = ptr<int>(*prev);
  }
  if (pair_table.has_value()) {
    same_act(*pair_table, f32, "pair_table");
    TORCH_CHECK(pair_table->dim() == 2 && pair_table->size(0) == buckets + 1 && pair_table->size(1) == d && buckets >= 1,
                "embed_pair_hash: pair_table [buckets + 1, d]");
    a.pair_table = pair_table->data_ptr();
  }
  if (save_slot.has_value()) {
    dtype(*save_slot, at::kInt, "save_slot");
    TORCH_CHECK(save_slot->numel() >= T, "embed_pair_hash: save_slot too short");
    a.save_slot = ptr<int>(*save_slot);
  }
  a.ids = ptr<int>(ids);
  a.table = table.data_ptr();
  a.buckets = buckets, a.mul_prev = mul_prev, a.mul_cur = mul_cur;
  a.prev_row = ptr<int>(prev_row);
  a.tok_state = ptr<int>(tok_state);
  a.x = ptr<float>(x);
  a.T = (int)T, a.S = (int)S, a.d = (int)d;
  launch_embed_pair_hash(a, f32, cur_stream(x));
}

void token_state_update(const Tensor& ids, Tensor& tok_state, const OptTensor& cu_q, const Tensor& save_slot, int64_t runs) {
  dtype(ids, at::kInt, "ids");
  dtype(tok_state, at::kInt, "tok_state");
  dtype(save_slot, at::kInt, "save_slot");
  if (cu_q.has_value()) {
    dtype(*cu_q, at::kInt, "cu_q");
    TORCH_CHECK(cu_q->numel() >= runs + 1, "token_state_update: cu_q too short");
  } else {
    TORCH_CHECK(runs <= ids.numel(), "token_state_update: more runs than rows");
  }
  launch_token_state_update(ptr<int>(ids), ptr<int>(tok_state), optptr<int>(cu_q), ptr<int>(save_slot), (int)runs,
                            cur_stream(ids));
}

void hyper_mix_norm(Tensor& xs, const OptTensor& a_, double sa, const OptTensor& b_, double sb, const OptTensor& mix,
                    const OptTensor& outc, const OptTensor& inc, const OptTensor& w, double eps, const OptTensor& rows,
                    const OptTensor& out) {
  dtype(xs, at::kFloat, "xs");
  TORCH_CHECK(xs.dim() == 3, "hyper_mix_norm: xs [T, S, d]");
  const int64_t T = xs.size(0), S = xs.size(1), d = xs.size(2);
  TORCH_CHECK(S >= 1 && S <= 8 && d >= 1 && d <= 15000, "hyper_mix_norm: at most 8 streams, width at most 15000");
  HyperMixArgs a{};
  a.xs = ptr<float>(xs);
  a.T = (int)T, a.S = (int)S, a.d = (int)d;
  if (a_.has_value()) {
    a.a_f32 = act(*a_, "a");
    TORCH_CHECK(a_->numel() == T * d && mix.has_value() && outc.has_value() && !rows.has_value(),
                "hyper_mix_norm: a [T, d] with mix and outc, no gathered rows");
    dtype(*mix, at::kFloat, "mix");
    dtype(*outc, at::kFloat, "outc");
    TORCH_CHECK(mix->numel() == S * S && outc->numel() == S, "hyper_mix_norm: mix [S, S], outc [S]");
    a.a = a_->data_ptr(), a.sa = (float)sa, a.mix = ptr<float>(*mix), a.outc = ptr<float>(*outc);
    if (b_.has_value()) {
      a.b_f32 = act(*b_, "b");
      TORCH_CHECK(b_->numel() == T * d, "hyper_mix_norm: b [T, d]");
      a.b = b_->data_ptr(), a.sb = (float)sb;
    }
  }
  int f32 = 0;
  if (out.has_value()) {
    f32 = act(*out, "out");
    TORCH_CHECK(out->dim() == 2 && out->size(1) == d && w.has_value(), "hyper_mix_norm: out [n, d] with w");
    dtype(*w, at::kFloat, "w");
    TORCH_CHECK(w->numel() == d, "hyper_mix_norm: w [d]");
    a.n = (int)out->size(0);
    if (rows.has_value()) {
      dtype(*rows, at::kLong, "rows");
      TORCH_CHECK(rows->numel() >= a.n, "hyper_mix_norm: rows too short");
      a.rows = reinterpret_cast<const long long*>(rows->data_ptr());
    } else {
      TORCH_CHECK(a.n <= T, "hyper_mix_norm: more output rows than rows");
    }
    if (inc.has_value()) {
      dtype(*inc, at::kFloat, "inc");
      TORCH_CHECK(inc->numel() == S, "hyper_mix_norm: inc [S]");
      a.inc = ptr<float>(*inc);
    }
    a.w = ptr<float>(*w), a.eps = (float)eps, a.out = out->data_ptr();
  }
  TORCH_CHECK(T <= 65535 * 1024 && a.n <= 65535 * 1024, "hyper_mix_norm: too many rows");
  launch_hyper_mix_norm(a, f32, cur_stream(xs));
}

void conv_qkv_cache(const Tensor& z, const Tensor& w, Tensor& state, const OptTensor& cu_q, const OptTensor& row_seq,
                    const Tensor& prev_row, const OptTensor& save_slot, int64_t runs, int64_t H, int64_t G, int64_t dk,
                    int64_t dv, double v_eps, const Tensor& slots, Tensor& q_out, Tensor& k_cache, Tensor& v_cache) {
  const int f32 = act(z, "z", false);
  TORCH_CHECK(z.dim() == 2 && state.dim() == 3 && w.dim() == 2, "conv_qkv_cache: z [T, C], w [C, taps], state [slots, taps - 1, C]");
  const int64_t T = z.size(0), C = H * dk + G * dk + G * dv;
  ConvQkvArgs a{};
  a.ldz = view2(z, f32, T, C, "z");
  same_act(w, f32, "w");
  same_act(state, f32, "state");
  same_act(q_out, f32, "q_out");
  same_act(k_cache, f32, "k_cache");
  same_act(v_cache, f32, "v_cache");
  dtype(prev_row, at::kInt, "prev_row");
  dtype(slots, at::kInt, "slots");
  const int64_t taps = w.size(1);
  TORCH_CHECK(w.size(0) == C && taps >= 1 && taps <= 16 && state.size(1) == taps - 1 && state.size(2) == C && dk <= 512 &&
                  dv <= 512 && H + 2 * G <= 65535 && H % G == 0 && q_out.numel() == T * H * dk && prev_row.numel() >= T &&
                  slots.numel() >= T && k_cache.dim() == 4 && v_cache.dim() == 4 && k_cache.size(2) == G &&
                  k_cache.size(3) == dk && v_cache.size(2) == G && v_cache.size(3) == dv && T <= 65535 * 1024,
              "conv_qkv_cache: shapes (at most 16 taps, heads at most 512 wide)");
  if (cu_q.has_value()) {
    TORCH_CHECK(row_seq.has_value(), "conv_qkv_cache: cu_q without row_seq");
    dtype(*cu_q, at::kInt, "cu_q");
    dtype(*row_seq, at::kInt, "row_seq");
    TORCH_CHECK(cu_q->numel() >= runs + 1 && row_seq->numel() >= T, "conv_qkv_cache: cu_q / row_seq too short");
    a.cu_q = ptr<int>(*cu_q), a.row_seq = ptr<int>(*row_seq);
  } else {
    TORCH_CHECK(runs <= T, "conv_qkv_cache: more runs than rows");
  }
  if (save_slot.has_value()) {
    TORCH_CHECK(!cu_q.has_value(), "conv_qkv_cache: save_slot only where every row is a run of its own");
    dtype(*save_slot, at::kInt, "save_slot");
    TORCH_CHECK(save_slot->numel() >= T, "conv_qkv_cache: save_slot too short");
    a.save_slot = ptr<int>(*save_slot);
  }
  a.z = z.data_ptr(), a.w = w.data_ptr(), a.state = state.data_ptr();
  a.state_stride = state.stride(0);
  a.prev_row = ptr<int>(prev_row), a.slots = ptr<int>(slots);
  a.q_out = q_out.data_ptr(), a.k_cache = k_cache.data_ptr(), a.v_cache = v_cache.data_ptr();
  a.v_eps = (float)v_eps;
  a.T = (int)T, a.C = (int)C, a.taps = (int)taps, a.H = (int)H, a.G = (int)G, a.dk = (int)dk, a.dv = (int)dv;
  launch_conv_qkv_cache(a, f32, cur_stream(z));
}

void memory_norm_gate(const Tensor& y, const Tensor& m, const Tensor& gate, const Tensor& w, double eps, Tensor& out) {
  const int f32 = act(out, "out");
  dtype(y, at::kFloat, "y");
  dtype(m, at::kFloat, "m");
  dtype(w, at::kFloat, "w");
  TORCH_CHECK(y.dim() == 3 && y.size(2) >= 2, "memory_norm_gate: y [T, H, P + 1]");
  const int64_t T = y.size(0), H = y.size(1), P = y.size(2) - 1;
  const int64_t ldg = view2(gate, f32, T, H * P, "gate");
  TORCH_CHECK(m.numel() == T * H && w.numel() == H * P && out.numel() == T * H * P && H <= 65535 && T <= 65535 * 1024,
              "memory_norm_gate: shapes");
  launch_memory_norm_gate(ptr<float>(y), ptr<float>(m), gate.data_ptr(), ldg, ptr<float>(w), (float)eps, out.data_ptr(),
                          (int)T, (int)H, (int)P, f32, cur_stream(y));
}

void hyb_clamped_glu(const Tensor& gu, double limit, double alpha, Tensor& out) {
  const int f32 = act(gu, "gu");
  same_act(out, f32, "out");
  TORCH_CHECK(gu.dim() == 2 && out.dim() == 2 && gu.size(0) == out.size(0) && gu.size(1) == 2 * out.size(1),
              "clamped_glu: gu [R, 2F], out [R, F]");
  launch_clamped_glu(gu.data_ptr(), out.data_ptr(), (int)out.size(0), (int)out.size(1), (float)limit, (float)alpha, f32,
                     cur_stream(gu));
}

void logit_softcap(Tensor& logits, double cap) {
  dtype(logits, at::kFloat, "logits");
  TORCH_CHECK(cap > 0, "logit_softcap: cap");
  launch_logit_softcap(ptr<float>(logits), logits.numel(), (float)cap, cur_stream(logits));
}

}  // namespace

TORCH_LIBRARY(symmetry_amd_hybrid, m) {
  m.def("embed_norm(Tensor ids, Tensor? src, Tensor? prev, Tensor table, Tensor w, float eps, float offset, Tensor(a!) x) -> ()",
        &embed_norm);
  m.def("rms_norm_rows(Tensor x, Tensor? rows, Tensor w, float eps, float offset, Tensor(a!) out) -> ()", &rms_norm_rows);
  m.def(
      "residual_mix_norm(Tensor(a!) x, Tensor a, float sa, Tensor? bias_a, Tensor? b, float sb, Tensor? c, float sc, "
      "Tensor? w, float eps, float offset, Tensor(b!)? out) -> ()",
      &residual_mix_norm);
  m.def(
      "qkv_rope_cache(Tensor z, Tensor? bias, int H, int G, int dk, int dv, Tensor positions, Tensor slots, Tensor? rope, "
      "Tensor(a!) q_out, Tensor(b!) k_cache, Tensor(c!) v_cache, int half_dims) -> ()",
      &qkv_rope_cache);
  m.def(
      "window_attn(Tensor q, Tensor k_cache, Tensor v_cache, Tensor block_tables, Tensor row_seq, Tensor positions, "
      "int window, float scale, Tensor? gate, Tensor(a!) out, Tensor? tiles, Tensor? cu_q, int impl, Tensor? bias, "
      "int keep_first, Tensor? sink) -> int",
      &window_attn);
  m.def(
      "decay_scan(int mode, Tensor q, Tensor k, Tensor v, Tensor dz, Tensor dbias, Tensor? rate, float tau, Tensor? skip, "
      "float q_scale, int H, int N, int P, int hpg, Tensor(a!) state, Tensor? cu_q, Tensor prev_row, Tensor save_slot, "
      "int runs, Tensor(b!) out, Tensor(c!)? mout) -> ()",
      &decay_scan);
  m.def("gated_group_norm(Tensor y, Tensor gate, Tensor w, float eps, int group, bool gate_first, Tensor(a!) out) -> ()",
        &gated_group_norm);
  m.def(
      "causal_conv_silu(Tensor xin, Tensor w, Tensor b, Tensor(a!) state, Tensor? cu_q, Tensor? row_seq, Tensor prev_row, "
      "int runs, Tensor(b!) out) -> ()",
      &causal_conv_silu);
  m.def("conv_state_update(Tensor xin, Tensor(a!) state, Tensor? cu_q, Tensor prev_row, Tensor save_slot, int runs) -> ()",
        &conv_state_update);
  m.def("relu_sq(Tensor a, Tensor(a!) out) -> ()", &relu_sq);
  m.def("silu_mul(Tensor gate, Tensor up, Tensor(a!) out) -> ()", &silu_mul);
  m.def(
      "softmax_topk(Tensor x, Tensor Wr, Tensor? corr, int k, Tensor(a!) ids, Tensor(b!) w, int groups, int keep, "
      "bool renorm) -> ()",
      &softmax_topk);
  m.def(
      "moe_mix(Tensor y, Tensor dst, Tensor ids, Tensor w, int k, int E, Tensor h, Tensor? shared, Tensor? sgate, "
      "Tensor(a!) out) -> ()",
      &moe_mix);
  m.def("expert_offsets(Tensor ids, int R, int E, Tensor(a!) offsets, Tensor(b!) cursor) -> ()", &expert_offsets);
  m.def(
      "scatter_scaled(Tensor x, Tensor ids, Tensor w, int k, Tensor offsets, Tensor(a!) cursor, Tensor(b!) xs, "
      "Tensor(c!) dst) -> ()",
      &scatter_scaled);
  m.def("grouped_linear(Tensor xs, Tensor W, Tensor offsets, Tensor(a!) y) -> ()", &grouped_linear);
  m.def("embed_scale(Tensor ids, Tensor? src, Tensor? prev, Tensor table, float scale, Tensor(a!) x) -> ()", &embed_scale);
  m.def(
      "residual_conv(Tensor x, Tensor w, Tensor(a!) state, Tensor? cu_q, Tensor? row_seq, Tensor prev_row, "
      "Tensor? save_slot, int runs, "
      "Tensor(b!) out) -> ()",
      &residual_conv);
  m.def(
      "post_rms_norm(Tensor(a!) x, float alpha, Tensor delta, Tensor w, float eps, Tensor? conv_w, Tensor(b!)? conv_state, "
      "Tensor? prev_row, Tensor? save_slot, Tensor(c!)? h) -> ()",
      &post_rms_norm);
  m.def(
      "qk_norm_cache(Tensor z, int H, int G, int dk, int dv, Tensor wq, Tensor wk, Tensor? q_mult, float eps, Tensor slots, "
      "Tensor(a!) q_out, Tensor(b!) k_cache, Tensor(c!) v_cache) -> ()",
      &qk_norm_cache);
  m.def("gelu_tanh_mul(Tensor gate, Tensor up, Tensor(a!) out) -> ()", &gelu_tanh_mul);
  m.def("sigmoid_mul(Tensor a, Tensor gate, Tensor(a!) out) -> ()", &sigmoid_mul);
  m.def(
      "embed_pair_hash(Tensor ids, Tensor? src, Tensor? prev, Tensor table, Tensor? pair_table, int buckets, int mul_prev, "
      "int mul_cur, Tensor prev_row, Tensor(a!) tok_state, Tensor? save_slot, Tensor(b!) x) -> ()",
      &embed_pair_hash);
  m.def("token_state_update(Tensor ids, Tensor(a!) tok_state, Tensor? cu_q, Tensor save_slot, int runs) -> ()",
        &token_state_update);
  m.def(
      "hyper_mix_norm(Tensor(a!) xs, Tensor? a, float sa, Tensor? b, float sb, Tensor? mix, Tensor? outc, Tensor? inc, "
      "Tensor? w, float eps, Tensor? rows, Tensor(b!)? out) -> ()",
      &hyper_mix_norm);
  m.def(
      "conv_qkv_cache(Tensor z, Tensor w, Tensor(a!) state, Tensor? cu_q, Tensor? row_seq, Tensor prev_row, "
      "Tensor? save_slot, int runs, int H, int G, int dk, int dv, float v_eps, Tensor slots, Tensor(b!) q_out, "
      "Tensor(c!) k_cache, Tensor(d!) v_cache) -> ()",
      &conv_qkv_cache);
  m.def("memory_norm_gate(Tensor y, Tensor m, Tensor gate, Tensor w, float eps, Tensor(a!) out) -> ()", &memory_norm_gate);
  m.def("clamped_glu(Tensor gu, float limit, float alpha, Tensor(a!) out) -> ()", &hyb_clamped_glu);
  m.def("logit_softcap(Tensor(a!) logits, float cap) -> ()", &logit_softcap);
}
