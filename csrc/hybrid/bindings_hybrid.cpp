// bindings_hybrid.cpp — registers the hybrid-decoder kernels (csrc/hybrid/*.hip) as torch.ops.chronos.hy_*.
//
// A library of its own (_H), so a model of this family compiles and loads only these kernels.  As in
// csrc/kernels/bindings.cpp every op checks dtypes, shapes and contiguity on the host before launching and launches on
// the current HIP stream (graph-capturable; outputs come from torch's caching allocator).
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include <hip/hip_runtime.h>
#include <cstdint>
#include <tuple>

namespace chronos {
void launch_hy_embed(const int32_t*, const void*, float*, int, int, float, bool, hipStream_t);
void launch_hy_cast_bf16(const float*, uint16_t*, int64_t, hipStream_t);
void launch_hy_layer_norm(const void*, bool, float*, const float*, void*, bool, int, int, float, hipStream_t);
void launch_hy_rowdot(const void*, const void*, const float*, float*, int, int, int, bool, hipStream_t);
void launch_hy_act(void*, int64_t, int, bool, hipStream_t);
void launch_hy_mlstm_scan(const void*, int, const float*, const int32_t*, const int32_t*, const int32_t*, float*, float*,
                          float*, float*, float*, float*, float*, int, int, int, int, float, bool, hipStream_t);
void launch_hy_mlstm_out(const float*, const void*, int, int, const float*, void*, int, int, int, float, bool,
                         hipStream_t);
void launch_hy_latent_prep(void*, const void*, const int32_t*, const int32_t*, const int32_t*, int, const float*, float,
                           const float*, int, int, int, int, int, void*, int, int, bool, hipStream_t);
bool launch_hy_latent_attention(const void*, const void*, const int32_t*, int, const int32_t*, const int32_t*,
                                const float*, void*, int, int, int, int, int, int, float, bool, int, float*, float*, int64_t,
                                hipStream_t);
bool hy_latent_use_mfma(bool, int, int);
int hy_latent_nsplit(int, int);
void launch_hy_moe_route(const void*, const void*, const float*, float*, int32_t*, float*, int, int, int, int, bool,
                         hipStream_t);
void launch_hy_moe_ffn_token(const void*, const int32_t*, const float*, const void*, const void*, void*, int, int, int,
                             int, int, int, bool, hipStream_t);
int hy_moe_max_tiles(int, int);
void launch_hy_moe_grouped(const uint16_t*, const int32_t*, const float*, const uint16_t*, const uint16_t*, uint16_t*,
                           int32_t*, uint16_t*, uint16_t*, int, int, int, int, int, int, hipStream_t);
void launch_hy_rms_norm(const void*, float*, const float*, void*, bool, int, int, float, float, hipStream_t);
void launch_hy_glu(const void*, void*, int64_t, int, float, float, float, bool, hipStream_t);
void launch_hy_decay_pow(float*, int64_t, float, hipStream_t);
void launch_hy_head_norm_gate(const float*, const void*, int, int, const float*, void*, int, int, int, float, bool, bool,
                              hipStream_t);
void launch_hy_window_prep(void*, int, int, int, int, int, const void*, const float*, const int32_t*, const int32_t*,
                           const int32_t*, int, const float*, const float*, float, const float*, int, void*, void*, int,
                           void*, int, const float*, int, bool, hipStream_t);
void launch_hy_pool_blocks(const void*, const void*, void*, void*, const int32_t*, int, const int32_t*, const int32_t*, int,
                           int, int, int, int, int, int, bool, hipStream_t);
void launch_hy_sandwich_join(const void*, const void*, float*, const float*, const float*, const float*, const float*,
                             void*, int, int, int, float, bool, bool, hipStream_t);
bool hy_sandwich_groups_ok(int, int);
void launch_hy_rotate_qk(void*, int, int, int, int, int, int, int, const float*, const int32_t*, float, float, int, bool,
                         hipStream_t);
void launch_hy_unrotate_gate(const void*, const int32_t*, const float*, const void*, int, int, void*, int, int, int, bool,
                             hipStream_t);
int hy_window_rows_cap(int, int, int, bool);
void launch_hy_window_attention(const void*, int, const void*, const void*, const int32_t*, int, const int32_t*,
                                const int32_t*, const float*, const float*, void*, int, int, int, int, int, int, int, float,
                                int, int, int, bool, int, float*, float*, int64_t, int, int, const void*, const void*, const float*, int, hipStream_t);
int hy_window_nsplit(bool, int, int, int, int, int, int, int, int, int, int, int, int);
void launch_hy_short_conv(const void*, int, const float*, const float*, const int32_t*, const int32_t*, const int32_t*,
                          const int32_t*, void*, void*, int, int, int, int, bool, bool, hipStream_t);
void launch_hy_delta_prep(const void*, int, const float*, const float*, float*, float*, float*, float*, int, int, int, int,
                          float, bool, hipStream_t);
bool launch_hy_linear_scan(const void*, int, int, int, int, const float*, const float*, float, const float*, bool, bool,
                           const float*, const int32_t*, const int32_t*, const int32_t*, float*, float*, int, int, int, int,
                           int, int, const float*, bool, hipStream_t);
void launch_hy_moe_route_topk(const void*, const void*, const float*, float*, int32_t*, float*, int, int, int, int, bool,
                              hipStream_t);
void launch_hy_moe_glu_grouped(const uint16_t*, const int32_t*, const float*, const uint16_t*, const uint16_t*, uint16_t*,
                               int32_t*, uint16_t*, uint16_t*, int, int, int, int, int, float, float, float, hipStream_t);
void launch_hy_moe_glu_token(const void*, const int32_t*, const float*, const void*, const void*, void*, int, int, int,
                             int, int, float, float, float, bool, bool, hipStream_t);
void launch_hy_add_rms_norm(const void*, const void*, const float*, const float*, float*, const float*, void*, int, int,
                            float, int, bool, hipStream_t);
void launch_hy_token_gate(const void*, const int32_t*, const void*, int, int, void*, int, int, bool, hipStream_t);
void launch_hy_ssm_prep(const float*, const float*, float*, float*, int, int, hipStream_t);
void launch_hy_gated_group_norm(const float*, const void*, int, int, const float*, const void*, int, int, const float*,
                                void*, int, int, int, int, float, bool, hipStream_t);
int hy_rglru_chunks(int);
void launch_hy_rglru_scan(const void*, const float*, const float*, float, const void*, int, int, const int32_t*,
                          const int32_t*, const int32_t*, float*, float*, float*, void*, int, int, int, int, int, bool,
                          hipStream_t);
void launch_hy_moe_route_group(const void*, const void*, float*, int32_t*, float*, int, int, int, int, int, int, float, bool,
                               hipStream_t);
}  // namespace chronos

namespace {

using at::Tensor;

hipStream_t stream() { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

void need(bool ok, const char* what) { TORCH_CHECK(ok, "chronos hybrid op: ", what); }

bool is_act(const Tensor& t) { return t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat; }
bool f32(const Tensor& t) { return t.scalar_type() == at::kFloat; }
void same_act(const Tensor& a, const Tensor& b, const char* what) {
    need(is_act(a) && a.scalar_type() == b.scalar_type(), what);
}
void i32(const Tensor& t, const char* what) { need(t.scalar_type() == at::kInt && t.is_contiguous() && t.is_cuda(), what); }
void flt(const Tensor& t, const char* what) { need(t.scalar_type() == at::kFloat && t.is_contiguous() && t.is_cuda(), what); }

Tensor hy_embed(const Tensor& ids, const Tensor& table, double scale) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(table.device());
    i32(ids, "embed: ids must be contiguous int32");
    need(is_act(table) && table.dim() == 2 && table.is_contiguous(), "embed: table [V, d] bf16 or f32");
    auto x = at::empty({ids.numel(), table.size(1)}, table.options().dtype(at::kFloat));
    chronos::launch_hy_embed(ids.data_ptr<int32_t>(), table.data_ptr(), x.data_ptr<float>(), (int)ids.numel(),
                             (int)table.size(1), (float)scale, f32(table), stream());
    return x;
}

Tensor hy_cast_bf16(const Tensor& x) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
    flt(x, "cast: float32 contiguous input");
    auto y = at::empty_like(x, x.options().dtype(at::kBFloat16));
    chronos::launch_hy_cast_bf16(x.data_ptr<float>(), (uint16_t*)y.data_ptr(), x.numel(), stream());
    return y;
}

Tensor hy_layer_norm(const Tensor& x, const Tensor& w, double eps, bool out_f32) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
    flt(x, "layer_norm: float32 rows");
    flt(w, "layer_norm: float32 weight");
    need(x.dim() == 2 && w.numel() == x.size(1), "layer_norm: weight size");
    auto h = at::empty_like(x, x.options().dtype(out_f32 ? at::kFloat : at::kBFloat16));
    chronos::launch_hy_layer_norm(x.data_ptr(), true, nullptr, w.data_ptr<float>(), h.data_ptr(), out_f32,
                                  (int)x.size(0), (int)x.size(1), (float)eps, stream());
    return h;
}

Tensor hy_add_layer_norm(const Tensor& y, Tensor& x, const Tensor& w, double eps, bool out_f32) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
    flt(x, "add_layer_norm: float32 residual");
    flt(w, "add_layer_norm: float32 weight");
    need(is_act(y) && y.is_contiguous() && y.dim() == 2 && y.sizes() == x.sizes(), "add_layer_norm: y shape");
    need(f32(y) == out_f32, "add_layer_norm: y must be in the activation dtype");
    need(w.numel() == x.size(1), "add_layer_norm: weight size");
    Tensor h = out_f32 ? at::empty({0}, x.options()) : at::empty_like(x, x.options().dtype(at::kBFloat16));
    chronos::launch_hy_layer_norm(y.data_ptr(), out_f32, x.data_ptr<float>(), w.data_ptr<float>(),
                                  out_f32 ? nullptr : h.data_ptr(), out_f32, (int)x.size(0), (int)x.size(1), (float)eps,
                                  stream());
    return h;
}

Tensor hy_rowdot(const Tensor& h, const Tensor& w, const c10::optional<Tensor>& bias) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(h.device());
    same_act(h, w, "rowdot: h and w in one activation dtype");
    need(h.dim() == 2 && w.dim() == 2 && h.is_contiguous() && w.is_contiguous() && h.size(1) == w.size(1), "rowdot: shapes");
    if (bias) { flt(*bias, "rowdot: float32 bias"); need(bias->numel() == w.size(0), "rowdot: bias size"); }
    auto out = at::empty({h.size(0), w.size(0)}, h.options().dtype(at::kFloat));
    chronos::launch_hy_rowdot(h.data_ptr(), w.data_ptr(), bias ? bias->data_ptr<float>() : nullptr, out.data_ptr<float>(),
                              (int)h.size(0), (int)h.size(1), (int)w.size(0), f32(h), stream());
    return out;
}

void hy_act(Tensor& x, int64_t kind) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
    need(is_act(x) && x.is_contiguous() && (kind == 0 || kind == 1), "act: contiguous activation tensor, kind 0/1");
    chronos::launch_hy_act(x.data_ptr(), x.numel(), (int)kind, f32(x), stream());
}

Tensor hy_mlstm_scan(const Tensor& proj, const Tensor& gate_pre, const Tensor& q_start, const Tensor& pos0,
                     const Tensor& slots, Tensor& S, Tensor& n, Tensor& m, int64_t H, int64_t D, int64_t Dv, double cap) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(proj.device());
    need(is_act(proj) && proj.dim() == 2 && proj.is_contiguous(), "mlstm_scan: proj [T, C]");
    need(proj.size(1) >= 2 * H * D + H * Dv, "mlstm_scan: proj narrower than q | k | v");
    flt(gate_pre, "mlstm_scan: float32 gate pre-activations");
    const int64_t T = proj.size(0);
    need(gate_pre.dim() == 2 && gate_pre.size(0) == T && gate_pre.size(1) == 2 * H, "mlstm_scan: gate_pre [T, 2H]");
    i32(q_start, "mlstm_scan: q_start"); i32(pos0, "mlstm_scan: pos0"); i32(slots, "mlstm_scan: slots");
    const int64_t B = slots.numel();
    need(q_start.numel() == B + 1 && pos0.numel() == B, "mlstm_scan: q_start [B+1], pos0 [B], slots [B]");
    flt(S, "mlstm_scan: S"); flt(n, "mlstm_scan: n"); flt(m, "mlstm_scan: m");
    need(S.dim() == 4 && S.size(1) == H && S.size(2) == D && S.size(3) == Dv, "mlstm_scan: S [NS, H, D, Dv]");
    need(n.dim() == 3 && n.size(0) == S.size(0) && n.size(1) == H && n.size(2) == D, "mlstm_scan: n [NS, H, D]");
    need(m.dim() == 2 && m.size(0) == S.size(0) && m.size(1) == H, "mlstm_scan: m [NS, H]");
    need(D >= 1 && D <= 512 && H >= 1 && Dv >= 1, "mlstm_scan: 1 <= D <= 512");
    auto o = at::empty({T, H, Dv}, proj.options().dtype(at::kFloat));
    auto scratch = at::empty({3, T, H}, proj.options().dtype(at::kFloat));
    float* sp = scratch.data_ptr<float>();
    chronos::launch_hy_mlstm_scan(proj.data_ptr(), (int)proj.size(1), gate_pre.data_ptr<float>(),
                                  q_start.data_ptr<int32_t>(), pos0.data_ptr<int32_t>(), slots.data_ptr<int32_t>(),
                                  S.data_ptr<float>(), n.data_ptr<float>(), m.data_ptr<float>(), sp, sp + T * H,
                                  sp + 2 * T * H, o.data_ptr<float>(), (int)B, (int)H, (int)D, (int)Dv, (float)cap,
                                  f32(proj), stream());
    return o;
}

Tensor hy_mlstm_out(const Tensor& o, const Tensor& proj, int64_t g_off, const Tensor& w, double eps, bool out_f32) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(o.device());
    flt(o, "mlstm_out: float32 read-out");
    flt(w, "mlstm_out: float32 weight");
    need(o.dim() == 3 && is_act(proj) && proj.dim() == 2 && proj.is_contiguous() && proj.size(0) == o.size(0), "mlstm_out: shapes");
    const int64_t T = o.size(0), H = o.size(1), Dv = o.size(2);
    need(f32(proj) == out_f32 && g_off >= 0 && g_off + H * Dv <= proj.size(1) && w.numel() == H * Dv, "mlstm_out: gate columns / weight");
    auto y = at::empty({T, H * Dv}, proj.options());
    chronos::launch_hy_mlstm_out(o.data_ptr<float>(), proj.data_ptr(), (int)proj.size(1), (int)g_off, w.data_ptr<float>(),
                                 y.data_ptr(), (int)T, (int)H, (int)Dv, (float)eps, out_f32, stream());
    return y;
}

void hy_latent_prep(Tensor& q, const Tensor& dkv, const Tensor& pos, const Tensor& tok_seq, const Tensor& block_table,
                    const Tensor& w_norm, double eps, const Tensor& cos_sin, int64_t dims, int64_t rank, Tensor& cache) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(q.device());
    same_act(q, dkv, "latent_prep: q and dkv in one activation dtype");
    same_act(q, cache, "latent_prep: the cache holds the activation dtype");
    need(q.dim() == 3 && q.is_contiguous() && dkv.dim() == 2 && dkv.is_contiguous() && cache.dim() == 3 && cache.is_contiguous(), "latent_prep: layouts");
    const int64_t T = q.size(0), H = q.size(1), DK = dkv.size(1), R = DK - rank, D = q.size(2) - R;
    need(dkv.size(0) == T && rank >= 1 && R >= 0 && D >= 0 && cache.size(2) == DK, "latent_prep: sizes");
    need(dims % 2 == 0 && dims <= R, "latent_prep: rotated columns");
    i32(pos, "latent_prep: pos"); i32(tok_seq, "latent_prep: tok_seq"); i32(block_table, "latent_prep: block_table");
    need(pos.numel() == T && tok_seq.numel() == T && block_table.dim() == 2, "latent_prep: per-token metadata");
    flt(w_norm, "latent_prep: float32 norm weight"); flt(cos_sin, "latent_prep: float32 cos/sin table");
    need(w_norm.numel() == rank && cos_sin.dim() == 2 && cos_sin.size(1) == dims, "latent_prep: norm weight / table width");
    chronos::launch_hy_latent_prep(q.data_ptr(), dkv.data_ptr(), pos.data_ptr<int32_t>(), tok_seq.data_ptr<int32_t>(),
                                   block_table.data_ptr<int32_t>(), (int)block_table.size(1), w_norm.data_ptr<float>(),
                                   (float)eps, cos_sin.data_ptr<float>(), (int)dims, (int)rank, (int)R, (int)H, (int)D,
                                   cache.data_ptr(), (int)cache.size(1), (int)T, f32(q), stream());
}

Tensor hy_latent_attention(const Tensor& qa, const Tensor& cache, const Tensor& block_table, const Tensor& q_start,
                           const Tensor& pos, const c10::optional<Tensor>& gate, double scale, int64_t rank,
                           int64_t max_q) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(qa.device());
    same_act(qa, cache, "latent_attention: queries and cache in one activation dtype");
    need(qa.dim() == 3 && qa.is_contiguous() && cache.dim() == 3 && cache.is_contiguous(), "latent_attention: layouts");
    const int64_t T = qa.size(0), H = qa.size(1), DK = qa.size(2);
    need(cache.size(2) == DK && rank >= 1 && rank <= DK, "latent_attention: key width");
    need(f32(qa) || DK % 2 == 0, "latent_attention: bf16 rows need an even width");
    i32(block_table, "latent_attention: block_table"); i32(q_start, "latent_attention: q_start"); i32(pos, "latent_attention: pos");
    const int64_t B = q_start.numel() - 1;
    need(block_table.dim() == 2 && block_table.size(0) >= B && pos.numel() == T, "latent_attention: metadata");
    if (gate) { flt(*gate, "latent_attention: float32 gate"); need(gate->numel() == T * H, "latent_attention: gate [T, H]"); }
    auto out = at::empty({T, H, rank}, qa.options());
    if (T == 0 || B <= 0) return out;
    // few workgroups over long contexts (decode rows, a lone short portion): split the key range over more workgroups
    // and merge the partials; the split count follows from sizes the host knows (the block table bounds the context)
    const int mq = (int)std::max<int64_t>(1, max_q);
    int nsplit = 1;
    Tensor part_o, part_ml;
    if (chronos::hy_latent_use_mfma(f32(qa), (int)DK, (int)rank)) {
        nsplit = chronos::hy_latent_nsplit((int)(B * ((mq * H + 63) / 64)), (int)(block_table.size(1) * cache.size(1)));
        if (nsplit > 1) {
            part_o = at::empty({T * H * nsplit, rank}, qa.options().dtype(at::kFloat));
            part_ml = at::empty({T * H * nsplit, 2}, qa.options().dtype(at::kFloat));
        }
    }
    const bool ok = chronos::launch_hy_latent_attention(
        qa.data_ptr(), cache.data_ptr(), block_table.data_ptr<int32_t>(), (int)block_table.size(1),
        q_start.data_ptr<int32_t>(), pos.data_ptr<int32_t>(), gate ? gate->data_ptr<float>() : nullptr, out.data_ptr(),
        (int)B, (int)H, (int)DK, (int)rank, (int)cache.size(1), mq, (float)scale, f32(qa), nsplit,
        nsplit > 1 ? part_o.data_ptr<float>() : nullptr, nsplit > 1 ? part_ml.data_ptr<float>() : nullptr, T * H, stream());
    TORCH_CHECK(ok, "chronos hybrid op: latent_attention has no launch geometry for heads=", H, " row width=", DK,
                " rank=", rank, " (rank <= 512; 16 keys and 4 query rows must fit the LDS)");
    return out;
}

std::tuple<Tensor, Tensor> hy_moe_route(const Tensor& h, const Tensor& w, const Tensor& corr, int64_t top) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(h.device());
    same_act(h, w, "moe_route: h and router in one activation dtype");
    need(h.dim() == 2 && w.dim() == 2 && h.is_contiguous() && w.is_contiguous() && h.size(1) == w.size(1), "moe_route: shapes");
    flt(corr, "moe_route: float32 correction");
    const int64_t N = w.size(0);
    need(corr.numel() == N && N <= 256 && top >= 1 && top <= N, "moe_route: 1 <= top <= outputs <= 256");
    auto idx = at::empty({h.size(0), top}, h.options().dtype(at::kInt));
    auto wt = at::empty({h.size(0), top}, h.options().dtype(at::kFloat));
    auto z = at::empty({h.size(0), N}, h.options().dtype(at::kFloat));
    chronos::launch_hy_moe_route(h.data_ptr(), w.data_ptr(), corr.data_ptr<float>(), z.data_ptr<float>(), idx.data_ptr<int32_t>(),
                                 wt.data_ptr<float>(), (int)h.size(0), (int)h.size(1), (int)N, (int)top, f32(h), stream());
    return {idx, wt};
}

Tensor hy_moe_ffn(const Tensor& h, const Tensor& idx, const Tensor& wt, const Tensor& w_up, const Tensor& w_down,
                  int64_t act) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(h.device());
    same_act(h, w_up, "moe_ffn: h and experts in one activation dtype");
    same_act(h, w_down, "moe_ffn: h and experts in one activation dtype");
    need(h.dim() == 2 && h.is_contiguous() && w_up.dim() == 3 && w_down.dim() == 3 && w_up.is_contiguous() && w_down.is_contiguous(), "moe_ffn: layouts");
    const int64_t T = h.size(0), d = h.size(1), E = w_up.size(0), F = w_up.size(1);
    need(w_up.size(2) == d && w_down.size(0) == E && w_down.size(1) == d && w_down.size(2) == F, "moe_ffn: expert shapes");
    i32(idx, "moe_ffn: idx"); flt(wt, "moe_ffn: weights");
    need(idx.dim() == 2 && idx.size(0) == T && wt.sizes() == idx.sizes(), "moe_ffn: idx / weights [T, top]");
    need((2 * d + F) * 4 <= 160 * 1024, "moe_ffn: a token's rows must fit the LDS");
    need(act == 0 || act == 1, "moe_ffn: activation kind");
    auto out = at::empty_like(h);
    // bfloat16 with tile-sized widths: the grouped MFMA GEMMs (each expert's weights once per 128 of its tokens);
    // float32, or widths off the 128 grid: the token-parallel kernel
    if (!f32(h) && d % 128 == 0 && F % 128 == 0 && E <= 256 && T > 0) {
        const int top = (int)idx.size(1), items = (int)T * top;
        const int maxTiles = chronos::hy_moe_max_tiles(items, (int)E);
        auto meta = at::empty({1 + (int64_t)maxTiles + (int64_t)maxTiles * 128 + items}, h.options().dtype(at::kInt));
        auto z = at::empty({(int64_t)maxTiles * 128, F}, h.options());
        auto yrows = at::empty({(int64_t)maxTiles * 128, d}, h.options());
        chronos::launch_hy_moe_grouped((const uint16_t*)h.data_ptr(), idx.data_ptr<int32_t>(), wt.data_ptr<float>(),
                                       (const uint16_t*)w_up.data_ptr(), (const uint16_t*)w_down.data_ptr(),
                                       (uint16_t*)out.data_ptr(), meta.data_ptr<int32_t>(), (uint16_t*)z.data_ptr(),
                                       (uint16_t*)yrows.data_ptr(), (int)T, (int)d, (int)F, (int)E, top, (int)act, stream());
        return out;
    }
    chronos::launch_hy_moe_ffn_token(h.data_ptr(), idx.data_ptr<int32_t>(), wt.data_ptr<float>(), w_up.data_ptr(),
                                     w_down.data_ptr(), out.data_ptr(), (int)T, (int)d, (int)F, (int)E, (int)idx.size(1),
                                     (int)act, f32(h), stream());
    return out;
}

Tensor hy_rms_norm(const Tensor& x, const Tensor& w, double eps, bool out_f32) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
    flt(x, "rms_norm: float32 rows");
    flt(w, "rms_norm: float32 weight");
    need(x.dim() == 2 && w.numel() == x.size(1), "rms_norm: weight size");
    auto h = at::empty_like(x, x.options().dtype(out_f32 ? at::kFloat : at::kBFloat16));
    chronos::launch_hy_rms_norm(nullptr, const_cast<float*>(x.data_ptr<float>()), w.data_ptr<float>(), h.data_ptr(),
                                out_f32, (int)x.size(0), (int)x.size(1), 1.f, (float)eps, stream());
    return h;
}

Tensor hy_scale_add_rms_norm(const Tensor& y, Tensor& x, const Tensor& w, double alpha, double eps, bool out_f32) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
    flt(x, "scale_add_rms_norm: float32 residual");
    flt(w, "scale_add_rms_norm: float32 weight");
    need(is_act(y) && y.is_contiguous() && y.dim() == 2 && y.sizes() == x.sizes(), "scale_add_rms_norm: y shape");
    need(f32(y) == out_f32, "scale_add_rms_norm: y must be in the activation dtype");
    need(w.numel() == x.size(1), "scale_add_rms_norm: weight size");
    Tensor h = out_f32 ? at::empty({0}, x.options()) : at::empty_like(x, x.options().dtype(at::kBFloat16));
    chronos::launch_hy_rms_norm(y.data_ptr(), x.data_ptr<float>(), w.data_ptr<float>(), out_f32 ? nullptr : h.data_ptr(),
                                out_f32, (int)x.size(0), (int)x.size(1), (float)alpha, (float)eps, stream());
    return h;
}

Tensor hy_glu(const Tensor& gu, double limit, double slope, double shift) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(gu.device());
    need(is_act(gu) && gu.dim() == 2 && gu.is_contiguous() && gu.size(1) % 2 == 0, "glu: [T, 2F] activation tensor");
    auto y = at::empty({gu.size(0), gu.size(1) / 2}, gu.options());
    chronos::launch_hy_glu(gu.data_ptr(), y.data_ptr(), gu.size(0), (int)(gu.size(1) / 2), (float)limit, (float)slope,
                           (float)shift, f32(gu), stream());
    return y;
}

void hy_decay_pow(Tensor& z, double p) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(z.device());
    flt(z, "decay_pow: float32 contiguous logits");
    chronos::launch_hy_decay_pow(z.data_ptr<float>(), z.numel(), (float)p, stream());
}

Tensor hy_head_norm_gate(const Tensor& o, const Tensor& src, int64_t g_off, const Tensor& w, double eps, bool silu_gate,
                         bool out_f32) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(o.device());
    flt(o, "head_norm_gate: float32 read-out");
    flt(w, "head_norm_gate: float32 weight");
    need(o.dim() == 3 && is_act(src) && src.dim() == 2 && src.is_contiguous() && src.size(0) == o.size(0), "head_norm_gate: shapes");
    const int64_t T = o.size(0), H = o.size(1), Dv = o.size(2);
    need(f32(src) == out_f32 && g_off >= 0 && g_off + H * Dv <= src.size(1) && w.numel() == H * Dv, "head_norm_gate: gate columns / weight");
    auto y = at::empty({T, H * Dv}, src.options());
    chronos::launch_hy_head_norm_gate(o.data_ptr<float>(), src.data_ptr(), (int)src.size(1), (int)g_off, w.data_ptr<float>(),
                                      y.data_ptr(), (int)T, (int)H, (int)Dv, (float)eps, silu_gate, out_f32, stream());
    return y;
}

Tensor hy_window_prep(Tensor& qkv, int64_t H, int64_t G, int64_t D, int64_t Dv, const c10::optional<Tensor>& v_first,
                      const c10::optional<Tensor>& lam, const Tensor& pos, const Tensor& tok_seq, const Tensor& block_table,
                      const c10::optional<Tensor>& q_norm, const c10::optional<Tensor>& k_norm, double eps,
                      const c10::optional<Tensor>& cos_sin, int64_t dims, Tensor& kc, Tensor& vc, bool emit_v,
                      int64_t v_off, const c10::optional<Tensor>& v_cos_sin) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(qkv.device());
    same_act(qkv, kc, "window_prep: the caches hold the activation dtype");
    same_act(qkv, vc, "window_prep: the caches hold the activation dtype");
    need(qkv.dim() == 2 && qkv.is_contiguous() && kc.dim() == 4 && vc.dim() == 4 && kc.is_contiguous() && vc.is_contiguous(), "window_prep: layouts");
    const int64_t T = qkv.size(0);
    if (v_off < 0) v_off = (H + G) * D;   // the values follow the keys
    need(H >= 1 && G >= 1 && H % G == 0 && D >= 1 && Dv >= 1 && qkv.size(1) >= (H + G) * D && v_off + G * Dv <= qkv.size(1), "window_prep: qkv width");
    if (v_cos_sin) {
        flt(*v_cos_sin, "window_prep: float32 cos/sin table of the values");
        need(Dv % 2 == 0 && v_cos_sin->dim() == 2 && v_cos_sin->size(1) == Dv, "window_prep: the values' table is [P, Dv], Dv even");
    }
    need(kc.size(2) == G && kc.size(3) == D && vc.size(2) == G && vc.size(3) == Dv && vc.size(0) == kc.size(0) && vc.size(1) == kc.size(1), "window_prep: cache shapes");
    i32(pos, "window_prep: pos"); i32(tok_seq, "window_prep: tok_seq"); i32(block_table, "window_prep: block_table");
    need(pos.numel() == T && tok_seq.numel() == T && block_table.dim() == 2, "window_prep: per-token metadata");
    need(q_norm.has_value() == k_norm.has_value(), "window_prep: queries and keys are normed together or not at all");
    if (q_norm) {
        flt(*q_norm, "window_prep: float32 norm weight"); flt(*k_norm, "window_prep: float32 norm weight");
        need(q_norm->numel() == D && k_norm->numel() == D, "window_prep: norm weights [D]");
    }
    need(dims >= 0 && dims % 2 == 0 && dims <= D, "window_prep: rotated columns");
    if (dims > 0) {
        need(cos_sin.has_value(), "window_prep: rotation needs the cos/sin table");
        flt(*cos_sin, "window_prep: float32 cos/sin table");
        need(cos_sin->dim() == 2 && cos_sin->size(1) == dims, "window_prep: table width");
    }
    if (v_first) {
        same_act(qkv, *v_first, "window_prep: v_first in the activation dtype");
        need(v_first->is_contiguous() && v_first->numel() == T * G * Dv, "window_prep: v_first [T, G Dv]");
        need(lam.has_value(), "window_prep: mixing needs its weight");
        flt(*lam, "window_prep: float32 mixing weight");
        need(lam->numel() == 1, "window_prep: one mixing weight");
    }
    Tensor v_out = emit_v ? at::empty({T, G * Dv}, qkv.options()) : at::empty({0}, qkv.options());
    chronos::launch_hy_window_prep(qkv.data_ptr(), (int)qkv.size(1), (int)H, (int)G, (int)D, (int)Dv,
                                   v_first ? v_first->data_ptr() : nullptr, v_first ? lam->data_ptr<float>() : nullptr,
                                   pos.data_ptr<int32_t>(), tok_seq.data_ptr<int32_t>(), block_table.data_ptr<int32_t>(),
                                   (int)block_table.size(1), q_norm ? q_norm->data_ptr<float>() : nullptr,
                                   k_norm ? k_norm->data_ptr<float>() : nullptr, (float)eps,
                                   dims > 0 ? cos_sin->data_ptr<float>() : nullptr, (int)dims, kc.data_ptr(), vc.data_ptr(),
                                   (int)kc.size(1), emit_v ? v_out.data_ptr() : nullptr, (int)v_off,
                                   v_cos_sin ? v_cos_sin->data_ptr<float>() : nullptr, (int)T, f32(qkv), stream());
    return v_out;
}

Tensor hy_window_attention(const Tensor& qkv, const Tensor& kc, const Tensor& vc, const Tensor& block_table,
                           const Tensor& q_start, const Tensor& pos, const c10::optional<Tensor>& sink,
                           const c10::optional<Tensor>& gate, double scale, int64_t window, int64_t keep, int64_t chunk,
                           int64_t H, int64_t max_q, int64_t pool, const c10::optional<Tensor>& kp,
                           const c10::optional<Tensor>& vp, const c10::optional<Tensor>& v_cos_sin, int64_t g_off) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(qkv.device());
    same_act(qkv, kc, "window_attention: queries and caches in one activation dtype");
    same_act(qkv, vc, "window_attention: queries and caches in one activation dtype");
    need(qkv.dim() == 2 && qkv.is_contiguous() && kc.dim() == 4 && vc.dim() == 4 && kc.is_contiguous() && vc.is_contiguous(), "window_attention: layouts");
    const int64_t T = qkv.size(0), G = kc.size(2), D = kc.size(3), Dv = vc.size(3);
    need(H >= 1 && H % G == 0 && qkv.size(1) >= H * D && vc.size(2) == G && vc.size(0) == kc.size(0) && vc.size(1) == kc.size(1), "window_attention: shapes");
    need(H / G <= 64 && Dv <= 256, "window_attention: at most 64 query heads per key/value head and 256 value columns");
    need(chronos::hy_window_rows_cap((int)(H / G), (int)D, (int)Dv, f32(qkv)) > 0, "window_attention: a key tile and a group's query rows must fit the LDS");
    i32(block_table, "window_attention: block_table"); i32(q_start, "window_attention: q_start"); i32(pos, "window_attention: pos");
    const int64_t B = q_start.numel() - 1;
    need(block_table.dim() == 2 && block_table.size(0) >= B && pos.numel() == T && window >= 0 && keep >= 0 && chunk >= 0, "window_attention: metadata");
    if (sink) { flt(*sink, "window_attention: float32 sinks"); need(sink->numel() == H, "window_attention: sink [H]"); }
    if (gate) { flt(*gate, "window_attention: float32 gate"); need(gate->numel() == T * H, "window_attention: gate [T, H]"); }
    int64_t EP = 1;
    if (pool > 0) {   // pooled pairs: block e of a sequence in row e % EP of its page e / EP
        need(kp.has_value() && vp.has_value() && window > 0, "window_attention: pooled blocks need their caches and a window");
        same_act(qkv, *kp, "window_attention: pooled caches in the activation dtype");
        same_act(qkv, *vp, "window_attention: pooled caches in the activation dtype");
        EP = (kc.size(1) + pool - 1) / pool;
        need(kp->is_contiguous() && vp->is_contiguous() && kp->dim() == 4 && vp->dim() == 4 && kp->size(0) == kc.size(0) &&
                 vp->size(0) == kc.size(0) && kp->size(1) == EP && vp->size(1) == EP && kp->size(2) == G && vp->size(2) == G &&
                 kp->size(3) == D && vp->size(3) == Dv, "window_attention: pooled caches [NB, ceil(BS / pool), G, .]");
    }
    if (v_cos_sin) {   // the outputs are turned back by the query's position
        flt(*v_cos_sin, "window_attention: float32 cos/sin table of the values");
        need(Dv % 2 == 0 && v_cos_sin->dim() == 2 && v_cos_sin->size(1) == Dv, "window_attention: the values' table is [P, Dv], Dv even");
    }
    need(g_off < 0 || g_off + H * Dv <= qkv.size(1), "window_attention: the gate columns lie in the projection's row");
    auto out = at::empty({T, H * Dv}, qkv.options());
    if (T == 0 || B <= 0) return out;
    const int mq = (int)std::max<int64_t>(1, max_q);
    const int nsplit = chronos::hy_window_nsplit(f32(qkv), (int)qkv.size(1), (int)B, mq, (int)H, (int)G, (int)D, (int)Dv,
                                                 (int)window, (int)keep, (int)chunk, (int)(block_table.size(1) * kc.size(1)),
                                                 (int)pool);
    Tensor part_o, part_ml;
    if (nsplit > 1) {
        part_o = at::empty({T * H * nsplit, Dv}, qkv.options().dtype(at::kFloat));
        part_ml = at::empty({T * H * nsplit, 2}, qkv.options().dtype(at::kFloat));
    }
    chronos::launch_hy_window_attention(qkv.data_ptr(), (int)qkv.size(1), kc.data_ptr(), vc.data_ptr(),
                                        block_table.data_ptr<int32_t>(), (int)block_table.size(1),
                                        q_start.data_ptr<int32_t>(), pos.data_ptr<int32_t>(),
                                        sink ? sink->data_ptr<float>() : nullptr, gate ? gate->data_ptr<float>() : nullptr,
                                        out.data_ptr(), (int)B, mq, (int)H, (int)G, (int)D, (int)Dv, (int)kc.size(1),
                                        (float)scale, (int)window, (int)keep, (int)chunk, f32(qkv), nsplit,
                                        nsplit > 1 ? part_o.data_ptr<float>() : nullptr,
                                        nsplit > 1 ? part_ml.data_ptr<float>() : nullptr, T * H, (int)pool, (int)EP,
                                        pool > 0 ? kp->data_ptr() : nullptr, pool > 0 ? vp->data_ptr() : nullptr,
                                        v_cos_sin ? v_cos_sin->data_ptr<float>() : nullptr, g_off >= 0 ? (int)g_off : -1,
                                        stream());
    return out;
}

Tensor hy_short_conv(const Tensor& x, const Tensor& w, const Tensor& tok_seq, const Tensor& q_start, const Tensor& pos0,
                     const Tensor& slots, Tensor& hist, bool silu, const c10::optional<Tensor>& bias, int64_t x_off) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
    same_act(x, hist, "short_conv: the history holds the activation dtype");
    flt(w, "short_conv: float32 taps");
    need(x.dim() == 2 && x.is_contiguous() && w.dim() == 2 && hist.dim() == 3 && hist.is_contiguous(), "short_conv: layouts");
    const int64_t T = x.size(0), C = w.size(0), K = w.size(1), B = slots.numel();
    need(x_off >= 0 && x_off + C <= x.size(1) && K >= 1 && hist.size(1) == K - 1 && hist.size(2) == C, "short_conv: channels / taps / history");
    if (bias) { flt(*bias, "short_conv: float32 bias"); need(bias->numel() == C, "short_conv: bias [C]"); }
    i32(tok_seq, "short_conv: tok_seq"); i32(q_start, "short_conv: q_start"); i32(pos0, "short_conv: pos0"); i32(slots, "short_conv: slots");
    need(tok_seq.numel() == T && q_start.numel() == B + 1 && pos0.numel() == B, "short_conv: metadata");
    auto y = at::empty({T, C}, x.options());
    const char* xp = (const char*)x.data_ptr() + x_off * x.element_size();
    chronos::launch_hy_short_conv(xp, (int)x.size(1), w.data_ptr<float>(), bias ? bias->data_ptr<float>() : nullptr,
                                  tok_seq.data_ptr<int32_t>(),
                                  q_start.data_ptr<int32_t>(), pos0.data_ptr<int32_t>(), slots.data_ptr<int32_t>(),
                                  hist.data_ptr(), y.data_ptr(), (int)T, (int)B, (int)C, (int)K, silu, f32(x), stream());
    return y;
}

std::tuple<Tensor, Tensor, Tensor, Tensor> hy_delta_prep(const Tensor& y, const Tensor& ab, const Tensor& a_log, int64_t HK,
                                                         int64_t H, int64_t D, double q_mul) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(y.device());
    need(is_act(y) && y.dim() == 2 && y.is_contiguous() && y.size(1) >= 2 * HK * D, "delta_prep: y [T, >= 2 HK D]");
    flt(ab, "delta_prep: float32 pre-activations"); flt(a_log, "delta_prep: float32 A_log");
    const int64_t T = y.size(0);
    need(ab.numel() == T * 2 * H && a_log.numel() == H, "delta_prep: ab [T, 2H], a_log [H]");
    auto fo = y.options().dtype(at::kFloat);
    auto qs = at::empty({T, HK}, fo), ks = at::empty({T, HK}, fo), dc = at::empty({T, H}, fo), bt = at::empty({T, H}, fo);
    chronos::launch_hy_delta_prep(y.data_ptr(), (int)y.size(1), ab.data_ptr<float>(), a_log.data_ptr<float>(),
                                  qs.data_ptr<float>(), ks.data_ptr<float>(), dc.data_ptr<float>(), bt.data_ptr<float>(),
                                  (int)T, (int)HK, (int)H, (int)D, (float)q_mul, f32(y), stream());
    return {qs, ks, dc, bt};
}

Tensor hy_linear_scan(const Tensor& proj, int64_t q_off, int64_t k_off, int64_t v_off, const c10::optional<Tensor>& qscale,
                      const c10::optional<Tensor>& kscale, double q_mul, const Tensor& decay,
                      const c10::optional<Tensor>& beta, const Tensor& q_start, const Tensor& pos0, const Tensor& slots,
                      Tensor& S, int64_t HK, int64_t H, int64_t D, int64_t Dv, const c10::optional<Tensor>& vscale) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(proj.device());
    need(is_act(proj) && proj.dim() == 2 && proj.is_contiguous(), "linear_scan: proj [T, C]");
    const int64_t T = proj.size(0), C = proj.size(1), B = slots.numel();
    need(HK >= 1 && H % HK == 0 && D >= 1 && Dv >= 1, "linear_scan: head counts");
    need(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + HK * D <= C && k_off + HK * D <= C && v_off + H * Dv <= C, "linear_scan: column ranges");
    flt(decay, "linear_scan: float32 decay");
    const bool fixed = decay.dim() == 1 && decay.numel() == H;   // one number per head, the same for every token
    const bool chd = !fixed && decay.numel() == T * H * D && D > 1;
    need(fixed || chd || decay.numel() == T * H, "linear_scan: decay [T, H], [T, H, D] or [H]");
    if (qscale) { flt(*qscale, "linear_scan: qscale"); need(qscale->numel() == T * HK, "linear_scan: qscale [T, HK]"); }
    if (kscale) { flt(*kscale, "linear_scan: kscale"); need(kscale->numel() == T * HK, "linear_scan: kscale [T, HK]"); }
    if (beta) { flt(*beta, "linear_scan: beta"); need(beta->numel() == T * H, "linear_scan: beta [T, H]"); }
    if (vscale) { flt(*vscale, "linear_scan: vscale"); need(vscale->numel() == T * H && !beta, "linear_scan: vscale [T, H], without the delta correction"); }
    i32(q_start, "linear_scan: q_start"); i32(pos0, "linear_scan: pos0"); i32(slots, "linear_scan: slots");
    need(q_start.numel() == B + 1 && pos0.numel() == B, "linear_scan: q_start [B+1], pos0 [B], slots [B]");
    flt(S, "linear_scan: S");
    need(S.dim() == 4 && S.size(1) == H && S.size(2) == D && S.size(3) == Dv, "linear_scan: S [NS, H, D, Dv]");
    auto o = at::empty({T, H, Dv}, proj.options().dtype(at::kFloat));
    if (T == 0) return o;
    const bool ok = chronos::launch_hy_linear_scan(
        proj.data_ptr(), (int)C, (int)q_off, (int)k_off, (int)v_off, qscale ? qscale->data_ptr<float>() : nullptr,
        kscale ? kscale->data_ptr<float>() : nullptr, (float)q_mul, decay.data_ptr<float>(), chd, fixed,
        beta ? beta->data_ptr<float>() : nullptr, q_start.data_ptr<int32_t>(), pos0.data_ptr<int32_t>(),
        slots.data_ptr<int32_t>(), S.data_ptr<float>(), o.data_ptr<float>(), (int)T, (int)B, (int)HK, (int)H, (int)D, (int)Dv,
        vscale ? vscale->data_ptr<float>() : nullptr, f32(proj), stream());
    TORCH_CHECK(ok, "chronos hybrid op: linear_scan keeps a state column in registers, D <= 256 (got ", D, ")");
    return o;
}

std::tuple<Tensor, Tensor> hy_moe_route_topk(const Tensor& h, const Tensor& w, const Tensor& bias, int64_t top) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(h.device());
    same_act(h, w, "moe_route_topk: h and router in one activation dtype");
    need(h.dim() == 2 && w.dim() == 2 && h.is_contiguous() && w.is_contiguous() && h.size(1) == w.size(1), "moe_route_topk: shapes");
    flt(bias, "moe_route_topk: float32 bias");
    const int64_t N = w.size(0);
    need(bias.numel() == N && N <= 256 && top >= 1 && top <= N && top <= 64, "moe_route_topk: 1 <= top <= min(outputs, 64), outputs <= 256");
    auto idx = at::empty({h.size(0), top}, h.options().dtype(at::kInt));
    auto wt = at::empty({h.size(0), top}, h.options().dtype(at::kFloat));
    auto z = at::empty({h.size(0), N}, h.options().dtype(at::kFloat));
    chronos::launch_hy_moe_route_topk(h.data_ptr(), w.data_ptr(), bias.data_ptr<float>(), z.data_ptr<float>(),
                                      idx.data_ptr<int32_t>(), wt.data_ptr<float>(), (int)h.size(0), (int)h.size(1), (int)N,
                                      (int)top, f32(h), stream());
    return {idx, wt};
}

Tensor hy_moe_glu_ffn(const Tensor& h, const Tensor& idx, const Tensor& wt, const Tensor& w_gu, const Tensor& w_down,
                      double limit, double slope, double shift, bool tiled) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(h.device());
    same_act(h, w_gu, "moe_glu_ffn: h and experts in one activation dtype");
    same_act(h, w_down, "moe_glu_ffn: h and experts in one activation dtype");
    need(h.dim() == 2 && h.is_contiguous() && w_gu.dim() == 3 && w_down.dim() == 3 && w_gu.is_contiguous() && w_down.is_contiguous(), "moe_glu_ffn: layouts");
    const int64_t T = h.size(0), d = h.size(1), E = w_gu.size(0), F = w_down.size(2);
    need(w_gu.size(1) == 2 * F && w_gu.size(2) == d && w_down.size(0) == E && w_down.size(1) == d, "moe_glu_ffn: expert shapes");
    i32(idx, "moe_glu_ffn: idx"); flt(wt, "moe_glu_ffn: weights");
    need(idx.dim() == 2 && idx.size(0) == T && wt.sizes() == idx.sizes(), "moe_glu_ffn: idx / weights [T, top]");
    auto out = at::empty_like(h);
    // bfloat16 with tile-sized widths and more than a few tokens: the grouped MFMA GEMMs over the tile-ordered copy
    // of the gate / up rows; otherwise the token-parallel kernel (which reads either row order)
    need(!tiled || (!f32(h) && d % 128 == 0 && F % 128 == 0), "moe_glu_ffn: the tile order is for bfloat16 experts with d and F on the 128 grid");
    if (tiled && E <= 256 && T * idx.size(1) >= 4 * E) {
        const int top = (int)idx.size(1), items = (int)T * top;
        const int maxTiles = chronos::hy_moe_max_tiles(items, (int)E);
        auto meta = at::empty({1 + (int64_t)maxTiles + (int64_t)maxTiles * 128 + items}, h.options().dtype(at::kInt));
        auto z = at::empty({(int64_t)maxTiles * 128, F}, h.options());
        auto yrows = at::empty({(int64_t)maxTiles * 128, d}, h.options());
        chronos::launch_hy_moe_glu_grouped((const uint16_t*)h.data_ptr(), idx.data_ptr<int32_t>(), wt.data_ptr<float>(),
                                           (const uint16_t*)w_gu.data_ptr(), (const uint16_t*)w_down.data_ptr(),
                                           (uint16_t*)out.data_ptr(), meta.data_ptr<int32_t>(), (uint16_t*)z.data_ptr(),
                                           (uint16_t*)yrows.data_ptr(), (int)T, (int)d, (int)F, (int)E, top, (float)limit,
                                           (float)slope, (float)shift, stream());
        return out;
    }
    need((2 * d + 2 * F) * 4 <= 160 * 1024, "moe_glu_ffn: a token's rows must fit the LDS");
    chronos::launch_hy_moe_glu_token(h.data_ptr(), idx.data_ptr<int32_t>(), wt.data_ptr<float>(), w_gu.data_ptr(),
                                     w_down.data_ptr(), out.data_ptr(), (int)T, (int)d, (int)F, (int)E, (int)idx.size(1),
                                     (float)limit, (float)slope, (float)shift, tiled, f32(h), stream());
    return out;
}

Tensor hy_add_rms_norm(const Tensor& y, Tensor& x, const c10::optional<Tensor>& w_out, double eps, bool out_f32,
                       const c10::optional<Tensor>& y2, const c10::optional<Tensor>& gate2,
                       const c10::optional<Tensor>& w_y, bool emit) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
    flt(x, "add_rms_norm: float32 residual");
    need(x.dim() == 2 && is_act(y) && y.is_contiguous() && y.sizes() == x.sizes() && f32(y) == out_f32, "add_rms_norm: y [T, d] in the activation dtype");
    const int64_t T = x.size(0), d = x.size(1);
    if (w_out) { flt(*w_out, "add_rms_norm: float32 weight"); need(w_out->numel() == d, "add_rms_norm: weight size"); }
    if (w_y) { flt(*w_y, "add_rms_norm: float32 weight"); need(w_y->numel() == d, "add_rms_norm: weight size"); }
    need(y2.has_value() == gate2.has_value(), "add_rms_norm: a second addend comes with its gate");
    if (y2) {
        same_act(y, *y2, "add_rms_norm: y2 in the activation dtype");
        need(y2->is_contiguous() && y2->sizes() == x.sizes(), "add_rms_norm: y2 shape");
        flt(*gate2, "add_rms_norm: float32 gate");
        need(gate2->numel() == T, "add_rms_norm: one gate per row");
    }
    const int mode = !emit ? 0 : (w_out ? 2 : 1);
    // float activations read the updated stream itself
    const bool has_h = mode == 2 || (mode == 1 && !out_f32);
    Tensor h = has_h ? at::empty({T, d}, x.options().dtype(out_f32 ? at::kFloat : at::kBFloat16)) : at::empty({0}, x.options());
    chronos::launch_hy_add_rms_norm(y.data_ptr(), y2 ? y2->data_ptr() : nullptr, gate2 ? gate2->data_ptr<float>() : nullptr,
                                    w_y ? w_y->data_ptr<float>() : nullptr, x.data_ptr<float>(),
                                    w_out ? w_out->data_ptr<float>() : nullptr, has_h ? h.data_ptr() : nullptr, (int)T, (int)d,
                                    (float)eps, has_h ? mode : 0, out_f32, stream());
    return h;
}

Tensor hy_token_gate(const Tensor& a, const Tensor& ids, const Tensor& table, int64_t col0) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(a.device());
    same_act(a, table, "token_gate: projection and table in one activation dtype");
    need(a.dim() == 2 && a.is_contiguous() && table.dim() == 2 && table.is_contiguous(), "token_gate: layouts");
    i32(ids, "token_gate: ids");
    need(ids.numel() == a.size(0) && col0 >= 0 && col0 + a.size(1) <= table.size(1), "token_gate: ids [T], columns inside the table");
    auto out = at::empty_like(a);
    chronos::launch_hy_token_gate(a.data_ptr(), ids.data_ptr<int32_t>(), table.data_ptr(), (int)table.size(1), (int)col0,
                                  out.data_ptr(), (int)a.size(0), (int)a.size(1), f32(a), stream());
    return out;
}

std::tuple<Tensor, Tensor> hy_ssm_prep(const Tensor& dt_pre, const Tensor& a_log) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(dt_pre.device());
    flt(dt_pre, "ssm_prep: float32 pre-activations"); flt(a_log, "ssm_prep: float32 A_log");
    need(dt_pre.dim() == 2 && dt_pre.size(1) == a_log.numel(), "ssm_prep: dt_pre [T, H], a_log [H]");
    auto decay = at::empty_like(dt_pre), dt = at::empty_like(dt_pre);
    chronos::launch_hy_ssm_prep(dt_pre.data_ptr<float>(), a_log.data_ptr<float>(), decay.data_ptr<float>(),
                                dt.data_ptr<float>(), (int)dt_pre.size(0), (int)dt_pre.size(1), stream());
    return {decay, dt};
}

Tensor hy_gated_group_norm(const Tensor& o, const Tensor& skip_src, int64_t skip_off, const Tensor& skip_w,
                           const Tensor& gate_src, int64_t g_off, const Tensor& w, int64_t groups, double eps, bool out_f32) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(o.device());
    flt(o, "gated_group_norm: float32 read-out"); flt(w, "gated_group_norm: float32 weight"); flt(skip_w, "gated_group_norm: float32 skip weights");
    need(o.dim() == 3, "gated_group_norm: o [T, H, Dv]");
    const int64_t T = o.size(0), H = o.size(1), Dv = o.size(2), n = H * Dv;
    same_act(skip_src, gate_src, "gated_group_norm: sources in one activation dtype");
    need(f32(gate_src) == out_f32 && skip_src.dim() == 2 && gate_src.dim() == 2 && skip_src.is_contiguous() && gate_src.is_contiguous() &&
         skip_src.size(0) == T && gate_src.size(0) == T, "gated_group_norm: sources [T, C]");
    need(skip_off >= 0 && skip_off + n <= skip_src.size(1) && g_off >= 0 && g_off + n <= gate_src.size(1), "gated_group_norm: column ranges");
    need(w.numel() == n && skip_w.numel() == H && groups >= 1 && n % groups == 0, "gated_group_norm: weight [H Dv], skip [H], equal groups");
    auto y = at::empty({T, n}, gate_src.options());
    chronos::launch_hy_gated_group_norm(o.data_ptr<float>(), skip_src.data_ptr(), (int)skip_src.size(1), (int)skip_off,
                                        skip_w.data_ptr<float>(), gate_src.data_ptr(), (int)gate_src.size(1), (int)g_off,
                                        w.data_ptr<float>(), y.data_ptr(), (int)T, (int)n, (int)groups, (int)Dv, (float)eps,
                                        out_f32, stream());
    return y;
}

Tensor hy_rglru_scan(const Tensor& u, const Tensor& gates, const Tensor& sp, double c, const Tensor& ysrc, int64_t y_off,
                     const Tensor& q_start, const Tensor& pos0, const Tensor& slots, Tensor& S, int64_t max_q) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(u.device());
    same_act(u, ysrc, "rglru_scan: branches in one activation dtype");
    need(u.dim() == 2 && u.is_contiguous() && ysrc.dim() == 2 && ysrc.is_contiguous() && ysrc.size(0) == u.size(0), "rglru_scan: layouts");
    const int64_t T = u.size(0), W = u.size(1), B = slots.numel();
    flt(gates, "rglru_scan: float32 gate pre-activations"); flt(sp, "rglru_scan: float32 decay parameter"); flt(S, "rglru_scan: S");
    need(gates.dim() == 3 && gates.size(1) == T && gates.size(0) >= 1 && W % gates.size(0) == 0 &&
         gates.size(2) == 2 * (W / gates.size(0)), "rglru_scan: gates [blocks, T, 2 W / blocks]");
    need(sp.numel() == W && y_off >= 0 && y_off + W <= ysrc.size(1) && S.dim() == 2 && S.size(1) == W, "rglru_scan: widths");
    i32(q_start, "rglru_scan: q_start"); i32(pos0, "rglru_scan: pos0"); i32(slots, "rglru_scan: slots");
    need(q_start.numel() == B + 1 && pos0.numel() == B, "rglru_scan: q_start [B+1], pos0 [B], slots [B]");
    auto out = at::empty_like(u);
    if (T == 0 || B == 0) return out;
    const int nch = chronos::hy_rglru_chunks((int)std::max<int64_t>(1, max_q > 0 ? max_q : T));
    Tensor pq, init;
    if (nch > 1) {
        pq = at::empty({B, nch, 2, W}, S.options());
        init = at::empty({B, W}, S.options());
    }
    chronos::launch_hy_rglru_scan(u.data_ptr(), gates.data_ptr<float>(), sp.data_ptr<float>(), (float)c, ysrc.data_ptr(),
                                  (int)ysrc.size(1), (int)y_off, q_start.data_ptr<int32_t>(), pos0.data_ptr<int32_t>(),
                                  slots.data_ptr<int32_t>(), S.data_ptr<float>(), nch > 1 ? pq.data_ptr<float>() : nullptr,
                                  nch > 1 ? init.data_ptr<float>() : nullptr, out.data_ptr(), (int)T, (int)B, (int)W,
                                  (int)(W / gates.size(0)), nch, f32(u), stream());
    return out;
}

std::tuple<Tensor, Tensor> hy_moe_route_group(const Tensor& h, const Tensor& w, int64_t top, int64_t n_groups, int64_t keep,
                                              double scale) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(h.device());
    same_act(h, w, "moe_route_group: h and router in one activation dtype");
    need(h.dim() == 2 && w.dim() == 2 && h.is_contiguous() && w.is_contiguous() && h.size(1) == w.size(1), "moe_route_group: shapes");
    const int64_t N = w.size(0);
    need(N <= 256 && n_groups >= 1 && n_groups <= 64 && N % n_groups == 0 && keep >= 1 && keep <= n_groups,
         "moe_route_group: outputs <= 256 in 1..64 equal groups, of which 1..all are kept");
    need(top >= 1 && top <= 64 && top <= keep * (N / n_groups), "moe_route_group: 1 <= top <= min(64, experts of the kept groups)");
    auto idx = at::empty({h.size(0), top}, h.options().dtype(at::kInt));
    auto wt = at::empty({h.size(0), top}, h.options().dtype(at::kFloat));
    auto z = at::empty({h.size(0), N}, h.options().dtype(at::kFloat));
    chronos::launch_hy_moe_route_group(h.data_ptr(), w.data_ptr(), z.data_ptr<float>(), idx.data_ptr<int32_t>(),
                                       wt.data_ptr<float>(), (int)h.size(0), (int)h.size(1), (int)N, (int)top, (int)n_groups,
                                       (int)keep, (float)scale, f32(h), stream());
    return {idx, wt};
}

void hy_pool_blocks(const Tensor& kc, const Tensor& vc, Tensor& kp, Tensor& vp, const Tensor& block_table,
                    const Tensor& q_start, const Tensor& pos0, int64_t pool, int64_t max_q) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(kc.device());
    same_act(kc, vc, "pool_blocks: caches in one activation dtype");
    same_act(kc, kp, "pool_blocks: caches in one activation dtype");
    same_act(kc, vp, "pool_blocks: caches in one activation dtype");
    need(kc.dim() == 4 && vc.dim() == 4 && kp.dim() == 4 && vp.dim() == 4 && kc.is_contiguous() && vc.is_contiguous() &&
             kp.is_contiguous() && vp.is_contiguous(), "pool_blocks: layouts");
    const int64_t BS = kc.size(1), G = kc.size(2), D = kc.size(3), Dv = vc.size(3);
    need(pool >= 1, "pool_blocks: pool >= 1");
    const int64_t EP = (BS + pool - 1) / pool;
    need(vc.size(0) == kc.size(0) && vc.size(1) == BS && vc.size(2) == G && kp.size(0) == kc.size(0) && vp.size(0) == kc.size(0) &&
             kp.size(1) == EP && vp.size(1) == EP && kp.size(2) == G && vp.size(2) == G && kp.size(3) == D && vp.size(3) == Dv,
         "pool_blocks: pooled caches [NB, ceil(BS / pool), G, .]");
    i32(block_table, "pool_blocks: block_table"); i32(q_start, "pool_blocks: q_start"); i32(pos0, "pool_blocks: pos0");
    const int64_t B = pos0.numel();
    need(block_table.dim() == 2 && block_table.size(0) >= B && q_start.numel() == B + 1, "pool_blocks: metadata");
    chronos::launch_hy_pool_blocks(kc.data_ptr(), vc.data_ptr(), kp.data_ptr(), vp.data_ptr(), block_table.data_ptr<int32_t>(),
                                   (int)block_table.size(1), q_start.data_ptr<int32_t>(), pos0.data_ptr<int32_t>(), (int)pool,
                                   (int)BS, (int)EP, (int)(G * D), (int)(G * Dv), (int)B, (int)std::max<int64_t>(1, max_q),
                                   f32(kc), stream());
}

// add: x <- x + norm(v) w_y with v from y (and y2); else the plain grouped norm of x.  emit: returns norm(x) w_out.
Tensor hy_sandwich_join(const c10::optional<Tensor>& y, const c10::optional<Tensor>& y2, Tensor& x,
                        const c10::optional<Tensor>& w_y, const c10::optional<Tensor>& w_out,
                        const c10::optional<Tensor>& w_a, const c10::optional<Tensor>& w_b, int64_t groups, double eps,
                        bool out_f32, bool add, bool emit) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
    flt(x, "sandwich_join: the stream is contiguous float32");
    need(x.dim() == 2, "sandwich_join: x [T, d]");
    const int64_t T = x.size(0), d = x.size(1);
    need(chronos::hy_sandwich_groups_ok((int)d, (int)groups), "sandwich_join: groups >= 1 and d % groups == 0");
    need(add == y.has_value() && (add || emit), "sandwich_join: an addend when adding, something to do otherwise");
    if (add) {
        need(is_act(*y) && y->is_contiguous() && y->dim() == 2 && y->size(0) == T && y->size(1) == d, "sandwich_join: y [T, d]");
        need(w_y.has_value(), "sandwich_join: the addend's norm weight");
        flt(*w_y, "sandwich_join: float32 norm weight");
        need(w_y->numel() == d, "sandwich_join: w_y [d]");
        if (y2) {
            same_act(*y, *y2, "sandwich_join: both addends in one dtype");
            need(y2->is_contiguous() && y2->numel() == T * d, "sandwich_join: y2 [T, d]");
        }
        need(w_a.has_value() == w_b.has_value() && (!w_a || y2), "sandwich_join: the pair form takes two addends and two weights");
        if (w_a) {
            flt(*w_a, "sandwich_join: float32 pair weight"); flt(*w_b, "sandwich_join: float32 pair weight");
            need(w_a->numel() == d && w_b->numel() == d, "sandwich_join: pair weights [d]");
        }
    }
    Tensor h;
    if (emit) {
        need(w_out.has_value(), "sandwich_join: the emitted norm's weight");
        flt(*w_out, "sandwich_join: float32 norm weight");
        need(w_out->numel() == d, "sandwich_join: w_out [d]");
        h = at::empty({T, d}, x.options().dtype(out_f32 ? at::kFloat : at::kBFloat16));
    } else {
        h = at::empty({0}, x.options());
    }
    chronos::launch_hy_sandwich_join(add ? y->data_ptr() : nullptr, (add && y2) ? y2->data_ptr() : nullptr, x.data_ptr<float>(),
                                     add ? w_y->data_ptr<float>() : nullptr, emit ? w_out->data_ptr<float>() : nullptr,
                                     (add && w_a) ? w_a->data_ptr<float>() : nullptr,
                                     (add && w_b) ? w_b->data_ptr<float>() : nullptr, emit ? h.data_ptr() : nullptr, (int)T,
                                     (int)d, (int)groups, (float)eps, add ? f32(*y) : true, out_f32, stream());
    return h;
}

void hy_rotate_qk(Tensor& proj, int64_t q_off, int64_t k_off, int64_t HQ, int64_t HK, int64_t D, int64_t dims,
                  const c10::optional<Tensor>& cos_sin, const Tensor& pos, double q_mul, double k_mul) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(proj.device());
    need(is_act(proj) && proj.dim() == 2 && proj.is_contiguous(), "rotate_qk: proj [T, C]");
    const int64_t T = proj.size(0), C = proj.size(1);
    need(HQ >= 0 && HK >= 0 && D >= 1 && q_off >= 0 && k_off >= 0 && q_off + HQ * D <= C && k_off + HK * D <= C, "rotate_qk: column ranges");
    need(dims >= 0 && dims % 2 == 0 && dims <= D, "rotate_qk: rotated columns");
    if (dims > 0) {
        need(cos_sin.has_value(), "rotate_qk: rotation needs the cos/sin table");
        flt(*cos_sin, "rotate_qk: float32 cos/sin table");
        need(cos_sin->dim() == 2 && cos_sin->size(1) == dims, "rotate_qk: table width");
    }
    i32(pos, "rotate_qk: pos");
    need(pos.numel() == T, "rotate_qk: pos [T]");
    chronos::launch_hy_rotate_qk(proj.data_ptr(), (int)C, (int)q_off, (int)k_off, (int)HQ, (int)HK, (int)D, (int)dims,
                                 dims > 0 ? cos_sin->data_ptr<float>() : nullptr, pos.data_ptr<int32_t>(), (float)q_mul,
                                 (float)k_mul, (int)T, f32(proj), stream());
}

Tensor hy_unrotate_gate(const Tensor& o, const Tensor& pos, const c10::optional<Tensor>& cos_sin,
                        const c10::optional<Tensor>& gate_src, int64_t g_off, int64_t H, int64_t Dv) {
    c10::hip::HIPGuardMasqueradingAsCUDA g(o.device());
    need(is_act(o) && o.dim() == 2 && o.is_contiguous() && o.size(1) == H * Dv, "unrotate_gate: o [T, H Dv]");
    const int64_t T = o.size(0);
    need(cos_sin.has_value() || gate_src.has_value(), "unrotate_gate: a table or a gate");
    if (cos_sin) {
        flt(*cos_sin, "unrotate_gate: float32 cos/sin table");
        need(Dv % 2 == 0 && cos_sin->dim() == 2 && cos_sin->size(1) == Dv, "unrotate_gate: table [P, Dv], Dv even");
    }
    if (gate_src) {
        same_act(o, *gate_src, "unrotate_gate: the gate's source in the activation dtype");
        need(gate_src->dim() == 2 && gate_src->is_contiguous() && gate_src->size(0) == T && g_off >= 0 &&
                 g_off + H * Dv <= gate_src->size(1), "unrotate_gate: gate columns");
    }
    i32(pos, "unrotate_gate: pos");
    need(pos.numel() == T, "unrotate_gate: pos [T]");
    auto out = at::empty_like(o);
    chronos::launch_hy_unrotate_gate(o.data_ptr(), pos.data_ptr<int32_t>(), cos_sin ? cos_sin->data_ptr<float>() : nullptr,
                                     gate_src ? gate_src->data_ptr() : nullptr, gate_src ? (int)gate_src->size(1) : 0,
                                     (int)g_off, out.data_ptr(), (int)T, (int)H, (int)Dv, f32(o), stream());
    return out;
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(chronos, m) {
    m.def("hy_embed(Tensor ids, Tensor table, float scale=1.0) -> Tensor");
    m.def("hy_cast_bf16(Tensor x) -> Tensor");
    m.def("hy_layer_norm(Tensor x, Tensor w, float eps, bool out_f32) -> Tensor");
    m.def("hy_add_layer_norm(Tensor y, Tensor(a!) x, Tensor w, float eps, bool out_f32) -> Tensor");
    m.def("hy_rowdot(Tensor h, Tensor w, Tensor? bias) -> Tensor");
    m.def("hy_act(Tensor(a!) x, int kind) -> ()");
    m.def("hy_mlstm_scan(Tensor proj, Tensor gate_pre, Tensor q_start, Tensor pos0, Tensor slots, Tensor(a!) S, "
          "Tensor(b!) n, Tensor(c!) m, int H, int D, int Dv, float cap) -> Tensor");
    m.def("hy_mlstm_out(Tensor o, Tensor proj, int g_off, Tensor w, float eps, bool out_f32) -> Tensor");
    m.def("hy_latent_prep(Tensor(a!) q, Tensor dkv, Tensor pos, Tensor tok_seq, Tensor block_table, Tensor w_norm, "
          "float eps, Tensor cos_sin, int dims, int rank, Tensor(b!) cache) -> ()");
    m.def("hy_latent_attention(Tensor qa, Tensor cache, Tensor block_table, Tensor q_start, Tensor pos, Tensor? gate, "
          "float scale, int rank, int max_q) -> Tensor");
    m.def("hy_moe_route(Tensor h, Tensor w, Tensor corr, int top) -> (Tensor, Tensor)");
    m.def("hy_moe_ffn(Tensor h, Tensor idx, Tensor wt, Tensor w_up, Tensor w_down, int act) -> Tensor");
    m.def("hy_rms_norm(Tensor x, Tensor w, float eps, bool out_f32) -> Tensor");
    m.def("hy_scale_add_rms_norm(Tensor y, Tensor(a!) x, Tensor w, float alpha, float eps, bool out_f32) -> Tensor");
    m.def("hy_glu(Tensor gu, float limit, float slope, float shift) -> Tensor");
    m.def("hy_decay_pow(Tensor(a!) z, float p) -> ()");
    m.def("hy_head_norm_gate(Tensor o, Tensor src, int g_off, Tensor w, float eps, bool silu_gate, bool out_f32) -> Tensor");
    m.def("hy_window_prep(Tensor(a!) qkv, int H, int G, int D, int Dv, Tensor? v_first, Tensor? lam, Tensor pos, "
          "Tensor tok_seq, Tensor block_table, Tensor? q_norm, Tensor? k_norm, float eps, Tensor? cos_sin, int dims, "
          "Tensor(b!) kc, Tensor(c!) vc, bool emit_v, int v_off=-1, Tensor? v_cos_sin=None) -> Tensor");
    m.def("hy_window_attention(Tensor qkv, Tensor kc, Tensor vc, Tensor block_table, Tensor q_start, Tensor pos, "
          "Tensor? sink, Tensor? gate, float scale, int window, int keep, int chunk, int H, int max_q, int pool=0, "
          "Tensor? kp=None, Tensor? vp=None, Tensor? v_cos_sin=None, int g_off=-1) -> Tensor");
    m.def("hy_pool_blocks(Tensor kc, Tensor vc, Tensor(a!) kp, Tensor(b!) vp, Tensor block_table, Tensor q_start, "
          "Tensor pos0, int pool, int max_q) -> ()");
    m.def("hy_sandwich_join(Tensor? y, Tensor? y2, Tensor(a!) x, Tensor? w_y, Tensor? w_out, Tensor? w_a, Tensor? w_b, "
          "int groups, float eps, bool out_f32, bool add, bool emit) -> Tensor");
    m.def("hy_rotate_qk(Tensor(a!) proj, int q_off, int k_off, int HQ, int HK, int D, int dims, Tensor? cos_sin, Tensor pos, "
          "float q_mul, float k_mul) -> ()");
    m.def("hy_unrotate_gate(Tensor o, Tensor pos, Tensor? cos_sin, Tensor? gate_src, int g_off, int H, int Dv) -> Tensor");
    m.def("hy_short_conv(Tensor x, Tensor w, Tensor tok_seq, Tensor q_start, Tensor pos0, Tensor slots, Tensor(a!) hist, "
          "bool silu, Tensor? bias, int x_off) -> Tensor");
    m.def("hy_delta_prep(Tensor y, Tensor ab, Tensor a_log, int HK, int H, int D, float q_mul) -> (Tensor, Tensor, Tensor, Tensor)");
    m.def("hy_linear_scan(Tensor proj, int q_off, int k_off, int v_off, Tensor? qscale, Tensor? kscale, float q_mul, "
          "Tensor decay, Tensor? beta, Tensor q_start, Tensor pos0, Tensor slots, Tensor(a!) S, int HK, int H, int D, "
          "int Dv, Tensor? vscale) -> Tensor");
    m.def("hy_moe_route_topk(Tensor h, Tensor w, Tensor bias, int top) -> (Tensor, Tensor)");
    m.def("hy_add_rms_norm(Tensor y, Tensor(a!) x, Tensor? w_out, float eps, bool out_f32, Tensor? y2, Tensor? gate2, "
          "Tensor? w_y, bool emit) -> Tensor");
    m.def("hy_token_gate(Tensor a, Tensor ids, Tensor table, int col0) -> Tensor");
    m.def("hy_ssm_prep(Tensor dt_pre, Tensor a_log) -> (Tensor, Tensor)");
    m.def("hy_gated_group_norm(Tensor o, Tensor skip_src, int skip_off, Tensor skip_w, Tensor gate_src, int g_off, Tensor w, "
          "int groups, float eps, bool out_f32) -> Tensor");
    m.def("hy_rglru_scan(Tensor u, Tensor gates, Tensor sp, float c, Tensor ysrc, int y_off, Tensor q_start, Tensor pos0, "
          "Tensor slots, Tensor(a!) S, int max_q) -> Tensor");
    m.def("hy_moe_route_group(Tensor h, Tensor w, int top, int n_groups, int keep, float scale) -> (Tensor, Tensor)");
    m.def("hy_moe_glu_ffn(Tensor h, Tensor idx, Tensor wt, Tensor w_gu, Tensor w_down, float limit, float slope, "
          "float shift, bool tiled) -> Tensor");
}

TORCH_LIBRARY_IMPL(chronos, CUDA, m) {
    m.impl("hy_embed", &hy_embed);
    m.impl("hy_cast_bf16", &hy_cast_bf16);
    m.impl("hy_layer_norm", &hy_layer_norm);
    m.impl("hy_add_layer_norm", &hy_add_layer_norm);
    m.impl("hy_rowdot", &hy_rowdot);
    m.impl("hy_act", &hy_act);
    m.impl("hy_mlstm_scan", &hy_mlstm_scan);
    m.impl("hy_mlstm_out", &hy_mlstm_out);
    m.impl("hy_latent_prep", &hy_latent_prep);
    m.impl("hy_latent_attention", &hy_latent_attention);
    m.impl("hy_moe_route", &hy_moe_route);
    m.impl("hy_moe_ffn", &hy_moe_ffn);
    m.impl("hy_rms_norm", &hy_rms_norm);
    m.impl("hy_scale_add_rms_norm", &hy_scale_add_rms_norm);
    m.impl("hy_glu", &hy_glu);
    m.impl("hy_decay_pow", &hy_decay_pow);
    m.impl("hy_head_norm_gate", &hy_head_norm_gate);
    m.impl("hy_window_prep", &hy_window_prep);
    m.impl("hy_window_attention", &hy_window_attention);
    m.impl("hy_pool_blocks", &hy_pool_blocks);
    m.impl("hy_sandwich_join", &hy_sandwich_join);
    m.impl("hy_rotate_qk", &hy_rotate_qk);
    m.impl("hy_unrotate_gate", &hy_unrotate_gate);
    m.impl("hy_short_conv", &hy_short_conv);
    m.impl("hy_delta_prep", &hy_delta_prep);
    m.impl("hy_linear_scan", &hy_linear_scan);
    m.impl("hy_moe_route_topk", &hy_moe_route_topk);
    m.impl("hy_add_rms_norm", &hy_add_rms_norm);
    m.impl("hy_token_gate", &hy_token_gate);
    m.impl("hy_ssm_prep", &hy_ssm_prep);
    m.impl("hy_gated_group_norm", &hy_gated_group_norm);
    m.impl("hy_rglru_scan", &hy_rglru_scan);
    m.impl("hy_moe_route_group", &hy_moe_route_group);
    m.impl("hy_moe_glu_ffn", &hy_moe_glu_ffn);
}
