// dgi/csrc/mix/bindings.cpp — torch.ops.dgi.* entries of the mixer-block kernels (dgi/_C_mix.so):
// Dynamic-Tanh norms, per-head q/k norm + rotary + paged KV write, row-wise masked attention,
// clamped GLU and soft-capped logits.  A library of its own, so a model that needs only these
// builds in seconds; it registers into the same `dgi` namespace as dgi/_C.so (as a fragment).
// Shapes are checked here, on the host, before any launch; every op runs on the current stream
// and allocates nothing.
#include <torch/library.h>
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

extern "C" {
int dgi_dyt(const float* x, const float* alpha, const float* w, const float* b, void* y, int is_f32, int T, int W,
            hipStream_t s);
int dgi_dyt_add(const void* h, int h_stride, const float* alpha1, const float* w1, const float* b1, const float* ls,
                float* res, const float* alpha2, const float* w2, const float* b2, void* y, int is_f32, int T, int W,
                hipStream_t s);
int dgi_embed_dyt(const long long* ids, const void* table, int vocab, float scale, const float* alpha, const float* w,
                  const float* b, float* res, int is_f32, int T, int W, hipStream_t s);
int dgi_qknorm_rope_cache(void* qkv, int is_f32, int T, int stride, const int* positions, const int* slots,
                          const float* qw, const float* kw, float eps, const float* cos_sin, int rd, int H, int G,
                          int dk, int dv, void* k_cache, void* v_cache, int block_size, hipStream_t s);
int dgi_masked_attn_rows(const void* q, int q_stride, const void* k_cache, const void* v_cache, const int* block_tables,
                         int bt_stride, const int* cu_seqlens, int n_seqs, const int* positions, int rows, int H, int G,
                         int dk, int dv, int block_size, float scale, int mask, const void* gate, int gate_stride,
                         void* out, int out_stride, int is_f32, hipStream_t s);
int dgi_paged_prefill_masked(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                             const int* block_tables, int bt_stride, const int* cu_seqlens_q, const int* context_lens,
                             const int* tiles, int n_tiles, void* out, int out_stride, int nh, int nkv, int hd,
                             int block_size, float scale, int mask, const void* gate, int gate_stride, hipStream_t s);
int dgi_glu_clamped(const void* gu, int gu_stride, void* out, int is_f32, int T, int I, float limit, float alpha,
                    hipStream_t s);
int dgi_scale_softcap(const void* x, int x_stride, float* out, int is_f32, int T, int V, float scale, float cap,
                      hipStream_t s);
}

namespace {

hipStream_t cur_stream() { return c10::hip::getCurrentHIPStream().stream(); }

void check_rc(int rc, const char* what) {
  TORCH_CHECK(rc == 0, "dgi kernel ", what, " failed with code ", rc,
              rc > 0 ? (std::string(" (") + hipGetErrorString((hipError_t)rc) + ")") : std::string());
}

// activation tensors: bf16 or fp32; returns 1 for fp32
int act_kind(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
  TORCH_CHECK(t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat, name, " must be bfloat16 or float32");
  return t.scalar_type() == at::kFloat ? 1 : 0;
}
void check_f32(const at::Tensor& t, const char* name, int64_t numel = -1) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous(), name, " must be a contiguous fp32 GPU tensor");
  TORCH_CHECK(numel < 0 || t.numel() == numel, name, " has ", t.numel(), " elements, expected ", numel);
}
void check_i32(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), name, " must be a contiguous int32 GPU tensor");
}
void check_rows(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 2 && t.stride(1) == 1, name, " must be 2-D with unit column stride");
  TORCH_CHECK(t.size(0) == 0 || t.stride(0) < (int64_t(1) << 31), name, " row stride too large");
}

void dyt(at::Tensor y, const at::Tensor& x, const at::Tensor& alpha, const at::Tensor& w, const at::Tensor& b) {
  const int f = act_kind(y, "y");
  TORCH_CHECK(x.dim() == 2 && y.dim() == 2 && y.is_contiguous() && y.sizes() == x.sizes());
  const int T = (int)x.size(0), W = (int)x.size(1);
  check_f32(x, "x"); check_f32(alpha, "alpha", 1); check_f32(w, "w", W); check_f32(b, "b", W);
  check_rc(dgi_dyt(x.data_ptr<float>(), alpha.data_ptr<float>(), w.data_ptr<float>(), b.data_ptr<float>(), y.data_ptr(), f,
                   T, W, cur_stream()), "dyt");
}

void dyt_add(at::Tensor res, const at::Tensor& h, const at::Tensor& alpha1, const at::Tensor& w1, const at::Tensor& b1,
             const at::Tensor& ls, const c10::optional<at::Tensor>& y, const c10::optional<at::Tensor>& alpha2,
             const c10::optional<at::Tensor>& w2, const c10::optional<at::Tensor>& b2) {
  const int f = act_kind(h, "h");
  check_rows(h, "h");
  TORCH_CHECK(res.dim() == 2 && h.size(0) == res.size(0) && h.size(1) == res.size(1));
  const int T = (int)res.size(0), W = (int)res.size(1);
  check_f32(res, "res"); check_f32(alpha1, "alpha1", 1); check_f32(w1, "w1", W); check_f32(b1, "b1", W); check_f32(ls, "ls", W);
  void* yp = nullptr;
  const float *a2 = nullptr, *w2p = nullptr, *b2p = nullptr;
  if (y.has_value()) {
    TORCH_CHECK(alpha2.has_value() && w2.has_value() && b2.has_value(), "dyt_add: y needs the next norm");
    TORCH_CHECK(act_kind(*y, "y") == f && y->is_contiguous() && y->sizes() == res.sizes());
    check_f32(*alpha2, "alpha2", 1); check_f32(*w2, "w2", W); check_f32(*b2, "b2", W);
    yp = y->data_ptr(); a2 = alpha2->data_ptr<float>(); w2p = w2->data_ptr<float>(); b2p = b2->data_ptr<float>();
  }
  check_rc(dgi_dyt_add(h.data_ptr(), (int)h.stride(0), alpha1.data_ptr<float>(), w1.data_ptr<float>(), b1.data_ptr<float>(),
                       ls.data_ptr<float>(), res.data_ptr<float>(), a2, w2p, b2p, yp, f, T, W, cur_stream()), "dyt_add");
}

void embed_dyt(at::Tensor res, const at::Tensor& ids, const at::Tensor& table, double scale, const at::Tensor& alpha,
               const at::Tensor& w, const at::Tensor& b) {
  const int f = act_kind(table, "table");
  TORCH_CHECK(ids.is_cuda() && ids.scalar_type() == at::kLong && ids.is_contiguous(), "ids must be contiguous int64");
  TORCH_CHECK(table.dim() == 2 && table.is_contiguous() && res.dim() == 2);
  const int T = (int)ids.numel(), W = (int)table.size(1);
  TORCH_CHECK(res.size(0) == T && res.size(1) == W);
  check_f32(res, "res"); check_f32(alpha, "alpha", 1); check_f32(w, "w", W); check_f32(b, "b", W);
  check_rc(dgi_embed_dyt((const long long*)ids.data_ptr<int64_t>(), table.data_ptr(), (int)table.size(0), (float)scale,
                         alpha.data_ptr<float>(), w.data_ptr<float>(), b.data_ptr<float>(), res.data_ptr<float>(), f, T, W,
                         cur_stream()), "embed_dyt");
}

// qkv rows: [q: H*dk | k: G*dk | v: G*dv | ...]; k_cache [NB, G, bs, dk], v_cache [NB, G, bs, dv]
void qknorm_rope_cache(at::Tensor qkv, const at::Tensor& positions, const at::Tensor& slots, const at::Tensor& qw,
                       const at::Tensor& kw, double eps, const c10::optional<at::Tensor>& cos_sin, int64_t H, int64_t G,
                       int64_t dk, int64_t dv, at::Tensor k_cache, at::Tensor v_cache) {
  const int f = act_kind(qkv, "qkv");
  check_rows(qkv, "qkv");
  check_i32(positions, "positions"); check_i32(slots, "slots");
  check_f32(qw, "qw", dk); check_f32(kw, "kw", dk);
  const int T = (int)qkv.size(0);
  TORCH_CHECK(positions.numel() == T && slots.numel() == T);
  TORCH_CHECK(qkv.size(1) >= (H + G) * dk + G * dv, "qkv rows too short");
  TORCH_CHECK(act_kind(k_cache, "k_cache") == f && act_kind(v_cache, "v_cache") == f);
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() && k_cache.dim() == 4 && v_cache.dim() == 4);
  TORCH_CHECK(k_cache.size(1) == G && k_cache.size(3) == dk && v_cache.size(1) == G && v_cache.size(3) == dv &&
              v_cache.size(0) == k_cache.size(0) && v_cache.size(2) == k_cache.size(2), "cache geometry");
  int rd = 0;
  const float* cs = nullptr;
  if (cos_sin.has_value()) {
    check_f32(*cos_sin, "cos_sin");
    TORCH_CHECK(cos_sin->dim() == 2);
    rd = (int)cos_sin->size(1);
    cs = cos_sin->data_ptr<float>();
  }
  check_rc(dgi_qknorm_rope_cache(qkv.data_ptr(), f, T, (int)qkv.stride(0), positions.data_ptr<int>(), slots.data_ptr<int>(),
                                 qw.data_ptr<float>(), kw.data_ptr<float>(), (float)eps, cs, rd, (int)H, (int)G, (int)dk,
                                 (int)dv, k_cache.data_ptr(), v_cache.data_ptr(), (int)k_cache.size(2), cur_stream()),
           "qknorm_rope_cache");
}

// rows of q (stride q.stride(0), H*dk used columns) attend over their sequence's pages;
// cu_seqlens (n_seqs + 1) maps rows to block-table rows, absent: row i <-> block-table row i
void masked_attn_rows(at::Tensor out, const at::Tensor& q, const at::Tensor& k_cache, const at::Tensor& v_cache,
                      const at::Tensor& block_tables, const c10::optional<at::Tensor>& cu_seqlens,
                      const at::Tensor& positions, int64_t H, int64_t G, double scale, int64_t mask,
                      const c10::optional<at::Tensor>& gate) {
  const int f = act_kind(q, "q");
  check_rows(q, "q"); check_rows(out, "out");
  TORCH_CHECK(act_kind(out, "out") == f && act_kind(k_cache, "k_cache") == f && act_kind(v_cache, "v_cache") == f);
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() && k_cache.dim() == 4 && v_cache.dim() == 4);
  check_i32(block_tables, "block_tables"); check_i32(positions, "positions");
  TORCH_CHECK(block_tables.dim() == 2);
  const int rows = (int)q.size(0);
  const int dk = (int)k_cache.size(3), dv = (int)v_cache.size(3);
  TORCH_CHECK(k_cache.size(1) == G && v_cache.size(1) == G && v_cache.size(2) == k_cache.size(2));
  TORCH_CHECK(q.size(1) >= H * dk && out.size(0) == rows && out.size(1) >= H * dv && positions.numel() == rows);
  int n_seqs = (int)block_tables.size(0);
  const int* cu = nullptr;
  if (cu_seqlens.has_value()) {
    check_i32(*cu_seqlens, "cu_seqlens");
    TORCH_CHECK(cu_seqlens->numel() == n_seqs + 1);
    cu = cu_seqlens->data_ptr<int>();
  } else {
    TORCH_CHECK(n_seqs >= rows, "one block-table row per query row");
  }
  const void* gp = nullptr;
  int gs = 0;
  if (gate.has_value()) {
    check_rows(*gate, "gate");
    TORCH_CHECK(act_kind(*gate, "gate") == f && gate->size(0) == rows && gate->size(1) >= H * dv);
    gp = gate->data_ptr();
    gs = (int)gate->stride(0);
  }
  check_rc(dgi_masked_attn_rows(q.data_ptr(), (int)q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
                                block_tables.data_ptr<int>(), (int)block_tables.stride(0), cu, n_seqs,
                                positions.data_ptr<int>(), rows, (int)H, (int)G, dk, dv, (int)k_cache.size(2), (float)scale,
                                (int)mask, gp, gs, out.data_ptr(), (int)out.stride(0), f, cur_stream()),
           "masked_attn_rows");
}

// bf16, key size == value size in {64, 128}: packed prompt portions (cu_seqlens_q) over
// [cached prefix | new keys]; tiles [n, 2] = (sequence, first row of a 128-row tile)
void paged_prefill_masked(at::Tensor out, const at::Tensor& q, const at::Tensor& k_cache, const at::Tensor& v_cache,
                          const at::Tensor& block_tables, const at::Tensor& cu_seqlens_q, const at::Tensor& context_lens,
                          const at::Tensor& tiles, int64_t nh, int64_t nkv, double scale, int64_t mask,
                          const c10::optional<at::Tensor>& gate) {
  TORCH_CHECK(act_kind(q, "q") == 0 && act_kind(out, "out") == 0 && act_kind(k_cache, "k_cache") == 0 &&
              act_kind(v_cache, "v_cache") == 0, "paged_prefill_masked: bfloat16 only");
  check_rows(q, "q"); check_rows(out, "out");
  check_i32(block_tables, "block_tables"); check_i32(cu_seqlens_q, "cu_seqlens_q");
  check_i32(context_lens, "context_lens"); check_i32(tiles, "tiles");
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() && k_cache.dim() == 4 && k_cache.sizes() == v_cache.sizes());
  const int hd = (int)k_cache.size(3);
  TORCH_CHECK(k_cache.size(1) == nkv && q.size(1) >= nh * hd && out.size(1) >= nh * hd && out.size(0) == q.size(0));
  TORCH_CHECK(q.stride(0) % 8 == 0 && out.stride(0) % 4 == 0 && q.data_ptr<at::BFloat16>() != nullptr);
  TORCH_CHECK(reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 == 0 && reinterpret_cast<uintptr_t>(out.data_ptr()) % 8 == 0,
              "paged_prefill_masked: q must be 16-byte and out 8-byte aligned");
  const int nb = (int)cu_seqlens_q.numel() - 1;
  TORCH_CHECK(block_tables.dim() == 2 && block_tables.size(0) >= nb && context_lens.numel() >= nb);
  TORCH_CHECK(tiles.dim() == 2 && tiles.size(1) == 2);
  const void* gp = nullptr;
  int gs = 0;
  if (gate.has_value()) {
    check_rows(*gate, "gate");
    TORCH_CHECK(act_kind(*gate, "gate") == 0 && gate->size(0) == q.size(0) && gate->size(1) >= nh * hd);
    TORCH_CHECK(gate->stride(0) % 4 == 0 && reinterpret_cast<uintptr_t>(gate->data_ptr()) % 8 == 0, "gate alignment");
    gp = gate->data_ptr();
    gs = (int)gate->stride(0);
  }
  check_rc(dgi_paged_prefill_masked(q.data_ptr(), (int)q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
                                    block_tables.data_ptr<int>(), (int)block_tables.stride(0), cu_seqlens_q.data_ptr<int>(),
                                    context_lens.data_ptr<int>(), tiles.data_ptr<int>(), (int)tiles.size(0), out.data_ptr(),
                                    (int)out.stride(0), (int)nh, (int)nkv, hd, (int)k_cache.size(2), (float)scale, (int)mask,
                                    gp, gs, cur_stream()), "paged_prefill_masked");
}

void glu_clamped(at::Tensor out, const at::Tensor& gu, double limit, double alpha) {
  const int f = act_kind(gu, "gu");
  check_rows(gu, "gu");
  TORCH_CHECK(act_kind(out, "out") == f && out.is_contiguous() && out.dim() == 2 && out.size(0) == gu.size(0) &&
              2 * out.size(1) == gu.size(1));
  check_rc(dgi_glu_clamped(gu.data_ptr(), (int)gu.stride(0), out.data_ptr(), f, (int)gu.size(0), (int)out.size(1),
                           (float)limit, (float)alpha, cur_stream()), "glu_clamped");
}

void scale_softcap(at::Tensor out, const at::Tensor& x, double scale, double cap) {
  const int f = act_kind(x, "x");
  check_rows(x, "x");
  check_f32(out, "out", x.numel());
  check_rc(dgi_scale_softcap(x.data_ptr(), (int)x.stride(0), out.data_ptr<float>(), f, (int)x.size(0), (int)x.size(1),
                             (float)scale, (float)cap, cur_stream()), "scale_softcap");
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(dgi, m) {
  m.def("dyt(Tensor(a!) y, Tensor x, Tensor alpha, Tensor w, Tensor b) -> ()");
  m.def("dyt_add(Tensor(a!) res, Tensor h, Tensor alpha1, Tensor w1, Tensor b1, Tensor ls, Tensor(b!)? y, "
        "Tensor? alpha2, Tensor? w2, Tensor? b2) -> ()");
  m.def("embed_dyt(Tensor(a!) res, Tensor ids, Tensor table, float scale, Tensor alpha, Tensor w, Tensor b) -> ()");
  m.def("qknorm_rope_cache(Tensor(a!) qkv, Tensor positions, Tensor slots, Tensor qw, Tensor kw, float eps, "
        "Tensor? cos_sin, int H, int G, int dk, int dv, Tensor(b!) k_cache, Tensor(c!) v_cache) -> ()");
  m.def("masked_attn_rows(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, Tensor block_tables, "
        "Tensor? cu_seqlens, Tensor positions, int H, int G, float scale, int mask, Tensor? gate) -> ()");
  m.def("paged_prefill_masked(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, Tensor block_tables, "
        "Tensor cu_seqlens_q, Tensor context_lens, Tensor tiles, int nh, int nkv, float scale, int mask, "
        "Tensor? gate) -> ()");
  m.def("glu_clamped(Tensor(a!) out, Tensor gu, float limit, float alpha) -> ()");
  m.def("scale_softcap(Tensor(a!) out, Tensor x, float scale, float cap) -> ()");
}

TORCH_LIBRARY_IMPL(dgi, CUDA, m) {
  m.impl("dyt", &dyt);
  m.impl("dyt_add", &dyt_add);
  m.impl("embed_dyt", &embed_dyt);
  m.impl("qknorm_rope_cache", &qknorm_rope_cache);
  m.impl("masked_attn_rows", &masked_attn_rows);
  m.impl("paged_prefill_masked", &paged_prefill_masked);
  m.impl("glu_clamped", &glu_clamped);
  m.impl("scale_softcap", &scale_softcap);
}
