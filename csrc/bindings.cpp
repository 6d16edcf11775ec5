// Python bindings for the gfx950 kernel library (torch tensors -> raw launchers).
// Every entry point validates shapes/dtypes/devices on the host BEFORE launching, so a
// mis-shaped call raises instead of faulting the GPU, and launches on torch's current HIP
// stream (graph-capturable: no allocation, no sync inside).
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

#include "kernels/tgemm_args.h"

extern "C" {
int dllm_norm(const void*, const void*, void*, const void*, const void*, void*, int, int, long, long, float, int,
              hipStream_t);
int dllm_rope_kv(const void*, long, const int*, const float*, const int*, void*, void*, void*, int, int, int, int, int,
                 hipStream_t);
int dllm_kv_write(const void*, const void*, long, const int*, void*, void*, int, int, int, int, hipStream_t);
int dllm_paged_attention(const void*, const void*, const void*, const int*, const int*, const int*, const int*,
                         const int*, const int*, void*, float*, float*, int*, const int*, const int*, int, int, int,
                         int, int, int, int, int, int, float, const void*, hipStream_t);
int dllm_silu_mul(const void*, void*, long, int, long, hipStream_t);
int dllm_embed(const int*, const void*, void*, long, int, long, long, float*, int*, const int*, int, hipStream_t);
int dllm_gemv(const void*, long, const void*, void*, long, int, int, int, int, int, const void*, void*, const void*,
              float, hipStream_t);
int dllm_gelu(const void*, void*, long, hipStream_t);
int dllm_mean_pool_l2(const void*, const int*, float*, int, int, int, hipStream_t);
int dllm_moe_gate(const float*, int, int, int, int*, float*, hipStream_t);
int dllm_moe_router(const void*, long, const void*, int, int, int, int, int*, float*, float*, hipStream_t);
int dllm_scatter_pairs(int*, const int*, int, hipStream_t);
int dllm_step_fetch(const int*, int*, int, int, int, int, const int*, const int*, int*, int, hipStream_t);
int dllm_step_store(const int*, int*, int, hipStream_t);
int dllm_argmax(const void*, long, int, int, int, int*, hipStream_t);
int dllm_sample_topp(const float*, const long*, int, int, const float*, const float*, const float*, int*, hipStream_t);
int dllm_cosine_scores(const float*, const float*, float*, int, int, int, hipStream_t);
int dllm_sample_rows(const void*, long, int, int, const float*, const float*, const int*, const unsigned*, int*,
                     hipStream_t);
int dllm_tp_cands_k();
int dllm_tp_cands(const void*, long, int, int, int, void*, hipStream_t);
int dllm_tp_sample(const void*, int, int, const float*, const float*, const int*, const unsigned*, int*, hipStream_t);
int dllm_sample_split(const void*, long, int, int, int, const float*, const float*, const int*, const unsigned*, void*,
                      long, int*, int*, hipStream_t);
int dllm_sample_split_maxp();
int dllm_sample_split_kmax();
int dllm_skinny_epi(const void*, long, const void*, int, void*, long, int, int, int, int, int, int, float*, int*, void*,
                    long, float*, long, const float*, int, long, float, float, const int*, const float*, const int*,
                    void*, void*, void*, int, int, int, hipStream_t);
int dllm_skinny_gemm(const void*, long, const void*, void*, long, int, int, int, int, int, int, float*, int*,
                     hipStream_t);
int dllm_moe_max_tiles(int, int);
int dllm_moe_ffn(const void*, long, long, int, const int*, const float*, int, int, const void*, const void*, int, int*,
                 int*, void*, float*, void*, int, hipStream_t);
int dllm_rms_rows(const void*, long, int, const float*, void*, long, int, int, int, float, int, hipStream_t);
int dllm_norm_resadd(const void*, long, int, const float*, float*, void*, int, int, float, int, const float*, hipStream_t);
int dllm_polynorm(const void*, long, int, const float*, void*, long, int, float, hipStream_t);
int dllm_route_topk(const float*, long, int, int, int, int, int, int, int, const float*, int, int*, float*, float*, hipStream_t);
int dllm_ls_resadd_ln(const void*, long, int, const float*, const float*, const void*, long, const float*, long, const void*, long,
                      const float*, float*, const float*, const float*, void*, long, int, float, hipStream_t);
int dllm_glu_act(const void*, long, int, const float*, int, int, float, float, void*, long, hipStream_t);
int dllm_proj_norm_prep(const void*, long, int, int, int, int, int, const float*, const float*, const float*, int, int, int, float,
                        const float*, int, const int*, const int*, void*, void*, void*, long, int, void*, int, hipStream_t);
int dllm_group_router(const float*, int, int, int, int, int, int*, float*, hipStream_t);
int dllm_swiglu_scale(const void*, int, const float*, int, int, void*, long, hipStream_t);
int dllm_softcap(const void*, int, float, float*, long, hipStream_t);
int dllm_gated_group_norm(const float*, const void*, long, int, const float*, void*, int, int, int, float, hipStream_t);
int dllm_outer_scan_cols();
int dllm_ssd_scan(const void*, long, const void*, long, int, int, int, int, int, int, const float*, const float*, const float*,
                  float*, const int*, const int*, const int*, const int*, int, float*, hipStream_t);
int dllm_mlstm(const void*, long, int, int, int, int, const float*, float, float*, float*, int, float, const float*, const int*,
               const int*, const int*, const int*, int, long, float*, void*, hipStream_t);
int dllm_qk_norm_prep(const void*, long, int, const float*, int, int, int, int, int, const float*, const float*, const float*,
                      int, int, float, float, const int*, const int*, void*, void*, void*, long, int, hipStream_t);
int dllm_diff_combine(const float*, void*, int, long, int, int, int, float, float, float, hipStream_t);
int dllm_conv_silu(const void*, long, int, const float*, const float*, void*, const int*, const int*, const int*,
                   const int*, void*, int, int, int, int, int, int, hipStream_t);
int dllm_selective_scan(const void*, const void*, int, const float*, const float*, const void*, long, int, const float*,
                        const void*, long, float*, void*, int, const int*, const int*, const int*, const int*, void*, int,
                        int, int, hipStream_t);
long dllm_retention_lds(int, int);
int dllm_retention(const void*, long, int, int, int, int, const float*, int, int, const float*, float*, float,
                   const int*, const int*, const int*, const int*, void*, int, int, float, float*, hipStream_t);
long dllm_retention_chunk_lds(int);
int dllm_retention_chunked(const void*, long, int, int, int, int, const float*, int, int, const float*, float*, float,
                           const int*, const int*, const int*, const int*, float*, void*, int, long, int, float, int,
                           hipStream_t);
int dllm_heads_norm_gate(const float*, const void*, long, int, long, int, const float*, float, const int*, const int*, int,
                         void*, long, hipStream_t);
int dllm_resadd_norm(const void*, long, const void*, long, int, const float*, const float*, const float*, float*,
                     const float*, void*, int, int, float, const float*, int, hipStream_t);
int dllm_depth_mix(float*, const float*, int, long, int, const float*, void*, int, float, hipStream_t);
int dllm_gelu_erf(const void*, void*, int, long, hipStream_t);
int dllm_conv_refill(const void*, long, int, void*, int, int, const int*, const int*, const int*, const int*, int,
                     hipStream_t);
int dllm_delta_rule(const void*, long, const void*, long, int, int, int, int, int, const float*, const float*, const float*,
                    float, float*, const int*, const int*, const int*, const int*, float*, void*, int, long, hipStream_t);
int dllm_attn_prep(const void*, long, int, int, int, int, int, const float*, int, int, float, const float*, const int*,
                   const int*, void*, void*, void*, long, int, hipStream_t);
int dllm_gqa_tile_tokens(int, int, int);
int dllm_gqa_mfma_ok(int, int, int, int, int, int);
int dllm_paged_gqa(const void*, const void*, const void*, int, const int*, int, int, const int*, const int*, const int*,
                   const int*, const int*, int, const void*, long, void*, int, int, int, int, int, int, float*, int, int, int,
                   int, float, hipStream_t);
int dllm_relu2_scale(const void*, int, const float*, int, int, void*, long, int, hipStream_t);
int dllm_dense_gate(const int*, const float*, float*, long, int, int, hipStream_t);
int dllm_latent_kv_write(const void*, long, int, int, int, const float*, float, const int*, const float*, int, const int*,
                         void*, int, hipStream_t);
int dllm_latent_attention(const void*, const void*, long, int, int, int, int, int, long, const float*, int, const void*,
                          const int*, int, const int*, const int*, const int*, const int*, const int*, int, float, void*,
                          int, float*, float*, int, int, hipStream_t);
int dllm_latent_mfma_ok(int, int, int);
int dllm_car_alloc(long, void**);
int dllm_car_get_handle(void*, char*);
int dllm_car_handle_size();
int dllm_car_open_handle(const char*, void**);
int dllm_car_close_handle(void*);
int dllm_car_free(void*);
int dllm_car_allreduce(const void*, void*, long, void* const*, int, int, long, unsigned*, int*, long, hipStream_t);
int dllm_car_resadd_slots(int);
int dllm_car_resadd(const void*, void*, long, float*, long, int, int, int, void* const*, int, int, long, unsigned*, int*,
                    long, hipStream_t);
int dllm_car_allgather(const void*, void*, long, void* const*, int, int, long, unsigned*, int*, long, hipStream_t);
int dllm_car_vote(int, int*, void*, int*, hipStream_t);
int dllm_tgemm(const void*, int, int, int, int, int, int, int, hipStream_t, int);
int dllm_moe_max_tiles_bm(int, int, int);
int dllm_moe_ffn_tg(const void*, long, long, int, const int*, const float*, int, int, const void*, const void*, int,
                    int*, int*, int*, void*, void*, void*, const int*, hipStream_t);
int dllm_encoder_attention(const void*, const int*, void*, int, int, int, int, float, hipStream_t);
int dllm_embed_ln(const int*, const void*, const void*, const void*, const void*, const void*, void*, int, int, int, int,
                  float, hipStream_t);
int dllm_res_add_ssq(const void*, long, void*, long, float*, long, int, int, int, hipStream_t);
int dllm_gemv_slots(int, int, int);
void dllm_gemv_set_grid(int, int, int);
int dllm_gemv_epi(const void*, long, const void*, void*, long, int, int, int, int, int, void*, long, float*, long,
                  const float*, int, long, float, float, const int*, const float*, const int*, void*, void*, void*, int,
                  int, int, hipStream_t);
int dllm_qkv_post(const void*, long, const float*, int, long, float, float, const int*, const float*, const int*, void*,
                  void*, void*, void*, int, int, int, int, hipStream_t);
int dllm_swiglu_post(const void*, long, const float*, int, long, float, float, void*, long, int, int, hipStream_t);
int dllm_flash_prefill(const void*, const void*, const void*, const int*, const int*, const int*, const int*, const int*,
                       const int*, void*, int, int, int, int, int, int, float, int, float*, float*, int*, hipStream_t);
int dllm_cache_scan(const unsigned long long*, const int*, int, const float*, const int*, long, int, float,
                    unsigned long long*, hipStream_t);
int dllm_cache_write(const unsigned long long*, const long long*, const int*, int, float*, int*, int, hipStream_t);
}

namespace {
hipStream_t stream() { return c10::hip::getCurrentHIPStream().stream(); }

void check_dev(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
}
void check_bf16(const torch::Tensor& t, const char* name) {
  check_dev(t, name);
  TORCH_CHECK(t.scalar_type() == torch::kBFloat16, name, " must be bf16");
}
void check_i32(const torch::Tensor& t, const char* name) {
  check_dev(t, name);
  TORCH_CHECK(t.scalar_type() == torch::kInt32 && t.is_contiguous(), name, " must be contiguous int32");
}
void check_f32(const torch::Tensor& t, const char* name) {
  check_dev(t, name);
  TORCH_CHECK(t.scalar_type() == torch::kFloat32 && t.is_contiguous(), name, " must be contiguous f32");
}
void ok(int rc, const char* what) { TORCH_CHECK(rc == 0, what, " launch failed, code ", rc); }

// y = norm(x (+ residual)) * w (+ b); residual (if given) is updated in place to x + residual.
void norm(torch::Tensor x, c10::optional<torch::Tensor> residual, torch::Tensor w, c10::optional<torch::Tensor> b,
          torch::Tensor y, double eps, bool layernorm) {
  check_bf16(x, "x");
  check_bf16(w, "w");
  check_bf16(y, "y");
  TORCH_CHECK(x.dim() == 2 && y.dim() == 2 && x.stride(1) == 1 && y.stride(1) == 1, "x, y: 2-D row-major");
  const int rows = x.size(0), H = x.size(1);
  TORCH_CHECK(y.size(0) == rows && y.size(1) == H && w.numel() == H, "shape mismatch");
  const void* rp = nullptr;
  if (residual) {
    check_bf16(*residual, "residual");
    TORCH_CHECK(residual->is_contiguous() && residual->size(0) == rows && residual->size(1) == H, "residual shape");
    rp = residual->data_ptr();
  }
  const void* bp = nullptr;
  if (layernorm) {
    TORCH_CHECK(b.has_value(), "layernorm needs bias");
    check_bf16(*b, "b");
    bp = b->data_ptr();
  }
  ok(dllm_norm(x.data_ptr(), rp, residual ? residual->data_ptr() : nullptr, w.data_ptr(), bp, y.data_ptr(), rows, H,
               x.stride(0), y.stride(0), (float)eps, layernorm ? 1 : 0, stream()),
     "norm");
}

void rope_kv(torch::Tensor qkv, torch::Tensor pos, torch::Tensor cos_sin, torch::Tensor slots, torch::Tensor q_out,
             torch::Tensor kc, torch::Tensor vc, int64_t nq, int64_t nkv, int64_t d) {
  check_bf16(qkv, "qkv");
  check_i32(pos, "positions");
  check_f32(cos_sin, "cos_sin");
  check_i32(slots, "slot_mapping");
  check_bf16(q_out, "q_out");
  check_bf16(kc, "k_cache");
  check_bf16(vc, "v_cache");
  TORCH_CHECK(qkv.dim() == 2 && qkv.stride(1) == 1 && qkv.size(1) >= (nq + 2 * nkv) * d, "qkv shape");
  const int T = qkv.size(0);
  TORCH_CHECK(pos.numel() == T && slots.numel() == T, "positions/slots length");
  TORCH_CHECK(q_out.is_contiguous() && q_out.numel() == (int64_t)T * nq * d, "q_out shape");
  TORCH_CHECK(cos_sin.dim() == 2 && cos_sin.size(1) == d, "cos_sin must be [max_pos, d]");
  TORCH_CHECK(kc.is_contiguous() && vc.is_contiguous() && kc.dim() == 4 && kc.size(1) == nkv && kc.size(2) == 16 &&
                  kc.size(3) == d && vc.size(2) == d && vc.size(3) == 16,
              "cache layout: K [blocks, nkv, 16, d], V [blocks, nkv, d, 16]");
  if (T == 0) return;
  ok(dllm_rope_kv(qkv.data_ptr(), qkv.stride(0), pos.data_ptr<int>(), cos_sin.data_ptr<float>(),
                  slots.data_ptr<int>(), q_out.data_ptr(), kc.data_ptr(), vc.data_ptr(), T, nq, nkv, d, 16, stream()),
     "rope_kv");
}

void kv_write(torch::Tensor k, torch::Tensor v, torch::Tensor slots, torch::Tensor kc, torch::Tensor vc) {
  check_bf16(k, "k");
  check_bf16(v, "v");
  check_i32(slots, "slots");
  TORCH_CHECK(k.dim() == 3 && k.is_contiguous() && v.is_contiguous() && v.sizes() == k.sizes(), "k/v [T, nkv, d]");
  const int T = k.size(0), nkv = k.size(1), d = k.size(2);
  TORCH_CHECK(kc.size(1) == nkv && kc.size(3) == d, "cache shape");
  if (T == 0) return;
  ok(dllm_kv_write(k.data_ptr(), v.data_ptr(), (long)nkv * d, slots.data_ptr<int>(), kc.data_ptr(), vc.data_ptr(), T,
                   nkv, d, 16, stream()),
     "kv_write");
}

void paged_attention(torch::Tensor q, torch::Tensor kc, torch::Tensor vc, torch::Tensor block_tables,
                     torch::Tensor qstart, torch::Tensor qlen, torch::Tensor ctx, torch::Tensor tile_seq,
                     torch::Tensor tile_tok0, torch::Tensor out, c10::optional<torch::Tensor> part_o,
                     c10::optional<torch::Tensor> part_ml, c10::optional<torch::Tensor> counters, int64_t splits,
                     bool causal, double scale, c10::optional<torch::Tensor> split_len, bool xcd_remap,
                     c10::optional<torch::Tensor> items, int64_t grid_items, c10::optional<torch::Tensor> v_new) {
  check_bf16(q, "q");
  check_bf16(kc, "k_cache");
  check_bf16(vc, "v_cache");
  check_bf16(out, "out");
  for (auto* t : {&block_tables, &qstart, &qlen, &ctx, &tile_seq, &tile_tok0}) check_i32(*t, "attention metadata");
  TORCH_CHECK(q.dim() == 3 && q.is_contiguous() && out.is_contiguous() && out.sizes() == q.sizes(), "q/out [T, nq, d]");
  const int nq = q.size(1), d = q.size(2);
  TORCH_CHECK(kc.dim() == 4 && kc.size(2) == 16 && kc.size(3) == d && vc.size(2) == d && vc.size(3) == 16,
              "cache layout");
  const int nkv = kc.size(1);
  TORCH_CHECK(nq % nkv == 0 && 16 % (nq / nkv) == 0, "GQA group must divide 16");
  TORCH_CHECK(d == 64 || d == 96 || d == 128, "head_dim must be 64, 96 or 128");
  TORCH_CHECK(block_tables.dim() == 2, "block_tables [num_seqs, max_blocks]");
  const int num_seqs = block_tables.size(0);
  TORCH_CHECK(qstart.numel() == num_seqs && qlen.numel() == num_seqs && ctx.numel() == num_seqs, "seq metadata len");
  const int num_tiles = tile_seq.numel();
  TORCH_CHECK(tile_tok0.numel() == num_tiles, "tile metadata len");
  float* po = nullptr;
  float* pml = nullptr;
  int* cnt = nullptr;
  if (splits > 1) {
    TORCH_CHECK(counters.has_value(), "split-K needs a zeroed counter buffer");
    check_i32(*counters, "counters");
    TORCH_CHECK(counters->numel() >= (int64_t)num_tiles * nkv, "counter buffer too small");
    cnt = counters->data_ptr<int>();
    TORCH_CHECK(part_o.has_value() && part_ml.has_value(), "split-K needs workspaces");
    check_f32(*part_o, "part_o");
    check_f32(*part_ml, "part_ml");
    TORCH_CHECK(part_o->numel() >= (int64_t)num_tiles * nkv * splits * 16 * d &&
                    part_ml->numel() >= (int64_t)num_tiles * nkv * splits * 16 * 2,
                "workspace too small");
    po = part_o->data_ptr<float>();
    pml = part_ml->data_ptr<float>();
  }
  const int* sl = nullptr;
  if (split_len.has_value()) {
    check_i32(*split_len, "split_len");
    TORCH_CHECK(split_len->numel() >= 1, "split_len: device scalar");
    sl = split_len->data_ptr<int>();
  }
  const int* it = nullptr;
  if (items.has_value()) {
    // work list [1 + 2 * n]: units outside (num_tiles, nkv, splits) are skipped by the kernel; the
    // two ints after the tile counters hold the dynamic-fetch cursor and exit count (kept zeroed)
    check_i32(*items, "items");
    TORCH_CHECK(splits > 1 && cnt != nullptr, "work-list attention needs split-K workspaces");
    TORCH_CHECK(items->numel() >= 1, "work list [1 + 2n]");
    TORCH_CHECK(counters->numel() >= (int64_t)num_tiles * nkv + 2, "work list: counters need 2 cursor slots");
    TORCH_CHECK(grid_items >= 1 && !xcd_remap, "work-list attention: grid >= 1, no XCD remap");
    it = items->data_ptr<int>();
  }
  const void* vn = nullptr;
  if (v_new.has_value()) {   // decode: the newest token's V row-major [T, nkv * d] (tgemm v_rows)
    check_bf16(*v_new, "v_new");
    TORCH_CHECK(v_new->is_contiguous() && v_new->numel() >= (int64_t)q.size(0) * nkv * d, "v_new [T, nkv * d]");
    vn = v_new->data_ptr();
  }
  ok(dllm_paged_attention(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), block_tables.data_ptr<int>(),
                          qstart.data_ptr<int>(), qlen.data_ptr<int>(), ctx.data_ptr<int>(), tile_seq.data_ptr<int>(),
                          tile_tok0.data_ptr<int>(), out.data_ptr(), po, pml, cnt, sl, it, (int)grid_items,
                          xcd_remap ? 1 : 0, num_tiles, nq, nkv, d, block_tables.size(1), splits, causal ? 1 : 0,
                          (float)scale, vn, stream()),
     "paged_attention");
}

// Flash-style prefill attention (csrc/kernels/flash_prefill.hip): 256-row GQA tiles with K/V
// staged once per workgroup in LDS.  tile_seq/tile_tok0 hold 256 / G tokens per tile.
void flash_prefill(torch::Tensor q, torch::Tensor kc, torch::Tensor vc, torch::Tensor block_tables,
                   torch::Tensor qstart, torch::Tensor qlen, torch::Tensor ctx, torch::Tensor tile_seq,
                   torch::Tensor tile_tok0, torch::Tensor out, bool causal, double scale, int64_t splits,
                   c10::optional<torch::Tensor> part_o, c10::optional<torch::Tensor> part_ml,
                   c10::optional<torch::Tensor> counters) {
  check_bf16(q, "q");
  check_bf16(kc, "k_cache");
  check_bf16(vc, "v_cache");
  check_bf16(out, "out");
  for (auto* t : {&block_tables, &qstart, &qlen, &ctx, &tile_seq, &tile_tok0}) check_i32(*t, "attention metadata");
  TORCH_CHECK(q.dim() == 3 && q.is_contiguous() && out.is_contiguous() && out.sizes() == q.sizes(), "q/out [T, nq, d]");
  const int nq = q.size(1), d = q.size(2);
  TORCH_CHECK(d == 64 || d == 96 || d == 128, "flash prefill: head_dim 64, 96 or 128");
  TORCH_CHECK(kc.is_contiguous() && vc.is_contiguous() && kc.dim() == 4 && kc.size(2) == 16 && kc.size(3) == d &&
                  vc.size(2) == d && vc.size(3) == 16,
              "cache layout");
  const int nkv = kc.size(1);
  TORCH_CHECK(nq % nkv == 0 && 128 % (nq / nkv) == 0, "GQA group must divide 128");
  TORCH_CHECK(block_tables.dim() == 2 && block_tables.size(1) >= 1, "block_tables [S, max_blocks]");
  const int S = block_tables.size(0);
  TORCH_CHECK(qstart.numel() == S && qlen.numel() == S && ctx.numel() == S, "seq metadata len");
  TORCH_CHECK(tile_tok0.numel() == tile_seq.numel(), "tile metadata len");
  float* po = nullptr;
  float* pml = nullptr;
  int* cnt = nullptr;
  if (splits > 1) {
    TORCH_CHECK(splits <= 16 && part_o.has_value() && part_ml.has_value() && counters.has_value(),
                "flash_prefill: split-KV needs part_o / part_ml / counters, splits <= 16");
    const long units = (long)tile_seq.numel() * nkv * splits;
    check_f32(*part_o, "part_o");
    check_f32(*part_ml, "part_ml");
    check_i32(*counters, "counters");
    TORCH_CHECK(part_o->numel() >= units * 256 * d && part_ml->numel() >= units * 256 * 4 &&
                    counters->numel() >= (long)tile_seq.numel() * nkv,
                "flash_prefill: split-KV workspace too small");
    po = part_o->data_ptr<float>();
    pml = part_ml->data_ptr<float>();
    cnt = counters->data_ptr<int>();
  }
  ok(dllm_flash_prefill(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), block_tables.data_ptr<int>(), qstart.data_ptr<int>(),
                        qlen.data_ptr<int>(), ctx.data_ptr<int>(), tile_seq.data_ptr<int>(), tile_tok0.data_ptr<int>(),
                        out.data_ptr(), tile_seq.numel(), nq, nkv, d, block_tables.size(1), causal ? 1 : 0,
                        (float)scale, (int)std::max<int64_t>(1, splits), po, pml, cnt, stream()),
     "flash_prefill");
}

void silu_mul(torch::Tensor gu, torch::Tensor out) {
  check_bf16(gu, "gate_up");
  check_bf16(out, "out");
  TORCH_CHECK(gu.dim() == 2 && gu.stride(1) == 1 && out.is_contiguous(), "2-D row-major");
  const long T = gu.size(0);
  const int I = gu.size(1) / 2;
  TORCH_CHECK(out.size(0) == T && out.size(1) == I, "out shape");
  ok(dllm_silu_mul(gu.data_ptr(), out.data_ptr(), T, I, gu.stride(0), stream()), "silu_mul");
}

// token-embedding gather; ssq (optional, f32 [>= T]): each row's sum of squares
// sc_dst / sc_buf (optional, int32): a decode step's block-table updates (scatter_pairs layout),
// applied by one extra workgroup of the same launch.
void embed(torch::Tensor ids, torch::Tensor table, torch::Tensor out, int64_t lo, c10::optional<torch::Tensor> ssq,
           c10::optional<torch::Tensor> sc_dst, c10::optional<torch::Tensor> sc_buf) {
  TORCH_CHECK(ids.scalar_type() == torch::kInt && ids.is_contiguous() && ids.is_cuda(), "ids: contiguous int32");
  check_bf16(table, "table");
  check_bf16(out, "out");
  TORCH_CHECK(table.dim() == 2 && table.is_contiguous() && out.is_contiguous(), "table [rows, H] contiguous");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == ids.numel() && out.size(1) == table.size(1), "out [T, H]");
  float* sp = nullptr;
  if (ssq.has_value()) {
    check_f32(*ssq, "ssq");
    TORCH_CHECK(ssq->is_contiguous() && ssq->numel() >= ids.numel(), "ssq [>= T] contiguous");
    sp = ssq->data_ptr<float>();
  }
  int* dst = nullptr;
  const int* buf = nullptr;
  int cap = 0;
  if (sc_buf.has_value()) {
    TORCH_CHECK(sc_dst.has_value(), "embed: sc_buf needs sc_dst");
    for (auto* t : {&*sc_dst, &*sc_buf})
      TORCH_CHECK(t->scalar_type() == torch::kInt && t->is_contiguous() && t->is_cuda(), "embed: scatter operands int32");
    dst = sc_dst->data_ptr<int>();
    buf = sc_buf->data_ptr<int>();
    cap = (int)((sc_buf->numel() - 1) / 2);
  }
  ok(dllm_embed(ids.data_ptr<int>(), table.data_ptr(), out.data_ptr(), ids.numel(), table.size(1), lo,
                table.size(0), sp, dst, buf, cap, stream()),
     "embed");
}

void gelu(torch::Tensor x, torch::Tensor y) {
  check_bf16(x, "x");
  check_bf16(y, "y");
  TORCH_CHECK(x.is_contiguous() && y.is_contiguous() && x.numel() == y.numel(), "contiguous same-size");
  ok(dllm_gelu(x.data_ptr(), y.data_ptr(), x.numel(), stream()), "gelu");
}

void mean_pool_l2(torch::Tensor x, torch::Tensor lens, torch::Tensor out) {
  check_bf16(x, "x");
  check_i32(lens, "lens");
  check_f32(out, "out");
  TORCH_CHECK(x.dim() == 3 && x.is_contiguous(), "x [B, S, H]");
  const int B = x.size(0), S = x.size(1), H = x.size(2);
  TORCH_CHECK(lens.numel() == B && out.size(0) == B && out.size(1) == H, "shapes");
  ok(dllm_mean_pool_l2(x.data_ptr(), lens.data_ptr<int>(), out.data_ptr<float>(), B, S, H, stream()), "mean_pool_l2");
}

void moe_gate(torch::Tensor logits, int64_t k, torch::Tensor ids, torch::Tensor w) {
  check_f32(logits, "router_logits");
  check_i32(ids, "ids");
  check_f32(w, "weights");
  const int T = logits.size(0), E = logits.size(1);
  TORCH_CHECK(ids.numel() == (int64_t)T * k && w.numel() == (int64_t)T * k, "out shapes");
  ok(dllm_moe_gate(logits.data_ptr<float>(), T, E, k, ids.data_ptr<int>(), w.data_ptr<float>(), stream()), "moe_gate");
}

// fused router GEMV + top-k (batch-invariant): x [T, H] (row stride % 8), wg [E, H] -> ids/w [T, k]
void moe_router(torch::Tensor x, torch::Tensor wg, int64_t k, torch::Tensor ids, torch::Tensor w,
                c10::optional<torch::Tensor> logits) {
  check_bf16(x, "x");
  check_bf16(wg, "router weight");
  check_i32(ids, "ids");
  check_f32(w, "weights");
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && wg.dim() == 2 && wg.is_contiguous() && wg.size(1) == x.size(1),
              "x [T, H] row-major, wg [E, H] contiguous");
  const int T = x.size(0), E = wg.size(0), H = x.size(1);
  TORCH_CHECK(ids.numel() == (int64_t)T * k && w.numel() == (int64_t)T * k && ids.is_contiguous() && w.is_contiguous(),
              "out shapes");
  float* lp = nullptr;
  if (logits.has_value()) {
    check_f32(*logits, "logits");
    TORCH_CHECK(logits->is_contiguous() && logits->numel() == (int64_t)T * E, "logits [T, E]");
    lp = logits->data_ptr<float>();
  }
  ok(dllm_moe_router(x.data_ptr(), x.stride(0), wg.data_ptr(), T, E, H, k, ids.data_ptr<int>(), w.data_ptr<float>(),
                     lp, stream()),
     "moe_router");
}

// dst (int32, any shape, contiguous) flat[idx_i] = val_i for buf = [n, idx0, val0, ...]
// Device address of a pinned (hipHostMalloc'd) host tensor, for kernels that read / write it.
static void* mapped_ptr(const torch::Tensor& t, const char* what) {
  TORCH_CHECK(t.device().is_cpu() && t.is_pinned() && t.is_contiguous() && t.scalar_type() == torch::kInt,
              what, ": pinned contiguous int32 host tensor");
  void* dptr = nullptr;
  ok((int)hipHostGetDevicePointer(&dptr, t.data_ptr(), 0), what);
  return dptr;
}

// Decode-step inputs from the pinned staging buffer (device-mapped) into dec_dev, with the
// pipelined id gather (ids[i] = d_out[src[i]] where src[i] >= 0) and the attention work list.
void step_fetch(torch::Tensor dec_host, torch::Tensor dec_dev, int64_t ids_off, int64_t src_off, int64_t n_ids,
                torch::Tensor d_out, c10::optional<torch::Tensor> items_host, c10::optional<torch::Tensor> items_dev) {
  TORCH_CHECK(dec_dev.is_cuda() && dec_dev.scalar_type() == torch::kInt && dec_dev.is_contiguous() &&
                  dec_dev.numel() == dec_host.numel(), "step_fetch: dec_dev int32 like dec_host");
  TORCH_CHECK(d_out.is_cuda() && d_out.scalar_type() == torch::kInt && d_out.numel() > n_ids, "step_fetch: d_out");
  const int* ih = nullptr;
  int* idv = nullptr;
  int cap = 0;
  if (items_host.has_value()) {
    TORCH_CHECK(items_dev.has_value() && items_dev->is_cuda() && items_dev->scalar_type() == torch::kInt &&
                    items_dev->numel() >= items_host->numel(), "step_fetch: items_dev");
    ih = (const int*)mapped_ptr(*items_host, "step_fetch items_host");
    idv = items_dev->data_ptr<int>();
    cap = (int)items_host->numel();
  }
  ok(dllm_step_fetch((const int*)mapped_ptr(dec_host, "step_fetch dec_host"), dec_dev.data_ptr<int>(),
                     (int)dec_host.numel(), (int)ids_off, (int)src_off, (int)n_ids, d_out.data_ptr<int>(), ih, idv, cap,
                     stream()),
     "step_fetch");
}

// out_host[0:n] <- d_out[0:n] by a kernel (last node of a decode-step graph).
void step_store(torch::Tensor d_out, torch::Tensor out_host, int64_t n) {
  TORCH_CHECK(d_out.is_cuda() && d_out.scalar_type() == torch::kInt && d_out.numel() >= n && out_host.numel() >= n,
              "step_store: shapes");
  ok(dllm_step_store(d_out.data_ptr<int>(), (int*)mapped_ptr(out_host, "step_store out_host"), (int)n, stream()),
     "step_store");
}

void scatter_pairs(torch::Tensor dst, torch::Tensor buf) {
  check_i32(dst, "dst");
  check_i32(buf, "buf");
  TORCH_CHECK(buf.numel() >= 1 && buf.numel() % 2 == 1, "buf = [n, (idx, val)*]");
  ok(dllm_scatter_pairs(dst.data_ptr<int>(), buf.data_ptr<int>(), (int)(buf.numel() - 1) / 2, stream()),
     "scatter_pairs");
}

void argmax(torch::Tensor logits, torch::Tensor out) {
  check_dev(logits, "logits");
  check_i32(out, "out");
  TORCH_CHECK(logits.dim() == 2 && logits.stride(1) == 1, "logits [B, V] row-major");
  const bool bf = logits.scalar_type() == torch::kBFloat16;
  TORCH_CHECK(bf || logits.scalar_type() == torch::kFloat32, "logits bf16 or f32");
  TORCH_CHECK(logits.stride(0) % (bf ? 8 : 4) == 0, "row stride must keep 16-B alignment");
  TORCH_CHECK(out.numel() == logits.size(0), "out len");
  ok(dllm_argmax(logits.data_ptr(), logits.stride(0), logits.size(0), logits.size(1), bf ? 1 : 0,
                 out.data_ptr<int>(), stream()),
     "argmax");
}

void sample_topp(torch::Tensor vals, torch::Tensor idx, torch::Tensor temp, torch::Tensor top_p, torch::Tensor u,
                 torch::Tensor out) {
  check_f32(vals, "vals");
  check_dev(idx, "idx");
  TORCH_CHECK(idx.scalar_type() == torch::kInt64 && idx.is_contiguous(), "idx int64");
  check_f32(temp, "temperature");
  check_f32(top_p, "top_p");
  check_f32(u, "uniform");
  check_i32(out, "out");
  const int B = vals.size(0), K = vals.size(1);
  TORCH_CHECK(idx.size(0) == B && idx.size(1) == K && temp.numel() == B && top_p.numel() == B && u.numel() == B &&
                  out.numel() == B,
              "shapes");
  ok(dllm_sample_topp(vals.data_ptr<float>(), (const long*)idx.data_ptr<int64_t>(), B, K, temp.data_ptr<float>(),
                      top_p.data_ptr<float>(), u.data_ptr<float>(), out.data_ptr<int>(), stream()),
     "sample_topp");
}

// Fused per-row sampler: temp <= 0 -> arg-max; else exact top-k (k <= 256; 0 -> 256), temperature,
// top-p and an inverse-CDF draw with u = hash(seed, row).  seed: int32 device scalar.
void sample_rows(torch::Tensor logits, torch::Tensor temp, torch::Tensor top_p, torch::Tensor top_k,
                 torch::Tensor seed, torch::Tensor out) {
  check_bf16(logits, "logits");
  TORCH_CHECK(logits.dim() == 2 && logits.stride(1) == 1 && logits.stride(0) % 8 == 0,
              "logits [B, V] row-major, 16-B aligned rows");
  check_f32(temp, "temperature");
  check_f32(top_p, "top_p");
  check_i32(top_k, "top_k");
  check_i32(seed, "seed");
  check_i32(out, "out");
  const int B = logits.size(0);
  TORCH_CHECK(temp.numel() >= B && top_p.numel() >= B && top_k.numel() >= B && out.numel() >= B &&
                  seed.numel() >= 1,
              "per-row parameter lengths");
  ok(dllm_sample_rows(logits.data_ptr(), logits.stride(0), B, logits.size(1), temp.data_ptr<float>(),
                      top_p.data_ptr<float>(), top_k.data_ptr<int>(), (const unsigned*)seed.data_ptr<int>(),
                      out.data_ptr<int>(), stream()),
     "sample_rows");
}

// Split-vocab sampler for small batches: grid (P shards, B rows), same tokens as sample_rows.
// part: f32/int32 workspace >= B * P * KMAX * 2 elements; counters: int32 >= B, zero (re-armed).
int64_t sample_split_maxp() { return dllm_sample_split_maxp(); }
int64_t sample_split_kmax() { return dllm_sample_split_kmax(); }
void sample_split(torch::Tensor logits, torch::Tensor temp, torch::Tensor top_p, torch::Tensor top_k,
                  torch::Tensor seed, torch::Tensor part, torch::Tensor counters, torch::Tensor out, int64_t P) {
  check_bf16(logits, "logits");
  TORCH_CHECK(logits.dim() == 2 && logits.stride(1) == 1 && logits.stride(0) % 8 == 0,
              "logits [B, V] row-major, 16-B aligned rows");
  check_f32(temp, "temperature");
  check_f32(top_p, "top_p");
  check_i32(top_k, "top_k");
  check_i32(seed, "seed");
  check_i32(out, "out");
  check_i32(counters, "counters");
  const int B = logits.size(0);
  TORCH_CHECK(temp.numel() >= B && top_p.numel() >= B && top_k.numel() >= B && out.numel() >= B &&
                  seed.numel() >= 1 && counters.numel() >= B,
              "per-row parameter lengths");
  TORCH_CHECK(part.is_cuda() && part.is_contiguous() && part.element_size() == 4, "part: 4-byte workspace");
  TORCH_CHECK(P >= 1 && P <= dllm_sample_split_maxp(), "shards P");
  ok(dllm_sample_split(logits.data_ptr(), logits.stride(0), B, logits.size(1), (int)P, temp.data_ptr<float>(),
                       top_p.data_ptr<float>(), top_k.data_ptr<int>(), (const unsigned*)seed.data_ptr<int>(),
                       part.data_ptr(), (long)part.numel() * 4, counters.data_ptr<int>(), out.data_ptr<int>(), stream()),
     "sample_split");
}

// vocab-parallel sampler (csrc/kernels/sampling.hip): a shard's ranked top-KC candidates as int32
// pairs (value f32 bits, global id) [S, KC, 2], and the merge + draw over all-gathered [tp, S, KC, 2]
int64_t tp_cands_k() { return dllm_tp_cands_k(); }
void tp_cands(torch::Tensor logits, int64_t start, torch::Tensor cand) {
  check_bf16(logits, "logits");
  check_i32(cand, "cand");
  TORCH_CHECK(logits.dim() == 2 && logits.stride(1) == 1 && logits.stride(0) % 8 == 0,
              "logits [S, V] row-major, 16-B aligned rows");
  const int S = logits.size(0), KC = dllm_tp_cands_k();
  TORCH_CHECK(cand.is_contiguous() && cand.numel() == (int64_t)S * KC * 2, "cand [S, KC, 2] int32");
  ok(dllm_tp_cands(logits.data_ptr(), logits.stride(0), S, logits.size(1), (int)start, cand.data_ptr(), stream()),
     "tp_cands");
}
void tp_sample(torch::Tensor cands, torch::Tensor temp, torch::Tensor top_p, torch::Tensor top_k, torch::Tensor seed,
               torch::Tensor out) {
  check_i32(cands, "cands");
  check_f32(temp, "temperature");
  check_f32(top_p, "top_p");
  check_i32(top_k, "top_k");
  check_i32(seed, "seed");
  check_i32(out, "out");
  const int KC = dllm_tp_cands_k();
  TORCH_CHECK(cands.is_contiguous() && cands.dim() == 4 && cands.size(2) == KC && cands.size(3) == 2 &&
                  cands.size(0) >= 1 && cands.size(0) <= 8,
              "cands [tp <= 8, S, KC, 2] int32");
  const int tp = cands.size(0), S = cands.size(1);
  TORCH_CHECK(temp.numel() >= S && top_p.numel() >= S && top_k.numel() >= S && out.numel() >= S && seed.numel() >= 1,
              "per-row parameter lengths");
  ok(dllm_tp_sample(cands.data_ptr(), S, tp, temp.data_ptr<float>(), top_p.data_ptr<float>(), top_k.data_ptr<int>(),
                    (const unsigned*)seed.data_ptr<int>(), out.data_ptr<int>(), stream()),
     "tp_sample");
}

void cosine_scores(torch::Tensor q, torch::Tensor c, torch::Tensor s) {
  check_f32(q, "q");
  check_f32(c, "c");
  check_f32(s, "s");
  TORCH_CHECK(q.dim() == 2 && c.dim() == 2 && q.size(1) == c.size(1), "q [B,d], c [N,d]");
  TORCH_CHECK(s.size(0) == q.size(0) && s.size(1) == c.size(0), "s [B,N]");
  ok(dllm_cosine_scores(q.data_ptr<float>(), c.data_ptr<float>(), s.data_ptr<float>(), q.size(0), c.size(0),
                        q.size(1), stream()),
     "cosine_scores");
}

// one launch for up to 128 semantic-cache lookups (csrc/kernels/cosine.hip cache_scan_kernel):
// qptrs = device addresses of the queries' f32 [d] vectors (kept alive by the caller), qcids = their
// context ids; best[i] <- packed (orderable sim << 32 | ~row) key, 0 = no row >= thr
void cache_scan(std::vector<int64_t> qptrs, std::vector<int64_t> qcids, torch::Tensor table, torch::Tensor ctx,
                int64_t n_rows, double thr, torch::Tensor best) {
  check_f32(table, "table");
  check_i32(ctx, "ctx");
  check_dev(best, "best");
  TORCH_CHECK(table.dim() == 2 && table.size(1) % 4 == 0 && table.size(1) <= 1024, "table [N, d], d % 4 == 0, d <= 1024");
  TORCH_CHECK(n_rows >= 0 && n_rows <= table.size(0) && ctx.numel() >= n_rows, "rows within table/ctx");
  TORCH_CHECK(n_rows < 0xffffffffLL, "row index must fit the 32-bit key");
  const int nq = (int)qptrs.size();
  TORCH_CHECK(nq >= 1 && nq <= 128 && (int)qcids.size() == nq, "1..128 queries with one context id each");
  TORCH_CHECK(best.scalar_type() == torch::kInt64 && best.is_contiguous() && best.numel() >= nq, "best: int64[nq]");
  std::vector<unsigned long long> qp(nq);
  std::vector<int> qc(nq);
  for (int i = 0; i < nq; ++i) {
    TORCH_CHECK(qptrs[i] != 0 && (qptrs[i] & 15) == 0, "query vectors must be 16-B aligned device memory");
    qp[i] = (unsigned long long)qptrs[i];
    qc[i] = (int)qcids[i];
  }
  ok(dllm_cache_scan(qp.data(), qc.data(), nq, table.data_ptr<float>(), ctx.data_ptr<int>(), (long)n_rows,
                     (int)table.size(1), (float)thr, (unsigned long long*)best.data_ptr<int64_t>(), stream()),
     "cache_scan");
}

// deferred routing-cache table writes, <= 64 per launch: row slots[i] <- f32 [d] at srcs[i] (0: keep),
// ctx[slots[i]] <- cids[i]
void cache_write(std::vector<int64_t> srcs, std::vector<int64_t> slots, std::vector<int64_t> cids, torch::Tensor table,
                 torch::Tensor ctx) {
  check_f32(table, "table");
  check_i32(ctx, "ctx");
  const int n = (int)srcs.size();
  TORCH_CHECK(n <= 64 && (int)slots.size() == n && (int)cids.size() == n, "<= 64 writes");
  std::vector<unsigned long long> sp(n);
  std::vector<long long> sl(n);
  std::vector<int> ci(n);
  for (int i = 0; i < n; ++i) {
    TORCH_CHECK(slots[i] >= 0 && slots[i] < table.size(0) && slots[i] < ctx.numel(), "slot out of range");
    TORCH_CHECK((srcs[i] & 15) == 0, "source vectors must be 16-B aligned");
    sp[i] = (unsigned long long)srcs[i];
    sl[i] = slots[i];
    ci[i] = (int)cids[i];
  }
  ok(dllm_cache_write(sp.data(), sl.data(), ci.data(), n, table.data_ptr<float>(), ctx.data_ptr<int>(),
                      (int)table.size(1), stream()),
     "cache_write");
}
// y[M, N] = x[M, K] . w[N, K]^T   (swiglu: x is [M, 2K] gate|up, silu(gate)*up computed on load)
void skinny_gemm(torch::Tensor x, torch::Tensor w, torch::Tensor y, int64_t ntw, int64_t splits, bool swiglu,
                 torch::Tensor part, torch::Tensor counters) {
  check_bf16(x, "x");
  check_bf16(w, "w");
  check_bf16(y, "y");
  check_f32(part, "part");
  check_i32(counters, "counters");
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && w.dim() == 2 && w.is_contiguous() && y.dim() == 2 &&
                  y.stride(1) == 1,
              "2-D row-major operands");
  const int M = x.size(0), N = w.size(0), K = w.size(1);
  TORCH_CHECK(x.size(1) == (swiglu ? 2 * K : K), "x inner dim");
  TORCH_CHECK(y.size(0) == M && y.size(1) == N, "y shape");
  TORCH_CHECK(M >= 1 && M <= 128 && K % 32 == 0, "M in [1,128], K % 32 == 0");
  TORCH_CHECK(ntw == 1 || ntw == 2 || ntw == 4, "ntw in {1,2,4}");
  // slab rows = the kernel's row-tile height (MT x 16, MT in {1, 2, 4, 8}), not ceil(M / 16) x 16
  const int nc = 16 * ntw, tiles = (N + nc - 1) / nc,
            mp = 16 * (M <= 16 ? 1 : M <= 32 ? 2 : M <= 64 ? 4 : 8);
  if (splits > 1) {
    TORCH_CHECK(part.numel() >= (int64_t)splits * tiles * nc * mp, "split-K workspace too small");
    TORCH_CHECK(counters.numel() >= tiles, "counter buffer too small");
  }
  ok(dllm_skinny_gemm(x.data_ptr(), x.stride(0), w.data_ptr(), y.data_ptr(), y.stride(0), M, N, K, ntw, splits, swiglu ? 1 : 0,
        part.data_ptr<float>(), counters.data_ptr<int>(), stream()),
     "skinny_gemm");
}
// Small-batch (M <= 16) MFMA GEMM with a fused decoder epilogue (csrc/kernels/skinny_gemm.hip
// skinny_epi_kernel): epi 0 plain (y), 1 residual add (res in place + per-tile row sums -> ssq_out),
// 2 QKV (RoPE, q_out, paged K / V^T), 3 SwiGLU (y = act [M, N/2]).  w: [N, K] or the panel copy
// [K/64, N, 64].  Returns the row-sum slots written (RESADD) or 0.
int64_t skinny_epi(torch::Tensor x, torch::Tensor w, c10::optional<torch::Tensor> y, int64_t ntw, int64_t splits,
                   int64_t epi, torch::Tensor part, torch::Tensor counters, c10::optional<torch::Tensor> res,
                   c10::optional<torch::Tensor> ssq_out, c10::optional<torch::Tensor> ssq_in, int64_t ssq_n,
                   double scale, double eps, c10::optional<torch::Tensor> pos, c10::optional<torch::Tensor> cos_sin,
                   c10::optional<torch::Tensor> slots, c10::optional<torch::Tensor> q_out,
                   c10::optional<torch::Tensor> kc, c10::optional<torch::Tensor> vc, int64_t nq, int64_t nkv, int64_t d) {
  check_bf16(x, "x");
  check_bf16(w, "w");
  check_f32(part, "part");
  check_i32(counters, "counters");
  const bool panel = w.dim() == 3;
  TORCH_CHECK(((w.dim() == 2) || (panel && w.size(2) == 64)) && w.is_contiguous(), "w: [N, K] or [K / 64, N, 64]");
  const int M = x.size(0), N = panel ? w.size(1) : w.size(0), K = panel ? w.size(0) * 64 : w.size(1);
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && x.stride(0) % 8 == 0 && x.size(1) == K, "x [M, K], 16-B rows");
  TORCH_CHECK(M >= 1 && M <= 16 && K % 64 == 0, "M in [1, 16], K % 64 == 0");
  TORCH_CHECK(ntw == 1 || ntw == 2, "ntw 1 or 2");
  TORCH_CHECK(epi >= 0 && epi <= 3 && (epi < 2 || ntw == 2), "epi 0-3; QKV / SwiGLU need ntw 2");
  const int nc = 16 * (int)ntw, tiles = (N + nc - 1) / nc;
  int kchunk = (K + (int)splits - 1) / (int)splits;
  kchunk = (kchunk + 31) & ~31;
  const int S = (K + kchunk - 1) / kchunk;
  if (S > 1) {
    TORCH_CHECK(part.numel() >= (int64_t)S * tiles * nc * 16, "split-K workspace too small");
    TORCH_CHECK(counters.numel() >= tiles, "counter buffer too small");
  }
  void* yp = nullptr;
  long ldy = 0;
  if (epi == 0 || epi == 3) {
    TORCH_CHECK(y.has_value(), "y required");
    check_bf16(*y, "y");
    TORCH_CHECK(y->dim() == 2 && y->stride(1) == 1 && y->size(0) == M && y->size(1) == (epi == 3 ? N / 2 : N), "y shape");
    yp = y->data_ptr();
    ldy = y->stride(0);
  }
  void* rp = nullptr;
  long ldr = 0;
  float* so = nullptr;
  long so_ld = 0;
  if (epi == 1) {
    TORCH_CHECK(res.has_value() && ssq_out.has_value(), "residual epilogue: res and ssq_out");
    check_bf16(*res, "res");
    check_f32(*ssq_out, "ssq_out");
    TORCH_CHECK(res->dim() == 2 && res->stride(1) == 1 && res->size(0) == M && res->size(1) == N, "res [M, N]");
    TORCH_CHECK(ssq_out->dim() == 2 && ssq_out->size(0) >= tiles && ssq_out->size(1) >= M, "ssq_out [>= tiles, >= M]");
    rp = res->data_ptr();
    ldr = res->stride(0);
    so = ssq_out->data_ptr<float>();
    so_ld = ssq_out->size(1);
  }
  const float* si = nullptr;
  long si_ld = 0;
  if (epi >= 2) {
    TORCH_CHECK(ssq_in.has_value(), "row-scaled epilogue: ssq_in");
    check_f32(*ssq_in, "ssq_in");
    TORCH_CHECK(ssq_in->dim() == 2 && ssq_in->size(1) >= M && ssq_n >= 1 && ssq_n <= ssq_in->size(0), "ssq_in [slots, >= M]");
    si = ssq_in->data_ptr<float>();
    si_ld = ssq_in->size(1);
  }
  const int *pp = nullptr, *sl = nullptr;
  const float* cs = nullptr;
  void *qo = nullptr, *kp = nullptr, *vp = nullptr;
  if (epi == 2) {
    TORCH_CHECK(pos.has_value() && cos_sin.has_value() && slots.has_value() && q_out.has_value() && kc.has_value() &&
                    vc.has_value(), "qkv epilogue operands");
    check_i32(*pos, "positions");
    check_i32(*slots, "slots");
    check_f32(*cos_sin, "cos_sin");
    check_bf16(*q_out, "q_out");
    check_bf16(*kc, "k_cache");
    check_bf16(*vc, "v_cache");
    TORCH_CHECK(d % 32 == 0 && N == (nq + 2 * nkv) * d, "qkv: N == (nq + 2 nkv) d, d % 32 == 0");
    TORCH_CHECK(pos->numel() >= M && slots->numel() >= M && cos_sin->dim() == 2 && cos_sin->size(1) == d,
                "positions / slots / cos_sin");
    TORCH_CHECK(q_out->is_contiguous() && q_out->numel() >= (int64_t)M * nq * d, "q_out [M, nq, d]");
    TORCH_CHECK(kc->is_contiguous() && vc->is_contiguous() && kc->dim() == 4 && kc->size(1) == nkv &&
                    kc->size(2) == 16 && kc->size(3) == d && vc->size(1) == nkv && vc->size(2) == d && vc->size(3) == 16,
                "cache layout: K [blocks, nkv, 16, d], V [blocks, nkv, d, 16]");
    pp = pos->data_ptr<int>();
    sl = slots->data_ptr<int>();
    cs = cos_sin->data_ptr<float>();
    qo = q_out->data_ptr();
    kp = kc->data_ptr();
    vp = vc->data_ptr();
  }
  ok(dllm_skinny_epi(x.data_ptr(), x.stride(0), w.data_ptr(), panel ? 1 : 0, yp, ldy, M, N, K, (int)ntw, (int)splits,
                     (int)epi, part.data_ptr<float>(), counters.data_ptr<int>(), rp, ldr, so, so_ld, si, (int)ssq_n, si_ld,
                     (float)scale, (float)eps, pp, cs, sl, qo, kp, vp, (int)nq, (int)nkv, (int)d, stream()),
     "skinny_epi");
  return epi == 1 ? tiles : 0;
}

// Small-batch GEMV (M in {1, 2, 4, 8}; csrc/kernels/gemv.hip): y = x . w^T (x = silu(g)*u if swiglu).
void gemv(torch::Tensor x, torch::Tensor w, torch::Tensor y, int64_t R, bool swiglu) {
  check_bf16(x, "x");
  check_bf16(w, "w");
  check_bf16(y, "y");
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && w.dim() == 2 && w.is_contiguous() && y.dim() == 2 &&
                  y.stride(1) == 1,
              "2-D row-major operands");
  const int M = x.size(0), N = w.size(0), K = w.size(1);
  TORCH_CHECK(M == 1 || M == 2 || M == 4 || M == 8, "gemv: M in {1, 2, 4, 8}");
  TORCH_CHECK(x.size(1) == (swiglu ? 2 * K : K) && K % 8 == 0, "gemv: x inner dim, K % 8 == 0");
  TORCH_CHECK((int64_t)M * K * 2 <= 64 * 1024, "gemv: M x K bf16 must fit the 64 KB LDS stage");
  TORCH_CHECK(x.stride(0) % 8 == 0 && y.stride(0) >= N && y.size(0) == M && y.size(1) == N, "gemv: y shape / alignment");
  TORCH_CHECK(R == 1 || R == 2 || R == 4, "gemv: R in {1, 2, 4}");
  ok(dllm_gemv(x.data_ptr(), x.stride(0), w.data_ptr(), y.data_ptr(), y.stride(0), M, N, K, (int)R, swiglu ? 1 : 0,
               nullptr, nullptr, nullptr, 0.f, stream()),
     "gemv");
}

// RMSNorm-fused GEMV: r = x + res_in -> res_out (bf16), y = rmsnorm(r) * norm_w . w^T
void gemv_norm(torch::Tensor x, torch::Tensor res_in, torch::Tensor res_out, torch::Tensor norm_w, double eps,
               torch::Tensor w, torch::Tensor y, int64_t R) {
  for (auto* t : {&x, &res_in, &res_out, &norm_w, &w, &y}) check_bf16(*t, "gemv_norm operand");
  const int M = x.size(0), N = w.size(0), K = w.size(1);
  TORCH_CHECK(M == 1 || M == 2 || M == 4 || M == 8, "gemv_norm: M in {1, 2, 4, 8}");
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous() && x.size(1) == K && K % 8 == 0, "gemv_norm: x [M, K]");
  TORCH_CHECK(res_in.is_contiguous() && res_out.is_contiguous() && res_in.sizes() == x.sizes() &&
                  res_out.sizes() == x.sizes() && res_in.data_ptr() != res_out.data_ptr(),
              "gemv_norm: res_in/res_out [M, K], distinct");
  TORCH_CHECK(norm_w.numel() == K && w.is_contiguous() && y.dim() == 2 && y.size(0) == M && y.size(1) == N &&
                  y.stride(1) == 1,
              "gemv_norm: shapes");
  TORCH_CHECK((int64_t)M * K * 2 <= 64 * 1024 && (R == 1 || R == 2 || R == 4), "gemv_norm: LDS stage / R");
  ok(dllm_gemv(x.data_ptr(), K, w.data_ptr(), y.data_ptr(), y.stride(0), M, N, K, (int)R, 0, res_in.data_ptr(),
               res_out.data_ptr(), norm_w.data_ptr(), (float)eps, stream()),
     "gemv_norm");
}

// GEMV with a fused decoder-layer epilogue (csrc/kernels/gemv.hip EPI; batch <= 8):
//   gemv_resadd: r += x . w^T in place, partial row sums of r^2 -> ssq_out [slots, >= M]; returns slots
//   gemv_qkv   : q [M, nq, d] of rope(rinv * x . w^T), K / V^T into the paged caches
//   gemv_swiglu: act [M, N/2] = silu(g) * u of rinv * x . w^T (interleaved gate/up rows)
static void gemv_epi_checks(const torch::Tensor& x, const torch::Tensor& w, int64_t R, const char* what) {
  check_bf16(x, what);
  check_bf16(w, what);
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && w.dim() == 2 && w.is_contiguous(), what, ": 2-D row-major operands");
  const int64_t M = x.size(0), K = w.size(1);
  TORCH_CHECK(M == 1 || M == 2 || M == 4 || M == 8, what, ": M in {1, 2, 4, 8}");
  TORCH_CHECK(x.size(1) == K && K % 8 == 0 && x.stride(0) % 8 == 0, what, ": x [M, K], K % 8 == 0, aligned rows");
  TORCH_CHECK(M * K * 2 <= 64 * 1024 && (R == 1 || R == 2 || R == 4), what, ": LDS stage / R");
}

static void check_ssq_in(const torch::Tensor& ssq, int64_t ssq_n, int64_t M) {
  check_f32(ssq, "ssq");
  TORCH_CHECK(ssq.dim() == 2 && ssq.stride(1) == 1 && ssq.size(1) >= M && ssq_n >= 1 && ssq_n <= ssq.size(0),
              "ssq [slots, >= M]");
}

int64_t gemv_slots(int64_t M, int64_t N, int64_t R) { return dllm_gemv_slots((int)M, (int)N, (int)R); }
void gemv_set_grid(int64_t min_blocks, int64_t xdiv, int64_t n_min) {
  dllm_gemv_set_grid((int)min_blocks, (int)xdiv, (int)n_min);
}

int64_t gemv_resadd(torch::Tensor x, torch::Tensor w, torch::Tensor r, torch::Tensor ssq_out, int64_t R) {
  gemv_epi_checks(x, w, R, "gemv_resadd");
  check_bf16(r, "r");
  check_f32(ssq_out, "ssq_out");
  const int M = x.size(0), N = w.size(0), K = w.size(1);
  const int slots = dllm_gemv_slots(M, N, (int)R);
  TORCH_CHECK(r.dim() == 2 && r.stride(1) == 1 && r.size(0) == M && r.size(1) == N && r.stride(0) % 8 == 0, "r [M, N]");
  TORCH_CHECK(ssq_out.dim() == 2 && ssq_out.stride(1) == 1 && ssq_out.size(0) >= slots && ssq_out.size(1) >= M,
              "ssq_out [>= slots, >= M]");
  ok(dllm_gemv_epi(x.data_ptr(), x.stride(0), w.data_ptr(), nullptr, 0, M, N, K, (int)R, 1, r.data_ptr(), r.stride(0),
                   ssq_out.data_ptr<float>(), ssq_out.stride(0), nullptr, 0, 0, 0.f, 0.f, nullptr, nullptr, nullptr,
                   nullptr, nullptr, nullptr, 0, 0, 0, stream()),
     "gemv_resadd");
  return slots;
}

void gemv_qkv(torch::Tensor x, torch::Tensor w, torch::Tensor ssq, int64_t ssq_n, double scale, double eps,
              torch::Tensor pos, torch::Tensor cos_sin, torch::Tensor slots, torch::Tensor q_out, torch::Tensor kc,
              torch::Tensor vc, int64_t nq, int64_t nkv, int64_t d, int64_t R) {
  gemv_epi_checks(x, w, R, "gemv_qkv");
  const int M = x.size(0), N = w.size(0), K = w.size(1);
  check_ssq_in(ssq, ssq_n, M);
  check_i32(pos, "positions");
  check_i32(slots, "slots");
  check_f32(cos_sin, "cos_sin");
  for (auto* t : {&q_out, &kc, &vc}) check_bf16(*t, "qkv outputs");
  TORCH_CHECK(N == (nq + 2 * nkv) * d && d % 32 == 0, "gemv_qkv: w rows (nq + 2 nkv) d, d % 32 == 0");
  TORCH_CHECK(pos.numel() >= M && slots.numel() >= M && cos_sin.dim() == 2 && cos_sin.size(1) == d &&
                  cos_sin.is_contiguous(),
              "positions/slots/cos_sin");
  TORCH_CHECK(q_out.is_contiguous() && q_out.numel() >= (int64_t)M * nq * d, "q_out");
  TORCH_CHECK(kc.is_contiguous() && vc.is_contiguous() && kc.size(1) == nkv && kc.size(2) == 16 && kc.size(3) == d &&
                  vc.size(2) == d && vc.size(3) == 16,
              "cache layout");
  ok(dllm_gemv_epi(x.data_ptr(), x.stride(0), w.data_ptr(), nullptr, 0, M, N, K, (int)R, 2, nullptr, 0, nullptr, 0,
                   ssq.data_ptr<float>(), (int)ssq_n, ssq.stride(0), (float)scale, (float)eps, pos.data_ptr<int>(),
                   cos_sin.data_ptr<float>(), slots.data_ptr<int>(), q_out.data_ptr(), kc.data_ptr(), vc.data_ptr(),
                   (int)nq, (int)nkv, (int)d, stream()),
     "gemv_qkv");
}

void gemv_swiglu(torch::Tensor x, torch::Tensor w, torch::Tensor ssq, int64_t ssq_n, double scale, double eps,
                 torch::Tensor act, int64_t R) {
  gemv_epi_checks(x, w, R, "gemv_swiglu");
  const int M = x.size(0), N = w.size(0), K = w.size(1);
  check_ssq_in(ssq, ssq_n, M);
  check_bf16(act, "act");
  TORCH_CHECK(N % 32 == 0 && act.dim() == 2 && act.stride(1) == 1 && act.size(0) == M && act.size(1) == N / 2,
              "gemv_swiglu: act [M, N/2], N % 32 == 0");
  ok(dllm_gemv_epi(x.data_ptr(), x.stride(0), w.data_ptr(), act.data_ptr(), act.stride(0), M, N, K, (int)R, 3, nullptr,
                   0, nullptr, 0, ssq.data_ptr<float>(), (int)ssq_n, ssq.stride(0), (float)scale, (float)eps, nullptr,
                   nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 0, stream()),
     "gemv_swiglu");
}

// Mixtral-style MoE FFN: x [T, H] bf16, ids [T, k] int32, wts [T, k] f32, w13 [E, 2I, H], w2 [E, H, I]
// -> out [T, H] bf16 (partial sum over this rank's I shard under TP).  Workspace from torch's
// caching allocator, so the call is graph-capturable.
// grouped-tgemm MoE (csrc/kernels/moe.hip dllm_moe_ffn_tg): w13 interleaved per 16-row group
void moe_ffn_tg(torch::Tensor x, torch::Tensor ids, torch::Tensor wts, torch::Tensor w13, torch::Tensor w2,
                torch::Tensor out, std::vector<int64_t> plan) {
  check_bf16(x, "x");
  check_i32(ids, "ids");
  check_f32(wts, "wts");
  check_bf16(w13, "w13");
  check_bf16(w2, "w2");
  check_bf16(out, "out");
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && x.stride(0) % 8 == 0 && out.is_contiguous(), "x rows 16-B aligned");
  TORCH_CHECK(w13.dim() == 3 && w2.dim() == 3 && w13.is_contiguous() && w2.is_contiguous(), "w13/w2 [E, N, K]");
  const int64_t T = x.size(0), H = x.size(1), E = w13.size(0), I = w13.size(1) / 2;
  TORCH_CHECK(w13.size(2) == H && w2.size(0) == E && w2.size(1) == H && w2.size(2) == I, "expert weight shapes");
  TORCH_CHECK(H % 64 == 0 && I % 64 == 0 && E <= 64, "H, I multiples of 64; E <= 64");
  TORCH_CHECK(ids.dim() == 2 && ids.size(0) == T && wts.sizes() == ids.sizes() && ids.is_contiguous() &&
                  wts.is_contiguous(), "ids/wts [T, k]");
  TORCH_CHECK(out.size(0) == T && out.size(1) == H, "out shape");
  TORCH_CHECK(plan.size() == 9, "plan: bm, bn13, stages13, ks13, nw13, bn2, stages2, ks2, nw2");
  const int bm = (int)plan[0];
  for (int g = 0; g < 2; ++g) {
    const int bn = (int)plan[1 + 4 * g], st = (int)plan[2 + 4 * g], ks = (int)plan[3 + 4 * g], nw = (int)plan[4 + 4 * g];
    TORCH_CHECK((ks == 1 || ks == 2) && (nw == 4 || (nw == 8 && bn >= 128)) &&
                    (st == 2 || st == 3 || ((st == 4 || st == 6) && ks == 1 && bm <= 128)) &&
                    (bm == 64 || bm == 128 || ((bm == 192 || bm == 256) && nw == 8)) &&
                    (bn == 64 || bn == 128 || (bn == 256 && bm == 256)) && st * ks * (bm + bn) * 128 <= 150 * 1024,
                "moe plan tile / ring size");
    TORCH_CHECK((g == 0 ? H : I) % (64 * ks) == 0, "K % (64 ks)");
  }
  const int k = ids.size(1);
  auto iopt = ids.options();
  const int P = (int)(T * k), mt = dllm_moe_max_tiles_bm(P, (int)E, bm);
  auto perm = torch::empty({std::max(P, 1)}, iopt);
  auto inv = torch::empty({std::max(P, 1)}, iopt);
  auto tiles = torch::empty({4 * mt + 1}, iopt);
  auto act = torch::empty({std::max(P, 1), I}, x.options());
  auto y = torch::empty({std::max(P, 1), H}, x.options());
  int pl[9];
  for (int i = 0; i < 9; ++i) pl[i] = (int)plan[i];
  ok(dllm_moe_ffn_tg(x.data_ptr(), x.stride(0), T, (int)H, ids.data_ptr<int>(), wts.data_ptr<float>(), k, (int)E,
                     w13.data_ptr(), w2.data_ptr(), (int)I, perm.data_ptr<int>(), inv.data_ptr<int>(),
                     tiles.data_ptr<int>(), act.data_ptr(), y.data_ptr(), out.data_ptr(), pl, stream()),
     "moe_ffn_tg");
}

// act_mode 0: SwiGLU experts (w13 [E, 2I, H]); 1: squared-ReLU experts without a gate (w13 [E, I, H])
void moe_ffn(torch::Tensor x, torch::Tensor ids, torch::Tensor wts, torch::Tensor w13, torch::Tensor w2,
             torch::Tensor out, int64_t act_mode) {
  check_bf16(x, "x");
  check_i32(ids, "ids");
  check_f32(wts, "wts");
  check_bf16(w13, "w13");
  check_bf16(w2, "w2");
  check_bf16(out, "out");
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && out.is_contiguous(), "x 2-D row-major, out contiguous");
  TORCH_CHECK(w13.dim() == 3 && w2.dim() == 3 && w13.is_contiguous() && w2.is_contiguous(), "w13/w2 [E, N, K]");
  TORCH_CHECK(act_mode == 0 || act_mode == 1, "act_mode 0 or 1");
  const int64_t T = x.size(0), H = x.size(1), E = w13.size(0), I = w13.size(1) / (act_mode ? 1 : 2);
  TORCH_CHECK(w13.size(2) == H && w2.size(0) == E && w2.size(1) == H && w2.size(2) == I, "expert weight shapes");
  TORCH_CHECK(ids.dim() == 2 && ids.size(0) == T && wts.sizes() == ids.sizes(), "ids/wts [T, k]");
  TORCH_CHECK(out.size(0) == T && out.size(1) == H, "out shape");
  TORCH_CHECK(E <= 64 && H % 32 == 0 && I % 32 == 0 && x.stride(0) % 8 == 0, "E <= 64, H and I multiples of 32");
  const int k = ids.size(1);
  auto iopt = ids.options();
  const int P = (int)(T * k), mt = dllm_moe_max_tiles(P, (int)E);
  auto perm = torch::empty({std::max(P, 1)}, iopt);
  auto tiles = torch::empty({4 * mt}, iopt);
  auto act = torch::empty({std::max(P, 1), I}, x.options());
  auto y = torch::empty({std::max(P, 1), H}, wts.options());
  ok(dllm_moe_ffn(x.data_ptr(), x.stride(0), T, (int)H, ids.data_ptr<int>(), wts.data_ptr<float>(), k, (int)E,
                  w13.data_ptr(), w2.data_ptr(), (int)I, perm.data_ptr<int>(), tiles.data_ptr<int>(), act.data_ptr(),
                  y.data_ptr<float>(), out.data_ptr(), (int)act_mode, stream()),
     "moe_ffn");
}

// ---- one-shot all-reduce over IPC-mapped peer buffers (csrc/kernels/custom_ar.hip)
int64_t car_alloc(int64_t data_bytes) {
  void* p = nullptr;
  ok(dllm_car_alloc(data_bytes, &p), "car_alloc");
  return (int64_t)p;
}
py::bytes car_handle(int64_t base) {
  char buf[64] = {0};
  ok(dllm_car_get_handle((void*)base, buf), "hipIpcGetMemHandle");
  return py::bytes(buf, dllm_car_handle_size());
}
int64_t car_open(py::bytes h) {
  std::string s = h;
  TORCH_CHECK((int)s.size() == dllm_car_handle_size(), "bad IPC handle size");
  void* p = nullptr;
  ok(dllm_car_open_handle(s.data(), &p), "hipIpcOpenMemHandle");
  return (int64_t)p;
}
void car_close(int64_t base) { ok(dllm_car_close_handle((void*)base), "hipIpcCloseMemHandle"); }
void car_free(int64_t base) { ok(dllm_car_free((void*)base), "hipFree"); }
void car_allreduce(torch::Tensor x, torch::Tensor out, std::vector<int64_t> bases, int64_t rank, int64_t data_bytes,
                   torch::Tensor counters, torch::Tensor err, int64_t spin_limit) {
  check_bf16(x, "x");
  check_bf16(out, "out");
  check_i32(counters, "counters");
  check_i32(err, "err");
  TORCH_CHECK(x.is_contiguous() && out.is_contiguous() && x.numel() == out.numel(), "contiguous, same size");
  TORCH_CHECK(counters.numel() >= 2 && err.numel() >= 1, "counters[2], err[1]");
  const int64_t nbytes = x.numel() * 2;
  TORCH_CHECK(nbytes % 16 == 0 && nbytes <= data_bytes, "message must be a multiple of 16 B and fit the buffer");
  TORCH_CHECK(!bases.empty() && bases.size() <= 8 && rank >= 0 && rank < (int64_t)bases.size(), "bad ranks");
  void* b[8];
  for (size_t i = 0; i < bases.size(); ++i) b[i] = (void*)bases[i];
  ok(dllm_car_allreduce(x.data_ptr(), out.data_ptr(), nbytes, b, (int)bases.size(), (int)rank, data_bytes,
                        (unsigned*)counters.data_ptr<int>(), err.data_ptr<int>(), spin_limit, stream()),
     "car_allreduce");
}

// r = bf16(sum_p y_p) + r (add) or r = bf16(sum_p y_p), in place, and the new r's partial row sums
// of squares per column slice into ssq [slots, >= T]; returns the slot count (one-shot all-reduce
// with the fused residual / RMSNorm-statistics epilogue, csrc/kernels/custom_ar.hip)
int64_t car_resadd(torch::Tensor y, torch::Tensor r, torch::Tensor ssq, bool add, std::vector<int64_t> bases,
                   int64_t rank, int64_t data_bytes, torch::Tensor counters, torch::Tensor err, int64_t spin_limit) {
  check_bf16(y, "y");
  check_bf16(r, "r");
  check_f32(ssq, "ssq");
  check_i32(counters, "counters");
  check_i32(err, "err");
  TORCH_CHECK(y.dim() == 2 && y.is_contiguous() && r.dim() == 2 && r.stride(1) == 1 && r.sizes() == y.sizes(),
              "y [T, H] contiguous, r like y (row stride may differ)");
  const int H = (int)y.size(1), T = (int)y.size(0);
  const int slots = dllm_car_resadd_slots(H);
  TORCH_CHECK(slots >= 1, "hidden size has no column-slice split");
  TORCH_CHECK(ssq.dim() == 2 && ssq.size(0) >= slots && ssq.size(1) >= T && ssq.stride(1) == 1, "ssq [>= slots, >= T]");
  TORCH_CHECK((int64_t)T * H * 2 <= data_bytes, "message must fit the buffer");
  TORCH_CHECK(!bases.empty() && bases.size() <= 8 && rank >= 0 && rank < (int64_t)bases.size(), "bad ranks");
  void* b[8];
  for (size_t i = 0; i < bases.size(); ++i) b[i] = (void*)bases[i];
  const int n = dllm_car_resadd(y.data_ptr(), r.data_ptr(), r.stride(0), ssq.data_ptr<float>(), ssq.stride(0), T, H,
                                add ? 1 : 0, b, (int)bases.size(), (int)rank, data_bytes,
                                (unsigned*)counters.data_ptr<int>(), err.data_ptr<int>(), spin_limit, stream());
  TORCH_CHECK(n >= 1, "car_resadd failed (", n, ")");
  return n;
}
int64_t car_resadd_slots(int64_t H) { return dllm_car_resadd_slots((int)H); }
void car_allgather(torch::Tensor x, torch::Tensor out, std::vector<int64_t> bases, int64_t rank, int64_t data_bytes,
                   torch::Tensor counters, torch::Tensor err, int64_t spin_limit) {
  check_i32(counters, "counters");
  check_i32(err, "err");
  TORCH_CHECK(x.is_contiguous() && out.is_contiguous() && x.scalar_type() == out.scalar_type(), "contiguous, same dtype");
  TORCH_CHECK(out.numel() == x.numel() * (int64_t)bases.size(), "out = world x input");
  const int64_t nbytes = x.numel() * x.element_size();
  TORCH_CHECK(nbytes % 16 == 0 && nbytes <= data_bytes, "message must be a multiple of 16 B and fit the buffer");
  TORCH_CHECK(!bases.empty() && bases.size() <= 8 && rank >= 0 && rank < (int64_t)bases.size(), "bad ranks");
  void* b[8];
  for (size_t i = 0; i < bases.size(); ++i) b[i] = (void*)bases[i];
  ok(dllm_car_allgather(x.data_ptr(), out.data_ptr(), nbytes, b, (int)bases.size(), (int)rank, data_bytes,
                        (unsigned*)counters.data_ptr<int>(), err.data_ptr<int>(), spin_limit, stream()),
     "car_allgather");
}
// In-graph health vote glue around the 16-byte one-shot all-reduce (mode 0: stage, 1: decide).
void car_vote(int64_t mode, torch::Tensor err, torch::Tensor v, torch::Tensor out) {
  check_i32(err, "err");
  check_i32(out, "out");
  TORCH_CHECK(v.scalar_type() == torch::kBFloat16 && v.numel() >= 8 && v.is_contiguous(), "car_vote: v bf16 [>= 8]");
  TORCH_CHECK(err.numel() >= 2 && out.numel() >= 1, "car_vote: err [flag, staged snapshot] / out");
  ok(dllm_car_vote((int)mode, err.data_ptr<int>(), v.data_ptr(), out.data_ptr<int>(), stream()), "car_vote");
}

// ---- fused-epilogue LDS-tiled GEMM (csrc/kernels/tgemm.hip).  epi: 0 plain y = x.w^T (optionally
// row-scaled by rinv from ssq_in), 1 residual add (y = residual, in place; ssq_out partial row
// sums), 2 QKV (RoPE + q_out + paged K/V writes), 3 SwiGLU (y = [M, N/2]), 4 GELU (y = gelu(x.w^T +
// bias)).  bias [N] (epi 0, 1, 4) is added to the product before the epilogue op.
void tgemm(torch::Tensor x, torch::Tensor w, c10::optional<torch::Tensor> y, int64_t epi, int64_t bm, int64_t bn,
           int64_t stages, int64_t splits, int64_t ks, int64_t nw, c10::optional<torch::Tensor> part, c10::optional<torch::Tensor> counters,
           c10::optional<torch::Tensor> ssq_in, int64_t ssq_in_n, double norm_scale, double eps,
           c10::optional<torch::Tensor> ssq_out, c10::optional<torch::Tensor> pos,
           c10::optional<torch::Tensor> cos_sin, c10::optional<torch::Tensor> slots,
           c10::optional<torch::Tensor> q_out, c10::optional<torch::Tensor> kc, c10::optional<torch::Tensor> vc,
           int64_t nq, int64_t nkv, int64_t d, c10::optional<torch::Tensor> bias, int64_t wk, int64_t nl,
           c10::optional<torch::Tensor> sk_table, int64_t sk_cmax, c10::optional<torch::Tensor> v_rows,
           int64_t kdepth, int64_t mfma, int64_t raster) {
  check_bf16(x, "x");
  check_bf16(w, "w");
  TORCH_CHECK(mfma == 16 || mfma == 32, "tgemm: mfma 16 or 32");
  if (mfma == 32) {   // tgemm.hip by_tile_m32 minus kPruned: the whitelist, so a bad plan gets a clear error
    const bool known = wk == 1 && kdepth == 64 &&
                       ((nl == 0 && ks == 2 && stages == 3 && ((bm == 64 && bn == 64 && nw == 4) ||
                                                               (bm == 64 && bn == 128 && nw == 8))));
    TORCH_CHECK(known, "tgemm: no 32x32x16 plan (", bm, "x", bn, ", ", stages, " stages, ks ", ks, ", ", nw, "+", nl,
                " waves)");
    TORCH_CHECK(!sk_table.has_value(), "tgemm: 32x32x16 plans have no stream-K form");
  }
  if (kdepth == 32) {   // tgemm.hip by_tile_k32 minus kPruned: explicit whitelist
    const bool known = ks == 1 && wk == 1 && nw == 8 && bm == 256 && bn == 256 && stages == 4 && nl == 0;
    TORCH_CHECK(known, "tgemm: no 32-deep plan (", bm, "x", bn, ", ", stages, " stages, ", nw, "+", nl, " waves)");
  }
  if (nl > 0 && kdepth != 32 && mfma == 16) {  // loader-wave plans (tgemm.hip by_tile_nl minus kPruned): KS 1, one k-group
    const bool known = ks == 1 && wk == 1 &&
                       ((bm == 16 && bn == 128 && nw == 4 && nl == 6 && (stages == 4 || stages == 8)) ||
                        (bm == 64 && bn == 64 && nw == 4 && ((nl == 4 && stages == 4) || (nl == 8 && (stages == 4 || stages == 8)))) ||
                        (bm == 128 && bn == 64 && nw == 4 && (nl == 4 || nl == 8) && stages == 4) ||
                        (bm == 128 && bn == 128 && nw == 4 && nl == 8 && stages == 4) ||
                        (bm == 160 && bn == 128 && nw == 8 && (nl == 4 || nl == 6) && stages == 3) ||
                        (bm == 256 && bn == 128 && nw == 8 && (nl == 4 || nl == 8) && stages == 3));
    TORCH_CHECK(known, "tgemm: no loader-wave plan (", bm, "x", bn, ", ", stages, " stages, ", nw, "+", nl, " waves)");
  }
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && x.stride(0) % 8 == 0, "x: 2-D row-major, 16-B aligned rows");
  TORCH_CHECK(epi >= 0 && epi <= 4, "epi");
  // w: [N, K] row-major, or the K-panel-major copy [K / 64, N, 64] (models.llama.panel_weight)
  const bool panel = w.dim() == 3;
  TORCH_CHECK(((w.dim() == 2) || (panel && w.size(2) == 64)) && w.is_contiguous(),
              "w: [N, K] or [K / 64, N, 64] contiguous");
  const int M = x.size(0), N = panel ? w.size(1) : w.size(0), K = panel ? w.size(0) * 64 : w.size(1);
  TORCH_CHECK((ks == 1 || ks == 2) && (nw == 4 || (nw == 8 && bn >= 128)), "ks in {1,2}; nw 4, or 8 with bn >= 128");
  TORCH_CHECK(wk == 1 || (wk == 2 && nw == 4 && ks == 2 && stages <= 3 && bm <= 128 && bn <= 128),
              "wk 2: two k-groups of 4 waves, ks 2, 2-3 stages, tiles up to 128 x 128");
  TORCH_CHECK(x.size(1) == K && K % (64 * ks) == 0, "x [M, K], K % (64 ks) == 0");
  TORCH_CHECK(nl > 0 || kdepth == 32 || ((bm == 64 || bm == 128 || ((bm == 192 || bm == 256) && nw == 8)) && (bn == 64 || bn == 128 || (bn == 256 && bm == 256)) &&
                  (stages == 2 || stages == 3 || ((stages == 4 || stages == 6) && ks == 1 && bm <= 128)) &&
                  (int64_t)stages * ks * (bm + bn) * 128 <= 150 * 1024),
              "tile / ring size");
  TORCH_CHECK(splits >= 1 && splits <= 64, "splits");
  const int kq = 64 * (int)ks;
  int kchunk = (K + splits - 1) / splits;
  kchunk = (kchunk + kq - 1) / kq * kq;
  const int S = (K + kchunk - 1) / kchunk;
  const int64_t tiles = (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
  dllm::GemmArgs a{};
  a.A = (const uint16_t*)x.data_ptr();
  a.lda = x.stride(0);
  a.W = (const uint16_t*)w.data_ptr();
  a.M = M; a.N = N; a.K = K; a.kchunk = kchunk; a.splits = S;
  a.w_panel = panel ? 1 : 0;
  if (sk_table.has_value()) {   // stream-K: the host-built segment lists (ops.gemm.stream_k_table)
    check_i32(*sk_table, "sk_table");
    TORCH_CHECK(sk_table->dim() == 3 && sk_table->size(2) == 4 && sk_table->is_contiguous() &&
                    sk_table->size(0) >= 1 && sk_table->size(1) >= 1 && sk_cmax >= 1 && splits == 1,
                "sk_table [grid, segments, 4] int32, splits 1");
    TORCH_CHECK(part.has_value() && counters.has_value(), "stream-K needs part/counters workspaces");
    check_f32(*part, "part");
    check_i32(*counters, "counters");
    TORCH_CHECK(part->numel() >= sk_cmax * tiles * bm * bn && counters->numel() >= tiles,
                "stream-K workspace too small");
    a.part = part->data_ptr<float>();
    a.counters = counters->data_ptr<int>();
    a.sk_table = sk_table->data_ptr<int>();
    a.sk_grid = (int)sk_table->size(0);
    a.sk_segmax = (int)sk_table->size(1);
    a.sk_cmax = (int)sk_cmax;
  } else if (S > 1) {
    TORCH_CHECK(part.has_value() && counters.has_value(), "split-K needs part/counters workspaces");
    check_f32(*part, "part");
    check_i32(*counters, "counters");
    TORCH_CHECK(part->numel() >= (int64_t)S * tiles * bm * bn && counters->numel() >= tiles,
                "split-K workspace too small");
    a.part = part->data_ptr<float>();
    a.counters = counters->data_ptr<int>();
  }
  if (ssq_in.has_value()) {
    check_f32(*ssq_in, "ssq_in");
    TORCH_CHECK(ssq_in->dim() == 2 && ssq_in->size(1) >= M && ssq_in_n >= 1 && ssq_in_n <= ssq_in->size(0),
                "ssq_in [slots, >= M]");
    TORCH_CHECK(epi != 1, "residual epilogue takes no row scale");
    a.ssq_in = ssq_in->data_ptr<float>();
    a.ssq_in_n = ssq_in_n;
    a.ssq_in_ld = ssq_in->size(1);
    a.norm_scale = (float)norm_scale;
    a.eps = (float)eps;
  }
  if (bias.has_value()) {
    check_bf16(*bias, "bias");
    TORCH_CHECK(epi == 0 || epi == 1 || epi == 4, "bias: plain, residual or gelu epilogue");
    TORCH_CHECK(bias->is_contiguous() && bias->numel() == N, "bias [N]");
    a.bias = (const uint16_t*)bias->data_ptr();
  }
  if (epi == 0 || epi == 1 || epi == 3 || epi == 4) {
    TORCH_CHECK(y.has_value(), "y required");
    check_bf16(*y, "y");
    TORCH_CHECK(y->dim() == 2 && y->stride(1) == 1 && y->size(0) == M && y->size(1) == (epi == 3 ? N / 2 : N),
                "y shape");
    a.Y = (uint16_t*)y->data_ptr();
    a.ldy = y->stride(0);
  }
  if (epi == 1 && ssq_out.has_value()) {
    check_f32(*ssq_out, "ssq_out");
    TORCH_CHECK(ssq_out->dim() == 2 && ssq_out->size(0) >= (N + bn - 1) / bn && ssq_out->size(1) >= M,
                "ssq_out [>= n_tiles, >= M]");
    a.ssq_out = ssq_out->data_ptr<float>();
    a.ssq_out_ld = ssq_out->size(1);
  }
  if (epi == 3) TORCH_CHECK(N % 32 == 0, "swiglu: N % 32 == 0");
  if (epi == 2) {
    TORCH_CHECK(pos.has_value() && cos_sin.has_value() && slots.has_value() && q_out.has_value() && kc.has_value() &&
                    vc.has_value(),
                "qkv epilogue operands");
    check_i32(*pos, "positions");
    check_i32(*slots, "slots");
    check_f32(*cos_sin, "cos_sin");
    check_bf16(*q_out, "q_out");
    check_bf16(*kc, "k_cache");
    check_bf16(*vc, "v_cache");
    TORCH_CHECK(d % 32 == 0 && N == (nq + 2 * nkv) * d, "qkv: N == (nq + 2 nkv) d, d % 32 == 0");
    TORCH_CHECK(pos->numel() >= M && slots->numel() >= M, "positions/slots length");
    TORCH_CHECK(cos_sin->dim() == 2 && cos_sin->size(1) == d, "cos_sin [max_pos, d]");
    TORCH_CHECK(q_out->is_contiguous() && q_out->numel() >= (int64_t)M * nq * d, "q_out [M, nq, d]");
    TORCH_CHECK(kc->is_contiguous() && vc->is_contiguous() && kc->dim() == 4 && kc->size(1) == nkv &&
                    kc->size(2) == 16 && kc->size(3) == d && vc->size(1) == nkv && vc->size(2) == d &&
                    vc->size(3) == 16,
                "cache layout: K [blocks, nkv, 16, d], V [blocks, nkv, d, 16]");
    a.pos = pos->data_ptr<int>();
    a.cos_sin = cos_sin->data_ptr<float>();
    a.slots = slots->data_ptr<int>();
    a.q_out = (uint16_t*)q_out->data_ptr();
    a.kc = (uint16_t*)kc->data_ptr();
    a.vc = (uint16_t*)vc->data_ptr();
    a.nq = nq; a.nkv = nkv; a.d = d;
    if (v_rows.has_value()) {   // V row-major [M, nkv * d] instead of the V^T cache (decode attention writes it)
      check_bf16(*v_rows, "v_rows");
      TORCH_CHECK(v_rows->dim() == 2 && v_rows->stride(1) == 1 && v_rows->size(0) >= M && v_rows->size(1) == nkv * d &&
                      v_rows->stride(0) % 8 == 0,
                  "v_rows [>= M, nkv * d], 16-B aligned rows");
      a.v_rows = (uint16_t*)v_rows->data_ptr();
      a.v_ld = v_rows->stride(0);
    }
  }
  TORCH_CHECK(kdepth == 64 || kdepth == 32, "tgemm: k depth 64 or 32");
  a.kdepth = (int)kdepth;
  a.mfma = (int)mfma;
  TORCH_CHECK(raster >= 0 && raster <= 64, "tgemm: raster 0..64");
  a.raster = (int)raster;
  ok(dllm_tgemm(&a, (int)bm, (int)bn, (int)stages, (int)ks, (int)nw, (int)wk, (int)epi, stream(), (int)nl), "tgemm");
}

// standalone EPI_QKV / EPI_SWIGLU for a vendor-GEMM output y (prefill)
void qkv_post(torch::Tensor y, torch::Tensor ssq, int64_t ssq_n, double scale, double eps, torch::Tensor pos,
              torch::Tensor cos_sin, torch::Tensor slots, torch::Tensor q_out, torch::Tensor kc, torch::Tensor vc,
              int64_t nq, int64_t nkv, int64_t d, c10::optional<torch::Tensor> v_rows) {
  check_bf16(y, "y");
  check_f32(ssq, "ssq");
  check_i32(pos, "positions");
  check_i32(slots, "slots");
  check_f32(cos_sin, "cos_sin");
  for (auto* t : {&q_out, &kc, &vc}) check_bf16(*t, "qkv outputs");
  const int M = y.size(0);
  TORCH_CHECK(y.dim() == 2 && y.stride(1) == 1 && y.size(1) == (nq + 2 * nkv) * d && d % 32 == 0, "y [M, (nq+2nkv) d]");
  TORCH_CHECK(ssq.dim() == 2 && ssq.size(1) >= M && ssq_n >= 1 && ssq_n <= ssq.size(0), "ssq [slots, >= M]");
  TORCH_CHECK(pos.numel() >= M && slots.numel() >= M && cos_sin.size(1) == d, "positions/slots/cos_sin");
  TORCH_CHECK(q_out.is_contiguous() && q_out.numel() >= (int64_t)M * nq * d, "q_out");
  TORCH_CHECK(kc.is_contiguous() && vc.is_contiguous() && kc.size(1) == nkv && kc.size(2) == 16 && kc.size(3) == d &&
                  vc.size(2) == d && vc.size(3) == 16,
              "cache layout");
  void* vr = nullptr;
  if (v_rows.has_value() && v_rows->defined()) {   // decode: V row-major, the attention kernel writes V^T
    check_bf16(*v_rows, "v_rows");
    TORCH_CHECK(v_rows->is_contiguous() && v_rows->numel() >= (int64_t)M * nkv * d, "v_rows [M, nkv d]");
    vr = v_rows->data_ptr();
  }
  ok(dllm_qkv_post(y.data_ptr(), y.stride(0), ssq.data_ptr<float>(), ssq_n, ssq.size(1), (float)scale, (float)eps,
                   pos.data_ptr<int>(), cos_sin.data_ptr<float>(), slots.data_ptr<int>(), q_out.data_ptr(), kc.data_ptr(),
                   vc.data_ptr(), vr, M, nq, nkv, d, stream()),
     "qkv_post");
}

void swiglu_post(torch::Tensor y, torch::Tensor ssq, int64_t ssq_n, double scale, double eps, torch::Tensor act) {
  check_bf16(y, "y");
  check_f32(ssq, "ssq");
  check_bf16(act, "act");
  const int M = y.size(0), N = y.size(1);
  TORCH_CHECK(y.dim() == 2 && y.stride(1) == 1 && N % 32 == 0, "y [M, 2I]");
  TORCH_CHECK(act.dim() == 2 && act.stride(1) == 1 && act.size(0) == M && act.size(1) == N / 2, "act [M, I]");
  TORCH_CHECK(ssq.dim() == 2 && ssq.size(1) >= M && ssq_n >= 1 && ssq_n <= ssq.size(0), "ssq [slots, >= M]");
  ok(dllm_swiglu_post(y.data_ptr(), y.stride(0), ssq.data_ptr<float>(), ssq_n, ssq.size(1), (float)scale, (float)eps,
                      act.data_ptr(), act.stride(0), M, N, stream()),
     "swiglu_post");
}

// r = h + r in place (h optional) and row sums of r^2: ssq f32 [M] (one slot) or [slots, >= M]
// (partial sums over up to ``slots`` column slices); returns the number of slots written
int64_t res_add_ssq(c10::optional<torch::Tensor> h, torch::Tensor r, torch::Tensor ssq) {
  check_bf16(r, "r");
  check_f32(ssq, "ssq");
  TORCH_CHECK(r.dim() == 2 && r.stride(1) == 1, "r [M, H]");
  TORCH_CHECK((ssq.dim() == 1 && ssq.numel() >= r.size(0)) ||
                  (ssq.dim() == 2 && ssq.size(1) >= r.size(0) && ssq.stride(1) == 1),
              "ssq [>= M] or [slots, >= M]");
  const void* hp = nullptr;
  long ldh = 0;
  if (h.has_value()) {
    check_bf16(*h, "h");
    TORCH_CHECK(h->dim() == 2 && h->stride(1) == 1 && h->sizes() == r.sizes(), "h like r");
    hp = h->data_ptr();
    ldh = h->stride(0);
  }
  const int slices = ssq.dim() == 2 ? (int)ssq.size(0) : 1;
  const long ld = ssq.dim() == 2 ? ssq.stride(0) : 0;
  const int n = dllm_res_add_ssq(hp, ldh, r.data_ptr(), r.stride(0), ssq.data_ptr<float>(), ld, slices, r.size(0),
                                 r.size(1), stream());
  TORCH_CHECK(n >= 1, "res_add_ssq failed (", n, ")");
  return n;
}


// router encoder (csrc/kernels/encoder.hip): bidirectional attention over a padded batch
void encoder_attention(torch::Tensor qkv, torch::Tensor lens, torch::Tensor out, int64_t B, int64_t S, int64_t nh,
                       int64_t d, double scale) {
  check_bf16(qkv, "qkv");
  check_bf16(out, "out");
  check_i32(lens, "lens");
  TORCH_CHECK(d == 32 || d == 64, "encoder attention: head_dim 32 or 64");
  TORCH_CHECK(S >= 1 && S <= 512, "encoder attention: 1 <= S <= 512");
  TORCH_CHECK(qkv.is_contiguous() && qkv.dim() == 2 && qkv.size(0) == B * S && qkv.size(1) == 3 * nh * d,
              "qkv [B*S, 3 nh d]");
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == B * S && out.size(1) == nh * d, "out [B*S, nh d]");
  TORCH_CHECK(lens.numel() >= B, "lens [B]");
  ok(dllm_encoder_attention(qkv.data_ptr(), lens.data_ptr<int>(), out.data_ptr(), B, S, nh, d, (float)scale, stream()),
     "encoder_attention");
}

void embed_ln(torch::Tensor ids, torch::Tensor word, torch::Tensor pos, torch::Tensor type0, torch::Tensor w,
              torch::Tensor b, torch::Tensor out, int64_t S, double eps) {
  check_i32(ids, "ids");
  for (auto* t : {&word, &pos, &type0, &w, &b, &out}) check_bf16(*t, "embed_ln operand");
  const int64_t T = ids.numel(), H = word.size(1);
  TORCH_CHECK(ids.is_contiguous() && word.is_contiguous() && pos.is_contiguous() && type0.is_contiguous() &&
                  w.is_contiguous() && b.is_contiguous() && out.is_contiguous(),
              "contiguous operands");
  TORCH_CHECK(S >= 1 && T % S == 0 && pos.size(0) >= S && pos.size(1) == H && type0.numel() == H && w.numel() == H &&
                  b.numel() == H && out.numel() == T * H && H % 8 == 0 && H <= 2048,
              "embed_ln shapes");
  ok(dllm_embed_ln(ids.data_ptr<int>(), word.data_ptr(), pos.data_ptr(), type0.data_ptr(), w.data_ptr(), b.data_ptr(),
                   out.data_ptr(), T, S, H, word.size(0), (float)eps, stream()),
     "embed_ln");
}
// ---- sequence mixers and the f32 residual stream (csrc/kernels/seqmix.hip, latent.hip).
// Activations are bf16 or f32; `act_f32` reports which and checks that a tensor is one of the two.
bool act_f32(const torch::Tensor& t, const char* name) {
  check_dev(t, name);
  TORCH_CHECK(t.scalar_type() == torch::kBFloat16 || t.scalar_type() == torch::kFloat32, name, " must be bf16 or f32");
  return t.scalar_type() == torch::kFloat32;
}
void check_rows2d(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 2 && t.stride(1) == 1, name, " must be 2-D with unit column stride");
}
struct SeqMeta { int S; const int *qstart, *qlen, *ctx, *rows; };
SeqMeta seq_meta(const torch::Tensor& qstart, const torch::Tensor& qlen, const torch::Tensor& ctx,
                 const torch::Tensor& rows, int64_t slots) {
  for (auto* t : {&qstart, &qlen, &ctx, &rows}) check_i32(*t, "sequence metadata");
  const int S = qstart.numel();
  TORCH_CHECK(qlen.numel() == S && ctx.numel() == S && rows.numel() >= S, "sequence metadata lengths");
  TORCH_CHECK(slots >= 1, "state slots");
  return {S, qstart.data_ptr<int>(), qlen.data_ptr<int>(), ctx.data_ptr<int>(), rows.data_ptr<int>()};
}

void rms_rows(torch::Tensor x, c10::optional<torch::Tensor> w, torch::Tensor y, double eps, int64_t groups) {
  const bool xf = act_f32(x, "x"), yf = act_f32(y, "y");
  check_rows2d(x, "x");
  check_rows2d(y, "y");
  TORCH_CHECK(x.sizes() == y.sizes(), "x / y shapes");
  const float* wp = nullptr;
  if (w) {
    check_f32(*w, "w");
    TORCH_CHECK(w->numel() == x.size(1), "w length");
    wp = w->data_ptr<float>();
  }
  TORCH_CHECK(groups >= 1 && x.size(1) % groups == 0, "row length must be a multiple of groups");
  ok(dllm_rms_rows(x.data_ptr(), x.stride(0), xf, wp, y.data_ptr(), y.stride(0), yf, (int)x.size(0), (int)x.size(1),
                   (float)eps, (int)groups, stream()),
     "rms_rows");
}

void norm_resadd(torch::Tensor y, torch::Tensor w, double eps, torch::Tensor x, c10::optional<torch::Tensor> xl,
                 int64_t groups, c10::optional<torch::Tensor> bias) {
  const bool f = act_f32(y, "y");
  check_rows2d(y, "y");
  check_f32(w, "w");
  check_f32(x, "x");
  TORCH_CHECK(x.dim() == 2 && x.sizes() == y.sizes() && w.numel() == x.size(1), "x / y / w shapes");
  void* lp = nullptr;
  if (xl) {
    TORCH_CHECK(xl->is_cuda() && xl->scalar_type() == y.scalar_type() && xl->is_contiguous() && xl->sizes() == x.sizes(),
                "x_lp: contiguous, the dtype of y, the shape of x");
    lp = xl->data_ptr();
  }
  TORCH_CHECK(groups >= 1 && x.size(1) % groups == 0 && x.is_contiguous(), "width must be a multiple of groups; x contiguous");
  const float* bp = nullptr;
  if (bias) {
    check_f32(*bias, "bias");
    TORCH_CHECK(bias->numel() == x.size(1), "bias length");
    bp = bias->data_ptr<float>();
  }
  ok(dllm_norm_resadd(y.data_ptr(), y.stride(0), f, w.data_ptr<float>(), x.data_ptr<float>(), lp, (int)x.size(0),
                      (int)x.size(1), (float)eps, (int)groups, bp, stream()),
     "norm_resadd");
}

void causal_conv_silu(torch::Tensor x, torch::Tensor w, torch::Tensor b, torch::Tensor state, torch::Tensor qstart,
                      torch::Tensor qlen, torch::Tensor ctx, torch::Tensor rows, torch::Tensor y, bool refill, int64_t act) {
  const bool f = act_f32(x, "x");
  TORCH_CHECK(act == 0 || act == 1, "act: 0 (SiLU) or 1 (input plus convolution)");
  check_rows2d(x, "x");
  check_f32(w, "w");
  check_f32(b, "b");
  TORCH_CHECK(w.dim() == 2, "w [C, K]");
  const int C = w.size(0), K = w.size(1), T = x.size(0);
  TORCH_CHECK(x.size(1) >= C && b.numel() == C, "x / b widths");
  TORCH_CHECK(state.is_cuda() && state.scalar_type() == x.scalar_type() && state.is_contiguous() && state.dim() == 3 &&
                  state.size(1) == K - 1 && state.size(2) == C,
              "conv state [slots, K - 1, C] in the dtype of x");
  TORCH_CHECK(y.is_cuda() && y.scalar_type() == x.scalar_type() && y.is_contiguous() && y.dim() == 2 && y.size(0) == T &&
                  y.size(1) == C,
              "y [T, C]");
  TORCH_CHECK(y.data_ptr() != x.data_ptr() || (refill && x.stride(0) == C),
              "in place only for steps of single tokens (refill) over exactly the convolved columns");
  auto m = seq_meta(qstart, qlen, ctx, rows, state.size(0));
  ok(dllm_conv_silu(x.data_ptr(), x.stride(0), f, w.data_ptr<float>(), b.data_ptr<float>(), state.data_ptr(), m.qstart,
                    m.qlen, m.ctx, m.rows, y.data_ptr(), T, m.S, C, K, (int)refill, (int)act, stream()),
     "causal_conv_silu");
}

void selective_scan(torch::Tensor xc, torch::Tensor dt_raw, torch::Tensor dt_bias, torch::Tensor A, torch::Tensor dbc,
                    int64_t dt_rank, torch::Tensor D, torch::Tensor xz, torch::Tensor ssm, torch::Tensor conv,
                    torch::Tensor qstart, torch::Tensor qlen, torch::Tensor ctx, torch::Tensor rows, torch::Tensor out) {
  const bool f = act_f32(xc, "xc");
  for (auto* t : {&dt_raw, &dbc, &xz, &out, &conv})
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == xc.scalar_type(), "activations share one dtype");
  check_f32(dt_bias, "dt_bias");
  check_f32(A, "A");
  check_f32(D, "D");
  check_f32(ssm, "ssm_state");
  TORCH_CHECK(A.dim() == 2, "A [C, N]");
  const int C = A.size(0), N = A.size(1), T = xc.size(0);
  TORCH_CHECK(xc.dim() == 2 && xc.is_contiguous() && xc.size(1) == C, "xc [T, C]");
  TORCH_CHECK(dt_raw.dim() == 2 && dt_raw.is_contiguous() && dt_raw.size(0) == T && dt_raw.size(1) == C, "dt_raw [T, C]");
  TORCH_CHECK(out.is_contiguous() && out.sizes() == xc.sizes(), "out [T, C]");
  check_rows2d(dbc, "dbc");
  check_rows2d(xz, "xz");
  TORCH_CHECK(dbc.size(0) == T && dt_rank >= 0 && dbc.size(1) >= dt_rank + 2 * N, "dbc [T, dt_rank + 2N]");
  TORCH_CHECK(xz.size(0) == T && xz.size(1) >= 2 * C, "xz [T, 2C]");
  TORCH_CHECK(dt_bias.numel() == C && D.numel() == C, "dt_bias / D length");
  TORCH_CHECK(ssm.dim() == 3 && ssm.size(1) == C && ssm.size(2) == N, "ssm_state [slots, C, N]");
  TORCH_CHECK(conv.is_contiguous() && conv.dim() == 3 && conv.size(0) == ssm.size(0) && conv.size(2) == C,
              "conv_state [slots, K - 1, C]");
  auto m = seq_meta(qstart, qlen, ctx, rows, ssm.size(0));
  ok(dllm_selective_scan(xc.data_ptr(), dt_raw.data_ptr(), f, dt_bias.data_ptr<float>(), A.data_ptr<float>(),
                         dbc.data_ptr(), dbc.stride(0), (int)dt_rank, D.data_ptr<float>(), xz.data_ptr(), xz.stride(0),
                         ssm.data_ptr<float>(), conv.data_ptr(), (int)conv.size(1), m.qstart, m.qlen, m.ctx, m.rows,
                         out.data_ptr(), m.S, C, N, stream()),
     "selective_scan");
}

void retention(torch::Tensor qkvg, int64_t H, int64_t d, int64_t dv, torch::Tensor cos_sin, int64_t rot,
               torch::Tensor decay, torch::Tensor state, double eps, torch::Tensor pos, torch::Tensor qstart,
               torch::Tensor qlen, torch::Tensor ctx, torch::Tensor rows, torch::Tensor out,
               c10::optional<torch::Tensor> raw) {
  const bool f = act_f32(qkvg, "qkvg");
  check_rows2d(qkvg, "qkvg");
  check_f32(cos_sin, "cos_sin");
  check_f32(decay, "decay");
  check_f32(state, "state");
  check_i32(pos, "positions");
  const int T = qkvg.size(0);
  TORCH_CHECK(H >= 1 && d >= 1 && dv >= 1 && qkvg.size(1) >= 2 * H * d + 2 * H * dv, "qkvg [T, 2 H d + 2 H dv]");
  TORCH_CHECK(cos_sin.dim() == 2 && rot >= 0 && rot % 2 == 0 && rot <= d && cos_sin.size(1) >= rot, "rotation table");
  TORCH_CHECK(decay.numel() == H, "decay per head");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == d && state.size(3) == dv,
              "state [slots, H, d, dv]");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == qkvg.scalar_type() && out.is_contiguous() && out.dim() == 2 &&
                  out.size(0) == T && out.size(1) == H * dv,
              "out [T, H dv]");
  auto m = seq_meta(qstart, qlen, ctx, rows, state.size(0));
  if (raw) {   // chunked form (prompt portions): f32 scratch [T, H, dv]
    check_f32(*raw, "raw");
    TORCH_CHECK(raw->numel() >= (int64_t)T * H * dv, "raw scratch [T, H, dv]");
    TORCH_CHECK(dllm_retention_chunk_lds((int)d) <= 150 * 1024, "dim does not fit the LDS");
    ok(dllm_retention_chunked(qkvg.data_ptr(), qkvg.stride(0), f, (int)H, (int)d, (int)dv, cos_sin.data_ptr<float>(),
                              (int)cos_sin.size(1), (int)rot, decay.data_ptr<float>(), state.data_ptr<float>(), (float)eps,
                              m.qstart, m.qlen, m.ctx, m.rows, raw->data_ptr<float>(), out.data_ptr(), m.S, (long)T, 0,
                              1.f / std::sqrt((float)d), 1, stream()),
       "retention (chunked)");
    return;
  }
  TORCH_CHECK(dllm_retention_lds((int)d, (int)dv) <= 150 * 1024, "dim x vdim state does not fit the LDS");
  ok(dllm_retention(qkvg.data_ptr(), qkvg.stride(0), f, (int)H, (int)d, (int)dv, cos_sin.data_ptr<float>(),
                    (int)cos_sin.size(1), (int)rot, decay.data_ptr<float>(), state.data_ptr<float>(), (float)eps, m.qstart,
                    m.qlen, m.ctx, m.rows, out.data_ptr(), m.S, 0, 1.f / std::sqrt((float)d), nullptr, stream()),
     "retention");
}

// Lightning attention on the retention kernels: SiLU'd q / k / v, no rotation, no key scale, raw f32
// outputs [T, H, dv]; then the heads of a token are normed together and gated by a sigmoid.
void lightning_attention(torch::Tensor qkvg, int64_t H, int64_t d, int64_t dv, torch::Tensor decay, torch::Tensor state,
                         double eps, torch::Tensor norm_w, torch::Tensor qstart, torch::Tensor qlen, torch::Tensor ctx,
                         torch::Tensor rows, torch::Tensor out, torch::Tensor raw, bool chunked) {
  const bool f = act_f32(qkvg, "qkvg");
  check_rows2d(qkvg, "qkvg");
  check_f32(decay, "decay");
  check_f32(state, "state");
  check_f32(norm_w, "norm weight");
  check_f32(raw, "raw");
  const int T = qkvg.size(0);
  TORCH_CHECK(H >= 1 && d >= 1 && dv >= 1 && qkvg.size(1) >= 2 * H * d + 2 * H * dv, "qkvg [T, 2 H d + 2 H dv]");
  TORCH_CHECK(decay.numel() == H && norm_w.numel() == H * dv, "decay per head, norm weight [H dv]");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == d && state.size(3) == dv,
              "state [slots, H, d, dv]");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == qkvg.scalar_type() && out.is_contiguous() && out.dim() == 2 &&
                  out.size(0) == T && out.size(1) == H * dv,
              "out [T, H dv]");
  TORCH_CHECK(raw.numel() >= (int64_t)T * H * dv, "raw scratch [T, H, dv]");
  auto m = seq_meta(qstart, qlen, ctx, rows, state.size(0));
  if (chunked) {
    TORCH_CHECK(dllm_retention_chunk_lds((int)d) <= 150 * 1024, "dim does not fit the LDS");
    ok(dllm_retention_chunked(qkvg.data_ptr(), qkvg.stride(0), f, (int)H, (int)d, (int)dv, decay.data_ptr<float>(), 0, 0,
                              decay.data_ptr<float>(), state.data_ptr<float>(), (float)eps, m.qstart, m.qlen, m.ctx, m.rows,
                              raw.data_ptr<float>(), out.data_ptr(), m.S, (long)T, 1, 1.f, 0, stream()),
       "lightning attention (chunked)");
  } else {
    TORCH_CHECK(dllm_retention_lds((int)d, (int)dv) <= 150 * 1024, "dim x vdim state does not fit the LDS");
    ok(dllm_retention(qkvg.data_ptr(), qkvg.stride(0), f, (int)H, (int)d, (int)dv, decay.data_ptr<float>(), 0, 0,
                      decay.data_ptr<float>(), state.data_ptr<float>(), (float)eps, m.qstart, m.qlen, m.ctx, m.rows,
                      out.data_ptr(), m.S, 1, 1.f, raw.data_ptr<float>(), stream()),
       "lightning attention");
  }
  ok(dllm_heads_norm_gate(raw.data_ptr<float>(), qkvg.data_ptr(), qkvg.stride(0), f, 2 * H * d + H * dv, (int)(H * dv),
                          norm_w.data_ptr<float>(), (float)eps, m.qstart, m.qlen, m.S, out.data_ptr(), (long)T, stream()),
     "heads_norm_gate");
}

void resadd_norm(torch::Tensor a, c10::optional<torch::Tensor> b, c10::optional<torch::Tensor> wa,
                 c10::optional<torch::Tensor> wb, torch::Tensor w_post, double eps, torch::Tensor x,
                 c10::optional<torch::Tensor> w_next, c10::optional<torch::Tensor> xn,
                 c10::optional<torch::Tensor> stack, c10::optional<torch::Tensor> dw, int64_t dn) {
  const bool f = act_f32(a, "a");
  check_rows2d(a, "a");
  check_f32(w_post, "w_post");
  check_f32(x, "x");
  const float* dwp = nullptr;
  if (stack) {   // x must be slot dn - 1 of the stack; slot dn receives the weighted sum over depth
    TORCH_CHECK(dw.has_value(), "depth weights");
    check_f32(*stack, "stack");
    check_f32(*dw, "depth weights");
    TORCH_CHECK(stack->dim() == 3 && stack->is_contiguous() && dn >= 1 && dn < stack->size(0) && dw->numel() >= dn &&
                    stack->size(1) == x.size(0) && stack->size(2) == x.size(1) &&
                    x.data_ptr<float>() == stack->data_ptr<float>() + (dn - 1) * stack->size(1) * stack->size(2),
                "stack [slots, T, H] with x its slot dn - 1, dn < slots");
    dwp = dw->data_ptr<float>();
  }
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous() && x.sizes() == a.sizes() && w_post.numel() == x.size(1),
              "x / a / w_post shapes");
  const void* bp = nullptr;
  const float *wap = nullptr, *wbp = nullptr, *wnp = nullptr;
  long ldb = 0;
  if (b) {
    TORCH_CHECK(wa && wb, "two branches need both norm weights");
    check_rows2d(*b, "b");
    check_f32(*wa, "wa");
    check_f32(*wb, "wb");
    TORCH_CHECK(b->is_cuda() && b->scalar_type() == a.scalar_type() && b->sizes() == a.sizes() &&
                    wa->numel() == x.size(1) && wb->numel() == x.size(1),
                "b / wa / wb shapes");
    bp = b->data_ptr();
    ldb = b->stride(0);
    wap = wa->data_ptr<float>();
    wbp = wb->data_ptr<float>();
  }
  void* xp = nullptr;
  if (xn) {
    TORCH_CHECK(xn->is_cuda() && xn->scalar_type() == a.scalar_type() && xn->is_contiguous() && xn->sizes() == x.sizes(),
                "x_next: contiguous, the dtype of a, the shape of x");
    xp = xn->data_ptr();
    if (w_next) {
      check_f32(*w_next, "w_next");
      TORCH_CHECK(w_next->numel() == x.size(1), "w_next length");
      wnp = w_next->data_ptr<float>();
    }
  }
  ok(dllm_resadd_norm(a.data_ptr(), a.stride(0), bp, ldb, f, wap, wbp, w_post.data_ptr<float>(), x.data_ptr<float>(), wnp,
                      xp, (int)x.size(0), (int)x.size(1), (float)eps, dwp, (int)dn, stream()),
     "resadd_norm");
}

void depth_mix(torch::Tensor X, torch::Tensor w, int64_t n, c10::optional<torch::Tensor> w_next, double eps,
               c10::optional<torch::Tensor> xn) {
  check_f32(X, "X");
  check_f32(w, "w");
  TORCH_CHECK(X.dim() == 3 && X.is_contiguous() && n >= 1 && n < X.size(0) && w.numel() >= n, "X [slots, T, H], n < slots");
  void* xp = nullptr;
  const float* wnp = nullptr;
  bool f = true;
  if (xn) {
    f = act_f32(*xn, "out_next");
    TORCH_CHECK(xn->is_contiguous() && xn->dim() == 2 && xn->size(0) == X.size(1) && xn->size(1) == X.size(2), "out_next [T, H]");
    xp = xn->data_ptr();
    if (w_next) {
      check_f32(*w_next, "w_next");
      TORCH_CHECK(w_next->numel() == X.size(2), "w_next length");
      wnp = w_next->data_ptr<float>();
    }
  }
  ok(dllm_depth_mix(X.data_ptr<float>(), w.data_ptr<float>(), (int)n, X.size(1), (int)X.size(2), wnp, xp, f, (float)eps,
                    stream()),
     "depth_mix");
}

void gelu_erf(torch::Tensor x, torch::Tensor y) {
  const bool f = act_f32(x, "x");
  TORCH_CHECK(x.is_contiguous() && y.is_cuda() && y.is_contiguous() && y.scalar_type() == x.scalar_type() &&
                  y.sizes() == x.sizes(),
              "x / y contiguous, same dtype and shape");
  ok(dllm_gelu_erf(x.data_ptr(), y.data_ptr(), f, x.numel(), stream()), "gelu_erf");
}

void conv_state_refill(torch::Tensor x, torch::Tensor state, torch::Tensor qstart, torch::Tensor qlen, torch::Tensor ctx,
                       torch::Tensor rows) {
  const bool f = act_f32(x, "x");
  check_rows2d(x, "x");
  TORCH_CHECK(state.is_cuda() && state.scalar_type() == x.scalar_type() && state.is_contiguous() && state.dim() == 3 &&
                  state.size(2) <= x.size(1) && state.size(1) <= 8,
              "conv state [slots, taps - 1 <= 8, C <= columns of x]");
  auto m = seq_meta(qstart, qlen, ctx, rows, state.size(0));
  ok(dllm_conv_refill(x.data_ptr(), x.stride(0), f, state.data_ptr(), (int)state.size(1), (int)state.size(2), m.qstart, m.qlen,
                      m.ctx, m.rows, m.S, stream()),
     "conv_state_refill");
}

void delta_rule(torch::Tensor qkv, torch::Tensor gba, int64_t H, int64_t G, int64_t d, int64_t dv, torch::Tensor neg_a,
                torch::Tensor dt_bias, torch::Tensor norm_w, double eps, torch::Tensor state, torch::Tensor qstart,
                torch::Tensor qlen, torch::Tensor ctx, torch::Tensor rows, torch::Tensor out) {
  const bool f = act_f32(qkv, "qkv");
  check_rows2d(qkv, "qkv");
  check_rows2d(gba, "gba");
  check_f32(neg_a, "neg_a");
  check_f32(dt_bias, "dt_bias");
  check_f32(norm_w, "norm weight");
  check_f32(state, "state");
  const int64_t T = qkv.size(0);
  TORCH_CHECK(H >= 1 && G >= 1 && H % G == 0 && d >= 1 && d <= 256 && dv >= 1, "heads / kv_heads / dim <= 256 / vdim");
  TORCH_CHECK(qkv.size(1) >= 2 * G * d + H * dv, "qkv [T, 2 G d + H dv]");
  TORCH_CHECK(gba.is_cuda() && gba.scalar_type() == qkv.scalar_type() && gba.size(0) == T && gba.size(1) >= H * dv + 2 * H,
              "gba [T, H dv + 2 H]");
  TORCH_CHECK(neg_a.numel() == H && dt_bias.numel() == H && norm_w.numel() == dv, "per-head constants, norm weight [dv]");
  TORCH_CHECK(state.dim() == 4 && state.is_contiguous() && state.size(1) == H && state.size(2) == dv && state.size(3) == d,
              "state [slots, H, dv, d]");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == qkv.scalar_type() && out.is_contiguous() && out.dim() == 2 &&
                  out.size(0) == T && out.size(1) == H * dv,
              "out [T, H dv]");
  auto m = seq_meta(qstart, qlen, ctx, rows, state.size(0));
  // f32 outputs before the per-head norm: written and read for tokens of live sequences only
  auto raw = torch::empty({T, H, dv}, torch::TensorOptions().dtype(torch::kFloat32).device(qkv.device()));
  ok(dllm_delta_rule(qkv.data_ptr(), qkv.stride(0), gba.data_ptr(), gba.stride(0), f, (int)H, (int)G, (int)d, (int)dv,
                     neg_a.data_ptr<float>(), dt_bias.data_ptr<float>(), norm_w.data_ptr<float>(), (float)eps,
                     state.data_ptr<float>(), m.qstart, m.qlen, m.ctx, m.rows, raw.data_ptr<float>(), out.data_ptr(), m.S,
                     (long)T, stream()),
     "delta_rule");
}

void attn_prep(torch::Tensor proj, int64_t H, int64_t G, int64_t d, int64_t dv, torch::Tensor cos_sin, int64_t rot,
               double eps, torch::Tensor qscale, torch::Tensor pos, torch::Tensor slots, torch::Tensor kc, torch::Tensor vc,
               torch::Tensor q) {
  const bool f = act_f32(proj, "proj");
  check_rows2d(proj, "proj");
  check_f32(cos_sin, "cos_sin");
  check_f32(qscale, "qscale");
  check_i32(pos, "positions");
  check_i32(slots, "slots");
  const int64_t T = proj.size(0);
  TORCH_CHECK(H >= 1 && G >= 1 && H % G == 0 && proj.size(1) >= (H + G) * d + G * dv, "proj [T, (H + G) d + G dv]");
  TORCH_CHECK(cos_sin.dim() == 2 && rot >= 0 && rot % 2 == 0 && rot <= d && (rot == 0 || cos_sin.size(1) >= rot),
              "rotation table");
  TORCH_CHECK(qscale.numel() == H && pos.numel() == T && slots.numel() == T, "qscale / positions / slots lengths");
  for (auto* c : {&kc, &vc})
    TORCH_CHECK(c->is_cuda() && c->scalar_type() == proj.scalar_type() && c->is_contiguous() && c->dim() == 4 &&
                    c->size(1) == G,
                "paged caches K [blocks, G, block, d], V [blocks, G, dv, block] in the activations' dtype");
  TORCH_CHECK(kc.size(3) == d && vc.size(2) == dv && kc.size(0) == vc.size(0) && kc.size(2) == vc.size(3), "cache widths");
  TORCH_CHECK(q.is_cuda() && q.scalar_type() == proj.scalar_type() && q.is_contiguous() && q.numel() == T * H * d, "q [T, H, d]");
  ok(dllm_attn_prep(proj.data_ptr(), proj.stride(0), f, (int)H, (int)G, (int)d, (int)dv, cos_sin.data_ptr<float>(),
                    (int)cos_sin.size(1), (int)rot, (float)eps, qscale.data_ptr<float>(), pos.data_ptr<int>(),
                    slots.data_ptr<int>(), kc.data_ptr(), vc.data_ptr(), q.data_ptr(), (long)T, (int)kc.size(2), stream()),
     "attn_prep");
}

void paged_gqa_attention(torch::Tensor q, torch::Tensor kc, torch::Tensor vc, torch::Tensor bt, torch::Tensor qstart,
                         torch::Tensor qlen, torch::Tensor ctx, torch::Tensor tile_seq, torch::Tensor tile_tok0,
                         c10::optional<torch::Tensor> gate, torch::Tensor out, bool mfma, int64_t splits,
                         c10::optional<torch::Tensor> part, int64_t window, int64_t keep_first, double sink) {
  const bool f = act_f32(q, "q");
  TORCH_CHECK(keep_first >= 0 && sink >= 0.0, "keep_first >= 0, sink >= 0");
  TORCH_CHECK(q.dim() == 3 && q.is_contiguous(), "q [T, H, d]");
  const int64_t T = q.size(0), H = q.size(1), d = q.size(2);
  for (auto* c : {&kc, &vc})
    TORCH_CHECK(c->is_cuda() && c->scalar_type() == q.scalar_type() && c->is_contiguous() && c->dim() == 4,
                "paged caches K [blocks, G, block, d], V [blocks, G, dv, block] in the dtype of q");
  const int64_t G = kc.size(1), dv = vc.size(2);
  const int64_t GV = vc.size(1);      // fewer value heads than key heads: neighbouring key heads share one
  TORCH_CHECK(G >= 1 && H % G == 0 && kc.size(3) == d && GV >= 1 && G % GV == 0 && kc.size(0) == vc.size(0) &&
                  kc.size(2) == vc.size(3) && dv <= 256 && window >= 0,
              "cache shapes; vdim <= 256; window >= 0");
  TORCH_CHECK(!mfma || dllm_gqa_mfma_ok(f, (int)H, (int)G, (int)d, (int)dv, (int)kc.size(2)),
              "shape outside the matrix-core kernel's range");
  check_i32(bt, "block_tables");
  TORCH_CHECK(bt.dim() == 2 && bt.stride(1) == 1, "block_tables [S, blocks]");
  for (auto* t : {&qstart, &qlen, &ctx, &tile_seq, &tile_tok0}) check_i32(*t, "sequence / tile metadata");
  TORCH_CHECK(qlen.numel() == qstart.numel() && ctx.numel() == qstart.numel() && tile_tok0.numel() >= tile_seq.numel() &&
                  bt.size(0) >= qstart.numel(),
              "metadata lengths");
  const void* gp = nullptr;
  long ldg = 0;
  if (gate) {
    check_rows2d(*gate, "gate");
    TORCH_CHECK(gate->is_cuda() && gate->scalar_type() == q.scalar_type() && gate->size(0) == T && gate->size(1) == H * dv,
                "gate [T, H dv]");
    gp = gate->data_ptr();
    ldg = gate->stride(0);
  }
  const bool of32 = out.scalar_type() == torch::kFloat32;
  TORCH_CHECK(out.is_cuda() && (of32 || out.scalar_type() == q.scalar_type()) && out.is_contiguous() && out.dim() == 2 &&
                  out.size(0) == T && out.size(1) == H * dv,
              "out [T, H dv] in the dtype of q or f32");
  float* pptr = nullptr;
  TORCH_CHECK(splits >= 1 && splits <= 64 && (splits == 1 || mfma), "key splits: 1..64, matrix-core kernel only");
  if (splits > 1) {
    TORCH_CHECK(part.has_value(), "key splits need a workspace");
    check_f32(*part, "split workspace");
    TORCH_CHECK(part->numel() >= (int64_t)tile_seq.numel() * G * splits * 64 * (dv + 2), "split workspace size");
    pptr = part->data_ptr<float>();
  }
  const int rc = dllm_paged_gqa(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), f, bt.data_ptr<int>(), (int)bt.stride(0),
                                (int)kc.size(2), qstart.data_ptr<int>(), qlen.data_ptr<int>(), ctx.data_ptr<int>(),
                                tile_seq.data_ptr<int>(), tile_tok0.data_ptr<int>(), (int)tile_seq.numel(), gp, ldg,
                                out.data_ptr(), (int)H, (int)G, (int)d, (int)dv, (int)mfma, (int)splits, pptr, (int)window,
                                (int)GV, (int)of32, (int)keep_first, (float)sink, stream());
  TORCH_CHECK(rc != -2, "head widths do not fit the LDS");
  ok(rc, "paged_gqa_attention");
}

// ---- differential attention, Mamba-2 / mLSTM recurrences, PolyNorm, grouped router (gqa.hip, outer_scan.hip, seqmix.hip)
void qk_norm_prep(torch::Tensor proj, c10::optional<torch::Tensor> bias, int64_t H, int64_t G, int64_t M, int64_t d, int64_t dv,
                  torch::Tensor qw, torch::Tensor kw, torch::Tensor cos_sin, int64_t rot, double eps, double qscale,
                  torch::Tensor pos, torch::Tensor slots, c10::optional<torch::Tensor> kc, c10::optional<torch::Tensor> vc,
                  torch::Tensor q) {
  const bool f = act_f32(proj, "proj");
  check_rows2d(proj, "proj");
  check_f32(cos_sin, "cos_sin");
  check_f32(qw, "q norm weight");
  check_f32(kw, "k norm weight");
  check_i32(pos, "positions");
  check_i32(slots, "slots");
  const int64_t T = proj.size(0);
  const bool own = kc.has_value();
  TORCH_CHECK(own == vc.has_value(), "both caches or none");
  const int64_t cols = H * M * d + (own ? G * M * d + G * dv : 0);
  TORCH_CHECK(H >= 1 && G >= 1 && M >= 1 && H % G == 0 && d >= 1 && dv >= 1 && proj.size(1) >= cols, "proj [T, q | k | v]");
  TORCH_CHECK(cos_sin.dim() == 2 && rot >= 0 && rot % 2 == 0 && rot <= d && (rot == 0 || cos_sin.size(1) >= rot),
              "rotation table");
  TORCH_CHECK(qw.numel() == d && kw.numel() == d && pos.numel() == T && slots.numel() == T, "norm weights / positions / slots");
  const float* bp = nullptr;
  if (bias) {
    check_f32(*bias, "bias");
    TORCH_CHECK(bias->numel() == cols, "bias length");
    bp = bias->data_ptr<float>();
  }
  void *kp = nullptr, *vp = nullptr;
  int bsz = 16;
  if (own) {
    for (auto* c : {&*kc, &*vc})
      TORCH_CHECK(c->is_cuda() && c->scalar_type() == proj.scalar_type() && c->is_contiguous() && c->dim() == 4,
                  "paged caches K [blocks, G M, block, d], V [blocks, G, dv, block] in the activations' dtype");
    TORCH_CHECK(kc->size(1) == G * M && vc->size(1) == G && kc->size(3) == d && vc->size(2) == dv &&
                    kc->size(0) == vc->size(0) && kc->size(2) == vc->size(3),
                "cache shapes");
    kp = kc->data_ptr();
    vp = vc->data_ptr();
    bsz = (int)kc->size(2);
  }
  TORCH_CHECK(q.is_cuda() && q.scalar_type() == proj.scalar_type() && q.is_contiguous() && q.numel() == T * H * M * d,
              "q [T, H M, d]");
  ok(dllm_qk_norm_prep(proj.data_ptr(), proj.stride(0), f, bp, (int)H, (int)G, (int)M, (int)d, (int)dv, qw.data_ptr<float>(),
                       kw.data_ptr<float>(), cos_sin.data_ptr<float>(), (int)cos_sin.size(1), (int)rot, (float)eps,
                       (float)qscale, pos.data_ptr<int>(), slots.data_ptr<int>(), kp, vp, q.data_ptr(), (long)T, bsz, stream()),
     "qk_norm_prep");
}

void diff_combine(torch::Tensor a, int64_t H, int64_t G, int64_t dv, double lam, double eps, double scale, torch::Tensor out) {
  check_f32(a, "a");
  const bool f = act_f32(out, "out");
  TORCH_CHECK(a.dim() == 2 && a.is_contiguous() && H >= 1 && G >= 1 && H % G == 0 && a.size(1) == 2 * H * dv, "a [T, 2 H dv]");
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == a.size(0) && out.size(1) == H * dv, "out [T, H dv]");
  ok(dllm_diff_combine(a.data_ptr<float>(), out.data_ptr(), f, (long)a.size(0), (int)H, (int)G, (int)dv, (float)lam,
                       (float)eps, (float)scale, stream()),
     "diff_combine");
}

void ssd_scan(torch::Tensor xbc, torch::Tensor proj, int64_t dt_col, int64_t H, int64_t dv, int64_t N, int64_t G,
              torch::Tensor dt_bias, torch::Tensor neg_a, torch::Tensor D, torch::Tensor state, torch::Tensor qstart,
              torch::Tensor qlen, torch::Tensor ctx, torch::Tensor rows, torch::Tensor out) {
  const bool f = act_f32(xbc, "xbc");
  check_rows2d(xbc, "xbc");
  check_rows2d(proj, "proj");
  TORCH_CHECK(proj.scalar_type() == xbc.scalar_type() && proj.size(0) == xbc.size(0), "proj: the dtype and rows of xbc");
  for (auto* t : {&dt_bias, &neg_a, &D}) {
    check_f32(*t, "per-head parameter");
    TORCH_CHECK(t->numel() == H, "per-head parameter length");
  }
  check_f32(state, "state");
  check_f32(out, "out");
  TORCH_CHECK(H >= 1 && G >= 1 && H % G == 0 && N >= 1 && dv >= 1 && xbc.size(1) >= H * dv + 2 * G * N, "xbc [T, x | B | C]");
  TORCH_CHECK(dt_col >= 0 && proj.size(1) >= dt_col + H, "step logits outside proj");
  TORCH_CHECK(state.is_contiguous() && state.dim() == 4 && state.size(1) == H && state.size(2) == N && state.size(3) == dv,
              "state [slots, H, N, dv]");
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == xbc.size(0) && out.size(1) == H * dv, "out [T, H dv] f32");
  auto m = seq_meta(qstart, qlen, ctx, rows, state.size(0));
  const int rc = dllm_ssd_scan(xbc.data_ptr(), xbc.stride(0), proj.data_ptr(), proj.stride(0), (int)dt_col, f, (int)H, (int)dv,
                               (int)N, (int)G, dt_bias.data_ptr<float>(), neg_a.data_ptr<float>(), D.data_ptr<float>(),
                               state.data_ptr<float>(), m.qstart, m.qlen, m.ctx, m.rows, m.S, out.data_ptr<float>(), stream());
  TORCH_CHECK(rc != -2, "state size outside the kernel's range");
  ok(rc, "ssd_scan");
}

void mlstm(torch::Tensor proj, int64_t H, int64_t d, int64_t dv, torch::Tensor gate_b, double cap, torch::Tensor state,
           torch::Tensor nm, double eps, torch::Tensor norm_w, torch::Tensor qstart, torch::Tensor qlen, torch::Tensor ctx,
           torch::Tensor rows, torch::Tensor raw, torch::Tensor out) {
  const bool f = act_f32(proj, "proj");
  check_rows2d(proj, "proj");
  check_f32(gate_b, "gate biases");
  check_f32(state, "state");
  check_f32(nm, "normaliser state");
  check_f32(norm_w, "norm weight");
  check_f32(raw, "raw");
  const int64_t T = proj.size(0);
  TORCH_CHECK(H >= 1 && d >= 1 && dv >= 1 && proj.size(1) >= 2 * H * (d + dv + 1), "proj [T, q | k | v | gate | i | f]");
  TORCH_CHECK(gate_b.numel() == 2 * H && norm_w.numel() == H * dv && cap > 0, "gate biases / norm weight / cap");
  TORCH_CHECK(state.is_contiguous() && state.dim() == 4 && state.size(1) == H && state.size(2) == d && state.size(3) == dv,
              "state [slots, H, d, dv]");
  const int64_t ncb = (dv + dllm_outer_scan_cols() - 1) / dllm_outer_scan_cols();
  TORCH_CHECK(nm.is_contiguous() && nm.dim() == 4 && nm.size(0) == state.size(0) && nm.size(1) == H && nm.size(2) == ncb &&
                  nm.size(3) == d + 1,
              "normaliser state [slots, H, column blocks, d + 1]");
  TORCH_CHECK(raw.is_contiguous() && raw.numel() == T * H * dv, "raw [T, H dv] f32");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == proj.scalar_type() && out.is_contiguous() && out.numel() == T * H * dv,
              "out [T, H dv]");
  auto m = seq_meta(qstart, qlen, ctx, rows, state.size(0));
  const int rc = dllm_mlstm(proj.data_ptr(), proj.stride(0), f, (int)H, (int)d, (int)dv, gate_b.data_ptr<float>(), (float)cap,
                            state.data_ptr<float>(), nm.data_ptr<float>(), (int)ncb, (float)eps, norm_w.data_ptr<float>(),
                            m.qstart, m.qlen, m.ctx, m.rows, m.S, (long)T, raw.data_ptr<float>(), out.data_ptr(), stream());
  TORCH_CHECK(rc != -2, "key width outside the kernel's range");
  ok(rc, "mlstm");
}

void gated_group_norm(torch::Tensor y, torch::Tensor z, torch::Tensor w, int64_t groups, double eps, torch::Tensor out) {
  check_f32(y, "y");
  check_f32(w, "w");
  const bool f = act_f32(z, "z");
  check_rows2d(z, "z");
  TORCH_CHECK(y.dim() == 2 && y.is_contiguous() && z.size(0) == y.size(0) && z.size(1) >= y.size(1) && w.numel() == y.size(1) &&
                  groups >= 1 && y.size(1) % groups == 0,
              "y [T, n] f32, z [T, >= n], w [n], n a multiple of groups");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == z.scalar_type() && out.is_contiguous() && out.sizes() == y.sizes(),
              "out [T, n] in the dtype of z");
  ok(dllm_gated_group_norm(y.data_ptr<float>(), z.data_ptr(), z.stride(0), f, w.data_ptr<float>(), out.data_ptr(),
                           (int)y.size(0), (int)y.size(1), (int)groups, (float)eps, stream()),
     "gated_group_norm");
}

void polynorm(torch::Tensor z, torch::Tensor coef, double eps, torch::Tensor y) {
  const bool f = act_f32(z, "z");
  check_rows2d(z, "z");
  check_f32(coef, "coef");
  TORCH_CHECK(coef.numel() == 4, "coef = (a, b, c, e)");
  TORCH_CHECK(y.is_cuda() && y.scalar_type() == z.scalar_type() && y.is_contiguous() && y.sizes() == z.sizes(), "y like z");
  ok(dllm_polynorm(z.data_ptr(), z.stride(0), f, coef.data_ptr<float>(), y.data_ptr(), (long)z.size(0), (int)z.size(1),
                   (float)eps, stream()),
     "polynorm");
}

void group_router(torch::Tensor logits, int64_t top, int64_t count, int64_t keep, torch::Tensor ids, torch::Tensor wts) {
  check_f32(logits, "logits");
  check_i32(ids, "ids");
  check_f32(wts, "wts");
  TORCH_CHECK(logits.dim() == 2 && logits.is_contiguous(), "logits [T, E] contiguous");
  const int64_t T = logits.size(0), E = logits.size(1);
  TORCH_CHECK(E >= 1 && E <= 1024 && count >= 1 && E % count == 0 && keep >= 1 && keep <= count && top >= 1 &&
                  top <= keep * (E / count),
              "experts <= 1024, groups divide the experts, top fits the kept groups");
  TORCH_CHECK(ids.is_contiguous() && wts.is_contiguous() && ids.numel() == T * top && wts.numel() == T * top, "ids / wts [T, top]");
  ok(dllm_group_router(logits.data_ptr<float>(), (int)T, (int)E, (int)top, (int)count, (int)keep, ids.data_ptr<int>(),
                       wts.data_ptr<float>(), stream()),
     "group_router");
}

void swiglu_scale(torch::Tensor gu, torch::Tensor gate, int64_t ff, torch::Tensor y) {
  const bool f = act_f32(gu, "gu");
  check_f32(gate, "gate");
  TORCH_CHECK(gu.dim() == 2 && gu.is_contiguous() && gate.dim() == 2 && gate.is_contiguous() && gate.size(0) == gu.size(0) &&
                  ff >= 1 && gate.size(1) * 2 * ff == gu.size(1),
              "gu [T, E 2 ff] contiguous, gate [T, E]");
  TORCH_CHECK(y.is_cuda() && y.scalar_type() == gu.scalar_type() && y.is_contiguous() && y.dim() == 2 &&
                  y.size(0) == gu.size(0) && y.size(1) * 2 == gu.size(1),
              "y [T, E ff]");
  ok(dllm_swiglu_scale(gu.data_ptr(), f, gate.data_ptr<float>(), (int)gate.size(1), (int)ff, y.data_ptr(), (long)gu.size(0),
                       stream()),
     "swiglu_scale");
}

void route_topk(torch::Tensor logits, int64_t E, int64_t top, int64_t count, int64_t keep, int64_t smode, int64_t gmode,
                c10::optional<torch::Tensor> corr, int64_t real, torch::Tensor ids, torch::Tensor wts, torch::Tensor idw) {
  check_f32(logits, "logits");
  check_i32(ids, "ids");
  check_f32(wts, "wts");
  check_f32(idw, "idw");
  TORCH_CHECK(logits.dim() == 2 && logits.stride(1) == 1 && logits.size(1) >= E, "logits [T, >= E], rows contiguous");
  const int64_t T = logits.size(0);
  TORCH_CHECK(E >= 1 && E <= 1024 && count >= 1 && E % count == 0 && keep >= 1 && keep <= count && top >= 1 &&
                  top <= keep * (E / count) && real >= 0 && real <= E,
              "outputs <= 1024, groups divide the outputs, top fits the kept groups");
  TORCH_CHECK((smode == 0 || smode == 1) && (gmode == 0 || gmode == 1), "score / group score mode");
  TORCH_CHECK(ids.is_contiguous() && wts.is_contiguous() && ids.numel() == T * top && wts.numel() == T * top &&
                  idw.is_contiguous() && idw.numel() == T,
              "ids / wts [T, top], idw [T]");
  const float* cp = nullptr;
  if (corr) {
    check_f32(*corr, "correction");
    TORCH_CHECK(corr->is_contiguous() && corr->numel() == E, "correction [E]");
    cp = corr->data_ptr<float>();
  }
  ok(dllm_route_topk(logits.data_ptr<float>(), (long)logits.stride(0), (int)T, (int)E, (int)top, (int)count, (int)keep,
                     (int)smode, (int)gmode, cp, (int)real, ids.data_ptr<int>(), wts.data_ptr<float>(), idw.data_ptr<float>(),
                     stream()),
     "route_topk");
}

void ls_resadd_ln(torch::Tensor x, torch::Tensor w, torch::Tensor b, double eps, torch::Tensor out,
                  c10::optional<torch::Tensor> y, c10::optional<torch::Tensor> ls, c10::optional<torch::Tensor> bias,
                  c10::optional<torch::Tensor> y2, c10::optional<torch::Tensor> g2, c10::optional<torch::Tensor> h,
                  c10::optional<torch::Tensor> hw) {
  check_f32(x, "x");
  check_f32(w, "w");
  check_f32(b, "b");
  const bool f = act_f32(out, "out");
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous(), "x [T, width] f32 contiguous");
  const int64_t T = x.size(0), H = x.size(1);
  TORCH_CHECK(w.numel() == H && b.numel() == H && w.is_contiguous() && b.is_contiguous(), "norm weight / bias [width]");
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == H, "out [T, width]");
  auto act2d = [&](const torch::Tensor& t, const char* what) {
    check_rows2d(t, what);
    TORCH_CHECK(t.is_cuda() && t.scalar_type() == out.scalar_type() && t.size(0) == T && t.size(1) == H, what,
                ": [T, width] in the dtype of out");
  };
  auto vec = [&](const torch::Tensor& t, const char* what) {
    check_f32(t, what);
    TORCH_CHECK(t.is_contiguous() && t.numel() == H, what, ": [width] f32");
  };
  const void *yp = nullptr, *y2p = nullptr, *hp = nullptr;
  const float *lsp = nullptr, *bp = nullptr, *g2p = nullptr, *hwp = nullptr;
  long ldy = 0, ldy2 = 0, ldg2 = 0, ldh = 0;
  TORCH_CHECK(y.has_value() || !(ls || bias || y2 || g2 || h || hw), "terms without y");
  if (y) { act2d(*y, "y"); yp = y->data_ptr(); ldy = y->stride(0); }
  if (ls) { vec(*ls, "ls"); lsp = ls->data_ptr<float>(); }
  if (bias) { vec(*bias, "bias"); bp = bias->data_ptr<float>(); }
  if (y2) { act2d(*y2, "y2"); y2p = y2->data_ptr(); ldy2 = y2->stride(0); }
  if (g2) {
    check_dev(*g2, "g2");
    TORCH_CHECK(g2->scalar_type() == torch::kFloat32 && y2.has_value() && g2->dim() == 1 && g2->size(0) == T,
                "g2 [T] f32 (may be a column of a matrix), with y2");
    g2p = g2->data_ptr<float>();
    ldg2 = g2->stride(0);
  }
  TORCH_CHECK(h.has_value() == hw.has_value(), "h and hw come together");
  if (h) {
    act2d(*h, "h");
    check_f32(*hw, "hw");
    TORCH_CHECK(hw->is_contiguous() && hw->numel() == T, "hw [T] f32");
    hp = h->data_ptr();
    ldh = h->stride(0);
    hwp = hw->data_ptr<float>();
  }
  const int rc = dllm_ls_resadd_ln(yp, ldy, f, lsp, bp, y2p, ldy2, g2p, ldg2, hp, ldh, hwp, x.data_ptr<float>(),
                                   w.data_ptr<float>(), b.data_ptr<float>(), out.data_ptr(), (long)T, (int)H, (float)eps,
                                   stream());
  ok(rc, "ls_resadd_ln");
}

void glu_act(torch::Tensor gu, c10::optional<torch::Tensor> bias, int64_t mode, double limit, double alpha, torch::Tensor y) {
  const bool f = act_f32(gu, "gu");
  check_rows2d(gu, "gu");
  TORCH_CHECK(gu.size(1) % 2 == 0 && (mode == 0 || mode == 1), "gu [T, 2 ff]; mode 0 or 1");
  const int64_t ff = gu.size(1) / 2;
  TORCH_CHECK(y.is_cuda() && y.scalar_type() == gu.scalar_type() && y.is_contiguous() && y.dim() == 2 &&
                  y.size(0) == gu.size(0) && y.size(1) == ff,
              "y [T, ff]");
  const float* bp = nullptr;
  if (bias) {
    check_f32(*bias, "bias");
    TORCH_CHECK(bias->is_contiguous() && bias->numel() == 2 * ff, "bias [2 ff]");
    bp = bias->data_ptr<float>();
  }
  ok(dllm_glu_act(gu.data_ptr(), gu.stride(0), f, bp, (int)ff, (int)mode, (float)limit, (float)alpha, y.data_ptr(),
                  (long)gu.size(0), stream()),
     "glu_act");
}

void proj_norm_prep(torch::Tensor proj, int64_t H, int64_t G, int64_t d, int64_t dv, torch::Tensor qw, torch::Tensor kw,
                    torch::Tensor cos_sin, int64_t rot, bool interleaved, double eps, torch::Tensor qscale, bool vnorm,
                    torch::Tensor pos, torch::Tensor slots, c10::optional<torch::Tensor> kc, c10::optional<torch::Tensor> vc,
                    torch::Tensor q, c10::optional<torch::Tensor> zero_rows) {
  const bool f = act_f32(proj, "proj");
  check_rows2d(proj, "proj");
  check_f32(cos_sin, "cos_sin");
  check_f32(qw, "q norm weight");
  void* zp = nullptr;
  int zn = 0;
  if (zero_rows) {
    TORCH_CHECK(zero_rows->is_cuda() && zero_rows->scalar_type() == proj.scalar_type() && zero_rows->is_contiguous() &&
                    zero_rows->dim() == 2 && zero_rows->size(0) == proj.size(0),
                "zero_rows [T, n] contiguous in the activations' dtype");
    zp = zero_rows->data_ptr();
    zn = (int)zero_rows->size(1);
  }
  check_f32(kw, "k norm weight");
  check_f32(qscale, "q scale");
  check_i32(pos, "positions");
  check_i32(slots, "slots");
  const int64_t T = proj.size(0);
  const bool own = kc.has_value();
  TORCH_CHECK(own == vc.has_value(), "both caches or none");
  const int64_t cols = H * d + (own ? G * (d + dv) : 0);
  TORCH_CHECK(H >= 1 && G >= 1 && H % G == 0 && d >= 1 && dv >= 1 && proj.size(1) >= cols, "proj [T, q | k | v]");
  TORCH_CHECK(cos_sin.dim() == 2 && cos_sin.is_contiguous() && rot >= 0 && rot % 2 == 0 && rot <= d &&
                  (rot == 0 || cos_sin.size(1) >= rot),
              "rotation table");
  TORCH_CHECK(qw.is_contiguous() && qw.numel() == H * d && (!own || (kw.is_contiguous() && kw.numel() == G * d)) &&
                  qscale.is_contiguous() && qscale.numel() == H && pos.numel() == T && slots.numel() == T,
              "norm weights [H d] / [G d], q scale [H], positions / slots [T]");
  void *kp = nullptr, *vp = nullptr;
  int bsz = 16;
  if (own) {
    for (auto* c : {&*kc, &*vc})
      TORCH_CHECK(c->is_cuda() && c->scalar_type() == proj.scalar_type() && c->is_contiguous() && c->dim() == 4,
                  "paged caches K [blocks, G, block, d], V [blocks, G, dv, block] in the activations' dtype");
    TORCH_CHECK(kc->size(1) == G && vc->size(1) == G && kc->size(3) == d && vc->size(2) == dv && kc->size(0) == vc->size(0) &&
                    kc->size(2) == vc->size(3),
                "cache shapes");
    kp = kc->data_ptr();
    vp = vc->data_ptr();
    bsz = (int)kc->size(2);
  }
  TORCH_CHECK(q.is_cuda() && q.scalar_type() == proj.scalar_type() && q.is_contiguous() && q.numel() == T * H * d, "q [T, H, d]");
  ok(dllm_proj_norm_prep(proj.data_ptr(), proj.stride(0), f, (int)H, (int)G, (int)d, (int)dv, qw.data_ptr<float>(),
                         kw.data_ptr<float>(), cos_sin.data_ptr<float>(), (int)cos_sin.size(1), (int)rot, (int)interleaved,
                         (float)eps, qscale.data_ptr<float>(), (int)vnorm, pos.data_ptr<int>(), slots.data_ptr<int>(), kp, vp,
                         q.data_ptr(), (long)T, bsz, zp, zn, stream()),
     "proj_norm_prep");
}

void softcap(torch::Tensor x, double cap, torch::Tensor y) {
  const bool f = act_f32(x, "x");
  check_f32(y, "y");
  TORCH_CHECK(x.is_contiguous() && y.is_contiguous() && x.numel() == y.numel() && cap > 0, "x / y contiguous, cap > 0");
  ok(dllm_softcap(x.data_ptr(), f, (float)cap, y.data_ptr<float>(), (long)x.numel(), stream()), "softcap");
}

void relu2_scale(torch::Tensor x, c10::optional<torch::Tensor> gate, int64_t ff, torch::Tensor y) {
  const bool f = act_f32(x, "x");
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous() && y.is_cuda() && y.scalar_type() == x.scalar_type() && y.is_contiguous() &&
                  y.sizes() == x.sizes(),
              "x / y contiguous [T, n]");
  const float* gp = nullptr;
  int E = 0;
  if (gate) {
    check_f32(*gate, "gate");
    TORCH_CHECK(gate->dim() == 2 && gate->size(0) == x.size(0) && ff >= 1 && gate->size(1) * ff == x.size(1),
                "gate [T, n / ff]");
    gp = gate->data_ptr<float>();
    E = gate->size(1);
  }
  ok(dllm_relu2_scale(x.data_ptr(), f, gp, E, (int)std::max<int64_t>(ff, 1), y.data_ptr(), x.size(0), (int)x.size(1),
                      stream()),
     "relu2_scale");
}

void dense_gate(torch::Tensor ids, torch::Tensor wts, torch::Tensor g) {
  check_i32(ids, "ids");
  check_f32(wts, "wts");
  check_f32(g, "gate");
  TORCH_CHECK(ids.dim() == 2 && wts.sizes() == ids.sizes() && g.dim() == 2 && g.size(0) == ids.size(0), "ids / wts / gate");
  ok(dllm_dense_gate(ids.data_ptr<int>(), wts.data_ptr<float>(), g.data_ptr<float>(), ids.size(0), (int)ids.size(1),
                     (int)g.size(1), stream()),
     "dense_gate");
}

void latent_kv_write(torch::Tensor ckv, int64_t rank, torch::Tensor w, double eps, torch::Tensor pos,
                     torch::Tensor cos_sin, torch::Tensor slots, torch::Tensor cache) {
  const bool f = act_f32(ckv, "ckv");
  check_rows2d(ckv, "ckv");
  check_f32(w, "norm weight");
  check_f32(cos_sin, "cos_sin");
  check_i32(pos, "positions");
  check_i32(slots, "slots");
  const int T = ckv.size(0);
  const int64_t rot = ckv.size(1) - rank;
  TORCH_CHECK(rank >= 1 && rot >= 0 && rot % 2 == 0 && w.numel() == rank, "latent / rotated widths");
  TORCH_CHECK(cos_sin.dim() == 2 && cos_sin.size(1) >= rot, "rotation table");
  TORCH_CHECK(pos.numel() == T && slots.numel() == T, "positions / slots length");
  TORCH_CHECK(cache.is_cuda() && cache.scalar_type() == ckv.scalar_type() && cache.is_contiguous() && cache.dim() == 3 &&
                  cache.size(1) == 16 && cache.size(2) == rank + rot,
              "cache [blocks, 16, rank + rot] in the dtype of ckv");
  ok(dllm_latent_kv_write(ckv.data_ptr(), ckv.stride(0), f, (int)rank, (int)rot, w.data_ptr<float>(), (float)eps,
                          pos.data_ptr<int>(), cos_sin.data_ptr<float>(), (int)cos_sin.size(1), slots.data_ptr<int>(),
                          cache.data_ptr(), T, stream()),
     "latent_kv_write");
}

void latent_attention(torch::Tensor qa, torch::Tensor q, int64_t dim, int64_t rot, torch::Tensor pos, torch::Tensor cos_sin,
                      torch::Tensor cache, torch::Tensor bt, torch::Tensor qstart, torch::Tensor qlen, torch::Tensor ctx,
                      torch::Tensor tile_seq, torch::Tensor tile_tok0, double scale, torch::Tensor out, int64_t splits,
                      c10::optional<torch::Tensor> part_o, c10::optional<torch::Tensor> part_ml, bool mfma,
                      int64_t rows) {
  const bool f = act_f32(qa, "qa");
  TORCH_CHECK(rows == 16 || (rows == 32 && mfma && !f && dllm_latent_mfma_ok((int)qa.size(2), (int)rot, 32)),
              "rows per workgroup: 16, or 32 where the matrix-core kernel takes the shape");
  TORCH_CHECK(qa.dim() == 3 && qa.is_contiguous(), "qa [H, T, rank] contiguous");
  const int64_t H = qa.size(0), T = qa.size(1), rank = qa.size(2);
  TORCH_CHECK(q.is_cuda() && q.scalar_type() == qa.scalar_type(), "q dtype");
  check_rows2d(q, "q");
  TORCH_CHECK(q.size(0) == T && q.size(1) >= H * (dim + rot), "q [T, H (dim + rot)]");
  check_f32(cos_sin, "cos_sin");
  check_i32(pos, "positions");
  for (auto* t : {&bt, &qstart, &qlen, &ctx, &tile_seq, &tile_tok0}) check_i32(*t, "attention metadata");
  TORCH_CHECK(cos_sin.dim() == 2 && rot >= 0 && rot % 2 == 0 && cos_sin.size(1) >= rot, "rotation table");
  TORCH_CHECK(cache.is_cuda() && cache.scalar_type() == qa.scalar_type() && cache.is_contiguous() && cache.dim() == 3 &&
                  cache.size(1) == 16 && cache.size(2) == rank + rot,
              "cache [blocks, 16, rank + rot]");
  TORCH_CHECK(bt.dim() == 2 && qstart.numel() == bt.size(0) && qlen.numel() == bt.size(0) && ctx.numel() == bt.size(0),
              "block tables [S, max_blocks] and per-sequence metadata");
  TORCH_CHECK(tile_tok0.numel() == tile_seq.numel(), "tile tables");
  TORCH_CHECK(rank <= 512, "latent rank <= 512");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == qa.scalar_type() && out.is_contiguous() && out.sizes() == qa.sizes(),
              "out like qa");
  float *po = nullptr, *pml = nullptr;
  TORCH_CHECK(splits >= 1 && splits <= 64, "splits in [1, 64]");
  if (splits > 1) {
    TORCH_CHECK(part_o && part_ml, "split partial buffers");
    check_f32(*part_o, "part_o");
    check_f32(*part_ml, "part_ml");
    const int64_t gx = ((H >= rows ? 1 : rows / H) * H + rows - 1) / rows, prow = tile_seq.numel() * gx * rows * splits;
    TORCH_CHECK(part_o->numel() >= prow * rank && part_ml->numel() >= prow * 2, "split partial buffers too small");
    po = part_o->data_ptr<float>();
    pml = part_ml->data_ptr<float>();
  }
  ok(dllm_latent_attention(qa.data_ptr(), q.data_ptr(), q.stride(0), f, (int)H, (int)dim, (int)rot, (int)rank, T,
                           cos_sin.data_ptr<float>(), (int)cos_sin.size(1), cache.data_ptr(), bt.data_ptr<int>(),
                           (int)bt.size(1), qstart.data_ptr<int>(), qlen.data_ptr<int>(), ctx.data_ptr<int>(),
                           tile_seq.data_ptr<int>(), tile_tok0.data_ptr<int>(), (int)tile_seq.numel(), (float)scale,
                           out.data_ptr(), (int)splits, po, pml, mfma ? 1 : 0, (int)rows, stream()),
     "latent_attention");
}
}  // namespace

PYBIND11_MODULE(_hip_kernels, m) {
  m.def("rms_rows", &rms_rows, py::arg("x"), py::arg("w"), py::arg("y"), py::arg("eps"), py::arg("groups") = 1);
  m.def("norm_resadd", &norm_resadd, py::arg("y"), py::arg("w"), py::arg("eps"), py::arg("x"), py::arg("x_lp"),
        py::arg("groups") = 1, py::arg("bias") = py::none());
  m.def("polynorm", &polynorm);
  m.def("group_router", &group_router);
  m.def("swiglu_scale", &swiglu_scale);
  m.def("route_topk", &route_topk);
  m.def("ls_resadd_ln", &ls_resadd_ln);
  m.def("glu_act", &glu_act);
  m.def("proj_norm_prep", &proj_norm_prep, py::arg("proj"), py::arg("heads"), py::arg("kv_heads"), py::arg("dim"), py::arg("vdim"),
        py::arg("qw"), py::arg("kw"), py::arg("cos_sin"), py::arg("rot"), py::arg("interleaved"), py::arg("eps"), py::arg("qscale"),
        py::arg("vnorm"), py::arg("pos"), py::arg("slots"), py::arg("k_cache"), py::arg("v_cache"), py::arg("q"),
        py::arg("zero_rows") = py::none());
  m.def("softcap", &softcap);
  m.def("gated_group_norm", &gated_group_norm);
  m.def("outer_scan_cols", []() { return dllm_outer_scan_cols(); });
  m.def("ssd_scan", &ssd_scan);
  m.def("mlstm", &mlstm);
  m.def("qk_norm_prep", &qk_norm_prep);
  m.def("diff_combine", &diff_combine);
  m.def("causal_conv_silu", &causal_conv_silu, py::arg("x"), py::arg("w"), py::arg("b"), py::arg("state"), py::arg("qstart"),
        py::arg("qlen"), py::arg("ctx"), py::arg("rows"), py::arg("y"), py::arg("refill") = false, py::arg("act") = 0);
  m.def("selective_scan", &selective_scan);
  m.def("retention", &retention, py::arg("qkvg"), py::arg("heads"), py::arg("dim"), py::arg("vdim"), py::arg("cos_sin"),
        py::arg("rot"), py::arg("decay"), py::arg("state"), py::arg("eps"), py::arg("positions"), py::arg("qstart"),
        py::arg("qlen"), py::arg("ctx"), py::arg("rows"), py::arg("out"), py::arg("raw") = py::none());
  m.def("relu2_scale", &relu2_scale);
  m.def("dense_gate", &dense_gate);
  m.def("lightning_attention", &lightning_attention);
  m.def("resadd_norm", &resadd_norm, py::arg("a"), py::arg("b"), py::arg("wa"), py::arg("wb"), py::arg("w_post"),
        py::arg("eps"), py::arg("x"), py::arg("w_next"), py::arg("x_next"), py::arg("stack") = py::none(),
        py::arg("depth_w") = py::none(), py::arg("depth_n") = 0);
  m.def("depth_mix", &depth_mix);
  m.def("gelu_erf", &gelu_erf);
  m.def("conv_state_refill", &conv_state_refill);
  m.def("delta_rule", &delta_rule);
  m.def("attn_prep", &attn_prep);
  m.def("paged_gqa_attention", &paged_gqa_attention, py::arg("q"), py::arg("k_cache"), py::arg("v_cache"),
        py::arg("block_tables"), py::arg("qstart"), py::arg("qlen"), py::arg("ctx"), py::arg("tile_seq"),
        py::arg("tile_tok0"), py::arg("gate"), py::arg("out"), py::arg("mfma"), py::arg("splits") = 1,
        py::arg("part") = py::none(), py::arg("window") = 0, py::arg("keep_first") = 0, py::arg("sink") = 0.0);
  m.def("gqa_tile_tokens",
        [](int64_t H, int64_t G, bool mfma) { return (int64_t)dllm_gqa_tile_tokens((int)H, (int)G, (int)mfma); });
  m.def("gqa_mfma_ok", [](bool f32, int64_t H, int64_t G, int64_t d, int64_t dv, int64_t bs) {
    return (bool)dllm_gqa_mfma_ok((int)f32, (int)H, (int)G, (int)d, (int)dv, (int)bs);
  });
  m.def("latent_kv_write", &latent_kv_write);
  m.def("latent_attention", &latent_attention, py::arg("qa"), py::arg("q"), py::arg("dim"), py::arg("rot"),
        py::arg("positions"), py::arg("cos_sin"), py::arg("cache"), py::arg("block_tables"), py::arg("qstart"),
        py::arg("qlen"), py::arg("ctx"), py::arg("tile_seq"), py::arg("tile_tok0"), py::arg("scale"), py::arg("out"),
        py::arg("splits") = 1, py::arg("part_o") = py::none(), py::arg("part_ml") = py::none(), py::arg("mfma") = true,
        py::arg("rows") = 16);
  m.def("latent_mfma_ok", [](int64_t rank, int64_t rot, int64_t rows) { return dllm_latent_mfma_ok((int)rank, (int)rot, (int)rows) != 0; });
  m.def("encoder_attention", &encoder_attention);
  m.def("embed_ln", &embed_ln);
  m.def("moe_ffn", &moe_ffn, py::arg("x"), py::arg("ids"), py::arg("wts"), py::arg("w13"), py::arg("w2"), py::arg("out"),
        py::arg("act_mode") = 0);
  m.def("moe_ffn_tg", &moe_ffn_tg);
  m.def("tgemm", &tgemm);
  m.def("res_add_ssq", &res_add_ssq);
  m.def("qkv_post", &qkv_post, py::arg("y"), py::arg("ssq"), py::arg("ssq_n"), py::arg("scale"), py::arg("eps"),
        py::arg("pos"), py::arg("cos_sin"), py::arg("slots"), py::arg("q_out"), py::arg("kc"), py::arg("vc"),
        py::arg("nq"), py::arg("nkv"), py::arg("d"), py::arg("v_rows") = py::none());
  m.def("swiglu_post", &swiglu_post);
  m.def("car_alloc", &car_alloc);
  m.def("car_handle", &car_handle);
  m.def("car_open", &car_open);
  m.def("car_close", &car_close);
  m.def("car_free", &car_free);
  m.def("car_allreduce", &car_allreduce);
  m.def("car_vote", &car_vote);
  m.def("car_resadd", &car_resadd);
  m.def("car_resadd_slots", &car_resadd_slots);
  m.def("car_allgather", &car_allgather);
  m.doc() = "gfx950 HIP kernels for distributed_llm_amd";
  m.def("norm", &norm);
  m.def("rope_kv", &rope_kv);
  m.def("kv_write", &kv_write);
  m.def("paged_attention", &paged_attention);
  m.def("flash_prefill", &flash_prefill, py::arg("q"), py::arg("kc"), py::arg("vc"), py::arg("block_tables"),
        py::arg("qstart"), py::arg("qlen"), py::arg("ctx"), py::arg("tile_seq"), py::arg("tile_tok0"), py::arg("out"),
        py::arg("causal"), py::arg("scale"), py::arg("splits") = 1, py::arg("part_o") = py::none(),
        py::arg("part_ml") = py::none(), py::arg("counters") = py::none());
  m.def("silu_mul", &silu_mul);
  m.def("embed", &embed, py::arg("ids"), py::arg("table"), py::arg("out"), py::arg("lo"), py::arg("ssq") = py::none(),
        py::arg("sc_dst") = py::none(), py::arg("sc_buf") = py::none());
  m.def("gelu", &gelu);
  m.def("mean_pool_l2", &mean_pool_l2);
  m.def("moe_gate", &moe_gate);
  m.def("moe_router", &moe_router, py::arg("x"), py::arg("wg"), py::arg("k"), py::arg("ids"), py::arg("w"),
        py::arg("logits") = py::none());
  m.def("argmax", &argmax);
  m.def("scatter_pairs", &scatter_pairs);
  m.def("step_fetch", &step_fetch);
  m.def("step_store", &step_store);
  m.def("sample_topp", &sample_topp);
  m.def("sample_rows", &sample_rows);
  m.def("sample_split", &sample_split);
  m.def("sample_split_maxp", &sample_split_maxp);
  m.def("sample_split_kmax", &sample_split_kmax);
  m.def("tp_cands_k", &tp_cands_k);
  m.def("tp_cands", &tp_cands);
  m.def("tp_sample", &tp_sample);
  m.def("cosine_scores", &cosine_scores);
  m.def("cache_scan", &cache_scan);
  m.def("cache_write", &cache_write);
  m.def("skinny_gemm", &skinny_gemm);
  m.def("skinny_epi", &skinny_epi);
  m.def("gemv", &gemv);
  m.def("gemv_norm", &gemv_norm);
  m.def("gemv_slots", &gemv_slots);
  m.def("gemv_set_grid", &gemv_set_grid);
  m.def("gemv_resadd", &gemv_resadd);
  m.def("gemv_qkv", &gemv_qkv);
  m.def("gemv_swiglu", &gemv_swiglu);
}
