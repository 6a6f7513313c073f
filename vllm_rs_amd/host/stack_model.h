// stack_model.h — a decoder described by a LIST OF LAYERS instead of one fixed block: every layer names its mixer (attention with its own
// head counts, score scale, soft cap, query temperature, optionally reading another layer's keys and values) and its feed-forward
// (none, dense with a PolyNorm activation, or a mixture of clamped gated experts with a sigmoid router and a gated shared expert);
// layers are parallel blocks  x <- x + m * (mixer(h) + ff(h)),  h = grouped RMS norm of x;  positions enter as a sinusoidal vector added
// to the embedding.  The Ditilix design is such a list (vllm_rs_amd/checkpoint.py turns its config.json into the spec text below).
//
// Precision: the residual stream, norms, router, attention scores and weights are f32; projections, the cache and activations are
// bf16 (f32 accumulation) or, for a VRA_F32 model, f32 throughout.
//
// Spec text, one record per line, `key=value` fields:
//   stack width=.. vocab=.. eps=.. groups=.. residual_mult=.. logit_scale=.. pos_base=..
//   layer heads=.. kv_heads=.. dim=.. vdim=.. scale=.. softcap=.. temp_coef=.. temp_every=.. kv_from=.. mlp=none|dense|moe ff=..
//         experts=.. top=.. limit=.. shared_ff=.. shared_limit=..
#pragma once
#include <map>
#include <string>
#include <vector>

#include "model_base.h"

namespace vra {

struct StackLayer {
  // mixer
  int heads = 0, kv_heads = 0, dim = 0, vdim = 0, temp_every = 0, kv_from = -1;
  float scale = 1.f, softcap = 0.f, temp_coef = 0.f;
  // feed-forward: 0 none, 1 dense (PolyNorm), 2 mixture of experts
  int mlp = 0, ff = 0, experts = 0, top = 0, shared_ff = 0;
  float limit = 0.f, shared_limit = 0.f;
  // derived
  int cache = -1;          // index of the paged cache this layer reads (its own, or the one of layer kv_from)
  bool owns_cache = false;
  int ffp = 0, sffp = 0;   // expert / shared widths rounded up to 16 (zero rows and columns)
  int nq() const { return heads * dim; }
  int nk() const { return kv_heads * dim; }
  int nv() const { return kv_heads * vdim; }
  int nqkv() const { return nq() + (owns_cache ? nk() + nv() : 0); }
  // device weights
  float* norm_w = nullptr;
  void* qkv = nullptr;     // [nq (+ nk + nv), width]
  void* o = nullptr;       // [width, heads * vdim]
  void* up = nullptr;      // dense [ff, width]
  void* down = nullptr;    // dense [width, ff]
  float* act = nullptr;    // PolyNorm a, b, c, e
  void* router = nullptr;  // [experts (+ 1: the shared expert's gate), width]
  void* e_gu = nullptr;    // [experts][2 * ffp][width], gate / up rows interleaved in blocks of 16
  void* e_down = nullptr;  // [experts][width][ffp]
  void* s_gu = nullptr;    // [2 * sffp][width]
  void* s_down = nullptr;  // [width][sffp]
};

class StackModel : public ModelBase {
 public:
  StackModel(const vra_model_config& mc, const vra_engine_config& ec, const char* spec);
  ~StackModel() override;
  bool init_synthetic(uint64_t seed) override;
  bool load_tensor(const std::string& name, const void* host, const int64_t* shape, int ndim, int elem_bytes) override;
  bool finalize_weights() override;
  bool init_kv_cache(int num_blocks) override;
  int num_blocks() const override { return num_blocks_; }
  int kv_layers() const override { return (int)kc_.size(); }
  size_t k_block_bytes(int c) const override;
  size_t v_block_bytes(int c) const override;
  void* k_cache(int c) const override { return kc_[c]; }
  void* v_cache(int c) const override { return vc_[c]; }
  int64_t kv_bytes_per_block() const override;
  bool init_buffers(int max_tokens, int max_seqs) override;
  int max_logit_rows() const override { return logit_rows_cap_; }
  void set_comm(void*) override {}
  bool has_comm() const override { return false; }
  int world() const override { return 1; }
  bool forward(const InputMetadata& md, int64_t stream, uint32_t* tokens = nullptr) override;
  float* logits() const override { return logits_; }
  size_t weight_bytes() const override { return weight_bytes_; }
  void set_layer_trace(bool on) override { trace_on_ = on; }
  int64_t read_layer_trace(void* host, int64_t max_bytes, int64_t stream) override;
  const std::vector<StackLayer>& layers() const { return layers_; }

 private:
  struct HostTensor {
    std::vector<uint8_t> data;
    std::vector<int64_t> shape;
    int elem_bytes = 0;
  };
  void* dalloc(size_t bytes);
  void* upload(const void* host, size_t bytes);
  bool need(const std::string& name, int64_t d0, int64_t d1, const HostTensor** out);
  float* upload_f32(const HostTensor& t);
  bool parse_spec(const char* spec);
  bool feed_forward(const StackLayer& L, int T, int64_t stream);
  bool expert_pair(const void* a, int lda, const void* w_gu, int64_t gu_stride, const void* w_down, int64_t down_stride, int rows, int fp, int f,
                   float limit, const int* tile_group, int granule, const int* a_row, const float* a_scale, const int* out_row, float* out,
                   int64_t stream);
  vra_model_config mc_;
  vra_engine_config ec_;
  std::string spec_error_;
  int dt_ = 0;
  size_t es_ = 2;
  int width_ = 0, vocab_ = 0, groups_ = 1;
  float eps_ = 1e-6f, residual_mult_ = 1.f, logit_scale_ = 1.f;
  double pos_base_ = 10000.0;
  std::vector<StackLayer> layers_;
  std::map<std::string, HostTensor> staged_;
  bool finalized_ = false;
  std::vector<void*> allocs_;
  size_t weight_bytes_ = 0;
  void* embed_ = nullptr;
  void* head_ = nullptr;
  float* final_norm_ = nullptr;
  float* inv_freq_ = nullptr;
  // paged caches of the layers that own one: K [blocks * BS, kv_heads * dim], V [blocks * BS, kv_heads * vdim]
  std::vector<void*> kc_, vc_;
  std::vector<int> cache_layer_;
  int num_blocks_ = 0;
  // activations
  int max_tokens_ = 0, max_seqs_ = 0, logit_rows_cap_ = 0, max_rows_ = 0;
  float *x_ = nullptr, *o_ = nullptr, *z_ = nullptr, *pair_out_ = nullptr, *sh_ = nullptr, *xl_ = nullptr, *logits_ = nullptr;
  void *h_ = nullptr, *qkv_ = nullptr, *attn_ = nullptr, *act_ = nullptr, *hl_ = nullptr;
  int *pair_expert_ = nullptr, *row_token_ = nullptr, *row_pair_ = nullptr, *tile_group_ = nullptr;
  float *pair_weight_ = nullptr, *row_scale_ = nullptr, *gate_ = nullptr;
  bool trace_on_ = false;
  float* trace_ = nullptr;
  size_t trace_cap_ = 0, trace_bytes_ = 0;
};

}  // namespace vra
