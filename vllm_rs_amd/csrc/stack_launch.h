// stack_launch.h — internal entry points of stack_ops.hip: the operators of config-driven layer stacks (host/stack_model.cpp).
// Element type `dtype`: VRA_BF16 (16-bit storage, f32 accumulation; norms, routers, attention scores and weights and the residual stay f32) or
// VRA_F32 (everything in 32-bit, no reduced-precision matrix mode).  All pointers are device pointers; launches are asynchronous
// on `stream` and graph-capturable (no allocation, no synchronisation, no memset nodes).
#pragma once
#include <stdint.h>

// out[r', n] = alpha * sum_k A[row(r), k] * scale(r) * W_g[n, k]  for logical rows r < M ("NT" GEMM, weights stored [N, K]).
// Grouped form: the logical rows are cut into granules of `granule` rows, granule t uses the weights of group tile_group[t]
// (w + group * w_group_stride elements; -1 = an empty granule).  a_row gathers (logical row -> row of A, -1 = no row),
// a_scale multiplies the gathered row (bf16: the product is rounded to bf16 before the matrix product), out_row scatters
// (logical row -> row of out, -1 = not written).  Null pointers = identity / one group.
// epi 0: plain.  epi 1: gated pair — W holds gate and up rows interleaved in blocks of 16 (block 2b = gate rows 16b.., block 2b+1 =
// up rows 16b..), N counts both; out gets N/2 columns of  g' * sigmoid(act_alpha * g') * (u' + 1),  g' = min(g, limit),
// u' = clamp(u, -limit, limit)  (limit <= 0: no clamp).
struct StkGemmArgs {
  const void* a = nullptr;
  int lda = 0;
  const void* w = nullptr;
  int64_t w_group_stride = 0;
  void* out = nullptr;
  int ldo = 0;
  int out_f32 = 0;
  int M = 0, N = 0, K = 0;
  float alpha = 1.f;
  const int* tile_group = nullptr;
  int granule = 0;
  const int* a_row = nullptr;
  const float* a_scale = nullptr;
  const int* out_row = nullptr;
  int epi = 0;
  float limit = 0.f, act_alpha = 1.702f;
};
void vra_stack_gemm(const StkGemmArgs& g, int dtype, int64_t stream);
// rows per granule the grouped launches of an M-row problem over `groups` groups want (16 or 64)
int vra_stack_gemm_granule(int rows, int groups);

// x[t, c] = embed[ids[t], c] + pe(positions[t], c),  pe(p, 2i) = sin(p * inv_freq[i]),  pe(p, 2i+1) = cos(p * inv_freq[i])  (f32)
void vra_stack_embed_sinpos(const uint32_t* ids, const int64_t* positions, const void* embed, const float* inv_freq, float* x, int T, int W, int V,
                            int dtype, int64_t stream);

// RMS norm in `groups` equal consecutive parts: h = x / sqrt(mean_part(x^2) + eps) * w   (x, w f32; h in dtype).
// Router (router_w != null, [n_router (+1 when gate_row), W] in dtype): z = router_w . h in f32 on the unrounded h; the `top` largest of the
// first n_router give pair_expert / pair_weight [T, top] (weight = sigmoid(z), not renormalised; ties: the lower index); with
// gate_row the last row gives gate_out[t] = sigmoid(z_last).
struct StkNormArgs {
  const float* x = nullptr;
  const float* w = nullptr;
  void* h = nullptr;
  int T = 0, W = 0, groups = 1;
  float eps = 1e-6f;
  const void* router_w = nullptr;
  int n_router = 0, top = 0, gate_row = 0;
  int* pair_expert = nullptr;
  float* pair_weight = nullptr;
  float* gate_out = nullptr;
};
void vra_stack_group_norm(const StkNormArgs& a, int dtype, int64_t stream);

// Token-expert pairs -> granule-padded rows sorted by expert: row_token / row_scale / row_pair [max_rows] (-1 / 0 in padding rows),
// tile_group [max_rows / granule].  max_rows >= P + n_groups * granule rounded up to the granule.
void vra_stack_moe_sort(const int* pair_expert, const float* pair_weight, int P, int top, int n_groups, int granule, int max_rows, int* row_token,
                        float* row_scale, int* row_pair, int* tile_group, int64_t stream);

// the gated pair of epi 1 on an f32 [M, 2 * F] matrix whose column blocks of 16 alternate gate / up -> out [M, F] in dtype
void vra_stack_gated_act(const float* gu, void* out, int M, int F, float limit, float act_alpha, int dtype, int64_t stream);

// PolyNorm: out = a N(z) + b N(z^2) + c N(z^3) + e,  N(v) = v / sqrt(mean(v^2) + eps) over a token's F values; coef = {a, b, c, e} (device, f32)
void vra_stack_polynorm(const float* z, void* out, const float* coef, int M, int F, float eps, int dtype, int64_t stream);

// x[t] += mult * (o[t] + sum_{j < n1} p1[t * n1 + j] + gate[t] * p2[t])     (all f32 [*, W]; null pointers drop their term; gate null = 1)
void vra_stack_residual_combine(float* x, const float* o, const float* p1, int n1, const float* p2, const float* gate, float mult, int T, int W,
                                int64_t stream);

// k / v rows of a step -> the paged cache of their layer: K [slots, G * dim], V [slots, G * vdim]; slot < 0: nothing written
void vra_stack_kv_store(const void* k, const void* v, int ld, void* kc, void* vc, const int64_t* slots, int T, int kdim, int vdim, int dtype,
                        int64_t stream);

// Causal softmax attention over the paged cache, scores and weights in f32:
//   s(i, j) = (q_i . k_j) * temp(p_i) * scale,  temp(p) = 1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)  (temp_every <= 0: 1),
//   s <- softcap * tanh(s / softcap) (softcap > 0),  key j visible iff j <= p_i.
// q [T, ldq] (head h at column h * dim), out [T, H * vdim]; query head h reads kv head h / (H / G).
struct StkAttnArgs {
  const void* q = nullptr;
  int ldq = 0;
  void* out = nullptr;
  const void* kc = nullptr;
  const void* vc = nullptr;
  const int64_t* positions = nullptr;
  const uint32_t* block_tables = nullptr;
  const uint32_t* context_lens = nullptr;
  const uint32_t* cu_q = nullptr;  // prefill form: [B + 1]; null: decode form, one token per sequence
  int B = 0, T = 0, max_q = 1, H = 0, G = 0, dim = 0, vdim = 0, BS = 64, max_blocks = 0;
  float scale = 1.f, softcap = 0.f, temp_coef = 0.f;
  int temp_every = 0;
};
void vra_stack_attention(const StkAttnArgs& a, int dtype, int64_t stream);

// rows of a [*, W] f32 matrix picked by index -> dst (f32)
void vra_stack_gather_rows_f32(const float* src, const uint32_t* rows, float* dst, int n, int W, int64_t stream);
