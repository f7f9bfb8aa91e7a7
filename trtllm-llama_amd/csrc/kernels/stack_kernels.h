// Host-side launch interface of the kernels behind the ragged-batch stack engine (runtime/stack_engine.cpp): decoder
// stacks whose layers are described at run time (grouped RMS norms, gated residuals, looped layer ranges, differential
// attention over a paged cache, HGRN2 recurrences over per-sequence state slots).
//
// A step is one packed batch of `tokens` rows: portions of prompts and single decoded tokens of several sequences side
// by side.  Row t belongs to batch entry tok_entry[t] and sits at position tok_pos[t] of its sequence.  Every kernel is
// built for two element types: DT_BF16 (activations, weights and caches in bfloat16; what a recurrence, a norm, a
// softmax or the residual touches in fp32) and DT_FLOAT (everything in fp32, plain FMA, no reduced-precision matrix
// mode).  Same conventions as kernels.h: enqueue on `stream`, never synchronise, 0 on success, negative + set_error on a
// shape that cannot run.
#pragma once
#include "kernels.h"

namespace tllm
{
namespace kernels
{

constexpr int32_t DT_BF16 = 7; // nvinfer1::DataType::kBF16

// ---------------------------------------------------------------------------------------------
// Dense product C[m,n] = sum_k A[m,k] * W[n,k] for the stack engine, with the layer's seam in the epilogue.
//   dtype DT_BF16: MFMA tiles (gemm_mfma.hip, v_mfma_f32_32x32x16_bf16) for M > 8, the streaming skinny kernel below it;
//   dtype DT_FLOAT: fp32 FMA tiles (stack_gemm.hip).
// Epilogue, when `resid` is set: resid[m, n] += sigmoid(gate[m, n] + gate_bias[n]) * C[m, n]  (fp32 residual stream, the
// sublayer's gate taken from another projection's columns); nothing is written to `c` then.
// ---------------------------------------------------------------------------------------------
struct StackGemmParams
{
    int32_t dtype = DT_BF16;     // element type of a, w (and of c unless out_f32)
    int32_t out_f32 = 0;         // c is fp32 (logits)
    int32_t M = 0, N = 0, K = 0;
    const void* a = nullptr;
    int64_t lda = 0;             // elements
    const void* w = nullptr;     // [N, K] row-major, K contiguous
    void* c = nullptr;
    int64_t ldc = 0;
    float* resid = nullptr;      // fp32 [M, ldr]
    int64_t ldr = 0;
    const void* gate = nullptr;  // element type `dtype`, [M, ldg]: pre-activation of the gate (null: plain accumulate into resid)
    int64_t ldg = 0;
    const float* gate_bias = nullptr; // fp32 [N] or null
};
int launch_stack_gemm(const StackGemmParams& p, hipStream_t stream);

// ---------------------------------------------------------------------------------------------
// Pointwise pieces.
// ---------------------------------------------------------------------------------------------
// x[t, :] = table[ids[t], :] * scale (fp32 residual stream); keep (optional) receives the same rows
int launch_stack_embed(float* x, float* keep, const int32_t* ids, const void* table, int32_t dtype, int32_t tokens, int32_t width,
    int32_t vocab, float scale, hipStream_t stream);
// x[t, :] += (add ? add[t, :] : 0) + (row ? row[:] : 0): the entry of a pass over a looped layer range
int launch_stack_pass_entry(float* x, const float* add, const float* row, int32_t tokens, int32_t width, hipStream_t stream);
// RMS norm in `groups` equal consecutive parts of the row, every part divided by its own sqrt(mean(part^2) + eps); the two
// outputs share the normalised row and differ in their weights (the parallel layer's two norms of the same x).  rows: optional
// gather (row r reads x[rows[r]]).  y2 / w2 may be null.
int launch_stack_group_rmsnorm(void* y1, void* y2, const float* x, const int32_t* rows, const float* w1, const float* w2, int32_t dtype,
    int32_t n_rows, int32_t width, int32_t groups, float eps, hipStream_t stream);
// y[t, c] = gelu_tanh(gu[t, c]) * gu[t, ff + c] over a [tokens, ld] projection that holds gate then up columns
int launch_stack_gelu_gate(void* y, const void* gu, int32_t dtype, int32_t tokens, int32_t ff, int64_t ld, hipStream_t stream);

// ---------------------------------------------------------------------------------------------
// Rotary positions: pair (2i, 2i + 1) of the first `dims` dimensions of every map of every head, angle = pos * freq[i]
// (fp32), cos / sin scaled by `mscale`; freq carries whatever frequency scaling the model uses (host: stack_rope_freqs).
// Paged cache of one attention layer: K pool [blocks, kv_heads * maps, page, dim], V pool [blocks, kv_heads, vdim, page] (values
// channel-major inside a page: the MFMA kernel reads V^T rows).
// ---------------------------------------------------------------------------------------------
struct StackAttnParams
{
    int32_t dtype = DT_BF16;
    int32_t tokens = 0, entries = 0;
    int32_t heads = 0, kv_heads = 0, maps = 1, dim = 0, vdim = 0;
    int32_t rot_dims = 0;
    const float* freq = nullptr; // fp32 [rot_dims / 2], device
    float mscale = 1.f;
    float scale = 1.f, softcap = 0.f; // score = softcap * tanh(q.k * scale / softcap) when softcap > 0
    // maps == 2: o = a1 - lambda * a2; head_norm: o /= sqrt(mean(o^2) + eps) over vdim, then * out_scale
    float lambda = 0.f, out_scale = 1.f, eps = 1e-5f;
    int32_t head_norm = 0;
    const void* proj = nullptr; // [tokens, ldp]: q rows (heads * maps * dim), k rows (kv_heads * maps * dim), v rows (kv_heads * vdim)
    int64_t ldp = 0;
    void* q = nullptr;          // scratch [tokens, heads * maps * dim]: rotated queries
    void* k_pool = nullptr;
    void* v_pool = nullptr;
    int32_t page = 64, max_blocks = 0;
    const int32_t* block_table = nullptr; // [entries, max_blocks]
    const int32_t* tok_entry = nullptr;   // [tokens]
    const int32_t* tok_pos = nullptr;     // [tokens]
    const int32_t* ent_first = nullptr;   // [entries] first row of the entry in the packed batch
    const int32_t* ent_count = nullptr;   // [entries] rows of the entry
    const int32_t* ent_pos0 = nullptr;    // [entries] position of its first row
    int32_t max_count = 0;                // host: the largest ent_count of the step
    int32_t max_context = 0;              // host: the largest pos0 + count of the step
    void* out = nullptr;                  // [tokens, heads * vdim]
    float* split_ws = nullptr;            // decoding steps: partials of the cross-workgroup key split (stack_attn_workspace_floats); null: no split
};
// rotates q and k, appends k and v of the step's rows to the paged cache
int launch_stack_rope_kv(const StackAttnParams& p, hipStream_t stream);
// causal attention of the step's rows over their sequences' cache (which already holds the step's own keys)
int launch_stack_attention(const StackAttnParams& p, hipStream_t stream);
size_t stack_attn_workspace_floats(int32_t heads, int32_t maps, int32_t vdim); // floats of split_ws a layer of this shape needs
// frequencies of the rotation with YaRN-style scaling (factor <= 0: none): fills freq[dims / 2], returns the cos / sin multiplier
float stack_rope_freqs(float* freq, int32_t dims, double base, double factor, double original, double fast, double slow);

// ---------------------------------------------------------------------------------------------
// HGRN2: per head a state S [dim, vdim] (fp32, one per sequence slot), S <- diag(f) S + (1 - f) v^T, o = S^T q with
// q = silu(q_raw), f = lower + (1 - lower) * sigmoid(f_raw + f_bias); then o / sqrt(mean(o^2) + eps) * norm_w per head.
// proj [tokens, ldp]: q_raw (heads * dim), f_raw (heads * dim), v (heads * vdim).  An entry whose pos0 is 0 starts from zero.
// ---------------------------------------------------------------------------------------------
struct StackHgrnParams
{
    int32_t dtype = DT_BF16;
    int32_t tokens = 0, entries = 0;
    int32_t heads = 0, dim = 0, vdim = 0;
    const void* proj = nullptr;
    int64_t ldp = 0;
    const float* f_bias = nullptr; // [heads * dim]
    const float* lower = nullptr;  // [heads * dim]
    const float* norm_w = nullptr; // [vdim]
    float eps = 1e-5f;
    float* state = nullptr;        // [slots, heads, dim, vdim]
    const int32_t* ent_slot = nullptr;
    const int32_t* ent_first = nullptr;
    const int32_t* ent_count = nullptr;
    const int32_t* ent_pos0 = nullptr;
    int32_t max_count = 0;         // host: the largest ent_count of the step
    float* o32 = nullptr;          // scratch [tokens, heads * vdim]
    void* out = nullptr;           // [tokens, heads * vdim]
};
int launch_stack_hgrn2(const StackHgrnParams& p, hipStream_t stream);
bool stack_hgrn2_serves(int32_t dim, int32_t vdim); // shapes one of its two forms takes

} // namespace kernels
} // namespace tllm
