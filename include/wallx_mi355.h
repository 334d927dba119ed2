/*
 * wallx_mi355.h -- C ABI of libwallx_mi355.so: the wall-x per-layer MoE hot path on MI355X (gfx950).
 *
 * Every entry point takes raw device pointers, sizes, strides (in elements) and a HIP stream, enqueues
 * its kernels on that stream and returns immediately: no allocation, no host synchronisation, no
 * torch types.  Return value: WX_OK (0) or a negative wx_status; wx_last_error_string() describes the
 * last failure on the calling thread.  Inputs are never modified.
 *
 * Each entry point names the reference interface it replaces (paths relative to the wall-x repository:
 * csrc/ = native ops bound by csrc/ops.cu:11-21 into module `wallx_csrc`, ops.py =
 * wall_x/fusions/ops.py, act.py / vl.py = wall_x/model/qwen2_5_based/modeling_qwen2_5_vl{_act,}.py).
 */
#ifndef WALLX_MI355_H
#define WALLX_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* wx_stream_t; /* hipStream_t */

typedef enum {
  WX_OK = 0,
  WX_ERR_INVALID_ARGUMENT = -1, /* null pointer, negative size, misaligned row, bad enum */
  WX_ERR_UNSUPPORTED = -2,      /* dtype / size outside what the kernels implement */
  WX_ERR_WORKSPACE = -3,        /* workspace too small */
  WX_ERR_LAUNCH = -4            /* hipGetLastError() after a launch */
} wx_status;

typedef enum { WX_F32 = 0, WX_F16 = 1, WX_BF16 = 2 } wx_dtype;
typedef enum { WX_I32 = 0, WX_I64 = 1, WX_U8 = 2 /* torch.bool */ } wx_itype;
/* Which rotary channel takes which of the (t, h, w) position planes:
 * WX_MROPE_HF   sections [s0,s1,s2,s0,s1,s2] cycling t,h,w,t,h,w     (vl.py:763-769, the PyTorch path)
 * WX_MROPE_CSRC sections [2*s0, 2*s1, 2*s2] contiguous t,h,w           (csrc/rope.cu:104-117) */
typedef enum { WX_MROPE_HF = 0, WX_MROPE_CSRC = 1 } wx_mrope_layout;

const char* wx_last_error_string(void);
/* Which kernels the last wx_dual_gemm / wx_dual_gemm_add call on the calling thread launched, as a bit set (0 before
 * the first call and after a call that launched nothing).  No counterpart in the reference; for tests and callers that
 * want to assert the code path rather than time it: a problem that should run on the matrix cores must not have gone
 * to the plain FMA kernel. */
enum {
  WX_GEMM_PATH_MFMA = 1,      /* the MFMA kernel (either tile shape) */
  WX_GEMM_PATH_ZERO_FILL = 2, /* an empty contraction (k == 0): its output was filled with zeros */
  WX_GEMM_PATH_FMA = 4,       /* the plain FMA kernel (K-major operands of 4 GiB or more) */
  WX_GEMM_PATH_ADD_COPY = 8   /* an empty contraction with an addend: the addend was copied to the output */
};
int wx_last_gemm_path(void);
int wx_abi_version(void);
/* 1 and *id = the capture's id when `stream` is being captured into a HIP graph, 0 and *id = 0 when it is not
 * (negative on error).  No counterpart in the reference; for hosts that keep results between calls (a cached token
 * partition, work buffers) and must not carry them from inside a capture, where nothing has executed yet, to
 * outside it. */
int wx_stream_capture_id(wx_stream_t stream, unsigned long long* id);

/* ------------------------------------------------------------------------------------------------
 * Token partition.  Replaces cub::DeviceRadixSort::SortPairs + moe_permute_topK_row_map
 * (csrc/permute.cu:39-67, 472-494) and the caller's per-expert bookkeeping (act.py:1274-1283).
 *
 * ids[num_tokens * num_topk] (row-major [T, K]) hold expert ids in [0, num_experts), num_experts <= 256.
 * Stable counting partition:  row_id_map[k*T + t] = sorted position of (t, k), or -1 when that position
 * is >= num_out_tokens (num_out_tokens <= 0 means T*K).  sorted_row_id[p] = t*K + k (may be NULL).
 * expert_offsets[num_experts + 1] = exclusive prefix of per-expert counts (may be NULL).
 * status (may be NULL): device word, set to 1 when an id lies outside [0, num_experts) (such ids are
 * clamped into range so the outputs stay a permutation), otherwise left untouched.
 * workspace: wx_partition_workspace_bytes(T*K) bytes of device memory, 256-byte aligned. */
size_t wx_partition_workspace_bytes(int64_t num_expanded_tokens);
int wx_partition_build(const void* ids, int id_type /* wx_itype */, int64_t num_tokens, int num_topk,
                       int num_experts, int64_t num_out_tokens, int32_t* row_id_map,
                       int32_t* sorted_row_id, int32_t* expert_offsets, int32_t* status,
                       void* workspace, size_t workspace_bytes, wx_stream_t stream);

/* wx_partition_build for callers that cannot allocate device memory or hand over a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference, whose
 * permute op allocates its sort workspace with torch (csrc/permute.cu:462-482).  Same arguments, outputs and
 * status codes as wx_partition_build minus the workspace pair: the per-segment histograms go to a 1 MiB device
 * array built into the library (one copy per GPU, held until the process ends), which covers every size the
 * partition takes (up to 2^31 - 1 expanded tokens; larger counts are refused with WX_ERR_UNSUPPORTED, a count whose
 * histograms would not fit with WX_ERR_WORKSPACE).  The call allocates nothing and does not synchronise.  The
 * array's address is looked up once per device (hipGetSymbolAddress) by wx_partition_noalloc_init(), or by the first
 * call on that device when it is not being captured; a first use from inside a stream capture is refused with
 * WX_ERR_INVALID_ARGUMENT (call the init function, with the device current, before capturing).
 * All calls on one GPU share the array: calls that overlap there (different streams or threads) race -- order them
 * on one stream.  Nothing in the array needs clearing between calls (every word read is written first). */
int wx_partition_build_noalloc(const void* ids, int id_type /* wx_itype */, int64_t num_tokens, int num_topk,
                               int num_experts, int64_t num_out_tokens, int32_t* row_id_map,
                               int32_t* sorted_row_id, int32_t* expert_offsets, int32_t* status,
                               wx_stream_t stream);
/* Set-up of wx_partition_build_noalloc for the current device: resolves the address of the built-in scratch array.
 * Idempotent, launches nothing; it has no counterpart in the reference either. */
int wx_partition_noalloc_init(void);

/* Row scatter of the permute op: out[row_id_map[k*T + t], :] = x[t, :] for every k with a map entry
 * != -1.  Replaces moe_permute_topK_kernel, forward branch (csrc/permute.cu:156-262, 294-305).
 * num_cols * sizeof(dtype) must be a multiple of 16 and rows 16-byte aligned. */
int wx_permute_rows(const void* x, void* out, const int32_t* row_id_map, int64_t num_tokens,
                    int num_topk, int64_t num_cols, int dtype /* wx_dtype */, wx_stream_t stream);

/* out[t, :] = sum_k prob[t, k] * y[row_id_map[k*T + t], :] (entries == -1 skipped; all skipped -> 0).
 * probs == NULL or num_topk == 1: no scaling (csrc/permute.cu:405-415 drops probs at K == 1).
 * Replaces moe_recover_topK_kernel (csrc/permute.cu:69-154, 398-441, 638-779). */
int wx_unpermute_rows(const void* y, void* out, const int32_t* row_id_map, const float* probs,
                      int64_t num_tokens, int num_topk, int64_t num_cols, int dtype,
                      wx_stream_t stream);

/* Backward of wx_unpermute_rows: act_grad[row_id_map[k*T+t], :] = grad_out[t, :] * prob[t, k]
 * (no factor at K == 1), prob_grad[t, k] = <grad_out[t, :], y_fwd[row, :]> in fp32 (written only when
 * K > 1; prob_grad may be NULL at K == 1).  Rows of act_grad that no token maps to are not written.
 * Replaces moe_permute_topK_kernel, unpermute-backward branch (csrc/permute.cu:156-262, 781-942). */
int wx_unpermute_rows_bwd(const void* grad_out, const void* y_fwd, void* act_grad, float* prob_grad,
                          const int32_t* row_id_map, const float* probs, int64_t num_tokens,
                          int num_topk, int64_t num_cols, int dtype, wx_stream_t stream);

/* ------------------------------------------------------------------------------------------------
 * Dual asymmetric grouped GEMM: out_e = op(in_e) @ op(w_e), e in {0, 1}, in ONE launch; bf16 in/out,
 * fp32 accumulate.  Replaces AsymmetricDualExpertGemm (csrc/dual_asym_grouped_gemm.cu:308-366,
 * ops.py:6-165).  trans_a: in_e stored [k_e, m_e]; trans_b: w_e stored [n_e, k_e] (nn.Linear layout).
 * All matrices packed row-major.  Every layout is read in place by the same MFMA kernel (an operand whose slow
 * dimension is K is transposed on its way from LDS to the registers), which covers the forward (trans_b) and
 * both backward GEMMs of ops.py:78-144 (dX: neither flag; dW: trans_a only).  n_e multiples of 8; m_e multiples
 * of 8 under trans_a; k_e multiples of 8 unless both operands are stored [k, .] (trans_a without trans_b), where
 * k_e -- the token count of a weight gradient -- is free.  m_e == 0 is allowed. */
int wx_dual_gemm(const void* in0, const void* in1, const void* w0, const void* w1, void* out0,
                 void* out1, int64_t m0, int64_t n0, int64_t k0, int64_t m1, int64_t n1, int64_t k1,
                 int trans_a, int trans_b, wx_stream_t stream);

/* wx_dual_gemm with an addend per expert: out_e = op(in_e) @ op(w_e) + add_e, where add_e is [m_e, n_e] bf16
 * row-major like out_e, may be out_e itself and may be NULL (plain product).  The product is rounded to bf16 and
 * the sum formed in fp32 and rounded once, i.e. the result of two eager bf16 ops.  For sums of products over
 * several weight matrices, as in the input gradient of a gated FFN, dX = dG @ Wg + dU @ Wu (the backward of
 * act.py:79-82, ops.py:78-144): the second product accumulates onto the first instead of a separate add pass. */
int wx_dual_gemm_add(const void* in0, const void* in1, const void* w0, const void* w1, void* out0,
                     void* out1, const void* add0, const void* add1, int64_t m0, int64_t n0, int64_t k0,
                     int64_t m1, int64_t n1, int64_t k1, int trans_a, int trans_b, wx_stream_t stream);

/* ------------------------------------------------------------------------------------------------
 * K-tiled operands of the fused FFN.  The MFMA kernels read activations and weights from a block layout in
 * which every 16-row x 32-column block (1 KiB, bank-swizzled for LDS) is contiguous and the 256 x 32 slab a
 * workgroup consumes per K step is one contiguous run -- the access pattern the memory pipeline serves fastest.
 * The layout is internal to this library: weights are packed once (wx_pack_tiled), activations are written in
 * it by wx_permute_rows_tiled, the intermediate never leaves it.  Only bf16; cols must be a multiple of 32.
 * wx_tiled_bytes: size of a packed [rows, cols] matrix (rows padded to 16).  wx_padded_sorted_rows: rows of the
 * expert-sorted space for `rows` tokens once each expert's range starts at a multiple of 256 (an upper bound that
 * depends on `rows` only).  These have no counterpart in the reference (its GEMMs read nn.Linear weights in place). */
size_t wx_tiled_bytes(int64_t rows, int64_t cols);
int64_t wx_padded_sorted_rows(int64_t rows);
int wx_pack_tiled(const void* src_row_major, void* dst_tiled, int64_t rows, int64_t cols,
                  wx_stream_t stream);

/* Permute straight into the K-tiled activation matrix of the FFN: row t of x goes to sorted row
 * row_id_map[t], shifted for expert 1 so that its rows start at a multiple of 256.  Replaces
 * moe_permute_topK_kernel's forward branch (csrc/permute.cu:156-262) for topK == 1 when the consumer is
 * wx_dual_swiglu_ffn.  out_tiled: wx_tiled_bytes(wx_padded_sorted_rows(T), num_cols) bytes.
 * expert_offsets: device int32[3] from wx_partition_build.  Either map may be NULL, not both: with
 * sorted_row_id (the partition's inverse map) rows are gathered block by block and every store is a whole
 * contiguous KiB (the faster form; padding rows are zero-filled); with row_id_map alone rows are scattered. */
int wx_permute_rows_tiled(const void* x, void* out_tiled, const int32_t* row_id_map,
                          const int32_t* sorted_row_id, const int32_t* expert_offsets,
                          int64_t num_tokens, int64_t num_cols, wx_stream_t stream);

/* Both experts' SwiGLU FFN over expert-sorted rows, two launches (gate/up + SwiGLU, then down), each
 * covering both experts:  out[r, :] = down_e( silu(x[r] @ gate_e^T) * (x[r] @ up_e^T) ) for sorted rows
 * r in [expert_offsets[e], expert_offsets[e+1]).  Replaces the per-expert loop of
 * SparseMoeBlock.forward over BlockSparseMLP (act.py:79-82, 142-154).
 * x_tiled: K-tiled activations from wx_permute_rows_tiled.  out: [num_rows, hidden] bf16 row-major in sorted
 * order (what wx_unpermute_rows reads).  gate_e, up_e: packed [inter_e, hidden]; down_e: packed
 * [hidden, inter_e] (wx_pack_tiled of the nn.Linear weights).
 * expert_offsets: DEVICE int32[3] (from wx_partition_build), read by the kernels -- no host sync.
 * hmid: device scratch, wx_padded_sorted_rows(num_rows) * max(inter0, inter1) bf16.
 * hidden, inter0, inter1 must be multiples of 32.
 * Intermediate rounding follows eager bf16 evaluation: gate, up, silu(gate) and the product are each
 * rounded to bf16 (fp32 accumulation inside each contraction). */
int wx_dual_swiglu_ffn(const void* x_tiled, void* out, const int32_t* expert_offsets, const void* gate0,
                       const void* up0, const void* down0, const void* gate1, const void* up1,
                       const void* down1, void* hmid, int64_t num_rows, int64_t hidden,
                       int64_t inter0, int64_t inter1, const int64_t* host_rows_per_expert,
                       const int32_t* out_row_id, wx_stream_t stream);

/* wx_dual_swiglu_ffn (optionally with the permute in front and wx_dual_down_proj_residual's closing add behind) as
 * ONE launch where that pays: when host_rows_per_expert is given and each of the two GEMMs is a single round of
 * 128 x 128 tiles (at most one per CU: the denoise step's few thousand action tokens), or, without the host's row
 * counts, for up to two rows per CU (512 on an MI355X), gate/up tiles and down tiles share one grid, and a down tile
 * starts as soon as the gate/up tiles of its 128 rows have finished instead of after a launch boundary.  Every other shape, or a NULL workspace, runs the launches of wx_[permute_rows_tiled +]
 * wx_dual_swiglu_ffn; results are bit-identical either way.  The host's row counts only choose the form.
 * x_rows: NULL, or the activations in token order, [num_rows, hidden] bf16 (out_row_id required): the permute is then
 * part of the call and x_tiled only a work buffer -- in the one launch the gate/up tiles read the token rows through
 * out_row_id and x_tiled is not touched; the other shapes fill it with wx_permute_rows_tiled first.
 * residual: NULL or as for wx_dual_down_proj_residual (then out_row_id is required).
 * workspace: wx_ffn_fused_workspace_bytes() bytes of device memory, 4-byte aligned, ZERO before its first use; a
 * launch leaves it zero again.  Calls that share a workspace must not overlap (one workspace per stream).
 * Inside the one launch tiles wait on counters in the workspace that other tiles advance; every wait is bounded
 * (seconds), and a wait that runs into its bound stores 1 into the workspace's last int (the result is then undefined).
 * A launch alone on the GPU, or two of them at once on two streams, cannot run into the bound (the tiles waited for
 * always hold or get a place on the chip); a caller that keeps three or more in flight together on one GPU should
 * read that int, or pass a NULL workspace.
 * Unless the previous one launch of the calling thread on the same workspace ran on the same six weight tensors (a
 * loop over one layer), the one launch also requests the gate/up weights ahead of its K loops, for weights that come
 * from HBM as every layer of a model's do.
 * No counterpart in the reference, whose experts are separate nn.Linear launches (act.py:79-82, 142-154). */
size_t wx_ffn_fused_workspace_bytes(void);
int wx_dual_swiglu_ffn_fused(const void* x_rows, void* x_tiled, void* out, const void* residual,
                             const int32_t* expert_offsets, const void* gate0, const void* up0, const void* down0,
                             const void* gate1, const void* up1, const void* down1, void* hmid, int64_t num_rows,
                             int64_t hidden, int64_t inter0, int64_t inter1, const int64_t* host_rows_per_expert,
                             const int32_t* out_row_id, void* workspace, wx_stream_t stream);

/* The two launches of wx_dual_swiglu_ffn on their own, for callers that put work between them (and for
 * timing each kernel): hmid = silu(x @ gate^T) * (x @ up^T), then out = hmid @ down^T, per expert.
 * Same arguments and layouts as above; they replace the same reference lines (act.py:79-82, 142-154). */
int wx_dual_swiglu_gate_up(const void* x_tiled, void* hmid, const int32_t* expert_offsets,
                           const void* gate0, const void* up0, const void* gate1, const void* up1,
                           int64_t num_rows, int64_t hidden, int64_t inter0, int64_t inter1,
                           const int64_t* host_rows_per_expert, wx_stream_t stream);
int wx_dual_down_proj(const void* hmid, void* out, const int32_t* expert_offsets, const void* down0,
                      const void* down1, int64_t num_rows, int64_t hidden, int64_t inter0,
                      int64_t inter1, const int64_t* host_rows_per_expert, const int32_t* out_row_id,
                      wx_stream_t stream);
/* wx_dual_down_proj with the decoder layer's closing residual add (act.py:256-265: `hidden_states = residual +
 * hidden_states` after the MoE block) in its epilogue: out[t, :] = residual[t, :] + y[t, :] in token order, where
 * y is the block's bf16 result and the sum is formed in fp32 and rounded once, like the eager add.  residual is
 * [num_rows, hidden] bf16 laid out like out and may be out itself; out_row_id (the partition's sorted_row_id) is
 * required.  Replaces wx_dual_down_proj + wx_unpermute_rows_add: the sorted result is never written. */
int wx_dual_down_proj_residual(const void* hmid, void* out, const void* residual,
                               const int32_t* expert_offsets, const void* down0, const void* down1,
                               int64_t num_rows, int64_t hidden, int64_t inter0, int64_t inter1,
                               const int64_t* host_rows_per_expert, const int32_t* out_row_id,
                               wx_stream_t stream);
/* wx_dual_swiglu_gate_up for a forward pass whose backward will follow: besides hmid it stores the two projections
 * themselves (rounded to bf16, before the SwiGLU) into gate_keep / up_keep, K-tiled buffers of hmid's size and
 * geometry, so that the backward does not run the two projections again.  The reference keeps these activations
 * through autograd (act.py:79-82 under torch.autograd saves gate, up, act_fn(gate) and the product). */
int wx_dual_swiglu_gate_up_keep(const void* x_tiled, void* hmid, void* gate_keep, void* up_keep,
                                const int32_t* expert_offsets, const void* gate0, const void* up0,
                                const void* gate1, const void* up1, int64_t num_rows, int64_t hidden,
                                int64_t inter0, int64_t inter1, const int64_t* host_rows_per_expert,
                                wx_stream_t stream);
/* out_row_id (optional, may be NULL): DEVICE int32[num_rows], the partition's sorted_row_id (sorted position ->
 * token).  When given, the down launch stores sorted row r of the result at row out_row_id[r] of `out`, i.e. `out`
 * comes back in token order and the separate unpermute (ops.unpermute at topK 1, act.py:157-161) is not needed:
 * its row-granular stores are the same 256-byte runs either way. */
/* host_rows_per_expert (optional, may be NULL): HOST int64[2], the rows of each expert when the caller already
 * has them on the host (the reference computes them there, act.py:1274-1283).  They only steer the choice between
 * the two tile shapes: without them, a call whose bounds on the tile count straddle the threshold launches both
 * shapes and the device decides (one of the launches returns at once).  The kernels always take the row ranges
 * from expert_offsets on the device; a hint that disagrees with them costs speed, never correctness. */

/* ------------------------------------------------------------------------------------------------
 * 3D multimodal RoPE:  out = x * cos_sel + rotate_half(x) * sin_sel for q and k, where channel d of
 * cos_sel / sin_sel comes from plane axis(d) of cos / sin [3, B, S, D] (contiguous, dtype of q).
 * Replaces launch_multimodal_rope_forward (csrc/rope.cu:48-178, 453-509; ops.py:402-497) and follows
 * apply_multimodal_rotary_pos_emb (vl.py:731-773) when layout == WX_MROPE_HF.
 * q is addressed as q[b, h, s, d] = q + b*q_sb + h*q_sh + s*q_ss + d (strides in elements, d
 * contiguous), so the [B, S, H, D] projection output can be passed without a transposing copy; same for
 * k and the two outputs.  Each product and the sum are rounded to the storage dtype, as eager
 * evaluation does.  D must be a multiple of 16 and at most 256. */
int wx_mrope_apply(const void* q, const void* k, const void* cos, const void* sin, void* q_out,
                   void* k_out, int64_t batch, int64_t seq, int n_q_heads, int n_kv_heads,
                   int head_dim, const int64_t q_strides[3] /* b, h, s */, const int64_t k_strides[3],
                   const int64_t qo_strides[3], const int64_t ko_strides[3],
                   const int mrope_section[3], int layout /* wx_mrope_layout */, int dtype,
                   wx_stream_t stream);

/* Adjoint w.r.t. q and k: g_in = g*cos_sel + rotate_half^T(g*sin_sel).  Replaces
 * launch_multimodal_rope_backward (csrc/rope.cu:181-330, 511-571).  fp32 math, one rounding. */
int wx_mrope_apply_bwd(const void* gq_out, const void* gk_out, const void* cos, const void* sin,
                       void* gq, void* gk, int64_t batch, int64_t seq, int n_q_heads,
                       int n_kv_heads, int head_dim, const int64_t gqo_strides[3],
                       const int64_t gko_strides[3], const int64_t gq_strides[3],
                       const int64_t gk_strides[3], const int mrope_section[3], int layout,
                       int dtype, wx_stream_t stream);

/* The same rotation with the cos/sin builder folded in: instead of the two [3, B, S, D] tables the call takes
 * what they are built from, position_ids [3, B, S] int64 (contiguous) and inv_freq [D/2] fp32, and every thread
 * evaluates cos/sin of its own channels like Qwen2_5_VLRotaryEmbedding.forward does (vl.py:679-712): angle =
 * fp32(position) * inv_freq[d mod D/2] in fp32, cos and sin in fp32, rounded to the dtype of q (attention_scaling
 * is 1 for the default rope type, vl.py:635-678).  Replaces that builder plus apply_multimodal_rotary_pos_emb
 * (vl.py:731-773) / the rope op (ops.py:402-497) in one pass; backward != 0 gives the adjoint (arguments as in
 * wx_mrope_apply_bwd).  Results equal wx_mrope_apply on tables built in fp32 up to the last-place difference of
 * the device's sincosf against the table builder's (a rounded bf16 cos/sin then differs in well under 1e-4 of the
 * entries).  Heads must be 2..64 16-byte chunks, a power of two, with section ends on chunk boundaries;
 * other shapes return WX_ERR_UNSUPPORTED (build the tables and call wx_mrope_apply). */
int wx_mrope_apply_positions(const void* q, const void* k, const int64_t* position_ids, const float* inv_freq,
                             void* q_out, void* k_out, int64_t batch, int64_t seq, int n_q_heads, int n_kv_heads,
                             int head_dim, const int64_t q_strides[3], const int64_t k_strides[3],
                             const int64_t qo_strides[3], const int64_t ko_strides[3],
                             const int mrope_section[3], int layout, int dtype, int backward,
                             wx_stream_t stream);

/* The attention block's q / k / v projections with the rotary embedding in the GEMM's epilogue: replaces
 * q_proj / k_proj / v_proj (nn.Linear with bias, vl.py:821-832, 955-957) followed by the rope op
 * (vl.py:962-964, ops.py:402-497) -- one launch, and q / k are not written and read again for the rotation.
 * wx_mrope_table builds what the epilogue reads: table[token][d], d < W, = bf16 cos | bf16 sin << 16 of
 * position_ids[plane(d)][token] * inv_freq[d mod head_dim / 2] (fp32 angle, fp32 cos / sin, rounded to bf16 as
 * vl.py:679-712 does); position_ids [3, B, S] int64, inv_freq [head_dim / 2] fp32, table uint32 [B * S, W].
 * W = wx_mrope_table_width(head_dim, mrope_section, layout): head_dim / 2 when channels d and d + head_dim / 2 share a
 * position plane (WX_MROPE_HF: one entry serves both), head_dim when they do not (WX_MROPE_CSRC: one entry per
 * channel); negative status on bad arguments.
 * wx_qkv_rope_proj: out [num_tokens, (n_q + 2 n_kv) * head_dim] = x [num_tokens, hidden] @ weight^T + bias, weight
 * [(n_q + 2 n_kv) * head_dim, hidden] = the three nn.Linear weights stacked q, k, v (row-major, read in place), bias
 * likewise or NULL; the q and k heads (the first (n_q + n_kv) * head_dim columns) come out rotated:
 * head[d] * cos[d] + rotate_half(head)[d] * sin[d], evaluated like eager bf16 code (the projection rounded once, every
 * product and the sum rounded).  bf16; head_dim must be 128 (a wavefront's 128 output columns are one head), hidden a
 * multiple of 8.  Row t of the table belongs to row t of x; table_width is the W the table was built with (either
 * layout is served: with WX_MROPE_HF this is the eager attention path of vl.py:860-862 / 1075-1077, with WX_MROPE_CSRC
 * the flash-attention class's rope op, vl.py:962-964 on csrc/rope.cu:104-117). */
int wx_mrope_table_width(int head_dim, const int mrope_section[3], int layout /* wx_mrope_layout */);
int wx_mrope_table(const int64_t* position_ids, const float* inv_freq, int64_t batch, int64_t seq, int head_dim,
                   const int mrope_section[3], int layout /* wx_mrope_layout */, uint32_t* table,
                   wx_stream_t stream);

/* wx_mrope_apply / wx_mrope_apply_bwd (backward != 0) with cos and sin read from the packed table of wx_mrope_table
 * instead of the two [3, B, S, D] tables: 256 bytes per token (512 for WX_MROPE_CSRC, whose table has one entry per
 * channel) where the selected channels of three planes of two tables touch twelve cache lines.  bf16; `layout` and
 * `mrope_section` must be the ones the table was built with; heads as for wx_mrope_apply_positions.  The table is
 * built once per forward and serves every layer.  Results equal
 * wx_mrope_apply_positions bit for bit (the same device cos / sin).  No counterpart in the reference beyond the rope
 * op itself (ops.py:402-497, vl.py:731-773). */
int wx_mrope_apply_packed(const void* q, const void* k, const uint32_t* table, void* q_out, void* k_out,
                          int64_t batch, int64_t seq, int n_q_heads, int n_kv_heads, int head_dim,
                          const int64_t q_strides[3], const int64_t k_strides[3], const int64_t qo_strides[3],
                          const int64_t ko_strides[3], const int mrope_section[3], int layout, int dtype,
                          int backward, wx_stream_t stream);
int wx_qkv_rope_proj(const void* x, const void* weight, const void* bias, const uint32_t* rope_table,
                     int table_width, void* out, int64_t num_tokens, int64_t hidden, int n_q_heads, int n_kv_heads,
                     int head_dim, wx_stream_t stream);

/* ------------------------------------------------------------------------------------------------
 * 3D position ids.  Replaces get_rope_index (csrc/rope_index.cu:464-569) with the semantics of the
 * PyTorch path (act.py:929-1149), exact integer arithmetic.
 * input_ids [B, S] int64; attention_mask [B, S] int64 or NULL (all ones);
 * image_grid_thw [n_image, 3] / video_grid_thw [n_video, 3] int64 (NULL when absent);
 * second_per_grid_ts [n_video] fp32 or NULL (1.0).  Both grids NULL selects the text-only branch
 * (act.py:1123-1149).  position_ids [3, B, S] int64, deltas [B] int64.
 * status (may be NULL): device word set to 1 when a row is malformed in a way that makes the PyTorch
 * path raise (a vision item without its tokens, more items than grids, a fully masked row).
 * workspace: wx_rope_index_workspace_bytes(B, S) bytes (a few bytes per row; rows longer than 30720 tokens also
 * keep their compacted form there, 5 bytes per token, instead of in LDS).  No cap on S or on images per row (the
 * reference kernel stops at 64 segments per row, csrc/rope_index.cu). */
size_t wx_rope_index_workspace_bytes(int64_t batch, int64_t seq);
int wx_rope_index(const int64_t* input_ids, const int64_t* attention_mask,
                  const int64_t* image_grid_thw, int64_t n_image, const int64_t* video_grid_thw,
                  int64_t n_video, const float* second_per_grid_ts, int64_t batch, int64_t seq,
                  int spatial_merge_size, int64_t image_token_id, int64_t video_token_id,
                  int64_t vision_start_token_id, float tokens_per_second, int64_t* position_ids,
                  int64_t* deltas, int32_t* status, void* workspace, size_t workspace_bytes,
                  wx_stream_t stream);

/* Vision-tower rotary table.  Replaces fused_rot_pos_emb_cuda (csrc/rot_pos.cu:187-312) and follows
 * rot_pos_emb (vl.py:473-500).  grid_thw [n_grid, 3] int32 or int64 on the device; total_patches =
 * sum t*h*w (the caller sizes the outputs from its host copy of grid_thw).
 * table (may be NULL): fp32 [total_patches, 2*n_freq] = [h_pos * inv_freq, w_pos * inv_freq].
 * pos_ids (may be NULL): int64 [total_patches, 2] = (h_pos, w_pos). */
int wx_rot_pos_emb(const float* inv_freq, int n_freq, const void* grid_thw, int grid_type,
                   int64_t n_grid, int spatial_merge_size, int64_t total_patches, float* table,
                   int64_t* pos_ids, wx_stream_t stream);

/* Vision-tower window permutation.  Replaces get_window_index_cuda (csrc/window_index.cu:208-286)
 * and follows get_window_index (vl.py:502-547) with one cumulative entry per non-empty window.
 * grid_thw [n_grid, 3] int32 or int64 on the device.  window_index int32 [total_tokens], total_tokens =
 * sum t*(h/m)*(w/m); cu_window_seqlens int32 [total_windows + 1], total_windows =
 * sum t*ceil(h/m/ws)*ceil(w/m/ws) (the caller sizes both from its host copy of grid_thw). */
int wx_window_index(const void* grid_thw, int grid_type, int64_t n_grid, int spatial_merge_size,
                    int vit_merger_window_size, int spatial_merge_unit, int64_t total_tokens,
                    int64_t total_windows, int32_t* window_index, int32_t* cu_window_seqlens,
                    wx_stream_t stream);

/* Caller fusions around the FFN (act.py:256-265: residual; post_attention_layernorm; moe; residual add), bf16:
 * wx_rmsnorm_permute_rows_tiled = RMSNorm (the module at act.py:190-193: fp32 variance, x * rsqrt(var + eps) rounded
 * to bf16, times the bf16 weight) followed by wx_permute_rows_tiled in its gather form, in one pass;
 * sorted_row_id is the inverse map from wx_partition_build.  num_cols: a multiple of 128, at most 4096.
 * wx_unpermute_rows_add = wx_unpermute_rows at topK 1 followed by `residual + .` (one rounding), in one pass.
 * The reference runs these as separate PyTorch ops; listed as the next step after the ops themselves. */
int wx_rmsnorm_permute_rows_tiled(const void* x, const void* weight, float eps, void* out_tiled,
                                  const int32_t* sorted_row_id, const int32_t* expert_offsets,
                                  int64_t num_tokens, int64_t num_cols, wx_stream_t stream);
int wx_unpermute_rows_add(const void* y, const void* residual, void* out, const int32_t* row_id_map,
                          int64_t num_tokens, int64_t num_cols, wx_stream_t stream);
/* wx_unpermute_rows_add with the RMSNorm that consumes its result next folded in: out = residual + unpermuted y
 * (the residual stream after the layer, act.py:265) and normed = weight * rmsnorm(out, eps), i.e. the following
 * layer's input_layernorm (act.py:240) or the model's final norm (act.py:506), computed from the bf16-rounded
 * sum as the separate module would.  num_cols: a multiple of 8, at most 4096. */
int wx_unpermute_rows_add_rmsnorm(const void* y, const void* residual, void* out, void* normed,
                                  const void* weight, float eps, const int32_t* row_id_map,
                                  int64_t num_tokens, int64_t num_cols, wx_stream_t stream);
/* The training step's side of the two fusions above (the reference trains through act.py:256-265 with autograd):
 * wx_rmsnorm_permute_rows = the same RMSNorm followed by wx_permute_rows at topK 1 -- out_sorted[p] = weight *
 * rmsnorm(x[sorted_row_id[p]]), row-major in expert-sorted order: the normed rows the experts' weight gradients
 * contract over, recomputed in the backward instead of kept by the forward.
 * wx_unpermute_rows_rmsnorm_bwd = backward of "normed = weight * rmsnorm(x); sorted = permute(normed)" for the
 * gradient grad_sorted of the sorted rows (wx_unpermute_rows_bwd at topK 1, then the norm's backward), in one pass:
 *   grad_x[t] = (add[t] +) inv * (g w - xhat * mean(g w xhat)),  g = grad_sorted[row_id_map[t]] (0 where the map holds
 *   -1), xhat = x[t] * inv, inv = rsqrt(mean(x[t]^2) + eps), fp32 math and one rounding;  `add` (optional, [T, H]) is
 *   the gradient that reaches x along the residual branch (act.py:256,265: the layer's output gradient itself);
 *   grad_weight[c] = sum over t of g[c] * bf16(xhat[c]), fp32 accumulation, bf16 [H].
 * workspace: wx_rmsnorm_bwd_workspace_bytes(num_cols) bytes of device memory (per-wavefront partial sums of
 * grad_weight).  num_cols: a multiple of 8, at most 4096. */
int wx_rmsnorm_permute_rows(const void* x, const void* weight, float eps, void* out_sorted,
                            const int32_t* sorted_row_id, int64_t num_tokens, int64_t num_cols, wx_stream_t stream);
size_t wx_rmsnorm_bwd_workspace_bytes(int64_t num_cols);
int wx_unpermute_rows_rmsnorm_bwd(const void* grad_sorted, const void* x, const void* weight, float eps,
                                  const void* add, void* grad_x, void* grad_weight, const int32_t* row_id_map,
                                  int64_t num_tokens, int64_t num_cols, void* workspace, size_t workspace_bytes,
                                  wx_stream_t stream);

/* One call for the block's forward as the decoder layer uses it (act.py:256-265 around act.py:105-162):
 * [RMSNorm ->] permute into the K-tiled activations -> gate/up + SwiGLU -> down with every row stored at its token's
 * position [+ residual].  Exactly the launches of wx_rmsnorm_permute_rows_tiled / wx_permute_rows_tiled,
 * wx_dual_swiglu_gate_up and wx_dual_down_proj / wx_dual_down_proj_residual in that order, with their argument rules:
 * a host that issues a layer per call (36 per forward, 360 per denoised action chunk) pays for one library call
 * instead of three.  x, out: [num_rows, hidden] bf16 in token order; row_id_map, sorted_row_id, expert_offsets: the
 * partition's outputs (sorted_row_id required); the six weights packed (wx_pack_tiled); x_tiled and hmid: work
 * buffers of wx_tiled_bytes(wx_padded_sorted_rows(num_rows), hidden) bytes and wx_padded_sorted_rows(num_rows) *
 * max(inter0, inter1) bf16; norm_weight: bf16 [hidden] or NULL (no norm); add_residual != 0 returns x + block(x).
 * ffn_workspace: NULL, or the workspace of wx_dual_swiglu_ffn_fused (same rules), which then runs the two GEMMs
 * and, when there is no norm, the permute as well. */
int wx_moe_block_forward(const void* x, void* out, const int32_t* row_id_map, const int32_t* sorted_row_id,
                         const int32_t* expert_offsets, const void* gate0, const void* up0, const void* down0,
                         const void* gate1, const void* up1, const void* down1, void* x_tiled, void* hmid,
                         int64_t num_rows, int64_t hidden, int64_t inter0, int64_t inter1,
                         const int64_t* host_rows_per_expert, const void* norm_weight, float eps,
                         int add_residual, void* ffn_workspace, wx_stream_t stream);

/* Elementwise backward of h = silu(g) * u inside an expert FFN (act.py:79-82; the reference leaves it to autograd):
 * from gate, up (the two projections, kept by the forward or recomputed) and dh (gradient w.r.t. h) in one pass:
 * hmid = bf16(bf16(silu(g)) * u) as the forward fed it to the down projection, dgate = dh * u * s * (1 + g * (1 - s))
 * with s = sigmoid(g), dup = dh * silu(g).  bf16 in and out, fp32 math; num_elems a multiple of 8. */
int wx_swiglu_bwd(const void* gate, const void* up, const void* dh, void* hmid, void* dgate, void* dup,
                  int64_t num_elems, wx_stream_t stream);
/* The same with gate and up of ONE expert read from the K-tiled buffers wx_dual_swiglu_gate_up_keep filled:
 * gate_tiled / up_tiled point at that expert's tiled matrix of tiled_rows rows (its row count rounded up to 256) and
 * cols columns; dh and the three outputs are row-major [rows, cols].  cols a multiple of 64.  hmid may be NULL when
 * the caller does not need it (the expert's down projection does not train). */
int wx_swiglu_bwd_tiled(const void* gate_tiled, const void* up_tiled, int64_t tiled_rows, const void* dh, void* hmid,
                        void* dgate, void* dup, int64_t rows, int64_t cols, wx_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* WALLX_MI355_H */
