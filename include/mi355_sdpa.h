/*
 * mi355_sdpa.h - C ABI of the MI355X (gfx950) fused scaled-dot-product-attention library.
 *
 * Every entry point is extern "C", takes plain pointers / sizes / POD structs, never
 * allocates device memory, never synchronises, launches on the stream it is given
 * (a hipStream_t passed as void*; NULL = the default stream) and reports failure with a
 * negative return code plus a thread-local message (mi355_sdpa_last_error).  No C++
 * exception crosses this boundary.
 *
 * Each declaration names the piece of aws-neuron/torch-neuronx it stands in for
 * (paths relative to that tree).
 *
 * Tensor convention: 4-D (batch, heads, sequence, head_dim), sizes and strides in
 * ELEMENTS.  The fast kernels need unit stride on the last dimension; everything else is
 * free (the usual (B,S,H,D).transpose(1,2) views are consumed in place).
 */
#ifndef MI355_SDPA_H
#define MI355_SDPA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_SDPA_ABI_VERSION 6

/* element types */
enum mi355_sdpa_dtype {
  MI355_SDPA_F32 = 0,
  MI355_SDPA_F16 = 1,
  MI355_SDPA_BF16 = 2,
  MI355_SDPA_F64 = 3,       /* descriptors only: validated, then computed as f32 by the host */
  MI355_SDPA_BOOL = 4,      /* attention mask only: 1 byte, non-zero = attend               */
  MI355_SDPA_FP8_E4M3 = 5,  /* OCP e4m3fn, decode K/V cache only                            */
  MI355_SDPA_OTHER = 99
};

/* return codes */
enum mi355_sdpa_status {
  MI355_SDPA_OK = 0,
  MI355_SDPA_ERR_INVALID = -1,     /* argument breaks the operator contract        */
  MI355_SDPA_ERR_UNSUPPORTED = -2, /* valid, but no kernel in this library takes it */
  MI355_SDPA_ERR_LAUNCH = -3       /* HIP reported an error at launch               */
};

/* backend ids: numerically equal to at::SDPBackend */
enum mi355_sdpa_backend { MI355_SDPA_BACKEND_MATH = 0, MI355_SDPA_BACKEND_OVERRIDEABLE = 4 };

/* which kernel family a call is served by */
enum mi355_sdpa_kernel {
  MI355_SDPA_KERNEL_NONE = 0,
  MI355_SDPA_KERNEL_GENERIC = 1, /* fp32-accumulate kernel: any head dim, bias, masks, dropout */
  MI355_SDPA_KERNEL_MFMA = 2,    /* matrix-op flash kernels: bf16/f16 (head dims up to 256, masks,
                                    functors, dropout) and float32
                                    (the same head dims; masks, key counts, dropout, functors) */
  /* forward only, for tests and tuning: pin the query rows per workgroup of the MFMA kernel */
  MI355_SDPA_KERNEL_MFMA_T128 = 3,
  MI355_SDPA_KERNEL_MFMA_T256 = 4
};

typedef struct mi355_sdpa_tensor {
  void* data; /* device pointer; NULL = absent */
  int64_t size[4];
  int64_t stride[4];
} mi355_sdpa_tensor;

/* Shape/dtype description used by the host-logic entry points (no device pointers read). */
typedef struct mi355_sdpa_desc {
  int32_t q_dim, k_dim, v_dim;       /* tensor ranks                                  */
  int64_t q_size[4], k_size[4], v_size[4];
  int32_t q_dtype, k_dtype, v_dtype; /* enum mi355_sdpa_dtype                         */
  int32_t on_device;                 /* 1 if all three live on the GPU                */
  int32_t has_symbolic_shape;        /* 1 if any size is symbolic (tracing)           */
  int32_t has_attn_bias;             /* a mask / bias tensor is present               */
  int32_t is_causal;
  int32_t return_debug_mask;
  int32_t has_scale;                 /* 0: scale = 1/sqrt(E)                          */
  float scale;
  float dropout_p;
  int32_t requires_lse;
  int32_t q_last_stride, k_last_stride, v_last_stride; /* stride of head_dim           */
} mi355_sdpa_desc;

/* Mask and score functors that need no mask tensor: the kernels derive them from the query and
 * key indices (and a few small captured vectors) and skip the key tiles they drop whole.  They
 * stand in for the specialisations the reference renders into its templated kernels
 * (torch_neuronx/neuron_dynamo_backend/flex_attention/flex_attention.py.jinja: mask_mod /
 * score_mod hooks :74-92, applied :2495-2660 - score = scale * q.k first, then score_mod, then the
 * mask; the `sliding_window` and `sink` arguments :94-117; static tile elimination :15-33; and
 * flex_attention_bwd.py.jinja: joint_mod, the derivative of score_mod, :958-988, applied
 * :1261-1271).
 *   window > 0   sliding window, needs is_causal: query i sees keys i-window+1 .. i
 *   sink_keys    with a window: keys 0 .. sink_keys-1 stay visible to every later query
 *   sink_logit   optional (B,Hq,n_sink_logits) contiguous float32 (n_sink_logits = 0 means 1, i.e.
 *                (B,Hq); the reference's kernels take both shapes, flex_attention_bwd.py.jinja:103,
 *                :316-320): logits without a value that join every row's softmax (maximum and
 *                sum): out = sum_j p_j v_j with p = softmax([scores, sink logits])[:S]; lse
 *                includes them.  Works with any mask.
 * Score functors, applied to s = scale * q.k of query i, key j, head h in this order (each optional;
 * what the reference's tests render as score_mods: ALiBi, a captured per-head per-key bias or
 * weight, a tanh soft cap - tests/neuron_dynamo_backend/unit/fx/passes/
 * test_flex_attention_legalization.py:1051-1066, :1207-1218):
 *   key_weight   (Hq,S) contiguous float32     s *= key_weight[h][j]
 *   key_bias     (Hq,S) contiguous float32     s += key_bias[h][j]
 *   alibi_slopes (Hq,)  float32                s += alibi_slopes[h] * (j - i)
 *   softcap > 0                                s  = softcap * tanh(s / softcap)
 * The backward multiplies the gradient of the scores by the derivative of that chain,
 * key_weight[h][j] * (1 - tanh^2), before it forms dQ and dK; the captured vectors get no
 * gradient of their own.
 * Index-computed masks with captured vectors (document masks of packed sequences):
 *   doc_ids_q (B,L), doc_ids_k (B,S) contiguous int32: the score of (i, j) is kept iff
 *                doc_ids_q[b][i] == doc_ids_k[b][j]; composes with is_causal and the window
 *   doc_ids_sorted  the caller's promise that both vectors are non-decreasing along the sequence
 *                (documents packed one after the other): the kernels then find, per block of query
 *                rows, the range of key tiles that can hold an equal id and walk only those, and
 *                test whole tiles with two loads.  Without the promise every tile is walked and
 *                every score compared: same results, no skipping.
 * Score functors and document ids run in the matrix-op kernels for bf16 / f16 at every head dim up
 * to 256 (D_v <= D_qk), and for float32 at the same head dims, without attn_bias and dropout; other calls take
 * the generic kernels.
 * Tile skip tables for a mask that only exists as a tensor (the run-time counterpart of the
 * reference's static tile elimination, flex_attention.py.jinja:15-33), built from the bias /
 * keep-mask by mi355_sdpa_mask_tiles and valid as long as that tensor is unchanged:
 *   live_tiles    forward: per (mask batch, mask head, block of 64 query rows) a bitmap of the
 *                 32-key tiles that hold at least one kept score; a workgroup walks only those
 *   live_tiles_t  backward (dK/dV): per (mask batch, mask head, block of 128 keys) a bitmap of
 *                 the 64-row query tiles that hold at least one kept score
 * Both optional; ignored together with is_causal, a window, or more than 32768 keys. */
typedef struct mi355_sdpa_mask_spec {
  int32_t window;
  int32_t sink_keys;
  const float* sink_logit;
  const uint32_t* live_tiles;
  const uint32_t* live_tiles_t;
  int32_t n_sink_logits;
  float softcap;
  const float* alibi_slopes;
  const float* key_bias;
  const float* key_weight;
  const int32_t* doc_ids_q;
  const int32_t* doc_ids_k;
  int32_t doc_ids_sorted;
  const int32_t* mask_verdict; /* optional, with a bias / keep-mask: what mi355_sdpa_mask_verdict wrote
                                  about that tensor.  The call is then put on the stream as a pair of
                                  kernels - with the mask, and with the causal flag, the window and
                                  key counts - whose first instructions read the verdict: a mask that is
                                  the keep-everything or the causal pattern or a sliding window with
                                  sink keys (each with or without right padding) is never read.  Matrix-op kernels for 16-bit inputs, head dims up to
                                  128 (the forward: up to 256), a mask with a row per query, nothing else
                                  shaping the scores; every other call uses the mask itself           */
} mi355_sdpa_mask_spec;

typedef struct mi355_sdpa_fwd_params {
  mi355_sdpa_tensor q;    /* (B,Hq,L,E)                                               */
  mi355_sdpa_tensor k;    /* (B,Hkv,S,E)   Hq % Hkv == 0; query head h reads h/(Hq/Hkv) */
  mi355_sdpa_tensor v;    /* (B,Hkv,S,Dv)                                             */
  mi355_sdpa_tensor out;  /* (B,Hq,L,Dv)   same dtype as q                            */
  float* lse;             /* (B,Hq,L) contiguous float32, natural log; may be NULL    */
  mi355_sdpa_tensor bias; /* optional additive bias or bool keep-mask, sizes (B,Hq,L,S),
                             stride 0 on broadcast dims.  A BOOL bias (1 byte per score,
                             non-zero = keep, zero = the score is -inf) is an extension of
                             this boundary: the reference's operator only ever sees additive
                             masks, because its caller turns a bool mask into 0 / -inf first
                             (decompositions.py:2101-2102); here that conversion, a pass over
                             L*S elements, is left out and the kernels read the bytes        */
  int32_t bias_dtype;     /* F32/F16/BF16/BOOL                                        */
  const int32_t* kv_lens; /* optional (B,): key j of batch b takes part iff j<kv_lens[b] */
  const uint8_t* dropout_keep; /* optional (B,Hq,L,S), 1 = keep: contiguous, or with rows
                                  dropout_keep_ld bytes apart (below)                  */
  float dropout_p;
  int32_t dtype;          /* dtype of q/k/v/out                                       */
  int32_t is_causal;      /* lower-triangular, anchored top-left (also when L != S)   */
  float scale;            /* multiplies Q K^T in float32                              */
  int32_t force_kernel;   /* 0 = library picks; else enum mi355_sdpa_kernel           */
  mi355_sdpa_mask_spec mask; /* all zero = none                                       */
  void* workspace;        /* optional: mi355_sdpa_fwd_workspace_bytes() bytes, 256-aligned.  With it,
                             a call with few query rows and few (batch, kv head) pairs splits its
                             keys over more workgroups (partial results here, merged by a second
                             kernel); without it the same call runs unsplit                    */
  size_t workspace_bytes;
  int64_t dropout_keep_ld; /* 0, or the bytes from one row of dropout_keep to the next (>= S; the
                              (B,Hq,L) rows stay densely packed at that pitch, the last row
                              included).  The matrix-op kernels for 16-bit inputs read the bytes a
                              dword at a time and need rows that start on dwords: a caller whose S
                              is no multiple of 4 pads the rows to one, or the call runs in the
                              generic kernels                                                */
} mi355_sdpa_fwd_params;

typedef struct mi355_sdpa_bwd_params {
  mi355_sdpa_tensor grad_out; /* (B,Hq,L,Dv) */
  mi355_sdpa_tensor q, k, v, out;
  const float* lse;           /* (B,Hq,L) contiguous float32                          */
  mi355_sdpa_tensor grad_q;   /* (B,Hq,L,E)                                           */
  mi355_sdpa_tensor grad_k;   /* (B,Hkv,S,E)   summed over each query-head group      */
  mi355_sdpa_tensor grad_v;   /* (B,Hkv,S,Dv)                                         */
  mi355_sdpa_tensor bias;     /* as in forward                                        */
  int32_t bias_dtype;
  mi355_sdpa_tensor grad_bias; /* optional (B,Hq,L,S), dtype of q.  The matrix-op kernels for 16-bit
                                  inputs write it four keys at a time: S a multiple of 4, or rows
                                  padded to one (a row stride >= S rounded up to 4 is the caller's
                                  word that every row, the last included, has that room)       */
  const int32_t* kv_lens;
  const uint8_t* dropout_keep;
  float dropout_p;
  int32_t dtype;
  int32_t is_causal;
  float scale;
  void* workspace;            /* mi355_sdpa_bwd_workspace_bytes() bytes, 256-aligned  */
  size_t workspace_bytes;
  int32_t force_kernel;
  mi355_sdpa_mask_spec mask;  /* as in forward                                          */
  float* grad_sink_logit;     /* optional, shape of mask.sink_logit: its gradient       */
  int64_t dropout_keep_ld;    /* as in forward                                          */
} mi355_sdpa_bwd_params;

typedef struct mi355_sdpa_decode_params {
  mi355_sdpa_tensor q;      /* (B,Hq,Lq,D) bf16/f16/f32, D = 64, 128 or 256, Lq*Hq/Hkv <= 16.
                               The query is carried exactly (bf16), with 12 to 16 significant
                               bits (f16) or with 16 (f32; 12 at D = 256 with more than 8
                               rows per kv head): see decode_fp8kv.hip                     */
  mi355_sdpa_tensor k;      /* (B,Hkv,S,D)  fp8 e4m3fn, 1 byte per element             */
  mi355_sdpa_tensor v;      /* (B,Hkv,S,D)  fp8 e4m3fn                                 */
  const float* k_scale;     /* (B,Hkv) contiguous: real K = fp8 value * k_scale        */
  const float* v_scale;     /* (B,Hkv)                                                 */
  const int32_t* kv_lens;   /* (B,) or NULL (= S everywhere)                           */
  mi355_sdpa_tensor out;    /* (B,Hq,Lq,D) dtype of q                                  */
  float* lse;               /* (B,Hq,Lq) float32 or NULL                               */
  int32_t q_dtype;
  float scale;
  int32_t num_splits;       /* 0 = library picks; N > 0: cut a full-length sequence into
                               about N pieces at most (fewer, larger partial results)  */
  void* workspace;          /* mi355_sdpa_decode_workspace_bytes() bytes               */
  size_t workspace_bytes;
} mi355_sdpa_decode_params;

/* ---- kernels -------------------------------------------------------------------------- */

/* Fused forward: O = softmax(scale*Q K^T + causal + bias) V and LSE.
 * Stands in for the device kernel launched at
 *   torch_neuronx/neuron_dynamo_backend/decompositions.py:2233-2262 (_compute_attention_nki)
 * and, for inputs the flash kernel refuses, for the math path
 *   torch_neuronx/_sdpa_math.py:51-95 (compute_attention). */
int mi355_sdpa_fwd(const mi355_sdpa_fwd_params* p, void* stream);
/* Bytes of workspace with which this forward call would split its keys (0: it would not).  No
 * counterpart in the reference; the workspace is optional. */
size_t mi355_sdpa_fwd_workspace_bytes(const mi355_sdpa_fwd_params* p);

/* Fused backward: dQ, dK, dV (dK/dV already reduced over each GQA group), optional dBias.
 * Stands in for decompositions.py:2467-2477 (_compute_attention_backward_nki),
 * _sdpa_math.py:98-176 (compute_attention_backward) and decompositions.py:2569-2599
 * (_reduce_gqa_gradients). */
int mi355_sdpa_bwd(const mi355_sdpa_bwd_params* p, void* stream);
/* Bytes of workspace this backward call needs: the row terms (rowsum(dO * O) and the log-sum-exp in
 * the log2 domain), and for a call with few key blocks the float32 partial dK / dV rows of the
 * workgroups that share a key block.  Ask per call: the size depends on every shape. */
size_t mi355_sdpa_bwd_workspace_bytes(const mi355_sdpa_bwd_params* p);

/* Decode-step attention over an fp8 e4m3 K/V cache with per-sequence lengths.
 * No counterpart in the reference (it has no fp8 attention path); defined as
 * compute_attention (_sdpa_math.py:51-95) on the dequantised cache with a key-padding bias. */
int mi355_sdpa_decode_fp8kv(const mi355_sdpa_decode_params* p, void* stream);
size_t mi355_sdpa_decode_workspace_bytes(const mi355_sdpa_decode_params* p);

/* The same decode step for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid it).  No counterpart in the reference.
 * p->workspace and p->workspace_bytes are ignored: partial results and step counts go to a
 * static device array of MI355_SDPA_DECODE_STATIC_SCRATCH_BYTES that every GPU holds from the
 * first call on it until the process ends.  A call that would need more scratch than that
 * (mi355_sdpa_decode_workspace_bytes tells) fails with MI355_SDPA_ERR_UNSUPPORTED.  The entry
 * point calls no allocating routine; the caller passes inputs and outputs as for
 * mi355_sdpa_decode_fp8kv, and the results are the same bit for bit.  All calls on one GPU
 * share the array: calls that overlap there (different streams, different threads) race; keep
 * them on one stream or order them with events.  The first call on a device looks the array's
 * address up (hipGetSymbolAddress): make it outside a stream capture. */
#define MI355_SDPA_DECODE_STATIC_SCRATCH_BYTES (32u << 20)
int mi355_sdpa_decode_fp8kv_static(const mi355_sdpa_decode_params* p, void* stream);

/* Row summary of an attention mask (L rows of S keys, unit stride over keys, row_stride in
 * elements; bool, or float with 0 = keep and -inf = drop): rows_out receives four int32 per row
 *   { last kept key, number of kept keys (-1 if some value is neither 0 nor -inf), length of the
 *     kept run starting at key 0, first key of the kept run ending at the last kept key }
 * from which the host recognises masks that a kernel can generate by itself (causal, sliding
 * window with sink keys, keep-everything) and calls the unmasked kernels instead.  The run-time
 * stand-in for the causal-mask recovery of
 *   torch_neuronx/neuron_dynamo_backend/fx/passes/sdpa_causal_mask.py:162-289 (SdpaCausalMaskRewrite). */
int mi355_sdpa_mask_rows(const void* mask, int32_t dtype, int64_t L, int64_t S, int64_t row_stride,
                         int32_t* rows_out, void* stream);

/* The same decision taken on the device, with no trip to the host: row summaries of every (mask
 * batch, row) and a verdict, in `verdict` (mi355_sdpa_mask_verdict_words(mask) int32 of device
 * memory; 0 = this mask cannot have one: it depends on the head, its keys are not unit-stride):
 *   verdict[0] kind: 0 not a pattern, 1 keep-everything, 2 causal, 3 sliding window with sink keys
 *   verdict[1] window, verdict[2] sink keys, verdict[3] 1 if some batch keeps fewer than S keys
 *   verdict[8 + b] keys of batch b that take part (right padding becomes a key count under every kind)
 * `mask` is the bias / keep-mask expanded to (B,Hq,L,S), stride 0 on broadcast dims.  Nothing
 * synchronises: the call records into a HIP graph in front of the attention call that is given
 * the verdict (mi355_sdpa_mask_spec.mask_verdict), and then follows a mask that is updated in place
 * between replays.  Stand-in, like mi355_sdpa_mask_rows, for
 *   torch_neuronx/neuron_dynamo_backend/fx/passes/sdpa_causal_mask.py:162-289. */
size_t mi355_sdpa_mask_verdict_words(const mi355_sdpa_tensor* mask, int32_t dtype);
int mi355_sdpa_mask_verdict(const mi355_sdpa_tensor* mask, int32_t dtype, int32_t* verdict, void* stream);

/* Tile skip tables of a bias / keep-mask (sizes (B,Hq,L,S), stride 0 on broadcast dims, unit stride
 * over keys, rows and data dword aligned as the MFMA kernels want them; bool, or float where
 * -inf = dropped): which 64-row x 32-key blocks hold at least one kept score.  The mask's own
 * batch and head extents count (a broadcast dim has extent 1).  Layouts, in uint32 words:
 *   live_tiles    [batch][head][ceil(L/64)][W],   W  = ceil(ceil(S/32)/32), bit t of a row block =
 *                 key tile t (word t/32, bit t%32)
 *   live_tiles_t  [batch][head][ceil(S/128)][Wt], Wt = ceil(ceil(L/64)/32), bit q of a key block =
 *                 query tile q
 * mi355_sdpa_mask_tiles_words returns the two sizes (words = 0: the mask cannot have tables).
 * No counterpart in the reference as a function: its templated kernel eliminates dropped tiles
 * when the kernel is rendered (flex_attention.py.jinja:15-33); here the mask is data. */
int mi355_sdpa_mask_tiles_words(const mi355_sdpa_tensor* bias, int32_t bias_dtype, size_t* words, size_t* words_t);
int mi355_sdpa_mask_tiles(const mi355_sdpa_tensor* bias, int32_t bias_dtype, uint32_t* live_tiles,
                          uint32_t* live_tiles_t, void* stream);

/* ---- host logic (no GPU needed) --------------------------------------------------------- */

/* Backend choice for F.scaled_dot_product_attention.  Rules of
 *   torch_neuronx/csrc/aten/SdpBackendSelection.cpp:14-68 (_fused_sdp_choice_neuron):
 * overrideable (4) for on-device, 4-D, concrete, non-empty q/k/v; otherwise math (0). */
int mi355_sdpa_choose_backend(const mi355_sdpa_desc* d);

/* Operator-boundary validation with the reference's messages.  Follows
 *   torch_neuronx/csrc/core/dispatch/NeuronDispatcher.cpp:2377-2459 (DispatchSdpaFwdImpl).
 * Returns 0 or MI355_SDPA_ERR_INVALID and writes the message (NUL-terminated) to msg. */
int mi355_sdpa_validate(const mi355_sdpa_desc* d, char* msg, size_t msg_len);

/* Strides of an output that keeps the dimension order of a reference tensor: the rule of
 * at::native::alloc_with_matching_layout used at NeuronDispatcher.cpp:2485-2491 and
 * :2554-2558 (dims sorted by descending stride of ref, dense strides for out_sizes). */
int mi355_sdpa_out_strides(const int64_t ref_sizes[4], const int64_t ref_strides[4],
                           const int64_t out_sizes[4], int64_t out_strides[4]);

/* Kernel eligibility: which kernel family serves a forward / backward call.  The analogue
 * of decompositions.py:2161-2207 (_can_use_nki_flash_attention) and :2371-2424
 * (_can_use_nki_flash_attention_backward) for this library's own kernels.
 * Returns an enum mi355_sdpa_kernel. */
int mi355_sdpa_can_use_fused_fwd(const mi355_sdpa_desc* d);
int mi355_sdpa_can_use_fused_bwd(const mi355_sdpa_desc* d);

/* Message of the last failing call on this thread ("" if none). */
const char* mi355_sdpa_last_error(void);
int mi355_sdpa_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MI355_SDPA_H */
