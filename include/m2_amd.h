/* libm2_amd.so -- C ABI of the MI355X (gfx950) Monarch-Mixer forward kernels.
 *
 * Every entry point takes raw device pointers, sizes and a HIP stream (as void*; pass 0 for the
 * null stream) and enqueues work on that stream without synchronising.  The library allocates no
 * device memory and keeps no device state: inputs, outputs and workspaces belong to the caller and
 * must stay valid until the stream has run the enqueued kernels.  Return value: M2_OK (0) or a
 * negative M2_ERR_* code, with a human-readable message available from m2_last_error() on the
 * calling thread.  All matrices are dense and contiguous in the layouts stated per argument.
 *
 * The reference (HazyResearch/m2) binds its optional native kernels through the pybind11 module
 * `flashmm` (csrc/flashmm/flash_mm.cpp:364-368: mm_block_fwd, hyena_filter_fwd,
 * exp_mod_in_place_fwd) and otherwise runs the path as PyTorch ops.  The entry points below are
 * what a binding for the same path would call; each cites the reference interface it stands in for.
 */
#ifndef M2_AMD_H_
#define M2_AMD_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define M2_AMD_VERSION 100 /* major*10000 + minor*100 + patch */

#define M2_OK 0
#define M2_ERR_ARG (-1)         /* null pointer, non-positive size, bad enum */
#define M2_ERR_UNSUPPORTED (-2) /* a size the kernels have no plan for */
#define M2_ERR_LAUNCH (-3)      /* HIP reported an error at launch */

#define M2_DTYPE_F32 0
#define M2_DTYPE_BF16 1

int m2_version(void);
const char* m2_last_error(void);

/* ---------------------------------------------------------------------------------------------
 * Implicit long-filter generation (HyenaFilter.filter / filter_rev + ExponentialModulation).
 * Stands in for: bert/src/mm/hyena_utils.py:201-217 (filter, filter_rev), :50-63 (Sin),
 * :110-112 (modulation) and :231-236 (bidirectional padding/flip); native counterpart in the
 * reference: flashmm.hyena_filter_fwd + exp_mod_in_place_fwd (csrc/flashmm/flash_mm.cpp:301-362).
 * ------------------------------------------------------------------------------------------- */
typedef struct m2_hyena_filter_params {
  const float* z;      /* (L, emb_dim)  pos_emb.z[0, :L]                                  */
  const float* t;      /* (L)           pos_emb.t[0, :L, 0]                               */
  const float* freq;   /* (order)       Sin.freq (one tensor shared by all activations)   */
  const float* deltas; /* (d)           modulation.deltas                                 */
  const float* w0;     /* (order, emb_dim)  implicit_filter.0.weight                      */
  const float* b0;     /* (order)           implicit_filter.0.bias                        */
  const float* w1;     /* (order, order)    implicit_filter.2.weight                      */
  const float* b1;     /* (order)                                                          */
  const float* w2;     /* (order, order)    implicit_filter.4.weight                      */
  const float* b2;     /* (order)                                                          */
  const float* w3;     /* (d, order)        implicit_filter.6.weight (no bias)            */
  const float* rw0;    /* same seven tensors of implicit_filter_rev; all NULL when the     */
  const float* rb0;    /* filter is not bidirectional                                      */
  const float* rw1;
  const float* rb1;
  const float* rw2;
  const float* rb2;
  const float* rw3;
} m2_hyena_filter_params;

/* Bytes of workspace m2_hyena_filter_fwd needs for `nfilters` filters of length L and width d: the last hidden
 * layer's activations (2 nfilters L order fp32-sized values) and the weights re-split for the matrix cores
 * (2 nfilters x (2 layers x 3 bf16 parts x order^2 + 2 bf16 parts x d x order)). */
size_t m2_hyena_filter_workspace_bytes(int nfilters, int L, int d, int order);

/* taps[f] (d, 2L) fp32, f < nfilters:  taps[f][c][l]      = k_fwd[c][l]       for l < L
 *                                      taps[f][c][L + l]  = k_rev[c][L-1-l]   (0 if not bidirectional)
 * with k[c][l] = (W3 sin(f.(W2 sin(f.(W1 sin(f.(W0 z_l + b0)) + b1)) + b2)))[c] * (exp(-t_l |delta_c|) + shift),
 * f = w_mod * freq.  `params` is a HOST array of nfilters structs holding DEVICE pointers.
 * Supported: order == 128, 3 <= emb_dim <= 8, d % 64 == 0, L % 32 == 0. */
int m2_hyena_filter_fwd(const m2_hyena_filter_params* params, int nfilters, int L, int d, int order, int emb_dim,
                        float w_mod, float shift, float* workspace, float* taps, void* stream);

/* The same computation as m2_hyena_filter_fwd without the workspace argument.  This entry point has no
 * counterpart in the reference: it exists for callers that cannot allocate device memory around the call (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  The intermediate activations
 * go through a device array of M2_HYENA_FILTER_STATIC_SCRATCH_BYTES that is part of the library itself (every GPU
 * the library runs on holds one copy until the process ends); the call allocates and frees nothing.  Limit:
 * m2_hyena_filter_workspace_bytes(nfilters, L, d, order) must not exceed that size: 20 MiB holds both filters of a
 * mixer up to L = 8192, or one filter up to L = 16384, for every d <= 1536 (two filters at L = 8192 need 19,136,512
 * bytes at d = 768 and 20,709,376 at d = 1536); beyond it the call fails with M2_ERR_UNSUPPORTED.  All calls on one GPU share
 * the array: two such calls whose kernels may overlap on the same GPU (different streams, or different host threads
 * on different streams) race; calls on one stream are ordered and safe.  The first call on a device looks up the
 * array's device address (hipGetSymbolAddress): make that call outside a stream capture. */
#define M2_HYENA_FILTER_STATIC_SCRATCH_BYTES (20u << 20)
int m2_hyena_filter_fwd_static(const m2_hyena_filter_params* params, int nfilters, int L, int d, int order,
                               int emb_dim, float w_mod, float shift, float* taps, void* stream);

/* All implicit filters of a batch of mixers -> the spectra m2_mixer_core_fwd reads, in one call: the whole of
 * HyenaFilter.filter / filter_rev (+ modulation), the bidirectional window, the skip weight and rfft(k) / 2L for
 * every mixer of a model at once (bert/src/mm/monarch_mixer_sequence_mixer.py:120-139 with
 * bert/src/mm/hyena_utils.py:201-236 and :24-33; the reference's native filter kernel is batched over filters the
 * same way, csrc/flashmm/flash_mm.cpp:301-338).  Same arithmetic as m2_hyena_filter_fwd followed by
 * m2_filter_spectrum_fwd per mixer, in three or four launches for ALL mixers; for L <= 512 the output projection,
 * the decay and the transform are one kernel and the taps never exist in memory.
 * params_dev  DEVICE array of nmixers * filters_per_mixer structs (of device pointers): filter_fn of mixer 0,
 *             filter_fn2 of mixer 0 (when filters_per_mixer == 2), filter_fn of mixer 1, ...  All filters share L, d,
 *             order, emb_dim; a filter is bidirectional when its rw0 .. rw3 are non-null.  The library cannot check
 *             pointers that live in device memory: the caller guarantees the forward-MLP pointers are valid.
 * skip_dev    DEVICE array of nmixers * filters_per_mixer pointers to the (d) fp32 skip weights (filter_fn.bias),
 *             entries may be null; the array itself may be NULL (no skip weights).
 * workspace   m2_mixer_filters_workspace_bytes(...) bytes of device memory, 256-byte aligned.
 * spec        nmixers consecutive buffers of m2_filter_spectrum_bytes(d, L) bytes.
 * At most 65535 MLPs per call (two per filter): nmixers * filters_per_mixer * 2 <= 65535. */
size_t m2_mixer_filters_workspace_bytes(int nmixers, int filters_per_mixer, int L, int d, int order);
int m2_mixer_filters_fwd(const m2_hyena_filter_params* params_dev, const float* const* skip_dev, int nmixers,
                         int filters_per_mixer, int L, int d, int order, int emb_dim, float w_mod, float shift,
                         void* workspace, float* spec, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Long convolution: filter spectra and the fused mixer core.
 * Stand in for: bert/src/mm/hyena_utils.py:16-42 (fftconv_ref), :219-248 (HyenaFilter.forward) and
 * bert/src/mm/monarch_mixer_sequence_mixer.py:112-147 (short conv, gates, two long convs, add);
 * native counterpart in the reference: flashmm.mm_block_fwd (csrc/flashmm/flash_mm.cpp:70-226).
 * ------------------------------------------------------------------------------------------- */

/* 1 if sequence length L is supported: a power of two in [128, 32768] (one LDS-resident transform per
 * row up to 1024, two half-length transforms per row for 2048 .. 16384; at 32768 each of the two real signals
 * of a row is convolved on its own in polyphase form, again as two LDS-resident half transforms). */
int m2_fftconv_supported_seqlen(int L);

/* Bytes of the opaque spectrum buffer for d channels and sequence length L (both filters): 16 d L, the size of
 * the four L-tap fp32 filters it is made from.  Always ask. */
size_t m2_filter_spectrum_bytes(int d, int L);

/* taps1, taps2: (d, 2L) fp32 bidirectional taps of filter_fn and filter_fn2 (taps2 may be NULL:
 * treated as zero).  D1, D2: (d) fp32 skip weights (`filter_fn.bias`, `filter_fn2.bias`; either
 * may be NULL = 0): the reference's "+ u * D" term (hyena_utils.py:35) equals adding D to tap 0,
 * which is done here.  spec: m2_filter_spectrum_bytes(d, L) bytes; receives
 * rfft(taps + D e0, 2L)/(2L) of both filters (at L = 32768: of their even and odd samples) in the order
 * m2_mixer_core_fwd reads them. */
int m2_filter_spectrum_fwd(const float* taps1, const float* taps2, const float* D1, const float* D2, float* spec,
                           int d, int L, void* stream);

/* y[c,b,:] = (fftconv(a; k1)[:L] + D1[c] a) * sc(x2) + fftconv(u; k2)[:L] + D2[c] u,
 *            a = sc(v) * sc(x1),  sc = depthwise 3-tap causal conv + bias (cross-correlation,
 *            out[t] = bias + w0 in[t-2] + w1 in[t-1] + w2 in[t]);  D1, D2 are already inside spec.
 * xproj  (3d, B, L)  in_linear output, CHANNEL-MAJOR, channels [0,d)=x1, [d,2d)=x2, [2d,3d)=v; act_dtype
 * proj_bias (3d)     fp32, added to xproj as it is read (the in_linear bias, so the projection GEMM can
 *                    run without a bias pass); NULL when xproj already contains it
 * u      (d, B, L)   fp32 layer input, channel-major; NULL when there is no residual long conv
 * short_w (3d, 3), short_b (3d)  fp32
 * spec   from m2_filter_spectrum_fwd with the same d and L
 * y      (d, B, L)   act_dtype (M2_DTYPE_F32 or M2_DTYPE_BF16); FFT arithmetic is fp32 either way */
int m2_mixer_core_fwd(const void* xproj, const float* proj_bias, const float* u, const float* short_w,
                      const float* short_b, const float* spec, void* y, int B, int L, int d, int act_dtype,
                      void* stream);

/* Plain long convolution y[c,b,:] = fftconv(x[c,b,:]; k1)[:L] + D1[c] x[c,b,:] with the first filter
 * of `spec` (HyenaFilter.forward on its own, bert/src/mm/hyena_utils.py:219-248).
 * x, y (d, B, L) channel-major, act_dtype. */
int m2_fftconv_fwd(const void* x, const float* spec, void* y, int B, int L, int d, int act_dtype, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Block-diagonal ("Monarch") linear layers of the GLU MLP, bf16 MFMA with fp32 accumulation.
 * Stand in for: bert/src/mm/blockdiag_multiply.py:49-60 (BlockdiagMultiply.forward, bf16 under
 * autocast), bert/src/mm/structured_linear.py:65-69 (bias add) and bert/src/bert_layers.py:482-506
 * (GLU, residual).  The reference has no native kernel for these (torch.bmm).
 * ------------------------------------------------------------------------------------------- */

/* out[m, j] = gelu_erf(h[m, j]) * h[m, I + j],  h = blockdiag_multiply(x, w),  j < I = intermediate.
 * x (M, in_features) bf16 row-major; w (nblocks, 2I/nblocks, in_features/nblocks) bf16 (the
 * `gated_layers.weight` tensor); out (M, I) bf16.  Needs nblocks even, (in/nblocks) % 8 == 0,
 * (2I/nblocks) % 8 == 0 (block sizes off the kernels' 64-wide tile grid, such as the 240-wide blocks of the
 * reference's 960-wide model, run on a masked variant of the general kernel). */
int m2_blockdiag_glu_fwd(const void* x, const void* w, void* out, int M, int in_features, int intermediate,
                         int nblocks, void* stream);

/* out = blockdiag_multiply(x, w) (+ bias) (+ residual).
 * x (M, in_features) bf16; w (nblocks, out/nblocks, in/nblocks) bf16; bias (out_features) fp32 or NULL;
 * residual (M, out_features) bf16 or NULL; out (M, out_features) of out_dtype (M2_DTYPE_F32 / _BF16).
 * Needs (in/nblocks) % 8 == 0, (out/nblocks) % 8 == 0. */
int m2_blockdiag_linear_fwd(const void* x, const void* w, const float* bias, const void* residual, void* out, int M,
                            int in_features, int out_features, int nblocks, int out_dtype, void* stream);

/* The fp32 form: out = blockdiag_multiply(x, w) (+ bias) with fp32 operands, exact fp32 products and fp32
 * accumulation -- what the reference computes when BlockdiagLinear is called with fp32 tensors outside CUDA autocast
 * (bert/src/mm/blockdiag_multiply.py:50 casts to bf16 only under autocast).  x (M, in_features) fp32; w (nblocks,
 * out/nblocks, in/nblocks) fp32; bias (out_features) fp32 or NULL; out (M, out_features) fp32.
 * Needs (in_features / nblocks) % 8 == 0. */
int m2_blockdiag_linear_f32_fwd(const float* x, const float* w, const float* bias, float* out, int M, int in_features,
                                int out_features, int nblocks, void* stream);

/* The whole GLU MLP up to the LayerNorm input in one kernel, the (M, 2I) and (M, I) intermediates never leaving the
 * chip:  out = blockdiag_multiply(gelu_erf(h[:, :I]) * h[:, I:], w_out) (+ bias) (+ residual),
 * h = blockdiag_multiply(x, w_gated)  (bert/src/bert_layers.py:482-506: gated_layers, act, wo, residual).  Same
 * arithmetic as m2_blockdiag_glu_fwd followed by m2_blockdiag_linear_fwd (bf16 operands, fp32 accumulation, the
 * gated values rounded to bf16 between the two products).
 * The kernel streams the weights from L2 once per 128-row tile and is bound by that stream, so it reads them from a
 * packed copy in which every 1 KB the kernel moves at a time is contiguous: m2_mlp_fused_pack writes it, once per
 * set of weights (w_gated (nblocks, 2I/nblocks, in/nblocks) bf16, gated_layers.weight; w_out (nblocks, in/nblocks,
 * I/nblocks) bf16, wo.weight; packed: m2_mlp_fused_packed_bytes bytes of device memory, 16-byte aligned; the size is
 * that of the two weights together).  m2_mlp_fused_fwd: x (M, in_features) bf16; w_packed as written by
 * m2_mlp_fused_pack for the same in_features / intermediate / nblocks; bias (in_features) fp32 or NULL; residual
 * (M, in_features) bf16 or NULL; out (M, in_features) of out_dtype.  m2_mlp_fused_supported returns 1 for the shapes
 * the kernel is built for (nblocks == 4, in_features == 768, intermediate % 128 == 0); for others
 * m2_mlp_fused_packed_bytes returns 0, the other two return M2_ERR_UNSUPPORTED and the caller uses the two separate
 * entry points. */
int m2_mlp_fused_supported(int in_features, int intermediate, int nblocks);
long m2_mlp_fused_packed_bytes(int in_features, int intermediate, int nblocks);
int m2_mlp_fused_pack(const void* w_gated, const void* w_out, void* packed, int in_features, int intermediate,
                      int nblocks, void* stream);
int m2_mlp_fused_fwd(const void* x, const void* w_packed, const float* bias, const void* residual, void* out, int M,
                     int in_features, int intermediate, int nblocks, int out_dtype, void* stream);

/* The gated block-diagonal GEMM with the GLU on its accumulators for 384-wide blocks, from packed weights:
 * out (M, I) bf16 = gelu_erf(h[:, :I]) * h[:, I:], h = blockdiag_multiply(x, w_gated)  (bert/src/bert_layers.py:494-502,
 * bert/src/mm/blockdiag_multiply.py:49-60).  Same arithmetic and result layout as m2_blockdiag_glu_fwd; the x rows stay
 * in registers and the weights stream through LDS from a packed copy in which every 1 KB the kernel moves at a time is
 * contiguous.  m2_glu_stream_pack writes that copy once per set of weights (w_gated (nblocks, 2I/nblocks,
 * in/nblocks) bf16, gated_layers.weight; packed: m2_glu_stream_packed_bytes bytes of device memory, 16-byte aligned,
 * the size of the weight, or of the weight with its blocks padded to 256 columns when they are narrower).  m2_glu_stream_fwd: x (M, in_features) bf16, w_packed as written by m2_glu_stream_pack for
 * the same shape, out (M, intermediate) bf16.  m2_glu_stream_supported returns 1 for the shapes the kernel is built for
 * (nblocks == 4, in_features / 4 == 384, 448 or a multiple of 8 in [224, 248], intermediate % 128 == 0); for others m2_glu_stream_packed_bytes returns 0, the
 * other two return M2_ERR_UNSUPPORTED and the caller uses m2_blockdiag_glu_fwd. */
int m2_glu_stream_supported(int in_features, int intermediate, int nblocks);
long m2_glu_stream_packed_bytes(int in_features, int intermediate, int nblocks);
int m2_glu_stream_pack(const void* w_gated, void* packed, int in_features, int intermediate, int nblocks, void* stream);
int m2_glu_stream_fwd(const void* x, const void* w_packed, void* out, int M, int in_features, int intermediate,
                      int nblocks, void* stream);

/* LayerNorm over the last dimension of x (M, d) fp32 (torch.nn.LayerNorm semantics, biased variance,
 * eps inside the root; bert/src/bert_layers.py:478-479,506 and :185-186,247).  Any of the three
 * outputs may be NULL: out_f32 (M, d) fp32, out_bf16 (M, d) bf16, out_channel_major (d, M) fp32 (the
 * layout m2_mixer_core_fwd reads its `u` in).  Needs d % 64 == 0, d <= 2048. */
int m2_layernorm_fwd(const float* x, const float* gamma, const float* beta, float eps, float* out_f32, void* out_bf16,
                     float* out_channel_major, int M, int d, void* stream);
/* The same for x (M, d) stored as bf16: what the reference's LayerNorm receives under CUDA autocast, where the sum
 * wo(...) + residual is a bf16 tensor (bert/src/bert_layers.py:504-506); statistics and outputs in fp32 as above. */
int m2_layernorm_bf16_fwd(const void* x, const float* gamma, const float* beta, float eps, float* out_f32,
                          void* out_bf16, float* out_channel_major, int M, int d, void* stream);

/* out = LayerNorm(blockdiag_multiply(x, w) + bias + residual) in one kernel: m2_blockdiag_linear_fwd followed by
 * m2_layernorm_fwd without the fp32 intermediate (bert/src/bert_layers.py:504-506: wo, dropout, residual,
 * layernorm).  Arguments as in those two; any of the three outputs may be NULL.
 * m2_blockdiag_linear_layernorm_supported returns 1 for the shapes the fused kernel covers: nblocks == 4,
 * (in_features / 4) % 64 == 0, (out_features / 4) % 32 == 0, out_features <= 768; for other shapes the fused
 * entry point returns M2_ERR_UNSUPPORTED and the caller uses the two separate entry points. */
int m2_blockdiag_linear_layernorm_supported(int in_features, int out_features, int nblocks);
int m2_blockdiag_linear_layernorm_fwd(const void* x, const void* w, const float* bias, const void* residual,
                                      const float* gamma, const float* beta, float eps, float* out_f32,
                                      void* out_bf16, float* out_channel_major, int M, int in_features,
                                      int out_features, int nblocks, void* stream);

/* Embedding sum + LayerNorm in one pass (BertEmbeddings.forward in eval mode, bert/src/bert_layers.py:191-252):
 * row m = b L + l:  e = word_emb[input_ids[m]] + type_emb[token_type_ids[m]] (+ pos_emb[position_ids[m]]),
 * out = LayerNorm(e) in the same three forms as m2_layernorm_fwd (any may be NULL).
 * input_ids (B, L) int64; token_type_ids (B, L) int64 or NULL (all zero); pos_emb NULL when the model has no
 * position embeddings, else position_ids (B, L) int64 or NULL (positions 0 .. L-1 in every sequence).
 * Tables are fp32 row-major: word_emb (vocab_size, d), type_emb (type_vocab_size, d), pos_emb (max_positions, d).
 * An index outside its table (the reference's nn.Embedding raises there) never reads foreign memory: the kernel
 * uses the nearest valid row instead and, when bad_index is not NULL, stores 1 to *bad_index (device memory, one
 * int, which the caller zeroed before the call and reads after the stream has run).  Without position_ids the
 * call fails with M2_ERR_ARG when L > max_positions.  Needs d % 64 == 0, d <= 2048. */
int m2_embed_layernorm_fwd(const long long* input_ids, const long long* token_type_ids, const long long* position_ids,
                           const float* word_emb, const float* type_emb, const float* pos_emb, int vocab_size,
                           int type_vocab_size, int max_positions, const float* gamma, const float* beta, float eps,
                           float* out_f32, void* out_bf16, float* out_channel_major, int* bad_index, int B, int L,
                           int d, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* M2_AMD_H_ */
