"""M2-BERT encoder stack (Monarch-Mixer branch) over the HIP kernels, module and state-dict names as
in the reference (bert/src/bert_layers.py:131-252 BertEmbeddings, :457-508 BertGatedLinearUnitMLP,
:511-599 BertLayer, :602-813 BertEncoder, :880-1021 BertModel).

`BertEncoder.forward` does not call its layers module by module: it runs one fused schedule per
layer so that no activation is transposed or re-read in between:

    h32 (M,d) f32, h16 (M,d) bf16, hT (d,M) f32   <- LayerNorm of the previous layer (three forms, one kernel)
    xproj (3d,M) bf16 = W_in h16^T                library GEMM, channel-major output (bias added by K2)
    spec              = filter spectra            K1 (hidden MLP, projection+decay) + spectrum FFT
    y (d,M) bf16      = mixer core(xproj, hT)     K2
    a (M,d) bf16      = y^T W_out^T + b           library GEMM
    g (M,I) bf16      = GLU(blockdiag(a, Wg))     K3
    s (M,d) f32       = blockdiag(g, Wo) + b + a  K3
    LayerNorm(s)      -> next layer's three forms

The individual modules keep working on their own (same call signatures as the reference) and give
the same numbers; they just pay for the layout changes the fused schedule avoids.
"""
from __future__ import annotations

from functools import partial
from typing import List, Optional

import torch
import torch.nn as nn

from . import ops
from .blockdiag import BlockdiagLinear
from .config import M2BertConfig
from .mixer import MonarchMixerSequenceMixing


class BertEmbeddings(nn.Module):
    def __init__(self, config: M2BertConfig):
        super().__init__()
        self.word_embeddings = nn.Embedding(config.vocab_size, config.hidden_size, padding_idx=config.pad_token_id)
        if config.use_positional_encodings:
            self.position_embeddings = nn.Embedding(config.max_position_embeddings, config.hidden_size)
        self.use_positional_encodings = config.use_positional_encodings
        self.token_type_embeddings = nn.Embedding(config.type_vocab_size, config.hidden_size)
        self.LayerNorm = nn.LayerNorm(config.hidden_size, eps=config.layer_norm_eps)
        self.dropout = nn.Dropout(config.hidden_dropout_prob)
        if config.use_positional_encodings:
            self.register_buffer("position_ids", torch.arange(config.max_position_embeddings).expand((1, -1)))
        self.register_buffer("token_type_ids", torch.zeros(config.max_position_embeddings, dtype=torch.long),
                             persistent=False)
        # set by the embedding kernel when an id lies outside its table (the kernel then reads the nearest valid
        # row); `check_indices()` reads it.  Not part of the state dict.
        self.register_buffer("_bad_index", torch.zeros(1, dtype=torch.int32), persistent=False)

    def check_indices(self) -> None:
        """Raises IndexError if a lookup since the last check used an id outside its table (nn.Embedding raises at
        the lookup in the reference; here the kernel flags it and this call, which waits for the stream, reports)."""
        ops.raise_on_bad_index(self._bad_index)

    def summed(self, input_ids=None, token_type_ids=None, position_ids=None, inputs_embeds=None,
               past_key_values_length: int = 0) -> torch.Tensor:
        """word + token-type (+ position) embeddings before the LayerNorm, (B, L, d) fp32."""
        if (input_ids is not None) == (inputs_embeds is not None):
            raise ValueError("Must specify either input_ids or input_embeds!")
        shape = input_ids.size() if input_ids is not None else inputs_embeds.size()[:-1]
        L = shape[1]
        if inputs_embeds is None:
            inputs_embeds = self.word_embeddings(input_ids)
        if token_type_ids is None:
            tt = self.token_type_embeddings.weight[0]            # all-zero type ids
            e = inputs_embeds + tt
        else:
            e = inputs_embeds + self.token_type_embeddings(token_type_ids)
        if self.use_positional_encodings:
            if position_ids is None:
                position_ids = self.position_ids[:, past_key_values_length:L + past_key_values_length]
            e = e + self.position_embeddings(position_ids)
        return e

    def forward(self, input_ids=None, token_type_ids=None, position_ids=None, inputs_embeds=None,
                past_key_values_length: int = 0) -> torch.Tensor:
        if self.training and self.dropout.p > 0:
            raise NotImplementedError("m2_amd is a forward/inference path: call .eval() first")
        o32, _, _ = self.forward_forms(input_ids, token_type_ids, position_ids, inputs_embeds, past_key_values_length,
                                       want_f32=True, want_bf16=False, want_channel_major=False)
        if not torch.cuda.is_current_stream_capturing():
            self.check_indices()
        return o32

    def forward_forms(self, input_ids=None, token_type_ids=None, position_ids=None, inputs_embeds=None,
                      past_key_values_length: int = 0, want_f32: bool = True, want_bf16: bool = True,
                      want_channel_major: bool = True):
        """The embedding LayerNorm written in the forms the first encoder layer reads, by one kernel:
        (B, L, d) fp32 | (B*L, d) bf16 | (d, B*L) fp32; forms not asked for are None."""
        if self.training and self.dropout.p > 0:
            raise NotImplementedError("m2_amd is a forward/inference path: call .eval() first")
        gamma, beta = self.LayerNorm.weight.detach().float(), self.LayerNorm.bias.detach().float()
        tables_f32 = self.word_embeddings.weight.dtype == torch.float32
        if input_ids is not None and inputs_embeds is None and past_key_values_length == 0 and tables_f32:
            # gather + sum + LayerNorm as one kernel
            B, L = input_ids.shape
            d = self.word_embeddings.weight.shape[1]
            pos = position_ids
            if pos is not None:
                pos = pos.expand(B, L).contiguous()
            o32, o16, oT = ops.embed_layernorm(
                input_ids.contiguous(), None if token_type_ids is None else token_type_ids.expand(B, L).contiguous(), pos,
                self.word_embeddings.weight.detach(), self.token_type_embeddings.weight.detach(),
                self.position_embeddings.weight.detach() if self.use_positional_encodings else None, gamma, beta,
                self.LayerNorm.eps, want_f32=want_f32, want_bf16=want_bf16, want_channel_major=want_channel_major,
                bad_index=self._bad_index)
        else:
            e = self.summed(input_ids, token_type_ids, position_ids, inputs_embeds, past_key_values_length).float()
            B, L, d = e.shape
            o32, o16, oT = ops.layernorm(e.reshape(B * L, d).contiguous(), gamma, beta, self.LayerNorm.eps,
                                         want_f32=want_f32, want_bf16=want_bf16, want_channel_major=want_channel_major)
        return (None if o32 is None else o32.view(B, L, d)), o16, oT


class BertGatedLinearUnitMLP(nn.Module):
    def __init__(self, config: M2BertConfig):
        super().__init__()
        if not config.use_monarch_mlp:
            raise NotImplementedError("only the Monarch (block-diagonal) GLU MLP is built")
        self.config = config
        self.is_padded = config.monarch_mixer_sequence_mixing
        linear_cls = partial(BlockdiagLinear, nblocks=config.monarch_mlp_nblocks)
        self.gated_layers = linear_cls(config.hidden_size, config.intermediate_size * 2, bias=False)
        self.act = nn.GELU(approximate="none")
        self.wo = linear_cls(config.intermediate_size, config.hidden_size)
        self.dropout = nn.Dropout(config.hidden_dropout_prob)
        self.layernorm = nn.LayerNorm(config.hidden_size, eps=config.layer_norm_eps)

    # True: wo + bias + residual + LayerNorm as one kernel (d <= 768).  Off by default: the 256 x 192-tile wo
    # kernel followed by the LayerNorm kernel measured faster on MI355X (9.06 against 9.13 ms per forward at
    # L = 8192, B = 4; 2.00 against 2.24 ms at L = 128, B = 32), although it writes and re-reads the fp32 sum.
    fuse_wo_layernorm = False
    # True: gated_layers, GLU and wo + bias + residual as one kernel that keeps the (M, I) intermediate on chip
    # (d = 768, four blocks; other shapes take the two kernels).  Measured on MI355X at M = 32768: 175 - 183 us against
    # 191 us for the two kernels it replaces.  It streams the weights from a packed copy (3.5 MB per layer at
    # I = 3072) that is rebuilt when the weights change.
    fuse_mlp = True
    _packed = None
    # True: the sum wo(...) + bias + residual goes to the LayerNorm as bf16 instead of fp32 -- the rounding the
    # reference's autocast path applies at this point (its wo output, residual and their sum are bf16 tensors) --
    # which halves the bytes written by the MLP kernel and read by the LayerNorm: -1.9 % per forward at L = 8192,
    # B = 4; per-layer deviation from the fp32 oracle 0.89 % instead of 0.78 % (max), end to end unchanged.
    bf16_presum = True

    def presum(self, a16: torch.Tensor) -> torch.Tensor:
        """a16 (M, d) bf16 -> wo(glu(a16)) + bias + a16, (M, d) fp32 (the LayerNorm input; bf16 with `bf16_presum`)."""
        sum_dtype = torch.bfloat16 if self.bf16_presum else torch.float32
        if self.fuse_mlp and ops.mlp_fused_supported(a16.shape[1], self.config.intermediate_size,
                                                     self.config.monarch_mlp_nblocks):
            wg, wo = self.gated_layers.weight_bf16(), self.wo.weight_bf16()
            # the packed copy the kernel streams: rebuilt whenever one of the bf16 copies has been rebuilt
            if self._packed is None or self._packed[0] is not wg or self._packed[1] is not wo:
                self._packed = (wg, wo, ops.mlp_fused_pack(wg, wo))
            return ops.mlp_fused(a16, wg, wo, self.wo.bias.detach().float().contiguous(), a16, out_dtype=sum_dtype,
                                 packed=self._packed[2])
        g = self.glu(a16)
        return ops.blockdiag_linear(g, self.wo.weight_bf16(), self.wo.bias.detach().float().contiguous(), a16,
                                    out_dtype=sum_dtype)

    # True: for 384-wide blocks (d = 1536, four blocks), 448-wide (d = 1792) and 240-wide ones (d = 960) the gated product + GLU runs as the kernel that keeps the x rows
    # in registers and streams packed weights through LDS (m2_glu_stream_fwd) instead of the LDS-tiled GEMM with a GLU
    # epilogue (m2_blockdiag_glu_fwd).  Same arithmetic; other shapes take the tiled kernel.
    stream_glu = True
    _packed_glu = None

    def glu(self, a16: torch.Tensor) -> torch.Tensor:
        """a16 (M, d) bf16 -> gelu(gate) * value of gated_layers(a16), (M, I) bf16."""
        wg = self.gated_layers.weight_bf16()
        if self.stream_glu and ops.glu_stream_supported(a16.shape[1], self.config.intermediate_size,
                                                        self.config.monarch_mlp_nblocks):
            if self._packed_glu is None or self._packed_glu[0] is not wg:      # rebuilt with the bf16 copy
                self._packed_glu = (wg, ops.glu_stream_pack(wg))
            return ops.glu_stream(a16, wg, packed=self._packed_glu[1])
        return ops.blockdiag_glu(a16, wg)

    def ln_params(self):
        return self.layernorm.weight.detach().float(), self.layernorm.bias.detach().float(), self.layernorm.eps

    def normed(self, a16: torch.Tensor, want_f32: bool, want_bf16: bool, want_channel_major: bool):
        """a16 (M, d) bf16 -> LayerNorm(wo(glu(a16)) + bias + a16) in the requested forms (f32 | None, bf16 | None,
        channel-major f32 | None).  With `fuse_wo_layernorm`, `wo` and the LayerNorm are one kernel where the shape
        allows it."""
        gamma, beta, eps = self.ln_params()
        w = self.wo.weight_bf16()
        nb, q, p = w.shape
        if self.fuse_wo_layernorm and ops.blockdiag_linear_layernorm_supported(nb * p, nb * q, nb):
            g = self.glu(a16)
            return ops.blockdiag_linear_layernorm(g, w, self.wo.bias.detach().float().contiguous(), a16, gamma, beta, eps,
                                                  want_f32=want_f32, want_bf16=want_bf16,
                                                  want_channel_major=want_channel_major)
        return ops.layernorm(self.presum(a16), gamma, beta, eps, want_f32=want_f32, want_bf16=want_bf16,
                             want_channel_major=want_channel_major)

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """fp32 input outside CUDA autocast runs in fp32 throughout, as the reference's modules do there
        (bert/src/bert_layers.py:482-508 with bert/src/mm/blockdiag_multiply.py:50 casting only under autocast);
        bf16 input or an enclosing autocast takes the bf16 kernels of the fused schedule."""
        if self.training and self.dropout.p > 0:
            raise NotImplementedError("m2_amd is a forward/inference path: call .eval() first")
        shape = hidden_states.shape
        gamma, beta, eps = self.ln_params()
        if hidden_states.dtype == torch.float32 and not torch.is_autocast_enabled():
            x = hidden_states.reshape(-1, shape[-1]).contiguous()
            h = self.gated_layers(x)                                   # fp32 block-diagonal kernel
            I = self.config.intermediate_size
            g = self.act(h[:, :I]) * h[:, I:]
            s = self.wo(g.contiguous()) + x
            o32, _, _ = ops.layernorm(s.contiguous(), gamma, beta, eps, want_f32=True)
            return o32.view(shape)
        a16 = hidden_states.reshape(-1, shape[-1]).to(torch.bfloat16).contiguous()
        o32, _, _ = self.normed(a16, True, False, False)
        return o32.view(shape)


class BertLayer(nn.Module):
    def __init__(self, config: M2BertConfig):
        super().__init__()
        if not config.monarch_mixer_sequence_mixing or not config.use_glu_mlp:
            raise NotImplementedError("only the Monarch-Mixer branch with the GLU MLP is built")
        self.monarch_mixer_sequence_mixing = True
        self.attention = MonarchMixerSequenceMixing(
            config.hidden_size, l_max=config.long_conv_l_max, hyena_kernel_lr=config.long_conv_kernel_learning_rate,
            bidirectional=config.bidirectional, hyena_lr_pos_emb=config.hyena_lr_pos_emb, hyena_w=config.hyena_w,
            hyena_w_mod=config.hyena_w_mod, hyena_wd=config.hyena_wd, hyena_emb_dim=config.hyena_emb_dim,
            hyena_filter_dropout=config.hyena_filter_dropout, hyena_filter_order=config.hyena_filter_order,
            residual_long_conv=config.residual_long_conv, hyena_training_additions=config.hyena_training_additions)
        self.mlp = BertGatedLinearUnitMLP(config)

    def forward(self, hidden_states, cu_seqlens=None, seqlen=None, subset_idx=None, indices=None, attn_mask=None,
                bias=None) -> torch.Tensor:
        # No autocast is forced here: like the reference's layer (bert/src/bert_layers.py:575-599) this runs in
        # whatever precision the caller set up -- fp32 input outside autocast stays fp32 end to end, bf16 input or an
        # enclosing torch.autocast("cuda", dtype=torch.bfloat16) takes the bf16 GEMM kernels.
        a, _ = self.attention(hidden_states)
        return self.mlp(a)

    def fused(self, h16: Optional[torch.Tensor], hT: Optional[torch.Tensor], B: int, L: int, want_f32: bool,
              spec: Optional[torch.Tensor] = None, spec_ready=None, after_core=None,
              h32: Optional[torch.Tensor] = None):
        """One layer of the fused schedule.  h16 (M,d) bf16, hT (d,M) f32 -> (f32 | None, bf16, (d,M) f32).
        `spec`: this layer's filter spectra when the caller has generated them already (`spec_ready`: the event
        the current stream must wait for before reading them); `after_core()` is called once the mixer core
        has been enqueued."""
        at = self.attention
        d = at.d_model
        if at.hyena_training_additions:      # extra input LayerNorm: needs the fp32 form, replaces h16 / hT
            _, h16, hT = at.pre_norm(h32, want_f32=False, want_bf16=True)
        w_in = at._cast("in_w", at.in_linear.weight, torch.bfloat16)
        w_out = at._cast("out_w", at.out_linear.weight, torch.bfloat16)
        b_out = at._cast("out_b", at.out_linear.bias, torch.bfloat16)
        # (3d, M) channel-major, bias added in the core.  Written as h16 @ W^T into the transposed view of the
        # output: the same product as W @ h16^T, for which the library picks a faster kernel (126 against 144 us at
        # M = 32768, d = 768)
        xproj = torch.empty(3 * d, B * L, dtype=torch.bfloat16, device=h16.device)
        torch.mm(h16, w_in.t(), out=xproj.t())
        if spec_ready is not None:
            torch.cuda.current_stream().wait_event(spec_ready)
        y = at.core(xproj.view(3 * d, B, L), hT.view(d, B, L) if at.residual_long_conv else None, B, L, spec=spec)
        if after_core is not None:
            after_core()
        a16 = torch.addmm(b_out, y.view(d, B * L).t(), w_out.t())                    # (M, d)
        pre = at.hyena_training_additions        # the next layer then reads the fp32 form only
        return self.mlp.normed(a16, want_f32, not pre, not pre)


class BertEncoder(nn.Module):
    """`use_hip_graph=True` captures the whole stack of layers into one HIP graph per input shape and replays
    it: at short sequence lengths the forward is launch-bound (about ten small kernels per layer) and the
    replay removes the per-launch host cost.  The graph holds device pointers of the weights (and of their
    cached bf16 copies): it is dropped by `load_state_dict` (of this module or of any module that contains
    it), `.to()` / `.cuda()` and `reset_graphs()`; call `reset_graphs()` after changing a parameter in place.
    Nothing in the captured region uses a memset."""

    UPFRONT_MAX_BYTES = 16 << 30
    # device memory one batched filter-generation call may use for its workspace (hidden activations; for L > 512
    # also the taps, 8 d L bytes per filter): the layers are generated in as few calls as stay below it
    FILTER_WORKSPACE_BYTES = 2 << 30

    def __init__(self, config: M2BertConfig, use_hip_graph: bool = False):
        super().__init__()
        self.layer = nn.ModuleList([BertLayer(config) for _ in range(config.num_hidden_layers)])
        self.monarch_mixer_sequence_mixing = config.monarch_mixer_sequence_mixing
        self.num_attention_heads = config.num_attention_heads
        self.use_hip_graph = use_hip_graph
        self._graphs = {}
        # Filter generation depends on the weights only.
        # batch_filters = True (default): the filters of ALL layers are generated at the start of the forward by
        #   one library call per group of layers (m2_mixer_filters_fwd: a few launches for all of them; groups are
        #   as large as FILTER_WORKSPACE_BYTES allows) -- on a second stream (default priority) beside the layers
        #   unless overlap_filters is False, each layer waiting for its group.  Holds all spectra at once (16 d L
        #   bytes per layer: 100 MB at L = 8192, d = 768) and is used while they stay below UPFRONT_MAX_BYTES.
        # batch_filters = False, or spectra beyond UPFRONT_MAX_BYTES, or a layer with cache_filters: per layer, with
        #   overlap_filters =
        #   "upfront"  all layers' spectra one after the other on the second stream from the start of the forward;
        #   True       the spectra of layer i + 1 behind the mixer core of layer i;
        #   False      in line, on the main stream;
        #   None       "upfront" while all layers' spectra together stay below UPFRONT_MAX_BYTES, else True.
        self.batch_filters = True
        self.overlap_filters = None
        self._filter_stream = None
        self._filter_table = None
        # nn.Module.load_state_dict of a parent never calls a child's load_state_dict, but it does run the
        # post hooks of every module it recursed into: new weights drop the captured graphs
        self.register_load_state_dict_post_hook(BertEncoder._drop_graphs_after_load)

    # -- graph bookkeeping -------------------------------------------------------------------
    def reset_graphs(self) -> None:
        self._graphs = {}

    def _apply(self, fn, *args, **kwargs):
        self._graphs = {}
        return super()._apply(fn, *args, **kwargs)

    @staticmethod
    def _drop_graphs_after_load(module, incompatible_keys) -> None:
        module._graphs = {}

    # -- the fused schedule --------------------------------------------------------------------
    def _run_layers(self, h32: Optional[torch.Tensor], B: int, L: int, all_layers: bool,
                    h16: Optional[torch.Tensor] = None, hT: Optional[torch.Tensor] = None) -> List[torch.Tensor]:
        """h32 (M, d) fp32 contiguous -> list of (M, d) fp32: every layer's output, or only the last.  A caller
        that already holds the bf16 and the channel-major fp32 form of the input passes them as h16 / hT (and
        may then pass h32 = None)."""
        with torch.autocast("cuda", enabled=False):
            pre_norm = self.layer[0].attention.hyena_training_additions       # layers then start from the fp32 form
            if not pre_norm:
                if h16 is None:
                    h16 = h32.to(torch.bfloat16)
                if hT is None:
                    hT = h32.t().contiguous()
            outs = []
            n = len(self.layer)
            o32 = h32
            cur = torch.cuda.current_stream()
            overlap = self.overlap_filters
            if overlap is None:
                d = self.layer[0].attention.d_model
                total = len(self.layer) * ops.lib.m2_filter_spectrum_bytes(d, L)
                overlap = "upfront" if total <= self.UPFRONT_MAX_BYTES else True
            nxt = [None, None]                       # spectra of the next layer and the event that says they are ready
            ahead = []
            upfront = False
            batched = self._batched_filter_plan(L)
            if batched is not None:
                # all layers' filters by a few launches per group of layers, beside the layers or ahead of them
                table, groups = batched
                f0 = self.layer[0].attention.filter_fn
                side = None
                if overlap is not False:
                    if self._filter_stream is None:
                        self._filter_stream = torch.cuda.Stream()          # default priority
                    side = self._filter_stream
                    side.wait_stream(cur)
                with torch.cuda.stream(side if side is not None else cur):
                    for first, count in groups:
                        sp = ops.mixer_filter_spectra(table, w_mod=float(f0.w_mod), shift=float(f0.modulation.shift),
                                                      first=first, count=count)
                        ev = None
                        if side is not None:
                            sp.record_stream(cur)
                            ev = torch.cuda.Event()
                            ev.record(side)
                        ahead += [(sp[j], ev) for j in range(count)]
                upfront = True
                overlap = "upfront" if side is not None else "inline-batched"
            elif overlap:
                if self._filter_stream is None:
                    self._filter_stream = torch.cuda.Stream()          # default priority
                side = self._filter_stream

                def generate(i, after_event):
                    if after_event is None:
                        side.wait_stream(cur)
                    else:
                        side.wait_event(after_event)
                    with torch.cuda.stream(side):
                        sp = self.layer[i].attention.filter_spectrum(L)
                        sp.record_stream(cur)
                        ev = torch.cuda.Event()
                        ev.record(side)
                    nxt[0], nxt[1] = sp, ev

                upfront = overlap == "upfront"
                if upfront:          # all layers' spectra at once, in order, while the main stream runs the layers
                    side.wait_stream(cur)
                    with torch.cuda.stream(side):
                        for lay in self.layer:
                            sp = lay.attention.filter_spectrum(L)
                            sp.record_stream(cur)
                            ev = torch.cuda.Event()
                            ev.record(side)
                            ahead.append((sp, ev))
                else:
                    generate(0, None)
            for i, layer in enumerate(self.layer):
                want = all_layers or i == n - 1
                keep32 = want or pre_norm
                spec, ready, hook = None, None, None
                if overlap and upfront:
                    spec, ready = ahead[i]
                elif overlap:
                    spec, ready = nxt
                    if i + 1 < n:
                        def hook(i=i):
                            ev = torch.cuda.Event()
                            ev.record(cur)
                            generate(i + 1, ev)
                o32, h16, hT = layer.fused(h16, hT, B, L, want_f32=keep32, spec=spec, spec_ready=ready,
                                           after_core=hook, h32=o32)
                if want:
                    outs.append(o32)
            if overlap and overlap != "inline-batched":
                cur.wait_stream(self._filter_stream)
        return outs

    def _batched_filter_plan(self, L: int):
        """(pointer table of all layers' filters, [(first layer, count), ...]) when the filters of all layers are
        generated by batched calls, else None."""
        if not self.batch_filters:
            return None
        mixers = [lay.attention for lay in self.layer]
        m0 = mixers[0]
        if any(m.cache_filters for m in mixers):
            return None
        same = all(m.d_model == m0.d_model and m.residual_long_conv == m0.residual_long_conv
                   and m.bidirectional == m0.bidirectional and m.filter_fn.order == m0.filter_fn.order
                   and m.filter_fn.emb_dim == m0.filter_fn.emb_dim and m.filter_fn.w_mod == m0.filter_fn.w_mod
                   and m.filter_fn.modulation.shift == m0.filter_fn.modulation.shift for m in mixers)
        d, n = m0.d_model, len(mixers)
        if not same or n * ops.lib.m2_filter_spectrum_bytes(d, L) > self.UPFRONT_MAX_BYTES:
            return None
        entries = [m.filter_table_entry() for m in mixers]
        probe = (L,) + tuple(t.data_ptr() for filters, skips in entries for f in filters for v in f.values()
                             for t in (v if isinstance(v, list) else [v])) + tuple(b.data_ptr() for _, skips in entries
                                                                                   for b in skips)
        if self._filter_table is None or self._filter_table[0] != probe:
            self._filter_table = (probe, ops.FilterTable([e[0] for e in entries], [e[1] for e in entries], L, d,
                                                         m0.filter_fn.order, m0.filter_fn.emb_dim))
        table = self._filter_table[1]
        fpm = table.fpm
        per = max(1, ops.lib.m2_mixer_filters_workspace_bytes(1, fpm, L, d, table.order))
        group = max(1, min(n, self.FILTER_WORKSPACE_BYTES // per))
        return table, [(i, min(group, n - i)) for i in range(0, n, group)]

    def _run_graphed(self, h32: Optional[torch.Tensor], B: int, L: int, all_layers: bool,
                     h16: Optional[torch.Tensor] = None, hT: Optional[torch.Tensor] = None) -> List[torch.Tensor]:
        given = [t for t in (h32, h16, hT) if t is not None]
        key = (B, L, given[0].shape[-1] if h32 is not None else h16.shape[-1], all_layers, given[0].device,
               h32 is None, h16 is None, hT is None)
        entry = self._graphs.get(key)
        if entry is None:
            static = [None if t is None else t.clone() for t in (h32, h16, hT)]
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):                  # warm-up outside the capture (allocator, lazy inits)
                self._run_layers(static[0], B, L, all_layers, h16=static[1], hT=static[2])
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                static_out = self._run_layers(static[0], B, L, all_layers, h16=static[1], hT=static[2])
            entry = (graph, static, static_out)
            self._graphs[key] = entry
        graph, static, static_out = entry
        for dst, src in zip(static, (h32, h16, hT)):
            if dst is not None:
                dst.copy_(src)
        graph.replay()
        return [o.clone() for o in static_out]

    def forward(self, hidden_states: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                output_all_encoded_layers: Optional[bool] = True, subset_mask: Optional[torch.Tensor] = None,
                position_encodings: Optional[torch.Tensor] = None) -> List[torch.Tensor]:
        """hidden_states (B, L, d) -> list of (B, L, d) fp32.  `attention_mask` is accepted and, as in the
        reference's Monarch-Mixer branch (bert/src/bert_layers.py:577,721-726), never used."""
        if not hidden_states.is_cuda:
            raise RuntimeError("BertEncoder (m2_amd) runs on the GPU only")
        if position_encodings is not None:
            raise NotImplementedError("position_encodings added after every layer is not built")
        B, L, d = hidden_states.shape
        M = B * L
        h32 = hidden_states.reshape(M, d).float().contiguous()
        run = self._run_graphed if self.use_hip_graph else self._run_layers
        outs = [o.view(B, L, d) for o in run(h32, B, L, bool(output_all_encoded_layers))]
        if subset_mask is not None:
            outs[-1] = outs[-1][subset_mask]
        return outs


class BertPooler(nn.Module):
    """tanh(dense(first token)), or with config.pool_all tanh(dense(mean over unmasked positions))
    (bert/src/bert_layers.py:816-859).  A (B, d) x (d, d) product: plain torch ops."""

    def __init__(self, config: M2BertConfig):
        super().__init__()
        if getattr(config, "sequence_token_planting", False):
            raise NotImplementedError("sequence_token_planting pooling is not built")
        self.dense = nn.Linear(config.hidden_size, config.hidden_size)
        self.activation = nn.Tanh()
        self.pool_all = getattr(config, "pool_all", False)
        self.use_cls_token = getattr(config, "use_cls_token", False)
        self.sequence_token_planting = False

    def forward(self, hidden_states: torch.Tensor, pool: Optional[bool] = True, mask=None) -> torch.Tensor:
        if not self.pool_all:
            first = hidden_states[:, 0] if pool else hidden_states
            return self.activation(self.dense(first))
        m = mask.to(hidden_states.dtype)
        mean = torch.sum(hidden_states * m.unsqueeze(-1), dim=1) / torch.sum(m, dim=1, keepdim=True)
        return self.activation(self.dense(mean))


class BertModel(nn.Module):
    """Embeddings + encoder + pooler; returns (sequence output or list of layer outputs, pooled output or None)
    like the reference (bert/src/bert_layers.py:880-1010)."""

    def __init__(self, config: M2BertConfig, add_pooling_layer: bool = True, use_hip_graph: bool = False):
        super().__init__()
        if getattr(config, "attention_pooling", False):
            raise NotImplementedError("attention_pooling is not built")
        self.config = config
        self.embeddings = BertEmbeddings(config)
        self.encoder = BertEncoder(config, use_hip_graph=use_hip_graph)
        self.pooler = BertPooler(config) if add_pooling_layer else None
        # True: every forward ends by reading the embedding kernel's out-of-range flag (one stream
        # synchronisation) and raises IndexError like nn.Embedding would; False leaves the flag to
        # `embeddings.check_indices()`.  The embedding tables are part of the captured graph too:
        self.validate_ids = True
        self.register_load_state_dict_post_hook(lambda module, keys: module.encoder.reset_graphs())

    def get_input_embeddings(self):
        return self.embeddings.word_embeddings

    def forward(self, input_ids: torch.Tensor, token_type_ids: Optional[torch.Tensor] = None,
                attention_mask: Optional[torch.Tensor] = None, position_ids: Optional[torch.Tensor] = None,
                output_all_encoded_layers: Optional[bool] = False, masked_tokens_mask: Optional[torch.Tensor] = None,
                **kwargs):
        if masked_tokens_mask is not None:
            raise NotImplementedError("masked_tokens_mask subsetting belongs to the MLM head, which is not built")
        B, L = input_ids.shape
        all_layers = bool(output_all_encoded_layers)

        pre_norm = self.encoder.layer[0].attention.hyena_training_additions

        def run(ids, tt, pos):
            # the embedding LayerNorm writes the bf16 and channel-major forms the first layer reads itself
            # (or the fp32 form when the layers start with their own LayerNorm)
            h32, h16, hT = self.embeddings.forward_forms(ids, tt, pos, want_f32=pre_norm, want_bf16=not pre_norm,
                                                         want_channel_major=not pre_norm)
            return self.encoder._run_layers(None if h32 is None else h32.view(B * L, -1), B, L, all_layers,
                                            h16=h16, hT=hT)

        if not self.encoder.use_hip_graph:
            outs = run(input_ids, token_type_ids, position_ids)
        else:
            # embeddings and layer stack as one captured graph per input shape; only the index tensors are copied in
            given = (input_ids, token_type_ids, position_ids)
            key = ("model", B, L, all_layers, input_ids.device) + tuple(None if t is None else tuple(t.shape) for t in given)
            entry = self.encoder._graphs.get(key)
            if entry is None:
                static = [None if t is None else t.clone() for t in given]
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):              # warm-up outside the capture (allocator, lazy inits)
                    run(*static)
                torch.cuda.current_stream().wait_stream(side)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    static_out = run(*static)
                entry = (graph, static, static_out)
                self.encoder._graphs[key] = entry
            graph, static, static_out = entry
            for dst, src in zip(static, given):
                if dst is not None:
                    dst.copy_(src)
            graph.replay()
            outs = [o.clone() for o in static_out]
        if self.validate_ids and not torch.cuda.is_current_stream_capturing():
            self.embeddings.check_indices()
        enc = [o.view(B, L, -1) for o in outs]
        pooled = None
        if self.pooler is not None:
            if attention_mask is None:
                attention_mask = torch.ones_like(input_ids)
            pooled = self.pooler(enc[-1], mask=attention_mask)
        return (enc if output_all_encoded_layers else enc[-1]), pooled
