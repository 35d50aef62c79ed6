"""Tensor-level wrappers over the C ABI of libm2_amd.so.

PyTorch is used here for device memory and streams only: each function validates shapes, dtypes,
devices and contiguity in Python (the library re-checks sizes), allocates the output with
`torch.empty`, and enqueues the HIP kernels on torch's current stream.  CPU tensors are rejected:
there is no fallback path.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import torch

from . import _lib
from ._lib import HyenaFilterParams, M2_DTYPE_BF16, M2_DTYPE_F32, check, lib

Tensor = torch.Tensor


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _require(t: Tensor, name: str, dtype=None, shape=None) -> None:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name}: expected a tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name}: must live on the GPU (m2_amd has no CPU path); got device {t.device}")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name}: expected dtype {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name}: must be contiguous")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name}: expected shape {tuple(shape)}, got {tuple(t.shape)}")


def _ptr(t: Optional[Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _act_code(dtype) -> int:
    if dtype == torch.float32:
        return M2_DTYPE_F32
    if dtype == torch.bfloat16:
        return M2_DTYPE_BF16
    raise TypeError(f"activation dtype must be float32 or bfloat16, got {dtype}")


def fftconv_supported(L: int) -> bool:
    return bool(lib.m2_fftconv_supported_seqlen(int(L)))


# ------------------------------------------------------------------------------------------------
def hyena_filter_taps(filters: Sequence[dict], L: int, d: int, order: int, emb_dim: int, w_mod: float = 1.0,
                      shift: float = 0.0, static_scratch: bool = False, out: Optional[Tensor] = None) -> Tensor:
    """Bidirectional taps (nfilters, d, 2L) fp32 of `filters`.

    Each entry is a dict with fp32 GPU tensors: z (>=L, emb), t (>=L), freq (order), deltas (d),
    `fwd` = [w0, b0, w1, b1, w2, b2, w3] and optionally `rev` = the same seven of the reverse MLP.
    `static_scratch=True` takes the library's allocation-free entry point (m2_hyena_filter_fwd_static: no
    workspace tensor; the 20 MiB static array holds two filters up to L = 8192 or one up to L = 16384 for d <= 1536); with `out` given as well
    nothing is allocated at all.
    """
    nf = len(filters)
    arr = (HyenaFilterParams * nf)()
    keep = []
    for i, f in enumerate(filters):
        z = f["z"].reshape(-1, emb_dim)[:L].contiguous()
        t = f["t"].reshape(-1)[:L].contiguous()
        freq = f["freq"].reshape(-1).contiguous()
        deltas = f["deltas"].reshape(-1).contiguous()
        _require(z, "z", torch.float32, (L, emb_dim))
        _require(t, "t", torch.float32, (L,))
        _require(freq, "freq", torch.float32, (order,))
        _require(deltas, "deltas", torch.float32, (d,))
        keep += [z, t, freq, deltas]
        arr[i].z, arr[i].t, arr[i].freq, arr[i].deltas = z.data_ptr(), t.data_ptr(), freq.data_ptr(), deltas.data_ptr()
        shapes = [(order, emb_dim), (order,), (order, order), (order,), (order, order), (order,), (d, order)]
        for key, names in (("fwd", ("w0", "b0", "w1", "b1", "w2", "b2", "w3")),
                           ("rev", ("rw0", "rb0", "rw1", "rb1", "rw2", "rb2", "rw3"))):
            ws = f.get(key)
            if ws is None:
                if key == "fwd":
                    raise ValueError("filter without forward MLP")
                continue
            for w, n, s in zip(ws, names, shapes):
                w = w.contiguous()
                _require(w, f"{key}.{n}", torch.float32, s)
                keep.append(w)
                setattr(arr[i], n, w.data_ptr())
    dev = keep[0].device
    if out is None:
        taps = torch.empty(nf, d, 2 * L, dtype=torch.float32, device=dev)
    else:
        _require(out, "out", torch.float32, (nf, d, 2 * L))
        taps = out
    if static_scratch:
        check(lib.m2_hyena_filter_fwd_static(arr, nf, L, d, order, emb_dim, float(w_mod), float(shift), _ptr(taps),
                                             _stream()))
        return taps
    ws_bytes = lib.m2_hyena_filter_workspace_bytes(nf, L, d, order)
    workspace = torch.empty(ws_bytes // 4, dtype=torch.float32, device=dev)
    check(lib.m2_hyena_filter_fwd(arr, nf, L, d, order, emb_dim, float(w_mod), float(shift), _ptr(workspace),
                                  _ptr(taps), _stream()))
    return taps


class FilterTable:
    """Pointer table, in device memory, of the implicit filters of a batch of mixers (what `m2_mixer_filters_fwd`
    reads), with the tensors it points to kept alive.  Built once per set of parameter tensors (`key` = their
    addresses): building it copies from the host, so it must happen outside a stream capture."""

    def __init__(self, mixers: Sequence[Sequence[dict]], skips: Sequence[Sequence[Optional[Tensor]]], L: int, d: int,
                 order: int, emb_dim: int):
        self.nmixers = len(mixers)
        self.fpm = len(mixers[0])
        if self.fpm not in (1, 2) or any(len(m) != self.fpm for m in mixers) or any(len(k) != self.fpm for k in skips):
            raise ValueError("every mixer must bring the same number (1 or 2) of filters and skip weights")
        self.L, self.d, self.order, self.emb_dim = L, d, order, emb_dim
        shapes = [(order, emb_dim), (order,), (order, order), (order,), (order, order), (order,), (d, order)]
        rows, skip_row, keep = [], [], []
        for filters, sk in zip(mixers, skips):
            for f, D in zip(filters, sk):
                z = f["z"].reshape(-1, emb_dim)[:L]
                t = f["t"].reshape(-1)[:L]
                freq = f["freq"].reshape(-1)
                deltas = f["deltas"].reshape(-1)
                _require(z, "z", torch.float32, (L, emb_dim))
                _require(t, "t", torch.float32, (L,))
                _require(freq, "freq", torch.float32, (order,))
                _require(deltas, "deltas", torch.float32, (d,))
                row = [z.data_ptr(), t.data_ptr(), freq.data_ptr(), deltas.data_ptr()]
                keep += [z, t, freq, deltas]
                for key in ("fwd", "rev"):
                    ws = f.get(key)
                    if ws is None:
                        if key == "fwd":
                            raise ValueError("filter without forward MLP")
                        row += [0] * 7
                        continue
                    for w, s_ in zip(ws, shapes):
                        _require(w, f"{key} MLP tensor", torch.float32, s_)
                        keep.append(w)
                        row.append(w.data_ptr())
                rows.append(row)
                if D is not None:
                    _require(D, "skip weight", torch.float32, (d,))
                    keep.append(D)
                skip_row.append(0 if D is None else D.data_ptr())
        self.keep = keep
        self.key = (L, d, order, emb_dim) + tuple(v for r in rows for v in r) + tuple(skip_row)
        dev = keep[0].device
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("a filter pointer table cannot be built during a stream capture: run one forward "
                               "with these parameter tensors before capturing")
        self.table = torch.tensor(rows, dtype=torch.int64).to(dev)
        self.skip = torch.tensor(skip_row, dtype=torch.int64).to(dev)

    def spectrum_floats(self) -> int:
        return lib.m2_filter_spectrum_bytes(self.d, self.L) // 4


def mixer_filter_spectra(table: FilterTable, w_mod: float = 1.0, shift: float = 0.0, first: int = 0,
                         count: Optional[int] = None, out: Optional[Tensor] = None) -> Tensor:
    """Spectra (count, m2_filter_spectrum_bytes / 4) fp32 of the mixers [first, first + count) of `table`, generated
    from the filter parameters in a few launches for all of them (m2_mixer_filters_fwd)."""
    count = table.nmixers - first if count is None else count
    if first < 0 or count < 1 or first + count > table.nmixers:
        raise ValueError(f"mixers [{first}, {first + count}) outside the table of {table.nmixers}")
    dev = table.table.device
    n = table.spectrum_floats()
    if out is None:
        out = torch.empty(count, n, dtype=torch.float32, device=dev)
    else:
        _require(out, "out", torch.float32, (count, n))
    ws_bytes = lib.m2_mixer_filters_workspace_bytes(count, table.fpm, table.L, table.d, table.order)
    workspace = torch.empty((ws_bytes + 3) // 4, dtype=torch.float32, device=dev)
    check(lib.m2_mixer_filters_fwd(ctypes.c_void_p(table.table.data_ptr() + first * table.fpm * 18 * 8),
                                   ctypes.c_void_p(table.skip.data_ptr() + first * table.fpm * 8), count, table.fpm,
                                   table.L, table.d, table.order, table.emb_dim, float(w_mod), float(shift),
                                   _ptr(workspace), _ptr(out), _stream()))
    return out


def filter_spectrum(taps1: Tensor, taps2: Optional[Tensor], D1: Optional[Tensor], D2: Optional[Tensor]) -> Tensor:
    """Opaque spectrum buffer for `mixer_core` from (d, 2L) taps of one or two filters."""
    d, n = taps1.shape
    L = n // 2
    _require(taps1, "taps1", torch.float32, (d, 2 * L))
    if taps2 is not None:
        _require(taps2, "taps2", torch.float32, (d, 2 * L))
    for nm, D in (("D1", D1), ("D2", D2)):
        if D is not None:
            _require(D, nm, torch.float32, (d,))
    spec = torch.empty(lib.m2_filter_spectrum_bytes(d, L) // 4, dtype=torch.float32, device=taps1.device)
    check(lib.m2_filter_spectrum_fwd(_ptr(taps1), _ptr(taps2), _ptr(D1), _ptr(D2), _ptr(spec), d, L, _stream()))
    return spec


def mixer_core(xproj: Tensor, u: Optional[Tensor], short_w: Tensor, short_b: Tensor, spec: Tensor, B: int, L: int,
               d: int, out: Optional[Tensor] = None, proj_bias: Optional[Tensor] = None) -> Tensor:
    """y (d, B, L) from the channel-major in-projection (3d, B, L) and layer input (d, B, L).
    `proj_bias` (3d) fp32 is added to xproj on load (pass the in_linear bias when the GEMM ran without it)."""
    _require(xproj, "xproj", None, (3 * d, B, L))
    code = _act_code(xproj.dtype)
    if proj_bias is not None:
        _require(proj_bias, "proj_bias", torch.float32, (3 * d,))
    if u is not None:
        _require(u, "u", torch.float32, (d, B, L))
    _require(short_w, "short_w", torch.float32, (3 * d, 3))
    _require(short_b, "short_b", torch.float32, (3 * d,))
    _require(spec, "spec", torch.float32, (lib.m2_filter_spectrum_bytes(d, L) // 4,))
    if out is None:
        out = torch.empty(d, B, L, dtype=xproj.dtype, device=xproj.device)
    else:
        _require(out, "out", xproj.dtype, (d, B, L))
    check(lib.m2_mixer_core_fwd(_ptr(xproj), _ptr(proj_bias), _ptr(u), _ptr(short_w), _ptr(short_b), _ptr(spec),
                                _ptr(out), B, L, d, code, _stream()))
    return out


def fftconv(x: Tensor, spec: Tensor, B: int, L: int, d: int) -> Tensor:
    """Plain long convolution of x (d, B, L) with the first filter held in `spec` (skip term included)."""
    _require(x, "x", None, (d, B, L))
    code = _act_code(x.dtype)
    _require(spec, "spec", torch.float32, (lib.m2_filter_spectrum_bytes(d, L) // 4,))
    out = torch.empty_like(x)
    check(lib.m2_fftconv_fwd(_ptr(x), _ptr(spec), _ptr(out), B, L, d, code, _stream()))
    return out


def blockdiag_glu(x: Tensor, w: Tensor, out: Optional[Tensor] = None) -> Tensor:
    """gelu_erf(h[:, :I]) * h[:, I:] with h = blockdiag_multiply(x, w); x (M, in) bf16, w (nb, 2I/nb, in/nb) bf16."""
    M, in_f = x.shape
    nb, q, p = w.shape
    _require(x, "x", torch.bfloat16)
    _require(w, "w", torch.bfloat16)
    if nb * p != in_f:
        raise ValueError(f"x has {in_f} features, weight expects {nb}*{p}")
    I = nb * q // 2
    if out is None:
        out = torch.empty(M, I, dtype=torch.bfloat16, device=x.device)
    else:
        _require(out, "out", torch.bfloat16, (M, I))
    check(lib.m2_blockdiag_glu_fwd(_ptr(x), _ptr(w), _ptr(out), M, in_f, I, nb, _stream()))
    return out


def blockdiag_linear(x: Tensor, w: Tensor, bias: Optional[Tensor] = None, residual: Optional[Tensor] = None,
                     out_dtype=torch.bfloat16, out: Optional[Tensor] = None) -> Tensor:
    """blockdiag_multiply(x, w) (+ bias) (+ residual); x (M, in) bf16, w (nb, out/nb, in/nb) bf16."""
    M, in_f = x.shape
    nb, q, p = w.shape
    _require(x, "x", torch.bfloat16)
    _require(w, "w", torch.bfloat16)
    if nb * p != in_f:
        raise ValueError(f"x has {in_f} features, weight expects {nb}*{p}")
    out_f = nb * q
    if bias is not None:
        _require(bias, "bias", torch.float32, (out_f,))
    if residual is not None:
        _require(residual, "residual", torch.bfloat16, (M, out_f))
    if out is None:
        out = torch.empty(M, out_f, dtype=out_dtype, device=x.device)
    else:
        _require(out, "out", out_dtype, (M, out_f))
    check(lib.m2_blockdiag_linear_fwd(_ptr(x), _ptr(w), _ptr(bias), _ptr(residual), _ptr(out), M, in_f, out_f, nb,
                                      _act_code(out_dtype), _stream()))
    return out


def blockdiag_linear_f32(x: Tensor, w: Tensor, bias: Optional[Tensor] = None) -> Tensor:
    """blockdiag_multiply(x, w) (+ bias) in fp32 (exact fp32 products, fp32 accumulation); x (M, in) fp32,
    w (nb, out/nb, in/nb) fp32."""
    M, in_f = x.shape
    nb, q, p = w.shape
    _require(x, "x", torch.float32)
    _require(w, "w", torch.float32)
    if nb * p != in_f:
        raise ValueError(f"x has {in_f} features, weight expects {nb}*{p}")
    if bias is not None:
        _require(bias, "bias", torch.float32, (nb * q,))
    out = torch.empty(M, nb * q, dtype=torch.float32, device=x.device)
    check(lib.m2_blockdiag_linear_f32_fwd(_ptr(x), _ptr(w), _ptr(bias), _ptr(out), M, in_f, nb * q, nb, _stream()))
    return out


def mlp_fused_supported(in_features: int, intermediate: int, nblocks: int) -> bool:
    return bool(lib.m2_mlp_fused_supported(int(in_features), int(intermediate), int(nblocks)))


def mlp_fused_pack(w_gated: Tensor, w_out: Tensor) -> Tensor:
    """gated_layers.weight (nb, 2I/nb, d/nb) bf16 and wo.weight (nb, d/nb, I/nb) bf16 -> the packed copy `mlp_fused`
    streams (flat bf16 tensor, as many elements as the two weights together).  Once per set of weights."""
    nb, q, p = w_gated.shape
    _require(w_gated, "w_gated", torch.bfloat16)
    d, I = nb * p, nb * q // 2
    _require(w_out, "w_out", torch.bfloat16, (nb, d // nb, I // nb))
    nbytes = int(lib.m2_mlp_fused_packed_bytes(d, I, nb))
    if nbytes == 0:
        raise RuntimeError(f"mlp_fused is built for nblocks=4, in_features=768, intermediate % 128 == 0; got {nb}, {d}, {I}")
    packed = torch.empty(nbytes // 2, dtype=torch.bfloat16, device=w_gated.device)
    check(lib.m2_mlp_fused_pack(_ptr(w_gated), _ptr(w_out), _ptr(packed), d, I, nb, _stream()))
    return packed


def mlp_fused(x: Tensor, w_gated: Tensor, w_out: Tensor, bias: Optional[Tensor] = None, residual: Optional[Tensor] = None,
              out_dtype=torch.float32, out: Optional[Tensor] = None, packed: Optional[Tensor] = None) -> Tensor:
    """blockdiag(gelu_erf(h[:, :I]) * h[:, I:], w_out) (+ bias) (+ residual) with h = blockdiag(x, w_gated), one kernel.
    x (M, d) bf16, w_gated (nb, 2I/nb, d/nb) bf16, w_out (nb, d/nb, I/nb) bf16; `packed` = mlp_fused_pack(w_gated,
    w_out), which a caller with fixed weights computes once (without it the weights are packed on every call)."""
    M, d = x.shape
    nb, q, p = w_gated.shape
    _require(x, "x", torch.bfloat16)
    I = nb * q // 2
    if nb * p != d:
        raise ValueError(f"x has {d} features, w_gated expects {nb}*{p}")
    if packed is None:
        packed = mlp_fused_pack(w_gated, w_out)
    else:
        _require(packed, "packed", torch.bfloat16, (int(lib.m2_mlp_fused_packed_bytes(d, I, nb)) // 2,))
    if bias is not None:
        _require(bias, "bias", torch.float32, (d,))
    if residual is not None:
        _require(residual, "residual", torch.bfloat16, (M, d))
    if out is None:
        out = torch.empty(M, d, dtype=out_dtype, device=x.device)
    else:
        _require(out, "out", out_dtype, (M, d))
    check(lib.m2_mlp_fused_fwd(_ptr(x), _ptr(packed), _ptr(bias), _ptr(residual), _ptr(out), M, d, I, nb,
                               _act_code(out_dtype), _stream()))
    return out


def glu_stream_supported(in_features: int, intermediate: int, nblocks: int) -> bool:
    return bool(lib.m2_glu_stream_supported(int(in_features), int(intermediate), int(nblocks)))


def glu_stream_pack(w_gated: Tensor) -> Tensor:
    """gated_layers.weight (nb, 2I/nb, d/nb) bf16 -> the packed copy `glu_stream` streams (flat bf16 tensor of the
    weight's size; blocks narrower than 256 are padded to 256 with zeros).  Once per set of weights."""
    nb, q, p = w_gated.shape
    _require(w_gated, "w_gated", torch.bfloat16)
    d, I = nb * p, nb * q // 2
    nbytes = int(lib.m2_glu_stream_packed_bytes(d, I, nb))
    if nbytes == 0:
        raise RuntimeError("glu_stream is built for nblocks=4, blocks 384 or 448 wide or a multiple of 8 in [224, 248], "
                           f"intermediate % 128 == 0; got {nb}, {d}, {I}")
    packed = torch.empty(nbytes // 2, dtype=torch.bfloat16, device=w_gated.device)
    check(lib.m2_glu_stream_pack(_ptr(w_gated), _ptr(packed), d, I, nb, _stream()))
    return packed


def glu_stream(x: Tensor, w_gated: Tensor, out: Optional[Tensor] = None, packed: Optional[Tensor] = None) -> Tensor:
    """gelu_erf(h[:, :I]) * h[:, I:] with h = blockdiag(x, w_gated), as `blockdiag_glu`, for 384-wide blocks (d = 1536), 448-wide ones (d = 1792) and blocks of 224 .. 248 (d = 960).
    x (M, d) bf16, w_gated (nb, 2I/nb, d/nb) bf16; `packed` = glu_stream_pack(w_gated), which a caller with fixed
    weights computes once (without it the weight is packed on every call)."""
    M, d = x.shape
    nb, q, p = w_gated.shape
    _require(x, "x", torch.bfloat16)
    I = nb * q // 2
    if nb * p != d:
        raise ValueError(f"x has {d} features, w_gated expects {nb}*{p}")
    if packed is None:
        packed = glu_stream_pack(w_gated)
    else:
        _require(packed, "packed", torch.bfloat16, (int(lib.m2_glu_stream_packed_bytes(d, I, nb)) // 2,))
    if out is None:
        out = torch.empty(M, I, dtype=torch.bfloat16, device=x.device)
    else:
        _require(out, "out", torch.bfloat16, (M, I))
    check(lib.m2_glu_stream_fwd(_ptr(x), _ptr(packed), _ptr(out), M, d, I, nb, _stream()))
    return out


def layernorm(x: Tensor, gamma: Tensor, beta: Tensor, eps: float, want_f32: bool = True, want_bf16: bool = False,
              want_channel_major: bool = False):
    """LayerNorm over the last dim of x (M, d) fp32 or bf16 -> (f32 (M,d) | None, bf16 (M,d) | None, f32 (d,M) | None)."""
    M, d = x.shape
    if x.dtype != torch.bfloat16:
        _require(x, "x", torch.float32)
    else:
        _require(x, "x", torch.bfloat16)
    _require(gamma, "gamma", torch.float32, (d,))
    _require(beta, "beta", torch.float32, (d,))
    o32 = torch.empty(M, d, dtype=torch.float32, device=x.device) if want_f32 else None
    o16 = torch.empty(M, d, dtype=torch.bfloat16, device=x.device) if want_bf16 else None
    ot = torch.empty(d, M, dtype=torch.float32, device=x.device) if want_channel_major else None
    fn = lib.m2_layernorm_bf16_fwd if x.dtype == torch.bfloat16 else lib.m2_layernorm_fwd
    check(fn(_ptr(x), _ptr(gamma), _ptr(beta), float(eps), _ptr(o32), _ptr(o16), _ptr(ot), M, d, _stream()))
    return o32, o16, ot


def embed_layernorm(input_ids: Tensor, token_type_ids: Optional[Tensor], position_ids: Optional[Tensor], word_emb: Tensor,
                    type_emb: Tensor, pos_emb: Optional[Tensor], gamma: Tensor, beta: Tensor, eps: float,
                    want_f32: bool = True, want_bf16: bool = False, want_channel_major: bool = False,
                    bad_index: Optional[Tensor] = None):
    """LayerNorm(word_emb[ids] + type_emb[token_type_ids or 0] (+ pos_emb[position_ids or 0..L-1])) for ids (B, L)
    -> (f32 (B*L, d) | None, bf16 (B*L, d) | None, f32 (d, B*L) | None).

    An index outside its table never reads out of bounds (the kernel takes the nearest valid row); `bad_index`,
    a zeroed int32 GPU tensor of one element, receives 1 when that happened: see `raise_on_bad_index`."""
    B, L = input_ids.shape
    d = word_emb.shape[1]
    _require(input_ids, "input_ids", torch.int64)
    _require(word_emb, "word_emb", torch.float32)
    _require(type_emb, "type_emb", torch.float32, (type_emb.shape[0], d))
    _require(gamma, "gamma", torch.float32, (d,))
    _require(beta, "beta", torch.float32, (d,))
    if token_type_ids is not None:
        _require(token_type_ids, "token_type_ids", torch.int64, (B, L))
    if pos_emb is not None:
        _require(pos_emb, "pos_emb", torch.float32, (pos_emb.shape[0], d))
        if position_ids is None and pos_emb.shape[0] < L:
            raise ValueError(f"position table has {pos_emb.shape[0]} rows, sequence length is {L}")
    if position_ids is not None:
        if pos_emb is None:
            raise ValueError("position_ids given but the model has no position embeddings")
        _require(position_ids, "position_ids", torch.int64, (B, L))
    if bad_index is not None:
        _require(bad_index, "bad_index", torch.int32, (1,))
    M = B * L
    dev = input_ids.device
    o32 = torch.empty(M, d, dtype=torch.float32, device=dev) if want_f32 else None
    o16 = torch.empty(M, d, dtype=torch.bfloat16, device=dev) if want_bf16 else None
    ot = torch.empty(d, M, dtype=torch.float32, device=dev) if want_channel_major else None
    check(lib.m2_embed_layernorm_fwd(_ptr(input_ids), _ptr(token_type_ids), _ptr(position_ids), _ptr(word_emb),
                                     _ptr(type_emb), _ptr(pos_emb), word_emb.shape[0], type_emb.shape[0],
                                     0 if pos_emb is None else pos_emb.shape[0], _ptr(gamma), _ptr(beta), float(eps),
                                     _ptr(o32), _ptr(o16), _ptr(ot), _ptr(bad_index), B, L, d, _stream()))
    return o32, o16, ot


def raise_on_bad_index(bad_index: Tensor) -> None:
    """Reads the flag `embed_layernorm` sets (this waits for the stream) and raises IndexError, as nn.Embedding
    does in the reference, when a token, token-type or position id lay outside its table."""
    if int(bad_index.item()) != 0:
        bad_index.zero_()
        raise IndexError("index out of range in the embedding lookup: a token id, token-type id or position id "
                         "lies outside its table (the output of this forward used the nearest valid rows)")


def blockdiag_linear_layernorm_supported(in_features: int, out_features: int, nblocks: int) -> bool:
    return bool(lib.m2_blockdiag_linear_layernorm_supported(int(in_features), int(out_features), int(nblocks)))


def blockdiag_linear_layernorm(x: Tensor, w: Tensor, bias: Optional[Tensor], residual: Optional[Tensor], gamma: Tensor,
                               beta: Tensor, eps: float, want_f32: bool = True, want_bf16: bool = False,
                               want_channel_major: bool = False):
    """LayerNorm(blockdiag_multiply(x, w) + bias + residual) in one kernel, outputs as `layernorm`."""
    M, in_f = x.shape
    nb, q, p = w.shape
    _require(x, "x", torch.bfloat16)
    _require(w, "w", torch.bfloat16)
    if nb * p != in_f:
        raise ValueError(f"x has {in_f} features, weight expects {nb}*{p}")
    d = nb * q
    if bias is not None:
        _require(bias, "bias", torch.float32, (d,))
    if residual is not None:
        _require(residual, "residual", torch.bfloat16, (M, d))
    _require(gamma, "gamma", torch.float32, (d,))
    _require(beta, "beta", torch.float32, (d,))
    o32 = torch.empty(M, d, dtype=torch.float32, device=x.device) if want_f32 else None
    o16 = torch.empty(M, d, dtype=torch.bfloat16, device=x.device) if want_bf16 else None
    ot = torch.empty(d, M, dtype=torch.float32, device=x.device) if want_channel_major else None
    check(lib.m2_blockdiag_linear_layernorm_fwd(_ptr(x), _ptr(w), _ptr(bias), _ptr(residual), _ptr(gamma), _ptr(beta),
                                                float(eps), _ptr(o32), _ptr(o16), _ptr(ot), M, in_f, d, nb, _stream()))
    return o32, o16, ot
