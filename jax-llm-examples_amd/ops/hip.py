"""The engine's kernel set on the GPU: hand-written HIP kernels (``csrc/``) called
through a C interface, plus library matrix products for the dense projections
(where the reference uses its library's ``einsum``, ``llama4/llama4_jax/model.py:907-909,
952-954, 1146-1152, 1204``).  Kernels run on PyTorch's current stream.  There is no
fallback: if the library cannot be built or loaded, constructing :class:`HipOps` fails.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import build as _build

# the rules under which the attention kernels here read keys ("window_keep": the general kernel alone)
_RET_MODES = {"all": 0, "chunk": 1, "window": 2, "window_keep": 2}


def _ret_mode(retention) -> int:
    try:
        return _RET_MODES[retention[0]]
    except KeyError:
        raise KernelError(f"the attention kernels read keys under the rules {', '.join(_RET_MODES)}; a mixer with the "
                          f"rule {retention!r} brings kernels of its own") from None

_vp, _i, _f, _ll = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_longlong

_SIGNATURES = {
    "jle_embed": [_vp, _vp, _i, _vp, _i, _i, _vp],
    "jle_add_rmsnorm": [_vp, _i, _vp, _vp, _vp, _i, _vp, _i, _vp, _f, _vp, _i, _vp, _i, _i, _vp],
    "jle_add_residual": [_vp, _vp, _i, _ll, _vp],
    "jle_gather_rows": [_vp, _vp, _vp, _i, _i, _vp],
    "jle_silu_mul": [_vp, _vp, _i, _i, _i, _vp],
    "jle_moe_combine": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "jle_qk_prepare": [_vp, _vp, _vp, _vp, _vp, _vp, _f, _f, _f, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _i,
                       _vp],
    "jle_paged_attention_generic": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _f, _i, _i, _i, _i, _i, _i, _i, _i, _vp,
                                    _vp, _vp],
    "jle_attention_f32_tiles": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _f, _i, _i, _i, _i, _vp],
    "jle_attention_f32_heads": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _f, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp],
    "jle_attention_merge": [_vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "jle_moe_route": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "jle_norm_route": [_vp, _i, _vp, _vp, _vp, _i, _vp, _i, _vp, _f, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                       _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "jle_moe_align": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "jle_moe_route_align": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "jle_gemm_generic": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "jle_gemm_f32_skinny": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    "jle_gemm_f32_stream": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "jle_sample": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "jle_attention_mfma_supported": [_i, _i, _i, _i],
    "jle_attention_prefill": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _vp, _i, _i, _i, _f, _i, _i, _i, _i, _vp,
                              _i, _vp, _vp],
    "jle_attention_decode": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _f, _i, _i, _i, _i,
                             _vp, _i, _vp, _vp],
    "jle_attention_decode_fused": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _f, _i, _i,
                                   _i, _i, _vp, _f, _f, _f, _vp, _i, _vp],
    "jle_gemm_grouped": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    "jle_gemm_skinny": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _i, _i, _i, _i, _vp, _vp,
                        _vp],
    "jle_add_norm_shift": [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _f, _i, _vp, _f, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                           _vp, _i, _i, _i, _i, _vp],
    "jle_polynorm": [_vp, _i, _vp, _vp, _f, _vp, _i, _i, _i, _vp],
    "jle_latent_prepare": [_vp, _i, _i, _i, _i, _i, _vp, _vp, _i, _i, _f, _vp, _f, _vp, _vp, _vp, _i, _vp, _i, _i, _i,
                           _vp],
    "jle_swap_leading": [_vp, _vp, _i, _i, _i, _vp],
    "jle_latent_attention_lds": [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _f, _vp, _i, _i, _i,
                                 _i, _i, _vp, _vp],
    "jle_latent_attention_mfma": [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _f, _vp, _i, _i, _i,
                                  _i, _i, _i, _i, _vp, _vp, _vp, _vp],
    "jle_latent_attention": [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _f, _i, _i, _i, _i, _i, _i, _i,
                             _vp, _vp, _vp, _vp],
    "jle_embed_pair": [_vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _ll, _ll, _vp],
    "jle_act_mul": [_vp, _vp, _i, _i, _i, _i, _vp],
    "jle_softcap": [_vp, _ll, _f, _vp],
    "jle_sigmoid_mul": [_vp, _vp, _i, _vp, _i, _i, _i, _vp],
    "jle_add_norm_pair": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _vp, _vp, _i, _i, _i, _vp],
    "jle_conv_rows": [_vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "jle_conv_qk_prepare": [_vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _f, _f, _vp, _vp, _i, _i,
                            _i, _i, _i, _i, _i, _i, _i, _vp],
    "jle_gemm_stream": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    "jle_streams_mix_norm": [_vp, _i, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _f, _vp, _i, _vp, _i, _i, _i, _i,
                             _vp],
    "jle_embed_sinusoid": [_vp, _vp, _vp, _i, _f, _vp, _vp, _i, _i, _i, _vp],
    "jle_mlstm": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _f, _f, _vp],
    "jle_mlstm_chunked": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i,
                          _i, _i, _f, _f, _f, _vp],
    "jle_span_prepare": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _f, _f, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    "jle_row_gate": [_vp, _i, _vp, _vp, _i, _i, _i, _vp],
    "jle_scaled_add_norm": [_vp, _vp, _i, _f, _vp, _i, _f, _vp, _vp, _f, _vp, _i, _vp, _i, _i, _vp, _i, _vp],
    "jle_moe_logits": [_vp, _vp, _vp, _i, _i, _i, _vp],
    "jle_heads_prepare": [_vp, _vp, _vp, _vp, _i, _i, _f, _f, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i,
                          _vp],
    "jle_diff_combine": [_vp, _vp, _vp, _f, _f, _f, _i, _i, _i, _i, _i, _i, _vp],
    "jle_gated_delta": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i,
                        _i, _i, _i, _i, _f, _f, _vp],
    "jle_moe_choose": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "jle_relu2": [_vp, _vp, _i, _ll, _vp],
    "jle_conv_rows_act": [_vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "jle_attention_prefill_kept": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _f, _i, _i, _i, _i, _vp],
    "jle_paged_attention_kept": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _f, _i, _i, _i, _i, _i, _i, _i, _i, _vp,
                                 _vp, _vp],
    "jle_paged_attention_biased": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _f, _i, _i, _i, _i, _i, _i, _i, _i, _vp,
                                   _vp, _vp, _i, _vp, _vp],
}


class KernelError(RuntimeError):
    pass


class ExpertSum:
    """A feed-forward output that is not formed yet: ``sum_j routed[inv[n * k + j]] + shared[n]``.  The kernel
    that adds it to the residual and norms the result reads the pieces directly."""

    def __init__(self, routed, inv, k: int, shared, n: int, d: int) -> None:
        self.routed, self.inv, self.k, self.shared = routed, inv, k, shared
        self.shape = torch.Size((n, d))
        self.dtype = routed.dtype


class PendingNorm:
    """The rows a norm will give, not computed yet: the residual, the branch output still to be added to it, the
    norm's weight and eps.  Whoever consumes it computes it - inside its own launch where a kernel can (the
    router of a step of few tokens does), else with the norm's own kernel (:meth:`rows`).  ``x_out`` is the
    residual after the addition, ``h`` / ``h32`` the normed rows in the run dtype / float32, once computed."""

    def __init__(self, ops, x, delta, weight, eps: float, out_dtype) -> None:
        self.ops, self.x, self.delta, self.weight, self.eps = ops, x, delta, weight, float(eps)
        self.dtype, self.shape, self.device = out_dtype, x.shape, x.device
        self.x_out = self.h = self.h32 = None

    @property
    def done(self) -> bool:
        return self.x_out is not None

    def rows(self, want32: bool = False):
        if not self.done:
            self.h, self.h32 = self.ops.add_rmsnorm(self.x, self.delta, self.weight, self.eps, self.dtype, want32=True)
            self.x_out = self.x  # (added in place)
        if want32 and self.h32 is None:  # (computed by a kernel that kept the float32 rows to itself)
            self.h32 = self.h.float() if self.dtype != torch.float32 else self.h
        return self.h32 if want32 else self.h

    def residual(self):
        self.rows()
        return self.x_out


_LIB = None


def _bind(path: str):
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:
        raise KernelError(f"cannot load the HIP kernel library {path}: {e}") from e
    for name, args in _SIGNATURES.items():
        fn = getattr(lib, name, None)  # (a library of some of the sources lacks the others' entry points)
        if fn is not None:
            fn.argtypes = args
            fn.restype = ctypes.c_int
    for name, args in (("jle_attention_mfma_supported", [_i, _i, _i, _i]),  # queries, not launches: no stream
                       ("jle_gemm_stream_supported", [_i, _i, _i]), ("jle_gemm_f32_stream_supported", [_i, _i, _i]),
                       ("jle_latent_attention_mfma_supported", [_i, _i, _i, _i, _i]), ("jle_attention_group_waves", []),
                       ("jle_mlstm_chunked_supported", [_i, _i]), ("jle_mlstm_chunk_tokens", []),
                       ("jle_gated_delta_padded", [_i])):
        fn = getattr(lib, name, None)
        if fn is not None:
            fn.argtypes = args
    lib._jle_path = path
    lib._jle_whole = "libjle-part-" not in path
    return lib


def load_library(kernel_sources=None):
    """Loads the compiled kernels (compiling them if no build is there).  ``kernel_sources``: the sources that the
    model to be run needs; if the library of all sources is not built yet, only those are compiled now.  A kernel
    that such a library lacks and that is called all the same brings the whole library in (:meth:`HipOps._whole`)."""
    global _LIB
    if _LIB is None:
        _LIB = _bind(_build.library_path(only=kernel_sources))
    return _LIB


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


class HipOps:
    name = "hip"

    def __init__(self, device, kernel_sources=None) -> None:
        self.device = torch.device(device)
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise KernelError("the HIP kernels need a GPU")
        self.lib = load_library(kernel_sources)
        self._fn = {name: getattr(self.lib, name) for name in _SIGNATURES if hasattr(self.lib, name)}
        self._device_index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        self._raw_stream = raw if raw is not None else (lambda i: torch.cuda.current_stream(i).cuda_stream)
        # true float32 products: no reduced-precision matrix mode
        # counters of the kernels in which the last wavefront (or block) to finish does the closing work: zero
        # between launches (whoever closes puts its counter back), so they are cleared here once
        self._tickets = torch.zeros(self.TICKETS, dtype=torch.int32, device=self.device)
        self._zero_bias = {}  # (heads, device) -> a distance table of zeros, for sinks without a bias
        self._slice_tickets = torch.zeros(self.SLICE_TICKETS, dtype=torch.int32, device=self.device)
        self._compute_units = torch.cuda.get_device_properties(self.device).multi_processor_count
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")

    # ------------------------------------------------------------------ helpers
    def _stream(self) -> int:
        """The current stream's handle (a decode step asks hundreds of times: the raw query, not a Stream object)."""
        return self._raw_stream(self._device_index)

    def _whole(self) -> None:
        """The library of all sources instead of the partial one this process began with (built now if need be)."""
        global _LIB
        if not self.lib._jle_whole:
            _LIB = _bind(_build.library_path())
        self.lib = _LIB
        self._fn = {name: getattr(self.lib, name) for name in _SIGNATURES}

    def _query(self, name: str, *args) -> int:
        """An entry point that answers a question about sizes (no launch, no stream)."""
        if not hasattr(self.lib, name):
            self._whole()
        return getattr(self.lib, name)(*args)

    def _call(self, name: str, *args) -> None:
        if name not in self._fn:
            self._whole()
        rc = self._fn[name](*args, self._stream())
        if rc != 0:
            if rc < 0:
                raise KernelError(f"{name}: the kernel refuses these sizes or options")
            raise KernelError(f"{name}: HIP error {rc}")

    @staticmethod
    def _is_bf16(t: torch.Tensor) -> int:
        if t.dtype == torch.bfloat16:
            return 1
        if t.dtype == torch.float32:
            return 0
        raise KernelError(f"unsupported dtype {t.dtype}")

    @staticmethod
    def _chk(t: torch.Tensor, dtype=None, shape=None, what: str = "tensor") -> torch.Tensor:
        if not t.is_cuda:
            raise KernelError(f"{what} must be on the GPU")
        if not t.is_contiguous():
            raise KernelError(f"{what} must be contiguous, got strides {t.stride()} for shape {tuple(t.shape)}")
        if dtype is not None and t.dtype != dtype:
            raise KernelError(f"{what} must be {dtype}, got {t.dtype}")
        if shape is not None and tuple(t.shape) != tuple(shape):
            raise KernelError(f"{what} must have shape {tuple(shape)}, got {tuple(t.shape)}")
        return t

    # ------------------------------------------------------------------ embedding, norms
    def embed(self, token_ids, table):
        n, (v, d) = token_ids.numel(), table.shape
        self._chk(token_ids, torch.int32, (n,), "token ids")
        self._chk(table, None, (v, d), "embedding table")
        out = torch.empty(n, d, dtype=torch.float32, device=table.device)
        self._call("jle_embed", _p(token_ids), _p(table), self._is_bf16(table), _p(out), n, d)
        return out

    def embed_pair(self, token_ids, prev_token_ids, table, pair_table, buckets: int, mul_prev: int, mul_cur: int):
        """``table[token] + pair_table[(prev * mul_prev + token * mul_cur) mod buckets]`` (row ``buckets`` where
        ``prev < 0``), float32."""
        n, (v, d) = token_ids.numel(), table.shape
        self._chk(token_ids, torch.int32, (n,), "token ids")
        self._chk(prev_token_ids, torch.int32, (n,), "tokens before")
        self._chk(table, None, (v, d), "embedding table")
        self._chk(pair_table, table.dtype, (buckets + 1, d), "pair table")
        out = torch.empty(n, d, dtype=torch.float32, device=table.device)
        self._call("jle_embed_pair", _p(token_ids), _p(prev_token_ids), _p(table), _p(pair_table), self._is_bf16(table),
                   _p(out), n, d, int(buckets), int(mul_prev), int(mul_cur))
        return out

    def embed_sinusoid(self, token_ids, positions, table, multiplier: float, rates):
        """``table[token] * multiplier`` plus the position's sinusoid (entry ``2i``: ``sin(pos * rates[i])``, entry
        ``2i + 1``: the cosine), float32."""
        n, (v, d) = token_ids.numel(), table.shape
        self._chk(token_ids, torch.int32, (n,), "token ids")
        self._chk(positions, torch.int32, (n,), "positions")
        self._chk(table, None, (v, d), "embedding table")
        self._chk(rates, torch.float32, ((d + 1) // 2,), "sinusoid rates")
        out = torch.empty(n, d, dtype=torch.float32, device=table.device)
        self._call("jle_embed_sinusoid", _p(token_ids), _p(positions), _p(table), self._is_bf16(table),
                   float(multiplier), _p(rates), _p(out), n, 1, d)
        return out

    # ------------------------------------------------------------------ several residual streams
    MAX_STREAMS = 16

    def streams_mix_norm(self, xs, update, inw, weight, eps: float, out_dtype, want32: bool = False, norm: bool = True):
        """``xs``: float32 ``[N, S, D]``, changed in place: the pending ``update`` (a branch output, a plain tensor or
        an :class:`ExpertSum`, with ``mix`` ``[from, to]`` and ``outw``) worked into all streams at once, then the
        norm of ``sum_s inw[s] X_s`` (``inw`` ``None``: the plain sum); one launch."""
        n, s_, d = xs.shape
        self._chk(xs, torch.float32, (n, s_, d), "residual streams")
        if s_ > self.MAX_STREAMS:
            raise KernelError(f"the streams kernel takes up to {self.MAX_STREAMS} streams, not {s_}")
        kind, plain, routed, inv, k, shared, is_bf16, mix, outw = 0, None, None, None, 0, None, 0, None, None
        if update is not None:
            y, mix, outw = update.y, update.mix, update.outw
            self._chk(mix, torch.float32, (s_, s_), "stream mix")
            self._chk(outw, torch.float32, (s_,), "stream output weights")
            if isinstance(y, ExpertSum):
                if tuple(y.shape) != (n, d):
                    raise KernelError("the branch output does not fit the streams")
                kind, routed, inv, k, shared = 2, y.routed, y.inv, y.k, y.shared
                is_bf16 = self._is_bf16(routed)
            else:
                self._chk(y, None, (n, d), "branch output")
                kind, plain, is_bf16 = 1, y, self._is_bf16(y)
        if inw is not None:
            self._chk(inw, torch.float32, (s_,), "stream input weights")
        if weight is not None:
            self._chk(weight, torch.float32, (d,), "norm weight")
        out = torch.empty(n, d, dtype=out_dtype, device=xs.device) if norm else None
        out32 = torch.empty(n, d, dtype=torch.float32, device=xs.device) if norm and want32 else None
        self._call("jle_streams_mix_norm", _p(xs), kind, _p(plain), _p(routed), _p(inv), k, _p(shared), is_bf16,
                   _p(mix), _p(outw), _p(inw), _p(weight), float(eps), _p(out),
                   self._is_bf16(out) if out is not None else 0, _p(out32), n, s_, d, int(bool(norm)))
        return out, out32

    # ------------------------------------------------------------------ a matrix memory per head
    MLSTM_CHUNKS_FROM = 8  # a step with a segment of this many tokens takes the matrix memory in chunks

    def mlstm(self, rows, gates, b_gates, norm_weight, num_heads: int, head_dim: int, value_dim: int, cap: float,
              eps: float, floor: float, state, ctx):
        """``rows``: q | k | v | output gate in the run dtype; ``gates``: float32 ``[N, 2 H]`` pre-activations without
        their biases (overwritten).  Every segment's tokens in order from its request's state (``state[slot, phase]``),
        the new state to the other half; ``[N, H dv]`` in the run dtype."""
        n = rows.shape[0]
        H, dk, dv = num_heads, head_dim, value_dim
        self._chk(rows, None, (n, 2 * H * dk + 2 * H * dv), "q|k|v|gate rows")
        self._chk(gates, torch.float32, (n, 2 * H), "gate pre-activations")
        self._chk(b_gates, torch.float32, (2 * H,), "gate biases")
        self._chk(norm_weight, torch.float32, (H * dv,), "head norm weight")
        self._chk(state, torch.float32, (state.shape[0], 2, H, dk * dv + dk + 1), "matrix-memory state")
        r = ctx.num_segments
        self._chk(ctx.cu_seqlens, torch.int32, (r + 1,), "segment bounds")
        self._chk(ctx.state_slots, torch.int32, (r,), "state slots")
        self._chk(ctx.state_phase, torch.int32, (r,), "state phases")
        if ctx.num_tokens != n:
            raise KernelError("the rows do not fit the step")
        if dk > 256:
            raise KernelError(f"matrix-memory kernel: key size {dk} must be at most 256")
        o_raw = torch.empty(n, H * dv, dtype=torch.float32, device=rows.device)
        out = torch.empty(n, H * dv, dtype=rows.dtype, device=rows.device)
        if (max(ctx.seg_lens, default=0) >= self.MLSTM_CHUNKS_FROM
                and self._query("jle_mlstm_chunked_supported", dk, dv)):
            # a segment of many tokens: all segments in chunks that are worked on side by side
            table = ctx.scratch.get("mlstm_chunks")
            if table is None:
                per = int(self._query("jle_mlstm_chunk_tokens"))
                flat, firsts, o = [], [0], 0
                for i, ln in enumerate(ctx.seg_lens):
                    for t in range(0, ln, per):
                        flat += [i, o + t, min(per, ln - t)]
                    firsts.append(len(flat) // 3)
                    o += ln
                both = torch.tensor(flat + firsts, dtype=torch.int32).to(rows.device)
                table = ctx.scratch["mlstm_chunks"] = (both[: len(flat)], both[len(flat):], len(flat) // 3)
            chunks, seg_chunk0, nc = table
            ws = torch.empty(nc * H * (dk * dv + dk + 3), dtype=torch.float32, device=rows.device)
            ws_c, ws_n = ws[: nc * H * dk * dv], ws[nc * H * dk * dv: nc * H * (dk * dv + dk)]
            ws_m, ws_m0 = ws[nc * H * (dk * dv + dk): nc * H * (dk * dv + dk + 2)], ws[nc * H * (dk * dv + dk + 2):]
            self._call("jle_mlstm_chunked", _p(rows), self._is_bf16(rows), _p(gates), _p(b_gates), _p(norm_weight),
                       _p(state), _p(ctx.state_slots), _p(ctx.state_phase), _p(chunks), nc, _p(seg_chunk0), _p(ws_c),
                       _p(ws_n), _p(ws_m), _p(ws_m0), _p(o_raw), _p(out), n, r, H, dk, dv, float(cap), float(eps),
                       float(floor))
            return out
        self._call("jle_mlstm", _p(rows), self._is_bf16(rows), _p(gates), _p(b_gates), _p(norm_weight), _p(state),
                   _p(ctx.cu_seqlens), _p(ctx.state_slots), _p(ctx.state_phase), _p(o_raw), _p(out), n, r, H, dk, dv,
                   float(cap), float(eps), float(floor))
        return out

    def add_norm_pair(self, x, delta, injected, weight_a, weight_b, eps: float, out_dtype, second: bool = False,
                      norm: bool = True):
        """``x += delta`` in place (``delta``: ``None``, a tensor, or a :class:`~..parts.residual.BranchSum` whose two
        tensors the kernel adds up in float32), ``x += rows + vector`` for ``injected = (rows or None, vector)``,
        then the row's statistics once and ``h * weight_a`` and (``second``) ``h * weight_b`` in the run dtype.
        ``norm=False``: the sums only."""
        n, d = x.shape
        self._chk(x, torch.float32, (n, d), "residual")
        a = b = None
        if delta is not None:
            delta = self.materialize(delta)
            a, b = (delta.a, delta.b) if hasattr(delta, "a") else (delta, None)
            self._chk(a, out_dtype, (n, d), "branch output")
            if b is not None:
                self._chk(b, out_dtype, (n, d), "second branch output")
        rows = vec = None
        if injected is not None:
            rows, vec = injected
            if rows is not None:
                self._chk(rows, torch.float32, (n, d), "injected rows")
            self._chk(vec, torch.float32, (d,), "injected vector")
        for w in (weight_a, weight_b):
            if w is not None:
                self._chk(w, torch.float32, (d,), "norm weight")
        h_a = torch.empty(n, d, dtype=out_dtype, device=x.device) if norm else None
        h_b = torch.empty(n, d, dtype=out_dtype, device=x.device) if norm and second else None
        self._call("jle_add_norm_pair", _p(x), _p(a), _p(b), _p(rows), _p(vec), _p(weight_a), _p(weight_b), float(eps),
                   _p(h_a), _p(h_b), 1 if out_dtype == torch.bfloat16 else 0, n, d)
        return h_a, h_b

    SHIFT_ROWS_PER_BLOCK = 4  # a block of the norm-and-shift kernel takes so many rows in a step of many tokens
    # (it forms the row before its first anew: with one row a block every row is formed twice)

    def add_norm_shift(self, x, delta, weight, eps: float, out_dtype, shift, ctx, do_norm: bool = True):
        """``x' = x + delta`` into a new tensor (``delta``: ``None``, a tensor, or a gated branch
        ``rmsnorm((y + b) * sigmoid(g + c)) * w_b`` that the kernel forms on the fly), ``h = rmsnorm(x') * weight``
        and, with ``shift = (w, state)``, ``hs = h + (h_prev - h) * w`` with the float32 ``h`` of the token before
        (from the request's two-halved state across steps).  Returns ``(x', h, hs or None)``."""
        n, d = x.shape
        self._chk(x, torch.float32, (n, d), "residual")
        delta = self.materialize(delta) if isinstance(delta, ExpertSum) else delta
        kind, y, yb, g, gb, pw, peps = 0, None, None, None, None, None, 0.0
        if hasattr(delta, "gate"):
            kind, y, yb, g, gb, pw, peps = 2, delta.y, delta.y_bias, delta.gate, delta.gate_bias, delta.weight, delta.eps
            self._chk(y, None, (n, d), "branch output")
            self._chk(g, y.dtype, (n, d), "gate")
            for t, what in ((yb, "branch bias"), (gb, "gate bias"), (pw, "norm weight")):
                if t is not None:
                    self._chk(t, torch.float32, (d,), what)
        elif delta is not None:
            kind, y = 1, self._chk(delta, None, (n, d), "branch output")
        if y is not None and y.dtype != out_dtype:
            raise KernelError(f"branch output in {y.dtype}, rows wanted in {out_dtype}")
        if weight is not None:
            self._chk(weight, torch.float32, (d,), "norm weight")
        x_out = torch.empty_like(x) if kind else None
        h = torch.empty(n, d, dtype=out_dtype, device=x.device) if do_norm else None
        hs = sw = state = None
        rows = 1
        if shift is not None:
            sw, state = shift
            self._chk(sw, torch.float32, (d,), "shift weight")
            self._chk(state, torch.float32, (state.shape[0], 2, d), "shift state")
            hs = torch.empty(n, d, dtype=out_dtype, device=x.device)
            rows = self.SHIFT_ROWS_PER_BLOCK if n >= self._compute_units * self.SHIFT_ROWS_PER_BLOCK else 1
        is_bf16 = 1 if out_dtype == torch.bfloat16 else 0
        self._call("jle_add_norm_shift", _p(x), _p(x_out), kind, _p(y), _p(yb), _p(g), _p(gb), _p(pw), float(peps),
                   int(do_norm), _p(weight), float(eps), _p(h), _p(sw), _p(hs), _p(state),
                   _p(ctx.positions) if shift is not None else None,
                   _p(ctx.token_segment) if shift is not None else None,
                   _p(ctx.cu_seqlens) if shift is not None else None,
                   _p(ctx.state_slots) if shift is not None else None,
                   _p(ctx.state_phase) if shift is not None else None, is_bf16, n, d, rows)
        return (x_out if kind else x), h, hs

    def polynorm(self, z, bias, coef, eps: float):
        """``c0 N(u) + c1 N(u^2) + c2 N(u^3) + c3`` with ``u = z + bias``, ``N`` a row's division by its root mean
        square (float32 inside)."""
        n, f = z.shape
        self._chk(z, None, (n, f), "feed-forward rows")
        self._chk(coef, torch.float32, (4,), "activation coefficients")
        if bias is not None:
            self._chk(bias, torch.float32, (f,), "bias")
        out = torch.empty_like(z)
        self._call("jle_polynorm", _p(z), f, _p(bias), _p(coef), float(eps), _p(out), self._is_bf16(z), n, f)
        return out

    def batched_linear(self, a, w, tokens_first: bool = False):
        """``out[b] = a[b] @ w[b]`` for ``a [B, N, K]``, ``w [B, K, M]`` (views with any strides): a library
        product, true float32 in float32.  ``[B, N, M]``, or with ``tokens_first`` laid out ``[N, B, M]``."""
        out = torch.bmm(a, w)
        if not tokens_first:
            return out
        b, n, m = out.shape
        row_bytes = m * out.element_size()
        if row_bytes % 4 or not out.is_contiguous():
            return out.transpose(0, 1).contiguous()
        swapped = torch.empty(n, b, m, dtype=out.dtype, device=out.device)
        self._call("jle_swap_leading", _p(out), _p(swapped), b, n, row_bytes)
        return swapped

    def latent_prepare(self, rows, num_heads: int, nope_dim: int, rope_dim: int, kv_rank: int, positions, rotation,
                       latent_norm, eps: float, latent_pages, rope_pages, slot_mapping, writes: bool,
                       latent_t_pages=None) -> None:
        """``latent_t_pages``: a second copy of the latent, per page ``[kv_rank, page_size]`` (the page's tokens
        side by side), which the matrix-core attention kernel reads for its second product."""
        n, ld = rows.shape
        self._chk(rows, None, None, "projected rows")
        self._chk(positions, torch.int32, (n,), "positions")
        pairing, rd, inv = 0, 0, None
        magnitude = 1.0 if rotation is None else float(getattr(rotation, "magnitude", 1.0))
        if rotation is not None:
            rd = int(rotation.rotary_dim) or rope_dim
            pairing = {"adjacent": 0, "half": 1}[rotation.pairing]
            inv = self._chk(rotation.inv_freq, torch.float32, (rd // 2,), "rotary frequencies")
        if writes:
            np_, ps = latent_pages.shape[0], latent_pages.shape[1]
            self._chk(latent_pages, rows.dtype, (np_, ps, kv_rank), "latent pages")
            self._chk(rope_pages, rows.dtype, (np_, ps, rope_dim), "rotated key pages")
            if latent_t_pages is not None:
                self._chk(latent_t_pages, rows.dtype, (np_, ps, kv_rank), "transposed latent pages")
            self._chk(slot_mapping, torch.int32, (n,), "slot mapping")
            if latent_norm is not None:
                self._chk(latent_norm, torch.float32, (kv_rank,), "latent norm weight")
        self._call("jle_latent_prepare", _p(rows), ld, num_heads, nope_dim, rope_dim, kv_rank, _p(positions), _p(inv),
                   pairing, rd, magnitude, _p(latent_norm) if writes else None, float(eps),
                   _p(latent_pages) if writes else None, _p(rope_pages) if writes else None,
                   _p(latent_t_pages) if writes else None, latent_pages.shape[1] if writes else 0,
                   _p(slot_mapping) if writes else None, int(bool(writes)), self._is_bf16(rows), n)

    LATENT_SPLIT_BELOW = 2048  # fewer (token, head) pairs than this: a query's key tiles are shared between wavefronts

    LATENT_MFMA_ITEMS = 1024  # the matrix-core kernel: fewer row tiles than this share their key steps between
    # wavefronts, about so many work items in all (measured at 256 / 512 / 1,024 / 2,048: batch 64 at 2,048 tokens of
    # context 296 / 168 / 117 / 130 us a layer, batch 16 80 / 58 / 48 / 63)
    LATENT_LDS_TILES = 1024  # from so many row tiles on: the kernel whose blocks share keys through shared memory

    def latent_attention(self, q_lat, q, nope_dim: int, latent_pages, rope_pages, block_table, positions,
                         token_segment, window, scale: float, meta=None, latent_t_pages=None, sink=None):
        """See ``attention_latent.hip``.  ``q_lat [H, N, kv_rank]``, ``q [N, H, nope + rope]`` (a view of the
        projected rows: the heads' queries lie at their start); returns ``[N, H, kv_rank]``.  In bfloat16, with the
        latent's transposed copy and sizes that fit, on the matrix cores; else in float32 arithmetic."""
        H, n, r = q_lat.shape
        dr = q.shape[2] - nope_dim
        np_, ps = latent_pages.shape[0], latent_pages.shape[1]
        self._chk(q_lat, latent_pages.dtype, (H, n, r), "queries in the latent's space")
        if q.dtype != q_lat.dtype or q.stride(2) != 1 or q.stride(1) != q.shape[2] or q.shape[:2] != (n, H):
            raise KernelError("the heads' queries must lie side by side at the start of contiguous rows")
        q_ld = q.stride(0)  # (rows that also hold the latent: a token's queries are addressed by the row's full width)
        self._chk(latent_pages, None, (np_, ps, r), "latent pages")
        self._chk(rope_pages, latent_pages.dtype, (np_, ps, dr), "rotated key pages")
        self._chk(block_table, torch.int32, None, "block table")
        self._chk(positions, torch.int32, (n,), "positions")
        self._chk(token_segment, torch.int32, (n,), "token segments")
        w = 0 if window is None else int(window)
        if sink is not None:
            self._chk(sink, torch.float32, (H,), "sinks")
        out = torch.empty(n, H, r, dtype=q_lat.dtype, device=q_lat.device)
        if (latent_t_pages is not None and q_lat.dtype == torch.bfloat16
                and self._query("jle_latent_attention_mfma_supported", r, nope_dim, dr, q_ld, ps)):
            self._chk(latent_t_pages, latent_pages.dtype, (np_, ps, r), "transposed latent pages")
            return self._latent_attention_mfma(q_lat, q, q_ld, nope_dim, dr, latent_pages, latent_t_pages, rope_pages,
                                               out, block_table, positions, token_segment, w, scale, meta, sink)
        splits, tiles_per_split, ws_ml, ws_o = 1, 0, None, None
        waves = n * H
        if waves < self.LATENT_SPLIT_BELOW:
            if meta is not None and meta.decode_bucket is not None:
                longest = meta.decode_bucket  # (a step of single tokens: laid out for the bound, see GroupContext)
            elif meta is not None and meta.seg_starts is not None:
                longest = max(s0 + ln for s0, ln in zip(meta.seg_starts, meta.seg_lens))
            else:
                longest = int(positions.max()) + 1
            span = min(w, longest) if w else longest
            tiles = -(-span // 64) + 1
            want = min(tiles, -(-self.LATENT_SPLIT_BELOW // waves))
            if want > 1:
                tiles_per_split = -(-tiles // want)
                splits = -(-tiles // tiles_per_split)
                ws_ml = torch.empty(waves * splits * 2, dtype=torch.float32, device=q.device)
                ws_o = torch.empty(waves * splits * r, dtype=torch.float32, device=q.device)
        self._call("jle_latent_attention", _p(q_lat), _p(q), q_ld, nope_dim, dr, _p(latent_pages), _p(rope_pages), _p(out),
                   _p(positions), _p(token_segment), _p(block_table), block_table.shape[1], w, float(scale),
                   self._is_bf16(q_lat), n, H, r, ps, splits, tiles_per_split, _p(ws_ml), _p(ws_o), _p(sink))
        return out

    def _latent_attention_mfma(self, q_lat, q, q_ld, dn, dr, latent_pages, latent_t_pages, rope_pages, out,
                               block_table, positions, token_segment, window, scale, meta, sink=None):
        H, n, r = q_lat.shape
        ps = latent_pages.shape[1]
        # row tiles: 16 consecutive (token, head) pairs of one segment
        key = f"latent_tiles_{H}"
        plan = meta.meta.get(key) if meta is not None else None
        if plan is None:
            seg_lens = meta.seg_lens if meta is not None and meta.seg_lens else \
                self._segments(meta, token_segment, positions)[0]
            flat, o = [], 0
            for ln in seg_lens:
                rows = ln * H
                for t in range(0, rows, 16):
                    flat += [o * H + t, min(16, rows - t)]
                o += ln
            plan = torch.tensor(flat, dtype=torch.int32).to(q_lat.device)
            if meta is not None:
                meta.meta[key] = plan
        tiles = plan.numel() // 2
        if tiles >= self.LATENT_LDS_TILES:
            # many rows: blocks of four neighbouring tiles that share their keys through shared memory
            key = f"latent_blocks_{H}"
            blocks = meta.meta.get(key) if meta is not None else None
            if blocks is None:
                seg_lens = meta.seg_lens if meta is not None and meta.seg_lens else \
                    self._segments(meta, token_segment, positions)[0]
                # (blocks with the most keys first: the compute units take them in order, and the last ones to start
                # should be the short ones)
                seg_starts = meta.seg_starts if meta is not None and meta.seg_starts else [0] * len(seg_lens)
                keyed, o = [], 0
                for ln, start in zip(seg_lens, seg_starts):
                    rows = ln * H
                    for t in range(0, rows, 64):
                        nrows = min(64, rows - t)
                        last = start + (t + nrows - 1) // H  # the position of the block's last token
                        keys = last + 1 if not window else min(last + 1, window + -(-nrows // H))
                        keyed.append((-keys, len(keyed), o * H + t, nrows))
                    o += ln
                keyed.sort()
                flat = [v for _, _, row0, nrows in keyed for v in (row0, nrows)]
                blocks = torch.tensor(flat, dtype=torch.int32).to(q_lat.device)
                if meta is not None:
                    meta.meta[key] = blocks
            self._call("jle_latent_attention_lds", _p(q_lat), _p(q), q_ld, dn, dr, _p(latent_pages),
                       _p(latent_t_pages), _p(rope_pages), _p(out), _p(positions), _p(token_segment), _p(block_table),
                       block_table.shape[1], window, float(scale), _p(blocks), blocks.numel() // 2, n, H, r, ps,
                       _p(sink))
            return out
        splits, steps_per_split, ws_ml, ws_o = 1, 0, None, None
        if tiles < self.LATENT_MFMA_ITEMS:
            if meta is not None and meta.decode_bucket is not None:
                longest = meta.decode_bucket  # (a step of single tokens: laid out for the bound, see GroupContext)
            elif meta is not None and meta.seg_starts is not None:
                longest = max(s0 + ln for s0, ln in zip(meta.seg_starts, meta.seg_lens))
            else:
                longest = int(positions.max()) + 1
            span = min(window, longest) if window else longest
            spanned = -(-16 // H) + 1 if H < 16 else 1  # tokens whose rows may share a tile
            steps = -(-(span + spanned + 31) // 32)
            want = min(steps, -(-self.LATENT_MFMA_ITEMS // tiles))
            if want > 1:
                steps_per_split = -(-steps // want)
                splits = -(-steps // steps_per_split)
                ws_ml = torch.empty(n * H * splits * 2, dtype=torch.float32, device=q_lat.device)
                ws_o = torch.empty(n * H * splits * r, dtype=torch.float32, device=q_lat.device)
        self._call("jle_latent_attention_mfma", _p(q_lat), _p(q), q_ld, dn, dr, _p(latent_pages), _p(latent_t_pages),
                   _p(rope_pages), _p(out), _p(positions), _p(token_segment), _p(block_table), block_table.shape[1],
                   window, float(scale), _p(plan), tiles, n, H, r, ps, splits, steps_per_split, _p(ws_ml), _p(ws_o),
                   _p(sink))
        return out

    def scaled_add_norm(self, x, delta, weight, eps: float, out_dtype, want32: bool = False, norm: bool = True):
        """``x += vector * sum_i factor_i * term_i`` in place for a :class:`~..parts.residual.ScaledSum` (terms in the
        run dtype or float32; a sum of expert outputs still in pieces is formed first), then (``norm``) ``h = x /
        sqrt(mean(x^2) + eps) * weight`` in the run dtype and, if wanted, float32; one launch."""
        n, d = x.shape
        self._chk(x, torch.float32, (n, d), "residual")
        terms = list(delta.terms)
        inv, inv_k = None, 0
        if isinstance(terms[0][0], ExpertSum) and terms[0][0].shared is None:  # (its pieces are added up by the kernel)
            pieces = terms[0][0]
            inv, inv_k = pieces.inv, pieces.k
            terms[0] = (pieces.routed, terms[0][1])
            self._chk(pieces.routed, None, (pieces.routed.shape[0], d), "expert outputs")
            self._chk(inv, torch.int32, (n * inv_k,), "rows of the expert outputs")
        terms = [(self.materialize(t), f) for t, f in terms]
        for t, _ in terms[(1 if inv is not None else 0):]:
            self._chk(t, None, (n, d), "branch output")
        kind = lambda t: 1 if t.dtype == torch.bfloat16 else 2 if t.dtype == torch.float32 else self._is_bf16(t)
        (a, fa), (b, fb) = terms[0], (terms[1] if len(terms) > 1 else (None, 0.0))
        if delta.vector is not None:
            self._chk(delta.vector, torch.float32, (d,), "channel scale")
        if weight is not None:
            self._chk(weight, torch.float32, (d,), "norm weight")
        h = torch.empty(n, d, dtype=out_dtype, device=x.device) if norm else None
        h32 = torch.empty(n, d, dtype=torch.float32, device=x.device) if norm and want32 else None
        self._call("jle_scaled_add_norm", _p(x), _p(a), kind(a), float(fa), _p(b), 0 if b is None else kind(b),
                   float(fb), _p(delta.vector), _p(weight), float(eps), _p(h),
                   1 if out_dtype == torch.bfloat16 else 0, _p(h32), n, d, _p(inv), inv_k)
        return h, h32

    def add_rmsnorm(self, x, delta, weight, eps: float, out_dtype, want32: bool = False):
        if hasattr(delta, "terms"):  # a sum with factors: the kernel that knows it
            return self.scaled_add_norm(x, delta, weight, eps, out_dtype, want32)
        if hasattr(delta, "a"):  # the sum of two parallel branches: the kernel that knows it
            h, _ = self.add_norm_pair(x, delta, None, weight, None, eps, out_dtype)
            return h, (h.float() if want32 else None)
        if hasattr(delta, "gate"):  # a gated branch: the kernel that knows it (the sum goes into a new array)
            x_out, h, _ = self.add_norm_shift(x, delta, weight, eps, out_dtype, None, None)
            x.copy_(x_out)
            return h, (h.float() if want32 else None)
        n, d = x.shape
        self._chk(x, torch.float32, (n, d), "residual")
        kind, plain, routed, inv, k, shared, is_bf16 = 0, None, None, None, 0, None, 0
        if isinstance(delta, ExpertSum):
            kind, routed, inv, k, shared = 2, delta.routed, delta.inv, delta.k, delta.shared
            is_bf16 = self._is_bf16(routed)
        elif delta is not None:
            self._chk(delta, None, (n, d), "branch output")
            kind, plain, is_bf16 = 1, delta, self._is_bf16(delta)
        if weight is not None:
            self._chk(weight, torch.float32, (d,), "norm weight")
        out = torch.empty(n, d, dtype=out_dtype, device=x.device)
        out32 = torch.empty(n, d, dtype=torch.float32, device=x.device) if want32 else None
        self._call("jle_add_rmsnorm", _p(x), kind, _p(plain), _p(routed), _p(inv), k, _p(shared), is_bf16, _p(weight),
                   float(eps), _p(out), self._is_bf16(out), _p(out32), n, d)
        return out, out32

    def defer_norm(self, x, delta, weight, eps: float, out_dtype) -> PendingNorm:
        """``add_rmsnorm`` put off until a consumer asks for the rows (see :class:`PendingNorm`).  Only for
        consumers that say they take one."""
        return PendingNorm(self, x, delta, weight, eps, out_dtype)

    @staticmethod
    def _rows(h, want32: bool = False):
        return h.rows(want32) if isinstance(h, PendingNorm) else h

    def materialize(self, delta):
        """The tensor an :class:`ExpertSum` (or a sum with factors) stands for (float32); anything else as it is."""
        if hasattr(delta, "terms"):
            first = delta.terms[0][0]
            total = torch.zeros(first.shape[0], first.shape[1], dtype=torch.float32, device=self.device)
            self.scaled_add_norm(total, delta, None, 0.0, torch.float32, norm=False)
            return total
        if not isinstance(delta, ExpertSum):
            return delta
        n, d = delta.shape
        out = torch.empty(n, d, dtype=torch.float32, device=delta.routed.device)
        self._call("jle_moe_combine", _p(delta.routed), _p(delta.inv), _p(delta.shared), _p(out),
                   self._is_bf16(delta.routed), n, delta.k, d)
        return out

    def add_residual(self, x, delta) -> None:
        if hasattr(delta, "terms"):
            self.scaled_add_norm(x, delta, None, 0.0, torch.float32, norm=False)
            return
        if hasattr(delta, "a"):
            self.add_norm_pair(x, delta, None, None, None, 0.0, delta.dtype, norm=False)
            return
        if hasattr(delta, "gate"):
            x_out, _, _ = self.add_norm_shift(x, delta, None, 0.0, delta.y.dtype, None, None, do_norm=False)
            x.copy_(x_out)
            return
        delta = self.materialize(delta)
        self._chk(x, torch.float32, None, "residual")
        self._chk(delta, None, x.shape, "branch output")
        self._call("jle_add_residual", _p(x), _p(delta), self._is_bf16(delta), x.numel())

    def gather_rows(self, x, idx):
        x = self.materialize(x)
        m = idx.numel()
        self._chk(x, None, None, "rows")
        self._chk(idx, torch.int32, (m,), "row indices")
        out = torch.empty(m, x.shape[1], dtype=x.dtype, device=x.device)
        self._call("jle_gather_rows", _p(x), _p(idx), _p(out), m, x.shape[1] * x.element_size())
        return out

    # ------------------------------------------------------------------ matrix products
    def linear(self, h, w, out_dtype=None):
        """``h @ w.T``: through the BLAS library (float32: true float32); a few bfloat16 rows through the
        weight-streaming kernel, which is as fast there or faster and much cheaper to launch."""
        h = self._rows(h)
        if (h.dtype == torch.bfloat16 and h.shape[0] <= self.SKINNY_LINEAR_ROWS and w.dim() == 2
                and w.dtype == torch.bfloat16 and w.shape[1] % 8 == 0 and h.is_contiguous() and w.is_contiguous()):
            out = self.gemm_skinny(h, w)
            return out if out_dtype is None or out_dtype == out.dtype else out.to(out_dtype)
        out = torch.matmul(h, w.t())
        return out if out_dtype is None or out_dtype == out.dtype else out.to(out_dtype)

    def linear_bias(self, h, w, bias, bias_run=None):
        """``h @ w.T + bias``.  Returns ``(rows, bias still to be added or None)``: the library's product adds the
        bias itself (``bias_run``: the bias in the operands' dtype) and rounds once; the weight-streaming kernel
        for few rows hands out float32 rows and leaves the bias to the kernel that reads them next."""
        h = self._rows(h)
        if bias is None:
            return self.linear(h, w), None
        if (h.dtype == torch.bfloat16 and h.shape[0] <= self.SKINNY_LINEAR_ROWS and w.dtype == torch.bfloat16
                and w.shape[1] % 8 == 0 and h.is_contiguous() and w.is_contiguous()):
            return self.gemm_skinny(h, w, out_f32=True), bias
        if bias_run is None:
            bias_run = bias.to(h.dtype)
        return torch.addmm(bias_run, h, w.t()), None

    _ACTS = {"silu": 0, "gelu_tanh": 1}

    def swiglu_linear(self, h, w_gate_up, activation: str = "silu"):
        """``act(h @ Wg.T) * (h @ Wu.T)`` with ``w_gate_up`` = gate rows, then up rows; ``act``: ``silu`` or
        ``gelu_tanh``."""
        h = self._rows(h)
        act = self._ACTS[activation]
        if h.dtype == torch.bfloat16 and h.shape[0] <= self.SKINNY_DENSE_ROWS and h.shape[1] % 8 == 0:
            return self.gemm_skinny(h, w_gate_up, swiglu=1 + act)  # (the activation in the product's epilogue)
        return self.silu_mul(torch.matmul(h, w_gate_up.t()), activation)

    def sigmoid_mul(self, o, gate):
        """``o * sigmoid(gate)``; ``gate`` may be a slice of wider rows (its last axis contiguous)."""
        n, c = o.shape
        self._chk(o, None, (n, c), "rows")
        if gate.dtype != o.dtype or tuple(gate.shape) != (n, c) or gate.stride(1) != 1 or not gate.is_cuda:
            raise KernelError("the gate must have the rows' shape and dtype, its last axis contiguous")
        out = torch.empty_like(o)
        self._call("jle_sigmoid_mul", _p(o), _p(gate), gate.stride(0) if n > 1 else c, _p(out), self._is_bf16(o), n, c)
        return out

    def conv_attention(self, proj, bias, conv_w, taps: int, state, num_heads: int, num_kv_heads: int, head_dim: int,
                       value_dim: int, page_dim: int, prep, ctx, kv_cache, writes: bool, slot_mapping, block_table,
                       retention, scale: float, meta=None):
        """From the projected q|k|v rows to the attention output ``[N, num_heads * page_dim]``.  Where queries, keys
        and values have one size and the rotation's magnitude can be told as a smaller eps of the norm behind it
        (a rotation over the whole head turns nothing's length: ``m x / sqrt(m^2 s + eps) = x / sqrt(s + eps /
        m^2)``), a kernel does bias, convolution and state, and the rows then go the way of any fused q|k|v rows
        (:meth:`attention_from_qkv`: a step of single tokens is one more launch).  Everything else goes through
        the kernel that also rotates, norms, fills heads up and writes the pages."""
        rot = prep.rotation
        rd = 0 if rot is None else (int(rot.rotary_dim) or head_dim)
        m = 1.0 if rot is None else float(rot.magnitude)
        if (head_dim == value_dim == page_dim and (m == 1.0 or (rd == head_dim and prep.norm_eps is not None))
                and prep.norm_weight_q is None and prep.norm_weight_k is None and not prep.norm_first
                and prep.query_scale is None):
            rows = self.conv_rows(proj, bias, conv_w, taps, state, ctx)
            plain = prep
            if m != 1.0:
                from ..parts.base import QKPreparation, Rotation

                plain = getattr(prep, "_told_plainly", None)  # (made once, kept on the preparation itself)
                if plain is None:
                    plain = QKPreparation(rotation=Rotation(rot.inv_freq, rot.pairing, rot.rotary_dim, 1.0),
                                          norm_eps=float(prep.norm_eps) / (m * m))
                    prep._told_plainly = plain
            return self.attention_from_qkv(rows, num_heads, num_kv_heads, head_dim, ctx.positions, ctx.token_segment,
                                           plain, kv_cache, writes, slot_mapping, block_table, retention, scale, meta)
        q = self.conv_qk_prepare(proj, bias, conv_w, taps, state, num_heads, num_kv_heads, head_dim, value_dim,
                                 page_dim, prep, ctx, kv_cache if writes else None, slot_mapping)
        return self.paged_attention(q, kv_cache, block_table, ctx.positions, ctx.token_segment, retention, scale, meta)

    def conv_rows(self, proj, bias, conv_w, taps: int, state, ctx, activation=None):
        """``y[t] = sum_j conv_w[j] * u[t - taps + 1 + j]`` (``conv_w``: ``[taps, channels]``) with ``u = proj + bias`` rounded to the run dtype, rows
        before a segment's start from the requests' two-halved state, whose other half gets the segment's last
        ``taps - 1`` rows of ``u``; ``[N, C]`` in the run dtype.  See ``attention_conv.hip``."""
        n, channels = proj.shape
        dt = ctx.dtype
        self._chk(proj, None, (n, channels), "projected rows")
        if proj.dtype not in (dt, torch.float32):
            raise KernelError(f"projected rows in {proj.dtype}, run dtype {dt}")
        if bias is not None:
            self._chk(bias, torch.float32, (channels,), "bias")
        if taps:
            self._chk(conv_w, torch.float32, (taps, channels), "convolution taps")
        if taps > 1:
            self._chk(state, dt, (state.shape[0], 2, taps - 1, channels), "convolution state")
        for t, what, shape in ((ctx.token_segment, "token segments", (n,)),
                               (ctx.cu_seqlens, "segment bounds", (ctx.num_segments + 1,)),
                               (ctx.state_slots, "state slots", (ctx.num_segments,)),
                               (ctx.state_phase, "state phases", (ctx.num_segments,))):
            self._chk(t, torch.int32, shape, what)
        y = torch.empty(n, channels, dtype=dt, device=proj.device)
        if activation is not None:  # (on the convolution's result, float32, before the rounding)
            if activation != "silu":
                raise KernelError(f"the convolution kernel knows the activation silu, not {activation!r}")
            self._call("jle_conv_rows_act", _p(proj), 1 if proj.dtype == torch.float32 else 0, _p(bias),
                       _p(conv_w) if taps else None, int(taps), _p(state) if taps > 1 else None,
                       _p(ctx.token_segment), _p(ctx.cu_seqlens), _p(ctx.state_slots), _p(ctx.state_phase), _p(y),
                       1 if dt == torch.bfloat16 else 0, n, ctx.num_segments, channels, 1)
            return y
        self._call("jle_conv_rows", _p(proj), 1 if proj.dtype == torch.float32 else 0, _p(bias),
                   _p(conv_w) if taps else None, int(taps), _p(state) if taps > 1 else None, _p(ctx.token_segment),
                   _p(ctx.cu_seqlens), _p(ctx.state_slots), _p(ctx.state_phase), _p(y),
                   1 if dt == torch.bfloat16 else 0, n, ctx.num_segments, channels)
        return y

    def heads_prepare(self, rows, q_heads: int, k_heads: int, v_heads: int, head_dim: int, value_dim: int,
                      page_dim: int, prep, positions, kv_cache, slot_mapping):
        """See ``attention_heads.hip``: q and k normed and rotated as ``prep`` says, keys and values into pages with
        heads of ``page_dim`` elements (a value head once for each of the ``k_heads / v_heads`` key heads that use
        it).  Returns q ``[N, q_heads, page_dim]``."""
        n = rows.shape[0]
        dk, dv, D = head_dim, value_dim, page_dim
        self._chk(rows, None, (n, (q_heads + k_heads) * dk + v_heads * dv), "projected rows")
        dt = rows.dtype
        if prep.query_scale is not None or prep.norm_span != "head":
            raise KernelError("this preparation kernel has no query scale and norms a head at a time")
        rot = prep.rotation
        inv_freq, rd, magnitude, half = None, 0, 1.0, 0
        if rot is not None:
            rd = int(rot.rotary_dim) or dk
            inv_freq, magnitude = self._chk(rot.inv_freq, torch.float32, (rd // 2,), "inv_freq"), float(rot.magnitude)
            half = 1 if rot.pairing == "half" else 0
        for w in (prep.norm_weight_q, prep.norm_weight_k):
            if w is not None:
                self._chk(w, torch.float32, (dk,), "q/k norm weight")
        self._chk(positions, torch.int32, (n,), "positions")
        ps = 1
        if kv_cache is not None:
            ps = kv_cache.shape[3]
            self._chk(kv_cache, dt, (kv_cache.shape[0], 2, k_heads, ps, D), "kv pages")
            self._chk(slot_mapping, torch.int32, (n,), "slot mapping")
        q = torch.empty(n, q_heads, D, dtype=dt, device=rows.device)
        self._call("jle_heads_prepare", _p(rows), _p(positions), _p(slot_mapping) if kv_cache is not None else None,
                   _p(inv_freq), rd, half, magnitude, -1.0 if prep.norm_eps is None else float(prep.norm_eps),
                   1 if prep.norm_first else 0, _p(prep.norm_weight_q), _p(prep.norm_weight_k), _p(q), _p(kv_cache),
                   self._is_bf16(rows), n, q_heads, k_heads, v_heads, dk, dv, D, ps)
        return q

    def diff_combine(self, o, lam: float, out_scale: float, eps: float, gate, num_heads: int, num_kv_heads: int,
                     page_dim: int, value_dim: int):
        """Two score maps' outputs ``[N, 2 H page_dim]`` (``[kv head][map][query head of the group]``) into ``(a1 - lam
        a2) / rms * out_scale * sigmoid(gate)``, ``[N, H value_dim]`` in the heads' own order."""
        n = o.shape[0]
        self._chk(o, None, (n, 2 * num_heads * page_dim), "attention output")
        if gate is not None:
            self._chk(gate, o.dtype, (n, num_heads * value_dim), "output gate")
        out = torch.empty(n, num_heads * value_dim, dtype=o.dtype, device=o.device)
        self._call("jle_diff_combine", _p(o), _p(gate), _p(out), float(lam), float(out_scale), float(eps),
                   self._is_bf16(o), n, num_heads, num_kv_heads, page_dim, value_dim)
        return out

    def gated_delta(self, rows, gates, a_log, dt_bias, norm_weight, out_gate, num_heads: int, num_kv_heads: int,
                    head_dim: int, value_dim: int, eps: float, floor: float, state, ctx):
        """See ``gated_delta.hip``: unit vectors, write strengths and decays of the step's tokens, the recurrence
        from and into the requests' two-halved memory, head norm and output gate.  ``[N, H dv]`` in the run dtype."""
        n = rows.shape[0]
        H, G, dk, dv = num_heads, num_kv_heads, head_dim, value_dim
        self._chk(rows, None, (n, 2 * G * dk + H * dv), "q | k | v rows")
        self._chk(out_gate, rows.dtype, (n, H * dv), "output gate")
        self._chk(gates, torch.float32, (n, 2 * H), "gate pre-activations")
        self._chk(state, torch.float32, (state.shape[0], 2, H, dv, dk), "memory")
        for t, shape, what in ((a_log, (H,), "a_log"), (dt_bias, (H,), "dt_bias"), (norm_weight, (dv,), "head norm weight")):
            self._chk(t, torch.float32, shape, what)
        for t, what, shape in ((ctx.cu_seqlens, "segment bounds", (ctx.num_segments + 1,)),
                               (ctx.state_slots, "state slots", (ctx.num_segments,)),
                               (ctx.state_phase, "state phases", (ctx.num_segments,))):
            self._chk(t, torch.int32, shape, what)
        dev = rows.device
        dkp = self._query("jle_gated_delta_padded", dk)  # (the unit vectors' rows, filled up to what the scan's lanes hold)
        if dkp < dk:
            raise KernelError(f"the gated delta rule's kernels take keys of up to 2048 elements, not {dk}")
        scratch = torch.empty(n * (2 * G * dkp + 2 * H + G + H * dv), dtype=torch.float32, device=dev)
        qn, kn = scratch[: n * G * dkp], scratch[n * G * dkp: 2 * n * G * dkp]
        o = 2 * n * G * dkp
        beta, decay, kq = scratch[o: o + n * H], scratch[o + n * H: o + 2 * n * H], scratch[o + 2 * n * H: o + 2 * n * H + n * G]
        o_raw = scratch[o + 2 * n * H + n * G:]
        out = torch.empty(n, H * dv, dtype=rows.dtype, device=dev)
        self._call("jle_gated_delta", _p(rows), self._is_bf16(rows), _p(gates), _p(a_log), _p(dt_bias), _p(norm_weight),
                   _p(out_gate), _p(state), _p(ctx.cu_seqlens), _p(ctx.state_slots), _p(ctx.state_phase), _p(qn), _p(kn),
                   _p(beta), _p(decay), _p(kq), _p(o_raw), _p(out), n, ctx.num_segments, H, G, dk, dv, float(eps),
                   float(floor))
        return out

    def conv_qk_prepare(self, proj, bias, conv_w, taps: int, state, num_heads: int, num_kv_heads: int, head_dim: int,
                        value_dim: int, page_dim: int, prep, ctx, kv_cache, slot_mapping):
        """See ``attention_conv.hip``: bias, causal convolution over time from the step's rows and the requests'
        two-halved state, rotation and weightless norm of q and k, pages written with heads of ``page_dim``
        elements.  Returns q ``[N, num_heads, page_dim]``."""
        n = proj.shape[0]
        hq, hk, dk, dv, D = num_heads, num_kv_heads, head_dim, value_dim, page_dim
        channels = (hq + hk) * dk + hk * dv
        dt = ctx.dtype
        self._chk(proj, None, (n, channels), "projected rows")
        if proj.dtype not in (dt, torch.float32):
            raise KernelError(f"projected rows in {proj.dtype}, run dtype {dt}")
        if prep.norm_weight_q is not None or prep.norm_weight_k is not None or prep.norm_first or prep.query_scale:
            raise KernelError("the convolution path norms q and k without weights after the rotation, no query scale")
        if bias is not None:
            self._chk(bias, torch.float32, (channels,), "bias")
        if taps:
            self._chk(conv_w, torch.float32, (taps, channels), "convolution taps")
        if taps > 1:
            self._chk(state, dt, (state.shape[0], 2, taps - 1, channels), "convolution state")
        rot = prep.rotation
        inv_freq, rd, magnitude = None, 0, 1.0
        if rot is not None:
            if rot.pairing != "adjacent":
                raise KernelError("the convolution path turns adjacent pairs")
            rd = int(rot.rotary_dim) or dk
            inv_freq, magnitude = self._chk(rot.inv_freq, torch.float32, (rd // 2,), "inv_freq"), float(rot.magnitude)
        ps = 0
        if kv_cache is not None:
            ps = kv_cache.shape[3]
            self._chk(kv_cache, dt, (kv_cache.shape[0], 2, hk, ps, D), "kv pages")
            self._chk(slot_mapping, torch.int32, (n,), "slot mapping")
        for t, what, shape in ((ctx.token_segment, "token segments", (n,)), (ctx.positions, "positions", (n,)),
                               (ctx.cu_seqlens, "segment bounds", (ctx.num_segments + 1,)),
                               (ctx.state_slots, "state slots", (ctx.num_segments,)),
                               (ctx.state_phase, "state phases", (ctx.num_segments,))):
            self._chk(t, torch.int32, shape, what)
        q = torch.empty(n, hq, D, dtype=dt, device=proj.device)
        self._call("jle_conv_qk_prepare", _p(proj), 1 if proj.dtype == torch.float32 else 0, _p(bias),
                   _p(conv_w) if taps else None, int(taps), _p(state) if taps > 1 else None, _p(ctx.token_segment),
                   _p(ctx.cu_seqlens), _p(ctx.state_slots), _p(ctx.state_phase), _p(ctx.positions),
                   _p(slot_mapping) if kv_cache is not None else None, _p(inv_freq), rd, magnitude,
                   -1.0 if prep.norm_eps is None else float(prep.norm_eps), _p(q), _p(kv_cache),
                   1 if dt == torch.bfloat16 else 0, n, ctx.num_segments, hq, hk, dk, dv, D, max(ps, 1))
        return q

    def gemm(self, a, b, *, offsets=None, a_rows=None, scale=None, out_f32=False, rows=None):
        """The hand-written product ``C[r] = scale[r] * A[a_rows[r]] @ B[g(r)].T`` (see ``gemm_generic.hip``)."""
        if b.dim() == 2:
            b = b.unsqueeze(0)
        g, nout, k = b.shape
        m = rows if rows is not None else (a_rows.numel() if a_rows is not None else a.shape[0])
        self._chk(a, b.dtype, None, "A")
        self._chk(b, None, None, "B")
        if a.shape[1] != k:
            raise KernelError(f"inner sizes differ: A {tuple(a.shape)}, B {tuple(b.shape)}")
        out = torch.empty(m, nout, dtype=torch.float32 if out_f32 else a.dtype, device=a.device)
        self._call("jle_gemm_generic", _p(a), _p(b), _p(out), _p(offsets), _p(a_rows), _p(scale), self._is_bf16(a),
                   1 if (out_f32 or a.dtype == torch.float32) else 0, m, nout, k, g)
        return out

    F32_SKINNY_ROWS = 128  # float32 grouped products: up to so many rows (of all groups together) the kernel whose
    # wavefronts split K; beyond, the one whose wavefronts hold up to 192 rows of a group (both on the float32 matrix
    # instructions); the general kernel where the sizes do not fit either

    def gemm_f32_skinny(self, a, b, *, offsets=None, a_rows=None, scale=None, swiglu=False, rows=None):
        """The float32 grouped product for few rows on the float32 matrix instructions (see ``gemm_f32.hip``):
        float32 operands, products and sums.  With ``swiglu`` the result is ``silu(gate) * up`` of the two halves
        of ``b``'s rows."""
        if b.dim() == 2:
            b = b.unsqueeze(0)
        g, nout, k = b.shape
        m = rows if rows is not None else (a_rows.numel() if a_rows is not None else a.shape[0])
        self._chk(a, torch.float32, None, "A")
        self._chk(b, torch.float32, None, "B")
        if a.shape[1] != k:
            raise KernelError(f"inner sizes differ: A {tuple(a.shape)}, B {tuple(b.shape)}")
        if k % 4 or a.data_ptr() % 16 or b.data_ptr() % 16:
            raise KernelError(f"the float32 matrix-core product needs an inner size that is a multiple of 4 and "
                              f"16-byte aligned rows, got K = {k}")
        out = torch.empty(m, nout // 2 if swiglu else nout, dtype=torch.float32, device=a.device)
        # (no more groups have rows than there are rows: so many group slots instead of every group)
        slots = m if offsets is not None and g > m else 0
        self._call("jle_gemm_f32_skinny", _p(a), _p(b), _p(out), _p(offsets), _p(a_rows), _p(scale), int(swiglu), m,
                   nout, k, g, m, slots)
        return out

    def f32_stream_supported(self, nout: int, k: int, swiglu: bool) -> bool:
        return bool(self._query("jle_gemm_f32_stream_supported", nout, k, int(swiglu)))

    def gemm_f32_stream(self, a, b, *, offsets=None, a_rows=None, scale=None, swiglu=False, rows=None):
        """The float32 grouped product for about a hundred rows per group on the float32 matrix instructions,
        the weights read once per 192 rows of a group (see ``gemm_f32.hip``)."""
        if b.dim() == 2:
            b = b.unsqueeze(0)
        g, nout, k = b.shape
        m = rows if rows is not None else (a_rows.numel() if a_rows is not None else a.shape[0])
        self._chk(a, torch.float32, None, "A")
        self._chk(b, torch.float32, None, "B")
        if a.shape[1] != k:
            raise KernelError(f"inner sizes differ: A {tuple(a.shape)}, B {tuple(b.shape)}")
        if a.numel() >= 2 ** 32:
            raise KernelError("the float32 weight-streaming grouped product addresses its rows with 32 bits")
        if not self.f32_stream_supported(nout, k, swiglu) or a.data_ptr() % 16 or b.data_ptr() % 16:
            raise KernelError(f"the float32 weight-streaming grouped product needs an inner size that is a multiple of "
                              f"64, whole tiles of 16 weight rows (32 with the fused activation) and 16-byte aligned "
                              f"rows, got {nout} x {k}")
        out = torch.empty(m, nout // 2 if swiglu else nout, dtype=torch.float32, device=a.device)
        self._call("jle_gemm_f32_stream", _p(a), _p(b), _p(out), _p(offsets), _p(a_rows), _p(scale), int(swiglu), m,
                   nout, k, g, m)
        return out

    SKINNY_MAX_ROWS = 64  # up to here a product is a stream of the weights: the MFMA weight-streaming kernel
    SKINNY_DENSE_ROWS = 16  # the fused gate|up projection of a dense feed-forward: beyond this the BLAS library
    SKINNY_LINEAR_ROWS = 8  # plain projections (q|k|v, o, down)
    SHARED_RIDES_ROWS = 16  # a shared expert's two products ride in the routed experts' launches as one more group

    SLICE_TICKETS = 1 << 14
    CUT_SLOTS = 2  # a grouped launch has its row tiles cut along K only with so many group slots at most
    SLICE_ROWS = 16  # up to so many rows the row tiles of a launch may be cut along K (see _k_slices)
    SLOT_ROWS = 16  # a grouped product of so few rows is launched over as many group slots as it has rows

    def _k_slices(self, tiles: int) -> tuple:
        """How a launch of ``tiles`` row tiles (a block each) is evened out over the compute units: ``(m, s)``
        = the first ``m`` tiles cut into ``s`` slices along K, so that the blocks are a multiple of the compute
        units; ``(0, 0)``: leave it (already even, or so many blocks that a part of a round does not matter)."""
        cus = self._compute_units
        m = tiles % cus
        # (measured on 256 compute units: 320 tiles gain a tenth to a fifth, 448 tiles lose as much: three
        # quarters of them would be cut)
        if m == 0 or tiles > 0.8 * (-(-tiles // cus) * cus):
            return 0, 0
        for s in (2, 4, 8):
            if (m * s) % cus == 0:
                return m, s
        return 0, 0

    def gemm_skinny(self, a, b, *, offsets=None, a_rows=None, scale=None, swiglu=False, out_f32=False, rows=None,
                    variant=0, tiled=False, b_last=None, tiled_last=False, balance=True):
        """bfloat16 weight-streaming product on MFMA for few rows (see ``gemm_skinny.hip``); with ``swiglu`` the
        result is ``silu(gate) * up`` of the two halves of ``b``'s rows.  ``b_last``: one more group behind
        ``b``'s, its matrix a tensor of its own (``offsets`` then has an entry more).  ``balance``: with up to 16
        rows, cut some row tiles along K so that the launch's blocks are a multiple of the compute units, and
        launch a grouped product over as many group slots as it has rows (not over every group)."""
        if b.dim() == 2:
            b = b.unsqueeze(0)
        g, nout, k = b.shape
        if b_last is not None:
            self._chk(b_last, torch.bfloat16, (nout, k), "the last group's matrix")
            if offsets is None or offsets.numel() != g + 2:
                raise KernelError("a last group with a matrix of its own needs offsets for one group more")
            g += 1
        m = rows if rows is not None else (a_rows.numel() if a_rows is not None else a.shape[0])
        self._chk(a, torch.bfloat16, None, "A")
        self._chk(b, torch.bfloat16, None, "B")
        if a.shape[1] != k:
            raise KernelError(f"inner sizes differ: A {tuple(a.shape)}, B {tuple(b.shape)}")
        if k % 8:
            raise KernelError(f"the MFMA product needs an inner size that is a multiple of 8, got {k}")
        out = torch.empty(m, nout // 2 if swiglu else nout, dtype=torch.float32 if out_f32 else torch.bfloat16,
                          device=a.device)
        slots = split_tiles = split = 0
        ws = None
        if balance and m <= self.SLICE_ROWS and variant <= 0:
            if offsets is not None and g > m and g <= 4096 and m <= self.SLOT_ROWS:
                slots = m  # (no more groups have rows than there are rows)
            # (several groups' tiles together fill their rounds well enough: measured at 2 to 8 tokens over 16
            # experts and a shared one, a 5,120 x 8,192 product takes 13 % longer with cut tiles than with whole ones)
            if not swiglu and (offsets is None or 0 < slots <= self.CUT_SLOTS):
                split_tiles, split = self._k_slices(-(-nout // 16))
                units = max(slots, 1) * split_tiles
                if units > self.SLICE_TICKETS or (k + 63) // 64 < split:
                    split_tiles = split = 0
                elif split_tiles:
                    ws = torch.empty(units * split * 256, dtype=torch.float32, device=a.device)
        self._call("jle_gemm_skinny", _p(a), _p(b), _p(out), _p(offsets), _p(a_rows), _p(scale), int(swiglu),
                   int(out_f32), m, nout, k, g, m, variant, int(tiled), _p(b_last), int(tiled_last), slots,
                   split_tiles, split, _p(ws), _p(self._slice_tickets))
        return out

    def gemm_grouped(self, a, b, *, offsets=None, a_rows=None, scale=None, swiglu=False, out_f32=False, rows=None,
                     tiled=False):
        """bfloat16 product on MFMA for many rows, grouped by ``offsets`` (see ``gemm_grouped.hip``)."""
        if b.dim() == 2:
            b = b.unsqueeze(0)
        g, nout, k = b.shape
        m = rows if rows is not None else (a_rows.numel() if a_rows is not None else a.shape[0])
        self._chk(a, torch.bfloat16, None, "A")
        self._chk(b, torch.bfloat16, None, "B")
        if a.shape[1] != k:
            raise KernelError(f"inner sizes differ: A {tuple(a.shape)}, B {tuple(b.shape)}")
        if k % 8:
            raise KernelError(f"the MFMA product needs an inner size that is a multiple of 8, got {k}")
        out = torch.empty(m, nout // 2 if swiglu else nout, dtype=torch.float32 if out_f32 else torch.bfloat16,
                          device=a.device)
        self._call("jle_gemm_grouped", _p(a), _p(b), _p(out), _p(offsets), _p(a_rows), _p(scale), int(swiglu),
                   int(out_f32), m, nout, k, g, int(tiled))
        return out


    def stream_supported(self, nout: int, k: int, swiglu: bool) -> bool:
        return bool(self._query("jle_gemm_stream_supported", nout, k, int(swiglu)))

    def gemm_stream(self, a, b, *, offsets=None, a_rows=None, scale=None, swiglu=False, out_f32=False, rows=None):
        """bfloat16 product on MFMA for about a hundred rows per group, weights in the streaming layout and
        read once per 192 rows of a group (see ``gemm_stream.hip``)."""
        if b.dim() == 2:
            b = b.unsqueeze(0)
        g, nout, k = b.shape
        m = rows if rows is not None else (a_rows.numel() if a_rows is not None else a.shape[0])
        self._chk(a, torch.bfloat16, None, "A")
        self._chk(b, torch.bfloat16, None, "B")
        if a.shape[1] != k:
            raise KernelError(f"inner sizes differ: A {tuple(a.shape)}, B {tuple(b.shape)}")
        if a.numel() >= 2 ** 32:
            raise KernelError("the weight-streaming grouped product addresses its rows with 32 bits")
        if not self.stream_supported(nout, k, swiglu):
            raise KernelError(f"the weight-streaming grouped product needs an inner size that is a multiple of 256 and "
                              f"whole tiles of 16 weight rows (32 with the fused activation), got {nout} x {k}")
        out = torch.empty(m, nout // 2 if swiglu else nout, dtype=torch.float32 if out_f32 else torch.bfloat16,
                          device=a.device)
        self._call("jle_gemm_stream", _p(a), _p(b), _p(out), _p(offsets), _p(a_rows), _p(scale), int(swiglu),
                   int(out_f32), m, nout, k, g, m)
        return out

    def lm_head(self, h, w, tiled: bool = False):
        """float32 logits; ``tiled``: ``w`` is in the streaming layout (``ops/layout.py``)."""
        if h.dtype == torch.float32:
            return torch.matmul(h, w.t())
        if h.shape[1] % 8 == 0:
            streams = tiled and self.stream_supported(w.shape[0], w.shape[1], False)
            # measured on a 202048 x 5120 head: up to 16 rows the skinny kernel is at the speed of reading the
            # weights; beyond, the kernel that shares the rows between wavefronts through shared memory
            if h.shape[0] <= (16 if streams else self.SKINNY_MAX_ROWS):
                return self.gemm_skinny(h, w, out_f32=True, tiled=tiled)
            if streams:
                return self.gemm_stream(h, w, out_f32=True)
            return self.gemm_grouped(h, w, out_f32=True, tiled=tiled)
        return self.gemm(h, w, out_f32=True)

    def softcap_(self, logits, cap: float):
        """``cap * tanh(logits / cap)`` in place (float32)."""
        self._chk(logits, torch.float32, None, "logits")
        self._call("jle_softcap", _p(logits), logits.numel(), float(cap))
        return logits

    def silu_mul(self, gate_up, activation: str = "silu"):
        n, f2 = gate_up.shape
        self._chk(gate_up, None, None, "gate|up")
        out = torch.empty(n, f2 // 2, dtype=gate_up.dtype, device=gate_up.device)
        if activation == "silu":
            self._call("jle_silu_mul", _p(gate_up), _p(out), self._is_bf16(gate_up), n, f2 // 2)
        else:
            self._call("jle_act_mul", _p(gate_up), _p(out), self._is_bf16(gate_up), n, f2 // 2, self._ACTS[activation])
        return out

    # ------------------------------------------------------------------ attention
    def qk_prepare_kv_write(self, qkv, num_heads, num_kv_heads, head_dim, positions, prep, kv_cache, slot_mapping):
        """``prep``: a :class:`~..parts.base.QKPreparation`."""
        n = qkv.shape[0]
        hq, hk, dh = num_heads, num_kv_heads, head_dim
        self._chk(qkv, None, (n, (hq + 2 * hk) * dh), "q|k|v")
        self._chk(positions, torch.int32, (n,), "positions")
        rot = prep.rotation
        inv_freq, pairing, rd = None, 0, 0
        if rot is not None:
            inv_freq, rd = rot.inv_freq, int(rot.rotary_dim) or dh
            if rot.pairing not in ("adjacent", "half"):
                raise KernelError(f"rotary/norm kernel: unknown pairing {rot.pairing!r}")
            pairing = 0 if rot.pairing == "adjacent" else 1
            if float(getattr(rot, "magnitude", 1.0)) != 1.0:
                raise KernelError("rotary/norm kernel: sines and cosines with a magnitude go through conv_qk_prepare")
            if rd % 2 or not 0 < rd <= dh:
                raise KernelError(f"rotary/norm kernel: {rd} rotated elements of a head of {dh}")
            self._chk(inv_freq, torch.float32, (rd // 2,), "inv_freq")
        for w, what in ((prep.norm_weight_q, "q norm weight"), (prep.norm_weight_k, "k norm weight")):
            if w is not None:
                if prep.norm_eps is None:
                    raise KernelError("rotary/norm kernel: norm weights without a norm")
                self._chk(w, torch.float32, (dh,), what)
        ps = 0
        if kv_cache is not None:
            ps = kv_cache.shape[3]
            self._chk(kv_cache, qkv.dtype, (kv_cache.shape[0], 2, hk, ps, dh), "kv pages")
            self._chk(slot_mapping, torch.int32, (n,), "slot mapping")
        if dh % 2 or dh > 512:
            raise KernelError(f"rotary/norm kernel: head size {dh} must be even and at most 512")
        q = torch.empty(n, hq, dh, dtype=qkv.dtype, device=qkv.device)
        fs, sc = (prep.query_scale if prep.query_scale is not None else (0.0, 0.0))
        self._call("jle_qk_prepare", _p(qkv), _p(q), _p(kv_cache), _p(positions),
                   _p(slot_mapping) if kv_cache is not None else None, _p(inv_freq),
                   -1.0 if prep.norm_eps is None else float(prep.norm_eps), float(fs), float(sc), self._is_bf16(qkv),
                   n, hq, hk, dh, max(ps, 1), 0 if kv_cache is None else 1, pairing, rd, _p(prep.norm_weight_q),
                   _p(prep.norm_weight_k), int(bool(prep.norm_first)))
        return q

    def qkv_span_prepare(self, rows, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, page_dim: int,
                         own_kv: bool, prep, positions, kv_cache, slot_mapping):
        """One RMS norm over all of a token's queries and one over all its keys (weights of those sizes), the queries
        times ``prep.query_scale``'s factor, keys and values into their pages with heads of ``page_dim`` elements
        (zeros behind the real ones).  Returns q ``[N, Hq, page_dim]``."""
        n = rows.shape[0]
        hq, hk, dk, dv, pd = num_heads, num_kv_heads, head_dim, value_dim, page_dim
        width = hq * dk + ((hk * dk + hk * dv) if own_kv else 0)
        self._chk(rows, None, (n, width), "projected rows")
        self._chk(positions, torch.int32, (n,), "positions")
        self._chk(prep.norm_weight_q, torch.float32, (hq * dk,), "q norm weight")
        if prep.norm_eps is None:
            raise KernelError("the norm over the projection needs its eps")
        ps = 1
        if kv_cache is not None:
            if not own_kv:
                raise KernelError("rows without keys and values cannot fill pages")
            ps = kv_cache.shape[3]
            self._chk(kv_cache, rows.dtype, (kv_cache.shape[0], 2, hk, ps, pd), "kv pages")
            self._chk(slot_mapping, torch.int32, (n,), "slot mapping")
            self._chk(prep.norm_weight_k, torch.float32, (hk * dk,), "k norm weight")
        q = torch.empty(n, hq, pd, dtype=rows.dtype, device=rows.device)
        fs, sc = (prep.query_scale if prep.query_scale is not None else (0.0, 0.0))
        self._call("jle_span_prepare", _p(rows), _p(q), _p(kv_cache), _p(positions),
                   _p(slot_mapping) if kv_cache is not None else None, _p(prep.norm_weight_q),
                   _p(prep.norm_weight_k) if kv_cache is not None else None, float(prep.norm_eps), float(fs), float(sc),
                   self._is_bf16(rows), n, hq, hk, dk, dv, pd, ps, int(bool(own_kv)))
        return q

    TICKETS = 1 << 16

    def attention_from_qkv(self, qkv, num_heads, num_kv_heads, head_dim, positions, token_segment, prep, kv_cache,
                           writes: bool, slot_mapping, block_table, retention, scale: float, meta=None):
        """From the fused q|k|v rows to the attention output ``[N, num_heads * head_dim]``: q and k prepared as
        ``prep`` says, k and v written into their pages (if this run ``writes`` its cache), attention over the
        pages.  A step of single tokens in bfloat16 is one launch (``attention_decode_fused_kernel``)."""
        n = qkv.shape[0]
        hq, hk, dh = num_heads, num_kv_heads, head_dim
        ps = kv_cache.shape[3]
        group = hq // max(hk, 1)
        whole_head = prep.rotation is None or (int(prep.rotation.rotary_dim) or dh) == dh
        if (meta is not None and meta.decode_bucket is not None and qkv.dtype == torch.bfloat16 and prep.plain
                and whole_head and group <= 32 and n * hk < self.TICKETS and 4 * (dh + 4 * group * (dh + 2)) <= 48 * 1024
                and self._query("jle_attention_mfma_supported", dh, hq, hk, ps)):
            self._chk(qkv, kv_cache.dtype, (n, (hq + 2 * hk) * dh), "q|k|v")
            self._chk(kv_cache, None, (kv_cache.shape[0], 2, hk, ps, dh), "kv pages")
            self._chk(block_table, torch.int32, None, "block table")
            self._chk(positions, torch.int32, (n,), "positions")
            self._chk(token_segment, torch.int32, (n,), "token segments")
            if writes:
                self._chk(slot_mapping, torch.int32, (n,), "slot mapping")
            inv_freq = None if prep.rotation is None else prep.rotation.inv_freq
            if inv_freq is not None:
                self._chk(inv_freq, torch.float32, (dh // 2,), "inv_freq")
            key = f"attn_plan_{hq // hk}"
            plan = meta.meta.get(key)
            if plan is None:
                plan = self.attention_plan(meta.seg_lens, meta.seg_starts, retention, qkv.device, hk, hq // hk,
                                           decode_bucket=meta.decode_bucket)
                meta.meta[key] = plan
            splits = -(-plan["max_splits"] // 4) * 4  # a block takes four ranges
            units = n * hk * (splits // 4) * group
            ws_ml = torch.empty(units * 2, dtype=torch.float32, device=qkv.device)
            ws_o = torch.empty(units * dh, dtype=torch.float32, device=qkv.device)
            out = torch.empty(n, hq * dh, dtype=qkv.dtype, device=qkv.device)
            fs, sc = (prep.query_scale if prep.query_scale is not None else (0.0, 0.0))
            mode = _ret_mode(retention)
            param = int(retention[1]) if len(retention) > 1 else 0
            self._call("jle_attention_decode_fused", _p(qkv), _p(kv_cache), _p(out), _p(ws_ml), _p(ws_o),
                       _p(self._tickets), _p(positions), _p(token_segment), _p(block_table), block_table.shape[1],
                       _p(plan["dec"]), n, splits, plan["split"], mode, param, float(scale), hq, hk, dh,
                       ps, _p(inv_freq), -1.0 if prep.norm_eps is None else float(prep.norm_eps), float(fs),
                       float(sc), _p(slot_mapping) if writes else None, int(bool(writes)))
            return out
        q = self.qk_prepare_kv_write(qkv, hq, hk, dh, positions, prep, kv_cache if writes else None, slot_mapping)
        return self.paged_attention(q, kv_cache, block_table, positions, token_segment, retention, scale, meta)

    PREFILL_TILE = 32  # tokens per prefill work item (the kernels take 16 or 32)
    BIASED_TILE = 16  # the same for the kernel with a distance bias and sinks
    GENERIC_SPLIT_BELOW = 2048  # the float32-arithmetic attention: fewer (token, head) pairs than this share their keys
    DECODE_MIN_SPLIT = 128  # decode attention: keys per work item (wavefront) at least ...
    DECODE_FIT_SPLIT = 1024  # ... and at most
    DECODE_MAX_SPLIT = 512  # (a step without single tokens: no matter)
    # measured on MI355X at head size 128 (bfloat16): a block of four wavefronts reads a key position (keys and values
    # of one kv head) of each in 0.073 us when every compute unit reads; results handed between blocks cost 5.5 us
    # and 0.09 us per block of the (token, kv head)
    DECODE_KEY_US, DECODE_MERGE_US, DECODE_RESULT_US = 0.073, 5.5, 0.09

    @staticmethod
    def _most_ranges(retention, bound: int, split: int) -> int:
        """The most key ranges of ``split`` positions that a query at a position below ``bound`` reads."""
        kind = retention[0]
        whole = (bound - 1) // split + 1
        if kind == "chunk":
            c = int(retention[1])
            most = 0
            for first in range(0, bound, c):
                last = min(first + c, bound) - 1
                most = max(most, last // split - first // split + 1)
            return most
        if kind == "window":
            return min(whole, (int(retention[1]) - 1) // split + 2)
        return whole

    def attention_plan(self, seg_lens, seg_starts, retention, device, num_kv_heads=1, group_size=1, decode_bucket=None,
                       tile=None):
        """Work lists of the MFMA attention kernels for one step and one retention rule: the rows that are
        single decode tokens (and into how many keys their work is split), tiles of up to 32 consecutive
        tokens of longer segments and, with ``group_size`` > 1 query heads per kv head, the packing of the
        (tile, head) items of a kv head into blocks of wavefronts that share keys.  ``decode_bucket``: the step
        holds single tokens only, none beyond this context length: the split is then chosen from the number of
        tokens and this bound alone (not from where each request stands), so the same launch fits every such
        step."""
        from ..parts.base import first_needed_position

        dec, tiles, spans, seg_tiles = [], [], [], []
        tile = tile or self.PREFILL_TILE
        o = 0
        for i, n in enumerate(seg_lens):
            if n == 1:
                dec.append(o)
                if decode_bucket is None:
                    spans.append((first_needed_position(retention, seg_starts[i]), seg_starts[i]))
            else:
                first = len(tiles) // 2
                for t in range(0, n, tile):
                    tiles += [o + t, min(tile, n - t)]
                seg_tiles.append((first, len(tiles) // 2 - first, seg_starts[i] + n - 1))
            o += n
        split, max_splits = self.DECODE_MAX_SPLIT, 1
        if dec:
            # Which range (a multiple of 32 keys): the one with which the busiest compute unit has the fewest keys
            # to read.  A block is four ranges of one (token, kv head); a compute unit reads about as fast with
            # two blocks as with one, so what counts is how many blocks it gets (the blocks over the compute
            # units, rounded up) times the block's keys; blocks that hand results to each other pay for the merge.
            if decode_bucket is not None:
                ranges_of = lambda cand: [self._most_ranges(retention, decode_bucket, cand)] * len(dec)
            else:
                ranges_of = lambda cand: [p // cand - f // cand + 1 for f, p in spans]
            best = None
            for cand in range(self.DECODE_MIN_SPLIT, self.DECODE_FIT_SPLIT + 1, 32):
                per_unit = [-(-r // 4) for r in ranges_of(cand)]  # blocks per (token, kv head)
                blocks = num_kv_heads * sum(per_unit)
                cost = (-(-blocks // self._compute_units) * cand * self.DECODE_KEY_US
                        + (self.DECODE_MERGE_US + self.DECODE_RESULT_US * max(per_unit) if max(per_unit) > 1 else 0.0))
                if best is None or cost <= best[0]:  # (equal: the longer range, fewer blocks)
                    best = (cost, cand)
            split = best[1]
            max_splits = max(ranges_of(split))
        groups = []
        if tiles and group_size > 1 and tile == 32:
            # consecutive (tile, head) items of one segment, `waves` per block; blocks with the most keys first
            waves = int(self._query("jle_attention_group_waves"))
            keyed = []
            for first, count, last_pos in seg_tiles:
                items = count * group_size
                for lo in range(0, items, waves):
                    n_items = min(waves, items - lo)
                    last_tile = first + (lo + n_items - 1) // group_size
                    end = last_pos - (first + count - 1 - last_tile) * tile  # about where its keys end
                    keyed.append((-end, len(keyed), [first + lo // group_size, lo % group_size, n_items, 0]))
            keyed.sort()
            groups = [v for _, _, quad in keyed for v in quad]
        flat = dec + tiles + groups
        flat = torch.tensor(flat, dtype=torch.int32).to(device) if flat else None
        nd, nt = len(dec), len(tiles)
        return {"num_dec": nd, "num_tiles": nt // 2, "max_splits": max_splits, "split": split,
                "dec": flat[:nd] if dec else None, "tiles": flat[nd: nd + nt] if tiles else None,
                "groups": flat[nd + nt:] if groups else None, "num_groups": len(groups) // 4}

    @staticmethod
    def _segments(meta, token_segment, positions):
        """The step's segments (lengths, first positions): from the step's context or, in a direct call (tests),
        recovered from the device arrays."""
        if meta is not None and meta.seg_starts is not None:
            return meta.seg_lens, meta.seg_starts
        seg = token_segment.cpu().tolist()
        pos = positions.cpu().tolist()
        seg_lens, seg_starts = [], []
        for i, sgm in enumerate(seg):
            if i == 0 or sgm != seg[i - 1]:
                seg_lens.append(0)
                seg_starts.append(pos[i])
            seg_lens[-1] += 1
        return seg_lens, seg_starts

    F32_TILE = 16  # tokens per work item of the float32 matrix-instruction attention
    F32_DECODE_ITEMS = 2048  # ... in a step of single tokens: about so many (token, kv head, key range) items

    def paged_attention(self, q, kv_cache, block_table, positions, token_segment, retention, scale: float, meta=None,
                        bias=None, sink=None):
        """``bias``: float32 ``[Hq, L]``: a key ``n`` places back adds ``bias[h, min(n, L - 1)]`` to head ``h``'s scaled
        score; ``sink``: float32 ``[Hq]``: ``exp(sink[h])`` is one more term of head ``h``'s denominator."""
        n, hq, dh = q.shape
        hk, ps = kv_cache.shape[2], kv_cache.shape[3]
        self._chk(q, kv_cache.dtype, None, "q")
        self._chk(kv_cache, None, (kv_cache.shape[0], 2, hk, ps, dh), "kv pages")
        self._chk(block_table, torch.int32, None, "block table")
        self._chk(positions, torch.int32, (n,), "positions")
        self._chk(token_segment, torch.int32, (n,), "token segments")
        mode = _ret_mode(retention)
        param = int(retention[1]) if len(retention) > 1 else 0
        out = torch.empty(n, hq * dh, dtype=q.dtype, device=q.device)
        biased = bias is not None or sink is not None
        if retention[0] == "window_keep":
            return self._attention_kept(q, kv_cache, out, block_table, positions, token_segment, mode, param,
                                        int(retention[2]), scale, meta, biased)
        if bias is not None:
            self._chk(bias, torch.float32, (hq, bias.shape[1]), "distance bias")
        if sink is not None:
            self._chk(sink, torch.float32, (hq,), "sinks")
        if (q.dtype == torch.bfloat16 and hq // hk <= 32
                and self._query("jle_attention_mfma_supported", dh, hq, hk, ps)):
            # (with a bias or sinks the kernel for heads of 128 alone shares keys between wavefronts; at other sizes
            # every (tile, head) is a wavefront of its own, in tiles of 16 tokens)
            grouped = hq // hk if (not biased or dh == 128) else 1
            if biased and bias is None:
                bias = self._zero_bias.get((hq, q.device))
                if bias is None:
                    bias = self._zero_bias[(hq, q.device)] = torch.zeros(hq, 1, dtype=torch.float32, device=q.device)
            bias_len = bias.shape[1] if biased else 0
            tile = self.BIASED_TILE if biased and grouped == 1 else self.PREFILL_TILE
            key = f"attn_plan_{grouped}_{tile}"
            plan = meta.meta.get(key) if meta is not None else None
            if plan is None:
                seg_lens, seg_starts = self._segments(meta, token_segment, positions)
                plan = self.attention_plan(seg_lens, seg_starts, retention, q.device, hk, grouped,
                                           decode_bucket=meta.decode_bucket if meta is not None else None, tile=tile)
                if meta is not None:
                    meta.meta[key] = plan
            if plan["num_tiles"]:
                self._call("jle_attention_prefill", _p(q), _p(kv_cache), _p(out), _p(positions), _p(token_segment),
                           _p(block_table), block_table.shape[1], _p(plan["tiles"]), plan["num_tiles"],
                           tile, _p(plan["groups"]), plan["num_groups"], mode, param, float(scale), hq,
                           hk, dh, ps, _p(bias), bias_len, _p(sink))
            if plan["num_dec"]:
                cols = 16 if hq // hk <= 16 else 32
                items = plan["num_dec"] * hk * plan["max_splits"]
                ws_ml = torch.empty(items * cols * 2, dtype=torch.float32, device=q.device)
                ws_o = torch.empty(items * cols * dh, dtype=torch.float32, device=q.device)
                self._call("jle_attention_decode", _p(q), _p(kv_cache), _p(out), _p(ws_ml), _p(ws_o), _p(positions),
                           _p(token_segment), _p(block_table), block_table.shape[1], _p(plan["dec"]), plan["num_dec"],
                           plan["max_splits"], plan["split"], mode, param, float(scale), hq, hk, dh, ps, _p(bias),
                           bias_len, _p(sink))
            return out
        if dh % 8 or dh > 256:
            raise KernelError(f"attention kernels: head size {dh} is not supported (a multiple of 8, at most 256)")
        if hq % hk:
            raise KernelError(f"attention kernels: {hq} query heads are no multiple of {hk} kv heads")
        if (not biased and q.dtype == torch.float32 and dh % 16 == 0 and ps % 16 == 0
                and n * hq >= self.GENERIC_SPLIT_BELOW and (meta is None or meta.decode_bucket is None)):
            # many tokens in float32: tiles of 16 tokens on the float32 matrix instructions
            tiles = meta.meta.get("f32_tiles") if meta is not None else None
            if tiles is None:
                seg_lens, _ = self._segments(meta, token_segment, positions)
                flat, o = [], 0
                for ln in seg_lens:
                    for t in range(0, ln, self.F32_TILE):
                        flat += [o + t, min(self.F32_TILE, ln - t)]
                    o += ln
                tiles = torch.tensor(flat, dtype=torch.int32).to(q.device)
                if meta is not None:
                    meta.meta["f32_tiles"] = tiles
            self._call("jle_attention_f32_tiles", _p(q), _p(kv_cache), _p(out), _p(positions), _p(token_segment),
                       _p(block_table), block_table.shape[1], _p(tiles), tiles.numel() // 2, mode, param, float(scale),
                       hq, hk, dh, ps)
            return out
        if (not biased and q.dtype == torch.float32 and dh % 16 == 0 and ps % 16 == 0 and hq // hk <= 16
                and ((meta is not None and meta.decode_bucket is not None)
                     or all(ln == 1 for ln in self._segments(meta, token_segment, positions)[0]))):
            # a step of single tokens in float32: the query heads of a kv head share a wavefront (its keys and
            # values are read once for all of them), the keys are shared between wavefronts and merged
            if meta is not None and meta.decode_bucket is not None:
                longest = meta.decode_bucket
            else:
                longest = int(positions.max()) + 1
            steps = -(-longest // 64)
            want = max(1, min(steps, -(-self.F32_DECODE_ITEMS // (n * hk))))
            per = -(-steps // want) * 64
            splits = -(-longest // per)
            ws_ml = ws_o = None
            if splits > 1:
                ws_ml = torch.empty(n * hq * splits * 2, dtype=torch.float32, device=q.device)
                ws_o = torch.empty(n * hq * splits * dh, dtype=torch.float32, device=q.device)
            self._call("jle_attention_f32_heads", _p(q), _p(kv_cache), _p(out), _p(positions), _p(token_segment),
                       _p(block_table), block_table.shape[1], n, mode, param, float(scale), hq, hk, dh, ps, splits,
                       per, _p(ws_ml), _p(ws_o))
            if splits > 1:
                self._call("jle_attention_merge", _p(ws_ml), _p(ws_o), _p(out), 0, n * hq, dh, splits)
            return out
        # few tokens with many keys (decode): each query's keys are shared between several wavefronts
        splits, tiles_per_split, ws_ml, ws_o = 1, 0, None, None
        waves = n * hq
        if waves < self.GENERIC_SPLIT_BELOW:
            if meta is not None and meta.decode_bucket is not None:
                longest = meta.decode_bucket  # (a step of single tokens: laid out for the bound, see GroupContext)
            elif meta is not None:
                longest = max(s0 + ln for s0, ln in zip(meta.seg_starts, meta.seg_lens))
            else:
                longest = int(positions.max()) + 1
            tiles = -(-longest // 64)
            want = min(tiles, -(-self.GENERIC_SPLIT_BELOW // waves))
            if want > 1:
                tiles_per_split = -(-tiles // want)
                splits = -(-tiles // tiles_per_split)
                ws_ml = torch.empty(waves * splits * 2, dtype=torch.float32, device=q.device)
                ws_o = torch.empty(waves * splits * dh, dtype=torch.float32, device=q.device)
        if biased:
            self._call("jle_paged_attention_biased", _p(q), _p(kv_cache), _p(out), _p(positions), _p(token_segment),
                       _p(block_table), block_table.shape[1], mode, param, float(scale), self._is_bf16(q), n, hq, hk,
                       dh, ps, splits, tiles_per_split, _p(ws_ml), _p(ws_o), _p(bias),
                       0 if bias is None else bias.shape[1], _p(sink))
            return out
        self._call("jle_paged_attention_generic", _p(q), _p(kv_cache), _p(out), _p(positions), _p(token_segment),
                   _p(block_table), block_table.shape[1], mode, param, float(scale), self._is_bf16(q), n, hq, hk, dh,
                   ps, splits, tiles_per_split, _p(ws_ml), _p(ws_o))
        return out

    def _attention_kept(self, q, kv_cache, out, block_table, positions, token_segment, mode: int, param: int,
                        keep: int, scale: float, meta, biased: bool):
        """A window whose queries also see the sequence's first ``keep`` keys: the general kernel (float32
        arithmetic, both dtypes) takes the kept keys that lie before the window as a range of their own."""
        n, hq, dh = q.shape
        hk, ps = kv_cache.shape[2], kv_cache.shape[3]
        if biased:
            raise KernelError("the attention kernel for kept first tokens takes no distance table and no sinks")
        if dh % 8 or dh > 256 or hq % hk:
            raise KernelError(f"attention kernels: head size {dh} (a multiple of 8, at most 256) or {hq} query heads "
                              f"on {hk} kv heads are not supported")
        single = meta is not None and meta.decode_bucket is not None
        if (not single and q.dtype == torch.bfloat16 and hq // hk <= 32
                and self._query("jle_attention_mfma_supported", dh, hq, hk, ps)):
            # portions of prompts in bfloat16: the matrix-core kernel, a wavefront per (tile of 32 tokens, head),
            # which takes the kept keys before a tile's window as a range of its own; a step of single tokens
            # goes on below (a query's keys shared between wavefronts)
            seg_lens, _ = self._segments(meta, token_segment, positions)
            if any(ln > 1 for ln in seg_lens):
                tiles = meta.meta.get("kept_tiles") if meta is not None else None
                if tiles is None:
                    flat, o = [], 0
                    for ln in seg_lens:
                        for t in range(0, ln, self.PREFILL_TILE):
                            flat += [o + t, min(self.PREFILL_TILE, ln - t)]
                        o += ln
                    tiles = torch.tensor(flat, dtype=torch.int32).to(q.device)
                    if meta is not None:
                        meta.meta["kept_tiles"] = tiles
                self._call("jle_attention_prefill_kept", _p(q), _p(kv_cache), _p(out), _p(positions),
                           _p(token_segment), _p(block_table), block_table.shape[1], _p(tiles), tiles.numel() // 2,
                           self.PREFILL_TILE, param, keep, float(scale), hq, hk, dh, ps)
                return out
        splits, tiles_per_split, ws_ml, ws_o = 1, 0, None, None
        waves = n * hq
        if waves < self.GENERIC_SPLIT_BELOW:  # few tokens with many keys: a query's keys shared between wavefronts
            if meta is not None and meta.decode_bucket is not None:
                longest = meta.decode_bucket
            elif meta is not None:
                longest = max(s0 + ln for s0, ln in zip(meta.seg_starts, meta.seg_lens))
            else:
                longest = int(positions.max()) + 1
            tiles = -(-min(longest, param + 64) // 64)  # (the window's keys; the kept ones ride with the first range)
            want = min(tiles, -(-self.GENERIC_SPLIT_BELOW // waves))
            if want > 1:
                tiles_per_split = -(-tiles // want)
                splits = -(-tiles // tiles_per_split)
                ws_ml = torch.empty(waves * splits * 2, dtype=torch.float32, device=q.device)
                ws_o = torch.empty(waves * splits * dh, dtype=torch.float32, device=q.device)
        self._call("jle_paged_attention_kept", _p(q), _p(kv_cache), _p(out), _p(positions), _p(token_segment),
                   _p(block_table), block_table.shape[1], mode, param, keep, float(scale), self._is_bf16(q), n, hq, hk,
                   dh, ps, splits, tiles_per_split, _p(ws_ml), _p(ws_o))
        return out

    # ------------------------------------------------------------------ routed experts
    def moe_choose(self, h32, router, correction, top_k: int, groups=None, keep_groups=None, group_terms: int = 2):
        """Router logits in float32 (the router kernel), then the choice by scores with a correction and groups
        (``moe_choose.hip``) and the grouping of the choices by expert.  Returns ``(ids, weights, grouping)``."""
        h32 = self._rows(h32, want32=True)
        n, d = h32.shape
        e = router.shape[0]
        self._chk(h32, torch.float32, None, "router input")
        self._chk(router, torch.float32, (e, d), "router matrix")
        if correction is not None:
            self._chk(correction, torch.float32, (e,), "correction")
        dev = h32.device
        logits = torch.empty(n, e, dtype=torch.float32, device=dev)
        self._call("jle_moe_logits", _p(h32), _p(router), _p(logits), n, d, e)
        ids = torch.empty(n, top_k, dtype=torch.int32, device=dev)
        weights = torch.empty(n, top_k, dtype=torch.float32, device=dev)
        self._call("jle_moe_choose", _p(logits), _p(correction), _p(ids), _p(weights), n, e, top_k,
                   0 if groups is None else int(groups), 0 if groups is None else int(keep_groups), int(group_terms))
        return ids, weights, self.moe_align(ids, weights, e)

    def relu2(self, x):
        """``relu(x)^2`` element by element."""
        self._chk(x, None, None, "rows")
        y = torch.empty_like(x)
        self._call("jle_relu2", _p(x), _p(y), self._is_bf16(x), x.numel())
        return y

    def moe_experts_scored(self, h, expert_ids, weights, w_up, w_down, activation: str = "relu2", tiled: bool = False,
                           grouping=None):
        """``sum_j weights[j] * W_down[e_j] relu(W_up[e_j] h)^2``: the choices grouped by expert, the first product
        plain, the activation a kernel of its own, the weights the second product's row scale (applied to its float32
        sums); the sum over a token's choices stays in pieces (:class:`ExpertSum`)."""
        if activation != "relu2":
            raise KernelError(f"unknown activation {activation!r}")
        h = self._rows(h)
        n, d = h.shape
        e, f, _ = w_up.shape
        k = expert_ids.shape[1]
        m = n * k
        if grouping is None:
            grouping = self.moe_align(expert_ids.contiguous(), weights.contiguous(), e)
        offsets, sorted_token, sorted_weight, inv = grouping
        mfma = h.dtype == torch.bfloat16 and d % 8 == 0 and f % 8 == 0

        def product(x, w, nout, kdim, **kw):
            if mfma and m <= 2 * self.SKINNY_MAX_ROWS:
                return self.gemm_skinny(x, w, offsets=offsets, tiled=tiled, **kw)
            if mfma and tiled and self.stream_supported(nout, kdim, False):
                return self.gemm_stream(x, w, offsets=offsets, **kw)
            if mfma:
                return self.gemm_grouped(x, w, offsets=offsets, tiled=tiled, **kw)
            if tiled:
                raise KernelError("weights in the streaming layout need the MFMA product kernels")
            if (x.dtype == torch.float32 and kdim % 4 == 0 and nout % 4 == 0 and m <= self.F32_SKINNY_ROWS):
                return self.gemm_f32_skinny(x, w, offsets=offsets, **kw)
            if (x.dtype == torch.float32 and self.f32_stream_supported(nout, kdim, False) and x.numel() < 2 ** 32
                    and m * nout < 2 ** 32 and not (x.data_ptr() | w.data_ptr()) % 16):
                return self.gemm_f32_stream(x, w, offsets=offsets, **kw)
            return self.gemm(x, w, offsets=offsets, **kw)

        up = product(h, w_up, f, d, a_rows=sorted_token)
        routed = product(self.relu2(up), w_down, d, f, scale=sorted_weight)
        return ExpertSum(routed, inv, k, None, n, d)

    def moe_route(self, h32, router, top_k: int, want_logits: bool = False, group: bool = False):
        """``group``: also return the grouping of the choices by expert (what ``moe_align`` gives), made in
        the same call; ``moe_experts`` takes it as ``grouping``."""
        n, d = h32.shape
        e = router.shape[0]
        if isinstance(h32, PendingNorm):
            fused = None if h32.done or not group else self._norm_route(h32, router, top_k)
            if fused is not None:
                ids, gates, logits, grouping = fused
                return (ids, gates, logits, grouping) if want_logits else (ids, gates, grouping)
            h32 = h32.rows(want32=True)
        self._chk(h32, torch.float32, None, "router input")
        self._chk(router, torch.float32, (e, d), "router matrix")
        if not 1 <= top_k <= min(8, e) or e > 4096:
            raise KernelError(f"router kernel: top_k {top_k} of {e} experts is not supported (top_k <= 8, experts <= 4096)")
        dev = h32.device
        ids = torch.empty(n, top_k, dtype=torch.int32, device=dev)
        gates = torch.empty(n, top_k, dtype=torch.float32, device=dev)
        logits = torch.empty(n, e, dtype=torch.float32, device=dev)
        if group:
            # (with one more group behind the experts' that holds every token once: a shared expert's rows)
            m = n * top_k
            offsets = torch.empty(e + 2, dtype=torch.int32, device=dev)
            sorted_token = torch.empty(m + n, dtype=torch.int32, device=dev)
            sorted_gate = torch.empty(m + n, dtype=torch.float32, device=dev)
            inv = torch.empty(m, dtype=torch.int32, device=dev)
            self._call("jle_moe_route_align", _p(h32), _p(router), _p(ids), _p(gates), _p(logits), _p(offsets),
                       _p(sorted_token), _p(sorted_gate), _p(inv), n, d, e, top_k, 1)
            grouping = (offsets, sorted_token, sorted_gate, inv)
            return (ids, gates, logits, grouping) if want_logits else (ids, gates, grouping)
        self._call("jle_moe_route", _p(h32), _p(router), _p(ids), _p(gates), _p(logits), n, d, e, top_k)
        return (ids, gates, logits) if want_logits else (ids, gates)

    NORM_ROUTE_ROWS = 256

    def _norm_route(self, pending: PendingNorm, router, top_k: int):
        """The pending addition and norm, the router's logits, the choice and the grouping (with the extra group
        of a shared expert's rows) in one launch, for a step of few tokens; ``None`` if the sizes do not fit."""
        x, delta = pending.x, pending.delta
        n, d = x.shape
        e = router.shape[0]
        words = 2 * e + 1 + 2 * n * top_k
        if (n > self.NORM_ROUTE_ROWS or d % 8 or not 1024 < d <= 8192 or not 1 <= top_k <= min(8, e) or e > 4096
                or 4 * max(words, d) > 48 * 1024 or x.dtype != torch.float32 or router.dtype != torch.float32):
            return None
        kind, plain, routed, inv_in, k_in, shared, is_bf16 = 0, None, None, None, 0, None, 0
        if isinstance(delta, ExpertSum):
            kind, routed, inv_in, k_in, shared = 2, delta.routed, delta.inv, delta.k, delta.shared
            is_bf16 = self._is_bf16(routed)
        elif delta is not None:
            self._chk(delta, None, (n, d), "branch output")
            kind, plain, is_bf16 = 1, delta, self._is_bf16(delta)
        tensors = [t for t in (x, plain, routed, shared, pending.weight, router) if t is not None]
        if any(t.data_ptr() % 16 or not t.is_contiguous() for t in tensors):
            return None
        self._chk(router, torch.float32, (e, d), "router matrix")
        if pending.weight is not None:
            self._chk(pending.weight, torch.float32, (d,), "norm weight")
        dev = x.device
        x_out = torch.empty_like(x)
        h = torch.empty(n, d, dtype=pending.dtype, device=dev)
        m = n * top_k
        ids = torch.empty(n, top_k, dtype=torch.int32, device=dev)
        gates = torch.empty(n, top_k, dtype=torch.float32, device=dev)
        logits = torch.empty(n, e, dtype=torch.float32, device=dev)
        offsets = torch.empty(e + 2, dtype=torch.int32, device=dev)
        sorted_token = torch.empty(m + n, dtype=torch.int32, device=dev)
        sorted_gate = torch.empty(m + n, dtype=torch.float32, device=dev)
        inv = torch.empty(m, dtype=torch.int32, device=dev)
        self._call("jle_norm_route", _p(x), kind, _p(plain), _p(routed), _p(inv_in), k_in, _p(shared), is_bf16,
                   _p(pending.weight), pending.eps, _p(x_out), _p(h), self._is_bf16(h), _p(router), _p(logits),
                   _p(ids), _p(gates), _p(offsets), _p(sorted_token), _p(sorted_gate), _p(inv),
                   self._tickets[-1:].data_ptr(), n, d, e, top_k, 1)
        pending.x_out, pending.h = x_out, h
        return ids, gates, logits, (offsets, sorted_token, sorted_gate, inv)

    def moe_align(self, expert_ids, gates, num_experts: int, extra_group: bool = False):
        """Stable grouping of the (token, choice) pairs by expert: offsets ``[E + 1]``, the token and the gate of
        every sorted row, and where each pair went.  ``extra_group``: one more group behind the experts' that
        holds every token once, in order, with gate 1 (the rows of a shared expert)."""
        n, k = expert_ids.shape
        m = n * k
        x = n if extra_group else 0
        dev = expert_ids.device
        self._chk(expert_ids, torch.int32, None, "expert ids")
        self._chk(gates, torch.float32, (n, k), "gates")
        offsets = torch.empty(num_experts + (2 if extra_group else 1), dtype=torch.int32, device=dev)
        sorted_token = torch.empty(m + x, dtype=torch.int32, device=dev)
        sorted_gate = torch.empty(m + x, dtype=torch.float32, device=dev)
        inv = torch.empty(m, dtype=torch.int32, device=dev)
        self._call("jle_moe_align", _p(expert_ids), _p(gates), _p(offsets), _p(sorted_token), _p(sorted_gate), _p(inv),
                   m, num_experts, k, int(extra_group))
        return offsets, sorted_token, sorted_gate, inv

    def row_gate_(self, rows, h32, w):
        """``rows[n] *= sigmoid(h32[n] . w)`` in place: one number a token, formed in float32."""
        n, d = rows.shape
        k = h32.shape[1]
        self._chk(rows, None, (n, d), "rows")
        self._chk(h32, torch.float32, (n, k), "gate input")
        self._chk(w, torch.float32, None, "gate row")
        if w.numel() != k:
            raise KernelError("the gate's row does not fit its input")
        self._call("jle_row_gate", _p(rows), self._is_bf16(rows), _p(h32), _p(w), n, k, d)
        return rows

    def moe_experts(self, h, expert_ids, gates, w_gate_up, w_down, shared=None, tiled: bool = False, grouping=None,
                    shared_weights=None, shared_gate=None):
        """``shared``: a shared expert's output, or ``shared_weights``: its (gate|up, down) matrices, row-major.
        ``shared_gate = (h32, w)``: the shared expert's output times ``sigmoid(h32 . w)``, one number a token."""
        if shared_gate is not None:
            total = self.moe_experts(h, expert_ids, gates, w_gate_up, w_down, shared=shared, tiled=tiled,
                                     grouping=grouping, shared_weights=shared_weights)
            if total.shared is not None:
                self.row_gate_(total.shared, self._rows(shared_gate[0], want32=True), shared_gate[1])
            return total
        h = self._rows(h)
        n, d = h.shape
        e, f2, _ = w_gate_up.shape
        k = expert_ids.shape[1]
        m = n * k
        mfma = h.dtype == torch.bfloat16 and d % 8 == 0 and (f2 // 2) % 8 == 0
        # a step of few tokens streams the shared expert's matrices in the launches of the routed experts', as one
        # more group: the cost of such a step is the kernels' getting started, not their work
        fuse = (shared is None and shared_weights is not None and mfma and n <= self.SHARED_RIDES_ROWS
                and m <= 2 * self.SKINNY_MAX_ROWS and tuple(shared_weights[0].shape) == (f2, d)
                and tuple(shared_weights[1].shape) == (d, f2 // 2))
        if grouping is None or (fuse and grouping[0].numel() != e + 2):
            grouping = self.moe_align(expert_ids.contiguous(), gates.contiguous(), e, extra_group=fuse)
        offsets, sorted_token, sorted_gate, inv = grouping
        if fuse:
            act = self.gemm_skinny(h, w_gate_up, offsets=offsets, a_rows=sorted_token, scale=sorted_gate, swiglu=True,
                                   tiled=tiled, b_last=shared_weights[0], rows=m + n)
            both = self.gemm_skinny(act, w_down, offsets=offsets, tiled=tiled, b_last=shared_weights[1])
            return ExpertSum(both[:m], inv, k, both[m:], n, d)
        if shared is None and shared_weights is not None:
            shared = self.linear(self.swiglu_linear(h, shared_weights[0]), shared_weights[1])
        if grouping[0].numel() != e + 1:  # (made with the extra group: the kernels below do not know of it)
            offsets, sorted_token, sorted_gate = offsets[: e + 1], sorted_token[:m], sorted_gate[:m]
        if mfma and m <= 2 * self.SKINNY_MAX_ROWS:  # few rows: the cost is streaming the chosen experts' weights
            act = self.gemm_skinny(h, w_gate_up, offsets=offsets, a_rows=sorted_token, scale=sorted_gate, swiglu=True,
                                   tiled=tiled)
            routed = self.gemm_skinny(act, w_down, offsets=offsets, tiled=tiled)
        elif mfma and tiled and self.stream_supported(f2, d, True) and self.stream_supported(d, f2 // 2, False):
            # around a hundred rows per expert the cost is reading the weights, which this kernel reads once per
            # 192 rows of an expert; with more rows it is still the faster one (measured up to 1024 per expert)
            act = self.gemm_stream(h, w_gate_up, offsets=offsets, a_rows=sorted_token, scale=sorted_gate, swiglu=True)
            routed = self.gemm_stream(act, w_down, offsets=offsets)
        elif mfma:
            act = self.gemm_grouped(h, w_gate_up, offsets=offsets, a_rows=sorted_token, scale=sorted_gate, swiglu=True,
                                    tiled=tiled)
            routed = self.gemm_grouped(act, w_down, offsets=offsets, tiled=tiled)
        elif tiled:
            raise KernelError("weights in the streaming layout need the MFMA product kernels")
        elif h.dtype == torch.float32 and d % 4 == 0 and (f2 // 2) % 4 == 0 and m <= self.F32_SKINNY_ROWS:
            # few rows in true float32: the weights streamed once through the float32 matrix instructions, the
            # activation fused into the first product
            act = self.gemm_f32_skinny(h, w_gate_up, offsets=offsets, a_rows=sorted_token, scale=sorted_gate,
                                       swiglu=True)
            routed = self.gemm_f32_skinny(act, w_down, offsets=offsets)
        elif (h.dtype == torch.float32 and self.f32_stream_supported(f2, d, True)
              and self.f32_stream_supported(d, f2 // 2, False) and h.numel() < 2 ** 32 and m * (f2 // 2) < 2 ** 32
              and not (h.data_ptr() | w_gate_up.data_ptr() | w_down.data_ptr()) % 16):
            # more rows in true float32 (a prefill): the same instructions, a wavefront holding up to 192 rows of
            # its expert, so that the weights are read once per so many rows
            act = self.gemm_f32_stream(h, w_gate_up, offsets=offsets, a_rows=sorted_token, scale=sorted_gate,
                                       swiglu=True)
            routed = self.gemm_f32_stream(act, w_down, offsets=offsets)
        else:
            gu = self.gemm(h, w_gate_up, offsets=offsets, a_rows=sorted_token, scale=sorted_gate)
            act = self.silu_mul(gu)
            routed = self.gemm(act, w_down, offsets=offsets)
        if shared is not None:
            self._chk(shared, h.dtype, (n, d), "shared expert output")
        return ExpertSum(routed, inv, k, shared, n, d)

    # ------------------------------------------------------------------ sampling
    def sample(self, logits, temperature, top_k, seeds, counters, any_top_k: bool = True):
        m, v = logits.shape
        self._chk(logits, torch.float32, None, "logits")
        self._chk(temperature, torch.float32, (m,), "temperature")
        for t, what in ((top_k, "top_k"), (seeds, "seeds"), (counters, "counters")):
            self._chk(t, torch.int32, (m,), what)
        out = torch.empty(m, dtype=torch.int32, device=logits.device)
        chunks = -(-v // 8192)
        part_v = torch.empty(m * chunks, dtype=torch.float32, device=logits.device)
        part_i = torch.empty(m * chunks, dtype=torch.int32, device=logits.device)
        self._call("jle_sample", _p(logits), _p(temperature), _p(top_k), _p(seeds), _p(counters), _p(out), _p(part_v),
                   _p(part_i), m, v, int(any_top_k))
        return out
