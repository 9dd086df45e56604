"""The engine's operations: thin, checked calls into the HIP libraries.

Every function takes torch tensors on the GPU, checks on the host what the
kernel assumes about shapes, strides and dtypes, and launches on torch's current
stream. There is no other implementation behind these names: without a GPU or
without the built library a call raises. (Tests may install another backend with
`set_backend` to exercise the engine's bookkeeping on a machine without a GPU.)

Reference counterparts: layers/ops.py:23-57 (attention/cache bindings and the
v1/v2 decode dispatcher), and the eager torch ops named in each docstring.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

import torch

from . import build

ME_BF16, ME_F32 = 0, 1
ACTIVATIONS = {"silu": 0, "relu2": 1, "tanh": 2, "gelu_tanh": 3}          # elementwise activations of `activation`
GATED_NORMS = {"silu_before": 0, "sigmoid_behind": 1, "silu_behind": 2}
DECAY_RULES = {"bonus": 0, "delta": 1, "gated": 2}         # update rules of `decay_rows_recurrence`
_DT = {torch.bfloat16: ME_BF16, torch.float32: ME_F32}


class KernelError(RuntimeError):
    pass


def _code(dtype: torch.dtype) -> int:
    try:
        return _DT[dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {dtype}; the kernels take bfloat16 and float32") from None


# --------------------------------------------------------------------------- libraries

class _Lib:
    def __init__(self, path: str, protos: dict):
        self.path = path
        self.cdll = ctypes.CDLL(path)
        self.cdll.me_last_error.restype = c_char_p
        self.fns = {}
        for name, argtypes in protos.items():
            fn = getattr(self.cdll, name)
            fn.argtypes = argtypes
            fn.restype = c_int
            self.fns[name] = fn
        self.protos = protos

    def call(self, name: str, *args):
        if self.fns[name](*args) != 0:
            raise KernelError(f"{name}: {self.cdll.me_last_error().decode()}")


P, I, L, F = c_void_p, c_int, c_int64, c_float
_CORE_PROTOS = {
    "me_gather_rows": [P, P, P, L, L, L, P],
    "me_gather_rows_scaled": [P, I, P, P, L, L, L, F, P],
    "me_take_tokens": [P, P, P, I, I, P],
    "me_rms_norm": [P, I, I, L, P, P, P, P, I, L, I, F, P],
    "me_silu_and_mul": [P, P, I, L, I, P],
    "me_qk_norm_rope_store": [P, I, L, L, P, P, F, P, L, L, P, P, P, P, I, I, I, I, I, P],
    "me_store_kv": [P, P, I, L, L, L, P, P, P, I, I, I, P],
    "me_attn_simple": [P, L, P, L, I, P, P, P, I, P, P, P, L, I, I, I, I, F, I, I, F, P, P],
    "me_attn_tail": [P, L, P, L, P, I, P, P, P, I, P, P, P, L, I, I, I, I, F, I, I, F, P, P],
    "me_gemm_tiled": [P, L, P, L, P, L, I, I, I, I, I, P],
    "me_gemm_skinny_bf16": [P, L, P, L, P, L, I, P, I, I, I, I, I, I, I, P],
    "me_gemm_rows_bf16": [P, L, P, L, P, L, I, P, I, I, I, I, I, P],
    "me_gemm_skinny_norm_bf16": [P, I, I, P, P, P, F, P, L, P, L, I, I, I, I, I, P],
    "me_gemm_mid_bf16": [P, L, P, L, P, L, I, I, I, I, I, I, P],
    "me_gemm_library_bf16": [P, L, P, L, P, L, I, P, ctypes.c_size_t, I, I, I, I, P],
    "me_add_rms_norm": [P, I, I, L, P, P, P, P, L, I, F, P],
    "me_add_rms_norm_partials": [P, I, L, P, P, P, P, L, I, F, P],
    "me_activation": [P, L, P, I, I, L, I, P],
    "me_head_gate": [P, P, L, I, L, I, I, P],
    "me_causal_conv": [P, L, I, P, P, P, L, P, P, I, P, L, I, I, I, P],
    "me_linear_recurrence": [P, L, P, L, P, L, I, P, L, P, P, P, P, P, L, P, P, P, L, I, I, I, I, I, I, I, I, I, I, P, P],
    "me_gated_rms_norm": [P, I, L, P, L, I, P, P, L, I, I, I, F, P],
    "me_scaled_sum_norm": [P, I, I, P, P, P, P, P, F, P, P, P, P, P, I, L, I, F, P],
    "me_softcap": [P, L, L, I, F, P],
    "me_qkv_prepare": [P, L, P, P, P, F, I, I, F, I, P, P, P, P, P, L, I, L, I, I, I, I, I, I, P, P, L, P],
    "me_moe_route": [P, L, I, P, L, I, I, I, I, I, P, P, P, I, I, I, I, F, P, P],
    "me_moe_sort": [P, L, I, I, I, P, P, P, P, P, P, I, I, I, I, I, I, F, P, P],
    "me_moe_gate_up": [P, L, P, P, P, P, P, P, L, I, I, I, I, I, I, P],
    "me_moe_down": [P, P, P, P, P, P, P, P, L, I, I, I, I, I, P],
    "me_moe_experts_simple": [P, L, I, P, P, P, P, P, P, L, I, I, I, I, I, P],
    "me_add_bias": [P, I, I, L, L, P, I, P, I, L, I, P],
    "me_sigmoid_gate": [P, L, P, L, I, L, I, P],
    "me_glu_clamped": [P, L, P, I, L, I, F, F, P],
    "me_weighted_sum": [I, P, P, P, P, P, P, P, P, F, P, P, P, I, L, I, P, P, P, P],
    "me_latent_prepare": [P, L, I, I, I, I, I, I, I, I, P, F, P, L, P, P, P, L, P, P, I, L, P],
    "me_heads_linear": [P, L, L, P, P, L, L, I, L, I, I, I, P],
    "me_token_shift": [P, L, I, P, I, P, L, P, P, P, P, L, I, P],
    "me_decay_rows_recurrence": [P, L, P, L, P, L, P, L, P, L, I, P, P, P, P, L, P, P, P, I, I, I, I, I, I, I, F, F, I, L, P, P],
    "me_sample": [P, L, P, P, P, P, I, I, P],
    "me_sample_static": [P, L, P, P, P, I, I, P],
}
_ATTN_PROTOS = {
    "me_attn_prefill": [P, L, P, L, P, P, P, I, P, P, I, L, I, I, I, F, I, I, I, I, I, I, P, P, I, F, P, P],
    "me_attn_decode": [P, L, P, L, P, P, P, I, P, I, I, I, I, F, I, I, I, P, I, F, P, P],
    "me_attn_decode_fused": [P, L, P, L, P, P, F, P, I, P, P, P, I, P, I, I, I, I, I, F, I, I, I, P, I, F, P, P],
}

_core: _Lib | None = None
_attn: dict = {}


def _require_gpu() -> None:
    if not torch.cuda.is_available():
        raise KernelError("mini_engine_amd needs an AMD GPU (gfx950): torch.cuda.is_available() is False "
                          "and there is no CPU implementation")


def core() -> _Lib:
    global _core
    if _core is None:
        _require_gpu()
        _core = _Lib(build.core_library(), _CORE_PROTOS)
    return _core


def attn_lib(head_dim: int, score_cap: bool = False) -> _Lib:
    key = (head_dim, bool(score_cap)) if score_cap else head_dim
    lib = _attn.get(key)
    if lib is None:
        _require_gpu()
        lib = _Lib(build.attention_library(head_dim, score_cap=bool(score_cap)), _ATTN_PROTOS)
        lib.cdll.me_attn_head_dim.restype = c_int
        if lib.cdll.me_attn_head_dim() != head_dim:
            raise KernelError(f"{lib.path} was built for head size {lib.cdll.me_attn_head_dim()}, not {head_dim}")
        _attn[key] = lib
    return lib


def loaded_libraries() -> list:
    return ([_core.path] if _core else []) + [l.path for l in _attn.values()]


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_device_index: int | None = None


def _stream() -> int:
    """The handle of torch's current stream (also inside a graph capture, which runs on a stream of its
    own). Asked for at every launch, so through the short way where torch offers it."""
    global _device_index
    if _raw_stream is None:
        return torch.cuda.current_stream().cuda_stream
    if _device_index is None:
        _device_index = torch.cuda.current_device()
    return _raw_stream(_device_index)


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _is_i32(t: torch.Tensor, n: int | None = None) -> bool:
    return t.dtype == torch.int32 and t.is_contiguous() and (n is None or t.numel() >= n)


# --------------------------------------------------------------------------- the HIP backend

LIBRARY_WORKSPACE_BYTES = 64 << 20
_library_workspaces: dict = {}            # slot -> workspace: products that run side by side on two streams must not share one
_workspace_slot = 0


class second_workspace:
    """While this is entered, library products use a workspace of their own: for work launched on a second stream beside
    the main one."""

    def __init__(self, slot: int = 1):
        self.slot = slot

    def __enter__(self):
        global _workspace_slot
        self.before, _workspace_slot = _workspace_slot, self.slot

    def __exit__(self, *exc):
        global _workspace_slot
        _workspace_slot = self.before
_library_direct: bool | None = None      # None: not asked yet


def library_is_direct() -> bool:
    """Whether the core library found a hipBLASLt in the process that it can call itself. Without a GPU
    (the dispatch rules are also asked on their own) the answer is yes, as on every GPU box."""
    global _library_direct
    if _library_direct is None:
        if not torch.cuda.is_available():
            return True
        core().cdll.me_gemm_library_available.restype = c_int
        _library_direct = bool(core().cdll.me_gemm_library_available())
    return _library_direct


def library_product(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, splits: int = 1,
                    out: torch.Tensor | None = None) -> torch.Tensor:
    """x [M, K] . w[N, K]^T through hipBLASLt, bfloat16 operands, float32 accumulation (reference
    layers/linear.py:25-26: its F.linear is a library product too).

    Called through the core library, which keeps the descriptors and the chosen algorithm of every
    shape, so a call costs a few microseconds of host time; torch's own route to the same library
    kernel costs several times that for every call, which is what bounds steps that are not replayed
    from a graph. torch's route stays as the way out when the process holds no hipBLASLt that the core
    library can find, or when it offers nothing for a shape. The workspace is allocated once, outside
    any graph capture (the first product of a process is never a captured one: a step runs eagerly
    before it is captured).

    splits > 1: K is cut in that many equal slices, computed as one strided batch; the result is their
    float32 partial sums [splits, M, N] for a consumer that adds them, or None where only torch's
    route is open (the caller then takes its other path)."""
    handle = _stream()
    _library_workspace = _library_workspaces.get(_workspace_slot)
    if library_is_direct() and _library_workspace is None and not torch.cuda.is_current_stream_capturing():
        _library_workspace = _library_workspaces[_workspace_slot] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=x.device)
    if _library_direct and _library_workspace is not None:
        M, K = x.shape
        N = w.shape[0]
        y = out if out is not None else torch.empty((M, N) if splits == 1 else (splits, M, N), dtype=out_dtype, device=x.device)
        rc = core().fns["me_gemm_library_bf16"](x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N,
                                               _code(out_dtype), _library_workspace.data_ptr(),
                                               LIBRARY_WORKSPACE_BYTES, M, N, K, splits, handle)
        if rc == 0:
            return y
        if rc != -3:
            raise KernelError(f"me_gemm_library_bf16: {core().cdll.me_last_error().decode()}")
    if splits > 1:
        return None                 # partial sums over slices of K only through the direct call
    y = torch.mm(x, w.t(), out_dtype=torch.float32) if out_dtype == torch.float32 else torch.matmul(x, w.t())
    if out is not None:
        out.copy_(y)
        return out
    return y


class RouteRule:
    """How a router's float32 logits become a choice of experts and their weights (`moe_route`). scoring: "softmax" over
    all experts or "sigmoid" per expert; correction: float32 [experts] added to the scores for the choice only, or None;
    group_top: a group of neighbours scores as the sum of its so many largest choice scores; normalise: the chosen
    experts' scores are divided by their sum; scale: a constant on the weights."""

    def __init__(self, scoring: str = "softmax", correction=None, group_top: int = 1, normalise: bool = True, scale: float = 1.0):
        if scoring not in ("softmax", "sigmoid") or group_top < 1:
            raise ValueError("scoring is 'softmax' or 'sigmoid', group_top positive")
        self.scoring, self.correction, self.group_top = scoring, correction, int(group_top)
        self.normalise, self.scale = bool(normalise), float(scale)

    def check(self, E: int) -> None:
        c = self.correction
        _check(c is None or (c.dtype == torch.float32 and c.shape == (E,) and c.is_contiguous()), "moe_route: the correction must be float32 [experts]")

    def args(self) -> tuple:
        return (self.group_top, int(self.scoring == "sigmoid"), int(self.normalise), self.scale, _ptr(self.correction))


class HipBackend:
    """Each method is one kernel (or one dispatch among kernels of the same meaning)."""

    name = "hip"

    # -- rows ----------------------------------------------------------------------------
    def gather_rows(self, src: torch.Tensor, idx: torch.Tensor, scale: float | None = None) -> torch.Tensor:
        """out[r] = src[idx[r]] (embedding lookup: reference layers/embed_head.py:10-11;
        rows that want logits: layers/embed_head.py:20-22). With `scale`: out[r] = scale * src[idx[r]] in float32
        (embedding rows under a multiplier: they start the 32-bit stream without a rounding of their own)."""
        _check(src.dim() == 2 and src.is_contiguous(), "gather_rows: source must be a contiguous matrix")
        _check(_is_i32(idx) and idx.dim() == 1, "gather_rows: indices must be int32 [n]")
        if scale is not None:
            out = torch.empty((idx.numel(), src.shape[1]), dtype=torch.float32, device=src.device)
            core().call("me_gather_rows_scaled", src.data_ptr(), _code(src.dtype), idx.data_ptr(), out.data_ptr(), idx.numel(),
                        src.shape[1], src.shape[0], float(scale), _stream())
            return out
        out = torch.empty((idx.numel(), src.shape[1]), dtype=src.dtype, device=src.device)
        core().call("me_gather_rows", src.data_ptr(), idx.data_ptr(), out.data_ptr(), idx.numel(),
                    src.shape[1] * src.element_size(), src.shape[0], _stream())
        return out

    def take_tokens(self, tokens: torch.Tensor, sampled: torch.Tensor, take: torch.Tensor) -> None:
        """tokens[r] = sampled[take[r]] where take[r] >= 0, in place (int32 [R], [S], [R]): the tokens of the last
        sampling call go into the rows of a step launched before they have reached the host."""
        R = tokens.numel()
        _check(_is_i32(tokens) and _is_i32(sampled) and _is_i32(take, R), "take_tokens: int32 tensors, one source row per token row")
        core().call("me_take_tokens", tokens.data_ptr(), sampled.data_ptr(), take.data_ptr(), R, sampled.numel(), _stream())

    # -- norm ----------------------------------------------------------------------------
    def rms_norm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, residual: torch.Tensor | None,
                 out_dtype: torch.dtype, want_residual: bool = True):
        """y = w * r * rsqrt(mean(r^2) + eps), r = x (+ residual) in float32 (reference
        layers/layernorm.py:11-24). x: [T, n], or float32 partial sums [P, T, n] that are added
        first. Returns (y [T, n] in out_dtype, r [T, n] float32 or None)."""
        parts = 1
        if x.dim() == 3:
            parts = x.shape[0]
            _check(x.dtype == torch.float32, "rms_norm: stacked partial sums must be float32")
        _check(x.is_contiguous(), "rms_norm: x must be contiguous")
        T, n = x.shape[-2], x.shape[-1]
        _check(weight.dtype == torch.float32 and weight.shape == (n,) and weight.is_contiguous(),
               "rms_norm: weight must be float32 [n]")
        if residual is not None:
            _check(residual.dtype == torch.float32 and residual.shape == (T, n) and residual.is_contiguous(),
                   "rms_norm: residual must be contiguous float32 [T, n]")
        y = torch.empty((T, n), dtype=out_dtype, device=x.device)
        res_out = torch.empty((T, n), dtype=torch.float32, device=x.device) if want_residual else None
        core().call("me_rms_norm", x.data_ptr(), _code(x.dtype), parts, T * n, _ptr(residual), _ptr(res_out),
                    weight.data_ptr(), y.data_ptr(), _code(out_dtype), T, n, float(eps), _stream())
        return y, res_out

    # -- feed-forward activation ---------------------------------------------------------
    def silu_and_mul(self, gu: torch.Tensor) -> torch.Tensor:
        """silu(gu[:, :I]) * gu[:, I:] (reference layers/activation.py:5-7)."""
        _check(gu.dim() == 2 and gu.is_contiguous() and gu.shape[1] % 2 == 0, "silu_and_mul: [T, 2I] contiguous")
        inter = gu.shape[1] // 2
        out = torch.empty((gu.shape[0], inter), dtype=gu.dtype, device=gu.device)
        core().call("me_silu_and_mul", gu.data_ptr(), out.data_ptr(), _code(gu.dtype), gu.shape[0], inter, _stream())
        return out

    # -- q/k norm + rotary + cache write -------------------------------------------------
    def qk_norm_rope_store(self, qkv, q_weight, k_weight, eps, table, positions, slots, k_cache, v_cache,
                           Hq: int, Hkv: int, D: int, page: int, store: bool = True, position_bound: int = 0) -> None:
        """In place on packed rows: per-head RMSNorm of q and k (weights float32 [D] or None), then
        rotary by `table` [P, D/2, 2] float32 (or None), q written back. `position_bound`: every position
        of the step is below it (the longest context the step's layout allows; 0: not told); a bound beyond
        the table's rows is refused.

        store=True: rows are [T, (Hq+2Hkv)*D]; k and v are scattered to the pages at `slots`
        (slots < 0 skipped). store=False: rows are [T, (Hq+Hkv)*D] (Hkv may be 0); k is written
        back in place and nothing is cached. (reference models/qwen3.py:34-36,
        layers/rotary_embedding.py:20-25, csrc/kv_cache.cu:10-31.)"""
        T = qkv.shape[0]
        width = (Hq + (2 * Hkv if store else Hkv)) * D
        _check(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == width,
               f"qk_norm_rope_store: rows must be [T, {width}] with unit inner stride, got {tuple(qkv.shape)}")
        for w in (q_weight, k_weight):
            _check(w is None or (w.dtype == torch.float32 and w.shape == (D,) and w.is_contiguous()),
                   "qk_norm_rope_store: norm weights must be float32 [D]")
        _check((q_weight is None) == (k_weight is None), "qk_norm_rope_store: give both norm weights or neither")
        if table is not None:
            _check(table.dtype == torch.float32 and table.is_contiguous() and table.shape[1:] == (D // 2, 2),
                   "qk_norm_rope_store: rotary table must be float32 [P, D/2, 2]")
        _check(_is_i32(positions, T), "qk_norm_rope_store: positions must be int32 [T]")
        if store:
            _check(_is_i32(slots, T), "qk_norm_rope_store: slots must be int32 [T]")
            _check(k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype and k_cache.is_contiguous()
                   and v_cache.is_contiguous(), "qk_norm_rope_store: caches must be contiguous and of the rows' dtype")
            _check(k_cache.shape[1:] == (Hkv, page, D) and v_cache.shape[1:] == (Hkv, D, page),
                   "qk_norm_rope_store: caches must be K [pages, Hkv, page, D] and V [pages, Hkv, D, page]")
        core().call("me_qk_norm_rope_store", qkv.data_ptr(), _code(qkv.dtype), T, qkv.stride(0), _ptr(q_weight),
                    _ptr(k_weight), float(eps), _ptr(table), 0 if table is None else table.shape[0], int(position_bound),
                    positions.data_ptr(), _ptr(slots) if store else None, _ptr(k_cache) if store else None,
                    _ptr(v_cache) if store else None, Hq, Hkv, D, page, int(store), _stream())

    def store_kv(self, k, v, slots, k_cache, v_cache, page: int) -> None:
        """Scatter k, v [T, Hkv, D] (views with a token stride are fine) into the pages; slots < 0
        are skipped (reference csrc/kv_cache.cu:10-31; the copy is bit-exact)."""
        T, Hkv, D = k.shape
        _check(v.shape == k.shape and k.dtype == v.dtype == k_cache.dtype == v_cache.dtype, "store_kv: dtype/shape mismatch")
        for t in (k, v):
            _check(t.stride(2) == 1 and t.stride(1) == D, "store_kv: heads of a token must be one contiguous row")
        _check(k_cache.shape[1:] == (Hkv, page, D) and v_cache.shape[1:] == (Hkv, D, page) and k_cache.is_contiguous()
               and v_cache.is_contiguous(), "store_kv: caches must be K [pages, Hkv, page, D], V [pages, Hkv, D, page]")
        _check(_is_i32(slots, T), "store_kv: slots must be int32 [T]")
        core().call("me_store_kv", k.data_ptr(), v.data_ptr(), _code(k.dtype), T, k.stride(0), v.stride(0),
                    slots.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), Hkv, D, page, _stream())

    # -- attention -----------------------------------------------------------------------
    def paged_attention(self, q, k_cache, v_cache, page: int, block_tables, context_lens, seq_of_token,
                        positions, prefill_cu, num_decodes: int, max_decode_context: int, scale: float,
                        window: int | None, Hq: int, Hkv: int, D: int, force_simple: bool = False,
                        max_prefill_context: int = 0, even_contexts: bool = False, decode_as_prefill: bool = False,
                        chunk: int | None = None, keep_first: int = 0, softcap: float | None = None, sinks=None):
        """Causal attention of this step's tokens over the paged keys of their requests. `chunk`: a block mask in
        place of a window: the query at position i sees the keys j <= i of its own block, floor(j / chunk) =
        floor(i / chunk) (the kernels take it as a negative window). `keep_first`: behind a window the keys j <
        keep_first stay visible. `softcap` c: every score becomes c * tanh(score / c) before the softmax. `sinks`
        (float32 [Hq]): exp(sink_h) joins the softmax's denominator of head h, a term without key or value. With any
        three. On the matrix-core path the cap runs inside the kernels (a library variant of its own), which also leave
        the logarithm of every softmax denominator; a second kernel (`attn_tail`) then joins the kept keys behind the
        window and the sink to that softmax. The float32 path and odd sizes take the exact kernel (`attn_simple`) for all of it.

        q: [T, Hq*D] (a strided view is fine). Rows are ordered decode requests first (one token
        each, `num_decodes` of them), then the others; `prefill_cu` int32 [B - num_decodes + 1]
        are prefix sums of the new-token counts of the others. `context_lens` int32 [B] counts keys
        after this step's write; `block_tables` int32 [B, MB]. `max_prefill_context`: the largest
        context among the others (a hint for cutting long key ranges; 0 = unknown). `even_contexts`: the
        decode requests' contexts are equally long (decode_contexts_even), which lets the decode kernel
        keep each request on one XCD. `decode_as_prefill` (or the module's DECODE_AS_PREFILL): the
        single-token rows go through the prefill kernel too, as prompts of one token: a second
        implementation of decoding to check the first against. Returns [T, Hq*D].
        (reference layers/attention.py:63-76: decode rows to the decode kernel, the rest to the
        prefill kernel, or all rows to the prefill kernel in its `unified` mode; csrc/paged_decode.cu,
        csrc/paged_prefill.cu.)"""
        T = q.shape[0]
        B = context_lens.numel()
        _check(q.dim() == 2 and q.shape[1] == Hq * D and q.stride(1) == 1, "attention: q must be [T, Hq*D], unit inner stride")
        _check(k_cache.shape[1:] == (Hkv, page, D) and v_cache.shape[1:] == (Hkv, D, page), "attention: cache layout mismatch")
        _check(k_cache.dtype == q.dtype and v_cache.dtype == q.dtype, "attention: cache dtype differs from q")
        _check(block_tables.dim() == 2 and block_tables.dtype == torch.int32 and block_tables.stride(1) == 1
               and block_tables.shape[0] >= B, "attention: block tables must be int32 [B, MB]")
        _check(_is_i32(context_lens) and _is_i32(seq_of_token, T) and _is_i32(positions, T), "attention: metadata must be int32")
        _check(0 <= num_decodes <= B and num_decodes <= T, "attention: bad decode count")
        out = torch.empty((T, Hq * D), dtype=q.dtype, device=q.device)
        _check(not (window and chunk), "attention: a window and a block mask exclude each other")
        win = -int(chunk) if chunk else int(window or 0)
        span = abs(win)          # no query sees more keys than this (0: all of them)
        _check(not keep_first or (window and keep_first > 0), "attention: keys are kept behind a window only")
        _check(sinks is None or (sinks.dtype == torch.float32 and sinks.shape == (Hq,) and sinks.is_contiguous()),
               "attention: sinks must be float32 [Hq]")
        tail = bool(keep_first) or sinks is not None
        mfma = (q.dtype == torch.bfloat16 and D % 16 == 0 and 16 <= D <= 512 and page >= 8 and page & (page - 1) == 0
                and not force_simple and (MFMA_WITH_EXTRAS or not (tail or softcap)))
        if not mfma:
            core().call("me_attn_simple", q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), _code(q.dtype),
                        k_cache.data_ptr(), v_cache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0),
                        seq_of_token.data_ptr(), positions.data_ptr(), context_lens.data_ptr(), T, Hq, Hkv, D, page,
                        float(scale), win, int(keep_first or 0), float(softcap or 0.0), _ptr(sinks), _stream())
            return out
        lib = attn_lib(D, score_cap=bool(softcap))
        cap = float(softcap or 0.0)
        lse = torch.empty((T, Hq), dtype=torch.float32, device=q.device) if tail else None
        es = q.element_size()
        if (decode_as_prefill or DECODE_AS_PREFILL) and num_decodes > 0:
            ones = torch.arange(num_decodes + 1, dtype=torch.int32, device=q.device)
            prefill_cu = ones if prefill_cu is None else torch.cat((ones[:-1], prefill_cu[:B - num_decodes + 1] + num_decodes))
            max_prefill_context = max(max_prefill_context, max_decode_context)
            num_decodes = 0
        if num_decodes > 0:
            part_size, num_parts = decode_partitions(num_decodes, Hq, Hkv, max_decode_context, even_contexts)
            if D > 128:
                part_size, num_parts = wide_head_partitions(part_size, num_parts, num_decodes * Hkv * ((Hq // Hkv + 15) // 16), max_decode_context)
            scratch = _scratch(num_decodes * Hq * num_parts * (D + 2), q.device) if num_parts > 1 else None
            lib.call("me_attn_decode", q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), k_cache.data_ptr(),
                     v_cache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0), context_lens.data_ptr(),
                     num_decodes, Hq, Hkv, page, float(scale), win, part_size, num_parts, _ptr(scratch),
                     0 if even_contexts else 1, cap, _ptr(lse), _stream())
        if T > num_decodes:
            _check(prefill_cu is not None and _is_i32(prefill_cu, B - num_decodes + 1), "attention: prefill_cu must be int32 [B-Dn+1]")
            Tp = T - num_decodes
            col_tiles = prefill_col_tiles(max_prefill_context, span, Tp, Hq, D)
            seg_keys, max_segs = prefill_segments(max_prefill_context, span, Tp, Hq, D, col_tiles)
            waves = prefill_waves(max_prefill_context, Tp, B - num_decodes, Hq, Hkv, col_tiles, max_segs)
            # the segments' partial results: in a buffer that is kept between steps (a step's decode rows have
            # finished with theirs before, on the same stream, but the two are kept apart all the same)
            pf = _scratch(Tp * Hq * max_segs * (D + 2), q.device, "prefill") if max_segs > 1 else None
            lib.call("me_attn_prefill", q.data_ptr() + num_decodes * q.stride(0) * es, q.stride(0),
                     out.data_ptr() + num_decodes * out.stride(0) * es, out.stride(0), k_cache.data_ptr(),
                     v_cache.data_ptr(), block_tables.data_ptr() + num_decodes * block_tables.stride(0) * 4,
                     block_tables.stride(0), context_lens.data_ptr() + num_decodes * 4, prefill_cu.data_ptr(),
                     B - num_decodes, Tp, Hq, Hkv, page, float(scale), win, col_tiles, PREFILL_THROUGH_LDS, waves, seg_keys, max_segs,
                     _ptr(pf), seq_of_token.data_ptr() + num_decodes * 4, num_decodes, cap,
                     None if lse is None else lse.data_ptr() + num_decodes * Hq * 4, _stream())
        if tail:
            core().call("me_attn_tail", q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), lse.data_ptr(), _code(q.dtype),
                        k_cache.data_ptr(), v_cache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0),
                        seq_of_token.data_ptr(), positions.data_ptr(), context_lens.data_ptr(), T, Hq, Hkv, D, page, float(scale),
                        win, int(keep_first or 0), cap, _ptr(sinks), _stream())
        return out

    def decode_step_attention(self, qkv, q_weight, k_weight, eps, table, k_cache, v_cache, page: int, block_tables,
                              context_lens, max_context: int, scale: float, window: int | None, Hq: int, Hkv: int,
                              D: int, even_contexts: bool = False, chunk: int | None = None):
        """A pure decode step's `qk_norm_rope_store` and `paged_attention` as one launch: rows [B, (Hq+2Hkv)*D]
        as the packed product left them (row r is request r's one new token, at position context_lens[r] - 1).
        The kernel norms and rotates q and the new key in float32, rounds them to bfloat16 as the separate
        kernel leaves them in the rows, writes the new key and value to the page the block table names for
        that position and attends over the pages. The rows stay as they were. Takes what `decode_step_fuses`
        admits. Returns [B, Hq*D]. (reference models/qwen3.py:34-38, layers/attention.py:63-70: the same
        four calls one after the other.)"""
        B = qkv.shape[0]
        _check(decode_step_fuses(qkv.dtype, D, page), "decode_step_attention: bfloat16 rows, head sizes in steps of 16 "
               "up to 512 and pages of a power of two from 8 on")
        _check(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == (Hq + 2 * Hkv) * D,
               f"decode_step_attention: rows must be [B, {(Hq + 2 * Hkv) * D}] with unit inner stride")
        for w in (q_weight, k_weight):
            _check(w is None or (w.dtype == torch.float32 and w.shape == (D,) and w.is_contiguous()),
                   "decode_step_attention: norm weights must be float32 [D]")
        _check((q_weight is None) == (k_weight is None), "decode_step_attention: give both norm weights or neither")
        if table is not None:
            _check(table.dtype == torch.float32 and table.is_contiguous() and table.shape[1:] == (D // 2, 2),
                   "decode_step_attention: rotary table must be float32 [P, D/2, 2]")
        _check(k_cache.shape[1:] == (Hkv, page, D) and v_cache.shape[1:] == (Hkv, D, page) and k_cache.is_contiguous()
               and v_cache.is_contiguous() and k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype,
               "decode_step_attention: caches must be K [pages, Hkv, page, D] and V [pages, Hkv, D, page] of the rows' dtype")
        _check(block_tables.dim() == 2 and block_tables.dtype == torch.int32 and block_tables.stride(1) == 1
               and block_tables.shape[0] >= B and _is_i32(context_lens) and context_lens.numel() >= B,
               "decode_step_attention: block tables int32 [B, MB], context lengths int32 [B]")
        _check(block_tables.shape[1] * page >= max_context, "decode_step_attention: block tables shorter than the longest context")
        out = torch.empty((B, Hq * D), dtype=qkv.dtype, device=qkv.device)
        part_size, num_parts = decode_partitions(B, Hq, Hkv, max_context, even_contexts)
        scratch = _scratch(B * Hq * num_parts * (D + 2), qkv.device) if num_parts > 1 else None
        attn_lib(D).call("me_attn_decode_fused", qkv.data_ptr(), qkv.stride(0), out.data_ptr(), out.stride(0),
                         _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(table), 0 if table is None else table.shape[0],
                         k_cache.data_ptr(), v_cache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0),
                         context_lens.data_ptr(), int(max_context), B, Hq, Hkv, page, float(scale),
                         -int(chunk) if chunk else int(window or 0),
                         part_size, num_parts, _ptr(scratch), 0 if even_contexts else 1, 0.0, None, _stream())
        return out

    # -- matrix products -----------------------------------------------------------------
    def linear(self, x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype | None = None,
               allow_partials: bool = False, out: torch.Tensor | None = None):
        """x [M, K] . w[N, K]^T (reference layers/linear.py:25-26: F.linear, no bias).

        float32: plain FMA kernel. bfloat16: the skinny MFMA kernel for up to 32 rows (64 for
        smaller weights or when K is split), the library product (hipBLASLt, library_product) above
        that, for the head over a large vocabulary and for large weights with several rows
        (library_streams_better), the FMA kernel for shapes the MFMA kernel refuses.
        With allow_partials the result may be float32 partial sums [S, M, N] over slices of K for a
        consumer that adds them: from the skinny kernel when the output features are few
        (choose_ksplit), from the rows kernel for 17-32 rows over large weights (rows_takes), from the tiled
        kernel for 33 to a few hundred rows over weights up to 27 M elements (mid_slices), from the
        library as a strided batch for 33-1,024 rows over larger weights (library_splits).
        `out` (not with allow_partials): a contiguous [M, N] tensor of the output dtype to write into."""
        _check(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1], f"linear: {tuple(x.shape)} x {tuple(w.shape)}^T")
        _check(x.dtype == w.dtype, f"linear: activation {x.dtype} and weight {w.dtype} differ")
        _check(x.stride(1) == 1 and w.stride(1) == 1, "linear: rows must be contiguous")
        M, K = x.shape
        N = w.shape[0]
        out_dtype = out_dtype or x.dtype
        if out is not None:
            _check(not allow_partials and out.shape == (M, N) and out.dtype == out_dtype and out.is_contiguous()
                   and out.device == x.device, "linear: `out` must be a contiguous [M, N] tensor of the output dtype")
        new = (lambda: out) if out is not None else (lambda: torch.empty((M, N), dtype=out_dtype, device=x.device))
        if x.dtype == torch.float32:
            _check(out_dtype == torch.float32, "linear: float32 inputs give float32 outputs")
            y = new()
            core().call("me_gemm_tiled", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N,
                        ME_F32, ME_F32, M, N, K, _stream())
            return y
        aligned = (K % 8 == 0 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
                   and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)
        if not aligned:
            y = new()
            core().call("me_gemm_tiled", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N,
                        ME_BF16, _code(out_dtype), M, N, K, _stream())
            return y
        mid_parts = mid_takes(M, N, K, True) if (allow_partials and out_dtype == x.dtype) else 0
        if mid_parts > 1:
            parts = torch.empty((mid_parts, M, N), dtype=torch.float32, device=x.device)
            core().call("me_gemm_mid_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), parts.data_ptr(), N,
                        ME_F32, mid_parts, M, N, K, 0, _stream())
            return parts
        splits = library_splits(M, N, K) if (allow_partials and out_dtype == x.dtype) else 1
        if splits > 1:
            parts = library_product(x, w, torch.float32, splits)
            if parts is not None:
                return parts
        if allow_partials and out_dtype == x.dtype and rows_takes(M, N, K):
            ksplit = rows_ksplit(K)
            parts = torch.empty((ksplit, M, N), dtype=torch.float32, device=x.device)
            core().call("me_gemm_rows_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), None, N,
                        ME_F32, parts.data_ptr(), ksplit, M, N, K, rows_wide(M, N, ksplit), _stream())
            return parts
        ksplit = choose_ksplit(M, N, K) if (allow_partials and M <= PARTIALS_MAX_M and out_dtype == x.dtype
                                            and (M <= SKINNY_MAX_M or N * K <= SKINNY_WIDE_MAX_WEIGHT)
                                            and not library_streams_better(M, N, K)) else 1
        if ksplit > 1:
            parts = torch.empty((ksplit, M, N), dtype=torch.float32, device=x.device)
            core().call("me_gemm_skinny_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), None, N,
                        ME_F32, parts.data_ptr(), ksplit, M, N, K, 0, 0, skinny_wide(N, K), _stream())
            return parts
        if skinny_takes(M, N, K):
            y = new()
            core().call("me_gemm_skinny_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N,
                        _code(out_dtype), None, 1, M, N, K, 0, 0, skinny_wide(N, K), _stream())
            return y
        if mid_takes(M, N, K, False) == 1:
            y = new()
            core().call("me_gemm_mid_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N,
                        _code(out_dtype), 1, M, N, K, 0, _stream())
            return y
        # many rows, or the head over a large vocabulary: the library product (float32 accumulation; the
        # float32 output form keeps the logits unrounded)
        return library_product(x, w, out_dtype, out=out)

    def gated_linear(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """silu(x . w[:I]^T) * (x . w[I:]^T) for a packed gate/up weight w [2 I, K] (gate rows first), as one
        launch: the product's workgroups pair each gate feature with its up feature when they merge their waves,
        from the unrounded sums (the separate kernels round the product to bfloat16 first). For the row counts
        `gated_linear_fuses` admits. Returns [M, I]. (reference layers/linear.py:29-45, layers/activation.py:5-7.)"""
        _check(gated_linear_fuses(x, w), "gated_linear: bfloat16, few rows, see gated_linear_fuses")
        M, K = x.shape
        N = w.shape[0]
        y = torch.empty((M, N // 2), dtype=x.dtype, device=x.device)
        if M > GATED_EPILOGUE_MAX_M:        # a few hundred rows over a small weight: the gating in that kernel's epilogue
            core().call("me_gemm_mid_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N // 2,
                        ME_BF16, 1, M, N, K, 1, _stream())
            return y
        core().call("me_gemm_skinny_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N // 2,
                    ME_BF16, None, 1, M, N, K, 0, 1, skinny_wide(N, K), _stream())
        return y

    def norm_linear(self, x: torch.Tensor, residual: torch.Tensor | None, norm_weight: torch.Tensor, eps: float,
                    w: torch.Tensor, out_dtype: torch.dtype | None = None, want_residual: bool = True,
                    gated: bool = False):
        """`rms_norm` and `linear` behind it as one launch, for the few rows `norm_linear_fuses` admits:
        r = x (+ residual), x being rows [M, K] or float32 partial sums [S, M, K]; y = (norm_weight * r
        rounded to bfloat16) . w^T, scaled by 1 / rms(r) in float32 (the scale is one number per row, so
        it is applied to the finished sums; the separate kernels round norm_weight * r / rms(r) instead:
        the same relative rounding). `gated`: w is a packed gate/up weight and y is silu(gate) * up, [M, N/2],
        as in `gated_linear`. Returns (y [M, N], r float32 [M, K] or None).
        (reference layers/layernorm.py:11-24, layers/linear.py:25-26.)"""
        _check(norm_linear_fuses(x, w), "norm_linear: bfloat16 weights, few rows, see norm_linear_fuses")
        _check(not gated or w.shape[0] % 2 == 0, "norm_linear: a packed gate/up weight has an even number of rows")
        S = x.shape[0] if x.dim() == 3 else 1
        M, K = x.shape[-2], x.shape[-1]
        N = w.shape[0]
        _check(norm_weight.dtype == torch.float32 and norm_weight.shape == (K,) and norm_weight.is_contiguous(),
               "norm_linear: the norm's weight must be float32 [K]")
        if residual is not None:
            _check(residual.dtype == torch.float32 and residual.shape == (M, K) and residual.is_contiguous(),
                   "norm_linear: residual must be contiguous float32 [M, K]")
        out_dtype = out_dtype or w.dtype
        cols = N // 2 if gated else N
        y = torch.empty((M, cols), dtype=out_dtype, device=x.device)
        res_out = torch.empty((M, K), dtype=torch.float32, device=x.device) if want_residual else None
        core().call("me_gemm_skinny_norm_bf16", x.data_ptr(), _code(x.dtype), S, _ptr(residual), _ptr(res_out),
                    norm_weight.data_ptr(), float(eps), w.data_ptr(), w.stride(0), y.data_ptr(), cols, _code(out_dtype),
                    M, N, K, int(gated), _stream())
        return y, res_out

    def silu_mul_linear(self, gu: torch.Tensor, w: torch.Tensor, allow_partials: bool = False):
        """(silu(gu[:, :I]) * gu[:, I:]) . w[N, I]^T: the gating fused into the product for few
        rows and a moderate width (bfloat16, M <= 16, I <= 4096, where the product is a weight stream
        and the gating is free);
        otherwise the two kernels one after the other (reference models/qwen3.py:50-51)."""
        M, two_i = gu.shape
        inter = two_i // 2
        _check(w.shape[1] == inter and two_i == 2 * inter, f"silu_mul_linear: {tuple(gu.shape)} against {tuple(w.shape)}")
        fused = (gu.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and M <= GATED_MAX_M and inter % 8 == 0
                 and inter <= GATED_MAX_K and not library_streams_better(M, w.shape[0], inter)
                 and gu.is_contiguous() and w.stride(1) == 1 and w.stride(0) % 8 == 0
                 and gu.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)
        if not fused:
            return self.linear(self.silu_and_mul(gu), w, None, allow_partials)
        N = w.shape[0]
        ksplit = choose_ksplit(M, N, inter) if allow_partials else 1      # fused only for M <= GATED_MAX_M <= PARTIALS_MAX_M
        if ksplit > 1:
            parts = torch.empty((ksplit, M, N), dtype=torch.float32, device=gu.device)
            core().call("me_gemm_skinny_bf16", gu.data_ptr(), gu.stride(0), w.data_ptr(), w.stride(0), None, N,
                        ME_F32, parts.data_ptr(), ksplit, M, N, inter, 1, 0, 0, _stream())
            return parts
        y = torch.empty((M, N), dtype=gu.dtype, device=gu.device)
        core().call("me_gemm_skinny_bf16", gu.data_ptr(), gu.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N,
                    ME_BF16, None, 1, M, N, inter, 1, 0, 0, _stream())
        return y

    # -- norms on a sublayer's output, activations, gates ----------------------------------
    def add_rms_norm(self, y: torch.Tensor, weight: torch.Tensor, eps: float, stream: torch.Tensor, out_dtype: torch.dtype):
        """stream + weight * y / sqrt(mean(y^2) + eps), all float32. y: [T, n] in the compute dtype, or float32
        partial sums [P, T, n] that are added first. Returns (the new stream rounded to out_dtype, the new stream
        float32 [T, n]); with out_dtype float32 both are one tensor."""
        parts = y.shape[0] if y.dim() == 3 else 1
        _check(y.is_contiguous() and (y.dim() == 2 or y.dtype == torch.float32), "add_rms_norm: y contiguous, partial sums float32")
        T, n = y.shape[-2], y.shape[-1]
        _check(weight.dtype == torch.float32 and weight.shape == (n,) and weight.is_contiguous(), "add_rms_norm: weight float32 [n]")
        _check(stream.dtype == torch.float32 and stream.shape == (T, n) and stream.is_contiguous(), "add_rms_norm: stream float32 [T, n]")
        new = torch.empty_like(stream)
        if out_dtype == torch.float32:
            _check(y.dtype == torch.float32, "add_rms_norm: a float32 stream copy needs float32 rows")
            core().call("me_add_rms_norm", y.data_ptr(), ME_F32, parts, T * n, weight.data_ptr(), stream.data_ptr(), new.data_ptr(),
                        None, T, n, float(eps), _stream())
            return new, new
        rounded = torch.empty((T, n), dtype=out_dtype, device=y.device)
        if y.dtype == torch.float32:
            core().call("me_add_rms_norm_partials", y.data_ptr(), parts, T * n, weight.data_ptr(), stream.data_ptr(), new.data_ptr(),
                        rounded.data_ptr(), T, n, float(eps), _stream())
        else:
            core().call("me_add_rms_norm", y.data_ptr(), _code(y.dtype), 1, 0, weight.data_ptr(), stream.data_ptr(), new.data_ptr(),
                        rounded.data_ptr(), T, n, float(eps), _stream())
        return rounded, new

    def activation(self, x: torch.Tensor, kind: str) -> torch.Tensor:
        """silu(x), relu(x)^2 or tanh(x) of a row view [T, n] (unit inner stride), float32 inside; contiguous result."""
        _check(x.dim() == 2 and x.stride(1) == 1 and kind in ACTIVATIONS, "activation: rows with unit inner stride, a known kind")
        T, n = x.shape
        out = torch.empty((T, n), dtype=x.dtype, device=x.device)
        core().call("me_activation", x.data_ptr(), x.stride(0), out.data_ptr(), _code(x.dtype), ACTIVATIONS[kind], T, n, _stream())
        return out

    def head_gate(self, o: torch.Tensor, gate: torch.Tensor, H: int, D: int) -> None:
        """o[t, h, :] *= sigmoid(gate[t, h]) in place; o contiguous [T, H * D], gate a view [T, H]."""
        T = o.shape[0]
        _check(o.is_contiguous() and o.shape == (T, H * D) and gate.shape == (T, H) and gate.stride(1) == 1
               and gate.dtype == o.dtype, "head_gate: o [T, H * D] contiguous, gate [T, H] of its dtype")
        core().call("me_head_gate", o.data_ptr(), gate.data_ptr(), gate.stride(0), _code(o.dtype), T, H, D, _stream())

    # -- mixers with a state of fixed size -------------------------------------------------
    def causal_conv(self, x, weight, bias, state, state_slots, cu_seqlens, q_lens) -> torch.Tensor:
        """silu(bias + sum_j weight[:, j] * x[t - (taps - 1) + j]) per channel (bias None: none) over every request's tokens of this step,
        continued from its state: x a row view [T, C]; weight float32 [C, taps] (the last tap is the current
        token's); state a float32 view [slots, C * (taps - 1)] (per channel the inputs before the request's next
        token, oldest first), rows `state_slots`; it moves on by this step's tokens. `q_lens`: the requests' token
        counts on the host (the launch is sized by the longest). Returns [T, C]."""
        T, C = x.shape
        taps = weight.shape[1]
        B = state_slots.numel()
        _check(x.stride(1) == 1 and weight.dtype == torch.float32 and weight.shape == (C, taps) and weight.is_contiguous()
               and (bias is None or (bias.dtype == torch.float32 and bias.shape == (C,) and bias.is_contiguous())), "causal_conv: bad operands")
        _check(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1 and state.shape[1] == C * (taps - 1),
               "causal_conv: state must be float32 [slots, C * (taps - 1)]")
        _check(_is_i32(state_slots) and _is_i32(cu_seqlens, B + 1) and len(q_lens) == B and sum(q_lens) == T,
               "causal_conv: metadata must be int32, one token count per request")
        out = torch.empty((T, C), dtype=x.dtype, device=x.device)
        core().call("me_causal_conv", x.data_ptr(), x.stride(0), _code(x.dtype), weight.data_ptr(), _ptr(bias),
                    state.data_ptr(), state.stride(0), state_slots.data_ptr(), cu_seqlens.data_ptr(), max(q_lens),
                    out.data_ptr(), T, B, C, taps, _stream())
        return out

    def linear_recurrence(self, q, k, v, state, state_slots, cu_seqlens, q_lens, H: int, G: int, N: int, P: int,
                          decay=None, dt=None, dt_bias=None, rate=None, skip=None, silu: bool = False) -> torch.Tensor:
        """Per request and head, over the request's tokens of this step in order, from its state row:
            S_t = a_t S_(t-1) + b_t k_t v_t^T,   y_t = S_t^T q_t (+ skip_h v_t),      S [N, P] float32.
        q, k: row views [T, G * N] (heads share them by groups of H / G), v: [T, H * P]; state: float32 view
        [slots, H * N * P], rows `state_slots`, left at the state behind the last token. a, b: `decay` (float32 [H])
        and 1; or exp(-rate_h dt), dt with dt = softplus(dt[t, h] + dt_bias_h) (`dt` a row view [T, H], the others
        float32 [H]). `silu`: q, k and v pass silu on their way in. `q_lens`: the requests' token counts on the host: long ones are cut into spans that run side
        by side (`recurrence_spans`). Returns float32 [T, H * P], or partial sums [S, T, H * P] over slices of N
        for a consumer that adds them."""
        T, B = v.shape[0], state_slots.numel()
        dtype = v.dtype
        for t, width in ((q, G * N), (k, G * N), (v, H * P)):
            _check(t.dim() == 2 and t.shape == (T, width) and t.stride(1) == 1 and t.dtype == dtype, "recurrence: bad q, k or v rows")
        _check(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1 and state.shape[1] == H * N * P,
               "recurrence: state must be float32 [slots, H * N * P]")
        _check((decay is None) != (dt is None), "recurrence: fixed decays or step sizes")
        for w in (decay, dt_bias, rate, skip):
            _check(w is None or (w.dtype == torch.float32 and w.shape == (H,) and w.is_contiguous()), "recurrence: per-head constants float32 [H]")
        if dt is not None:
            _check(dt.shape == (T, H) and dt.stride(1) == 1 and dt.dtype == dtype and dt_bias is not None and rate is not None,
                   "recurrence: step sizes [T, H] with bias and rates")
        _check(_is_i32(state_slots) and _is_i32(cu_seqlens, B + 1) and len(q_lens) == B, "recurrence: metadata")
        if T == B and N <= RECURRENCE_STEP_MAX_ROWS:
            # every request brings one token: the state streams through once, one output row per token
            y = torch.empty((T, H * P), dtype=torch.float32, device=v.device)
            core().call("me_linear_recurrence", q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0),
                        _code(dtype), _ptr(dt), 0 if dt is None else dt.stride(0), _ptr(decay), _ptr(dt_bias), _ptr(rate), _ptr(skip),
                        state.data_ptr(), state.stride(0), state_slots.data_ptr(), cu_seqlens.data_ptr(), y.data_ptr(), T * H * P,
                        B, H, G, N, P, 0, 1, int(silu), 0, 1, None, _stream())
            return y
        per_wave = recurrence_rows_per_wave(N)
        slices = -(-N // per_wave)
        columns = recurrence_columns(q_lens, H, G, P, slices)
        span, spans = recurrence_spans(q_lens, H * -(-P // 64) * slices // columns, 65535 // slices)
        scratch = _scratch(B * spans * (H * N * P + H), v.device, "recurrence") if spans > 1 else None
        y = torch.empty((slices, T, H * P) if slices > 1 else (T, H * P), dtype=torch.float32, device=v.device)
        core().call("me_linear_recurrence", q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0),
                    _code(dtype), _ptr(dt), 0 if dt is None else dt.stride(0), _ptr(decay), _ptr(dt_bias), _ptr(rate), _ptr(skip),
                    state.data_ptr(), state.stride(0), state_slots.data_ptr(), cu_seqlens.data_ptr(), y.data_ptr(), T * H * P,
                    B, H, G, N, P, per_wave, columns, int(silu), span, spans, _ptr(scratch), _stream())
        return y

    def gated_rms_norm(self, y, gate, weight, eps: float, groups: int, kind: str, out_dtype: torch.dtype) -> torch.Tensor:
        """`kind` "silu_before": u = y * silu(gate), out = u / rms(u) * weight with the root mean square taken over
        each of `groups` equal parts of a row; "sigmoid_behind": out = y / rms(y) * weight * sigmoid(gate); "silu_behind": the
        same with silu(gate). y float32
        [T, n] or slices [S, T, n] that are added first; gate a row view [T, n] of out_dtype. Returns [T, n]."""
        if y.dim() == 3 and y.shape[0] > 64:          # more slices than the kernel adds (a state of thousands of rows)
            y = y.sum(0)
        parts = y.shape[0] if y.dim() == 3 else 1
        T, n = y.shape[-2], y.shape[-1]
        _check(y.dtype == torch.float32 and y.is_contiguous() and kind in GATED_NORMS, "gated_rms_norm: float32 rows, a known kind")
        _check(gate.shape == (T, n) and gate.stride(1) == 1 and gate.dtype == out_dtype, "gated_rms_norm: gate [T, n] of the output dtype")
        _check(weight.dtype == torch.float32 and weight.shape == (n,) and weight.is_contiguous() and n % groups == 0,
               "gated_rms_norm: weight float32 [n], n a multiple of the groups")
        out = torch.empty((T, n), dtype=out_dtype, device=y.device)
        core().call("me_gated_rms_norm", y.data_ptr(), parts, T * n, gate.data_ptr(), gate.stride(0), _code(out_dtype),
                    weight.data_ptr(), out.data_ptr(), T, n, groups, GATED_NORMS[kind], float(eps), _stream())
        return out

    # -- sublayers side by side, attention with biases and whole-projection norms ------------
    def scaled_sum_norm(self, stream, terms, mult: float, w1, w2, eps: float, out_dtype: torch.dtype):
        """stream' = stream + mult * sum_i scale_i * term_i, then y1 = w1 * stream' / rms(stream') and the same with w2,
        one pass. stream: [T, n], float32 or the compute dtype (rows that start a stream); terms: up to four
        (rows [T, n] in the compute dtype or float32 partial sums [P, T, n], scale float32 [n] or None); w1, w2: float32
        [n] or None (w2 only with w1). Returns (stream' float32 [T, n], y1, y2) with y in out_dtype; without terms and
        with a float32 stream, stream' is the stream itself."""
        T, n = stream.shape
        _check(stream.dim() == 2 and stream.is_contiguous(), "scaled_sum_norm: stream must be contiguous [T, n]")
        _check(len(terms) <= 4, "scaled_sum_norm: up to four terms")
        for w in (w1, w2):
            _check(w is None or (w.dtype == torch.float32 and w.shape == (n,) and w.is_contiguous()), "scaled_sum_norm: norm weights float32 [n]")
        _check(w2 is None or w1 is not None, "scaled_sum_norm: a second norm needs the first")
        k = len(terms)
        ptrs, dts, parts, strides, scales = (c_void_p * 4)(), (c_int * 4)(), (c_int * 4)(), (c_int64 * 4)(), (c_void_p * 4)()
        for i, (t, sc) in enumerate(terms):
            _check(t.is_contiguous() and t.shape[-2:] == (T, n) and (t.dim() == 2 or (t.dim() == 3 and t.dtype == torch.float32)),
                   "scaled_sum_norm: a term is rows [T, n] or float32 partial sums [P, T, n]")
            _check(sc is None or (sc.dtype == torch.float32 and sc.shape == (n,) and sc.is_contiguous()), "scaled_sum_norm: scales float32 [n]")
            ptrs[i], dts[i], parts[i], strides[i] = t.data_ptr(), _code(t.dtype), (t.shape[0] if t.dim() == 3 else 1), T * n
            scales[i] = None if sc is None else sc.data_ptr()
        keep = k == 0 and stream.dtype == torch.float32
        new = stream if keep else torch.empty((T, n), dtype=torch.float32, device=stream.device)
        y1 = torch.empty((T, n), dtype=out_dtype, device=stream.device) if w1 is not None else None
        y2 = torch.empty((T, n), dtype=out_dtype, device=stream.device) if w2 is not None else None
        if keep and w1 is None:
            return new, None, None
        core().call("me_scaled_sum_norm", stream.data_ptr(), _code(stream.dtype), k, ptrs, dts, parts, strides, scales, float(mult),
                    None if keep else new.data_ptr(), _ptr(w1), _ptr(w2), _ptr(y1), _ptr(y2), _code(out_dtype), T, n, float(eps), _stream())
        return new, y1, y2

    def softcap_(self, z: torch.Tensor, cap: float) -> torch.Tensor:
        """z <- cap * tanh(z / cap) in place; float32 rows with unit inner stride."""
        _check(z.dim() == 2 and z.dtype == torch.float32 and z.stride(1) == 1, "softcap: float32 rows")
        core().call("me_softcap", z.data_ptr(), z.stride(0), z.shape[0], z.shape[1], float(cap), _stream())
        return z

    def qkv_prepare_store(self, rows, bias, q_weight, k_weight, eps: float, nq: int, nk: int, temperature, positions, slots,
                          k_cache, v_cache, Hq: int, Hkv: int, D: int, page: int, vdim: int, mix: int = 0, lam=None,
                          v_first=None) -> torch.Tensor:
        """The step between a packed q/k/v product and attention, for projections with biases that are normed as a whole.
        rows: float32 [T, (Hq + 2 Hkv) * D], the product's unrounded sums (heads in D slots each, slots beyond a head's
        stored size zero); bias: float32 of that width or None; q_weight [Hq * D], k_weight [Hkv * D]: float32 weights
        of an RMS norm over all of a token's query (key) slots at once, the mean taken over nq (nk) stored dimensions
        (None: no norm); temperature: (coef, every) or None: the query at position p is multiplied by
        1 + coef * ln(floor((p + 1) / every) + 1). mix 1: the first vdim slots of every value head are kept in v_first
        (float32 [T, Hkv * vdim]); mix 2: v <- (1 - lam) v + lam v_first (lam: float32 tensor of one element). Keys and
        values go to the pages at `slots` (K [pages, Hkv, page, D], V [pages, Hkv, D, page]; slots < 0 skipped).
        Returns the queries [T, Hq * D] in the caches' dtype."""
        T = rows.shape[0]
        width = (Hq + 2 * Hkv) * D
        _check(rows.dim() == 2 and rows.dtype == torch.float32 and rows.shape[1] >= width and rows.stride(1) == 1,
               f"qkv_prepare_store: rows must be float32 [T, >= {width}]")
        _check(bias is None or (bias.dtype == torch.float32 and bias.numel() >= width and bias.is_contiguous()), "qkv_prepare_store: bias float32")
        _check((q_weight is None) == (k_weight is None), "qkv_prepare_store: both norm weights or neither")
        if q_weight is not None:
            _check(q_weight.dtype == torch.float32 and q_weight.shape == (Hq * D,) and q_weight.is_contiguous()
                   and k_weight.dtype == torch.float32 and k_weight.shape == (Hkv * D,) and k_weight.is_contiguous(),
                   "qkv_prepare_store: norm weights float32 [Hq * D] and [Hkv * D]")
        _check(_is_i32(positions, T) and _is_i32(slots, T), "qkv_prepare_store: positions and slots int32 [T]")
        _check(k_cache.dtype == v_cache.dtype and k_cache.is_contiguous() and v_cache.is_contiguous()
               and k_cache.shape[1:] == (Hkv, page, D) and v_cache.shape[1:] == (Hkv, D, page),
               "qkv_prepare_store: caches must be K [pages, Hkv, page, D] and V [pages, Hkv, D, page]")
        if mix:
            _check(v_first is not None and v_first.dtype == torch.float32 and v_first.shape == (T, Hkv * vdim) and v_first.stride(1) == 1
                   and 1 <= vdim <= D, "qkv_prepare_store: v_first float32 [T, Hkv * vdim]")
            _check(mix == 1 or (lam is not None and lam.dtype == torch.float32 and lam.numel() == 1), "qkv_prepare_store: lam float32 scalar")
        coef, every = temperature if temperature else (0.0, 0)
        q = torch.empty((T, Hq * D), dtype=k_cache.dtype, device=rows.device)
        core().call("me_qkv_prepare", rows.data_ptr(), rows.stride(0), _ptr(bias), _ptr(q_weight), _ptr(k_weight), float(eps), int(nq),
                    int(nk), float(coef), int(every), positions.data_ptr(), slots.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                    q.data_ptr(), q.stride(0), _code(k_cache.dtype), T, Hq, Hkv, D, page, int(vdim), int(mix),
                    _ptr(lam) if mix == 2 else None, _ptr(v_first) if mix else None, v_first.stride(0) if mix else 0, _stream())
        return q

    # -- two mixers side by side: a recurrence with a decay per state row, and the steps around it -----------
    def add_bias(self, x, bias, out_dtype: torch.dtype) -> torch.Tensor:
        """(x summed over its slices) + bias, rounded once to out_dtype. x: a row view [T, n] or float32 partial sums
        [P, T, n]; bias: float32 [nb], nb <= n (columns beyond nb get none). Returns contiguous [T, n]."""
        parts = x.shape[0] if x.dim() == 3 else 1
        T, n = x.shape[-2], x.shape[-1]
        _check(x.stride(-1) == 1 and (x.dim() == 2 or (x.dtype == torch.float32 and x.is_contiguous())), "add_bias: rows or float32 partial sums")
        _check(bias.dtype == torch.float32 and bias.dim() == 1 and bias.numel() <= n and bias.is_contiguous(), "add_bias: bias float32 [<= n]")
        out = torch.empty((T, n), dtype=out_dtype, device=x.device)
        core().call("me_add_bias", x.data_ptr(), _code(x.dtype), parts, T * n if x.dim() == 3 else 0, x.stride(-2), bias.data_ptr(),
                    bias.numel(), out.data_ptr(), _code(out_dtype), T, n, _stream())
        return out

    def sigmoid_gate_(self, o: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
        """o *= sigmoid(gate), element by element, in place; row views [T, n] of one dtype."""
        T, n = o.shape
        _check(o.dim() == 2 and gate.shape == (T, n) and o.stride(1) == 1 and gate.stride(1) == 1 and gate.dtype == o.dtype,
               "sigmoid_gate: two row views [T, n] of one dtype")
        core().call("me_sigmoid_gate", o.data_ptr(), o.stride(0), gate.data_ptr(), gate.stride(0), _code(o.dtype), T, n, _stream())
        return o

    def glu_clamped(self, gu: torch.Tensor, limit: float, alpha: float) -> torch.Tensor:
        """g = min(gu[:, :I], limit), u = clamp(gu[:, I:], -limit, limit); g * sigmoid(alpha * g) * (u + 1): [T, I]."""
        _check(gu.dim() == 2 and gu.stride(1) == 1 and gu.shape[1] % 2 == 0, "glu_clamped: rows [T, 2 I]")
        T, inter = gu.shape[0], gu.shape[1] // 2
        out = torch.empty((T, inter), dtype=gu.dtype, device=gu.device)
        core().call("me_glu_clamped", gu.data_ptr(), gu.stride(0), out.data_ptr(), _code(gu.dtype), T, inter, float(limit), float(alpha), _stream())
        return out

    def weighted_sum(self, terms, norm_weight=None, eps: float = 0.0, stream=None, out_dtype: torch.dtype | None = None):
        """sum_i scale_i * gate_i * (term_i + bias_i) in float32. terms: up to four (rows [T, n] in the compute dtype or float32
        partial sums [P, T, n], a number, float32 bias [n] or None, and optionally gate rows: a view [T] or [T, 1] in the
        compute dtype or float32 whose sigmoid multiplies the term token by token). Without `norm_weight`: returns the sum, float32
        [T, n]. With it (float32 [n]) and `stream` (float32 [T, n]): the norm on the sum and the residual sum in the same
        pass, stream' = stream + norm_weight * s / sqrt(mean(s^2) + eps); returns (stream' rounded to out_dtype, stream')."""
        k = len(terms)
        _check(1 <= k <= 4, "weighted_sum: one to four terms")
        T, n = terms[0][0].shape[-2:]
        ptrs, dts, parts, strides, scales, biases = (c_void_p * 4)(), (c_int * 4)(), (c_int * 4)(), (c_int64 * 4)(), (c_float * 4)(), (c_void_p * 4)()
        gates, gate_dts, gate_strides = (c_void_p * 4)(), (c_int * 4)(), (c_int64 * 4)()
        for i, term in enumerate(terms):
            t, sc, b = term[:3]
            gate = term[3] if len(term) > 3 else None
            if gate is not None:
                _check(gate.shape[0] == T and gate.numel() == T, "weighted_sum: gate rows hold one number per token")
                gates[i], gate_dts[i], gate_strides[i] = gate.data_ptr(), _code(gate.dtype), gate.stride(0)
            else:
                gates[i], gate_dts[i], gate_strides[i] = None, ME_F32, 0
            _check(t.is_contiguous() and t.shape[-2:] == (T, n) and (t.dim() == 2 or (t.dim() == 3 and t.dtype == torch.float32)),
                   "weighted_sum: a term is rows [T, n] or float32 partial sums [P, T, n]")
            _check(b is None or (b.dtype == torch.float32 and b.shape == (n,) and b.is_contiguous()), "weighted_sum: biases float32 [n]")
            ptrs[i], dts[i], parts[i], strides[i] = t.data_ptr(), _code(t.dtype), (t.shape[0] if t.dim() == 3 else 1), T * n
            scales[i], biases[i] = float(sc), None if b is None else b.data_ptr()
        dev = terms[0][0].device
        if norm_weight is None:
            out = torch.empty((T, n), dtype=torch.float32, device=dev)
            core().call("me_weighted_sum", k, ptrs, dts, parts, strides, scales, biases, out.data_ptr(), None, 0.0, None, None, None, 0, T, n,
                        gates, gate_dts, gate_strides, _stream())
            return out
        _check(norm_weight.dtype == torch.float32 and norm_weight.shape == (n,) and norm_weight.is_contiguous()
               and stream is not None and stream.dtype == torch.float32 and stream.shape == (T, n) and stream.is_contiguous(),
               "weighted_sum: norm weight float32 [n], stream float32 [T, n]")
        new = torch.empty_like(stream)
        rounded = new if out_dtype in (None, torch.float32) else torch.empty((T, n), dtype=out_dtype, device=dev)
        core().call("me_weighted_sum", k, ptrs, dts, parts, strides, scales, biases, None, norm_weight.data_ptr(), float(eps),
                    stream.data_ptr(), new.data_ptr(), None if rounded is new else rounded.data_ptr(),
                    _code(rounded.dtype), T, n, gates, gate_dts, gate_strides, _stream())
        return rounded, new

    def token_shift(self, x, mu, state, state_slots, cu_seqlens, seq_of_token) -> torch.Tensor:
        """out[s, t] = x[t] + (x[t - 1] - x[t]) * mu[s] for every mix s, where x[t - 1] is the row of the request's previous
        token: for the first of a request's tokens in this step, what its state row holds (the step function has zeroed
        it for a request that starts at position 0); the state row then takes the request's last row of this step.
        x: a row view [T, n]; mu: float32 [S, n]; state: a float32 view [slots, n], rows `state_slots`. Returns [S, T, n]
        in x's dtype."""
        T, n = x.shape
        S = mu.shape[0]
        B = state_slots.numel()
        _check(x.stride(1) == 1 and mu.dtype == torch.float32 and mu.shape == (S, n) and mu.is_contiguous(), "token_shift: rows [T, n], mu float32 [S, n]")
        _check(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] == n and state.stride(1) == 1, "token_shift: state float32 [slots, n]")
        _check(_is_i32(state_slots) and _is_i32(cu_seqlens, B + 1) and _is_i32(seq_of_token, T), "token_shift: metadata must be int32")
        out = torch.empty((S, T, n), dtype=x.dtype, device=x.device)
        core().call("me_token_shift", x.data_ptr(), x.stride(0), _code(x.dtype), mu.data_ptr(), S, state.data_ptr(), state.stride(0),
                    state_slots.data_ptr(), cu_seqlens.data_ptr(), seq_of_token.data_ptr(), out.data_ptr(), T, n, _stream())
        return out

    def decay_rows_recurrence(self, q, k, v, raw, state, state_slots, cu_seqlens, q_lens, H: int, G: int, N: int, P: int, rule: str,
                              base, rate=None, bonus=None, beta=None, unit_eps: float | None = None, q_scale: float = 1.0) -> torch.Tensor:
        """Per request and head a float32 state S [N, P] whose rows decay each at a rate the token chooses, walked over
        the request's tokens of this step in order from its state row, which is left at the state behind the last token.
        rule "bonus":  d = exp(-exp(raw + base));  y = (S + diag(bonus) k v^T)^T q;  S <- diag(d) S + k v^T.
        rule "delta":  d = exp(-rate_h softplus(raw + base));  S <- diag(d) S;  u = sigmoid(beta) (v - S^T k);
                       S <- S + k u^T;  y = S^T q.
        rule "gated":  d = sigmoid(raw + base) ^ rate_h;  S <- diag(d) S + k v^T;  y = S^T q.
        q, k: row views [T, G * N] (heads share them by groups of H / G); v: [T, H * P]; raw: [T, H * N]; beta: [T, H];
        base, bonus: float32 [H * N]; rate: float32 [H]. `unit_eps`: q and k are made unit vectors per head first, x /
        sqrt(sum(x^2) + unit_eps); q is multiplied by q_scale. Everything but the rows read is float32. Returns float32
        [T, H * P]. (`q_lens`: the requests' token counts on the host.)"""
        T, B = v.shape[0], state_slots.numel()
        dtype = v.dtype
        _check(rule in DECAY_RULES, f"decay_rows_recurrence: rule must be one of {sorted(DECAY_RULES)}")
        for t, width in ((q, G * N), (k, G * N), (v, H * P), (raw, H * N)):
            _check(t.dim() == 2 and t.shape == (T, width) and t.stride(1) == 1 and t.dtype == dtype, "decay_rows_recurrence: bad q, k, v or decay rows")
        _check(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1 and state.shape[1] == H * N * P,
               "decay_rows_recurrence: state must be float32 [slots, H * N * P]")
        for w, width in ((base, H * N), (bonus, H * N), (rate, H)):
            _check(w is None or (w.dtype == torch.float32 and w.numel() == width and w.is_contiguous()), "decay_rows_recurrence: constants float32")
        _check(base is not None and (bonus is not None if rule == "bonus" else (rate is not None and (beta is not None or rule == "gated"))),
               "decay_rows_recurrence: the rule's constants are missing")
        if beta is not None:
            _check(beta.shape == (T, H) and beta.stride(1) == 1 and beta.dtype == dtype, "decay_rows_recurrence: write strengths [T, H]")
        _check(_is_i32(state_slots) and _is_i32(cu_seqlens, B + 1) and len(q_lens) == B and sum(q_lens) == T, "decay_rows_recurrence: metadata")
        _check(1 <= N <= 256 and H % G == 0, "decay_rows_recurrence: up to 256 state rows, heads a multiple of the groups")
        y = torch.empty((T, H * P), dtype=torch.float32, device=v.device)
        groups, prepared = decay_row_groups(B, H, N, P, max(q_lens))
        NR = 32 if N <= 32 else 64 if N <= 64 else 128 if N <= 128 else 256
        pre = _scratch(3 * T * H * NR + T * H, v.device, "decay_rows") if prepared else None
        core().call("me_decay_rows_recurrence", q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0),
                    raw.data_ptr(), raw.stride(0), _ptr(beta), 0 if beta is None else beta.stride(0), _code(dtype),
                    base.data_ptr(), _ptr(rate), _ptr(bonus), state.data_ptr(), state.stride(0), state_slots.data_ptr(),
                    cu_seqlens.data_ptr(), y.data_ptr(), B, H, G, N, P, DECAY_RULES[rule], int(unit_eps is not None),
                    float(unit_eps or 0.0), float(q_scale), groups, T, _ptr(pre), _stream())
        return y

    # -- routed experts ------------------------------------------------------------------
    def moe_route(self, x, router, top: int, group_count: int = 1, group_keep: int = 1, rule: "RouteRule | None" = None):
        """Which experts each token uses and with what weights. x: [T, n] rows; router: float32 [E, n]. The logits router . x
        are float32. `rule` (a `RouteRule`; None: its defaults) says how they become scores (their softmax over all E
        experts, or a sigmoid each), whether a correction per expert joins the scores for the choice, how a group of
        neighbours scores (the sum of its group_top largest choice scores), and what the weights are (the chosen
        experts' scores without the correction, divided by their sum + 1e-20 or not, times a constant). With
        group_count > 1 only experts of the group_keep best groups can be chosen. The `top` largest choice scores are
        chosen (ties: the lower index). Returns (ids int32 [T, top], weights float32 [T, top])."""
        T, n = x.shape
        E = router.shape[0]
        rule = rule or RouteRule()
        _check(x.stride(1) == 1 and router.dtype == torch.float32 and router.shape == (E, n) and router.is_contiguous(),
               "moe_route: rows [T, n], router float32 [E, n]")
        rule.check(E)
        ids = torch.empty((T, top), dtype=torch.int32, device=x.device)
        weights = torch.empty((T, top), dtype=torch.float32, device=x.device)
        logits = torch.empty((T, E), dtype=torch.float32, device=x.device)
        core().call("me_moe_route", x.data_ptr(), x.stride(0), _code(x.dtype), router.data_ptr(), T, n, E, int(top), int(group_count),
                    int(group_keep), logits.data_ptr(), ids.data_ptr(), weights.data_ptr(), 1, *rule.args(), _stream())
        return ids, weights

    def route_and_run_experts(self, x, router, top: int, group_count: int, group_keep: int, gate_up, down,
                              rule: "RouteRule | None" = None, gated: bool = True) -> torch.Tensor:
        """`moe_route` and `routed_experts` behind it: float32 [top, T, hidden]. For the few tokens `moe_sort_chooses` admits,
        the kernel that orders the pairs by expert makes the choice itself from the router's logits: one launch less in a
        decode step's chain."""
        T, n = x.shape
        E = router.shape[0]
        F = gate_up.shape[1] // 2 if gated else gate_up.shape[1]
        rule = rule or RouteRule()
        if not (moe_sort_chooses(T, E, group_count) and x.dtype == torch.bfloat16 and n % 8 == 0 and F % 8 == 0 and x.stride(0) % 8 == 0
                and x.data_ptr() % 16 == 0):
            ids, weights = self.moe_route(x, router, top, group_count, group_keep, rule)
            return self.routed_experts(x, ids, weights, gate_up, down, gated=gated)
        _check(x.stride(1) == 1 and router.dtype == torch.float32 and router.shape == (E, n) and router.is_contiguous(),
               "moe_route: rows [T, n], router float32 [E, n]")
        rule.check(E)
        ids = torch.empty((T, top), dtype=torch.int32, device=x.device)
        weights = torch.empty((T, top), dtype=torch.float32, device=x.device)
        logits = torch.empty((T, E), dtype=torch.float32, device=x.device)
        core().call("me_moe_route", x.data_ptr(), x.stride(0), _code(x.dtype), router.data_ptr(), T, n, E, int(top), int(group_count),
                    int(group_keep), logits.data_ptr(), ids.data_ptr(), weights.data_ptr(), 0, *rule.args(), _stream())
        return self.routed_experts(x, ids, weights, gate_up, down, choose_from=(logits, group_count, group_keep, rule), gated=gated)

    def routed_experts(self, x, ids, weights, gate_up, down, force_simple: bool = False, tile_rows: int | None = None,
                       choose_from=None, gated: bool = True) -> torch.Tensor:
        """Every token through its chosen experts: out[j, t] = weights[t, j] * W_down[e] (silu(W_gate[e] x_t) * (W_up[e] x_t)),
        e = ids[t, j]: float32 [top, T, hidden], one partial sum per choice for a consumer that adds them. x: [T, K];
        gate_up: [E, 2 F, K] (an expert's gate rows, then its up rows); down: [E, hidden, F]. With `gated` False the experts
        have no gate: gate_up is [E, F, K] (up rows only) and an expert is W_down[e] relu(W_up[e] x_t)^2. bfloat16 with K and F in
        whole steps of 8: the (token, choice) pairs are ordered by expert and cut into tiles that never span two experts, of
        64 rows (a workgroup's 64 x 64 tile of the matrix-core kernel) or, while an expert gets few rows (`expert_tile_rows`;
        `tile_rows` forces it), of 16 rows for the kernel that streams the chosen experts' weights with K cut over a
        workgroup's waves; otherwise (float32, other sizes) one wave per output element."""
        T, K = x.shape
        top = ids.shape[1]
        E, F2, _ = gate_up.shape
        F, N = (F2 // 2 if gated else F2), down.shape[1]
        _check(x.stride(1) == 1 and gate_up.is_contiguous() and down.is_contiguous() and gate_up.shape == (E, (2 if gated else 1) * F, K)
               and down.shape == (E, N, F) and gate_up.dtype == x.dtype and down.dtype == x.dtype, "routed_experts: operand shapes")
        _check(ids.dtype == torch.int32 and ids.is_contiguous() and weights.dtype == torch.float32 and weights.is_contiguous()
               and ids.shape == (T, top) and weights.shape == (T, top), "routed_experts: ids int32 [T, top], weights float32 [T, top]")
        out = torch.empty((top, T, N), dtype=torch.float32, device=x.device)
        Pn = T * top
        act = torch.empty((Pn, F), dtype=x.dtype, device=x.device)
        rows = tile_rows or expert_tile_rows(T, top, E)
        tiled = (x.dtype == torch.bfloat16 and K % 8 == 0 and F % 8 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
                 and not force_simple and Pn // rows + min(E, Pn) <= 65535)
        if not tiled:
            core().call("me_moe_experts_simple", x.data_ptr(), x.stride(0), _code(x.dtype), gate_up.data_ptr(), down.data_ptr(),
                        ids.data_ptr(), weights.data_ptr(), act.data_ptr(), out.data_ptr(), T, top, N, F, K, int(gated), _stream())
            return out
        max_tiles = Pn // rows + min(E, Pn)
        meta = torch.empty((Pn + E + 1 + 2 * max_tiles,), dtype=torch.int32, device=x.device)
        order, offsets = meta[:Pn], meta[Pn:Pn + E + 1]
        tile_expert, tile_row = meta[Pn + E + 1:Pn + E + 1 + max_tiles], meta[Pn + E + 1 + max_tiles:]
        # choose_from (logits, group_count, group_keep, rule): ids and weights are still empty and the sort kernel fills them
        logits, gc, gk, rule = choose_from if choose_from is not None else (None, 1, 1, RouteRule())
        _check(choose_from is None or tiled, "routed_experts: the choice inside the sort kernel needs the tiled path")
        core().call("me_moe_sort", ids.data_ptr(), Pn, E, max_tiles, rows, order.data_ptr(), offsets.data_ptr(), tile_expert.data_ptr(),
                    tile_row.data_ptr(), _ptr(logits), weights.data_ptr(), top, int(gc), int(gk), *rule.args(), _stream())
        core().call("me_moe_gate_up", x.data_ptr(), x.stride(0), gate_up.data_ptr(), order.data_ptr(), offsets.data_ptr(),
                    tile_expert.data_ptr(), tile_row.data_ptr(), act.data_ptr(), T, top, F, K, max_tiles, rows, int(gated), _stream())
        core().call("me_moe_down", act.data_ptr(), down.data_ptr(), order.data_ptr(), offsets.data_ptr(), tile_expert.data_ptr(),
                    tile_row.data_ptr(), weights.data_ptr(), out.data_ptr(), T, top, N, F, max_tiles, rows, _stream())
        return out

    # -- attention over a latent that all heads share ------------------------------------------
    def latent_prepare(self, rows, q_off: int, kv_off: int | None, H: int, dn: int, dr: int, R: int, D: int, norm_weight, eps: float,
                       table, positions, slots, k_cache, v_cache, page: int) -> torch.Tensor:
        """From the rows of a layer's packed product ([T, ...]: H query heads of dn unrotated and dr rotating dimensions from
        column q_off; from column kv_off the latent's R rows and dr rows of a key part that all heads share): the RMS norm
        of the latent with `norm_weight` (float32 [R]), the rotation of the shared key part and of every head's rotating
        query part in adjacent pairs by `table` (float32 [positions, dr / 2, 2]: cos, sin), and the write into the pages at
        `slots`: k_cache [pages, 1, page, D] takes [latent | rotated part | zeros], v_cache [pages, 1, D, page] the latent.
        kv_off None: a layer that reads another layer's pages writes none. Returns the queries' frame [T, H * D] in the
        rows' dtype with slots R .. R + dr of every head filled (the rotated part; zeros behind it): slots 0 .. R wait for
        the queries carried into the latent's space (`heads_linear`)."""
        T = rows.shape[0]
        _check(rows.dim() == 2 and rows.stride(1) == 1 and q_off + H * (dn + dr) <= rows.shape[1], "latent_prepare: rows [T, n], unit inner stride")
        _check(dr % 2 == 0 and D >= R + dr and (dr == 0 or (table is not None and table.dtype == torch.float32 and table.is_contiguous()
               and table.shape[1:] == (dr // 2, 2))), "latent_prepare: the rotation's table must be float32 [positions, dr / 2, 2]")
        _check(_is_i32(positions, T), "latent_prepare: positions must be int32")
        write = kv_off is not None
        if write:
            _check(kv_off + R + dr <= rows.shape[1] and _is_i32(slots, T) and norm_weight.dtype == torch.float32 and norm_weight.shape == (R,)
                   and norm_weight.is_contiguous(), "latent_prepare: slots int32, norm weight float32 [rank]")
            _check(k_cache.shape[1:] == (1, page, D) and v_cache.shape[1:] == (1, D, page) and k_cache.dtype == rows.dtype
                   and v_cache.dtype == rows.dtype, "latent_prepare: cache layout mismatch")
        qa = torch.empty((T, H * D), dtype=rows.dtype, device=rows.device)
        core().call("me_latent_prepare", rows.data_ptr(), rows.stride(0), _code(rows.dtype), int(q_off), int(kv_off or 0), H, dn, dr, R, D,
                    _ptr(norm_weight) if write else None, float(eps), _ptr(table), 0 if table is None else table.shape[0],
                    positions.data_ptr(), slots.data_ptr() if write else None, qa.data_ptr(), qa.stride(0),
                    k_cache.data_ptr() if write else None, v_cache.data_ptr() if write else None, int(page), T, _stream())
        return qa

    def heads_linear(self, x, w, out) -> torch.Tensor:
        """out[t, h, :] = w[h] x[t, h, :]: a product per head. x: a view [T, H, K], w: [H, N, K] contiguous, out: a view [T, H, N],
        all of one dtype; the views' inner strides are 1, their token and head strides are free (heads inside a wider row)."""
        T, H, K = x.shape
        N = w.shape[1]
        _check(w.shape == (H, N, K) and w.is_contiguous() and out.shape == (T, H, N) and x.stride(2) == 1 and out.stride(2) == 1
               and x.dtype == w.dtype == out.dtype, "heads_linear: x [T, H, K], w [H, N, K], out [T, H, N] of one dtype")
        core().call("me_heads_linear", x.data_ptr(), x.stride(0), x.stride(1), w.data_ptr(), out.data_ptr(), out.stride(0), out.stride(1),
                    _code(x.dtype), T, H, N, K, _stream())
        return out

    # -- sampling ------------------------------------------------------------------------
    def sample(self, logits: torch.Tensor, temperatures: torch.Tensor, keys: torch.Tensor) -> torch.Tensor:
        """Token ids int32 [S] from float32 logits [S, V]: argmax where temperature is 0, else
        argmax(logits/T - log E) with E ~ Exp(1) a hash of (keys[s], vocabulary id)
        (reference layers/sampler.py:5-11)."""
        S, V = logits.shape
        _check(logits.dtype == torch.float32 and logits.stride(1) == 1, "sample: logits must be float32 rows")
        _check(temperatures.dtype == torch.float32 and temperatures.numel() == S and temperatures.is_contiguous(),
               "sample: temperatures must be float32 [S]")
        _check(keys.dtype == torch.int32 and keys.shape == (S, 2) and keys.is_contiguous(), "sample: keys must be int32 [S, 2]")
        out = torch.empty((S,), dtype=torch.int32, device=logits.device)
        if S <= SAMPLE_STATIC_MAX_ROWS:
            # the per-chunk partial results stay in a device array of the library: nothing is allocated for them.
            # (All calls on a GPU share that array; the engine samples on one stream, one call after the other.)
            core().call("me_sample_static", logits.data_ptr(), logits.stride(0), temperatures.data_ptr(), keys.data_ptr(),
                        out.data_ptr(), S, V, _stream())
            return out
        scratch = _scratch(2 * S * 32, logits.device, "sample")
        core().call("me_sample", logits.data_ptr(), logits.stride(0), temperatures.data_ptr(), keys.data_ptr(),
                    out.data_ptr(), scratch.data_ptr(), S, V, _stream())
        return out


# Dispatch rules. Every threshold below was measured on one MI355X at the layer sizes of Qwen3-0.6B, 8B and 32B;
# the tables behind each constant are kept in the repository's design notes, one line of reason here.
SKINNY_MAX_M = 32                          # rows up to which the skinny kernel beats the library product
SKINNY_WIDE_MAX_M = 64                     # ... for weights of up to SKINNY_WIDE_MAX_WEIGHT elements
SKINNY_WIDE_MAX_WEIGHT = 5 * 1024 * 1024
PARTIALS_MAX_M = 64                        # rows up to which a product split over K (float32 partial sums) pays
LIBRARY_MIN_N = 32768                      # outputs this wide (the head over the vocabulary) go to the library ...
WIDE_OUTPUT_SKINNY_ROWS = 12               # ... except up to this many rows, where the skinny kernel's wide loads win
LIBRARY_MIN_ROWS = 4                       # large weights go to the library from this many rows on ...
LIBRARY_MIN_ROWS_WIDE = 17                 # ... with the wide loads and K up to 4,096: never within their 16 rows
LIBRARY_MIN_ROWS_WIDE_LONG_K = 11          # ... over a longer K
LIBRARY_MIN_WEIGHT = 15 * 1024 * 1024
LIBRARY_MAX_K = 16384                      # the library's choice for a longer K is poor
ROWS_MIN_WEIGHT = 10 * 1024 * 1024
ROWS_FEW_FEATURES = 3072
PREFILL_SEGMENT_KEYS = None    # None: chosen by prefill_segments(); an int forces that many keys per segment (0: never cut)
# prefill attention, keys and values shared by a workgroup's waves through LDS: 0 never, 1 wherever it fits (written there
# by the loads themselves at head size 128 and pages of 16 keys or more), 2 as 1 but always staged through registers
PREFILL_THROUGH_LDS = 1
PREFILL_COL_TILES = 0     # 0: chosen by prefill_col_tiles(); 1 or 2 force the column tiles per wave
MFMA_WITH_EXTRAS = True        # False: attention with kept first keys, a score cap or sinks always takes the exact kernel
DECODE_AS_PREFILL = False      # True: single-token rows go through the prefill kernel (cross-check of the decode kernel)
USE_MID_PRODUCT = True          # False: products of 33-512 rows over small weights go to the library like the larger ones
MID_MAX_WEIGHT = 8 << 20
MID_SMALL_WEIGHT = 13 << 19     # 6.5 M elements: gate/up at the 0.6B sizes (6.3 M) keeps the own kernel and its gating epilogue
FUSE_GATE_INTO_GATE_UP = True  # False: silu(gate) * up is formed in front of the down product, not behind gate_up
GATED_EPILOGUE_MAX_M = 16
FUSE_NORM_INTO_LINEAR = True   # False: the norm kernel and the product behind it always run as two launches
NORM_FUSE_MAX_M = 2
NORM_FUSE_MAX_WEIGHT = 8 << 20
FUSE_DECODE_STEP = True        # False: pure decode steps run norm/rotation/cache write and attention as two launches
GATED_MAX_K = 4096             # the gating in front of the down product is formed in every workgroup: not over a longer K
GATED_MAX_M = 16
_COMPUTE_UNITS = 256
_DECODE_WORKGROUPS = 4096
_PREFILL_THREE_WAVES_WORKGROUPS = 2048
_DECODE_WHOLE_WORKGROUPS = 768
_DECODE_ONE_ROUND = 768           # workgroups of the decode kernel that run at once: three to a compute unit
_DECODE_WHOLE_MAX_KEYS = 4096
_DECODE_EVEN_WHOLE_WORKGROUPS = 192
_DECODE_EVEN_WHOLE_MAX_KEYS = 8192
_DECODE_MAX_PARTITION = 2048
SAMPLE_STATIC_MAX_ROWS = 1024     # ME_SAMPLE_STATIC_MAX_ROWS of csrc/sampling.h
_scratch_buf: dict = {}
_scratch_retired: list = []      # outgrown buffers stay alive: a captured graph may still write to them


def _scratch(num_floats: int, device, use: str = "decode") -> torch.Tensor:
    """Device memory for a kernel's partial results (4-byte words), kept between calls: one buffer per device
    and use, grown when a call needs more (by half as much again, so that a slowly growing need does not
    allocate at every step), never shrunk."""
    key = (device, use)
    buf = _scratch_buf.get(key)
    if buf is None or buf.numel() < num_floats:
        if buf is not None:
            _scratch_retired.append(buf)
        buf = torch.empty((max(num_floats + num_floats // 2, 1 << 20),), dtype=torch.float32, device=device)
        _scratch_buf[key] = buf
    return buf


def prefill_col_tiles(max_context: int, window: int, num_tokens: int, Hq: int, D: int = 128) -> int:
    """Column tiles (of 16 (token, head) pairs) per wave of the prefill kernel: 2 halves the reads of keys and
    values per product but needs twice the columns per workgroup, so it is for launches with many columns (32,768
    or more: 2,048 tokens of 16 heads), and for portions of 256 tokens or more of a prompt over 4,096 keys or
    more, where each tile walks a long range and `prefill_segments` cuts that range into enough workgroups.
    PREFILL_COL_TILES forces it."""
    if PREFILL_COL_TILES in (1, 2):
        return PREFILL_COL_TILES
    if D > 128:
        return 1
    cols = num_tokens * Hq
    span = min(max_context, window + 256) if window else max_context
    return 2 if cols >= 32768 or (cols >= 4096 and span >= 4096) else 1


def prefill_segments(max_context: int, window: int, num_tokens: int, Hq: int, D: int = 128, col_tiles: int | None = None) -> tuple:
    """(keys per segment, most segments per tile) for the prefill kernel; (0, 1): no cutting.

    A tile's key range grows with its position, and a step with few new tokens over a long context
    gives the kernel few workgroups, each walking the whole context. Cutting the ranges into
    segments of at least 512 keys (1,024 over ranges beyond 4,096), run by different workgroups and merged by a
    second kernel, evens the work out and fills the GPU: two segments for launches of 257 to 640 workgroups; three
    for 129 to 256 when the ranges start short (a prompt from its beginning: tiles of 64 to all keys,
    which thirds balance better than halves) and two when they are all long (a later portion of a
    prompt: twice the workgroups fill the slots evenly); as many as give 768 workgroups below that.
    A portion of a prompt that runs with two column tiles per wave before its launch has 32,768 columns
    (`prefill_col_tiles`) gets segments of 512 to 1,024 keys, as many as give about 512 workgroups.
    PREFILL_SEGMENT_KEYS forces a size."""
    span = min(max_context, window + 256) if window else max_context
    if PREFILL_SEGMENT_KEYS is not None:
        seg = PREFILL_SEGMENT_KEYS
        return (seg, -(-span // seg) + 1) if seg > 0 and span > seg else (0, 1)
    cols = num_tokens * Hq
    if col_tiles is None:
        col_tiles = prefill_col_tiles(max_context, window, num_tokens, Hq, D)
    most_by_memory = (1 << 28) // (cols * (D + 2) * 4) - 1      # the partial results are float32 [tokens, heads, segments + 1, D + 2]: under 256 MB
    if col_tiles == 2 and cols < 32768:
        tiles = -(-cols // 128)
        seg = min(1024, max(512, -(-(-(-span // -(-512 // tiles))) // 32) * 32))
        segs = min(-(-span // seg), most_by_memory)
        if segs <= 1:
            return 0, 1
        seg = -(-(-(-span // segs)) // 32) * 32
        return seg, -(-span // seg) + 1
    workgroups = max(1, cols // (128 if col_tiles == 2 else 64))
    if workgroups > 640:
        segs = 1
    elif workgroups > 256:
        segs = 2
    elif workgroups > 128:
        segs = 3 if 2 * (max_context - num_tokens) < span else 2
    else:
        segs = -(-768 // workgroups)
    segs = min(segs, span // (512 if span <= 4096 else 1024))      # segments of 512 keys or more, 1,024 over long ranges
    segs = min(segs, most_by_memory)
    if segs <= 1:
        return 0, 1
    seg = -(-(-(-span // segs)) // 32) * 32
    return seg, -(-span // seg) + 1


SKINNY_WIDE_MIN_WEIGHT = 1 << 22


def skinny_wide(N: int, K: int) -> int:
    """Whether the skinny product reads a weight [N, K] with its wide loads: a wave's load takes 256 contiguous bytes
    of each of four rows, marked as not to be kept by the caches, and the pieces reach their lanes through LDS. For
    weights of SKINNY_WIDE_MIN_WEIGHT elements or more (the kernel applies them to up to 16 rows and a K in whole
    steps of 128); small weights are over before the mark matters."""
    return 1 if N * K >= SKINNY_WIDE_MIN_WEIGHT else 0


def skinny_takes(M: int, N: int, K: int) -> bool:
    """Whether the skinny kernel (without a split over K) takes an aligned bfloat16 product."""
    rows_ok = M <= SKINNY_MAX_M or (M <= SKINNY_WIDE_MAX_M and N * K <= SKINNY_WIDE_MAX_WEIGHT)
    if N >= LIBRARY_MIN_N:
        rows_ok = M <= WIDE_OUTPUT_SKINNY_ROWS and K % 128 == 0 and skinny_wide(N, K) == 1
    return rows_ok and not library_streams_better(M, N, K)


LIBRARY_SPLIT_MIN_ROWS = 33
LIBRARY_SPLIT_MAX_ROWS = 1024
LIBRARY_SPLIT_MIN_WEIGHT = 10 << 20
LIBRARY_SPLIT_SURE_WEIGHT = 16 << 20


def library_splits(M: int, N: int, K: int) -> int:
    """In how many slices of K the library computes a product whose consumer adds float32 partial sums
    (1: not this way). o and down have few output features and a long K, so the library's plain call
    covers the output with too few tiles to fill the GPU (it has no split over K of its own for these
    shapes); as a strided batch over slices of K it runs the same large-tile kernels on 2-8 times the
    tiles. From 33 rows (below, the skinny and the rows kernel are as fast or faster) to 1,024 (above,
    the tiles suffice and the partial sums, S x M x N x 4 bytes written and read again, cost more than
    the split gains), for weights of 10 M elements or more."""
    if not (LIBRARY_SPLIT_MIN_ROWS <= M <= LIBRARY_SPLIT_MAX_ROWS) or N * K < LIBRARY_SPLIT_MIN_WEIGHT:
        return 1
    if N * K < LIBRARY_SPLIT_SURE_WEIGHT and K < 6144 and M < 128:
        return 1          # the smaller of these weights over a short K: the plain call is ahead below 128 rows
    if rows_has_few_features(M, N, K):
        return 1
    if not library_is_direct():
        return 1
    splits = 8 if M <= 256 else 4 if M <= 512 else 2
    while splits > 1 and (K % (8 * splits) or K // splits < 512):
        splits //= 2
    return splits


def rows_has_few_features(M: int, N: int, K: int) -> bool:
    """33 to 64 rows over a weight of up to ROWS_FEW_FEATURES output features and a K of 8,192 or more (down at the 4B
    sizes): the rows kernel's own split over K is ahead of the library's slices and of its plain call."""
    return 32 < M <= 64 and N <= ROWS_FEW_FEATURES and K >= 8192 and K % 8 == 0 and N * K >= ROWS_MIN_WEIGHT


def rows_takes(M: int, N: int, K: int) -> bool:
    """Whether a product whose consumer adds float32 partial sums goes to the rows kernel (64 features per
    workgroup, the tokens staged once per workgroup in LDS, K split over up to 8 workgroups): large
    weights with 17 to 64 rows, where the skinny kernel reads the tokens again for every 16 features and
    the library streams at 1.7-3.5 TB/s, and from 8 rows on over a K too long for the library that is no multiple
    of 128 (otherwise the skinny kernel's wide loads are ahead up to 16 rows); and 33 to 64 rows over a weight with
    few output features (up to ROWS_FEW_FEATURES) and a K of 8,192 or more, where the library's slices of K are poor."""
    if N * K < ROWS_MIN_WEIGHT or K < 4096 or K % 8 or M > 64:
        return False
    if rows_has_few_features(M, N, K):
        return True       # few output features over a long K: the library's slices have too few tiles here too
    if library_splits(M, N, K) > 1:
        return False
    if M > 16:
        return M <= 32 or K >= 12288
    return M >= 8 and K > LIBRARY_MAX_K and not (K % 128 == 0 and skinny_wide(N, K))


def rows_wide(M: int, N: int, ksplit: int) -> int:
    """Whether the rows kernel reads its weights with the wide loads of the skinny kernel (`skinny_wide`): up to 32
    rows and with two workgroups or more to a compute unit. The pass through LDS lengthens a wave's chain from load
    to product, which other workgroups on the compute unit must fill, and the wave tiles' 17 KB beside 48-64 KB of
    staged tokens leave room for one workgroup only."""
    return 1 if M <= 32 and -(-N // 64) * ksplit >= 2 * _COMPUTE_UNITS else 0


def rows_ksplit(K: int) -> int:
    """The most splits up to 8 that leave no split without one of the K/512 chunks."""
    chunks = -(-K // 512)
    for ks in range(min(8, chunks), 0, -1):
        if (ks - 1) * -(-chunks // ks) < chunks:
            return ks
    return 1


def library_streams_better(M: int, N: int, K: int) -> bool:
    """Whether a product of few rows goes to the library rather than the skinny kernel: every workgroup of the
    skinny kernel reads all of x, which at 8 to 16 rows is as much traffic as a large weight itself."""
    if N * K < LIBRARY_MIN_WEIGHT or K > LIBRARY_MAX_K:
        return False
    if K % 128 == 0 and M <= 16 and skinny_wide(N, K):
        return M >= (LIBRARY_MIN_ROWS_WIDE if K <= 4096 else LIBRARY_MIN_ROWS_WIDE_LONG_K)
    return M >= LIBRARY_MIN_ROWS


def choose_ksplit(M: int, N: int, K: int) -> int:
    """Workgroups over K for a skinny product whose consumer adds float32 partial sums (1: K is not split).

    A product's time goes with the rounds its workgroups make over the 256 compute units, each round as long as
    a workgroup's share of K: rounds(tiles x splits) / splits, plus a little for every further set of partial sums
    that the consumer reads. The split with the least of that is taken, each split keeping 512 of K or more (4
    steps of 128, one per wave); with 256 feature tiles or more only over a K of 4,096 or more, where an uneven
    count (320 tiles: one round and a quarter) costs a quarter of the stream, and only up to 32 rows (beyond, the
    library is level or ahead)."""
    tiles = -(-N // 16) * -(-M // 64)
    if tiles >= _COMPUTE_UNITS and (K < 4096 or M > SKINNY_MAX_M):
        return 1
    best, least = 1, None
    for splits in range(1, 9):
        if splits > 1 and K // splits < 512:
            break
        cost = -(-tiles * splits // _COMPUTE_UNITS) / splits + 0.02 * splits
        if least is None or cost < least - 1e-9:
            best, least = splits, cost
    return best


MID_SLICES_MAX_WEIGHT = 27 << 20


def mid_slices(M: int, N: int, K: int) -> int:
    """In how many slices of K (2, 4 or 8; 1: not so) the tiled kernel of csrc/gemm_mid.hip computes M rows against a
    weight [N, K] as float32 partial sums for a consumer that adds them: o and down of a layer at 33 to a few hundred
    rows. A tile of 64 x 64 is one workgroup, and a compute unit that draws its operands alone gets them slowly, so
    what counts is how many workgroups there are: as many slices as keep tiles x slices within 256 workgroups (two
    slices up to 320), each slice with 8 steps of 64 or more (4 where the workgroups are 128 at most). Where it is
    ahead of the skinny split, the rows kernel and the library's strided batch (us with the norm that adds the slices
    behind, this / those): weights up to 8 M elements with up to 2,048 features (1024 x 3072 at 64 rows in 8 slices
    8.3 / 9.4 in 4); up to 13 M and 2,560 features at up to 256 rows (2048 x 6144 at 64 rows 11.6 / 14.7, 2560 x 4096 at
    128 rows 13.7 / 20.9); up to 27 M and 4,096 features at up to 128 rows (2560 x 9728 at 64 rows 20.1 / 24.7, 4096 x
    4096 at 64 rows 13.4 / 17.2). Beyond (4096 x 12288, 5120 x 5120, 5120 x 17408, more rows) the library's larger tiles
    are level or ahead."""
    weight = N * K
    # from 17 rows over the larger weights (2048 x 6144 at 24 rows 10.2 / 12.0, 2560 x 4096 10.3 / 12.8, 2560 x 9728 17.6 /
    # 20.3 with the rows kernel); over the small ones the skinny kernel's split keeps 17-32 rows (1024 x 2048: 6.8 / 7.2)
    if (not USE_MID_PRODUCT or K % 64 or N % 4 or K < 2048 or M <= (32 if weight <= MID_MAX_WEIGHT else 16)
            or weight > MID_SLICES_MAX_WEIGHT):
        return 1
    if weight <= MID_MAX_WEIGHT:
        if N > 2048 or M > (512 if N <= 1024 else 256):
            return 1
        if M > 256:
            return 4
    elif weight <= 13 << 20:
        if N > 2560 or M > 256:
            return 1
    elif N > 4096 or M > 128:
        return 1
    tiles = -(-N // 64) * -(-M // 64)
    steps = K // 64
    for slices in (8, 4, 2):
        per = -(-steps // slices)                       # steps of a slice; the last may have fewer, none has none
        fills = tiles * slices <= 256 or (slices == 2 and tiles <= 160)
        if fills and (slices - 1) * per < steps and (per >= 8 or (per >= 4 and tiles * slices <= 128)):
            return slices
    return 1


def mid_takes(M: int, N: int, K: int, partials: bool) -> int:
    """Whether the product of M rows against a bfloat16 weight [N, K] goes to the own kernel for a few hundred rows
    (csrc/gemm_mid.hip), and in how many slices of K: 0 no, 1 one result, 2, 4 or 8 float32 partial sums over
    that many slices (only when the consumer adds them, `partials`: `mid_slices`). One result: its time is 7 us
    whatever the row count up to 256 (tiles of 64 x 64, one workgroup to a compute unit), where the library's grows
    with the rows; beyond 8 M weight elements and beyond these row counts the library's larger tiles win."""
    if not USE_MID_PRODUCT or K % 64 or N % 4 or K < 256 or M <= 16:
        return 0
    if partials:
        slices = mid_slices(M, N, K)
        if slices > 1:
            return slices
    if M <= 32:
        return 0
    if N * K > MID_MAX_WEIGHT:
        return 0
    if N * K > MID_SMALL_WEIGHT and M < 128:
        return 0          # the larger of the small weights with few rows: the library's tiles are ahead
    return 1 if M <= 256 else 0


def prefill_waves(max_context: int, num_tokens: int, num_seqs: int, Hq: int, Hkv: int, col_tiles: int, max_segs: int) -> int:
    """Waves per SIMD (2 or 3) of the prefill attention kernel whose loads write LDS themselves (head size 128).

    Three waves of 168 registers where two column tiles per wave are in use, the tiles are left whole, there are
    2,048 workgroups or more, and the prompts start at their beginning (the longest context at most twice the mean
    number of new tokens per sequence): tiles of all lengths are then under way at once and the third wave fills
    the others' waits. Portions over a long prefix, whose tiles are equally long and walk the same keys together,
    run better with two waves and 205 registers, and so do launches of few workgroups."""
    if col_tiles != 2 or max_segs != 1 or num_seqs < 1 or max_context <= 0:
        return 2
    group = max(1, Hq // max(1, Hkv))
    tok_tile = max(1, 128 // group)
    tiles = num_tokens // tok_tile + num_seqs
    if tiles * Hkv < _PREFILL_THREE_WAVES_WORKGROUPS or max_context * num_seqs > 2 * num_tokens:
        return 2
    return 3


_DECODE_PART_SIZES = tuple(range(128, 577, 32)) + tuple(range(640, 1409, 64))


def _decode_partition_cost(base: int, ctx: int, part: int) -> float:
    """What a launch of the split decode kernel costs with partitions of `part` keys, in units of one key's work on a
    compute unit: the keys of the busiest compute unit (its workgroups, each with about 64 keys' worth of work before
    and after its keys; a few workgroups beyond a multiple of the 256 units already make some unit that busy), 80 for
    every block that a wave takes after another (a trip to memory that nothing hides), and 300 for every round of
    workgroups beyond the 768 that run at once. Fitted to 86 launches timed over all sizes (1-32 requests of 300-66,000
    keys, 8 key heads with 2, 4 and 8 query heads each, 2 key heads of 64 channels): the size it puts first is 2 %
    behind the fastest on average (12 % at worst)."""
    parts = -(-ctx // part)
    workgroups = base * parts
    per_unit = workgroups / _COMPUTE_UNITS
    busiest = int(per_unit) + min(1.0, (per_unit - int(per_unit)) * 3) if per_unit > 1 else 1.0
    rounds = -(-workgroups // _DECODE_ONE_ROUND)
    return busiest * (part + 64) + 80 * -(-part // 128) + 300 * (rounds - 1)


def decode_partitions(num_seqs: int, Hq: int, Hkv: int, max_context: int, even: bool = False) -> tuple:
    """(keys per partition, number of partitions) for the split decode kernel.

    A workgroup's 4 waves take the 32-key blocks of its partition in turn, and three workgroups share a compute
    unit: 768 run at once. While there are fewer (sequence, kv head) pairs than compute units, the partition size is
    the one of 128, 160, ... 576, 640, ... 1,408 keys that `_decode_partition_cost` puts first (8 requests of 2,048
    keys: 8 partitions of 256; of 2,070 keys: 11 of 192, 704 workgroups at once, where 17 of 128 keys, 1,088
    workgroups in a round and a third, cost a fifth more; of 8,200 keys: 12 of 704), never more than 64 partitions to
    merge. Beyond that list, and from 256 pairs on: one round of workgroups while the pairs stay below 768, at least
    128 keys (one block per wave) and at most 512, and at most 2,048 keys as long as 64 partitions cover the
    context: a workgroup goes through its keys round by round, so in a batch with a few long contexts among short
    ones the long partitions are what is still running at the end.
    From 768 workgroups on (96 sequences x 8 kv heads) a context up to 2,048 keys (4,096 from 2,048 workgroups
    on) is one partition and needs no reduce kernel. `even` (the contexts are equally long,
    `decode_contexts_even`): from 192 workgroups on, a context up to 8,192 keys is one partition if the workgroups
    then fill the compute units evenly (a multiple of 256: 32 or 64 requests x 8 kv heads; 24 or 48 requests leave
    compute units idle or doubly loaded and run 12-14 % faster in partitions): every workgroup then has the same
    work, none waits for another's partial results and no reduce kernel follows; contexts of different lengths
    gain nothing from it and long ones among short ones lose.
    (The reference's rule: layers/ops.py:44-51, split when sequences x kv heads cannot fill the SMs, 256-key
    partitions.)"""
    col_tiles = (Hq // Hkv + 15) // 16
    base = max(1, num_seqs * Hkv * col_tiles)
    ctx = max(1, max_context)
    if base >= _DECODE_WHOLE_WORKGROUPS and ctx <= (_DECODE_WHOLE_MAX_KEYS if base >= 2048 else _DECODE_WHOLE_MAX_KEYS // 2):
        return -(-ctx // 128) * 128, 1
    if even and base >= _DECODE_EVEN_WHOLE_WORKGROUPS and base % _COMPUTE_UNITS == 0 and ctx <= _DECODE_EVEN_WHOLE_MAX_KEYS:
        return -(-ctx // 128) * 128, 1
    if base < _COMPUTE_UNITS:
        # fewer (request, head block) pairs than compute units: the size that a simple reckoning of the launch's time
        # puts first (sizes beyond the list only where 64 partitions of the largest do not cover the context)
        sizes = [p for p in _DECODE_PART_SIZES if -(-ctx // p) <= 64]
        if sizes:
            part = min(sizes, key=lambda p: (_decode_partition_cost(base, ctx, p), -p))
            return part, max(1, -(-ctx // part))
    if base <= _DECODE_ONE_ROUND:
        # one round of workgroups where the batch allows it
        per = -(-ctx // max(1, _DECODE_ONE_ROUND // base))
        part = min(512, max(128, -(-per // 64) * 64))
        part = max(part, -(-(-(-ctx // 64)) // 128) * 128)          # 64 partitions at most
        return part, max(1, -(-ctx // part))
    want = max(1, -(-_DECODE_WORKGROUPS // base), -(-ctx // _DECODE_MAX_PARTITION))
    want = min(64, want)
    part = max(128, -(-(-(-ctx // want)) // 128) * 128)
    parts = max(1, -(-ctx // part))
    return part, parts


def wide_head_partitions(part: int, parts: int, base: int, max_context: int) -> tuple:
    """`decode_partitions` for head sizes above 128: the decode kernel then has two workgroups to a compute unit (its
    operands of a block need more registers than three leave) and a block costs it more, so more than one round of
    workgroups does not pay: partitions are doubled while more than one workgroup per compute unit remains (64 requests
    of 2,048 keys under one key/value head of 256: 8 partitions of 256 keys 60 us, 4 of 512 34 us; 8 requests keep
    their 16 partitions of 128 keys, 17 us, where 8 of 256 take 25)."""
    while parts > 1 and base * parts > _COMPUTE_UNITS and part < _DECODE_MAX_PARTITION:
        part *= 2
        parts = max(1, -(-max(1, max_context) // part))
    return part, parts


def recurrence_rows_per_wave(N: int) -> int:
    """State rows a wave of the recurrence kernel keeps in registers per lane (16, 32, 48 or 64): all of N up to 48,
    beyond that slices of 32 (or of 48 where they waste fewer rows): four waves to a SIMD then share its LDS reads
    and hide each other's waits, where slices of 64 leave two (a prompt of 2,048 tokens at 16 heads of 128 x 128: 185
    against 221 us; 8,192 tokens: 644 against 698)."""
    if N <= 48:
        return -(-N // 16) * 16
    return min((32, 48), key=lambda r: (-(-N // r) * r - N, r))


def recurrence_columns(q_lens: list, H: int, G: int, P: int, slices: int) -> int:
    """State columns a lane of the recurrence kernel keeps: 1. The kernel also has a form with 2 (two blocks of 64
    columns of one head where P exceeds 64, else the same columns of two neighbouring heads of a group, which needs
    an even number of heads per group): it halves the reads of k and q from LDS per product, but its 256 registers
    leave one wave to a SIMD, and it measured slower at every size tried (a prompt of 2,048 tokens at 16 heads of
    128 x 128: 283 against 222 us; 64 requests decoding: 98 against 54 us). ME_RECURRENCE_COLUMNS=2 forces it, for
    timing one against the other."""
    if RECURRENCE_COLUMNS == 2 and not (P <= 64 and (H // G) % 2):
        return 2
    return 1


import os as _os
RECURRENCE_STEP_MAX_ROWS = 4096     # state rows up to which the single-token kernel's k and q fit its LDS
RECURRENCE_COLUMNS = int(_os.environ.get("ME_RECURRENCE_COLUMNS", "0"))     # 1 or 2 force the columns per lane (for timing one against the other)
RECURRENCE_MIN_SPAN = 64
RECURRENCE_WAVES = 4096        # waves that keep the 256 compute units busy: 16 a unit, 4 a SIMD


def recurrence_spans(q_lens: list, waves_per_request: int, most_spans: int = 8191) -> tuple:
    """(tokens per span, most spans per request) for the recurrence kernel; (0, 1): every request in one pass.

    A request's tokens are a chain, and one pass gives the GPU only requests x heads x slices waves. A long prompt is
    therefore cut into spans that run side by side: each span first from zero, then a walk over the spans' end states
    carries the state on, then each span again from the state before it, which costs the work twice and pays as soon
    as the spans are many. Spans of RECURRENCE_MIN_SPAN tokens or more (shorter ones spend their time on reading and
    writing states), as many as bring the launch to RECURRENCE_WAVES waves, for steps whose longest request has two
    spans or more."""
    longest = max(q_lens, default=0)
    if longest < 2 * RECURRENCE_MIN_SPAN:
        return 0, 1
    total = sum(q_lens)
    want = max(1, RECURRENCE_WAVES // max(1, waves_per_request))        # spans over all requests
    span = max(RECURRENCE_MIN_SPAN, -(-total // want), -(-longest // most_spans))    # a launch holds `most_spans` spans a request
    span = -(-span // 16) * 16
    spans = -(-longest // span)
    return (span, spans) if spans >= 2 else (0, 1)


EXPERT_SKINNY_MAX_ROWS = 24       # mean rows per expert up to which the 16-row tiles of the streaming kernel are taken
EXPERT_LARGE_TILE_ROWS = 160      # ... from which tiles of 128 x 128 are taken


SORT_CHOOSES_MAX_TOKENS = 64


def moe_sort_chooses(T: int, E: int, group_count: int) -> bool:
    """Whether the kernel that orders the (token, choice) pairs also makes the choice: up to SORT_CHOOSES_MAX_TOKENS tokens
    (its one workgroup takes them 16 at a time, a wave each) and as many experts as leave its 16 waves their scratch
    memory."""
    return T <= SORT_CHOOSES_MAX_TOKENS and 16 * (2 * E + group_count) * 4 <= 40 * 1024


def expert_tile_rows(T: int, top: int, E: int) -> int:
    """Rows per tile of the routed experts' kernels: 16 while an expert gets EXPERT_SKINNY_MAX_ROWS rows or fewer on
    average (decode steps and short portions: the step is the stream of the chosen experts' weights, and a tile of 16
    rows reads an expert's weights once per 16 rows with K cut over a workgroup's waves), else 64 (the tiles of the
    matrix-core kernel that stages its operands in LDS), and 128 from EXPERT_LARGE_TILE_ROWS rows per expert on (tiles of
    128 x 128: twice the products per operand read from LDS; below, too many of their rows would be empty)."""
    if T * top <= EXPERT_SKINNY_MAX_ROWS * E:
        return 16
    return 128 if T * top >= EXPERT_LARGE_TILE_ROWS * E else 64


DECAY_PREPARE_MIN_TOKENS = 9      # requests of this many tokens or more: the tokens' values are shaped by a kernel of its own


def decay_row_groups(num_seqs: int, H: int, N: int, P: int, longest: int = 1) -> tuple:
    """(lanes that share a column of the state in `decay_rows_recurrence`, whether a first kernel shapes the tokens' values).
    A request is a chain: the fewer rows a lane walks per token, the shorter the chain's step, at the price of more waves
    and an exchange between lanes. Steps of long requests: the values of all tokens are shaped at once by a kernel of its
    own (unit lengths, decays and their exponentials leave the chain), and 16 lanes share a column while that keeps the
    launch within 16 waves a compute unit, else 4. Short steps shape inside the kernel: 4 lanes where a lane could not
    keep a whole column in registers, or while one lane to a column leaves compute units without a wave; else 1."""
    if longest >= DECAY_PREPARE_MIN_TOKENS:
        return (16 if num_seqs * H * -(-P // 4) <= 16 * _COMPUTE_UNITS else 4), True
    if N > 64:
        return 4, False
    return (4 if num_seqs * H * -(-P // 64) < 2 * _COMPUTE_UNITS and N >= 16 else 1), False


def gated_linear_rows(rows: int, w: torch.Tensor) -> bool:
    """Whether `rows` rows against the packed gate/up weight w [2 I, K] are few enough, and w of a kind, for the
    gating to happen in the product's epilogue: a bfloat16 product that the unsplit skinny kernel takes, up to
    GATED_EPILOGUE_MAX_M rows, or one of 17-256 rows that the tiled kernel for small weights takes (`mid_takes`).
    In front of the down product the gating costs every one of that product's workgroups about 2 us; behind
    gate/up every gate is formed once."""
    if not FUSE_GATE_INTO_GATE_UP or w.dtype != torch.bfloat16 or w.dim() != 2:
        return False
    N, K = w.shape
    # over large weights the library takes the product from a row count on (library_streams_better), and the gating is
    # then a kernel of its own; without the skinny kernel's wide loads (K no multiple of 128) the skinny kernel with the
    # gating in its epilogue is still ahead of the two up to 8 rows over a K of 4,096
    takes = skinny_takes(rows, N, K) or (rows <= 8 and K <= 4096 and N < LIBRARY_MIN_N and rows <= SKINNY_MAX_M)
    aligned = N % 2 == 0 and K % 8 == 0 and w.stride(1) == 1 and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0
    if rows > GATED_EPILOGUE_MAX_M:
        # the kernel for a few hundred rows over a small weight gates in its epilogue too, in place of a kernel of
        # its own behind it; and from 17 rows on, where the skinny kernel would have the product itself
        if not (aligned and N % 8 == 0):
            return False
        if rows <= 32:
            return mid_takes(33, N, K, False) == 1
        return not skinny_takes(rows, N, K) and mid_takes(rows, N, K, False) == 1
    return 1 <= rows and aligned and takes


def gated_linear_fuses(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether `gated_linear` takes rows x [M, K] and the packed gate/up weight w [2 I, K]."""
    return (x.dtype == torch.bfloat16 and x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1] and x.stride(1) == 1
            and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and gated_linear_rows(x.shape[0], w))


def norm_linear_fuses(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether `norm_linear` takes rows x ([M, K], or float32 partial sums [S, M, K]) and weight w: a
    bfloat16 weight that the unsplit skinny kernel would take, one or two rows, a weight of at most
    NORM_FUSE_MAX_WEIGHT elements. Every workgroup forms the normed rows for itself, which costs each about
    2 us; the norm kernel costs 3 us in a chain of decode kernels, so it pays for one and two rows only."""
    if not FUSE_NORM_INTO_LINEAR or w.dtype != torch.bfloat16 or w.dim() != 2 or x.dim() not in (2, 3):
        return False
    S = x.shape[0] if x.dim() == 3 else 1
    M, K = x.shape[-2], x.shape[-1]
    N = w.shape[0]
    if x.dtype not in (torch.float32, torch.bfloat16) or (S > 1 and x.dtype != torch.float32) or S > 8:
        return False
    if not (1 <= M <= NORM_FUSE_MAX_M and K == w.shape[1] and K % 8 == 0 and x.is_contiguous() and w.stride(1) == 1
            and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        return False
    if N * K > NORM_FUSE_MAX_WEIGHT or M * (K + 8) * 2 + 4416 > 64 * 1024:
        return False
    return skinny_takes(M, N, K)


def decode_step_fuses(dtype: torch.dtype, D: int, page: int) -> bool:
    """Whether `decode_step_attention` takes these rows: what the matrix-core attention kernels take."""
    return bool(FUSE_DECODE_STEP and dtype == torch.bfloat16 and D % 16 == 0 and 16 <= D <= 512 and page >= 8
                and page & (page - 1) == 0)


def decode_contexts_even(num_seqs: int, min_context: int, max_context: int) -> bool:
    """Whether the decode kernel may keep each request's work on one XCD (8 requests or more whose
    contexts differ by 5 % at most), or has to spread every request over the XCDs. With all of a request
    on one XCD, the XCD that draws the long contexts finishes last; with equal contexts the spread costs
    1-3 % for the block-table reads that a request's heads no longer share in one L2."""
    return num_seqs >= 8 and min_context > 0 and (max_context - min_context) * 20 <= max_context


# --------------------------------------------------------------------------- dispatch

_backend = None


def backend():
    global _backend
    if _backend is None:
        _require_gpu()
        _backend = HipBackend()
    return _backend


def set_backend(b) -> None:
    """Install another object with HipBackend's methods (tests only); None restores the default."""
    global _backend
    _backend = b


def gather_rows(*a, **k): return backend().gather_rows(*a, **k)
def take_tokens(*a, **k): return backend().take_tokens(*a, **k)
def rms_norm(*a, **k): return backend().rms_norm(*a, **k)
def silu_and_mul(*a, **k): return backend().silu_and_mul(*a, **k)
def qk_norm_rope_store(*a, **k): return backend().qk_norm_rope_store(*a, **k)
def store_kv(*a, **k): return backend().store_kv(*a, **k)
def paged_attention(*a, **k): return backend().paged_attention(*a, **k)
def decode_step_attention(*a, **k): return backend().decode_step_attention(*a, **k)
def linear(*a, **k): return backend().linear(*a, **k)
def silu_mul_linear(*a, **k): return backend().silu_mul_linear(*a, **k)
def norm_linear(*a, **k): return backend().norm_linear(*a, **k)
def gated_linear(*a, **k): return backend().gated_linear(*a, **k)
def sample(*a, **k): return backend().sample(*a, **k)
def add_rms_norm(*a, **k): return backend().add_rms_norm(*a, **k)
def activation(*a, **k): return backend().activation(*a, **k)
def head_gate(*a, **k): return backend().head_gate(*a, **k)
def causal_conv(*a, **k): return backend().causal_conv(*a, **k)
def linear_recurrence(*a, **k): return backend().linear_recurrence(*a, **k)
def gated_rms_norm(*a, **k): return backend().gated_rms_norm(*a, **k)
def scaled_sum_norm(*a, **k): return backend().scaled_sum_norm(*a, **k)
def softcap_(*a, **k): return backend().softcap_(*a, **k)
def qkv_prepare_store(*a, **k): return backend().qkv_prepare_store(*a, **k)
def add_bias(*a, **k): return backend().add_bias(*a, **k)
def sigmoid_gate_(*a, **k): return backend().sigmoid_gate_(*a, **k)
def glu_clamped(*a, **k): return backend().glu_clamped(*a, **k)
def weighted_sum(*a, **k): return backend().weighted_sum(*a, **k)
def token_shift(*a, **k): return backend().token_shift(*a, **k)
def decay_rows_recurrence(*a, **k): return backend().decay_rows_recurrence(*a, **k)
def moe_route(*a, **k): return backend().moe_route(*a, **k)
def routed_experts(*a, **k): return backend().routed_experts(*a, **k)
def route_and_run_experts(*a, **k): return backend().route_and_run_experts(*a, **k)
def latent_prepare(*a, **k): return backend().latent_prepare(*a, **k)
def heads_linear(*a, **k): return backend().heads_linear(*a, **k)
