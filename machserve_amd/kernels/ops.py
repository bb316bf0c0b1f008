"""The one boundary between Python and the HIP libraries (role of ``mach-kernel-sys`` in the
reference, ``crates/mach-kernel-sys/src/hip.rs``): torch tensors own the memory, every
operand is checked on the host against what the kernel and its grid assume, and the raw
pointers go to the ``extern "C"`` entry points on torch's current stream.

There is no fallback: without a GPU or without the libraries, construction raises.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import build

_c_float, _c_void = ctypes.c_float, ctypes.c_void_p


def _c_int(v) -> int:
    """An argument of C type int: ctypes passes a Python int as one by itself (and refuses one that does not
    fit), which spares an object per argument; pointers and floats need their wrappers."""
    return int(v)



class KernelError(RuntimeError):
    pass


def _ptr(t: Optional[torch.Tensor]):
    return _c_void(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """torch's current stream on the current device as a raw handle.  The private accessor costs a
    fraction of a microsecond; ``torch.cuda.current_stream()`` builds an object (several microseconds,
    and a step issues some two hundred launches)."""
    if _raw_stream is not None:
        return _c_void(_raw_stream(torch.cuda.current_device()))
    return _c_void(torch.cuda.current_stream().cuda_stream)


class HipOps:
    """Kernels of one element type: ``torch.bfloat16`` or ``torch.float16`` (serving; the same kernels with the
    other two-byte type, the reference's own fast precision, ``crates/mach-model/src/config.rs:3-11``) or
    ``torch.float32`` (true 32-bit)."""
    ELEMS = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}

    def __init__(self, dtype: torch.dtype, device: str = "cuda:0"):
        if dtype not in self.ELEMS:
            raise KernelError(f"no kernels for element type {dtype}; bfloat16, float16 and float32 are built")
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: the HIP kernels have no CPU fallback")
        self.dtype = dtype
        self.device = torch.device(device)
        self._index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        self.elem = self.ELEMS[dtype]
        self._libs: list = []
        self._core = self._load(build.ensure_library("core", self.elem))
        self._attn = {}
        self._extra: dict = {}  # libraries that only some models need, loaded (and built) when first asked for
        self._cus = torch.cuda.get_device_properties(self._index).multi_processor_count
        # what the library plans for a product depends on its sizes alone: asked once per size
        self._plans: dict = {}

    def _load(self, path: str):
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"cannot load {path}: {e}") from None
        lib.ms_last_error.restype = ctypes.c_char_p
        lib.ms_launch_count.restype = ctypes.c_long
        self._libs.append(lib)
        return lib

    def launch_count(self) -> int:
        """Kernels launched so far by the libraries this object has loaded."""
        return sum(int(lib.ms_launch_count()) for lib in self._libs)

    def _stream(self):
        """torch's current stream on this object's device as a raw handle."""
        if _raw_stream is not None:
            return _c_void(_raw_stream(self._index))
        return _c_void(torch.cuda.current_stream(self.device).cuda_stream)

    def _check(self, lib, rc: int):
        if rc != 0:
            raise KernelError(lib.ms_last_error().decode())

    def _want(self, t: torch.Tensor, dtype, name: str, *shape):
        """The operand is what the kernel assumes: on the GPU, of this type, contiguous, of this shape if one
        is given.  Runs for every operand of every launch, so the good case is a few attribute reads."""
        if not t.is_cuda or t.dtype is not dtype or not t.is_contiguous():
            raise KernelError(f"{name}: expected a contiguous {dtype} GPU tensor, got {t.dtype} on {t.device}"
                              f"{'' if t.is_contiguous() else ' (not contiguous)'}")
        if shape and t.shape != shape:
            raise KernelError(f"{name}: expected shape {tuple(shape)}, got {tuple(t.shape)}")

    def require_sizes(self, what: str, reductions=(), head_dim: Optional[int] = None, norm_width: Optional[int] = None,
                      rotated_row: Optional[int] = None) -> None:
        """Refuses, when a model is put together, sizes that the kernels do not take: a product sums over a
        multiple of 8 elements, a head has a multiple of 16 up to the largest attention tile, a normalised row
        and a row of q, k and v that is rotated and written to the cache fit a block's row buffer."""
        for name, k in reductions:
            if k <= 0 or k % 8:
                raise KernelError(f"{what}: {name} = {k} must be a positive multiple of 8 (the products sum over it in 16-byte chunks)")
        if norm_width is not None and not 0 < norm_width <= self._core.ms_max_norm_width():
            raise KernelError(f"{what}: width {norm_width} is outside what the norm kernel takes (1 to {self._core.ms_max_norm_width()})")
        if rotated_row is not None and not 0 < rotated_row <= self._core.ms_max_rope_row():
            raise KernelError(f"{what}: (heads + 2 x key/value heads) x head size = {rotated_row} is outside what the rotation "
                              f"kernel takes (1 to {self._core.ms_max_rope_row()})")
        if head_dim is not None:
            try:
                build.attention_tile_for(head_dim)
            except build.BuildError as e:
                raise KernelError(f"{what}: {e}") from None

    # ------------------------------------------------------------------ elementwise
    def embed(self, tokens: torch.Tensor, table: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
        T, (V, d) = tokens.numel(), table.shape
        self._want(tokens, torch.int32, "embed tokens", T)
        self._want(table, self.dtype, "embed table")
        x = torch.empty((T, d), dtype=torch.float32, device=table.device)
        self._check(self._core, self._core.ms_embed(_ptr(tokens), _ptr(table), _ptr(x), _c_int(T), _c_int(d), _c_float(scale),
                                                    self._stream()))
        return x

    def feed_tokens(self, tokens: torch.Tensor, sampled: torch.Tensor, rows: torch.Tensor, src: torch.Tensor) -> None:
        """``tokens[rows[i]] = sampled[src[i]]`` where ``rows[i]`` is no negative number: the rows of a step whose
        input the step before it sampled take it on the device."""
        n = rows.numel()
        self._want(tokens, torch.int32, "feed_tokens tokens")
        self._want(sampled, torch.int32, "feed_tokens sampled")
        self._want(rows, torch.int32, "feed_tokens rows", n)
        self._want(src, torch.int32, "feed_tokens src", n)
        self._check(self._core, self._core.ms_feed_tokens(_ptr(tokens), _ptr(sampled), _ptr(rows), _ptr(src), _c_int(n),
                                                          _c_int(tokens.numel()), _c_int(sampled.numel()), self._stream()))

    def rmsnorm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, rows: Optional[torch.Tensor] = None,
                out_f32: bool = False, partials: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Norm of ``x + sum(partials)`` (of its ``rows`` if given).  With ``partials [P, T, d]`` and
        no ``rows`` the sum is also written back into ``x``."""
        T, d = x.shape
        self._want(x, torch.float32, "rmsnorm input")
        self._want(weight, torch.float32, "rmsnorm weight", d)
        n, P = T, 0
        if rows is not None:
            self._want(rows, torch.int32, "rmsnorm rows")
            n = rows.numel()
        if partials is not None:
            P = partials.shape[0]
            self._want(partials, torch.float32, "rmsnorm partial sums", P, T, d)
        out = torch.empty((n, d), dtype=torch.float32 if out_f32 else self.dtype, device=x.device)
        self._check(self._core, self._core.ms_rmsnorm(_ptr(x), _ptr(partials), _c_int(P), _c_int(T), _ptr(rows),
                                                      _ptr(weight), _ptr(out), _c_int(int(out_f32)), _c_int(n), _c_int(d),
                                                      _c_float(eps), self._stream()))
        return out

    def layernorm(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float,
                  rows: Optional[torch.Tensor] = None, out_f32: bool = False, partials: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``(v - mean(v)) / sqrt(mean((v - mean(v))^2) + eps) * weight + bias`` for the rows ``v`` of ``x + sum(partials)``
        (of its ``rows`` if given); with ``partials [P, T, d]`` and no ``rows`` the sum is also written back into ``x``."""
        T, d = x.shape
        self._want(x, torch.float32, "layernorm input")
        self._want(weight, torch.float32, "layernorm weight", d)
        if bias is not None:
            self._want(bias, torch.float32, "layernorm bias", d)
        n, P = T, 0
        if rows is not None:
            self._want(rows, torch.int32, "layernorm rows")
            n = rows.numel()
        if partials is not None:
            P = partials.shape[0]
            self._want(partials, torch.float32, "layernorm partial sums", P, T, d)
        out = torch.empty((n, d), dtype=torch.float32 if out_f32 else self.dtype, device=x.device)
        self._check(self._core, self._core.ms_layernorm(_ptr(x), _ptr(partials), _c_int(P), _c_int(T), _ptr(rows), _ptr(weight),
                                                        _ptr(bias), _ptr(out), _c_int(int(out_f32)), _c_int(n), _c_int(d),
                                                        _c_float(eps), self._stream()))
        return out

    def add_partials(self, x: torch.Tensor, partials: torch.Tensor) -> None:
        """``x += sum(partials)`` in order."""
        T, d = x.shape
        self._want(x, torch.float32, "stream")
        self._want(partials, torch.float32, "partial sums", partials.shape[0], T, d)
        self._check(self._core, self._core.ms_add_partials(_ptr(x), _ptr(partials), _c_int(partials.shape[0]), _c_int(T),
                                                           _c_int(d), self._stream()))

    def rope_kv_write(self, qkv: torch.Tensor, bias: Optional[torch.Tensor], positions: torch.Tensor,
                      inv_freq: Optional[torch.Tensor], slot_map: Optional[torch.Tensor], kpool: Optional[torch.Tensor],
                      vpool: Optional[torch.Tensor], H: int, KV: int, hd: int, page_size: int) -> torch.Tensor:
        """``qkv [P, T, stride]`` are partial sums of the q/k/v projection (see :meth:`linear_split`);
        their sum plus ``bias`` is rotated (q and k) and written (k and v) into the pages.  Returns
        q ``[T, H * hd]`` in the element type."""
        if qkv.dim() == 2:
            qkv = qkv.unsqueeze(0)
        P, T, stride = qkv.shape
        self._want(qkv, torch.float32, "rope qkv")
        self._want(positions, torch.int32, "rope positions", T)
        if bias is not None:
            self._want(bias, torch.float32, "rope bias", stride)
        if inv_freq is not None:
            self._want(inv_freq, torch.float32, "rope inv_freq", hd // 2)
        if slot_map is not None:
            self._want(slot_map, torch.int32, "rope slot_map", T)
            pages = kpool.shape[0]
            self._want(kpool, self.dtype, "key pool", pages, KV, page_size, hd)
            self._want(vpool, self.dtype, "value pool", pages, KV, hd, page_size)
        q = torch.empty((T, H * hd), dtype=self.dtype, device=qkv.device)
        self._check(self._core, self._core.ms_rope_kv_write(
            _ptr(qkv), _c_int(P), _ptr(bias), _c_int(stride), _ptr(positions), _ptr(inv_freq), _ptr(slot_map), _ptr(q),
            _ptr(kpool), _ptr(vpool), _c_int(T), _c_int(H), _c_int(KV), _c_int(hd), _c_int(page_size), self._stream()))
        return q

    def rope_table(self, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
        """Float32 ``[T, hd / 2, 2]``: cosine and sine of ``positions[t] * inv_freq[j]``, as the rotation kernels
        compute them; for :meth:`linear_qkv_rope`."""
        T, half = positions.numel(), inv_freq.numel()
        self._want(positions, torch.int32, "rope table positions", T)
        self._want(inv_freq, torch.float32, "rope table inv_freq", half)
        cs = torch.empty((T, half, 2), dtype=torch.float32, device=inv_freq.device)
        self._check(self._core, self._core.ms_rope_table(_ptr(positions), _ptr(inv_freq), _ptr(cs), _c_int(T), _c_int(half), self._stream()))
        return cs

    def qkv_rope_takes(self, M: int, H: int, KV: int, hd: int, K: int) -> bool:
        """Whether :meth:`linear_qkv_rope` takes this shape (else: :meth:`linear_split` and :meth:`rope_kv_write`)."""
        return bool(self._plan("ms_qkv_rope_takes", M, H, KV, hd, K))

    def linear_qkv_rope(self, a: torch.Tensor, w_qkv: torch.Tensor, bias: Optional[torch.Tensor], rope_cs: torch.Tensor,
                        slot_map: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, H: int, KV: int, hd: int,
                        page_size: int) -> torch.Tensor:
        """The q/k/v projection ``a @ w_qkv.T + bias`` of a step of many rows with the rotation of queries and keys
        (by ``rope_cs`` of :meth:`rope_table`) and the write of keys and values into their pages in the product's own
        epilogue.  Returns q ``[T, H * hd]`` in the element type."""
        M, N, K = self._mm_operands(a, w_qkv, "linear_qkv_rope")
        if N != (H + 2 * KV) * hd:
            raise KernelError(f"linear_qkv_rope: weight of {N} rows for {H} + 2 x {KV} heads of {hd}")
        if bias is not None:
            self._want(bias, torch.float32, "linear_qkv_rope bias", N)
        self._want(rope_cs, torch.float32, "linear_qkv_rope angles", M, hd // 2, 2)
        self._want(slot_map, torch.int32, "linear_qkv_rope slot_map", M)
        pages = kpool.shape[0]
        self._want(kpool, self.dtype, "key pool", pages, KV, page_size, hd)
        self._want(vpool, self.dtype, "value pool", pages, KV, hd, page_size)
        q = torch.empty((M, H * hd), dtype=self.dtype, device=a.device)
        self._check(self._core, self._core.ms_linear_qkv_rope(
            _ptr(a), _ptr(w_qkv), _ptr(bias), _ptr(rope_cs), _ptr(slot_map), _ptr(q), _ptr(kpool), _ptr(vpool), _c_int(M), _c_int(H),
            _c_int(KV), _c_int(hd), _c_int(page_size), _c_int(K), self._stream()))
        return q

    # ------------------------------------------------------------------ matrix products
    def _mm_operands(self, a: torch.Tensor, w: torch.Tensor, what: str):
        self._want(a, self.dtype, f"{what} input")
        self._want(w, self.dtype, f"{what} weight")
        M, K = a.shape
        if w.shape[1] != K:
            raise KernelError(f"{what}: input has {K} columns, weight has {w.shape[1]}")
        return M, w.shape[0], K

    SKINNY_ROWS = 64  # at most this many rows: the weight-streaming kernels

    def _plan(self, what: str, *sizes: int, lib=None) -> int:
        key = (what, sizes)
        v = self._plans.get(key)
        if v is None:
            v = self._plans[key] = int(getattr(lib or self._core, what)(*[_c_int(x) for x in sizes]))
        return v

    def _tiled(self, M: int, N: int, K: int) -> bool:
        """Whether the tiled kernel takes this product: always above SKINNY_ROWS rows; below, where it was
        measured faster (in bfloat16 every large weight from one row on, because its blocks stream the
        weight with several K steps in flight, and smaller ones from 8 to 32 rows on; never in 32-bit)."""
        return M > self.SKINNY_ROWS or bool(self._plan("ms_prefers_tiled", M, N, K))

    def linear_split(self, a: torch.Tensor, w: torch.Tensor, allow_partials: bool = True) -> torch.Tensor:
        """Float32 ``[P, M, N]`` whose sum over P is ``a @ w.T``.  Within one kernel family the cut
        of K depends on N and K only, so the consumer that adds the parts sees the same sums for a row
        whatever else is in the batch; which family runs depends on the number of rows (see
        :meth:`_tiled`), and the two differ in rounding."""
        M, N, K = self._mm_operands(a, w, "linear_split")
        if self._tiled(M, N, K):
            P = self._plan("ms_tiled_partials", M, N, K) if allow_partials else 1
            if P == 1:
                return self.linear(a, w, None, out_f32=True).unsqueeze(0)
            out = torch.empty((P, M, N), dtype=torch.float32, device=a.device)
            self._check(self._core, self._core.ms_linear_split_tiled(_ptr(a), _ptr(w), _ptr(out), _c_int(M), _c_int(N),
                                                                     _c_int(K), self._stream()))
            return out
        P = self._plan("ms_skinny_partials", M, N, K, int(allow_partials))
        out = torch.empty((P, M, N), dtype=torch.float32, device=a.device)
        self._check(self._core, self._core.ms_linear_skinny(_ptr(a), _ptr(w), _ptr(out), _c_int(M), _c_int(N), _c_int(K),
                                                            _c_int(int(allow_partials)), self._stream()))
        return out

    def linear(self, a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
               out_f32: bool = False) -> torch.Tensor:
        """``a @ w.T (+ bias)``; 32-bit output on request (logits)."""
        M, N, K = self._mm_operands(a, w, "linear")
        if not self._tiled(M, N, K) and out_f32 and bias is None:
            return self.linear_split(a, w, allow_partials=False)[0]
        if bias is not None:
            self._want(bias, torch.float32, "linear bias", N)
        out = torch.empty((M, N), dtype=torch.float32 if out_f32 else self.dtype, device=a.device)
        self._check(self._core, self._core.ms_linear(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), _c_int(int(out_f32)),
                                                     _c_int(M), _c_int(N), _c_int(K), self._stream()))
        return out

    def linear_residual(self, a: torch.Tensor, w: torch.Tensor, x: torch.Tensor) -> Optional[torch.Tensor]:
        """``x += a @ w.T`` in the 32-bit residual stream.  When the product is cut along K over several
        blocks (a long K under few rows, or too few tiles to fill the chip) the sum is not added here:
        the float32 partial sums ``[P, M, N]`` are returned for the consumer (the next norm) to fold
        in; otherwise None."""
        M, N, K = self._mm_operands(a, w, "linear_residual")
        self._want(x, torch.float32, "residual stream", M, N)
        if not self._tiled(M, N, K):
            if M > 32 or self._plan("ms_skinny_partials", M, N, K, 1) > 1:
                return self.linear_split(a, w)
            # all of K inside one block: one writer an element, added in the epilogue (up to 32 rows the
            # kernel has registers to ask for the stream's values ahead; beyond, the next norm adds the sum)
            self._check(self._core, self._core.ms_linear_residual_skinny(_ptr(a), _ptr(w), _ptr(x), _c_int(M), _c_int(N),
                                                                         _c_int(K), self._stream()))
            return None
        if self._plan("ms_tiled_partials", M, N, K) > 1:
            return self.linear_split(a, w)
        self._check(self._core, self._core.ms_linear_residual(_ptr(a), _ptr(w), _ptr(x), _c_int(M), _c_int(N), _c_int(K),
                                                              self._stream()))
        return None

    def prenorm_swiglu_takes(self, M: int, N: int, K: int, n_gate_up: int) -> bool:
        """Whether ``x += a @ w.T`` (``w [N, K]``) followed by the gated product of ``rmsnorm(x)`` with an
        interleaved weight of ``n_gate_up`` rows can run as two kernels without a norm between them: the
        first leaves ``x * norm_w`` and the rows' sums of squares beside the sum, the second divides its
        finished sums by the root mean square (:meth:`linear_residual_prenorm`, :meth:`linear_swiglu_scaled`)."""
        return (not self._tiled(M, N, K) and self._plan("ms_skinny_prenorm_parts", M, N, K) > 0
                and bool(self._plan("ms_swiglu_scaled_takes", M, n_gate_up // 2, N)
                         or self._plan("ms_swiglu_scaled_skinny_takes", M, n_gate_up // 2, N)))

    def linear_residual_prenorm(self, a: torch.Tensor, w: torch.Tensor, x: torch.Tensor, norm_w: torch.Tensor):
        """``x += a @ w.T`` in place; returns ``(x * norm_w`` in the element type, float32 ``[parts, M]`` whose sum
        over parts is the rows' sums of squares of ``x``)``."""
        M, N, K = self._mm_operands(a, w, "linear_residual_prenorm")
        self._want(x, torch.float32, "residual stream", M, N)
        self._want(norm_w, torch.float32, "norm weight", N)
        parts = self._plan("ms_skinny_prenorm_parts", M, N, K)
        if parts < 1:
            raise KernelError(f"linear_residual_prenorm: M={M} N={N} K={K} is not taken")
        hn = torch.empty((M, N), dtype=self.dtype, device=a.device)
        ss = torch.empty((parts, M), dtype=torch.float32, device=a.device)
        self._check(self._core, self._core.ms_linear_residual_prenorm_skinny(
            _ptr(a), _ptr(w), _ptr(x), _ptr(norm_w), _ptr(hn), _ptr(ss), _c_int(M), _c_int(N), _c_int(K), self._stream()))
        return hn, ss

    def linear_swiglu_scaled(self, hn: torch.Tensor, row_ss: torch.Tensor, eps: float, w_gate_up: torch.Tensor,
                             intermediate: int, activation: str = "silu") -> torch.Tensor:
        """:meth:`linear_swiglu` of rows ``hn`` that lack their norm's division: both products of a row are
        divided by ``sqrt(sum(row_ss[:, row]) / K + eps)`` before the activation."""
        act = gate_activation_code(activation)
        M, N, K = self._mm_operands(hn, w_gate_up, "linear_swiglu_scaled")
        if N != 2 * ((intermediate + 15) // 16) * 16:
            raise KernelError(f"linear_swiglu_scaled: interleaved weight has {N} rows for intermediate size {intermediate}")
        self._want(row_ss, torch.float32, "linear_swiglu_scaled sums of squares", row_ss.shape[0], M)
        out = torch.empty((M, intermediate), dtype=self.dtype, device=hn.device)
        few_rows = bool(self._plan("ms_swiglu_scaled_skinny_takes", M, intermediate, K))
        fn = self._core.ms_linear_swiglu_scaled_skinny if few_rows else self._core.ms_linear_swiglu_scaled
        self._check(self._core, fn(_ptr(hn), _ptr(row_ss), _c_int(row_ss.shape[0]), _c_float(eps), _ptr(w_gate_up), _ptr(out),
                                   _c_int(M), _c_int(intermediate), _c_int(K), _c_int(act), self._stream()))
        return out

    def linear_swiglu(self, a: torch.Tensor, w_gate_up: torch.Tensor, intermediate: int, activation: str = "silu") -> torch.Tensor:
        """``act(a @ gate.T) * (a @ up.T)`` with gate and up rows interleaved in blocks of 16
        (see :func:`interleave_gate_up`); ``activation`` is one of :data:`GATE_ACTIVATIONS` (SiLU gives the
        method its name)."""
        act = gate_activation_code(activation)
        M, N, K = self._mm_operands(a, w_gate_up, "linear_swiglu")
        if N != 2 * ((intermediate + 15) // 16) * 16:
            raise KernelError(f"linear_swiglu: interleaved weight has {N} rows for intermediate size {intermediate}")
        out = torch.empty((M, intermediate), dtype=self.dtype, device=a.device)
        fn = self._core.ms_linear_swiglu if self._tiled(M, N, K) else self._core.ms_linear_swiglu_skinny
        self._check(self._core, fn(_ptr(a), _ptr(w_gate_up), _ptr(out), _c_int(M), _c_int(intermediate), _c_int(K),
                                   _c_int(act), self._stream()))
        return out

    # ------------------------------------------------------------------ products with the norm folded in
    def norm_folds_into(self, M: int, N: int, K: int, n_partials: int) -> bool:
        """Whether a few-rows product over the stream can apply the stream's RMS norm itself (at most
        16 rows, and a shape the few-rows kernel would take anyway)."""
        return (not self._tiled(M, N, K)
                and bool(self._plan("ms_skinny_norm_takes", M, N, K, n_partials)))

    def _normed_operands(self, x, partials, norm_w, w, what):
        M, K = x.shape
        self._want(x, torch.float32, f"{what} stream", M, K)
        self._want(norm_w, torch.float32, f"{what} norm weight", K)
        self._want(w, self.dtype, f"{what} weight")
        if w.dim() != 2 or w.shape[1] != K:
            raise KernelError(f"{what}: weight {tuple(w.shape)} for a stream of width {K}")
        P = 0
        if partials is not None:
            P = partials.shape[0]
            self._want(partials, torch.float32, f"{what} pending sums", P, M, K)
        x_new = torch.empty_like(x) if P else None
        return M, w.shape[0], K, P, x_new

    def linear_split_normed(self, x: torch.Tensor, partials: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float,
                            w: torch.Tensor):
        """``rmsnorm(x + sum(partials)) @ w.T`` as float32 ``[1, M, N]``, and the stream with the
        pending sums added (a new tensor; None if nothing was pending)."""
        M, N, K, P, x_new = self._normed_operands(x, partials, norm_w, w, "linear_split_normed")
        out = torch.empty((1, M, N), dtype=torch.float32, device=x.device)
        self._check(self._core, self._core.ms_linear_norm_skinny(
            _ptr(x), _ptr(partials), _c_int(P), _c_int(M), _ptr(norm_w), _c_float(eps), _ptr(x_new), _ptr(w), _ptr(out),
            _c_int(M), _c_int(N), _c_int(K), self._stream()))
        return out, x_new

    def linear_swiglu_normed(self, x: torch.Tensor, partials: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float,
                             w_gate_up: torch.Tensor, intermediate: int, activation: str = "silu"):
        """``act(h @ gate.T) * (h @ up.T)`` for ``h = rmsnorm(x + sum(partials))`` (see
        :meth:`linear_swiglu`), and the stream with the pending sums added (or None)."""
        act = gate_activation_code(activation)
        M, N, K, P, x_new = self._normed_operands(x, partials, norm_w, w_gate_up, "linear_swiglu_normed")
        if N != 2 * ((intermediate + 15) // 16) * 16:
            raise KernelError(f"linear_swiglu_normed: interleaved weight has {N} rows for intermediate size {intermediate}")
        out = torch.empty((M, intermediate), dtype=self.dtype, device=x.device)
        self._check(self._core, self._core.ms_linear_swiglu_norm_skinny(
            _ptr(x), _ptr(partials), _c_int(P), _c_int(M), _ptr(norm_w), _c_float(eps), _ptr(x_new), _ptr(w_gate_up), _ptr(out),
            _c_int(M), _c_int(intermediate), _c_int(K), _c_int(act), self._stream()))
        return out, x_new

    # ------------------------------------------------------------------ attention
    def _attention_lib(self, hd: int):
        nd = build.attention_tile_for(hd)
        if nd not in self._attn:
            lib = self._load(build.ensure_library("attention", self.elem, nd))
            self._attn[nd] = (lib, getattr(lib, f"ms_paged_attention_mask_nd{nd}"),
                              getattr(lib, f"ms_attention_rows_per_block_nd{nd}")(),
                              getattr(lib, f"ms_decode_attention_mask_nd{nd}"), getattr(lib, f"ms_attention_key_tile_nd{nd}")(),
                              getattr(lib, f"ms_decode_attention_fused_nd{nd}"))
        return self._attn[nd]

    def attention_rows_per_block(self, hd: int) -> int:
        return self._attention_lib(hd)[2]

    def paged_attention(self, q: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, block_table: torch.Tensor,
                        seq_q_start: torch.Tensor, seq_q_len: torch.Tensor, seq_pos0: torch.Tensor,
                        work: torch.Tensor, H: int, KV: int, hd: int, page_size: int, window: Optional[int],
                        scale: float, max_key_groups: int = 0, key_splits: int = 0, sinks: Optional[torch.Tensor] = None,
                        out_gate: Optional[torch.Tensor] = None, chunk: int = 0, softcap: float = 0.0) -> torch.Tensor:
        """``chunk`` > 0: a row at position p sees only keys from ``floor(p / chunk) * chunk`` on (chunks counted from the
        request's position 0); ``softcap`` > 0: a scaled score s becomes ``softcap * tanh(s / softcap)`` before the softmax.
        ``sinks`` float32 ``[H]``: the softmax's denominator also holds ``exp(sinks[h])``, a term without key or value;
        ``out_gate`` float32 ``[T, H]``: what the output of each (row, head) is multiplied by, in the kernel's last pass.
        ``max_key_groups`` asks for that many groups of waves sharing a block's keys (0: the kernel's
        choice); ``key_splits`` for that many blocks sharing them (0: the library's choice by the number of blocks
        of rows, the step's rows and the width of the block tables), merged by a second kernel."""
        lib, fn = self._attention_lib(hd)[:2]
        T = q.shape[0]
        self._want(q, self.dtype, "attention q", T, H * hd)
        pages = kpool.shape[0]
        self._want(kpool, self.dtype, "key pool", pages, KV, page_size, hd)
        self._want(vpool, self.dtype, "value pool", pages, KV, hd, page_size)
        S = seq_q_start.numel()
        self._want_softmax_extras(sinks, out_gate, T, H)
        self._want(block_table, torch.int32, "block table")
        if block_table.dim() != 2 or block_table.shape[0] != S:
            raise KernelError(f"attention: block table {tuple(block_table.shape)} for {S} requests")
        for t, n in ((seq_q_start, "seq_q_start"), (seq_q_len, "seq_q_len"), (seq_pos0, "seq_pos0")):
            self._want(t, torch.int32, n, S)
        self._want(work, torch.int32, "attention work")
        if work.dim() != 2 or work.shape[1] != 2 or work.shape[0] == 0:
            raise KernelError(f"attention: work list of shape {tuple(work.shape)}")
        out = torch.empty((T, H * hd), dtype=self.dtype, device=q.device)
        nsplit = key_splits or self._plan(f"ms_attention_splits_nd{build.attention_tile_for(hd)}", work.shape[0], KV, T, hd, page_size,
                                          block_table.shape[1], self._reach(window, chunk), lib=lib)
        part_o = part_ml = None
        if nsplit > 1:
            part_o = torch.empty((T, H, nsplit, hd), dtype=torch.float32, device=q.device)
            part_ml = torch.empty((T, H, nsplit, 2), dtype=torch.float32, device=q.device)
        self._check(lib, fn(_ptr(q), _ptr(kpool), _ptr(vpool), _ptr(out), _ptr(block_table), _c_int(block_table.shape[1]),
                            _ptr(seq_q_start), _ptr(seq_q_len), _ptr(seq_pos0), _ptr(work), _c_int(work.shape[0]),
                            _c_int(H), _c_int(KV), _c_int(hd), _c_int(page_size), _c_int(pages), _c_int(window or 0),
                            _c_float(scale), _c_int(max_key_groups), _c_int(T), _c_int(nsplit), _ptr(part_o), _ptr(part_ml),
                            _ptr(sinks), _ptr(out_gate), _c_int(chunk), _c_float(softcap), self._stream()))
        return out

    @staticmethod
    def _reach(window: Optional[int], chunk: int) -> int:
        """How far back a row can see under a window and a chunked mask (0: all the way)."""
        reaches = [r for r in (window or 0, chunk or 0) if r > 0]
        return min(reaches) if reaches else 0

    def _want_softmax_extras(self, sinks, out_gate, T: int, H: int) -> None:
        if sinks is not None:
            self._want(sinks, torch.float32, "attention sinks", H)
        if out_gate is not None:
            self._want(out_gate, torch.float32, "attention output gate", T, H)

    DECODE_MAX_GROUP = 16  # query heads per key/value head the decode kernel takes

    def _decode_splits(self, S: int, KV: int, table_width: int, page_size: int, window: Optional[int], key_tile: int,
                       hd: int = 64) -> int:
        """Blocks sharing a request's keys: as many as stay within one round of the chip, which holds two blocks a CU
        with small heads and one with heads above 64 (measured at head sizes 64 and 128, 1 to 200 requests: a split more
        than that starts a second round of blocks, and every round has the kernel's whole chain of latencies in it: 7B
        heads, 48 requests of 512 keys, 22 us uncut, 31 in two; 0.5B heads, 200 requests, 19 against 25), at least
        four key tiles each."""
        span = table_width * page_size if not window else min(table_width * page_size, window + key_tile)
        tiles = max(1, -(-span // key_tile))
        blocks = self._cus * (2 if hd <= 64 else 1)
        return max(1, min(blocks // (S * KV), -(-tiles // 4), 64))

    def decode_attention_fused(self, qkv: torch.Tensor, bias: Optional[torch.Tensor], inv_freq: Optional[torch.Tensor],
                               slot_map: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor,
                               block_table: torch.Tensor, seq_pos0: torch.Tensor, H: int, KV: int, hd: int,
                               page_size: int, window: Optional[int], scale: float) -> torch.Tensor:
        """Decode attention from the partial sums ``qkv [P, S, stride]`` of the q/k/v projection: bias,
        rotation, cache write and attention over the pages in one launch, the merge of the
        splits in a second."""
        lib, key_tile, fn = self._attention_lib(hd)[0], self._attention_lib(hd)[4], self._attention_lib(hd)[5]
        if qkv.dim() == 2:
            qkv = qkv.unsqueeze(0)
        P, S, stride = qkv.shape
        self._want(qkv, torch.float32, "attention qkv")
        if bias is not None:
            self._want(bias, torch.float32, "attention bias", stride)
        if inv_freq is not None:
            self._want(inv_freq, torch.float32, "attention inv_freq", hd // 2)
        self._want(slot_map, torch.int32, "attention slot_map", S)
        pages = kpool.shape[0]
        self._want(kpool, self.dtype, "key pool", pages, KV, page_size, hd)
        self._want(vpool, self.dtype, "value pool", pages, KV, hd, page_size)
        self._want(block_table, torch.int32, "block table")
        if block_table.dim() != 2 or block_table.shape[0] != S:
            raise KernelError(f"attention: block table {tuple(block_table.shape)} for {S} requests")
        self._want(seq_pos0, torch.int32, "seq_pos0", S)
        if H // KV > self.DECODE_MAX_GROUP:
            raise KernelError(f"decode attention: {H // KV} heads per key/value head, at most {self.DECODE_MAX_GROUP}")
        nsplit = self._decode_splits(S, KV, block_table.shape[1], page_size, window, key_tile, hd)
        out = torch.empty((S, H * hd), dtype=self.dtype, device=qkv.device)
        part_o = part_ml = None
        if nsplit > 1:
            part_o = torch.empty((S, H, nsplit, hd), dtype=torch.float32, device=qkv.device)
            part_ml = torch.empty((S, H, nsplit, 2), dtype=torch.float32, device=qkv.device)
        self._check(lib, fn(_ptr(qkv), _c_int(P), _c_int(stride), _ptr(bias), _ptr(inv_freq), _ptr(slot_map), _ptr(kpool),
                            _ptr(vpool), _ptr(out), _ptr(part_o), _ptr(part_ml), _ptr(block_table),
                            _c_int(block_table.shape[1]), _ptr(seq_pos0), _c_int(S), _c_int(H), _c_int(KV), _c_int(hd),
                            _c_int(page_size), _c_int(window or 0), _c_int(nsplit), _c_float(scale), self._stream()))
        return out

    def decode_attention(self, q: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, block_table: torch.Tensor,
                         seq_pos0: torch.Tensor, H: int, KV: int, hd: int, page_size: int, window: Optional[int],
                         scale: float, sinks: Optional[torch.Tensor] = None, out_gate: Optional[torch.Tensor] = None,
                         chunk: int = 0, softcap: float = 0.0) -> torch.Tensor:
        """Attention of a step in which request ``s`` has the single row ``s`` (``sinks``, ``out_gate``, ``chunk``, ``softcap``: see
        :meth:`paged_attention`).  The keys are cut
        into splits so that the grid fills the chip; how many follows from the number of
        requests and the width of the block table only."""
        lib, _, _, fn, key_tile = self._attention_lib(hd)[:5]
        S = q.shape[0]
        self._want(q, self.dtype, "attention q", S, H * hd)
        self._want_softmax_extras(sinks, out_gate, S, H)
        pages = kpool.shape[0]
        self._want(kpool, self.dtype, "key pool", pages, KV, page_size, hd)
        self._want(vpool, self.dtype, "value pool", pages, KV, hd, page_size)
        self._want(block_table, torch.int32, "block table")
        if block_table.dim() != 2 or block_table.shape[0] != S:
            raise KernelError(f"attention: block table {tuple(block_table.shape)} for {S} requests")
        self._want(seq_pos0, torch.int32, "seq_pos0", S)
        if H // KV > self.DECODE_MAX_GROUP:
            raise KernelError(f"decode attention: {H // KV} heads per key/value head, at most {self.DECODE_MAX_GROUP}")
        nsplit = self._decode_splits(S, KV, block_table.shape[1], page_size, self._reach(window, chunk) or None, key_tile, hd)
        out = torch.empty((S, H * hd), dtype=self.dtype, device=q.device)
        part_o = part_ml = None
        if nsplit > 1:
            part_o = torch.empty((S, H, nsplit, hd), dtype=torch.float32, device=q.device)
            part_ml = torch.empty((S, H, nsplit, 2), dtype=torch.float32, device=q.device)
        self._check(lib, fn(_ptr(q), _ptr(kpool), _ptr(vpool), _ptr(out), _ptr(part_o), _ptr(part_ml), _ptr(block_table),
                            _c_int(block_table.shape[1]), _ptr(seq_pos0), _c_int(S), _c_int(H), _c_int(KV), _c_int(hd),
                            _c_int(page_size), _c_int(window or 0), _c_int(nsplit), _c_float(scale), _ptr(sinks), _ptr(out_gate),
                            _c_int(chunk), _c_float(softcap), self._stream()))
        return out

    # ------------------------------------------------------------------ a branch's output, normalised, into the stream
    def norm_add(self, x: torch.Tensor, partials: torch.Tensor, weight: torch.Tensor, eps: float) -> None:
        """``x += rmsnorm(sum(partials)) * weight``: ``partials`` float32 ``[P, T, d]`` are the sums of a branch's last
        product (see :meth:`linear_split`)."""
        T, d = x.shape
        self._want(x, torch.float32, "norm_add stream")
        self._want(partials, torch.float32, "norm_add sums", partials.shape[0], T, d)
        self._want(weight, torch.float32, "norm_add weight", d)
        self._check(self._core, self._core.ms_norm_add(_ptr(x), _ptr(partials), _c_int(partials.shape[0]), _ptr(weight), _c_int(T),
                                                       _c_int(d), _c_float(eps), self._stream()))

    def softcap(self, logits: torch.Tensor, scale: float, cap: float) -> None:
        """In place ``v = logits * scale``, then ``cap * tanh(v / cap)`` (``cap`` 0: ``v`` as it is)."""
        self._want(logits, torch.float32, "softcap logits")
        self._check(self._core, self._core.ms_softcap(_ptr(logits), ctypes.c_long(logits.numel()), _c_float(scale), _c_float(cap),
                                                      self._stream()))

    # ------------------------------------------------------------------ mixers with state of fixed size
    def _extra_lib(self, kind: str):
        lib = self._extra.get(kind)
        if lib is None:
            lib = self._extra[kind] = self._load(build.ensure_library(kind, self.elem))
        return lib

    def _seq_operands(self, what, seq_q_start, seq_q_len, seq_slot):
        S = seq_q_start.numel()
        for t, n in ((seq_q_start, "seq_q_start"), (seq_q_len, "seq_q_len"), (seq_slot, "seq_slot")):
            self._want(t, torch.int32, f"{what} {n}", S)
        return S

    def recurrent_limits(self) -> dict:
        """The largest sizes the kernels of the mixers with state take."""
        lib = self._extra_lib("recurrent")
        return {"taps": lib.ms_conv_max_taps(), "states": lib.ms_scan_max_states(), "lightning_dim": lib.ms_lightning_max_dim()}

    def causal_conv(self, xz: torch.Tensor, channels: int, weight: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor,
                    seq_q_start: torch.Tensor, seq_q_len: torch.Tensor, seq_slot: torch.Tensor) -> torch.Tensor:
        """``silu(bias + causal convolution)`` per channel of the first ``channels`` columns of ``xz [T, ld]``, a request's
        earlier inputs coming from ``state [slots, taps - 1, channels]`` (float32), which is brought up to date."""
        lib = self._extra_lib("recurrent")
        T, ld = xz.shape
        taps = weight.shape[1]
        self._want(xz, self.dtype, "convolution input")
        self._want(weight, torch.float32, "convolution weight", channels, taps)
        if bias is not None:
            self._want(bias, torch.float32, "convolution bias", channels)
        self._want(state, torch.float32, "convolution state", state.shape[0], max(taps - 1, 1), channels)
        S = self._seq_operands("convolution", seq_q_start, seq_q_len, seq_slot)
        out = torch.empty((T, channels), dtype=self.dtype, device=xz.device)
        self._check(lib, lib.ms_causal_conv(_ptr(xz), _c_int(ld), _ptr(weight), _ptr(bias), _ptr(state), _ptr(seq_q_start),
                                            _ptr(seq_q_len), _ptr(seq_slot), _c_int(S), _ptr(out), _c_int(T), _c_int(channels),
                                            _c_int(taps), self._stream()))
        return out

    SCAN_CHUNK = 64           # tokens of a chunk of the scan
    SCAN_CHUNK_MIN_ROWS = 256  # steps of at least this many rows, half as many a request on average, are cut into chunks

    def selective_scan(self, x: torch.Tensor, xz: torch.Tensor, dbc: torch.Tensor, dt_rank: int, n_states: int, w_dt: torch.Tensor,
                       b_dt: Optional[torch.Tensor], a_log: torch.Tensor, d_skip: Optional[torch.Tensor], state: torch.Tensor,
                       seq_q_start: torch.Tensor, seq_q_len: torch.Tensor, seq_slot: torch.Tensor) -> torch.Tensor:
        """The scan of a Mamba layer over the step's rows.  ``x [T, C]``: the convolved input; ``xz [T, 2 C]``: its second
        half is the gate; ``dbc`` float32 ``[T, dt_rank + 2 n_states]``: step size input, B and C.  Step sizes are
        ``softplus(low @ w_dt + b_dt)`` with ``w_dt [dt_rank, C]``, the projection transposed; ``state`` float32 ``[slots, C, n_states]`` is carried on.  Returns
        ``y * silu(gate)`` ``[T, C]``."""
        lib = self._extra_lib("recurrent")
        T, C = x.shape
        self._want(x, self.dtype, "scan input")
        self._want(xz, self.dtype, "scan gate", T, 2 * C)
        self._want(dbc, torch.float32, "scan step input", T, dt_rank + 2 * n_states)
        self._want(w_dt, torch.float32, "scan step weight (transposed)", dt_rank, C)
        if b_dt is not None:
            self._want(b_dt, torch.float32, "scan step bias", C)
        self._want(a_log, torch.float32, "scan A_log", C, n_states)
        if d_skip is not None:
            self._want(d_skip, torch.float32, "scan D", C)
        self._want(state, torch.float32, "scan state", state.shape[0], C, n_states)
        S = self._seq_operands("scan", seq_q_start, seq_q_len, seq_slot)
        dt = torch.empty((T, C), dtype=torch.float32, device=x.device)
        ldb = dbc.shape[1]
        self._check(lib, lib.ms_dt_softplus(_ptr(dbc), _c_int(ldb), _ptr(w_dt), _ptr(b_dt), _ptr(dt), _c_int(T), _c_int(C),
                                            _c_int(dt_rank), self._stream()))
        y = torch.empty((T, C), dtype=self.dtype, device=x.device)
        z = _c_void(xz.data_ptr() + C * xz.element_size())
        # Long portions are cut into chunks that are walked side by side (each from zero, then each from the state that
        # comes into it): one walk over a long prompt keeps a sixteenth of the chip busy.  The cut follows from the
        # step's rows and requests alone.
        chunk = n_chunks = 0
        carry = csum = None
        if T >= self.SCAN_CHUNK_MIN_ROWS and T // S >= self.SCAN_CHUNK_MIN_ROWS // 2:
            n_chunks = -(-T // self.SCAN_CHUNK)
            if S * n_chunks * C * n_states * 4 <= (256 << 20):
                chunk = self.SCAN_CHUNK
                carry = torch.empty((S, n_chunks, C, n_states), dtype=torch.float32, device=x.device)
                csum = torch.empty((S, n_chunks, C), dtype=torch.float32, device=x.device)
        self._check(lib, lib.ms_selective_scan(_ptr(x), z, _c_int(2 * C), _ptr(dt), _ptr(dbc), _c_int(ldb), _c_int(dt_rank),
                                               _c_int(dt_rank + n_states), _ptr(a_log), _ptr(d_skip), _ptr(state), _ptr(seq_q_start),
                                               _ptr(seq_q_len), _ptr(seq_slot), _c_int(S), _ptr(y), _c_int(T), _c_int(C),
                                               _c_int(n_states), _c_int(chunk), _c_int(n_chunks if chunk else 0), _ptr(carry), _ptr(csum),
                                               self._stream()))
        return y

    LIGHTNING_SEGMENT = 128  # rows of a segment of lightning attention in chunks (a multiple of the chunk of 32)

    def lightning_attention(self, qkvg: torch.Tensor, heads: int, dim: int, vdim: int, decay: torch.Tensor, state: torch.Tensor,
                            seq_q_start: torch.Tensor, seq_q_len: torch.Tensor, seq_slot: torch.Tensor, chunked: bool = False) -> torch.Tensor:
        """Linear attention with a decay per head over the step's rows.  ``qkvg [T, ld]`` holds q ``[heads, dim]``, k
        ``[heads, dim]``, v ``[heads, vdim]`` (and whatever follows) before their SiLU; ``state`` float32
        ``[slots, heads, dim, vdim]`` is carried on.  Returns float32 ``[T, heads * vdim]``.  ``chunked``: a request's rows
        in chunks of 32 on the matrix cores (steps of many rows), else token after token (decoding)."""
        lib = self._extra_lib("recurrent")
        T, ld = qkvg.shape
        self._want(qkvg, self.dtype, "lightning q/k/v")
        self._want(decay, torch.float32, "lightning decay", heads)
        self._want(state, torch.float32, "lightning state", state.shape[0], heads, dim, vdim)
        S = self._seq_operands("lightning", seq_q_start, seq_q_len, seq_slot)
        o = torch.empty((T, heads * vdim), dtype=torch.float32, device=qkvg.device)
        if chunked and self._plan("ms_lightning_chunked_takes", dim, vdim, lib=lib):
            # long portions in segments that are walked side by side (see selective_scan); the cut follows from the step's
            # rows and requests alone
            seg = n_segs = 0
            carry = None
            if T >= 2 * self.LIGHTNING_SEGMENT and T // S >= self.LIGHTNING_SEGMENT:
                n_segs = -(-T // self.LIGHTNING_SEGMENT)
                if S * n_segs * heads * dim * vdim * 4 <= (256 << 20):
                    seg = self.LIGHTNING_SEGMENT
                    carry = torch.empty((S, n_segs, heads, dim, vdim), dtype=torch.float32, device=qkvg.device)
            self._check(lib, lib.ms_lightning_chunked(
                _ptr(qkvg), _c_int(ld), _c_int(0), _c_int(heads * dim), _c_int(2 * heads * dim), _ptr(decay), _ptr(state), _ptr(seq_q_start),
                _ptr(seq_q_len), _ptr(seq_slot), _c_int(S), _ptr(o), _c_int(T), _c_int(heads), _c_int(dim), _c_int(vdim), _c_int(seg),
                _c_int(n_segs if seg else 0), _ptr(carry), self._stream()))
            return o
        self._check(lib, lib.ms_lightning(_ptr(qkvg), _c_int(ld), _c_int(0), _c_int(heads * dim), _c_int(2 * heads * dim), _ptr(decay),
                                          _ptr(state), _ptr(seq_q_start), _ptr(seq_q_len), _ptr(seq_slot), _c_int(S), _ptr(o),
                                          _c_int(T), _c_int(heads), _c_int(dim), _c_int(vdim), self._stream()))
        return o

    def gated_rmsnorm(self, o: torch.Tensor, gate_of: torch.Tensor, gate_col: int, weight: torch.Tensor, eps: float) -> torch.Tensor:
        """``rmsnorm(o) * weight * sigmoid(gate)`` in the element type; the gate is columns ``gate_col`` onwards of
        ``gate_of [T, ld]``."""
        lib = self._extra_lib("recurrent")
        T, n = o.shape
        self._want(o, torch.float32, "gated norm input")
        self._want(gate_of, self.dtype, "gated norm gate")
        if gate_of.shape[0] != T or gate_col < 0 or gate_col + n > gate_of.shape[1]:
            raise KernelError(f"gated norm: gate columns {gate_col}..{gate_col + n} of {tuple(gate_of.shape)} for {T} rows")
        self._want(weight, torch.float32, "gated norm weight", n)
        out = torch.empty((T, n), dtype=self.dtype, device=o.device)
        gate = _c_void(gate_of.data_ptr() + gate_col * gate_of.element_size())
        self._check(lib, lib.ms_gated_rmsnorm(_ptr(o), gate, _c_int(gate_of.shape[1]), _ptr(weight), _ptr(out), _c_int(T), _c_int(n),
                                              _c_float(eps), self._stream()))
        return out

    # ------------------------------------------------------------------ attention whose heads exchange scores
    def talking_limits(self) -> dict:
        return {"row": self._extra_lib("talking").ms_talking_max_row()}

    def talking_prepare(self, qkv: torch.Tensor, q_norm: Optional[torch.Tensor], k_norm: Optional[torch.Tensor], eps: float,
                        positions: torch.Tensor, inv_freq: Optional[torch.Tensor], rot: int, cs_factor: float,
                        v_other: Optional[torch.Tensor], v_lambda: Optional[torch.Tensor], keep_values: bool, slot_map: torch.Tensor,
                        kpool: torch.Tensor, vpool: torch.Tensor, H: int, KV: int, d: int, dv: int, page_size: int):
        """Finishes the rows of a q/k/v product given as float32 partial sums ``[P, T, stride]`` (q ``[H, d]``, k
        ``[KV, d]``, v ``[KV, dv]``): RMS norm over the whole of q and of k (weights ``q_norm``, ``k_norm``; None: no
        norm), rotation of the first ``rot`` numbers of every head by ``positions * inv_freq`` with cosines and sines
        times ``cs_factor``, values blended as ``(1 - v_lambda) v + v_lambda v_other``, keys and values written to their
        pages.  Returns ``(q [T, H * d]`` in the element type, the rows' own values float32 ``[T, KV * dv]`` before the
        blend if ``keep_values`` else None)``."""
        lib = self._extra_lib("talking")
        if qkv.dim() == 2:
            qkv = qkv.unsqueeze(0)
        P, T, stride = qkv.shape
        self._want(qkv, torch.float32, "attention rows")
        if q_norm is not None:
            self._want(q_norm, torch.float32, "query norm weight", H * d)
        if k_norm is not None:
            self._want(k_norm, torch.float32, "key norm weight", KV * d)
        self._want(positions, torch.int32, "attention positions", T)
        if inv_freq is not None:
            self._want(inv_freq, torch.float32, "attention inv_freq", rot // 2)
        if v_other is not None:
            self._want(v_other, torch.float32, "values to blend with", T, KV * dv)
            self._want(v_lambda, torch.float32, "blend weight")
        self._want(slot_map, torch.int32, "attention slot_map", T)
        pages = kpool.shape[0]
        self._want(kpool, self.dtype, "key pool", pages, KV, page_size, d)
        self._want(vpool, self.dtype, "value pool", pages, KV, dv, page_size)
        q = torch.empty((T, H * d), dtype=self.dtype, device=qkv.device)
        v_raw = torch.empty((T, KV * dv), dtype=torch.float32, device=qkv.device) if keep_values else None
        self._check(lib, lib.ms_talking_prepare(
            _ptr(qkv), _c_int(P), _c_int(stride), _ptr(q_norm), _ptr(k_norm), _c_float(eps), _ptr(positions), _ptr(inv_freq), _c_int(rot),
            _c_float(cs_factor), _ptr(v_other), _ptr(v_lambda), _ptr(v_raw), _ptr(slot_map), _ptr(q), _ptr(kpool), _ptr(vpool), _c_int(T),
            _c_int(H), _c_int(KV), _c_int(d), _c_int(dv), _c_int(page_size), self._stream()))
        return q, v_raw

    TILE_MIN_ROWS = 8  # a step of at least this many rows that is not plain decoding runs in tiles of 16 rows

    def talking_tile_takes(self, H: int, KV: int, d: int, dv: int, page_size: int) -> bool:
        """Whether the kernel that takes 16 rows a block on the matrix cores is built for these sizes."""
        return bool(self._plan("ms_talking_tile_takes", H, KV, d, dv, page_size, lib=self._extra_lib("talking")))

    def talking_attention(self, q: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, talk: Optional[torch.Tensor],
                          block_table: torch.Tensor, seq_q_start: torch.Tensor, seq_pos0: torch.Tensor, H: int, KV: int, d: int, dv: int,
                          page_size: int, window: Optional[int], keep_first: int, scale: float,
                          seq_q_len: Optional[torch.Tensor] = None, tiles: bool = False) -> torch.Tensor:
        """Attention of every row over the keys it sees: the last ``window`` positions up to its own (None: all) and
        the request's first ``keep_first``.  ``talk`` float32 ``[H, H]`` mixes the heads' scaled scores before the
        softmax (None: no exchange).  Returns ``[T, H * dv]`` in the element type.  ``tiles``: 16 rows a block, for steps
        of many rows a request; else one row a block, for decoding.  With ``seq_q_len`` and sizes it takes, the kernel on
        the matrix cores runs either way; else the kernels of the vector units (one row a block)."""
        lib = self._extra_lib("talking")
        T = q.shape[0]
        self._want(q, self.dtype, "attention q", T, H * d)
        pages = kpool.shape[0]
        self._want(kpool, self.dtype, "key pool", pages, KV, page_size, d)
        self._want(vpool, self.dtype, "value pool", pages, KV, dv, page_size)
        if talk is not None:
            self._want(talk, torch.float32, "head exchange", H, H)
        S = seq_q_start.numel()
        self._want(block_table, torch.int32, "block table")
        if block_table.dim() != 2 or block_table.shape[0] != S:
            raise KernelError(f"attention: block table {tuple(block_table.shape)} for {S} requests")
        self._want(seq_q_start, torch.int32, "seq_q_start", S)
        self._want(seq_pos0, torch.int32, "seq_pos0", S)
        out = torch.empty((T, H * dv), dtype=self.dtype, device=q.device)
        if self.talking_tile_takes(H, KV, d, dv, page_size) and seq_q_len is not None:
            # On the matrix cores: tiles of 16 rows for steps of many rows a request; for single decoded rows a block a
            # row (a tile with one live query: the rows belong to different requests, which a tile takes one after the
            # other).  Too few tiles to fill the chip: several blocks share a tile's keys (at least four 32-key tiles each).
            self._want(seq_q_len, torch.int32, "seq_q_len", S)
            tile_rows = 16 if tiles else 1
            span = block_table.shape[1] * page_size
            key_tiles = -(-span // 32) if not window else min(-(-span // 32), -(-window // 32) + 2 + -(-keep_first // 32))
            n_split = max(1, min(8 if tiles else 16, (2 * self._cus) // -(-T // tile_rows), key_tiles // 4))
            part_o = part_ml = None
            if n_split > 1:
                part_o = torch.empty((T, n_split, H * dv), dtype=torch.float32, device=q.device)
                part_ml = torch.empty((T, n_split, H, 2), dtype=torch.float32, device=q.device)
            self._check(lib, lib.ms_talking_attention_tiles(
                _ptr(q), _ptr(kpool), _ptr(vpool), _ptr(talk), _ptr(block_table), _c_int(block_table.shape[1]), _ptr(seq_q_start),
                _ptr(seq_q_len), _ptr(seq_pos0), _c_int(S), _ptr(out), _c_int(T), _c_int(H), _c_int(KV), _c_int(d), _c_int(dv),
                _c_int(page_size), _c_int(window or 0), _c_int(keep_first), _c_float(scale), _c_int(n_split), _ptr(part_o), _ptr(part_ml),
                _c_int(tile_rows), self._stream()))
            return out
        if self._plan("ms_talking_split_takes", H, KV, d, dv, page_size, lib=lib):
            # blocks that share a row's keys, as many as fill the chip: how many follows from the step's rows and the
            # most 64-position tiles a row can see (its window and first tokens, or the width of the block tables)
            span = block_table.shape[1] * page_size
            tiles = -(-span // 64) if not window else min(-(-span // 64), -(-window // 64) + 1 + -(-keep_first // 64))
            n_split = max(1, min(tiles, -(-2 * self._cus // T), 64))
            part_o = part_ml = None
            if n_split > 1:
                part_o = torch.empty((T, n_split, H * dv), dtype=torch.float32, device=q.device)
                part_ml = torch.empty((T, n_split, H, 2), dtype=torch.float32, device=q.device)
            self._check(lib, lib.ms_talking_attention_split(
                _ptr(q), _ptr(kpool), _ptr(vpool), _ptr(talk), _ptr(block_table), _c_int(block_table.shape[1]), _ptr(seq_q_start),
                _ptr(seq_pos0), _c_int(S), _ptr(out), _c_int(T), _c_int(H), _c_int(KV), _c_int(d), _c_int(dv), _c_int(page_size),
                _c_int(window or 0), _c_int(keep_first), _c_float(scale), _c_int(n_split), _ptr(part_o), _ptr(part_ml), self._stream()))
            return out
        self._check(lib, lib.ms_talking_attention(
            _ptr(q), _ptr(kpool), _ptr(vpool), _ptr(talk), _ptr(block_table), _c_int(block_table.shape[1]), _ptr(seq_q_start),
            _ptr(seq_pos0), _c_int(S), _ptr(out), _c_int(T), _c_int(H), _c_int(KV), _c_int(d), _c_int(dv), _c_int(page_size),
            _c_int(window or 0), _c_int(keep_first), _c_float(scale), self._stream()))
        return out

    # ------------------------------------------------------------------ attention through a latent
    def latent_limits(self) -> dict:
        return {"row": self._extra_lib("latent").ms_latent_max_row()}

    def latent_rows(self, proj: torch.Tensor, q_norm: torch.Tensor, c_norm: Optional[torch.Tensor], eps: float, positions: torch.Tensor,
                    inv_freq: Optional[torch.Tensor], cs_factor: float, slot_map: Optional[torch.Tensor], kpool: Optional[torch.Tensor],
                    vpool: Optional[torch.Tensor], q_rank: int, rank: int, rot: int, page_size: int, halves: bool = False) -> Optional[torch.Tensor]:
        """Finishes the rows of the down projections given as float32 partial sums ``[P, T, stride]`` (query latent
        ``[q_rank]``, then, if the layer writes a cache (``c_norm`` given), latent ``[rank]`` and key part ``[rot]``): RMS
        norm with weight of the query latent, returned ``[T, q_rank up to a multiple of 8]`` in the element type (zeros behind); RMS norm with weight of the
        latent, written as columns ``0 .. rank`` of the row's key and as the row's value; the key part rotated in pairs
        ``(2i, 2i + 1)`` (with ``halves``: ``(i, i + rot / 2)``) by ``positions * inv_freq`` with cosines and sines times
        ``cs_factor``, written behind it.  ``q_rank`` 0: the rows hold no query latent, and nothing is returned."""
        lib = self._extra_lib("latent")
        if proj.dim() == 2:
            proj = proj.unsqueeze(0)
        P, T, stride = proj.shape
        self._want(proj, torch.float32, "latent rows")
        if q_rank:
            self._want(q_norm, torch.float32, "query latent norm weight", q_rank)
        elif c_norm is None:
            raise KernelError("latent rows: neither a query latent nor a cache to write")
        hd = 0
        if c_norm is not None:
            self._want(c_norm, torch.float32, "latent norm weight", rank)
            self._want(positions, torch.int32, "latent positions", T)
            if rot:
                self._want(inv_freq, torch.float32, "latent inv_freq", rot // 2)
            self._want(slot_map, torch.int32, "latent slot_map", T)
            pages, _, _, hd = kpool.shape
            self._want(kpool, self.dtype, "latent key pool", pages, 1, page_size, hd)
            self._want(vpool, self.dtype, "latent value pool", pages, 1, hd, page_size)
        cq = torch.empty((T, -(-q_rank // 8) * 8), dtype=self.dtype, device=proj.device) if q_rank else None
        self._check(lib, lib.ms_latent_rows(_ptr(proj), _c_int(P), _c_int(stride), _ptr(q_norm), _ptr(c_norm), _c_float(eps),
                                            _ptr(positions), _ptr(inv_freq), _c_float(cs_factor), _ptr(slot_map), _ptr(cq),
                                            _c_int(cq.shape[1] if q_rank else 0), _ptr(kpool), _ptr(vpool), _c_int(T), _c_int(q_rank), _c_int(rank), _c_int(rot), _c_int(hd),
                                            _c_int(page_size), _c_int(int(halves)), self._stream()))
        return cq

    def latent_query(self, q: torch.Tensor, positions: torch.Tensor, inv_freq: Optional[torch.Tensor], cs_factor: float, H: int, d: int,
                     rot: int, rank: int, hd: int, halves: bool = False):
        """From the up-projected queries ``q`` float32 ``[T, H * (d + rot)]``: ``(plain [T, H, dp], att [T, H, hd])`` in the
        element type, ``dp`` = ``d`` rounded up to 8.  ``plain`` holds the heads' first ``d`` numbers; ``att``, the queries
        of the attention over the latent cache, has its columns ``rank .. rank + rot`` set to the rotated rest and zeros
        behind; its first ``rank`` columns are left for the per-head product to fill."""
        lib = self._extra_lib("latent")
        T = q.shape[0]
        self._want(q, torch.float32, "latent queries", T, H * (d + rot))
        self._want(positions, torch.int32, "latent positions", T)
        if rot:
            self._want(inv_freq, torch.float32, "latent inv_freq", rot // 2)
        dp = -(-d // 8) * 8
        plain = torch.empty((T, H, dp), dtype=self.dtype, device=q.device)
        att = torch.empty((T, H, hd), dtype=self.dtype, device=q.device)
        self._check(lib, lib.ms_latent_query(_ptr(q), _ptr(positions), _ptr(inv_freq), _c_float(cs_factor), _ptr(plain), _ptr(att),
                                             _c_int(T), _c_int(H), _c_int(d), _c_int(dp), _c_int(rot), _c_int(rank), _c_int(hd),
                                             _c_int(int(halves)), self._stream()))
        return plain, att

    def sigmoid_rows(self, sums: torch.Tensor) -> torch.Tensor:
        """``sigmoid(sums)`` of float32 sums, float32: a gate per row and head."""
        lib = self._extra_lib("latent")
        self._want(sums, torch.float32, "gate sums")
        out = torch.empty_like(sums)
        self._check(lib, lib.ms_sigmoid_rows(_ptr(sums), _ptr(out), ctypes.c_long(sums.numel()), self._stream()))
        return out

    def heads_linear(self, a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """A product per head: ``out[t, b, :N] = w[b] @ a[t, b, :]`` for ``a [T, B, K]`` and ``w [B, N, K]``.  ``out``
        ``[T, B, >= N]`` receives the result in its first ``N`` columns of every head (None: a new ``[T, B, N]``)."""
        lib = self._extra_lib("latent")
        T, B, K = a.shape
        self._want(a, self.dtype, "heads_linear input")
        self._want(w, self.dtype, "heads_linear weight", B, w.shape[1], K)
        N = w.shape[1]
        if out is None:
            out = torch.empty((T, B, N), dtype=self.dtype, device=a.device)
        self._want(out, self.dtype, "heads_linear output", T, B, out.shape[2])
        if out.shape[2] < N:
            raise KernelError(f"heads_linear: output heads of {out.shape[2]} columns for {N}")
        self._check(lib, lib.ms_heads_linear(_ptr(a), ctypes.c_long(B * K), ctypes.c_long(K), _ptr(w), _ptr(out),
                                             ctypes.c_long(B * out.shape[2]), ctypes.c_long(out.shape[2]), _c_int(T), _c_int(B), _c_int(N),
                                             _c_int(K), self._stream()))
        return out

    # ------------------------------------------------------------------ attention behind a short convolution
    def conv_rows_limits(self) -> dict:
        lib = self._extra_lib("convattn")
        return {"row": lib.ms_conv_rows_max_row(), "taps": lib.ms_conv_rows_max_taps()}

    def conv_rows(self, proj: torch.Tensor, conv_w: Optional[torch.Tensor], state: Optional[torch.Tensor], seq_q_start: torch.Tensor,
                  seq_q_len: torch.Tensor, seq_slot: torch.Tensor, positions: torch.Tensor, unit_norm: bool, eps: float,
                  temp_coef: float, temp_every: int, values_are_keys: bool, gated: bool, slot_map: torch.Tensor, kpool: torch.Tensor,
                  vpool: torch.Tensor, H: int, KV: int, d: int, page_size: int):
        """Finishes the rows of a projection given as float32 partial sums ``[P, T, stride]`` (q ``[H, d]``, k ``[KV, d]``,
        then with ``gated`` one gate column per head): causal convolution per channel with ``conv_w [(H + KV) * d, taps]``
        over the request's earlier rows (``state [slots, taps - 1, (H + KV) * d]``, brought up to date; None: no
        convolution), unit norm per head, the queries' temperature ``1 + temp_coef ln(floor((p + 1) / temp_every) + 1)``,
        keys (and with ``values_are_keys`` the keys before their norm as values) written to their pages.  Returns
        ``(q [T, H * dp]`` in the element type with ``dp`` the pools' head size, ``sigmoid(gate)`` float32 ``[T, H]`` or None)``."""
        lib = self._extra_lib("convattn")
        if proj.dim() == 2:
            proj = proj.unsqueeze(0)
        P, T, stride = proj.shape
        C = (H + KV) * d
        self._want(proj, torch.float32, "conv rows")
        taps = 1
        if conv_w is not None:
            taps = conv_w.shape[1]
            self._want(conv_w, torch.float32, "convolution weight", C, taps)
            if taps > 1:
                self._want(state, torch.float32, "convolution state", state.shape[0], taps - 1, C)
            else:
                state = None
        S = self._seq_operands("conv rows", seq_q_start, seq_q_len, seq_slot)
        self._want(positions, torch.int32, "conv rows positions", T)
        self._want(slot_map, torch.int32, "conv rows slot_map", T)
        pages, _, _, dp = kpool.shape
        self._want(kpool, self.dtype, "key pool", pages, KV, page_size, dp)
        self._want(vpool, self.dtype, "value pool", pages, KV, dp, page_size)
        q = torch.empty((T, H * dp), dtype=self.dtype, device=proj.device)
        gate = torch.empty((T, H), dtype=torch.float32, device=proj.device) if gated else None
        self._check(lib, lib.ms_conv_rows(_ptr(proj), _c_int(P), _c_int(stride), _ptr(conv_w), _c_int(taps), _ptr(state), _ptr(seq_q_start),
                                          _ptr(seq_q_len), _ptr(seq_slot), _c_int(S), _ptr(positions), _c_int(int(unit_norm)), _c_float(eps),
                                          _c_float(temp_coef), _c_int(temp_every), _c_int(int(values_are_keys)), _ptr(slot_map), _ptr(q),
                                          _ptr(kpool), _ptr(vpool), _ptr(gate), _c_int(T), _c_int(H), _c_int(KV), _c_int(d), _c_int(dp),
                                          _c_int(page_size), self._stream()))
        return q, gate

    # ------------------------------------------------------------------ branches that end in a norm of their own
    def norm_add_bias(self, x: torch.Tensor, partials: torch.Tensor, bias: Optional[torch.Tensor], weight: torch.Tensor, eps: float) -> None:
        """``x += rmsnorm(sum(partials) + bias) * weight``: :meth:`norm_add` for a product that has a bias."""
        if bias is None:
            return self.norm_add(x, partials, weight, eps)
        T, d = x.shape
        self._want(x, torch.float32, "norm_add stream")
        self._want(partials, torch.float32, "norm_add sums", partials.shape[0], T, d)
        self._want(bias, torch.float32, "norm_add bias", d)
        self._want(weight, torch.float32, "norm_add weight", d)
        self._check(self._core, self._core.ms_norm_add_bias(_ptr(x), _ptr(partials), _c_int(partials.shape[0]), _ptr(bias), _ptr(weight),
                                                            _c_int(T), _c_int(d), _c_float(eps), self._stream()))

    def pair_norm_add(self, x: torch.Tensor, pa: torch.Tensor, wa: torch.Tensor, pb: torch.Tensor, wb: torch.Tensor, weight: torch.Tensor,
                      eps: float) -> None:
        """``y = (rmsnorm(sum(pa)) * wa + rmsnorm(sum(pb)) * wb) / 2;  x += rmsnorm(y) * weight``: two branches side by side,
        each given as the float32 partial sums ``[P, T, d]`` of its last product."""
        T, d = x.shape
        self._want(x, torch.float32, "pair_norm_add stream")
        self._want(pa, torch.float32, "pair_norm_add sums", pa.shape[0], T, d)
        self._want(pb, torch.float32, "pair_norm_add sums", pb.shape[0], T, d)
        for w in (wa, wb, weight):
            self._want(w, torch.float32, "pair_norm_add weight", d)
        self._check(self._core, self._core.ms_pair_norm_add(_ptr(x), _ptr(pa), _c_int(pa.shape[0]), _ptr(wa), _ptr(pb), _c_int(pb.shape[0]),
                                                            _ptr(wb), _ptr(weight), _c_int(T), _c_int(d), _c_float(eps), self._stream()))

    def gate_mul(self, sums: torch.Tensor, activation: str) -> torch.Tensor:
        """``act(sums[:, :n]) * sums[:, n:]`` in the element type for float32 ``sums [T, 2 n]``: the gated product of a
        feed-forward whose gate and up projections carry biases."""
        T, n2 = sums.shape
        self._want(sums, torch.float32, "gate_mul sums")
        if n2 % 2:
            raise KernelError(f"gate_mul: {n2} columns are not a gate and an up half")
        out = torch.empty((T, n2 // 2), dtype=self.dtype, device=sums.device)
        self._check(self._core, self._core.ms_gate_mul(_ptr(sums), _ptr(out), _c_int(T), _c_int(n2 // 2), _c_int(gate_activation_code(activation)),
                                                       self._stream()))
        return out

    def round_rows(self, x: torch.Tensor) -> torch.Tensor:
        """The 32-bit stream in the element type (a copy in the 32-bit build): the input of a branch that reads the stream as it is."""
        self._want(x, torch.float32, "round_rows stream")
        out = torch.empty(x.shape, dtype=self.dtype, device=x.device)
        self._check(self._core, self._core.ms_round_rows(_ptr(x), _ptr(out), ctypes.c_long(x.numel()), self._stream()))
        return out

    def embed_pair(self, tokens: torch.Tensor, table: torch.Tensor, pairs: torch.Tensor, prev: torch.Tensor, seq_q_start: torch.Tensor,
                   seq_q_len: torch.Tensor, seq_pos0: torch.Tensor, seq_slot: torch.Tensor, mul_prev: int, mul_cur: int, buckets: int) -> torch.Tensor:
        """``table[token] + pairs[(previous * mul_prev + token * mul_cur) mod buckets]`` (row ``buckets`` for a request's
        first token) as float32 rows; the token before a portion's first row is what ``prev [slots]`` holds, and the
        portion's last token is left there."""
        T, (V, d) = tokens.numel(), table.shape
        self._want(tokens, torch.int32, "embed tokens", T)
        self._want(table, self.dtype, "embed table")
        self._want(pairs, self.dtype, "embed pair table", buckets + 1, d)
        self._want(prev, torch.int32, "embed previous tokens")
        S = self._seq_operands("embed", seq_q_start, seq_q_len, seq_slot)
        self._want(seq_pos0, torch.int32, "embed seq_pos0", S)
        x = torch.empty((T, d), dtype=torch.float32, device=table.device)
        L = ctypes.c_long
        self._check(self._core, self._core.ms_embed_pair(_ptr(tokens), _ptr(table), _ptr(pairs), _ptr(prev), _ptr(seq_q_start), _ptr(seq_q_len),
                                                         _ptr(seq_pos0), _ptr(seq_slot), _c_int(S), _ptr(x), _c_int(T), _c_int(d), L(mul_prev),
                                                         L(mul_cur), L(buckets), self._stream()))
        return x

    # ------------------------------------------------------------------ q, k and v finished from 32-bit rows
    def finish_rows(self, rows: torch.Tensor, q_norm: Optional[torch.Tensor], k_norm: Optional[torch.Tensor], eps: float,
                    positions: torch.Tensor, inv_freq: Optional[torch.Tensor], rot: int, neighbours: bool, slot_map: torch.Tensor,
                    kpool: torch.Tensor, vpool: torch.Tensor, H: int, KV: int, d: int, dv: int, page_size: int,
                    queries_only: bool = False) -> torch.Tensor:
        """``queries_only``: the rows hold q alone and nothing is written to the pools, which belong to another layer.
        ``rows`` float32 ``[T, >= H d + KV d + KV dv]`` hold q, k and v: an RMS norm over all of q and one over all of k
        (weights; None: none), the rotation of the first ``rot`` numbers of every head of q and k by ``position * inv_freq``
        (pairs of neighbours, or ``(i, i + rot / 2)``), k and v written into their pages.  Returns q ``[T, H * dp]`` in the
        element type, ``dp`` the pools' head size (zeros beyond ``d``)."""
        lib = self._extra_lib("convattn")
        T, stride = rows.shape
        self._want(rows, torch.float32, "finish rows")
        if q_norm is not None:
            self._want(q_norm, torch.float32, "query norm weight", H * d)
        if k_norm is not None:
            self._want(k_norm, torch.float32, "key norm weight", KV * d)
        self._want(positions, torch.int32, "finish rows positions", T)
        if inv_freq is not None:
            self._want(inv_freq, torch.float32, "rotation frequencies", rot // 2)
        else:
            rot = 0
        self._want(slot_map, torch.int32, "finish rows slot_map", T)
        pages, _, _, dp = kpool.shape
        self._want(kpool, self.dtype, "key pool", pages, KV, page_size, dp)
        self._want(vpool, self.dtype, "value pool", pages, KV, dp, page_size)
        q = torch.empty((T, H * dp), dtype=self.dtype, device=rows.device)
        self._check(lib, lib.ms_finish_rows(_ptr(rows), _c_int(stride), _ptr(q_norm), _ptr(k_norm), _c_float(eps), _ptr(positions),
                                            _ptr(inv_freq), _c_int(rot), _c_int(int(neighbours)), _ptr(slot_map), _ptr(q), _ptr(kpool),
                                            _ptr(vpool), _c_int(T), _c_int(H), _c_int(0 if queries_only else KV), _c_int(d), _c_int(dv), _c_int(dp),
                                            _c_int(page_size), self._stream()))
        return q

    def diff_combine(self, o: torch.Tensor, gate: torch.Tensor, lam: float, eps: float, factor: float, H: int, KV: int, hd: int, dv: int,
                     out_cols: int) -> torch.Tensor:
        """Differential attention behind the attention kernel.  ``o [T, 2 H hd]`` in the element type holds two maps a head,
        ordered (key/value head, map, head of the group); a head's result is ``map0 - lam map1`` over its first ``dv``
        numbers, divided by its root mean square (``eps``), times ``factor`` and ``sigmoid(gate)`` (float32 ``[T, H dv]``).
        Heads side by side, ``[T, out_cols]`` in the element type with zeros behind ``H dv``."""
        lib = self._extra_lib("convattn")
        T = o.shape[0]
        self._want(o, self.dtype, "diff_combine maps", T, 2 * H * hd)
        self._want(gate, torch.float32, "diff_combine gate", T, H * dv)
        out = torch.empty((T, out_cols), dtype=self.dtype, device=o.device)
        self._check(lib, lib.ms_diff_combine(_ptr(o), _ptr(gate), _ptr(out), _c_float(lam), _c_float(eps), _c_float(factor), _c_int(T), _c_int(H),
                                             _c_int(KV), _c_int(hd), _c_int(dv), _c_int(out_cols), self._stream()))
        return out

    # ------------------------------------------------------------------ linear recurrences with gates that depend on the token
    def linrec_limits(self) -> dict:
        lib = self._extra_lib("linrec")
        return {"taps": lib.ms_linrec_max_taps(), "wkv_dim": lib.ms_wkv_max_dim(), "lru_block": lib.ms_lru_max_block()}

    def conv_sums(self, sums: torch.Tensor, col0: int, channels: int, bias_in: Optional[torch.Tensor], weight: torch.Tensor,
                  bias_out: Optional[torch.Tensor], state: Optional[torch.Tensor], seq_q_start: torch.Tensor, seq_q_len: torch.Tensor,
                  seq_slot: torch.Tensor) -> torch.Tensor:
        """A causal convolution per channel over a projection given as float32 partial sums ``[P, T, N]`` (columns ``col0``
        onwards, plus ``bias_in``): ``out[t] = bias_out + sum_k weight[:, k] u[t - (taps - 1 - k)]``, the inputs before a
        request's rows of this step from ``state [slots, taps - 1, channels]``, which is brought up to date.  Float32 ``[T, channels]``."""
        lib = self._extra_lib("linrec")
        if sums.dim() == 2:
            sums = sums.unsqueeze(0)
        P, T, N = sums.shape
        self._want(sums, torch.float32, "conv_sums input")
        taps = weight.shape[1]
        self._want(weight, torch.float32, "conv_sums weight", channels, taps)
        for b in (bias_in, bias_out):
            if b is not None:
                self._want(b, torch.float32, "conv_sums bias", channels)
        if taps > 1:
            self._want(state, torch.float32, "conv_sums state", state.shape[0], taps - 1, channels)
        else:
            state = None
        S = self._seq_operands("conv_sums", seq_q_start, seq_q_len, seq_slot)
        out = torch.empty((T, channels), dtype=torch.float32, device=sums.device)
        self._check(lib, lib.ms_conv_sums(_ptr(sums), _c_int(P), ctypes.c_long(T * N), _c_int(N), _c_int(col0), _ptr(bias_in), _ptr(weight),
                                          _ptr(bias_out), _ptr(state), _ptr(seq_q_start), _ptr(seq_q_len), _ptr(seq_slot), _c_int(S), _ptr(out),
                                          _c_int(channels), _c_int(0), _c_int(T), _c_int(channels), _c_int(taps), self._stream()))
        return out

    def lru_gates(self, u: torch.Tensor, wa_t: torch.Tensor, wi_t: torch.Tensor, ba: torch.Tensor, bi: torch.Tensor, lam: torch.Tensor,
                  factor: float):
        """Gates of the real-gated linear recurrent unit from ``u`` float32 ``[T, C]``: per block of channels
        ``r = sigmoid(Wa u + ba)``, ``i = sigmoid(Wi u + bi)`` (weights transposed, ``[blocks, in, out]``), ``a = exp(-factor r
        softplus(lam))``; returns float32 ``(a, sqrt(1 - a^2) i u)``."""
        lib = self._extra_lib("linrec")
        T, C = u.shape
        blocks, bw, _ = wa_t.shape
        self._want(u, torch.float32, "lru input")
        self._want(wa_t, self.dtype, "lru gate weight", blocks, bw, bw)
        self._want(wi_t, self.dtype, "lru gate weight", blocks, bw, bw)
        if blocks * bw != C:
            raise KernelError(f"lru_gates: {blocks} blocks of {bw} for {C} channels")
        for v in (ba, bi, lam):
            self._want(v, torch.float32, "lru gate vector", C)
        a = torch.empty((T, C), dtype=torch.float32, device=u.device)
        drive = torch.empty((T, C), dtype=torch.float32, device=u.device)
        self._check(lib, lib.ms_lru_gates(_ptr(u), _ptr(wa_t), _ptr(wi_t), _ptr(ba), _ptr(bi), _ptr(lam), _c_float(factor), _ptr(a), _ptr(drive),
                                          _c_int(T), _c_int(C), _c_int(blocks), self._stream()))
        return a, drive

    def lru_scan(self, a: torch.Tensor, drive: torch.Tensor, y: torch.Tensor, ycol: int, y_bias: Optional[torch.Tensor], state: torch.Tensor,
                 seq_q_start: torch.Tensor, seq_q_len: torch.Tensor, seq_slot: torch.Tensor) -> torch.Tensor:
        """``S <- a S + drive`` token after token from ``state [slots, C]`` (brought up to date);
        returns ``S * gelu_tanh(y[:, ycol : ycol + C] + y_bias)`` in the element type."""
        lib = self._extra_lib("linrec")
        T, C = a.shape
        self._want(a, torch.float32, "lru decay")
        self._want(drive, torch.float32, "lru drive", T, C)
        self._want(y, self.dtype, "lru gate branch")
        if y.shape[0] != T or ycol < 0 or ycol + C > y.shape[1]:
            raise KernelError(f"lru_scan: gate branch {tuple(y.shape)} for {T} rows of {C} channels at column {ycol}")
        if y_bias is not None:
            self._want(y_bias, torch.float32, "lru gate branch bias", C)
        self._want(state, torch.float32, "lru state", state.shape[0], C)
        S = self._seq_operands("lru_scan", seq_q_start, seq_q_len, seq_slot)
        out = torch.empty((T, C), dtype=self.dtype, device=a.device)
        seg, n_segs = self._walk_segments(T, S, self.LRU_SEGMENT, 2 * C)
        carry = torch.empty((S, n_segs, 2, C), dtype=torch.float32, device=a.device) if seg else None
        self._check(lib, lib.ms_lru_scan(_ptr(a), _ptr(drive), _ptr(y), _c_int(y.shape[1]), _c_int(ycol), _ptr(y_bias), _ptr(state),
                                         _ptr(seq_q_start), _ptr(seq_q_len), _ptr(seq_slot), _c_int(S), _ptr(out), _c_int(C),
                                         _c_int(seg), _c_int(n_segs), _ptr(carry), self._stream()))
        return out

    LRU_SEGMENT = 64  # rows of a segment of the gated recurrence
    WKV_SEGMENT = 32  # and of time mixing, whose walk does more a row

    def _walk_segments(self, T: int, S: int, seg: int, floats_per_segment: int) -> tuple:
        """``(segment length, segments a request)`` for a recurrence over a step of ``T`` rows in ``S`` requests, or ``(0, 0)``:
        long portions are cut into segments that are walked side by side (each from zero, then each from the state that
        comes into it), since one walk over a long prompt keeps a small part of the chip busy.  The cut follows from
        the step's rows and requests alone."""
        if T < self.SCAN_CHUNK_MIN_ROWS or T // S < self.SCAN_CHUNK_MIN_ROWS // 2:
            return 0, 0
        n_segs = -(-T // seg)
        while S * n_segs * floats_per_segment * 4 > (256 << 20) and n_segs > 1:
            seg *= 2
            n_segs = -(-T // seg)
        return (seg, n_segs) if n_segs > 1 else (0, 0)

    def shift_mix(self, x: torch.Tensor, prev: torch.Tensor, mu: torch.Tensor, seq_q_start: torch.Tensor, seq_q_len: torch.Tensor,
                  seq_slot: torch.Tensor) -> torch.Tensor:
        """``out[m, t] = x[t] + (x[t - 1] - x[t]) * mu[m]`` in the element type for float32 rows ``x [T, d]``; the row before a
        request's first row of the step is ``prev [slots, d]``, which then takes the request's last row."""
        lib = self._extra_lib("linrec")
        T, d = x.shape
        M = mu.shape[0]
        self._want(x, torch.float32, "shift_mix rows")
        self._want(prev, torch.float32, "shift_mix previous rows", prev.shape[0], d)
        self._want(mu, torch.float32, "shift_mix weights", M, d)
        S = self._seq_operands("shift_mix", seq_q_start, seq_q_len, seq_slot)
        out = torch.empty((M, T, d), dtype=self.dtype, device=x.device)
        self._check(lib, lib.ms_shift_mix(_ptr(x), _ptr(prev), _ptr(mu), _c_int(M), _ptr(seq_q_start), _ptr(seq_q_len), _ptr(seq_slot), _c_int(S),
                                          _ptr(out), _c_int(T), _c_int(d), self._stream()))
        return out

    def tanh_rows(self, sums: torch.Tensor) -> torch.Tensor:
        """``tanh`` of float32 sums, in the element type."""
        lib = self._extra_lib("linrec")
        self._want(sums, torch.float32, "tanh_rows sums")
        out = torch.empty(sums.shape, dtype=self.dtype, device=sums.device)
        self._check(lib, lib.ms_tanh_rows(_ptr(sums), _ptr(out), ctypes.c_long(sums.numel()), self._stream()))
        return out

    def wkv(self, r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gate: torch.Tensor, z: torch.Tensor, w0: torch.Tensor, u: torch.Tensor,
            norm_w: torch.Tensor, eps: float, state: torch.Tensor, seq_q_start: torch.Tensor, seq_q_len: torch.Tensor, seq_slot: torch.Tensor,
            heads: int, dim: int) -> torch.Tensor:
        """Time mixing with a decay per key channel and token, per head from ``state [slots, heads, dim, dim]``:
        ``o = (S + diag(u) k v^T)^T r``, ``S <- diag(exp(-exp(z + w0))) S + k v^T``; returns
        ``o / rms(o) * norm_w * silu(gate)`` (the root mean square per head) in the element type."""
        lib = self._extra_lib("linrec")
        T, n = r.shape
        if n != heads * dim:
            raise KernelError(f"wkv: rows of {n} for {heads} heads of {dim}")
        for t, name in ((r, "r"), (k, "k"), (v, "v"), (gate, "gate")):
            self._want(t, self.dtype, f"wkv {name}", T, n)
        self._want(z, torch.float32, "wkv decay input", T, n)
        for t in (w0, u, norm_w):
            self._want(t, torch.float32, "wkv vector", n)
        self._want(state, torch.float32, "wkv state", state.shape[0], heads, dim, dim)
        S = self._seq_operands("wkv", seq_q_start, seq_q_len, seq_slot)
        out = torch.empty((T, n), dtype=self.dtype, device=r.device)
        seg, n_segs = self._walk_segments(T, S, self.WKV_SEGMENT, heads * dim * dim)
        carry = torch.empty((S, n_segs, heads, dim, dim), dtype=torch.float32, device=r.device) if seg else None
        cdec = torch.empty((S, n_segs, heads, dim), dtype=torch.float32, device=r.device) if seg else None
        self._check(lib, lib.ms_wkv(_ptr(r), _ptr(k), _ptr(v), _ptr(gate), _ptr(z), _ptr(w0), _ptr(u), _ptr(norm_w), _c_float(eps), _ptr(state),
                                    _ptr(seq_q_start), _ptr(seq_q_len), _ptr(seq_slot), _c_int(S), _ptr(out), _c_int(heads), _c_int(dim),
                                    _c_int(seg), _c_int(n_segs), _ptr(carry), _ptr(cdec), self._stream()))
        return out

    # ------------------------------------------------------------------ routed experts
    EXPERT_ACTIVATIONS = {"gelu": 0, "gelu_tanh": 1, "silu": 2}

    def route_limits(self) -> dict:
        return {"experts": self._extra_lib("routed").ms_route_max_experts(), "top": 64}

    def route(self, h: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], top: int, correction: Optional[torch.Tensor] = None,
              softmax_all: bool = False) -> torch.Tensor:
        """Float32 ``[T, experts]``: for every row its weight for each expert, the softmax over the ``top`` largest of the
        logits ``h @ w.T + bias`` (32-bit sums, float32 weights; the lower index wins a tie), zero for the others.  With
        ``softmax_all`` the scores are the softmax over all logits, the ``top`` largest of score + ``correction`` are chosen,
        and the weights are the chosen scores over their sum (+ 1e-20)."""
        lib = self._extra_lib("routed")
        T, d = h.shape
        E = w.shape[0]
        self._want(h, self.dtype, "route rows")
        self._want(w, torch.float32, "route weight", E, d)
        if bias is not None:
            self._want(bias, torch.float32, "route bias", E)
        if correction is not None:
            self._want(correction, torch.float32, "route correction", E)
        gates = torch.empty((T, E), dtype=torch.float32, device=h.device)
        self._check(lib, lib.ms_route(_ptr(h), _ptr(w), _ptr(bias), _ptr(gates), _c_int(T), _c_int(d), _c_int(E), _c_int(top),
                                      _c_int(int(softmax_all)), _ptr(correction), self._stream()))
        return gates

    def expert_act(self, up: torch.Tensor, gates: torch.Tensor, ff: int, activation: str, experts: Optional[int] = None,
                   gated: bool = False) -> torch.Tensor:
        """``act(up[t, c]) * gates[t, c // ff]`` in the element type for float32 ``up [T, n]``; the columns beyond
        ``experts * ff`` (an expert every row uses) carry weight one.  ``experts``: how many of the gates' columns are
        experts with columns here (None: all).  ``gated``: ``up`` is ``[T, 2 n]``, the experts' gates and then their up
        projections, and the result ``act(gate) * up * weight``."""
        lib = self._extra_lib("routed")
        T, n = up.shape
        if gated:
            if n % 2:
                raise KernelError(f"experts: {n} columns are not gates and up projections")
            n //= 2
        E = gates.shape[1] if experts is None else experts
        self._want(up, torch.float32, "expert sums")
        self._want(gates, torch.float32, "expert weights", T, gates.shape[1])
        if E > gates.shape[1]:
            raise KernelError(f"experts: {E} experts for weights of {gates.shape[1]} columns")
        if activation not in self.EXPERT_ACTIVATIONS:
            raise KernelError(f"experts: activation {activation!r} is not built (built: {', '.join(sorted(self.EXPERT_ACTIVATIONS))})")
        out = torch.empty((T, n), dtype=self.dtype, device=up.device)
        self._check(lib, lib.ms_expert_act(_ptr(up), _ptr(gates), _ptr(out), _c_int(T), _c_int(n), _c_int(E), _c_int(ff),
                                           _c_int(self.EXPERT_ACTIVATIONS[activation]), _c_int(gates.shape[1]), _c_int(int(gated)), self._stream()))
        return out

    def add_scaled_rows(self, x: torch.Tensor, h: torch.Tensor, weights: torch.Tensor, first: int, count: int) -> None:
        """``x[t] += (sum of weights[t, first : first + count]) * h[t]`` for float32 ``x [T, d]``, ``h`` in the element type and
        float32 ``weights [T, n]``: rows of a part's own input added with a weight a row."""
        lib = self._extra_lib("routed")
        T, d = x.shape
        self._want(x, torch.float32, "add_scaled_rows sums")
        self._want(h, self.dtype, "add_scaled_rows rows", T, d)
        self._want(weights, torch.float32, "add_scaled_rows weights", T, weights.shape[1])
        self._check(lib, lib.ms_add_scaled_rows(_ptr(x), _ptr(h), _ptr(weights), _c_int(weights.shape[1]), _c_int(first), _c_int(count),
                                                _c_int(T), _c_int(d), self._stream()))

    # ------------------------------------------------------------------ several residual streams
    def streams_limits(self) -> dict:
        lib = self._extra_lib("multistream")
        return {"streams": lib.ms_streams_max(), "row": lib.ms_streams_max_row()}

    def _streams(self, xs: torch.Tensor):
        self._want(xs, torch.float32, "streams")
        if xs.dim() != 3:
            raise KernelError(f"streams of shape {tuple(xs.shape)}: [streams, rows, width] wanted")
        return xs.shape

    def streams_read(self, xs: torch.Tensor, w_in: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``sum_s w_in[s] xs[s]`` (None: the plain sum) of float32 ``xs [S, T, d]``, of the ``rows`` if given; float32."""
        lib = self._extra_lib("multistream")
        S, T, d = self._streams(xs)
        if w_in is not None:
            self._want(w_in, torch.float32, "streams' input weights", S)
        R = T
        if rows is not None:
            self._want(rows, torch.int32, "streams' rows")
            R = rows.numel()
        out = torch.empty((R, d), dtype=torch.float32, device=xs.device)
        self._check(lib, lib.ms_streams_read(_ptr(xs), _ptr(w_in), _ptr(rows), _c_int(R), _ptr(None), _c_float(0.0), _ptr(out), _ptr(None), _c_int(S),
                                             _c_int(T), _c_int(d), self._stream()))
        return out

    def streams_read_norm(self, xs: torch.Tensor, w_in: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float) -> torch.Tensor:
        """``rmsnorm(sum_s w_in[s] xs[s]) * norm_w`` in the element type, one kernel."""
        lib = self._extra_lib("multistream")
        S, T, d = self._streams(xs)
        if w_in is not None:
            self._want(w_in, torch.float32, "streams' input weights", S)
        self._want(norm_w, torch.float32, "streams' norm weight", d)
        out = torch.empty((T, d), dtype=self.dtype, device=xs.device)
        self._check(lib, lib.ms_streams_read(_ptr(xs), _ptr(w_in), _ptr(None), _c_int(T), _ptr(norm_w), _c_float(eps), _ptr(None), _ptr(out), _c_int(S),
                                             _c_int(T), _c_int(d), self._stream()))
        return out

    def streams_write(self, xs: torch.Tensor, sums: torch.Tensor, bias: Optional[torch.Tensor], mix: torch.Tensor, w_out: torch.Tensor) -> None:
        """In place, all streams at once from the old ones: ``xs[t] = sum_s mix[s, t] xs[s] + w_out[t] (sum(sums) + bias)`` for
        float32 ``xs [S, T, d]`` and the partial sums ``sums [P, T, d]`` of a branch's last product."""
        lib = self._extra_lib("multistream")
        S, T, d = self._streams(xs)
        self._want(sums, torch.float32, "streams' sums", sums.shape[0], T, d)
        if bias is not None:
            self._want(bias, torch.float32, "streams' bias", d)
        self._want(mix, torch.float32, "streams' mixing matrix", S, S)
        self._want(w_out, torch.float32, "streams' output weights", S)
        self._check(lib, lib.ms_streams_write(_ptr(xs), _ptr(sums), _c_int(sums.shape[0]), _ptr(bias), _ptr(mix), _ptr(w_out), _c_int(S),
                                              _c_int(T), _c_int(d), self._stream()))

    def streams_write_read_norm(self, xs: torch.Tensor, sums: torch.Tensor, bias: Optional[torch.Tensor], mix: torch.Tensor,
                                w_out: torch.Tensor, w_in: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float) -> torch.Tensor:
        """:meth:`streams_write` and, from the streams as they are written, :meth:`streams_read_norm` of the branch that
        follows, in one kernel: the same numbers as the two calls."""
        lib = self._extra_lib("multistream")
        S, T, d = self._streams(xs)
        self._want(sums, torch.float32, "streams' sums", sums.shape[0], T, d)
        if bias is not None:
            self._want(bias, torch.float32, "streams' bias", d)
        self._want(mix, torch.float32, "streams' mixing matrix", S, S)
        self._want(w_out, torch.float32, "streams' output weights", S)
        if w_in is not None:
            self._want(w_in, torch.float32, "streams' input weights", S)
        self._want(norm_w, torch.float32, "streams' norm weight", d)
        out = torch.empty((T, d), dtype=self.dtype, device=xs.device)
        self._check(lib, lib.ms_streams_write_read(_ptr(xs), _ptr(sums), _c_int(sums.shape[0]), _ptr(bias), _ptr(mix), _ptr(w_out), _ptr(w_in),
                                                   _ptr(norm_w), _c_float(eps), _ptr(out), _c_int(S), _c_int(T), _c_int(d), self._stream()))
        return out

    # ------------------------------------------------------------------ state-space duality
    def ssd_limits(self) -> dict:
        lib = self._extra_lib("ssd")
        return {"states": lib.ms_ssd_max_states(), "head_dim": lib.ms_ssd_max_head()}

    def ssd_scan(self, xbc: torch.Tensor, proj: torch.Tensor, dt_col: int, dt_bias: torch.Tensor, a_log: torch.Tensor, d_skip: torch.Tensor,
                 state: torch.Tensor, seq_q_start: torch.Tensor, seq_q_len: torch.Tensor, seq_slot: torch.Tensor, H: int, P: int, N: int,
                 G: int) -> torch.Tensor:
        """The recurrence of the second Mamba layer over the step's rows.  ``xbc`` float32 ``[T, H P + 2 G N]``: x, B and C
        behind their convolution, before their SiLU; ``proj`` float32 ``[T, ld]`` whose columns ``dt_col .. dt_col + H`` are the
        raw step sizes; ``dt = softplus(raw + dt_bias)``, ``S <- exp(-exp(a_log) dt) S + dt B x^T``, ``y = S^T C + d_skip x``;
        ``state`` float32 ``[slots, H, N, P]`` is carried on.  Returns float32 ``y [T, H P]``."""
        lib = self._extra_lib("ssd")
        T = xbc.shape[0]
        self._want(xbc, torch.float32, "ssd x, B and C", T, H * P + 2 * G * N)
        self._want(proj, torch.float32, "ssd projection", T, proj.shape[1])
        for t, n in ((dt_bias, "dt_bias"), (a_log, "A_log"), (d_skip, "D")):
            self._want(t, torch.float32, f"ssd {n}", H)
        self._want(state, torch.float32, "ssd state", state.shape[0], H, N, P)
        S = self._seq_operands("ssd", seq_q_start, seq_q_len, seq_slot)
        y = torch.empty((T, H * P), dtype=torch.float32, device=xbc.device)
        seg, n_segs = self._walk_segments(T, S, self.SSD_SEGMENT, H * N * P)
        carry = torch.empty((S, n_segs, H, N, P), dtype=torch.float32, device=xbc.device) if seg else None
        cdec = torch.empty((S, n_segs, H), dtype=torch.float32, device=xbc.device) if seg else None
        self._check(lib, lib.ms_ssd_scan(_ptr(xbc), _c_int(xbc.shape[1]), _ptr(proj), _c_int(proj.shape[1]), _c_int(dt_col), _ptr(dt_bias),
                                         _ptr(a_log), _ptr(d_skip), _ptr(state), _ptr(seq_q_start), _ptr(seq_q_len), _ptr(seq_slot), _c_int(S),
                                         _ptr(y), _c_int(T), _c_int(H), _c_int(P), _c_int(N), _c_int(G), _c_int(seg), _c_int(n_segs),
                                         _ptr(carry), _ptr(cdec), self._stream()))
        return y

    SSD_SEGMENT = 64  # rows of a segment of the state-space recurrence

    def gated_group_norm(self, y: torch.Tensor, proj: torch.Tensor, z_col: int, weight: torch.Tensor, eps: float, groups: int,
                         out_cols: int) -> torch.Tensor:
        """``y * silu(z)`` RMS-normed in ``groups`` equal parts, times ``weight``, in the element type ``[T, out_cols]`` (zeros
        behind the ``n`` columns of ``y``); ``z`` is columns ``z_col .. z_col + n`` of float32 ``proj``."""
        lib = self._extra_lib("ssd")
        T, n = y.shape
        self._want(y, torch.float32, "gated norm input")
        self._want(proj, torch.float32, "gated norm gate", T, proj.shape[1])
        if z_col < 0 or z_col + n > proj.shape[1] or out_cols < n:
            raise KernelError(f"gated norm: gate columns {z_col}..{z_col + n} of {tuple(proj.shape)}, {out_cols} columns out")
        self._want(weight, torch.float32, "gated norm weight", n)
        out = torch.empty((T, out_cols), dtype=self.dtype, device=y.device)
        z = _c_void(proj.data_ptr() + z_col * 4)
        self._check(lib, lib.ms_gated_group_norm(_ptr(y), z, _c_int(proj.shape[1]), _ptr(weight), _ptr(out), _c_int(out_cols), _c_int(T),
                                                 _c_int(n), _c_int(groups), _c_float(eps), self._stream()))
        return out

    # ------------------------------------------------------------------ sampling
    def sample(self, logits, temperature, top_k, top_p, state, any_greedy: bool = True):
        """One token per row; ``state`` (int64 SplitMix64 states) advances in place.
        Returns ``(tokens int32, logprobs float32)``."""
        both = self.sample_packed(logits, temperature, top_k, top_p, state, any_greedy)
        return both[0], both[1].view(torch.float32)

    def sample_packed(self, logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
                      state: torch.Tensor, any_greedy: bool = True, also_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        """:meth:`sample` with both results in one int32 tensor ``[2, W]`` (tokens, then the bits of
        the logprobs) so that one copy brings them to the host.  With ``any_greedy`` a first
        launch finds the maxima of 64 chunks of every row, so that a greedy row is not one
        block's serial scan.  ``also_tokens`` (int32 ``[W]``) receives the tokens as well: the
        place where a following step reads its input."""
        W, V = logits.shape
        self._want(logits, torch.float32, "sample logits")
        self._want(temperature, torch.float32, "sample temperature", W)
        self._want(top_k, torch.int32, "sample top_k", W)
        self._want(top_p, torch.float32, "sample top_p", W)
        self._want(state, torch.int64, "sample state", W)
        if also_tokens is not None:
            self._want(also_tokens, torch.int32, "sample also_tokens", W)
        both = torch.empty((2, W), dtype=torch.int32, device=logits.device)  # tokens, then logprob bits
        tok, lp = both[0], both[1].view(torch.float32)
        pv = pi = None
        if any_greedy:
            chunks = self._core.ms_sample_chunks()
            pv = torch.empty((W, chunks), dtype=torch.float32, device=logits.device)
            pi = torch.empty((W, chunks), dtype=torch.int32, device=logits.device)
        self._check(self._core, self._core.ms_sample(_ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(top_p),
                                                     _ptr(state), _ptr(tok), _ptr(lp), _ptr(pv), _ptr(pi),
                                                     _ptr(also_tokens), _c_int(W), _c_int(V), self._stream()))
        return both

    def top_logprobs(self, logits: torch.Tensor, inv_t: torch.Tensor, k: int):
        """The ``k`` most probable tokens of every row and their log-probabilities at the row's
        temperature (``inv_t``), ties to the smaller id.  Returns ``(tokens [W, k], logprobs [W, k])``."""
        W, V = logits.shape
        self._want(logits, torch.float32, "top_logprobs logits")
        self._want(inv_t, torch.float32, "top_logprobs inv_t", W)
        width = self._core.ms_top_logprobs_max()
        tok = torch.empty((W, width), dtype=torch.int32, device=logits.device)
        lp = torch.empty((W, width), dtype=torch.float32, device=logits.device)
        self._check(self._core, self._core.ms_top_logprobs(_ptr(logits), _ptr(inv_t), _ptr(tok), _ptr(lp), _c_int(W),
                                                           _c_int(V), _c_int(k), self._stream()))
        return tok[:, :k], lp[:, :k]

    def logit_edit(self, logits: torch.Tensor, row_of: torch.Tensor, token: torch.Tensor, delta: torch.Tensor) -> None:
        """``logits[row_of[e], token[e]] += delta[e]`` (penalties and biases merged on the host)."""
        n = row_of.numel()
        self._want(logits, torch.float32, "logit_edit logits")
        self._want(row_of, torch.int32, "logit_edit rows", n)
        self._want(token, torch.int32, "logit_edit tokens", n)
        self._want(delta, torch.float32, "logit_edit deltas", n)
        self._check(self._core, self._core.ms_logit_edit(_ptr(logits), _c_int(logits.shape[1]), _ptr(row_of), _ptr(token),
                                                         _ptr(delta), _c_int(n), self._stream()))


# The activations a gated product applies to its gate branch, by the name a specification gives them, and the
# number the kernels know them by.
GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def gate_activation_code(name: str) -> int:
    try:
        return GATE_ACTIVATIONS[name]
    except KeyError:
        raise KernelError(f"gated product: activation {name!r} is not built (built: {', '.join(sorted(GATE_ACTIVATIONS))})") from None


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``[2 * ceil16(I), d]``: blocks of 16 gate rows and the same 16 up rows alternate, zero
    rows pad the last block; the layout :meth:`HipOps.linear_swiglu` multiplies by."""
    I, d = gate.shape
    Ip = (I + 15) // 16 * 16
    g = torch.zeros((Ip, d), dtype=gate.dtype, device=gate.device)
    u = torch.zeros((Ip, d), dtype=gate.dtype, device=gate.device)
    g[:I] = gate
    u[:I] = up
    return torch.stack([g.view(Ip // 16, 16, d), u.view(Ip // 16, 16, d)], dim=1).reshape(2 * Ip, d).contiguous()


_OPS = {}


def get_ops(dtype: torch.dtype, device: str = "cuda:0") -> HipOps:
    key = (dtype, device)
    if key not in _OPS:
        _OPS[key] = HipOps(dtype, device)
    return _OPS[key]
