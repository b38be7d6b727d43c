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

_RET_MODES = {"all": 0, "chunk": 1, "window": 2}  # the rules under which the attention kernels here read keys


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
    "jle_attention_prefill": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _vp, _i, _i, _i, _f, _i, _i, _i, _i, _vp],
    "jle_attention_decode": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _f, _i, _i, _i, _i,
                             _vp],
    "jle_attention_decode_fused": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _f, _i, _i,
                                   _i, _i, _vp, _f, _f, _f, _vp, _i, _vp],
    "jle_gemm_grouped": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    "jle_gemm_skinny": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _i, _i, _i, _i, _vp, _vp,
                        _vp],
    "jle_gemm_stream": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
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


def load_library():
    """Loads the compiled kernels (compiling them if no build is there)."""
    global _LIB
    if _LIB is None:
        path = _build.library_path()
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"cannot load the HIP kernel library {path}: {e}") from e
        for name, args in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = ctypes.c_int
        lib.jle_attention_mfma_supported.argtypes = [_i, _i, _i, _i]  # a query, not a launch: no stream
        lib.jle_gemm_stream_supported.argtypes = [_i, _i, _i]
        lib.jle_gemm_f32_stream_supported.argtypes = [_i, _i, _i]
        lib.jle_attention_group_waves.argtypes = []
        lib._jle_path = path
        _LIB = lib
    return _LIB


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


class HipOps:
    name = "hip"

    def __init__(self, device) -> None:
        self.device = torch.device(device)
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise KernelError("the HIP kernels need a GPU")
        self.lib = load_library()
        self._fn = {name: getattr(self.lib, name) for name in _SIGNATURES}
        self._device_index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        self._raw_stream = raw if raw is not None else (lambda i: torch.cuda.current_stream(i).cuda_stream)
        # true float32 products: no reduced-precision matrix mode
        # counters of the kernels in which the last wavefront (or block) to finish does the closing work: zero
        # between launches (whoever closes puts its counter back), so they are cleared here once
        self._tickets = torch.zeros(self.TICKETS, dtype=torch.int32, device=self.device)
        self._slice_tickets = torch.zeros(self.SLICE_TICKETS, dtype=torch.int32, device=self.device)
        self._compute_units = torch.cuda.get_device_properties(self.device).multi_processor_count
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")

    # ------------------------------------------------------------------ helpers
    def _stream(self) -> int:
        """The current stream's handle (a decode step asks hundreds of times: the raw query, not a Stream object)."""
        return self._raw_stream(self._device_index)

    def _call(self, name: str, *args) -> None:
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

    def add_rmsnorm(self, x, delta, weight, eps: float, out_dtype, want32: bool = False):
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
        """The tensor an :class:`ExpertSum` stands for (float32)."""
        if not isinstance(delta, ExpertSum):
            return delta
        n, d = delta.shape
        out = torch.empty(n, d, dtype=torch.float32, device=delta.routed.device)
        self._call("jle_moe_combine", _p(delta.routed), _p(delta.inv), _p(delta.shared), _p(out),
                   self._is_bf16(delta.routed), n, delta.k, d)
        return out

    def add_residual(self, x, delta) -> None:
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

    def swiglu_linear(self, h, w_gate_up):
        """``silu(h @ Wg.T) * (h @ Wu.T)`` with ``w_gate_up`` = gate rows, then up rows."""
        h = self._rows(h)
        if h.dtype == torch.bfloat16 and h.shape[0] <= self.SKINNY_DENSE_ROWS and h.shape[1] % 8 == 0:
            return self.gemm_skinny(h, w_gate_up, swiglu=True)
        return self.silu_mul(torch.matmul(h, w_gate_up.t()))

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
        return bool(self.lib.jle_gemm_f32_stream_supported(nout, k, int(swiglu)))

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
        return bool(self.lib.jle_gemm_stream_supported(nout, k, int(swiglu)))

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

    def silu_mul(self, gate_up):
        n, f2 = gate_up.shape
        self._chk(gate_up, None, None, "gate|up")
        out = torch.empty(n, f2 // 2, dtype=gate_up.dtype, device=gate_up.device)
        self._call("jle_silu_mul", _p(gate_up), _p(out), self._is_bf16(gate_up), n, f2 // 2)
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
        if (meta is not None and meta.decode_bucket is not None and qkv.dtype == torch.bfloat16 and prep.plain
                and group <= 32 and n * hk < self.TICKETS and 4 * (dh + 4 * group * (dh + 2)) <= 48 * 1024
                and self.lib.jle_attention_mfma_supported(dh, hq, hk, ps)):
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

    def attention_plan(self, seg_lens, seg_starts, retention, device, num_kv_heads=1, group_size=1, decode_bucket=None):
        """Work lists of the MFMA attention kernels for one step and one retention rule: the rows that are
        single decode tokens (and into how many keys their work is split), tiles of up to 32 consecutive
        tokens of longer segments and, with ``group_size`` > 1 query heads per kv head, the packing of the
        (tile, head) items of a kv head into blocks of wavefronts that share keys.  ``decode_bucket``: the step
        holds single tokens only, none beyond this context length: the split is then chosen from the number of
        tokens and this bound alone (not from where each request stands), so the same launch fits every such
        step."""
        from ..parts.base import first_needed_position

        dec, tiles, spans, seg_tiles = [], [], [], []
        o = 0
        for i, n in enumerate(seg_lens):
            if n == 1:
                dec.append(o)
                if decode_bucket is None:
                    spans.append((first_needed_position(retention, seg_starts[i]), seg_starts[i]))
            else:
                first = len(tiles) // 2
                for t in range(0, n, self.PREFILL_TILE):
                    tiles += [o + t, min(self.PREFILL_TILE, n - t)]
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
        if tiles and group_size > 1 and self.PREFILL_TILE == 32:
            # consecutive (tile, head) items of one segment, `waves` per block; blocks with the most keys first
            waves = int(self.lib.jle_attention_group_waves())
            keyed = []
            for first, count, last_pos in seg_tiles:
                items = count * group_size
                for lo in range(0, items, waves):
                    n_items = min(waves, items - lo)
                    last_tile = first + (lo + n_items - 1) // group_size
                    end = last_pos - (first + count - 1 - last_tile) * self.PREFILL_TILE  # about where its keys end
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

    def paged_attention(self, q, kv_cache, block_table, positions, token_segment, retention, scale: float, meta=None):
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
        if (q.dtype == torch.bfloat16 and hq // hk <= 32
                and self.lib.jle_attention_mfma_supported(dh, hq, hk, ps)):
            key = f"attn_plan_{hq // hk}"
            plan = meta.meta.get(key) if meta is not None else None
            if plan is None:
                seg_lens, seg_starts = self._segments(meta, token_segment, positions)
                plan = self.attention_plan(seg_lens, seg_starts, retention, q.device, hk, hq // hk,
                                           decode_bucket=meta.decode_bucket if meta is not None else None)
                if meta is not None:
                    meta.meta[key] = plan
            if plan["num_tiles"]:
                self._call("jle_attention_prefill", _p(q), _p(kv_cache), _p(out), _p(positions), _p(token_segment),
                           _p(block_table), block_table.shape[1], _p(plan["tiles"]), plan["num_tiles"],
                           self.PREFILL_TILE, _p(plan["groups"]), plan["num_groups"], mode, param, float(scale), hq,
                           hk, dh, ps)
            if plan["num_dec"]:
                cols = 16 if hq // hk <= 16 else 32
                items = plan["num_dec"] * hk * plan["max_splits"]
                ws_ml = torch.empty(items * cols * 2, dtype=torch.float32, device=q.device)
                ws_o = torch.empty(items * cols * dh, dtype=torch.float32, device=q.device)
                self._call("jle_attention_decode", _p(q), _p(kv_cache), _p(out), _p(ws_ml), _p(ws_o), _p(positions),
                           _p(token_segment), _p(block_table), block_table.shape[1], _p(plan["dec"]), plan["num_dec"],
                           plan["max_splits"], plan["split"], mode, param, float(scale), hq, hk, dh, ps)
            return out
        if dh % 8 or dh > 256:
            raise KernelError(f"attention kernels: head size {dh} is not supported (a multiple of 8, at most 256)")
        if hq % hk:
            raise KernelError(f"attention kernels: {hq} query heads are no multiple of {hk} kv heads")
        if (q.dtype == torch.float32 and dh % 16 == 0 and ps % 16 == 0 and n * hq >= self.GENERIC_SPLIT_BELOW
                and (meta is None or meta.decode_bucket is None)):
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
        if (q.dtype == torch.float32 and dh % 16 == 0 and ps % 16 == 0 and hq // hk <= 16
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
        self._call("jle_paged_attention_generic", _p(q), _p(kv_cache), _p(out), _p(positions), _p(token_segment),
                   _p(block_table), block_table.shape[1], mode, param, float(scale), self._is_bf16(q), n, hq, hk, dh,
                   ps, splits, tiles_per_split, _p(ws_ml), _p(ws_o))
        return out

    # ------------------------------------------------------------------ routed experts
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

    def moe_experts(self, h, expert_ids, gates, w_gate_up, w_down, shared=None, tiled: bool = False, grouping=None,
                    shared_weights=None):
        """``shared``: a shared expert's output, or ``shared_weights``: its (gate|up, down) matrices, row-major."""
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
