"""The kernels as Python calls on torch tensors.

Every method checks on the host that shapes, dtypes, devices and contiguity match what the
kernel and its grid assume, then passes raw device pointers and the current HIP stream to
the library. Nothing here computes on the CPU and nothing falls back to a library routine
except where the matrix products say so (``linear``).
"""
import ctypes
from typing import Optional

import torch

from . import dispatch as D
from . import library
from .handles import DeferredLinear, PendingProduct, ScaledRows

F32 = 0
BF16 = 1


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise TypeError("kernels take float32 or bfloat16 tensors, got %s" % dtype)


try:
    _raw_stream, _current_device = torch._C._cuda_getCurrentRawStream, torch._C._cuda_getDevice
except AttributeError:      # a torch without these: the documented way

    def _raw_stream(device_index: int) -> int:
        return torch.cuda.current_stream(device_index).cuda_stream

    _current_device = torch.cuda.current_device


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


class HipOps:
    """Kernel calls of the product path. One instance per process is enough."""

    name = "hip"

    def __init__(self):
        if not torch.cuda.is_available():
            raise library.KernelLibraryError(
                "lmsf_amd needs a GPU: torch.cuda.is_available() is False and there is no CPU path")
        self.lib = library.load_library()
        buf = ctypes.create_string_buffer(256)
        if self.lib.lmsf_device_arch(buf, 256) != 0:
            raise library.KernelLibraryError(library.last_error(self.lib))
        self.device_arch = buf.value.decode()
        if not self.device_arch.startswith("gfx950"):
            raise library.KernelLibraryError(
                "the kernels are built for gfx950 only; this device reports %r" % self.device_arch)
        self._bad_flag = None
        # The switch points between the kernels live in one structure that the C++ side reads (csrc/dispatch.h says
        # what each means); they are attributes of this object all the same (see __setattr__).
        self.use_library_gemm = True   # bfloat16 matrix products of many rows go to the BLAS library
        self.prefill_attention_variant = 0
        self.decode_attention_order = 0
        self.decode_attention_splits = 0
        self.fuse_norm_rows = 16
        self.fuse_stream_rows = 1
        self.gemv_max_rows = 2
        self.skinny_variant = 0
        self.mid_wide_max_cols = 8192  # beyond 64 rows only products of up to this many columns: the library is good at the wide ones (measured)
        self.mid_max_rows = 128        # rows up to which the 17-and-more-rows kernel beats the library (64 with the gated activation)
        self.skinny_max_rows = 16      # rows up to which the few-rows kernel beats the library (measured)
        self.large_max_rows = 256      # rows up to which the many-rows kernel beats the library (measured; 0: never)
        self.large_deep_min_rows = 64    # products whose K is at least three times N go to the many-rows kernel from beyond this many rows already (down at 128 rows: 42.8 -> 38.0 us; decode at batch 128: 6.63 -> 6.53 ms a step, at 96: 5.83 -> 5.74)
        self.mid_scaled_rows = 16        # rows up to which the gated product after a norm runs in the 17-and-more-rows kernel where that kernel's workgroups fit on the chip at once (0: never)
        self.large_deep_max_rows = 1024  # the same for products whose K is at least three times N (down: 57 against 76 us at 320 rows, 74 against 94 at 512, 102 against 108 at 768, level at 1,024)
        self.qkv_fused_max_rows = 32     # rows up to which the QKV product with rotation and cache write runs in the few-rows kernel, beyond skinny_max_rows (one kernel against the 17-and-more-rows product and the rotary kernel over its partial sums: decode at batch 24 3.99 -> 3.92 ms a step, at 32 4.11 -> 3.99; level at 48, behind at 64: 4.80 -> 4.87)
        self.weight_row_pad_bytes = 512  # bytes left between two rows of a linear layer's weight (see weight_row_pad)
        # the BLAS library's products are called from C++ (csrc/blas.hip); its handle and workspace are made here
        if self.lib.lmsf_blas_init(self.blas_workspace_bytes) != 0:
            raise library.KernelLibraryError("the BLAS library cannot be used: " + library.last_error(self.lib))

    blas_workspace_bytes = 128 << 20

    def __setattr__(self, name, value):
        if name in D.TUNABLE_NAMES:
            setattr(self.__dict__.setdefault("_tun", D.Tunables()), name, int(value))
        else:
            object.__setattr__(self, name, value)

    def __getattr__(self, name):
        # (called only for names that are no ordinary attributes: the switch points)
        if name in D.TUNABLE_NAMES and "_tun" in self.__dict__:
            return int(getattr(self.__dict__["_tun"], name))
        raise AttributeError(name)

    def tunables(self) -> tuple:
        """The switch points as they are now, in the order of ``dispatch.TUNABLE_NAMES``."""
        return self._tun.as_tuple()

    def _shape(self, x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype) -> D.ProductShape:
        """What the C++ side wants to know of a product x weight^T before it names the kernel."""
        return D.ProductShape(x.shape[0], weight.shape[0], x.shape[1], _code(x.dtype), _code(weight.dtype),
                              _code(out_dtype), x.stride(0), weight.stride(0), 1 if x.data_ptr() % 16 == 0 else 0,
                              1 if weight.data_ptr() % 16 == 0 else 0)

    # ------------------------------------------------------------------ helpers

    def _stream(self):
        # (the raw handle of the current device's current stream; torch.cuda.current_stream() gives the same
        # handle wrapped in an object and costs 8 us a call, a third of the host's time in a step of few tokens)
        return ctypes.c_void_p(_raw_stream(_current_device()))

    def _check(self, rc: int):
        if rc != 0:
            raise RuntimeError("lmsf_amd kernel error: " + library.last_error(self.lib))

    @staticmethod
    def _dev(*tensors):
        for t in tensors:
            if t is not None and not t.is_cuda:
                raise ValueError("kernel operand is not on the GPU")

    @staticmethod
    def _i32(t: Optional[torch.Tensor], name: str, numel: Optional[int] = None):
        if t is None:
            return
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise ValueError("%s must be a contiguous int32 tensor" % name)
        if numel is not None and t.numel() < numel:
            raise ValueError("%s holds %d elements, %d needed" % (name, t.numel(), numel))

    # ------------------------------------------------------------------ embedding

    def embedding(self, ids: torch.Tensor, table: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
        """float32 [N, H] rows of ``table`` [V, H] selected by int32 ``ids`` [N], times ``scale``."""
        self._dev(ids, table)
        self._i32(ids, "ids")
        if table.dim() != 2 or not table.is_contiguous():
            raise ValueError("embedding table must be contiguous [V, H]")
        n, (V, H) = ids.numel(), table.shape
        out = torch.empty((n, H), dtype=torch.float32, device=table.device)
        if self._bad_flag is None or self._bad_flag.device != table.device:
            self._bad_flag = torch.zeros(1, dtype=torch.int32, device=table.device)
        self._check(self.lib.lmsf_embedding(_ptr(ids), _ptr(table), _code(table.dtype), _ptr(out), n, H, V,
                                            float(scale), _ptr(self._bad_flag), self._stream()))
        return out

    def patch_tokens(self, ids: torch.Tensor, src: torch.Tensor, prev: torch.Tensor) -> None:
        """ids[i] = prev[src[i]] where src[i] >= 0 (all int32, on the device): a step launched ahead takes the
        tokens that the step before it sampled from where the sampler left them."""
        self._dev(ids, src, prev)
        self._i32(ids, "ids")
        self._i32(src, "src", ids.numel())
        self._i32(prev, "prev")
        self._check(self.lib.lmsf_patch_tokens(_ptr(ids), _ptr(src), _ptr(prev), ids.numel(), prev.numel(),
                                               self._stream()))

    def bad_token_seen(self) -> bool:
        """True if an embedding call since the last query met an id outside the vocabulary."""
        if self._bad_flag is None:
            return False
        bad = bool(self._bad_flag.item())
        if bad:
            self._bad_flag.zero_()
        return bad

    # ------------------------------------------------------------------ norm

    def add_rms_norm(self, branch: Optional[torch.Tensor], residual: Optional[torch.Tensor], weight: torch.Tensor,
                     eps: float, out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                     weight_offset: float = 0.0, defer_ok: bool = False):
        """out = rms_norm(branch + residual) * (weight + weight_offset).

        ``residual`` (float32 [N, H]) is updated to the sum in place when both operands are given
        and ``rows`` is None. ``rows`` (int32 [R]) selects input rows; the output then has R rows.
        ``branch`` may be a ``PendingProduct``: its partial sums are added up on the way in; or a
        ``DeferredLinear``, which then runs as a product that adds into ``residual``. With ``defer_ok``
        the caller takes a ``ScaledRows`` as well (up to 16 rows, after a ``DeferredLinear``).
        """
        if isinstance(branch, PendingProduct):
            return self._add_rms_norm_pending(branch, residual, weight, eps, out_dtype, rows, weight_offset)
        if isinstance(branch, DeferredLinear):
            handle, branch = self._run_deferred(branch, residual, weight, eps, out_dtype, rows, weight_offset, defer_ok)
            if handle is not None:
                return handle
        self._dev(branch, residual, weight, rows)
        ref = branch if branch is not None else residual
        if ref is None:
            raise ValueError("add_rms_norm needs a branch or a residual")
        if ref.dim() != 2 or not ref.is_contiguous():
            raise ValueError("add_rms_norm operands must be contiguous [N, H]")
        N, H = ref.shape
        if branch is not None and residual is not None and branch.shape != residual.shape:
            raise ValueError("branch %s and residual %s differ in shape" % (tuple(branch.shape), tuple(residual.shape)))
        if residual is not None and (residual.dtype != torch.float32 or not residual.is_contiguous()):
            raise ValueError("the residual stream must be contiguous float32")
        if weight.shape != (H,) or not weight.is_contiguous():
            raise ValueError("norm weight must be [%d], got %s" % (H, tuple(weight.shape)))
        self._i32(rows, "rows")
        n_out = N if rows is None else rows.numel()
        out = torch.empty((n_out, H), dtype=out_dtype, device=ref.device)
        self._check(self.lib.lmsf_add_rms_norm(
            _ptr(branch), _code(branch.dtype) if branch is not None else F32, _ptr(residual), _ptr(weight),
            _code(weight.dtype), _ptr(out), _code(out_dtype), _ptr(rows), n_out, H, float(eps),
            float(weight_offset), self._stream()))
        return out

    def _run_deferred(self, branch: DeferredLinear, residual: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                      out_dtype: torch.dtype, rows: Optional[torch.Tensor], weight_offset: float, defer_ok: bool):
        """Runs the product that ``branch`` stands for, in the form that leaves the norm the least to do.
        Returns (handle, branch): a ``ScaledRows`` if the product did the norm's preparation as well (then the
        norm is done), else None and what is left to add: nothing if the product added into the stream itself,
        the product's tensor otherwise."""
        M, N = branch.shape
        K = branch.x.shape[1]
        fits = (rows is None and residual is not None and residual.dtype == torch.float32
                and residual.is_contiguous() and tuple(residual.shape) == branch.shape)
        prepares = (fits and defer_ok and out_dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
                    and weight.is_contiguous() and weight.shape == (N,))
        rt = D.Route()
        self.lib.lmsf_route_deferred_norm(ctypes.byref(self._tun), M, N, K, 1 if fits else 0, 1 if prepares else 0,
                                          ctypes.byref(rt))
        operands = (_ptr(branch.x), branch.x.stride(0), _ptr(branch.weight), branch.weight.stride(0), _ptr(branch.bias))
        if rt.route == D.GEMV_ADD_NORM:
            # adds into the stream, leaves stream * w and its workgroups' sums of squares
            self._dev(branch.x, branch.weight, branch.bias, residual, weight)
            parts = self.lib.lmsf_gemv_partials(N)
            xw = torch.empty((M, N), dtype=torch.bfloat16, device=residual.device)
            sumsq = torch.empty(parts * M, dtype=torch.float32, device=residual.device)
            self._check(self.lib.lmsf_gemv_add_norm(*operands, _ptr(residual), residual.stride(0), _ptr(weight),
                                                    float(weight_offset), _ptr(xw), xw.stride(0), _ptr(sumsq), M, N, K,
                                                    self._stream()))
            return ScaledRows(xw, sumsq, parts, M, residual, weight, float(eps), float(weight_offset), out_dtype), None
        if rt.route == D.SKINNY_ADD_NORM:
            # the same from the few-rows kernel: sums of squares per 16 columns
            self._dev(branch.x, branch.weight, branch.bias, residual, weight)
            tiles = -(-N // 16)
            xw = torch.empty((M, N), dtype=torch.bfloat16, device=residual.device)
            sumsq = torch.empty(tiles * 16, dtype=torch.float32, device=residual.device)
            self._check(self.lib.lmsf_gemm_skinny_add_norm(*operands, _ptr(residual), residual.stride(0), _ptr(weight),
                                                           float(weight_offset), _ptr(xw), xw.stride(0), _ptr(sumsq), M,
                                                           N, K, self.skinny_variant, self._stream()))
            return ScaledRows(xw, sumsq, tiles, 16, residual, weight, float(eps), float(weight_offset), out_dtype), None
        if rt.route == D.GEMV_ADD:
            # adds into the stream; the norm kernel follows
            self._dev(branch.x, branch.weight, branch.bias, residual)
            self._check(self.lib.lmsf_gemv_add(*operands, _ptr(residual), residual.stride(0), M, N, K, self._stream()))
            return None, None
        return None, self.materialize(branch)

    def _add_rms_norm_pending(self, branch: PendingProduct, residual: Optional[torch.Tensor], weight: torch.Tensor,
                              eps: float, out_dtype: torch.dtype, rows: Optional[torch.Tensor],
                              weight_offset: float) -> torch.Tensor:
        M, H = branch.shape
        fits = (H % 4 == 0 and H <= 16384 and weight.shape == (H,) and weight.is_contiguous()
                and weight.data_ptr() % 16 == 0
                and (residual is None or (residual.dtype == torch.float32 and residual.is_contiguous()
                                          and tuple(residual.shape) == (M, H) and residual.data_ptr() % 16 == 0)))
        if not fits:
            return self.add_rms_norm(self.materialize(branch), residual, weight, eps, out_dtype, rows, weight_offset)
        self._dev(residual, weight, rows)
        self._i32(rows, "rows")
        n_out = M if rows is None else rows.numel()
        out = torch.empty((n_out, H), dtype=out_dtype, device=branch.device)
        self._check(self.lib.lmsf_add_rms_norm_partial(
            _ptr(branch.partials), _ptr(branch.bias), branch.partials.shape[0], M, _ptr(residual), _ptr(weight),
            _code(weight.dtype), _ptr(out), _code(out_dtype), _ptr(rows), n_out, H, float(eps), float(weight_offset),
            self._stream()))
        return out

    def materialize(self, y):
        """The tensor behind ``y``: ``y`` itself, the finished sum of a ``PendingProduct``, the product of a
        ``DeferredLinear`` or the norm of a ``ScaledRows``."""
        if isinstance(y, DeferredLinear):
            return self.linear(y.x, y.weight, y.bias, out_dtype=y.dtype)
        if isinstance(y, ScaledRows):
            return self.add_rms_norm(None, y.stream, y.weight, y.eps, y.dtype, weight_offset=y.weight_offset)
        if not isinstance(y, PendingProduct):
            return y
        M, N = y.shape
        out = torch.empty((M, N), dtype=y.dtype, device=y.device)
        self._check(self.lib.lmsf_gemm_mid_reduce(_ptr(y.partials), _ptr(y.bias), _ptr(out), _code(y.dtype),
                                                  out.stride(0), M, N, y.partials.shape[0], self._stream()))
        return out

    # ------------------------------------------------------------------ rotary + cache write

    def rope_cache_write(self, qkv: torch.Tensor, nh: int, nkv: int, d: int, positions: Optional[torch.Tensor],
                         table: Optional[torch.Tensor], rot_dim: int, neox: bool, slots: Optional[torch.Tensor],
                         k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor]) -> None:
        """Rotate the q and k heads of the fused ``qkv`` [N, (nh + 2 nkv) d] in place and store k, v in
        the pages at ``slots``. ``table`` None: no rotation. ``slots`` None: no cache write."""
        self._dev(qkv, positions, table, slots, k_pages, v_pages)
        if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] != (nh + 2 * nkv) * d:
            raise ValueError("qkv must be [N, %d] with unit column stride, got %s" % ((nh + 2 * nkv) * d,
                                                                                      tuple(qkv.shape)))
        N = qkv.shape[0]
        es = qkv.element_size()
        max_pos = 0
        if table is not None:
            if table.dtype != torch.float32 or table.dim() != 2 or table.shape[1] != rot_dim or not table.is_contiguous():
                raise ValueError("rotary table must be contiguous float32 [max_pos, %d]" % rot_dim)
            self._i32(positions, "positions", N)
            if positions is None:
                raise ValueError("rotation needs positions")
            max_pos = table.shape[0]
        num_pages, ps = 0, 1
        if slots is not None:
            self._i32(slots, "slots", N)
            if k_pages is None or k_pages.dim() != 4 or k_pages.shape[1] != nkv or k_pages.shape[3] != d \
                    or not k_pages.is_contiguous() or k_pages.dtype != qkv.dtype:
                raise ValueError("k_pages must be contiguous [pages, %d, page_size, %d] of %s" % (nkv, d, qkv.dtype))
            num_pages, ps = k_pages.shape[0], k_pages.shape[2]
            if v_pages is None or tuple(v_pages.shape) != (num_pages, nkv, d, ps) or not v_pages.is_contiguous() \
                    or v_pages.dtype != qkv.dtype:
                raise ValueError("v_pages must be contiguous [%d, %d, %d, %d] of %s" % (num_pages, nkv, d, ps, qkv.dtype))
        base = qkv.data_ptr()
        q = ctypes.c_void_p(base)
        k = ctypes.c_void_p(base + nh * d * es)
        v = ctypes.c_void_p(base + (nh + nkv) * d * es)
        self._check(self.lib.lmsf_rope_cache_write(
            q, k, v, _code(qkv.dtype), N, qkv.stride(0), _ptr(positions), _ptr(table), rot_dim, 1 if neox else 0,
            max_pos, _ptr(slots), _ptr(k_pages), _ptr(v_pages), num_pages, nh, nkv, d, ps, self._stream()))

    def _check_qkv_fused(self, bias, weight, N, table, d, positions, slots, M, k_pages, v_pages, nkv):
        """Operand checks of the fused QKV forms; returns (pages, page size)."""
        if bias is not None and (bias.shape != (N,) or bias.dtype != weight.dtype or not bias.is_contiguous()):
            raise ValueError("qkv_rope_cache: bias must be [%d] of the weight's dtype" % N)
        if table.dtype != torch.float32 or table.dim() != 2 or table.shape[1] != d or not table.is_contiguous():
            raise ValueError("rotary table must be contiguous float32 [max_pos, %d]" % d)
        self._i32(positions, "positions", M)
        self._i32(slots, "slots", M)
        if k_pages.dim() != 4 or k_pages.shape[1] != nkv or k_pages.shape[3] != d or not k_pages.is_contiguous():
            raise ValueError("k_pages must be contiguous [pages, %d, page_size, %d]" % (nkv, d))
        num_pages, ps = k_pages.shape[0], k_pages.shape[2]
        if v_pages is None or tuple(v_pages.shape) != (num_pages, nkv, d, ps) or not v_pages.is_contiguous() \
                or v_pages.dtype != torch.bfloat16:
            raise ValueError("v_pages must be contiguous bfloat16 [%d, %d, %d, %d]" % (num_pages, nkv, d, ps))
        return num_pages, ps

    def qkv_rope_cache(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], nh: int, nkv: int,
                       d: int, positions: torch.Tensor, table: Optional[torch.Tensor], rot_dim: int, neox: bool,
                       slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor],
                       v_pages: Optional[torch.Tensor]) -> torch.Tensor:
        """The fused QKV projection, the rotation of its q and k heads and the write of k and v into the
        pages: ``linear`` followed by ``rope_cache_write``, with the same results. With few bfloat16 rows and
        a NeoX rotation over the whole head, the rotation and the write are the product's epilogue. ``x`` may
        be a ``ScaledRows``."""
        M, K = x.shape
        N = (nh + 2 * nkv) * d
        scaled = isinstance(x, ScaledRows)
        xt = x.xw if scaled else x
        fused_shape = (table is not None and slots is not None and neox and rot_dim == d and d % 32 == 0
                       and weight.dtype == torch.bfloat16 and tuple(weight.shape) == (N, K) and xt.stride(1) == 1
                       and weight.stride(1) == 1 and k_pages is not None and k_pages.dtype == torch.bfloat16)
        rt = D.Route()
        self.lib.lmsf_route_qkv(ctypes.byref(self._tun), ctypes.byref(self._shape(xt, weight, xt.dtype)),
                                1 if fused_shape else 0, x.rows_per_tile if scaled else 0, ctypes.byref(rt))
        if rt.route == D.MATERIALIZE:
            return self.qkv_rope_cache(self.materialize(x), weight, bias, nh, nkv, d, positions, table, rot_dim,
                                       neox, slots, k_pages, v_pages)
        if rt.route != D.SEPARATE:
            self._dev(xt, weight, bias, positions, table, slots, k_pages, v_pages)
            num_pages, ps = self._check_qkv_fused(bias, weight, N, table, d, positions, slots, M, k_pages, v_pages, nkv)
            y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
            head = (_ptr(xt), xt.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(y), y.stride(0), M, K,
                    _ptr(positions), _ptr(table), table.shape[0], _ptr(slots), _ptr(k_pages), _ptr(v_pages), num_pages,
                    nh, nkv, d, ps)
            if rt.route == D.GEMV_SCALED:
                self._dev(x.sumsq)
                self._check(self.lib.lmsf_gemv_scaled_qkv_rope_cache(*head, _ptr(x.sumsq), x.tiles, x.eps, self._stream()))
            elif rt.route == D.SKINNY_SCALED:
                self._dev(x.sumsq)
                self._check(self.lib.lmsf_gemm_qkv_rope_cache_scaled(*head, _ptr(x.sumsq), x.tiles, x.eps, self._stream()))
            elif rt.route == D.GEMV:
                self._check(self.lib.lmsf_gemv_qkv_rope_cache(*head, self._stream()))
            else:
                self._check(self.lib.lmsf_gemm_qkv_rope_cache(*head, self.skinny_variant, self._stream()))
            return y
        y = self.linear(x, weight, bias, pending_ok=bool(rt.pending))
        if isinstance(y, PendingProduct):
            # 17 and more rows with K split: the rotation and the cache write add up the partial sums themselves
            if (table is None and slots is None) or tuple(weight.shape) != (N, K):
                return self.materialize(y)
            return self._rope_cache_write_pending(y, nh, nkv, d, positions, table, rot_dim, neox, slots, k_pages,
                                                  v_pages)
        if table is not None or slots is not None:
            self.rope_cache_write(y, nh, nkv, d, positions, table, rot_dim, neox, slots, k_pages, v_pages)
        return y

    def _rope_cache_write_pending(self, p: PendingProduct, nh: int, nkv: int, d: int,
                                  positions: Optional[torch.Tensor], table: Optional[torch.Tensor], rot_dim: int,
                                  neox: bool, slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor],
                                  v_pages: Optional[torch.Tensor]) -> torch.Tensor:
        M, N = p.shape
        y = torch.empty((M, N), dtype=torch.bfloat16, device=p.device)
        self._dev(positions, table, slots, k_pages, v_pages)
        max_pos = 0
        if table is not None:
            if table.dtype != torch.float32 or table.dim() != 2 or table.shape[1] != rot_dim or not table.is_contiguous():
                raise ValueError("rotary table must be contiguous float32 [max_pos, %d]" % rot_dim)
            if positions is None:
                raise ValueError("rotation needs positions")
            self._i32(positions, "positions", M)
            max_pos = table.shape[0]
        num_pages, ps = 0, 1
        if slots is not None:
            self._i32(slots, "slots", M)
            if k_pages is None or k_pages.dim() != 4 or k_pages.shape[1] != nkv or k_pages.shape[3] != d \
                    or not k_pages.is_contiguous() or k_pages.dtype != torch.bfloat16:
                raise ValueError("k_pages must be contiguous bfloat16 [pages, %d, page_size, %d]" % (nkv, d))
            num_pages, ps = k_pages.shape[0], k_pages.shape[2]
            if v_pages is None or tuple(v_pages.shape) != (num_pages, nkv, d, ps) or not v_pages.is_contiguous() \
                    or v_pages.dtype != torch.bfloat16:
                raise ValueError("v_pages must be contiguous bfloat16 [%d, %d, %d, %d]" % (num_pages, nkv, d, ps))
        self._check(self.lib.lmsf_rope_cache_write_partial(
            _ptr(p.partials), _ptr(p.bias), p.partials.shape[0], _ptr(y), y.stride(0), M, _ptr(positions), _ptr(table),
            rot_dim, 1 if neox else 0, max_pos, _ptr(slots), _ptr(k_pages), _ptr(v_pages), num_pages, nh, nkv, d, ps,
            self._stream()))
        return y

    # ------------------------------------------------------------------ attention

    @staticmethod
    def check_head_dim(d: int, limit: int = 256) -> None:
        """Raises if no attention kernel takes head size ``d``: the matrix-core kernels take multiples of 16
        up to 256 (bfloat16), the general kernel multiples of 4 up to 1,024 (either dtype). Parts ask this when
        they are built, before any weight is loaded; ``limit`` is the widest head the part wants served (256
        keeps a part on kernels that have a matrix-core form)."""
        if d <= 0 or d % 4 != 0 or d > min(limit, 1024):
            raise ValueError("head size %d is not supported by the attention kernels: they take multiples of 4 "
                             "up to %d (multiples of 16 up to 256 on the matrix cores)" % (d, min(limit, 1024)))

    def paged_attention(self, q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                        block_tables: torch.Tensor, seg: torch.Tensor, pos: torch.Tensor, nh: int, nkv: int, d: int,
                        scale: float, window: int = 0, batch=None, kernel: Optional[str] = None,
                        chunk: int = 0, weights_f32: bool = False, softcap: float = 0.0) -> torch.Tensor:
        """Attention of every query token over the cached keys of its request: those at positions up to its own,
        within the last ``window`` positions if a window is given, or within its own chunk of ``chunk`` positions
        (chunks counted from position 0 of the request) if a chunk size is given. ``weights_f32``: in a bfloat16 run
        the softmax weights enter the product with the values in full float32 (as three bfloat16 parts on the
        matrix cores) instead of rounded to bfloat16; scores, maxima and sums are float32 either way. ``softcap``
        c > 0: a scaled score s enters the softmax as c tanh(s / c).

        ``q`` is [N, >= nh*d] with unit column stride (it may be the fused QKV buffer, of which the
        first nh*d columns are read). ``k_pages`` [pages, nkv, page_size, d], ``v_pages``
        [pages, nkv, d, page_size]. ``block_tables`` int32 [S, W]; ``seg``, ``pos`` int32 [N].
        ``batch`` (engine.batch.StepContext) carries host-side facts about the step for the choice of
        kernel; without it they are read back from ``seg`` and ``pos``. ``kernel`` forces "generic" or
        "mfma" (tests). Returns [N, nh*d] in q's dtype.
        """
        self._dev(q, k_pages, v_pages, block_tables, seg, pos)
        if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < nh * d:
            raise ValueError("q must be [N, >= %d] with unit column stride" % (nh * d))
        N = q.shape[0]
        if k_pages.dim() != 4 or k_pages.shape[1] != nkv or k_pages.shape[3] != d or not k_pages.is_contiguous() \
                or k_pages.dtype != q.dtype:
            raise ValueError("k_pages must be contiguous [pages, %d, page_size, %d] of %s" % (nkv, d, q.dtype))
        num_pages, ps = k_pages.shape[0], k_pages.shape[2]
        if tuple(v_pages.shape) != (num_pages, nkv, d, ps) or not v_pages.is_contiguous() or v_pages.dtype != q.dtype:
            raise ValueError("v_pages must be contiguous [%d, %d, %d, %d] of %s" % (num_pages, nkv, d, ps, q.dtype))
        if block_tables.dim() != 2:
            raise ValueError("block_tables must be [segments, width]")
        self._i32(block_tables, "block_tables")
        self._i32(seg, "seg", N)
        self._i32(pos, "pos", N)
        out = torch.empty((N, nh * d), dtype=q.dtype, device=q.device)
        if N == 0:
            return out
        if chunk:
            if window or chunk < 0:
                raise ValueError("paged_attention takes a window or a chunk size (> 0), not both")
            window = -int(chunk)        # the kernels' encoding of a chunk mask (csrc/common.h: first_visible_key)
        fast_ok = (q.dtype == torch.bfloat16 and d % 16 == 0 and 16 <= d <= 256 and ps % 4 == 0
                   and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0 and scale > 0)
        if kernel == "mfma" and not fast_ok:
            raise ValueError("the matrix-core attention kernels need bfloat16, a head size that is a multiple of 16 "
                             "up to 256, a page size that is a multiple of 4, 16-byte aligned query rows and a positive scale")
        if kernel == "generic" or not fast_ok:
            self._check(self.lib.lmsf_paged_attention_generic_capped(
                _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pages), _ptr(v_pages), num_pages,
                _ptr(block_tables), block_tables.shape[1], _ptr(seg), _ptr(pos), N, nh, nkv, d, ps, float(scale),
                int(window or 0), float(softcap), _code(q.dtype), self._stream()))
            return out
        plan = self._attention_plan(batch, seg, pos, nh, nkv)
        exact = self.ATTENTION_WEIGHTS_F32 if weights_f32 else 0
        common = (_ptr(k_pages), _ptr(v_pages), num_pages, _ptr(block_tables), block_tables.shape[1])
        if plan.tiles is not None:
            self._check(self.lib.lmsf_paged_attention_prefill_mfma_capped(
                _ptr(q), q.stride(0), _ptr(out), out.stride(0), *common, _ptr(plan.tiles), plan.n_tiles,
                _ptr(seg), _ptr(pos), nh, nkv, d, ps, float(scale), int(window or 0), float(softcap),
                self.prefill_attention_variant + exact, self._stream()))
        if plan.n_single:
            c_chunk, c_splits = ctypes.c_int(0), ctypes.c_int(0)
            self.lib.lmsf_route_decode_attention(ctypes.byref(self._tun), plan.n_single, nh, nkv, plan.max_context,
                                                 ctypes.byref(c_chunk), ctypes.byref(c_splits))
            chunk, n_splits = c_chunk.value, c_splits.value
            floats = self.lib.lmsf_attention_decode_scratch_floats(plan.n_single, nh, d, n_splits)
            scratch = torch.empty(floats if n_splits > 1 else 1, dtype=torch.float32, device=q.device)
            self._check(self.lib.lmsf_paged_attention_decode_mfma_capped(
                _ptr(q), q.stride(0), _ptr(out), out.stride(0), *common, _ptr(plan.single_tokens), plan.n_single,
                None if plan.token_is_request else _ptr(seg), _ptr(pos), nh, nkv, d, ps, float(scale),
                int(window or 0), float(softcap), chunk, n_splits, _ptr(scratch), self.decode_attention_order + exact,
                self._stream()))
        return out

    ATTENTION_WEIGHTS_F32 = 256     # csrc/entry_points.h: LMSF_ATTENTION_WEIGHTS_F32

    def _attention_plan(self, batch, seg: torch.Tensor, pos: torch.Tensor, nh: int, nkv: int) -> "_AttentionPlan":
        """How a step's tokens are split between the two matrix-core kernels: requests with one token go
        to the decode kernel, the others are cut into tiles for the prefill kernel. Computed once per step
        and tile size, and kept on the batch for the other layers."""
        tq = self.lib.lmsf_attention_tile_tokens(nh, nkv)
        if batch is not None:
            aux = batch.aux
            key = ("attention_plan", tq)
            if key in aux:
                return aux[key]
            lens, starts, max_context = batch.host_seg_lens, batch.host_seg_starts, batch.max_context
            first_pos = batch.host_seg_first_pos
            if batch.replayed or batch.all_single:
                # the order matters from 16 tokens on (the kernel starts the longest contexts first); below that
                # the tokens are taken as they come, which saves the kernel the trip to the list
                order = getattr(batch, "longest_first", None) if batch.n_tokens >= 16 else None
                plan = _AttentionPlan(None, 0, order, batch.n_tokens, max_context, token_is_request=True)
                aux[key] = plan
                return plan
        else:
            seg_h = seg.tolist()
            lens, starts = [], []
            for i, sg in enumerate(seg_h):
                if i == 0 or sg != seg_h[i - 1]:
                    starts.append(i)
                    lens.append(0)
                lens[-1] += 1
            pos_h = pos.tolist()
            max_context = max(pos_h) + 1
            first_pos = [pos_h[st] for st in starts]
            aux, key = None, None
        by_keys, single = [], []
        for st, n, p0 in zip(starts, lens, first_pos):
            if n == 1:
                single.append((p0, st))
            else:
                for t in range(0, n, tq):
                    by_keys.append((p0 + t + min(tq, n - t), st + t, min(tq, n - t)))
        # the tiles with the most keys first: the prefill kernel starts its workgroups in this order
        by_keys.sort(key=lambda e: -e[0])
        tiles = [x for e in by_keys for x in e[1:]]
        # likewise the single tokens with the longest contexts first
        single = [st for _, st in sorted(single, key=lambda e: -e[0])]
        dev = seg.device
        if len(single) == len(lens):
            plan = _AttentionPlan(None, 0, None, len(single), max_context)
        else:
            both = self.upload_ints(tiles + single, dev)
            plan = _AttentionPlan(both[:len(tiles)], len(tiles) // 2,
                                  both[len(tiles):] if single else None, len(single), max_context)
        if aux is not None:
            aux[key] = plan
        return plan

    def upload_ints(self, values, dev: torch.device) -> torch.Tensor:
        """int32 values to the device through pinned memory, without waiting for the copy. Four buffers take
        turns; before a buffer is written again its last copy's event is waited for (long past, as a rule)."""
        n = len(values)
        turn = self._pinned_turn = (getattr(self, "_pinned_turn", -1) + 1) % 4
        bufs = self.__dict__.setdefault("_pinned_ints", [None] * 4)
        events = self.__dict__.setdefault("_pinned_events", [None] * 4)
        if events[turn] is not None:
            events[turn].synchronize()
        if bufs[turn] is None or bufs[turn].numel() < n:
            bufs[turn] = torch.empty(max(n, 4096), dtype=torch.int32, pin_memory=True)
        host = bufs[turn][:n]
        host.numpy()[:] = values
        out = host.to(dev, non_blocking=True)
        if events[turn] is None:
            events[turn] = torch.cuda.Event()
        events[turn].record()
        return out

    # ------------------------------------------------------------------ norm in groups, latent attention, experts

    def group_norm(self, x: Optional[torch.Tensor] = None, x_weight: Optional[torch.Tensor] = None,
                   residual: Optional[torch.Tensor] = None, out_weight: Optional[torch.Tensor] = None, groups: int = 1,
                   x_eps: float = 1e-5, out_eps: float = 1e-5, out_dtype: Optional[torch.dtype] = None,
                   rows: Optional[torch.Tensor] = None, history: Optional[torch.Tensor] = None, index: int = 0,
                   mix: Optional[torch.Tensor] = None, want_out: bool = True) -> Optional[torch.Tensor]:
        """RMS norm in ``groups`` equal consecutive parts of a row, gn(v; w) = v / rms of v's part * w, around a
        float32 stream; every operand is optional (csrc/group_norm.hip):

            r = (residual[rows] if residual is given else 0) + (gn(x; x_weight) if x is given else 0)
            residual <- r                                     (x and residual given, no rows)
            history[index] <- r; r = sum_j<=index mix[j] history[j]; residual <- r        (history given)
            returns gn(r; out_weight) (or r itself without out_weight) in out_dtype, unless want_out is False

        ``x`` is [N, W] float32 or bfloat16 with unit column stride (a view of a wider buffer will do),
        ``residual`` contiguous float32 [N, W], ``history`` contiguous float32 [L, N, W], the weights float32 [W]."""
        self._dev(x, x_weight, residual, out_weight, rows, history, mix)
        ref = x if x is not None else residual
        if ref is None or ref.dim() != 2:
            raise ValueError("group_norm needs x or a residual, [N, W]")
        N, W = ref.shape
        if x is not None:
            if x.stride(1) != 1 or x_weight is None:
                raise ValueError("group_norm: x needs unit column stride and its weight")
        for w in (x_weight, out_weight, mix):
            if w is not None and (w.dtype != torch.float32 or not w.is_contiguous()):
                raise ValueError("group_norm: weights must be contiguous float32")
        if x_weight is not None and x_weight.shape != (W,) or out_weight is not None and out_weight.shape != (W,):
            raise ValueError("group_norm: weights must be [%d]" % W)
        if residual is not None:
            if residual.dtype != torch.float32 or not residual.is_contiguous() or residual.shape[1] != W:
                raise ValueError("group_norm: the residual stream must be contiguous float32 [N, %d]" % W)
            if rows is None and residual.shape[0] != N:
                raise ValueError("group_norm: x and the residual differ in rows")
        self._i32(rows, "rows")
        n_out = N if rows is None else rows.numel()
        if rows is not None and x is not None:
            raise ValueError("group_norm: rows select from the residual only")
        hist_stride = 0
        if history is not None:
            if history.dtype != torch.float32 or not history.is_contiguous() or tuple(history.shape[1:]) != (N, W) \
                    or not (0 <= index < history.shape[0]) or mix is None or mix.numel() < index + 1 \
                    or residual is None or rows is not None:
                raise ValueError("group_norm: history must be float32 [L > index, %d, %d] with index + 1 weights" % (N, W))
            hist_stride = history.stride(0)
        out = None
        if want_out:
            out = torch.empty((n_out, W), dtype=out_dtype or ref.dtype, device=ref.device)
        self._check(self.lib.lmsf_group_norm(
            _ptr(x), _code(x.dtype) if x is not None else F32, x.stride(0) if x is not None else W, _ptr(x_weight),
            _ptr(residual), _ptr(history), hist_stride, int(index), _ptr(mix), _ptr(out_weight), _ptr(out),
            _code(out.dtype) if out is not None else F32, W, _ptr(rows), n_out, W, int(groups), float(x_eps),
            float(out_eps), self._stream()))
        return out

    def latent_cache_write(self, x: torch.Tensor, weight: torch.Tensor, eps: float, rank: int, rot_width: int,
                           positions: torch.Tensor, table: torch.Tensor, slots: torch.Tensor, k_pages: torch.Tensor,
                           v_pages: torch.Tensor, also_norm: Optional[torch.Tensor] = None,
                           also_weight: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Per token: c = rms_norm(x[:rank]) * weight, r = rotate(x[rank:rank + rot_width]) by the token's position
        (``table`` float32 [max_pos, rot] = [cos | sin], the first ``rot`` entries of r in pairs (i, i + rot/2));
        [c | r | zeros] goes to the token's slot of ``k_pages`` [pages, 1, page_size, D] and of ``v_pages``
        [pages, 1, D, page_size]. A negative slot stores nothing. ``also_norm``: another view of the same rows (same
        row stride) whose plain RMS norm with ``also_weight`` and the same eps is returned, from the same launch."""
        self._dev(x, weight, positions, table, slots, k_pages, v_pages, also_norm, also_weight)
        q_out = None
        if also_norm is not None:
            if also_norm.stride(0) != x.stride(0) or also_norm.stride(1) != 1 or also_norm.shape[0] != x.shape[0] \
                    or also_norm.dtype != x.dtype or also_weight is None or also_weight.dtype != torch.float32 \
                    or also_weight.shape != (also_norm.shape[1],) or not also_weight.is_contiguous():
                raise ValueError("latent_cache_write: the second norm's operand must be a view of the same rows, its "
                                 "weight contiguous float32")
            q_out = torch.empty(tuple(also_norm.shape), dtype=x.dtype, device=x.device)
        N = x.shape[0]
        if x.dim() != 2 or x.stride(1) != 1 or x.shape[1] < rank + rot_width:
            raise ValueError("latent_cache_write: x must be [N, >= %d] with unit column stride" % (rank + rot_width))
        if weight.dtype != torch.float32 or weight.shape != (rank,) or not weight.is_contiguous():
            raise ValueError("latent_cache_write: weight must be contiguous float32 [%d]" % rank)
        if table.dtype != torch.float32 or table.dim() != 2 or not table.is_contiguous() or table.shape[1] > rot_width \
                or table.shape[1] % 2:
            raise ValueError("latent_cache_write: bad rotary table")
        self._i32(positions, "positions", N)
        self._i32(slots, "slots", N)
        if k_pages.dim() != 4 or k_pages.shape[1] != 1 or k_pages.shape[3] < rank + rot_width or k_pages.dtype != x.dtype \
                or not k_pages.is_contiguous():
            raise ValueError("latent_cache_write: k_pages must be contiguous [pages, 1, page_size, >= %d] of %s"
                             % (rank + rot_width, x.dtype))
        P, _, ps, D = k_pages.shape
        if tuple(v_pages.shape) != (P, 1, D, ps) or v_pages.dtype != x.dtype or not v_pages.is_contiguous():
            raise ValueError("latent_cache_write: v_pages must be contiguous [%d, 1, %d, %d] of %s" % (P, D, ps, x.dtype))
        self._check(self.lib.lmsf_latent_cache_write(
            _ptr(x), _code(x.dtype), x.stride(0), _ptr(weight), float(eps), _ptr(positions), _ptr(table),
            table.shape[1], table.shape[0], _ptr(slots), _ptr(k_pages), _ptr(v_pages), P, N, int(rank), int(rot_width),
            D, ps, _ptr(also_norm), _ptr(also_weight), _ptr(q_out), q_out.stride(0) if q_out is not None else 0,
            also_norm.shape[1] if also_norm is not None else 0, self._stream()))
        return q_out

    def head_linear(self, x: torch.Tensor, x_head: int, weight: torch.Tensor, out: torch.Tensor, out_head: int,
                    gate: Optional[torch.Tensor] = None, rope_tail=None, gate_wide: bool = False) -> torch.Tensor:
        """Per-head products: out[n, h * out_head + o] = sum_k weight[h, o, k] x[n, h * x_head + k], times
        sigmoid(gate[n, h]) if a gate is given (``gate_wide``: a gate per output, sigmoid(gate[n, h * O + o])).
        ``weight`` contiguous [H, O, K]; x, out and gate are views with
        unit column stride whose first column is head 0's first entry. ``rope_tail`` = (x_at, out_at, width,
        positions, table): also what ``rope_tail`` does with these arguments, from the same launch where it can be."""
        self._dev(x, weight, out, gate)
        x_at = out_at = width = rot = max_pos = 0
        positions = table = None
        if rope_tail is not None:
            x_at, out_at, width, positions, table = rope_tail
            self._dev(positions, table)
            if table.dtype != torch.float32 or table.dim() != 2 or not table.is_contiguous() or table.shape[1] > width:
                raise ValueError("head_linear: bad rotary table")
            self._i32(positions, "positions", x.shape[0])
            rot, max_pos = table.shape[1], table.shape[0]
        H, O, K = weight.shape
        N = x.shape[0]
        if not weight.is_contiguous() or weight.dtype != x.dtype or out.dtype != x.dtype:
            raise ValueError("head_linear: weight must be contiguous and of x's dtype, as the output")
        if x.stride(1) != 1 or out.stride(1) != 1 or x.shape[1] < (H - 1) * x_head + K \
                or out.shape[1] < (H - 1) * out_head + O or out.shape[0] != N:
            raise ValueError("head_linear: operands too narrow for %d heads" % H)
        need = H * O if gate_wide else H
        if gate is not None and (gate.dtype != x.dtype or gate.stride(1) != 1 or gate.shape[1] < need or gate.shape[0] != N):
            raise ValueError("head_linear: gate must be [N, >= %d] of x's dtype" % need)
        self._check(self.lib.lmsf_head_linear(
            _ptr(x), _code(x.dtype), x.stride(0), int(x_head), _ptr(weight), _ptr(out), out.stride(0), int(out_head),
            _ptr(gate), gate.stride(0) if gate is not None else 0, N, H, O, K, _ptr(positions), _ptr(table), rot, max_pos,
            int(x_at), int(out_at), int(width), 1 if (gate_wide and gate is not None) else 0, self._stream()))
        return out

    def rope_tail(self, x: torch.Tensor, x_head: int, x_at: int, out: torch.Tensor, out_head: int, out_at: int,
                  heads: int, width: int, positions: torch.Tensor, table: torch.Tensor) -> None:
        """For every head h: out[n, h * out_head + out_at + e] = rotate(x[n, h * x_head + x_at + e]) for e < width
        (the first ``rot`` = table.shape[1] of them in pairs (e, e + rot/2), the others as they are); the rest of
        the head behind them in ``out`` is zeroed."""
        self._dev(x, out, positions, table)
        N = x.shape[0]
        if x.stride(1) != 1 or out.stride(1) != 1 or x.shape[1] < heads * x_head or out.shape[1] < heads * out_head \
                or out.shape[0] != N or out.dtype != x.dtype:
            raise ValueError("rope_tail: operands too narrow for %d heads" % heads)
        if table.dtype != torch.float32 or table.dim() != 2 or not table.is_contiguous() or table.shape[1] > width:
            raise ValueError("rope_tail: bad rotary table")
        self._i32(positions, "positions", N)
        self._check(self.lib.lmsf_rope_tail(
            _ptr(x), _code(x.dtype), x.stride(0), int(x_head), int(x_at), _ptr(out), out.stride(0), int(out_head),
            int(out_at), _ptr(positions), _ptr(table), table.shape[1], table.shape[0], N, int(heads), int(width),
            self._stream()))

    def table_moe(self, h: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor, token_ids: Optional[torch.Tensor],
                  table: torch.Tensor, weight: float, base: Optional[torch.Tensor] = None,
                  pair_scale: Optional[torch.Tensor] = None, base_scale: Optional[torch.Tensor] = None,
                  out_scale: Optional[torch.Tensor] = None, gated: bool = True) -> torch.Tensor:
        """out[n] = base[n] + weight * sum_k down_e(silu(gate_e h[n]) * up_e h[n]) over e = table[token_ids[n], k].
        ``gated`` False: experts of one matrix, ``w_gate_up`` [E, F, W], down_e(relu(up_e h[n])^2). ``out_scale``
        (float32 [N, top]): what the expert of (n, k) returns is multiplied by out_scale[n, k].
        ``w_gate_up`` [E, 2 F, W] (gate rows first), ``w_down`` [E, W, F], ``table`` int32 [vocab, top].
        ``token_ids`` None: row n of the table is token n's choice (a router's, ``moe_route``). ``pair_scale``
        (float32 [N, top]): the expert of (n, k) gets pair_scale[n, k] * h[n] as its input. ``base_scale``
        (float32 [N]): base[n] is multiplied by it."""
        self._dev(h, w_gate_up, w_down, token_ids, table, base, pair_scale, base_scale)
        N, W = h.shape
        E, F2, _ = w_gate_up.shape
        F = F2 // 2 if gated else F2
        if tuple(w_gate_up.shape) != (E, (2 if gated else 1) * F, W) or tuple(w_down.shape) != (E, W, F) or not w_gate_up.is_contiguous() \
                or not w_down.is_contiguous() or w_gate_up.dtype != h.dtype or w_down.dtype != h.dtype:
            raise ValueError("table_moe: expert weights must be contiguous [E, 2F, W] and [E, W, F] of h's dtype")
        if h.stride(1) != 1 or (base is not None and (base.shape != h.shape or base.stride(1) != 1 or base.dtype != h.dtype)):
            raise ValueError("table_moe: h and base must be [N, W] with unit column stride")
        self._i32(token_ids, "token_ids", N)
        if table.dtype != torch.int32 or table.dim() != 2 or not table.is_contiguous():
            raise ValueError("table_moe: table must be contiguous int32 [vocab, top]")
        vocab, top = table.shape
        if token_ids is None and vocab < N:
            raise ValueError("table_moe: without token ids the table needs a row per token")
        if pair_scale is not None and (pair_scale.dtype != torch.float32 or pair_scale.numel() != N * top
                                       or not pair_scale.is_contiguous()):
            raise ValueError("table_moe: pair_scale must be contiguous float32 [%d, %d]" % (N, top))
        if base_scale is not None and (base is None or base_scale.dtype != torch.float32 or base_scale.numel() != N
                                       or not base_scale.is_contiguous()):
            raise ValueError("table_moe: base_scale must be contiguous float32 [%d] beside a base" % N)
        if out_scale is not None and (out_scale.dtype != torch.float32 or out_scale.numel() != N * top
                                      or not out_scale.is_contiguous()):
            raise ValueError("table_moe: out_scale must be contiguous float32 [%d, %d]" % (N, top))
        self._dev(out_scale)
        act = torch.empty((N * top, F), dtype=h.dtype, device=h.device)
        out = torch.empty((N, W), dtype=h.dtype, device=h.device)
        ints = rows = None
        if self.lib.lmsf_table_moe_grouped(_code(h.dtype), N, top, E, F, W, h.stride(0)):
            # many tokens: grouped by expert on the device, tiles on the matrix cores
            ints = torch.empty(self.lib.lmsf_table_moe_scratch_ints(N, top, E), dtype=torch.int32, device=h.device)
            rows = torch.empty((N * top, W), dtype=torch.float32, device=h.device)
        self._check(self.lib.lmsf_table_moe_act(
            _ptr(h), _code(h.dtype), h.stride(0), _ptr(w_gate_up), _ptr(w_down), _ptr(token_ids), _ptr(table), vocab,
            top, E, float(weight), _ptr(base), base.stride(0) if base is not None else 0, _ptr(pair_scale),
            _ptr(base_scale), _ptr(out_scale), 0 if gated else 1, _ptr(act), _ptr(out), out.stride(0), N, F, W,
            _ptr(ints), _ptr(rows), self._stream()))
        return out

    def moe_route_groups(self, logits: torch.Tensor, experts: int, top: int, softmax: bool = True, groups: int = 1,
                         keep: int = 1, renorm: bool = False):
        """A router's choice from float32 logits [N, >= experts] with scores softmax(logits) over all experts (or
        sigmoid), where only experts of the ``keep`` best of ``groups`` equal groups of neighbours may be chosen (a
        group's score is its best expert's): (choice int32 [N, top], weight float32 [N, top]), the weights the
        chosen experts' scores, over their sum with ``renorm``."""
        self._dev(logits)
        if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1 or logits.shape[1] < experts:
            raise ValueError("moe_route_groups: logits must be float32 [N, >= %d] with unit column stride" % experts)
        if not (0 < top <= experts and top <= 64) or not (0 < keep <= groups <= 256) or experts % groups \
                or keep * (experts // groups) < top:
            raise ValueError("moe_route_groups: %d of %d experts from %d of %d groups" % (top, experts, keep, groups))
        N = logits.shape[0]
        choice = torch.empty((N, top), dtype=torch.int32, device=logits.device)
        weight = torch.empty((N, top), dtype=torch.float32, device=logits.device)
        self._check(self.lib.lmsf_moe_route_groups(_ptr(logits), logits.stride(0), N, int(experts), int(top),
                                                   1 if softmax else 0, int(groups), int(keep), 1 if renorm else 0,
                                                   _ptr(choice), _ptr(weight), self._stream()))
        return choice, weight

    def moe_route(self, logits: torch.Tensor, experts: int, top: int, renorm: bool = False, extra: int = -1):
        """A router's choice from float32 logits [N, >= experts]: (choice int32 [N, top], weight float32 [N, top],
        gate float32 [N] or None). Scores are sigmoid(logits); the ``top`` largest choose (the largest first, the
        lower index among equals); the weights are their scores, divided by their sum with ``renorm``. ``extra``
        >= 0 names a column beside the experts' whose sigmoid is returned as ``gate``."""
        self._dev(logits)
        if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1 or logits.shape[1] < experts \
                or extra >= logits.shape[1]:
            raise ValueError("moe_route: logits must be float32 [N, >= %d] with unit column stride" % experts)
        if not (0 < top <= experts and top <= 64):
            raise ValueError("moe_route: %d of %d experts (at most 64 a token)" % (top, experts))
        N = logits.shape[0]
        choice = torch.empty((N, top), dtype=torch.int32, device=logits.device)
        weight = torch.empty((N, top), dtype=torch.float32, device=logits.device)
        gate = torch.empty((N,), dtype=torch.float32, device=logits.device) if extra >= 0 else None
        self._check(self.lib.lmsf_moe_route(_ptr(logits), logits.stride(0), N, int(experts), int(top), 1 if renorm else 0,
                                            int(extra), _ptr(choice), _ptr(weight), _ptr(gate), self._stream()))
        return choice, weight, gate

    # ------------------------------------------------------------------ what a token brings beside its embedding

    def hashed_pair_embedding(self, batch, table: torch.Tensor, pairs: torch.Tensor, prev_state: torch.Tensor,
                              mul_prev: int, mul_cur: int, keep: bool = False):
        """float32 [N, W] = table[id] + pairs[(previous id * mul_prev + id * mul_cur) mod buckets], the last row of
        ``pairs`` ([buckets + 1, W]) for a request's first token. The id before a segment's first token is
        ``prev_state[slot]`` (int32, an entry per state slot and the spare one), which is brought up to date.
        ``keep``: also returns a second copy of the result."""
        ids = batch.token_ids
        N = ids.numel()
        self._dev(ids, table, pairs, prev_state, batch.positions)
        if table.dim() != 2 or pairs.dim() != 2 or pairs.shape[1] != table.shape[1] or pairs.shape[0] < 2 \
                or table.dtype != pairs.dtype or not table.is_contiguous() or not pairs.is_contiguous():
            raise ValueError("hashed_pair_embedding: table [V, W] and pairs [buckets + 1, W] of one dtype are needed")
        if prev_state.dtype != torch.int32 or not prev_state.is_contiguous():
            raise ValueError("hashed_pair_embedding: prev_state must be contiguous int32")
        self._i32(ids, "token_ids", N)
        self._i32(batch.positions, "positions", N)
        seg_of, seg_starts, slots, S = self._segments(batch, N)
        V, W = table.shape
        out = torch.empty((N, W), dtype=torch.float32, device=table.device)
        kept = torch.empty((N, W), dtype=torch.float32, device=table.device) if keep else None
        self._check(self.lib.lmsf_hashed_pair_embedding(
            _ptr(ids), _ptr(batch.positions), _ptr(seg_of), _ptr(seg_starts), _ptr(slots), _ptr(prev_state), _ptr(table),
            _ptr(pairs), _code(table.dtype), _ptr(out), _ptr(kept), N, S, V, W, pairs.shape[0] - 1, int(mul_prev),
            int(mul_cur), self._stream()))
        return (out, kept) if keep else out

    def concat_rows(self, a: torch.Tensor, b: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        """[a | b] row by row in ``out_dtype``; a, b contiguous float32 [N, Wa], [N, Wb]."""
        self._dev(a, b)
        if a.dim() != 2 or b.dim() != 2 or a.shape[0] != b.shape[0] or a.dtype != torch.float32 \
                or b.dtype != torch.float32 or not a.is_contiguous() or not b.is_contiguous():
            raise ValueError("concat_rows: two contiguous float32 matrices of equal rows are needed")
        out = torch.empty((a.shape[0], a.shape[1] + b.shape[1]), dtype=out_dtype, device=a.device)
        self._check(self.lib.lmsf_concat_rows(_ptr(a), _ptr(b), _ptr(out), _code(out_dtype), a.shape[0], a.shape[1],
                                              b.shape[1], self._stream()))
        return out

    def gate_table(self, z: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, at: int) -> torch.Tensor:
        """gelu_tanh(z [N, dim]) * table[ids, at : at + dim], in z's dtype."""
        self._dev(z, ids, table)
        N, dim = z.shape
        if z.stride(1) != 1 or table.dim() != 2 or table.dtype != z.dtype or table.stride(1) != 1 \
                or not (0 <= at and at + dim <= table.shape[1]):
            raise ValueError("gate_table: z [N, dim] and a table [V, >= at + dim] of one dtype are needed")
        self._i32(ids, "token_ids", N)
        out = torch.empty((N, dim), dtype=z.dtype, device=z.device)
        self._check(self.lib.lmsf_gate_table(_ptr(z), z.stride(0), _ptr(ids), _ptr(table), table.stride(0), int(at),
                                             table.shape[0], _ptr(out), _code(z.dtype), N, dim, self._stream()))
        return out

    def relu_squared(self, z: torch.Tensor) -> torch.Tensor:
        """relu(z)^2, elementwise, in z's dtype; z [N, F] with unit column stride."""
        self._dev(z)
        if z.dim() != 2 or z.stride(1) != 1:
            raise ValueError("relu_squared: z must be [N, F] with unit column stride")
        out = torch.empty(tuple(z.shape), dtype=z.dtype, device=z.device)
        self._check(self.lib.lmsf_relu_squared(_ptr(z), z.stride(0), _ptr(out), _code(z.dtype), z.shape[0], z.shape[1],
                                               self._stream()))
        return out

    # ------------------------------------------------------------------ attention with norms and rotated values

    def attn_prepare_normed(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, heads: int, kv_heads: int, dim: int,
                            vdim: int, padded: int, positions: torch.Tensor, slots: Optional[torch.Tensor],
                            k_pages: torch.Tensor, v_pages: torch.Tensor, q_weight: Optional[torch.Tensor] = None,
                            k_weight: Optional[torch.Tensor] = None, eps: float = 1e-5,
                            table: Optional[torch.Tensor] = None, table_v: Optional[torch.Tensor] = None,
                            interleaved: bool = False, v_norm: bool = False) -> torch.Tensor:
        """Readies projected queries, keys and values for ``paged_attention`` at head size ``padded``, each step
        optional: one RMS norm over all of q with ``q_weight`` (float32 [heads * dim]) and one over all of k with
        ``k_weight``; rotation of the first table.shape[1] entries of every q and k head; every value head over its
        root mean square (``v_norm``); rotation of all of a value head (``table_v`` float32 [max_pos, vdim]). Pairs
        are (2m, 2m + 1) if ``interleaved`` else (m, m + rot / 2). k and v go to the tokens' slots of the pages.
        Returns q [N, heads * padded]."""
        self._dev(q, k, v, positions, slots, k_pages, v_pages, q_weight, k_weight, table, table_v)
        N = q.shape[0]
        for t, w, name in ((q, heads * dim, "q"), (k, kv_heads * dim, "k"), (v, kv_heads * vdim, "v")):
            if t.dim() != 2 or t.shape[0] != N or t.shape[1] < w or t.stride(1) != 1 or t.dtype != q.dtype:
                raise ValueError("attn_prepare_normed: %s must be [%d, >= %d] of q's dtype with unit column stride"
                                 % (name, N, w))
        self._i32(positions, "positions", N)
        self._i32(slots, "slots", N)
        if q_weight is not None:
            self._f32_vec(q_weight, heads * dim, "attn_prepare_normed: q_weight")
        if k_weight is not None:
            self._f32_vec(k_weight, kv_heads * dim, "attn_prepare_normed: k_weight")
        rot = 0
        max_pos = None
        for tb, width, name in ((table, None, "table"), (table_v, vdim, "table_v")):
            if tb is None:
                continue
            if tb.dtype != torch.float32 or tb.dim() != 2 or not tb.is_contiguous() or tb.shape[1] % 2 \
                    or (width is not None and tb.shape[1] != width) or (width is None and tb.shape[1] > dim) \
                    or (max_pos is not None and tb.shape[0] != max_pos):
                raise ValueError("attn_prepare_normed: %s must be contiguous float32 [max_pos, entries]" % name)
            max_pos = tb.shape[0]
        if table is not None:
            rot = table.shape[1]
        if k_pages.dim() != 4 or k_pages.shape[1] != kv_heads or k_pages.shape[3] != padded or not k_pages.is_contiguous() \
                or k_pages.dtype != q.dtype:
            raise ValueError("attn_prepare_normed: k_pages must be contiguous [pages, %d, page_size, %d] of %s"
                             % (kv_heads, padded, q.dtype))
        num_pages, ps = k_pages.shape[0], k_pages.shape[2]
        if tuple(v_pages.shape) != (num_pages, kv_heads, padded, ps) or not v_pages.is_contiguous() or v_pages.dtype != q.dtype:
            raise ValueError("attn_prepare_normed: v_pages must be contiguous [%d, %d, %d, %d] of %s"
                             % (num_pages, kv_heads, padded, ps, q.dtype))
        out = torch.empty((N, heads * padded), dtype=q.dtype, device=q.device)
        self._check(self.lib.lmsf_attn_prepare_normed(
            _ptr(q), q.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0), _code(q.dtype), _ptr(q_weight),
            _ptr(k_weight), float(eps), _ptr(positions), _ptr(table), rot, _ptr(table_v), int(max_pos or 1),
            1 if interleaved else 0, 1 if v_norm else 0, _ptr(slots), _ptr(out), out.stride(0), _ptr(k_pages),
            _ptr(v_pages), num_pages, N, int(heads), int(kv_heads), int(dim), int(vdim), int(padded), ps, self._stream()))
        return out

    def attn_finish(self, a: torch.Tensor, padded: int, heads: int, vdim: int, positions: torch.Tensor,
                    gate: Optional[torch.Tensor] = None, table_v: Optional[torch.Tensor] = None,
                    interleaved: bool = False) -> torch.Tensor:
        """The attention's result [N, heads * padded] made ready for the output projection: every head's first vdim
        entries, turned back by the token's position over all of them (``table_v`` float32 [max_pos, vdim]; None: not),
        times sigmoid(gate[n, h]) (``gate`` [N, >= heads], one number a head; None: none). Returns [N, heads * vdim]."""
        self._dev(a, positions, gate, table_v)
        N = a.shape[0]
        if a.dim() != 2 or a.stride(1) != 1 or a.shape[1] < heads * padded or padded < vdim:
            raise ValueError("attn_finish: a must be [N, >= %d] with unit column stride" % (heads * padded))
        self._i32(positions, "positions", N)
        if gate is not None and (gate.dim() != 2 or gate.shape[0] != N or gate.shape[1] < heads or gate.stride(1) != 1
                                 or gate.dtype != a.dtype):
            raise ValueError("attn_finish: gate must be [%d, >= %d] of a's dtype" % (N, heads))
        if table_v is not None and (table_v.dtype != torch.float32 or table_v.dim() != 2 or table_v.shape[1] != vdim
                                    or not table_v.is_contiguous()):
            raise ValueError("attn_finish: table_v must be contiguous float32 [max_pos, %d]" % vdim)
        out = torch.empty((N, heads * vdim), dtype=a.dtype, device=a.device)
        self._check(self.lib.lmsf_attn_finish(
            _ptr(a), a.stride(0), _ptr(gate), gate.stride(0) if gate is not None else 0, _code(a.dtype), _ptr(positions),
            _ptr(table_v), table_v.shape[0] if table_v is not None else 1, 1 if interleaved else 0, _ptr(out),
            out.stride(0), N, int(heads), int(vdim), int(padded), self._stream()))
        return out

    # ------------------------------------------------------------------ the gated delta rule

    def gated_delta_state_floats(self, heads: int, dim: int, vdim: int) -> int:
        return int(self.lib.lmsf_gated_delta_state_floats(heads, dim, vdim))

    def gated_delta(self, qkv: torch.Tensor, q_at: int, k_at: int, v_at: int, a: torch.Tensor, dt_bias: torch.Tensor,
                    a_log: torch.Tensor, b: torch.Tensor, state: torch.Tensor, batch, heads: int, kv_heads: int,
                    dim: int, vdim: int, q_scale: float, unit_eps: float = 1e-6) -> torch.Tensor:
        """The gated delta rule over each request's tokens, the memory S [heads, dim, vdim] carried in ``state``
        (float32 [slots, >= gated_delta_state_floats], laid out [heads, ceil(vdim / 4), dim, 4]): S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q, with
        q, k the unit vectors of columns q_at, k_at of ``qkv`` (kv_heads heads of dim; q times q_scale), v its columns
        from v_at (heads of vdim), beta = sigmoid(b [N, >= heads]) and g = exp(-exp(a_log [heads]) softplus(a + dt_bias))
        (``a`` float32 [N, heads * dim]). Returns the heads' o as float32 [N, heads * vdim]."""
        self._dev(qkv, a, dt_bias, a_log, b)
        N = qkv.shape[0]
        need = max(q_at + kv_heads * dim, k_at + kv_heads * dim, v_at + heads * vdim)
        if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < need:
            raise ValueError("gated_delta: qkv must be [N, >= %d] with unit column stride" % need)
        if a.dtype != torch.float32 or a.dim() != 2 or a.shape[0] != N or a.shape[1] < heads * dim or a.stride(1) != 1:
            raise ValueError("gated_delta: a must be float32 [%d, >= %d]" % (N, heads * dim))
        if b.dtype != torch.float32 or b.dim() != 2 or b.shape[0] != N or b.shape[1] < heads or b.stride(1) != 1:
            raise ValueError("gated_delta: b must be float32 [%d, >= %d]" % (N, heads))
        self._f32_vec(dt_bias, heads * dim, "gated_delta: dt_bias")
        self._f32_vec(a_log, heads, "gated_delta: a_log")
        if heads % kv_heads or dim > 256:
            raise ValueError("gated_delta: %d heads over %d key heads, keys of %d entries (at most 256)" % (heads, kv_heads, dim))
        self._state_view(state, self.gated_delta_state_floats(heads, dim, vdim), "gated_delta")
        seg_of, seg_starts, slots, S = self._segments(batch, N)
        out = torch.empty((N, heads * vdim), dtype=torch.float32, device=qkv.device)
        scratch = torch.empty(max(1, self.lib.lmsf_gated_delta_scratch_floats(N, S, int(heads), int(dim), int(vdim))),
                              dtype=torch.float32, device=qkv.device)
        self._check(self.lib.lmsf_gated_delta(
            _ptr(qkv), _code(qkv.dtype), qkv.stride(0), int(q_at), int(k_at), int(v_at), _ptr(a), a.stride(0),
            _ptr(dt_bias), _ptr(a_log), _ptr(b), b.stride(0), _ptr(state), state.stride(0), _ptr(seg_of), _ptr(seg_starts),
            _ptr(slots), _ptr(scratch), _ptr(out), out.stride(0), N, S,
            1 if (getattr(batch, "all_single", False) and S == N) else 0, int(heads), int(kv_heads), int(dim), int(vdim), float(q_scale),
            float(unit_eps), self._stream()))
        return out

    def head_rms_gate(self, raw: torch.Tensor, heads: int, vdim: int, eps: float, weight: Optional[torch.Tensor],
                      gate: Optional[torch.Tensor], out_dtype: torch.dtype, activation: str = "sigmoid") -> torch.Tensor:
        """Every head of ``raw`` (float32 [N, heads * vdim]) over its root mean square, times ``weight`` (float32
        [vdim], shared by the heads; None: none), times sigmoid or silu of ``gate`` ([N, >= heads * vdim] of
        ``out_dtype``; None: none). Returns [N, heads * vdim] in ``out_dtype``."""
        self._dev(raw, weight, gate)
        N = raw.shape[0]
        if raw.dtype != torch.float32 or raw.dim() != 2 or raw.shape[1] < heads * vdim or raw.stride(1) != 1:
            raise ValueError("head_rms_gate: raw must be float32 [N, >= %d]" % (heads * vdim))
        if weight is not None:
            self._f32_vec(weight, vdim, "head_rms_gate: weight")
        act = 0
        if gate is not None:
            if gate.dim() != 2 or gate.shape[0] != N or gate.shape[1] < heads * vdim or gate.stride(1) != 1 \
                    or gate.dtype != out_dtype:
                raise ValueError("head_rms_gate: gate must be [%d, >= %d] of the output's dtype" % (N, heads * vdim))
            act = {"sigmoid": 1, "silu": 2}[activation]
        out = torch.empty((N, heads * vdim), dtype=out_dtype, device=raw.device)
        self._check(self.lib.lmsf_head_rms_gate(
            _ptr(raw), raw.stride(0), _ptr(weight), _ptr(gate), gate.stride(0) if gate is not None else 0, act, _ptr(out),
            out.stride(0), _code(out_dtype), N, int(heads), int(vdim), float(eps), self._stream()))
        return out

    # ------------------------------------------------------------------ layer scale, logit cap

    def scale_add_norm(self, a: torch.Tensor, scale_a: torch.Tensor, b: Optional[torch.Tensor],
                       scale_b: Optional[torch.Tensor], residual: torch.Tensor, weight: Optional[torch.Tensor] = None,
                       eps: float = 1e-5) -> Optional[torch.Tensor]:
        """residual += scale_a * a + scale_b * b (float32, in place; b may be None), and with ``weight`` the RMS norm
        of the new rows times ``weight`` in a's dtype, from the same launch. a, b [N, W] with unit column stride;
        the scales float32 [W]; residual contiguous float32 [N, W]."""
        self._dev(a, scale_a, b, scale_b, residual, weight)
        if a.dim() != 2 or a.stride(1) != 1 or residual.dtype != torch.float32 or not residual.is_contiguous() \
                or residual.shape != a.shape:
            raise ValueError("scale_add_norm: a [N, W] and a contiguous float32 stream of that shape are needed")
        N, W = a.shape
        self._f32_vec(scale_a, W, "scale_add_norm: first scale")
        if b is not None:
            if b.shape != a.shape or b.dtype != a.dtype or b.stride(1) != 1 or scale_b is None:
                raise ValueError("scale_add_norm: b must be like a and have its scale")
            self._f32_vec(scale_b, W, "scale_add_norm: second scale")
        out = None
        if weight is not None:
            if weight.shape != (W,) or not weight.is_contiguous():
                raise ValueError("scale_add_norm: the norm's weight must be [%d]" % W)
            out = torch.empty((N, W), dtype=a.dtype, device=a.device)
        self._check(self.lib.lmsf_scale_add_norm(
            _ptr(a), a.stride(0), _ptr(scale_a), _ptr(b), b.stride(0) if b is not None else 0, _ptr(scale_b),
            _code(a.dtype), _ptr(residual), _ptr(weight), _code(weight.dtype) if weight is not None else F32, _ptr(out),
            N, W, float(eps), self._stream()))
        return out

    def logit_cap(self, logits: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> torch.Tensor:
        """logits <- cap tanh(logits * scale / cap) (cap 0: logits * scale), float32 [R, V], in place."""
        self._dev(logits)
        if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
            raise ValueError("logit_cap: logits must be float32 [R, V] with unit column stride")
        R, V = logits.shape
        for r0 in range(0, R, 65535):
            part = logits[r0:r0 + 65535]
            self._check(self.lib.lmsf_logit_cap(_ptr(part), part.stride(0), part.shape[0], V, float(scale), float(cap),
                                                self._stream()))
        return logits

    # ------------------------------------------------------------------ retention

    def retention_state_floats(self, heads: int, dim: int, vdim: int) -> int:
        return int(self.lib.lmsf_retention_state_floats(heads, dim, vdim))

    def retention(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, out_gate: torch.Tensor,
                  state: torch.Tensor, batch, heads: int, dim: int, vdim: int, k_scale: float, eps: float,
                  table: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Linear attention with a fixed decay per head over each request's tokens, the memory S [heads, dim, vdim]
        carried in ``state`` (float32 [slots, >= heads * dim * vdim]): S <- decay S + (k * k_scale) v^T, o = S^T q;
        returns every head's o over its root mean square times silu(out_gate), [N, heads * vdim] in q's dtype.
        q, k [N, heads * dim] and v [N, heads * vdim]: views of one buffer (equal row strides). ``decay``: float32
        [2 heads], the decays and then their logarithms. ``table`` (float32 [max_pos, rot] = [cos | sin]): q and k
        are first rotated by the token's position over their first rot entries, pairs (i, i + rot/2)."""
        self._dev(q, k, v, decay, out_gate, table)
        N = q.shape[0]
        for t, w, name in ((q, heads * dim, "q"), (k, heads * dim, "k"), (v, heads * vdim, "v"),
                           (out_gate, heads * vdim, "out_gate")):
            if t.dim() != 2 or t.shape[0] != N or t.shape[1] < w or t.stride(1) != 1 or t.dtype != q.dtype:
                raise ValueError("retention: %s must be [%d, >= %d] of q's dtype with unit column stride" % (name, N, w))
        if not (q.stride(0) == k.stride(0) == v.stride(0)):
            raise ValueError("retention: q, k and v must have one row stride")
        self._f32_vec(decay, 2 * heads, "retention: decay")
        rot = max_pos = 0
        if table is not None:
            if table.dtype != torch.float32 or table.dim() != 2 or not table.is_contiguous() or table.shape[1] > dim \
                    or table.shape[1] % 2:
                raise ValueError("retention: the rotary table must be contiguous float32 [max_pos, rot <= %d]" % dim)
            max_pos, rot = table.shape
            self._i32(batch.positions, "positions", N)
            self._dev(batch.positions)
        self._state_view(state, self.retention_state_floats(heads, dim, vdim), "retention")
        _, seg_starts, slots, S = self._segments(batch, N)
        out = torch.empty((N, heads * vdim), dtype=q.dtype, device=q.device)
        raw = torch.empty((N, heads * vdim), dtype=torch.float32, device=q.device)
        head = (_ptr(q), _ptr(k), _ptr(v), _code(q.dtype), q.stride(0), _ptr(batch.positions) if table is not None else None,
                _ptr(table), rot, max_pos, _ptr(decay), _ptr(out_gate), out_gate.stride(0), _ptr(state), state.stride(0),
                _ptr(seg_starts), _ptr(slots), _ptr(out), out.stride(0), _ptr(raw), N, S, int(heads), int(dim), int(vdim),
                float(k_scale), float(eps))
        lens = getattr(batch, "host_seg_lens", None)
        L = self.lib.lmsf_retention_chunk_tokens(int(dim))
        if not getattr(batch, "replayed", False) and not getattr(batch, "all_single", False) and lens and L > 0 \
                and max(lens) >= self.recurrent_chunked_min_tokens:
            bases = entries = None
            n_entries, most = 0, 1
            if max(lens) >= self.recurrent_parallel_min_chunks * L:
                key = ("retention_chunks", L)
                plan = batch.aux.get(key)
                if plan is None:
                    counts = [-(-n // L) for n in lens]
                    firsts = [sum(counts[:i]) for i in range(len(counts))]
                    plan = batch.aux[key] = (self.upload_ints(firsts, q.device), sum(counts), max(counts))
                bases, n_entries, most = plan
                entries = torch.empty(n_entries * self.lib.lmsf_retention_chunk_entry_floats(heads, dim, vdim),
                                      dtype=torch.float32, device=q.device)
            self._check(self.lib.lmsf_retention_chunked(*head, _ptr(bases), int(most), int(n_entries), _ptr(entries),
                                                        self._stream()))
            return out
        self._check(self.lib.lmsf_retention_tokens(*head, self._stream()))
        return out

    # ------------------------------------------------------------------ Dynamic Tanh, state-carrying mixers

    @staticmethod
    def _f32_vec(t: torch.Tensor, n: int, name: str) -> None:
        if t.dtype != torch.float32 or t.numel() != n or not t.is_contiguous():
            raise ValueError("%s must be contiguous float32 of %d elements" % (name, n))

    def dyt_norm(self, branch: Optional[torch.Tensor], residual: Optional[torch.Tensor], weight: torch.Tensor,
                 bias: torch.Tensor, alpha: torch.Tensor, out_dtype: torch.dtype,
                 rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """tanh(alpha * r) * weight + bias with r = residual + branch (either may be missing). ``residual``
        (float32 [N, H]) becomes the sum in place when both are given and ``rows`` is None; ``rows`` (int32 [R])
        selects rows, the output then has R. ``alpha`` is a float32 tensor of one element."""
        self._dev(branch, residual, weight, bias, alpha, rows)
        ref = branch if branch is not None else residual
        if ref is None or ref.dim() != 2 or not ref.is_contiguous():
            raise ValueError("dyt_norm needs a contiguous [N, H] branch or residual")
        N, H = ref.shape
        if branch is not None and residual is not None and branch.shape != residual.shape:
            raise ValueError("dyt_norm: branch %s and residual %s differ" % (tuple(branch.shape), tuple(residual.shape)))
        if residual is not None and (residual.dtype != torch.float32 or not residual.is_contiguous()):
            raise ValueError("the residual stream must be contiguous float32")
        self._f32_vec(weight, H, "dyt_norm: weight")
        self._f32_vec(bias, H, "dyt_norm: bias")
        self._f32_vec(alpha, 1, "dyt_norm: alpha")
        self._i32(rows, "rows")
        n_out = N if rows is None else rows.numel()
        out = torch.empty((n_out, H), dtype=out_dtype, device=ref.device)
        self._check(self.lib.lmsf_dyt_norm(_ptr(branch), _code(branch.dtype) if branch is not None else F32,
                                           _ptr(residual), _ptr(weight), _ptr(bias), _ptr(alpha), _ptr(out),
                                           _code(out_dtype), _ptr(rows), n_out, H, self._stream()))
        return out

    def _segments(self, batch, n_tokens: int):
        """(seg_of, seg_starts, state_slots, segments) of a step, checked."""
        self._dev(batch.seg_of_token, batch.seg_starts, batch.state_slots)
        S = batch.n_segments
        self._i32(batch.seg_of_token, "seg_of_token", n_tokens)
        self._i32(batch.seg_starts, "seg_starts", S + 1)
        self._i32(batch.state_slots, "state_slots", S)
        return batch.seg_of_token, batch.seg_starts, batch.state_slots, S

    @staticmethod
    def _state_view(state: torch.Tensor, need: int, name: str) -> None:
        if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < need \
                or not state.is_cuda:
            raise ValueError("%s: the state must be float32 [slots, >= %d] with unit column stride" % (name, need))

    def short_conv(self, u: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], state: Optional[torch.Tensor],
                   batch, activation: Optional[str] = None) -> torch.Tensor:
        """Causal convolution over time, channel by channel: out[t, c] = act(bias[c] + sum_j weight[c, j] u[t - taps + 1 + j, c])
        within each request. ``u`` [N, C] (a view with unit column stride will do), ``weight`` [C, taps]; ``state``
        float32 [slots, >= C (taps - 1)] holds every request's last taps - 1 inputs and is brought up to date (by a
        second launch, or by the same one in a step of single tokens).
        ``batch`` is the step (engine.batch.StepContext). activation None or "silu"."""
        self._dev(u, weight, bias)
        if u.dim() != 2 or u.stride(1) != 1 or weight.dim() != 2 or weight.shape[0] != u.shape[1] \
                or not weight.is_contiguous() or weight.dtype != u.dtype:
            raise ValueError("short_conv: u [N, C] and weight [C, taps] of one dtype are needed")
        N, C = u.shape
        taps = weight.shape[1]
        if bias is not None and (bias.shape != (C,) or bias.dtype != u.dtype or not bias.is_contiguous()):
            raise ValueError("short_conv: bias must be [%d] of u's dtype" % C)
        if activation not in (None, "silu"):
            raise ValueError("short_conv: activation %r unknown (None, silu)" % (activation,))
        if taps > 1:
            if state is None:
                raise ValueError("short_conv: a convolution over %d taps needs a state" % taps)
            self._state_view(state, C * (taps - 1), "short_conv")
        seg_of, seg_starts, slots, S = self._segments(batch, N)
        out = torch.empty((N, C), dtype=u.dtype, device=u.device)
        self._check(self.lib.lmsf_short_conv(
            _ptr(u), _code(u.dtype), u.stride(0), _ptr(weight), _ptr(bias), 1 if activation else 0, _ptr(state),
            state.stride(0) if state is not None else 0, _ptr(seg_of), _ptr(seg_starts), _ptr(slots), _ptr(out),
            out.stride(0), N, S, C, taps, 1 if (getattr(batch, "all_single", False) and S == N) else 0, self._stream()))
        return out

    def selective_scan(self, x: torch.Tensor, dt: torch.Tensor, bc: torch.Tensor, b_at: int, c_at: int, z: torch.Tensor,
                       a_log: torch.Tensor, d_skip: torch.Tensor, state: torch.Tensor, batch) -> torch.Tensor:
        """The selective scan over each request's tokens, the state carried in ``state`` (float32
        [slots, >= inner * n]): S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n, y_c = (sum_n S[c, n] C_n + D_c x_c)
        silu(z_c), with dt = softplus(``dt``) (float32 [N, inner], before the softplus), A = -exp(``a_log``)
        (float32 [inner, n]), B = bc[:, b_at:b_at + n], C = bc[:, c_at:c_at + n]. x, z, bc: views with unit column
        stride, one dtype. Returns y [N, inner] in x's dtype."""
        self._dev(x, dt, bc, z, a_log, d_skip)
        N, inner = x.shape
        if a_log.dim() != 2 or a_log.shape[0] != inner or a_log.dtype != torch.float32 or not a_log.is_contiguous():
            raise ValueError("selective_scan: a_log must be contiguous float32 [%d, n]" % inner)
        n = a_log.shape[1]
        self._f32_vec(d_skip, inner, "selective_scan: D")
        if dt.dtype != torch.float32 or tuple(dt.shape) != (N, inner) or dt.stride(1) != 1:
            raise ValueError("selective_scan: dt must be float32 [%d, %d]" % (N, inner))
        for t, w, name in ((x, inner, "x"), (z, inner, "z"), (bc, max(b_at, c_at) + n, "bc")):
            if t.dim() != 2 or t.shape[0] != N or t.shape[1] < w or t.stride(1) != 1 or t.dtype != x.dtype:
                raise ValueError("selective_scan: %s must be [%d, >= %d] of x's dtype with unit column stride" % (name, N, w))
        self._state_view(state, inner * n, "selective_scan")
        _, seg_starts, slots, S = self._segments(batch, N)
        y = torch.empty((N, inner), dtype=x.dtype, device=x.device)
        # segments longer than a chunk (portions of prompts) are cut into chunks that run side by side; which
        # segments, and where their chunks' summaries lie, is worked out once a step on the host
        chunk, max_chunks, bases, scratch = self.scan_chunk_tokens, 1, None, None
        plan = self._chunk_plan(batch, chunk)
        if plan is not None:
            bases, entries, max_chunks = plan
            scratch = torch.empty(entries * self.lib.lmsf_selective_scan_entry_floats(inner, n), dtype=torch.float32,
                                  device=x.device)
        self._check(self.lib.lmsf_selective_scan(
            _ptr(x), _code(x.dtype), x.stride(0), _ptr(dt), dt.stride(0), _ptr(bc), bc.stride(0), int(b_at), int(c_at),
            _ptr(z), z.stride(0), _ptr(a_log), _ptr(d_skip), _ptr(state), state.stride(0), _ptr(seg_starts), _ptr(slots),
            _ptr(y), y.stride(0), N, S, inner, n, int(chunk), int(max_chunks), _ptr(bases), _ptr(scratch), self._stream()))
        return y

    scan_chunk_tokens = 64         # tokens of a chunk of the selective scan's chunked form
    recurrent_chunked_min_tokens = 16   # segments from this many tokens on go to the matrix memory's chunked form
    recurrent_parallel_min_chunks = 3   # and from this many chunks on the chunks run side by side

    def _chunk_plan(self, batch, chunk: int):
        """(per segment its first entry of scratch or -1, entries in all, the most chunks of a segment) for a step
        that has segments longer than ``chunk`` tokens; None for a step without (and for a captured step, where
        nothing may hang on the host's view of the segments: those are steps of single tokens)."""
        if getattr(batch, "replayed", False) or getattr(batch, "all_single", False):
            return None
        key = ("chunk_plan", chunk)
        aux = getattr(batch, "aux", None)
        if aux is not None and key in aux:
            return aux[key]
        lens = getattr(batch, "host_seg_lens", None)
        plan = None
        if lens and max(lens) > chunk:
            bases, at, most = [], 0, 1
            for n in lens:
                c = -(-n // chunk)
                bases.append(at if c > 1 else -1)
                if c > 1:
                    at += c
                    most = max(most, c)
            plan = (self.upload_ints(bases, batch.seg_starts.device), at, most)
        if aux is not None:
            aux[key] = plan
        return plan

    def mlstm_state_floats(self, heads: int, dim: int, vdim: int) -> int:
        return int(self.lib.lmsf_mlstm_state_floats(heads, dim, vdim))

    def mlstm(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gates: torch.Tensor, out_gate: torch.Tensor,
              norm_weight: torch.Tensor, state: torch.Tensor, batch, heads: int, dim: int, vdim: int, q_scale: float,
              gate_cap: float, eps: float) -> torch.Tensor:
        """A matrix memory per head with exponential gates, over each request's tokens, the memory carried in
        ``state`` (csrc/recurrent.hip says how it is laid out and what is computed). q, k [N, heads * dim] and v
        [N, heads * vdim]: views of one buffer (equal row strides); ``gates`` float32 [N, 2 heads]: the input gates'
        pre-activations, then the forget gates'; ``out_gate`` [N, heads * vdim] before its sigmoid; ``norm_weight``
        float32 [heads * vdim]. Returns [N, heads * vdim] in q's dtype: every head's output over its root mean
        square, times the weight, times the gate."""
        self._dev(q, k, v, gates, out_gate, norm_weight)
        N = q.shape[0]
        for t, w, name in ((q, heads * dim, "q"), (k, heads * dim, "k"), (v, heads * vdim, "v"),
                           (out_gate, heads * vdim, "out_gate")):
            if t.dim() != 2 or t.shape[0] != N or t.shape[1] < w or t.stride(1) != 1 or t.dtype != q.dtype:
                raise ValueError("mlstm: %s must be [%d, >= %d] of q's dtype with unit column stride" % (name, N, w))
        if not (q.stride(0) == k.stride(0) == v.stride(0)):
            raise ValueError("mlstm: q, k and v must have one row stride")
        if gates.dtype != torch.float32 or tuple(gates.shape) != (N, 2 * heads) or gates.stride(1) != 1:
            raise ValueError("mlstm: gates must be float32 [%d, %d]" % (N, 2 * heads))
        self._f32_vec(norm_weight, heads * vdim, "mlstm: norm weight")
        self._state_view(state, self.mlstm_state_floats(heads, dim, vdim), "mlstm")
        _, seg_starts, slots, S = self._segments(batch, N)
        out = torch.empty((N, heads * vdim), dtype=q.dtype, device=q.device)
        lens = getattr(batch, "host_seg_lens", None)
        if not getattr(batch, "replayed", False) and not getattr(batch, "all_single", False) and lens \
                and max(lens) >= self.recurrent_chunked_min_tokens:
            # portions of prompts: chunks of tokens at a time (csrc/recurrent.hip: mlstm_chunk_kernel)
            raw = torch.empty(self.lib.lmsf_mlstm_chunk_scratch_floats(N, heads, vdim), dtype=torch.float32, device=q.device)
            # with segments of several chunks the chunks run side by side (three launches); their summaries and first
            # states lie in scratch, a segment's chunks one behind the other
            L = self.lib.lmsf_mlstm_chunk_tokens(int(dim))
            bases = entries = None
            n_entries, most = 0, 1
            if L > 0 and max(lens) >= self.recurrent_parallel_min_chunks * L:
                key = ("mlstm_chunks", L)
                plan = batch.aux.get(key)
                if plan is None:
                    counts = [-(-n // L) for n in lens]
                    firsts = [sum(counts[:i]) for i in range(len(counts))]
                    plan = batch.aux[key] = (self.upload_ints(firsts, q.device), sum(counts), max(counts))
                bases, n_entries, most = plan
                entries = torch.empty(n_entries * self.lib.lmsf_mlstm_chunk_entry_floats(heads, dim, vdim),
                                      dtype=torch.float32, device=q.device)
            self._check(self.lib.lmsf_mlstm_chunked(
                _ptr(q), _ptr(k), _ptr(v), _code(q.dtype), q.stride(0), _ptr(gates), gates.stride(0), _ptr(out_gate),
                out_gate.stride(0), _ptr(norm_weight), _ptr(state), state.stride(0), _ptr(seg_starts), _ptr(slots),
                _ptr(out), out.stride(0), _ptr(raw), N, S, int(heads), int(dim), int(vdim), float(q_scale),
                float(gate_cap), float(eps), _ptr(bases), int(most), int(n_entries), _ptr(entries), self._stream()))
            return out
        # steps of single tokens, and of portions of a few: one pass over every request's state
        raw = torch.empty(self.lib.lmsf_mlstm_chunk_scratch_floats(N, heads, vdim), dtype=torch.float32, device=q.device)
        self._check(self.lib.lmsf_mlstm_tokens(
            _ptr(q), _ptr(k), _ptr(v), _code(q.dtype), q.stride(0), _ptr(gates), gates.stride(0), _ptr(out_gate),
            out_gate.stride(0), _ptr(norm_weight), _ptr(state), state.stride(0), _ptr(seg_starts), _ptr(slots), _ptr(out),
            out.stride(0), _ptr(raw), N, S, int(heads), int(dim), int(vdim), float(q_scale), float(gate_cap), float(eps),
            self._stream()))
        return out

    # ------------------------------------------------------------------ attention with keys and values of two sizes

    def attn_prepare(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, heads: int, kv_heads: int, dim: int,
                     vdim: int, padded: int, positions: torch.Tensor, slots: Optional[torch.Tensor],
                     k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], table: Optional[torch.Tensor] = None,
                     unit_norm_eps: Optional[float] = None, temp_coef: float = 0.0, temp_every: int = 0) -> torch.Tensor:
        """Readies projected queries, keys and values for ``paged_attention`` at head size ``padded``: q and k are
        (each step optional) divided by their root mean square over the head (``unit_norm_eps``), rotated by the
        position over the first table.shape[1] entries in pairs (i, i + rot/2) (``table`` float32 [max_pos, rot] =
        [cos | sin]), q is multiplied by 1 + temp_coef ln(floor((p + 1) / temp_every) + 1); k and v go to the
        tokens' slots of the pages, everything padded with zeros to ``padded`` entries a head. q [N, heads * dim],
        k [N, kv_heads * dim], v [N, kv_heads * vdim]: views with unit column stride. Returns q [N, heads * padded]."""
        self._dev(q, k, v, positions, slots, k_pages, v_pages, table)
        N = q.shape[0]
        for t, w, name in ((q, heads * dim, "q"), (k, kv_heads * dim, "k"), (v, kv_heads * vdim, "v")):
            if t.dim() != 2 or t.shape[0] != N or t.shape[1] < w or t.stride(1) != 1 or t.dtype != q.dtype:
                raise ValueError("attn_prepare: %s must be [%d, >= %d] of q's dtype with unit column stride" % (name, N, w))
        self._i32(positions, "positions", N)
        rot = max_pos = 0
        if table is not None:
            if table.dtype != torch.float32 or table.dim() != 2 or not table.is_contiguous() or table.shape[1] > dim \
                    or table.shape[1] % 2:
                raise ValueError("attn_prepare: the rotary table must be contiguous float32 [max_pos, rot <= %d]" % dim)
            max_pos, rot = table.shape
        num_pages, ps = 0, 1
        if slots is not None:
            self._i32(slots, "slots", N)
            if k_pages is None or k_pages.dim() != 4 or k_pages.shape[1] != kv_heads or k_pages.shape[3] != padded \
                    or not k_pages.is_contiguous() or k_pages.dtype != q.dtype:
                raise ValueError("attn_prepare: k_pages must be contiguous [pages, %d, page_size, %d] of %s"
                                 % (kv_heads, padded, q.dtype))
            num_pages, ps = k_pages.shape[0], k_pages.shape[2]
            if v_pages is None or tuple(v_pages.shape) != (num_pages, kv_heads, padded, ps) or not v_pages.is_contiguous() \
                    or v_pages.dtype != q.dtype:
                raise ValueError("attn_prepare: v_pages must be contiguous [%d, %d, %d, %d] of %s"
                                 % (num_pages, kv_heads, padded, ps, q.dtype))
        out = torch.empty((N, heads * padded), dtype=q.dtype, device=q.device)
        self._check(self.lib.lmsf_attn_prepare(
            _ptr(q), q.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0), _code(q.dtype), _ptr(positions), _ptr(table),
            rot, max_pos, _ptr(slots), _ptr(out), out.stride(0), _ptr(k_pages), _ptr(v_pages), num_pages, N, int(heads),
            int(kv_heads), int(dim), int(vdim), int(padded), ps, 0 if unit_norm_eps is None else 1,
            float(unit_norm_eps or 0.0), float(temp_coef), int(temp_every), self._stream()))
        return out

    def head_gate(self, x: torch.Tensor, x_head: int, heads: int, vdim: int, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        """out[n, h * vdim + e] = x[n, h * x_head + e] * sigmoid(gate[n, h * vdim + e]) (no gate: the copy that drops
        what lies behind every head's first ``vdim`` entries)."""
        self._dev(x, gate)
        N = x.shape[0]
        if x.dim() != 2 or x.stride(1) != 1 or x.shape[1] < (heads - 1) * x_head + vdim or x_head < vdim:
            raise ValueError("head_gate: x too narrow for %d heads of %d" % (heads, x_head))
        if gate is not None and (gate.dim() != 2 or gate.shape[0] != N or gate.shape[1] < heads * vdim or gate.stride(1) != 1
                                 or gate.dtype != x.dtype):
            raise ValueError("head_gate: gate must be [%d, >= %d] of x's dtype" % (N, heads * vdim))
        out = torch.empty((N, heads * vdim), dtype=x.dtype, device=x.device)
        self._check(self.lib.lmsf_head_gate(_ptr(x), _code(x.dtype), x.stride(0), int(x_head), _ptr(gate),
                                            gate.stride(0) if gate is not None else 0, _ptr(out), out.stride(0), N,
                                            int(heads), int(vdim), self._stream()))
        return out

    def rms_pair(self, a: torch.Tensor, b: torch.Tensor, wa: torch.Tensor, wb: torch.Tensor, eps: float,
                 scale: float = 0.5) -> torch.Tensor:
        """scale * (a / rms(a) * wa + b / rms(b) * wb), row by row; a, b [N, W] of one dtype, the weights float32."""
        self._dev(a, b, wa, wb)
        if a.dim() != 2 or a.shape != b.shape or a.dtype != b.dtype or a.stride(1) != 1 or b.stride(1) != 1:
            raise ValueError("rms_pair: a and b must be [N, W] of one dtype with unit column stride")
        N, W = a.shape
        self._f32_vec(wa, W, "rms_pair: first weight")
        self._f32_vec(wb, W, "rms_pair: second weight")
        out = torch.empty((N, W), dtype=a.dtype, device=a.device)
        self._check(self.lib.lmsf_rms_pair(_ptr(a), a.stride(0), _ptr(b), b.stride(0), _code(a.dtype), _ptr(wa), _ptr(wb),
                                           _ptr(out), N, W, float(eps), float(scale), self._stream()))
        return out

    # ------------------------------------------------------------------ feed-forward

    def gated_act(self, gu: torch.Tensor, kind: str = "silu") -> torch.Tensor:
        """act(gu[:, :I]) * gu[:, I:] for gu [N, 2I]; kind "silu", "gelu" (erf form) or "gelu_tanh"."""
        self._dev(gu)
        if gu.dim() != 2 or gu.stride(1) != 1 or gu.shape[1] % 2 != 0:
            raise ValueError("gated_act input must be [N, 2I] with unit column stride")
        kinds = {"silu": 0, "gelu": 1, "gelu_tanh": 2}
        if kind not in kinds:
            raise ValueError("unknown activation %r (known: %s)" % (kind, ", ".join(kinds)))
        N, I = gu.shape[0], gu.shape[1] // 2
        out = torch.empty((N, I), dtype=gu.dtype, device=gu.device)
        self._check(self.lib.lmsf_gated_act(_ptr(gu), _ptr(out), _code(gu.dtype), N, I, gu.stride(0), kinds[kind],
                                            self._stream()))
        return out

    # ------------------------------------------------------------------ matrix products

    def weight_row_pad(self, in_features: int, dtype: torch.dtype) -> int:
        """Elements to leave between the end of one row of a linear layer's weight and the start of the next.
        With rows of 8 KB (or any multiple of 4 KB) lying back to back, the rows that a workgroup reads side by
        side begin on the same memory channels: a kernel that only reads a 28,672 x 4,096 matrix 64 rows at a
        time, 128 bytes of each, gets 4.8 TB/s, and 5.6 to 5.75 with 128 to 2,048 bytes between the rows; 16 rows
        at a time, 1 KB of each: 5.0 and 5.9 to 6.0. Which distances help depends on the row's length (rows of
        16 KB: 128 bytes hurt, 256 and more help; rows of 28 KB: 256 hurts); 512 bytes help or do no harm at 4,096,
        8,192, 14,336 and 28,672 columns, for the few-rows, the many-rows and the library's products alike (gate_up
        of 57,344 x 8,192 at 64 rows: 207 -> 181 us). Every product takes the distance between rows as an
        argument."""
        return self.weight_row_pad_bytes // torch.empty((), dtype=dtype).element_size()

    def linear(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
               out_dtype: Optional[torch.dtype] = None, pending_ok: bool = False,
               out: Optional[torch.Tensor] = None):
        """y = x weight^T (+ bias); x [M, K], weight [N, K]; y [M, N] in ``out_dtype`` (default x's).
        With ``pending_ok`` the caller takes a ``PendingProduct`` as well, which comes back where the
        product splits K over workgroups, or a ``DeferredLinear`` (few rows). ``out``: a contiguous [M, N]
        tensor of ``out_dtype`` that takes the result instead of a new one (not together with ``pending_ok``).

        Which kernel runs is decided by ``lmsf_route_linear`` (csrc/dispatch.hip), as for the step program:
        float32 operands always run the float32 multiply-add kernel; bfloat16 products with bfloat16 output
        and many rows go to the BLAS library, as the reference's do (core/src/model_executor/layers/linear.rs:44-106
        calls cuBLASLt), through csrc/blas.hip; the rest run in this package's kernels.
        """
        self._dev(x, weight, bias)
        if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
            raise ValueError("linear: x %s and weight %s do not match" % (tuple(x.shape), tuple(weight.shape)))
        if x.stride(1) != 1 or weight.stride(1) != 1:
            raise ValueError("linear: operands need unit column stride")
        M, K = x.shape
        N = weight.shape[0]
        if bias is not None and (bias.shape != (N,) or bias.dtype != weight.dtype or not bias.is_contiguous()):
            raise ValueError("linear: bias must be [%d] of the weight's dtype" % N)
        out_dtype = out_dtype or x.dtype
        if out is not None:
            if pending_ok or tuple(out.shape) != (M, N) or out.dtype != out_dtype or not out.is_contiguous() \
                    or out.device != x.device:
                raise ValueError("linear: out must be a contiguous [%d, %d] %s tensor on x's device" % (M, N, out_dtype))
        rt = D.Route()
        self.lib.lmsf_route_linear(ctypes.byref(self._tun), ctypes.byref(self._shape(x, weight, out_dtype)),
                                   1 if pending_ok else 0, ctypes.byref(rt))
        if rt.route == D.MID:
            return self._linear_mid(x, weight, bias, 0, out_dtype, rt, out=out)
        if rt.route == D.LARGE:
            return self._linear_large(x, weight, bias, 0, bool(rt.pending), out=out, plan=rt.plan)
        if rt.route == D.DEFERRED:
            return DeferredLinear(x, weight, bias, out_dtype)
        y = out if out is not None else torch.empty((M, N), dtype=out_dtype, device=x.device)
        if rt.route == D.GEMV:
            self._check(self.lib.lmsf_gemv(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(y),
                                           _code(out_dtype), y.stride(0), M, N, K, 0, self._stream()))
        elif rt.route == D.CHUNKS:
            for r0 in range(0, M, rt.chunk_rows):
                rows = min(rt.chunk_rows, M - r0)
                self.linear(x[r0:r0 + rows], weight, bias, out_dtype=out_dtype, out=y[r0:r0 + rows])
        elif rt.route == D.SKINNY:
            for r0 in range(0, M, 64):
                rows = min(64, M - r0)
                xs, ys = x[r0:r0 + rows], y[r0:r0 + rows]
                self._check(self.lib.lmsf_gemm_skinny(
                    _ptr(xs), xs.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(ys),
                    _code(out_dtype), ys.stride(0), rows, N, K, self.skinny_variant, 0, self._stream()))
        elif rt.route == D.BLAS:
            self._check(self.lib.lmsf_blas_linear(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(bias),
                                                  _ptr(y), y.stride(0), M, N, K, self._stream()))
        else:
            self._check(self.lib.lmsf_gemm_plain(_ptr(x), _code(x.dtype), x.stride(0), _ptr(weight),
                                                 _code(weight.dtype), weight.stride(0), _ptr(bias), _ptr(y),
                                                 _code(out_dtype), y.stride(0), M, N, K, self._stream()))
        return y

    def linear_wide(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                    out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x weight^T + bias in float32, for results that enter a recurrence (a step size, a gate). With many
        bfloat16 rows the product runs in the many-rows matrix-core kernel with K in two parts, whose float32 partial
        sums the reduction kernel adds up with the bias (the BLAS library's plans of this package write bfloat16
        only, and ``linear`` would cut the rows into pieces of ``mid_max_rows``: 16 launches for 2,048 rows);
        otherwise it is ``linear`` with float32 output. ``out``: a contiguous float32 [M, N] tensor that takes the
        result (not an operand of the product)."""
        M, K = x.shape
        N = weight.shape[0]
        if out is not None and (tuple(out.shape) != (M, N) or out.dtype != torch.float32 or not out.is_contiguous()
                                or out.device != x.device):
            raise ValueError("linear_wide: out must be a contiguous float32 [%d, %d] tensor on x's device" % (M, N))
        if (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and M > self.mid_max_rows and x.dim() == 2
                and weight.dim() == 2 and weight.shape[1] == K and K % 64 == 0 and K >= 128 and N % 8 == 0
                and x.stride(1) == 1 and weight.stride(1) == 1 and x.stride(0) % 8 == 0 and weight.stride(0) % 8 == 0
                and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0
                and (bias is None or (bias.shape == (N,) and bias.dtype == weight.dtype and bias.is_contiguous()))):
            self._dev(x, weight, bias)
            plan = self.lib.lmsf_gemm_large_plan(M, N, K, 0) // 16 * 16 + 2
            parts = torch.empty((2, M, N), dtype=torch.float32, device=x.device)
            self._check(self.lib.lmsf_gemm_large(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), None, None, 0,
                                                 M, N, K, 0, plan, _ptr(parts), 0, self._stream()))
            y = out if out is not None else torch.empty((M, N), dtype=torch.float32, device=x.device)
            self._check(self.lib.lmsf_gemm_mid_reduce(_ptr(parts), _ptr(bias), _ptr(y), F32, y.stride(0), M, N, 2,
                                                      self._stream()))
            return y
        if (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.dim() == 2 and weight.dim() == 2
                and M > self.mid_max_rows and weight.shape[1] == K and K < 128 and x.stride(1) == 1
                and weight.stride(1) == 1 and (bias is None or (bias.shape == (N,) and bias.dtype == weight.dtype
                                                                and bias.is_contiguous()))):
            # a product over few columns (the second half of a low-rank pair): one launch of the plain kernel instead
            # of pieces of ``mid_max_rows`` rows
            self._dev(x, weight, bias)
            y = out if out is not None else torch.empty((M, N), dtype=torch.float32, device=x.device)
            self._check(self.lib.lmsf_gemm_plain(_ptr(x), _code(x.dtype), x.stride(0), _ptr(weight), _code(weight.dtype),
                                                 weight.stride(0), _ptr(bias), _ptr(y), F32, y.stride(0), M, N, K,
                                                 self._stream()))
            return y
        if out is not None:
            return self.linear(x, weight, bias, out_dtype=torch.float32, out=out)
        return self.linear(x, weight, bias, out_dtype=torch.float32)

    def linear_gated(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                     kind: str = "silu") -> torch.Tensor:
        """act(x Wg^T + bg) * (x Wu^T + bu) for the fused weight [2 I, K] = [Wg; Wu] (bias [2 I] likewise);
        [M, I] in x's dtype. Where ``lmsf_route_linear_gated`` says so the activation is the epilogue of the
        product; otherwise the product and the activation kernel run one after the other. Both ways round
        the two products to the storage type before the activation, so they give the same bits wherever
        they add up K in the same order (the default tilings of the fused and the plain product do not: they
        split K over 8 and over 16 waves). ``x`` may be a ``ScaledRows``."""
        if weight.dim() != 2 or weight.shape[0] % 2 != 0:
            raise ValueError("linear_gated: weight must be [2 I, K]")
        kinds = {"silu": 1, "gelu": 2, "gelu_tanh": 5}
        if kind not in kinds:
            raise ValueError("unknown activation %r (known: %s)" % (kind, ", ".join(kinds)))
        M, I = x.shape[0], weight.shape[0] // 2
        scaled = isinstance(x, ScaledRows)
        xt = x.xw if scaled else x
        if xt.dim() != 2 or xt.shape[1] != weight.shape[1] or xt.stride(1) != 1 or weight.stride(1) != 1:
            raise ValueError("linear_gated: x %s and weight %s do not match" % (tuple(xt.shape), tuple(weight.shape)))
        K = xt.shape[1]
        rt = D.Route()
        self.lib.lmsf_route_linear_gated(ctypes.byref(self._tun), ctypes.byref(self._shape(xt, weight, xt.dtype)),
                                         x.rows_per_tile if scaled else 0, x.tiles if scaled else 0, ctypes.byref(rt))
        if rt.route == D.MATERIALIZE:
            return self.linear_gated(self.materialize(x), weight, bias, kind)
        if rt.route == D.SEPARATE or (kind == "gelu_tanh" and rt.route not in (D.GEMV, D.SKINNY)):
            # (the tanh form of GELU is an epilogue of the one-row and the few-rows product only)
            return self.gated_act(self.linear(self.materialize(x), weight, bias), kind)
        self._dev(xt, weight, bias)
        if bias is not None and (bias.shape != (2 * I,) or bias.dtype != weight.dtype or not bias.is_contiguous()):
            raise ValueError("linear_gated: bias must be [%d] of the weight's dtype" % (2 * I))
        if rt.route == D.MID:
            return self._linear_mid(x, weight, bias, kinds[kind], torch.bfloat16, rt)
        if rt.route == D.LARGE:
            return self._linear_large(x, weight, bias, kinds[kind], plan=rt.plan)
        y = torch.empty((M, I), dtype=torch.bfloat16, device=x.device)
        head = (_ptr(xt), xt.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(y))
        if rt.route == D.MID_SCALED:
            self._check(self.lib.lmsf_gemm_mid_scaled(*head, y.stride(0), M, I, K, kinds[kind], _ptr(x.sumsq), x.tiles,
                                                      x.eps, self._stream()))
        elif rt.route == D.GEMV_SCALED:
            self._check(self.lib.lmsf_gemv_scaled(*head, y.stride(0), M, I, K, kinds[kind], _ptr(x.sumsq), x.tiles,
                                                  x.eps, self._stream()))
        elif rt.route == D.SKINNY_SCALED:
            self._check(self.lib.lmsf_gemm_skinny_scaled(*head, y.stride(0), M, I, K, kinds[kind], _ptr(x.sumsq),
                                                         x.tiles, x.eps, self.skinny_variant, self._stream()))
        elif rt.route == D.GEMV:
            self._check(self.lib.lmsf_gemv(*head, BF16, y.stride(0), M, I, K, kinds[kind], self._stream()))
        else:
            self._check(self.lib.lmsf_gemm_skinny(*head, BF16, y.stride(0), M, I, K, self.skinny_variant, kinds[kind],
                                                  self._stream()))
        return y

    def _linear_mid(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], act: int,
                    out_dtype: torch.dtype, rt: D.Route, out: Optional[torch.Tensor] = None):
        """The 17-and-more-rows product (csrc/gemm_mid.hip) as ``rt`` says."""
        self._dev(x, weight, bias)
        M, K = x.shape
        N = weight.shape[0] // 2 if act else weight.shape[0]
        if bias is not None and (bias.shape != (weight.shape[0],) or bias.dtype != weight.dtype
                                 or not bias.is_contiguous()):
            raise ValueError("linear: bias must be [%d] of the weight's dtype" % weight.shape[0])
        splits = rt.splits
        if rt.pending:
            partials = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
            self._check(self.lib.lmsf_gemm_mid_partial(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), M, N, K,
                                                       splits, _ptr(partials), self._stream()))
            return PendingProduct(partials, bias, out_dtype)
        floats = self.lib.lmsf_gemm_mid_scratch_floats(M, N, splits, act)
        scratch = torch.empty(floats, dtype=torch.float32, device=x.device) if floats else None
        y = out if out is not None else torch.empty((M, N), dtype=out_dtype, device=x.device)
        self._check(self.lib.lmsf_gemm_mid(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(y),
                                           _code(out_dtype), y.stride(0), M, N, K, act, splits, _ptr(scratch),
                                           self._stream()))
        return y

    def _linear_large(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], act: int,
                      pending_ok: bool = False, out: Optional[torch.Tensor] = None, plan: Optional[int] = None):
        """The many-rows product (csrc/gemm_large.hip); K a multiple of 64, W's rows of 8, row strides of 8,
        16-byte aligned bases. ``plan``: tiling and split (``lmsf_gemm_large_plan`` proposes one)."""
        self._dev(x, weight, bias)
        M, K = x.shape
        N = weight.shape[0] // 2 if act else weight.shape[0]
        if bias is not None and (bias.shape != (weight.shape[0],) or bias.dtype != weight.dtype
                                 or not bias.is_contiguous()):
            raise ValueError("linear: bias must be [%d] of the weight's dtype" % weight.shape[0])
        if plan is None:
            plan = self.lib.lmsf_gemm_large_plan(M, N, K, act)
        splits = plan % 16
        scratch = None
        if splits > 1:
            scratch = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
            if pending_ok:
                self._check(self.lib.lmsf_gemm_large(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), None, None, 0,
                                                     M, N, K, 0, plan, _ptr(scratch), 0, self._stream()))
                return PendingProduct(scratch, bias, torch.bfloat16)
        y = out if out is not None else torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
        self._check(self.lib.lmsf_gemm_large(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(y),
                                             y.stride(0), M, N, K, act, plan, _ptr(scratch), 1, self._stream()))
        return y

    def tune_products(self, x: torch.Tensor, weights, bias: Optional[torch.Tensor] = None, candidates: int = 16,
                      reps: int = 5):
        """Lets the BLAS library's candidates for the product of ``x`` [M, K] with matrices like ``weights`` (a list of
        [N, K] tensors of one shape and row distance: the same product of several layers, so that no run finds its
        weights in cache) race, and keeps the fastest for later products of that shape
        (tops/src/cublas.rs:121-223 profiles cuBLASLt's tactics likewise). Returns (first choice's us, fastest's us)."""
        w0 = weights[0]
        self._dev(x, bias, *weights)
        if any(w.shape != w0.shape or w.stride(0) != w0.stride(0) or w.dtype != torch.bfloat16 or w.stride(1) != 1
               for w in weights) or x.dtype != torch.bfloat16 or x.shape[1] != w0.shape[1] or x.stride(1) != 1:
            raise ValueError("tune_products: bfloat16 operands of one shape are needed")
        M, K = x.shape
        N = w0.shape[0]
        y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
        ptrs = (ctypes.c_void_p * len(weights))(*[w.data_ptr() for w in weights])
        times = (ctypes.c_float * 2)()
        self._check(self.lib.lmsf_blas_tune(_ptr(x), x.stride(0), ptrs, len(weights), w0.stride(0), _ptr(bias), _ptr(y),
                                            y.stride(0), M, N, K, int(candidates), int(reps), times, self._stream()))
        return float(times[0]), float(times[1])

    # ------------------------------------------------------------------ sampling

    def sample(self, logits: torch.Tensor, temperature: Optional[torch.Tensor] = None,
               top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
               min_p: Optional[torch.Tensor] = None, seeds: Optional[torch.Tensor] = None,
               draws: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One token per row of float32 ``logits`` [R, V]; int32 [R]. All parameters are per-row device
        tensors: temperature/top_p/min_p float32, top_k int32, seeds int64, draws int32."""
        self._dev(logits, temperature, top_k, top_p, min_p, seeds, draws)
        if logits.dim() != 2 or logits.dtype != torch.float32 or logits.stride(1) != 1:
            raise ValueError("sample: logits must be float32 [R, V] with unit column stride")
        R, V = logits.shape
        for name, t, dt in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                            ("top_p", top_p, torch.float32), ("min_p", min_p, torch.float32),
                            ("seeds", seeds, torch.int64), ("draws", draws, torch.int32)):
            if t is not None and (t.dtype != dt or t.numel() != R or not t.is_contiguous()):
                raise ValueError("sample: %s must be a contiguous %s tensor of %d elements" % (name, dt, R))
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
        scratch = None
        if temperature is None or (top_k is None and top_p is None and min_p is None):
            elems = self.lib.lmsf_sample_scratch_elems(R, V)
            if elems:
                scratch = torch.empty(2 * elems, dtype=torch.float32, device=logits.device)
        self._check(self.lib.lmsf_sample(_ptr(logits), logits.stride(0), R, V, _ptr(temperature), _ptr(top_k),
                                         _ptr(top_p), _ptr(min_p), _ptr(seeds), _ptr(draws), _ptr(out),
                                         _ptr(scratch), self._stream()))
        return out

    def apply_penalties(self, logits: torch.Tensor, tokens: torch.Tensor, offsets: torch.Tensor,
                        prompt_lens: torch.Tensor, presence: torch.Tensor, frequency: torch.Tensor,
                        repetition: torch.Tensor) -> None:
        """Presence, frequency and repetition penalties on float32 ``logits`` [R, V], in place.
        ``tokens`` int32: each row's prompt then output tokens, concatenated; ``offsets`` int32 [R+1];
        ``prompt_lens`` int32 [R]; the penalties float32 [R]."""
        self._dev(logits, tokens, offsets, prompt_lens, presence, frequency, repetition)
        if logits.dim() != 2 or logits.dtype != torch.float32 or logits.stride(1) != 1:
            raise ValueError("apply_penalties: logits must be float32 [R, V] with unit column stride")
        R, V = logits.shape
        self._i32(tokens, "tokens")
        self._i32(offsets, "offsets", R + 1)
        self._i32(prompt_lens, "prompt_lens", R)
        for name, t in (("presence", presence), ("frequency", frequency), ("repetition", repetition)):
            if t.dtype != torch.float32 or t.numel() != R or not t.is_contiguous():
                raise ValueError("apply_penalties: %s must be contiguous float32 [%d]" % (name, R))
        counts = torch.zeros((R, V), dtype=torch.int32, device=logits.device)
        self._check(self.lib.lmsf_apply_penalties(_ptr(logits), logits.stride(0), R, V, _ptr(tokens), _ptr(offsets),
                                                  _ptr(prompt_lens), _ptr(counts), _ptr(presence), _ptr(frequency),
                                                  _ptr(repetition), self._stream()))


    # ------------------------------------------------------------------ what the machine gives

    def measure(self, nbytes: int = 4 << 30, reps: int = 5) -> dict:
        """Measured rates of this GPU: reading and copying ``nbytes`` of device memory with plain kernels (GB/s,
        a copy counted as bytes read plus bytes written) and the bfloat16 matrix-core instruction in a loop
        without memory traffic (TFLOP/s). The best of ``reps`` runs each, timed with events."""
        dev = torch.device("cuda", _current_device())
        src = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        src.random_(0, 255)
        dst = torch.empty_like(src)
        sink = torch.zeros(64, dtype=torch.float32, device=dev)

        def timed(launch):
            best = None
            for _ in range(reps + 1):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                launch()
                b.record()
                b.synchronize()
                ms = a.elapsed_time(b)
                best = ms if best is None else min(best, ms)
            return best * 1e-3

        t_read = timed(lambda: self._check(self.lib.lmsf_measure_read(_ptr(src), nbytes, _ptr(sink), self._stream())))
        t_copy = timed(lambda: self._check(self.lib.lmsf_measure_copy(_ptr(src), _ptr(dst), nbytes, self._stream())))
        flops = [0.0]

        def mfma():
            flops[0] = self.lib.lmsf_measure_mfma(_ptr(sink), 4096, 256 * 8, self._stream())
            if flops[0] == 0.0:
                self._check(1)
        t_mfma = timed(mfma)
        return {"read_GBps": nbytes / t_read / 1e9, "copy_GBps": 2 * nbytes / t_copy / 1e9,
                "mfma_bf16_TFLOPs": flops[0] / t_mfma / 1e12}


class _AttentionPlan:
    __slots__ = ("tiles", "n_tiles", "single_tokens", "n_single", "max_context", "token_is_request")

    def __init__(self, tiles, n_tiles, single_tokens, n_single, max_context, token_is_request=False):
        self.tiles = tiles                    # int32 [n_tiles, 2] on the device, or None
        self.n_tiles = n_tiles
        self.single_tokens = single_tokens    # int32 flat indices of the one-token requests; None: every token
        self.n_single = n_single
        self.max_context = max_context
        self.token_is_request = token_is_request   # a step of single tokens: token i is request i of the tables


_default_ops: Optional[HipOps] = None


def get_ops() -> HipOps:
    """The process-wide kernel object; raises if the GPU or the library is missing."""
    global _default_ops
    if _default_ops is None:
        _default_ops = HipOps()
    return _default_ops
