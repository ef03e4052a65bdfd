"""The kernels the engine computes with: hand-written HIP for gfx950, called through ctypes.

Every wrapper checks on the host that operand shapes, dtypes and strides are what
its kernel and grid assume before anything is launched, launches on torch's
current stream, and raises with the library's message on a refusal.  Matrix
products of the bfloat16 path with many rows go to the library GEMM behind
torch (hipBLASLt), as the reference's go to cuBLAS (inference_engine/model.py:172-185);
everything else, and every product of the float32 path, is a kernel of this
package.  There is no CPU path and no fallback: a missing library is an error.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p

import torch

from . import library
from .api import KernelBackend, Normed, Sink

F32, BF16 = 0, 1


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise TypeError(f"kernels take float32 or bfloat16, not {dtype}")


def _ptr(t) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


def _rows_ok(t: torch.Tensor, what: str) -> None:
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{what}: expected a 2-d tensor with unit inner stride, got shape {tuple(t.shape)} "
                         f"strides {t.stride()}")


class ProjectionSums:
    """The q/k/v projection of a step as float32 sums [splits, tokens, (Hq + 2 Hkv) D], not yet added up, rotated
    or written to the cache (operands checked).  ``finish()`` does that in a kernel of its own and gives q
    [tokens, Hq * D]; ``paged_attention`` lets its decode kernel do it instead where that kernel has a workgroup
    of its own for every row and kv head."""

    def __init__(self, ops, part, positions, cos, sin, slots, k_cache, v_cache, Hq, Hkv, D, page):
        self.ops, self.part, self.positions, self.cos, self.sin, self.slots = ops, part, positions, cos, sin, slots
        self.k_cache, self.v_cache, self.Hq, self.Hkv, self.D, self.page = k_cache, v_cache, Hq, Hkv, D, page

    def finish(self):
        ops, part = self.ops, self.part
        splits, M, _ = part.shape
        q = torch.empty((M, self.Hq * self.D), dtype=torch.bfloat16, device=part.device)
        if splits == 1:
            lib = ops.lib("rope_kv")
            library.check(lib, lib.mie_rotary_kv_store_sums(
                _ptr(part), part.stride(1), _ptr(q), q.stride(0), _ptr(self.positions), _ptr(self.cos), _ptr(self.sin),
                _ptr(self.slots), _ptr(self.k_cache), _ptr(self.v_cache), self.Hq, self.Hkv, self.D, self.page, M,
                ops._stream()))
        else:
            lib = ops.lib("gemm_mid_bf16")
            library.check(lib, lib.mie_mid_reduce_rope_kv(
                _ptr(part), splits, M, _ptr(q), q.stride(0), _ptr(self.positions), _ptr(self.cos), _ptr(self.sin),
                _ptr(self.slots), _ptr(self.k_cache), _ptr(self.v_cache), self.Hq, self.Hkv, self.D, self.page,
                ops._stream()))
        return q


class HipBackend(KernelBackend):
    name = "hip-gfx950"

    def __init__(self, act_dtype: torch.dtype, device="cuda"):
        self.act_dtype = act_dtype
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("the HIP kernels run on the GPU only; there is no CPU path")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU visible to torch: the engine needs an MI355X (gfx950)")
        self._libs = {}
        self._zeros = None          # 256 zero bytes on the device, what masked loads of the mid-row product read
        self._lt_workspace = None   # device memory the library's product kernels may use
        self._lt_rows = set()       # row counts whose library products get their kernel chosen by timing (prefer_rows)
        self._lt_tuned = set()      # (M, N, K, kind, leading dims) already chosen that way
        self._log2_tables = {}      # distance-bias tables in units of log2 e, by the address of the table they were made of
        self.true_fp32 = act_dtype == torch.float32
        self._device_index = self.device.index if self.device.index is not None else torch.cuda.current_device()

    # ------------------------------------------------------------ plumbing
    def lib(self, module: str, defines: tuple = ()):
        """The loaded library of a registered kernel module (library.register_kernel_module), entry points
        declared with the argument types it was registered with."""
        key = (module, defines)
        if key not in self._libs:
            self._libs[key] = library.load(module, defines)
        return self._libs[key]

    def _stream(self) -> c_void_p:
        # the handle alone: building torch's Stream object costs several microseconds a launch
        return c_void_p(torch._C._cuda_getCurrentRawStream(self._device_index))

    def _on_device(self, *tensors) -> None:
        for t in tensors:
            if t is not None and t.device.type != "cuda":
                raise ValueError(f"tensor on {t.device}; the kernels take GPU tensors only")

    # ---- library matrix products (many rows): hipBLASLt through csrc/lt_gemm.hip
    LT_BF16, LT_F32, LT_ADD = 0, 1, 2
    LT_WORKSPACE_BYTES = 128 << 20
    LT_COLD_BYTES = 384 << 20       # overwritten before each timed launch of a finalist: more than the memory-side cache

    def prefer_rows(self, counts) -> None:
        self._lt_rows.update(int(c) for c in counts)

    def _lt_ok(self, x, w) -> bool:
        """Whether the engine's own call into the library takes x w^T (else torch's call does)."""
        return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.stride(1) == 1 and w.stride(1) == 1
                and w.shape[0] % 8 == 0 and w.shape[1] % 8 == 0 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
                and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)

    def _lt_product(self, x, w, kind, out):
        """out (+)= x w^T by the library; out [M, N] contiguous, bfloat16 (LT_BF16) or float32."""
        lib = self.lib("lt_gemm")
        M, K = x.shape
        N = w.shape[0]
        if self._lt_workspace is None:
            self._lt_workspace = torch.empty(self.LT_WORKSPACE_BYTES, dtype=torch.uint8, device=w.device)
        ws = self._lt_workspace
        if M in self._lt_rows:
            key = (M, N, K, kind, x.stride(0), w.stride(0), out.stride(0))
            if key not in self._lt_tuned and not torch.cuda.is_current_stream_capturing():
                if not lib.mie_lt_is_tuned(x.stride(0), w.stride(0), out.stride(0), M, N, K, kind):
                    # choose this shape's kernel by timing the library's suggestions, on a buffer that may be spoilt
                    # (every kernel the library has for the shape; the finalists with the weights cold, as a step finds them)
                    spoilt = out if kind != self.LT_ADD else torch.empty_like(out)
                    cold = torch.empty(self.LT_COLD_BYTES, dtype=torch.uint8, device=w.device)
                    best, first = c_float(0), c_float(0)
                    library.check(lib, lib.mie_lt_tune(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(spoilt), spoilt.stride(0),
                                                       M, N, K, kind, _ptr(ws), ws.numel(), 0, 5, _ptr(cold), cold.numel(),
                                                       ctypes.byref(best), ctypes.byref(first), self._stream()))
                    torch.cuda.current_stream().synchronize()
                    del cold
                self._lt_tuned.add(key)
        library.check(lib, lib.mie_lt_gemm(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(0), M, N, K, kind,
                                           _ptr(ws), ws.numel(), self._stream()))
        return out

    # ----------------------------------------------------------------- ops
    def embedding(self, ids, table, taken_from=None, earlier_tokens=None, scale=1.0):
        self._on_device(ids, table, taken_from, earlier_tokens)
        if ids.dtype != torch.int32 or ids.dim() != 1 or not ids.is_contiguous():
            raise ValueError("embedding: ids must be contiguous int32 [T]")
        if taken_from is not None:
            if earlier_tokens is None or taken_from.dtype != torch.int32 or earlier_tokens.dtype != torch.int32 \
                    or taken_from.shape != ids.shape or not taken_from.is_contiguous() or not earlier_tokens.is_contiguous():
                raise ValueError("embedding: taken_from must be contiguous int32 [T] beside int32 earlier_tokens")
        if table.dim() != 2 or not table.is_contiguous():
            raise ValueError("embedding: table must be contiguous [vocab, width]")
        T, (V, W) = ids.shape[0], table.shape
        out = torch.empty((T, W), dtype=torch.float32, device=table.device)
        lib = self.lib("embed_norm")
        library.check(lib, lib.mie_embedding(_ptr(ids), _ptr(table), _code(table.dtype), _ptr(out), T, W, V,
                                             _ptr(taken_from), _ptr(earlier_tokens), float(scale), self._stream()))
        return out

    def add_rmsnorm(self, x, residual, weight, eps, out_dtype=None, rows=None):
        self._on_device(x, residual, weight, rows)
        out_dtype = out_dtype or self.act_dtype
        if residual.dtype != torch.float32 or residual.dim() != 2 or not residual.is_contiguous():
            raise ValueError("add_rmsnorm: the residual stream must be contiguous float32 [T, width]")
        T, W = residual.shape
        if x is not None and (tuple(x.shape) != (T, W) or not x.is_contiguous()):
            raise ValueError(f"add_rmsnorm: x {tuple(x.shape)} does not match the stream {(T, W)}")
        if tuple(weight.shape) != (W,) or not weight.is_contiguous():
            raise ValueError(f"add_rmsnorm: weight {tuple(weight.shape)} for width {W}")
        n = T
        if rows is not None:
            if rows.dtype != torch.int32 or rows.dim() != 1 or not rows.is_contiguous():
                raise ValueError("add_rmsnorm: rows must be contiguous int32")
            n = rows.shape[0]
        y = torch.empty((n, W), dtype=out_dtype, device=residual.device)
        lib = self.lib("embed_norm")
        library.check(lib, lib.mie_add_rmsnorm(
            _ptr(x), _code(x.dtype) if x is not None else F32, _ptr(residual), _ptr(weight), _code(weight.dtype),
            _ptr(y), _code(out_dtype), _ptr(rows), n, W, float(eps), self._stream()))
        return y

    def _gemm(self, x, w, bias, out_dtype):
        M, K = x.shape
        N = w.shape[0]
        y = torch.empty((M, N), dtype=out_dtype, device=x.device)
        if bias is not None:
            bias = bias.float().contiguous()
        lib = self.lib("gemm")
        library.check(lib, lib.mie_gemm_nt(_ptr(x), _code(x.dtype), x.stride(0), _ptr(w), _code(w.dtype), w.stride(0),
                                           _ptr(y), _code(out_dtype), y.stride(0), _ptr(bias), M, N, K,
                                           self._stream()))
        return y

    # ---- few-row products of the bfloat16 path: one fused kernel each
    SKINNY_MAX_ROWS = 16      # the kernel's own limit (one tile of rows); a decode step of 16 rows of 512 keys at the
                              # benchmark's sizes takes 1.15 ms, one of 17 rows with the split product 1.27
    EPI_BF16, EPI_F32, EPI_ADD, EPI_SWIGLU, EPI_GEGLU = 0, 1, 2, 3, 5

    def _skinny_ok(self, x, w, bias, rows=None) -> bool:
        """Whether the fused few-row kernel takes this product (x a bfloat16 tensor)."""
        m = x.shape[0] if rows is None else rows.shape[0]
        return (not self.true_fp32 and bias is None and w.dtype == torch.bfloat16 and x.dtype == torch.bfloat16
                and m <= self.SKINNY_MAX_ROWS and x.shape[0] <= 64 and w.shape[1] % 8 == 0 and w.stride(0) % 8 == 0
                and x.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0 and x.data_ptr() % 16 == 0)

    def _prepared(self, x, w, bias):
        """If ``x`` is a Normed whose input an earlier product already prepared (weighted, rounded values
        and per-tile sums of squares) and the fused kernel takes the product: that preparation."""
        if (isinstance(x, Normed) and x.ready is not None and x.pending is None and x._value is None
                and self._skinny_ok(x.ready["x"], w, bias, x.rows)):
            return x.ready
        return None

    def _skinny(self, x, w, epi, out, n_out, sink=None, prepared=None, rows=None, eps=0.0):
        """One launch of the few-row kernel.  ``sink`` naming a norm: also prepare that norm's input
        (returned).  ``prepared``: x is such a preparation; the norm is finished inside this product."""
        lib = self.lib("gemm_bf16")
        M = x.shape[0] if rows is None else rows.shape[0]
        made = None
        norm_args = [None, 0, None, 0, None, None, 0, 0.0, None]
        if sink is not None and sink.norm_weight is not None:
            g = sink.norm_weight
            tiles = -(-n_out // 16)
            # rows 64 bytes apart from a multiple of 4 KB: rows that are exactly 4 KB long fall on the same cache
            # channels when every workgroup reads all of them at once (qkv and o products 0.4 us faster at 8 rows)
            made = {"x": torch.empty((M, n_out + 32), dtype=torch.bfloat16, device=w.device)[:, :n_out],
                    "ss": torch.empty((M, (tiles + 3) // 4 * 4), dtype=torch.float32, device=w.device), "tiles": tiles}
            norm_args = [_ptr(g), int(g.dtype == torch.float32), _ptr(made["x"]), made["x"].stride(0), _ptr(made["ss"]), None, 0,
                         0.0, None]
        elif prepared is not None:
            norm_args = [None, 0, None, 0, None, _ptr(prepared["ss"]), prepared["tiles"], float(eps), _ptr(rows)]
        library.check(lib, lib.mie_skinny_gemm(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(0), epi,
                                               M, n_out, w.shape[1], *norm_args, self._stream()))
        return made

    # ---- products of 17 to 128 rows on a narrow weight: split over K, partial results, one kernel that adds
    # them up and does what follows the product
    MID_MAX_ROWS = 128
    MID_MAX_COLS = 4096        # wider weights have tiles enough for the library product without a split of K (8192 measured
                               # at hidden sizes of 4096: the same step times)
    RED_BF16, RED_F32, RED_ADD, RED_ADD_NORM = 0, 1, 2, 3

    def _mid_ok(self, x, w, bias) -> bool:
        """Whether the split product takes x w^T: more rows than the few-row kernel takes, up to 128 (measured at
        the benchmark's shapes, decode steps of 80 / 96 / 128 rows with every narrow product here against the
        library product and its separate epilogue kernel: 1.81 / 1.84 / 1.92 ms against 1.93 / 1.95 / 2.07)."""
        M = x.shape[0]
        return (not self.true_fp32 and bias is None and w.dtype == torch.bfloat16 and x.dtype == torch.bfloat16
                and self.SKINNY_MAX_ROWS < M <= self.MID_MAX_ROWS and w.shape[0] <= self.MID_MAX_COLS
                and w.shape[0] % 4 == 0 and w.shape[1] % 8 == 0 and w.stride(0) % 8 == 0 and x.stride(0) % 8 == 0
                and w.data_ptr() % 16 == 0 and x.data_ptr() % 16 == 0)

    @staticmethod
    def mid_splits(N: int, K: int) -> int:
        """Splits of K wanted for a weight [N, K]: enough for 256 workgroups of 64 weight rows, each split
        at least 256 wide.  A function of the weight's shape alone: a row's sums do not depend on its batch."""
        tiles = -(-N // 64)
        return max(1, min(8, 256 // tiles, K // 256))

    def _mid_partials(self, x, w):
        """part [splits, M, N] float32 of x w^T."""
        lib = self.lib("gemm_mid_bf16")
        M, K = x.shape
        N = w.shape[0]
        wanted = self.mid_splits(N, K)
        splits = lib.mie_mid_splits(K, wanted)
        part = torch.empty((splits, M, N), dtype=torch.float32, device=w.device)
        if self._zeros is None:
            self._zeros = torch.zeros(64, dtype=torch.int32, device=w.device)
        library.check(lib, lib.mie_mid_gemm(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(part), M, N, K, wanted,
                                            _ptr(self._zeros), self._stream()))
        return part

    def _mid_reduce(self, part, mode, out=None, stream=None, g=None, x_next=None, eps=0.0):
        lib = self.lib("gemm_mid_bf16")
        splits, M, N = part.shape
        library.check(lib, lib.mie_mid_reduce(
            _ptr(part), splits, M, N, mode, _ptr(out), out.stride(0) if out is not None else 0, _ptr(stream), _ptr(g),
            int(g is not None and g.dtype == torch.float32), _ptr(x_next), x_next.stride(0) if x_next is not None else 0,
            float(eps), self._stream()))

    def linear(self, x, w, bias=None, out_dtype=None, add_to=None):
        self._on_device(w, bias)
        _rows_ok(w, "linear: w")
        out_dtype = out_dtype or self.act_dtype
        M, K = x.shape
        if K != w.shape[1]:
            raise ValueError(f"linear: x {tuple(x.shape)} against w {tuple(w.shape)}")
        N = w.shape[0]
        sink = add_to if isinstance(add_to, Sink) or add_to is None else Sink(add_to)
        if sink is not None:
            st = sink.stream
            self._on_device(st)
            if st.dtype != torch.float32 or tuple(st.shape) != (M, N) or not st.is_contiguous():
                raise ValueError(f"linear: add_to must be the contiguous float32 stream {(M, N)}")
        prepared = self._prepared(x, w, bias)
        if prepared is not None and sink is None and out_dtype in (torch.bfloat16, torch.float32):
            out = torch.empty((M, N), dtype=out_dtype, device=w.device)
            self._skinny(prepared["x"], w, self.EPI_BF16 if out_dtype == torch.bfloat16 else self.EPI_F32, out, N,
                         prepared=prepared, rows=x.rows, eps=x.eps)
            return out
        if isinstance(x, Normed):
            x = x.materialize()
        self._on_device(x)
        _rows_ok(x, "linear: x")
        if self._skinny_ok(x, w, bias) and out_dtype in (torch.bfloat16, torch.float32):
            if sink is not None:
                made = self._skinny(x, w, self.EPI_ADD, sink.stream, N, sink=sink)
                if made is None:
                    return None
                return Normed(self, None, sink.stream, sink.norm_weight, sink.norm_eps, ready=made)
            out = torch.empty((M, N), dtype=out_dtype, device=w.device)
            self._skinny(x, w, self.EPI_BF16 if out_dtype == torch.bfloat16 else self.EPI_F32, out, N)
            return out
        if self._mid_ok(x, w, bias) and out_dtype in (torch.bfloat16, torch.float32):
            part = self._mid_partials(x, w)
            if sink is None:
                out = torch.empty((M, N), dtype=out_dtype, device=w.device)
                self._mid_reduce(part, self.RED_BF16 if out_dtype == torch.bfloat16 else self.RED_F32, out=out)
                return out
            g = sink.norm_weight
            if g is None or g.dtype not in (torch.bfloat16, torch.float32) or tuple(g.shape) != (N,) or not g.is_contiguous():
                self._mid_reduce(part, self.RED_ADD, stream=sink.stream)
                return None
            normed = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
            self._mid_reduce(part, self.RED_ADD_NORM, stream=sink.stream, g=g, x_next=normed, eps=sink.norm_eps)
            done = Normed(self, None, sink.stream, g, sink.norm_eps)
            done._value = normed            # the norm is computed: materialize() hands this out
            return done
        if not self.true_fp32 and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
            # library matrix product, 32-bit accumulation, as the reference's F.linear.  What goes into the
            # float32 stream or out as logits leaves the product in float32: the sums are not rounded to
            # bfloat16 on their way there, whatever the number of rows.
            own_call = bias is None and self._lt_ok(x, w)
            if bias is None and sink is not None:
                # the product adds its float32 sums to the stream itself (C = C + A B in place): the stream is
                # not read and written once more by a kernel of its own
                if own_call:
                    self._lt_product(x, w, self.LT_ADD, sink.stream)
                else:
                    torch.ops.aten.addmm.dtype_out(sink.stream, x, w.t(), torch.float32, out=sink.stream)
                if sink.norm_weight is None:
                    return None
                return Normed(self, None, sink.stream, sink.norm_weight, sink.norm_eps)
            if bias is None and out_dtype == torch.float32:
                if own_call:
                    return self._lt_product(x, w, self.LT_F32, torch.empty((M, N), dtype=torch.float32, device=w.device))
                return torch.mm(x, w.t(), out_dtype=torch.float32)
            if own_call and out_dtype == torch.bfloat16:
                return self._lt_product(x, w, self.LT_BF16, torch.empty((M, N), dtype=torch.bfloat16, device=w.device))
            y = torch.nn.functional.linear(x, w, None if bias is None else bias.to(torch.bfloat16))
            return y if out_dtype == torch.bfloat16 else y.to(out_dtype)
        return self._gemm(x, w, bias, out_dtype)

    def silu_mul(self, gu, intermediate):
        _rows_ok(gu, "silu_mul: gu")
        if gu.shape[1] != 2 * intermediate:
            raise ValueError(f"silu_mul: {gu.shape[1]} columns for intermediate {intermediate}")
        out = torch.empty((gu.shape[0], intermediate), dtype=gu.dtype, device=gu.device)
        lib = self.lib("gemm")
        library.check(lib, lib.mie_silu_mul(_ptr(gu), gu.stride(0), _ptr(out), out.stride(0), _code(gu.dtype),
                                            gu.shape[0], intermediate, self._stream()))
        return out

    def linear_silu_mul(self, x, w_gate_up, intermediate):
        if w_gate_up.shape[0] != 2 * intermediate:
            raise ValueError(f"linear_silu_mul: weight of {w_gate_up.shape[0]} rows for intermediate {intermediate}")
        if x.shape[1] != w_gate_up.shape[1]:
            raise ValueError(f"linear_silu_mul: x {tuple(x.shape)} against w {tuple(w_gate_up.shape)}")
        prepared = self._prepared(x, w_gate_up, None)
        if prepared is not None:
            out = torch.empty((x.shape[0], intermediate), dtype=torch.bfloat16, device=w_gate_up.device)
            self._skinny(prepared["x"], w_gate_up, self.EPI_SWIGLU, out, intermediate, prepared=prepared, rows=x.rows,
                         eps=x.eps)
            return out
        if isinstance(x, Normed):
            x = x.materialize()
        if self._skinny_ok(x, w_gate_up, None):
            out = torch.empty((x.shape[0], intermediate), dtype=torch.bfloat16, device=w_gate_up.device)
            self._skinny(x, w_gate_up, self.EPI_SWIGLU, out, intermediate)
            return out
        return self.silu_mul(self.linear(x, w_gate_up), intermediate)

    ACT_CODES = {"none": 0, "silu": 1, "gelu_tanh": 2, "relu2": 3}

    def linear_act_mul(self, x, w_gate_up, intermediate, activation="silu"):
        if activation == "silu":
            return self.linear_silu_mul(x, w_gate_up, intermediate)
        if activation not in self.ACT_CODES:
            raise ValueError(f"linear_act_mul: activation {activation!r}")
        if w_gate_up.shape[0] != 2 * intermediate or x.shape[1] != w_gate_up.shape[1]:
            raise ValueError(f"linear_act_mul: x {tuple(x.shape)}, w {tuple(w_gate_up.shape)}, intermediate {intermediate}")
        if isinstance(x, Normed):
            x = x.materialize()
        if activation == "gelu_tanh" and self._skinny_ok(x, w_gate_up, None):      # few rows: the gate in the product's epilogue
            out = torch.empty((x.shape[0], intermediate), dtype=torch.bfloat16, device=w_gate_up.device)
            self._skinny(x, w_gate_up, self.EPI_GEGLU, out, intermediate)
            return out
        gu = self.linear(x, w_gate_up)
        out = torch.empty((gu.shape[0], intermediate), dtype=gu.dtype, device=gu.device)
        lib = self.lib("gemm")
        library.check(lib, lib.mie_act_mul(_ptr(gu), gu.stride(0), _ptr(out), out.stride(0), _code(gu.dtype), gu.shape[0],
                                           intermediate, self.ACT_CODES[activation], self._stream()))
        return out

    def linear_act(self, x, w, activation="relu2"):
        if activation not in self.ACT_CODES:
            raise ValueError(f"linear_act: activation {activation!r}")
        sums = self.linear(x, w, out_dtype=torch.float32)
        out = torch.empty(sums.shape, dtype=self.act_dtype, device=sums.device)
        lib = self.lib("gemm")
        library.check(lib, lib.mie_act_store(_ptr(sums), sums.stride(0), _ptr(out), out.stride(0), _code(out.dtype),
                                             sums.shape[0], sums.shape[1], self.ACT_CODES[activation], self._stream()))
        return out

    def scale_(self, t, factor):
        self._on_device(t)
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise ValueError("scale_: a contiguous float32 tensor")
        lib = self.lib("embed_norm")
        library.check(lib, lib.mie_scale(_ptr(t), t.numel(), float(factor), self._stream()))
        return t

    def scale_softcap_(self, t, scale, cap):
        self._on_device(t)
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise ValueError("scale_softcap_: a contiguous float32 tensor")
        if cap is not None and not cap > 0:
            raise ValueError(f"scale_softcap_: cap {cap}")
        lib = self.lib("layer_norm")
        library.check(lib, lib.mie_scale_softcap(_ptr(t), t.numel(), float(scale), float(cap or 0.0), self._stream()))
        return t

    def add_layernorm(self, x, residual, weight, bias, eps, out_dtype=None, rows=None):
        self._on_device(x, residual, weight, bias, rows)
        out_dtype = out_dtype or self.act_dtype
        if residual.dtype != torch.float32 or residual.dim() != 2 or not residual.is_contiguous():
            raise ValueError("add_layernorm: the residual stream must be contiguous float32 [T, width]")
        T, W = residual.shape
        if x is not None and (tuple(x.shape) != (T, W) or not x.is_contiguous()):
            raise ValueError(f"add_layernorm: x {tuple(x.shape)} does not match the stream {(T, W)}")
        self._f32_vector(weight, W, "add_layernorm: weight")
        self._f32_vector(bias, W, "add_layernorm: bias")
        n = T
        if rows is not None:
            if rows.dtype != torch.int32 or rows.dim() != 1 or not rows.is_contiguous():
                raise ValueError("add_layernorm: rows must be contiguous int32")
            n = rows.shape[0]
        y = torch.empty((n, W), dtype=out_dtype, device=residual.device)
        lib = self.lib("layer_norm")
        library.check(lib, lib.mie_add_layernorm(_ptr(x), _code(x.dtype) if x is not None else F32, _ptr(residual), _ptr(weight),
                                                 _ptr(bias), _ptr(y), _code(out_dtype), _ptr(rows), n, W, float(eps),
                                                 self._stream()))
        return y

    def branch_layernorm_add(self, y, stream, weight, bias, eps, next_norm=None):
        self._on_device(y, stream, weight, bias)
        if stream.dtype != torch.float32 or stream.dim() != 2 or not stream.is_contiguous():
            raise ValueError("branch_layernorm_add: the stream must be contiguous float32 [T, width]")
        T, W = stream.shape
        if tuple(y.shape) != (T, W) or not y.is_contiguous():
            raise ValueError(f"branch_layernorm_add: y {tuple(y.shape)} does not match the stream {(T, W)}")
        self._f32_vector(weight, W, "branch_layernorm_add: weight")
        self._f32_vector(bias, W, "branch_layernorm_add: bias")
        x, nw, nb, ne = None, None, None, 0.0
        if next_norm is not None:
            nw, nb, ne = next_norm
            self._on_device(nw, nb)
            self._f32_vector(nw, W, "branch_layernorm_add: the next norm's weight")
            self._f32_vector(nb, W, "branch_layernorm_add: the next norm's bias")
            x = torch.empty((T, W), dtype=self.act_dtype, device=stream.device)
        lib = self.lib("layer_norm")
        library.check(lib, lib.mie_branch_layernorm_add(_ptr(y), _code(y.dtype), _ptr(stream), _ptr(weight), _ptr(bias), float(eps),
                                                        _ptr(nw), _ptr(nb), float(ne), _ptr(x), _code(self.act_dtype), T, W,
                                                        self._stream()))
        return x

    def branch_norm_add(self, y, stream, weight, eps, copy=True):
        self._on_device(y, stream, weight)
        if stream.dtype != torch.float32 or stream.dim() != 2 or not stream.is_contiguous():
            raise ValueError("branch_norm_add: the stream must be contiguous float32 [T, width]")
        T, W = stream.shape
        if y is not None:
            if tuple(y.shape) != (T, W) or not y.is_contiguous():
                raise ValueError(f"branch_norm_add: y {tuple(y.shape)} does not match the stream {(T, W)}")
            if weight is None or tuple(weight.shape) != (W,) or not weight.is_contiguous():
                raise ValueError(f"branch_norm_add: a contiguous weight of {W}")
        want_copy = copy
        copy = None if self.act_dtype == torch.float32 or not want_copy else torch.empty((T, W), dtype=self.act_dtype,
                                                                                         device=stream.device)
        if y is not None or copy is not None:
            lib = self.lib("embed_norm")
            library.check(lib, lib.mie_branch_norm_add(
                _ptr(y), _code(y.dtype) if y is not None else F32, _ptr(stream), _ptr(weight),
                _code(weight.dtype) if weight is not None else F32, _ptr(copy), _code(copy.dtype) if copy is not None else F32,
                T, W, float(eps), self._stream()))
        if not want_copy:
            return None
        return stream if copy is None else copy

    @staticmethod
    def _f32_columns(x, col, n, what):
        if x.dtype != torch.float32 or x.dim() != 2 or x.stride(1) != 1 or col < 0 or col + n > x.shape[1]:
            raise ValueError(f"{what}: columns {col} .. {col + n} of a float32 matrix with unit inner stride, got "
                             f"{tuple(x.shape)} {x.dtype}")
        return c_void_p(x.data_ptr() + 4 * col)

    @staticmethod
    def _f32_vector(t, n, what):
        if t is None or t.dtype != torch.float32 or t.numel() != n or not t.is_contiguous():
            raise ValueError(f"{what}: {n} contiguous float32 numbers expected")
        return _ptr(t)

    def rmsnorm_columns(self, x, col, n, weight, eps):
        self._on_device(x, weight)
        xp = self._f32_columns(x, col, n, "rmsnorm_columns")
        if tuple(weight.shape) != (n,) or not weight.is_contiguous():
            raise ValueError(f"rmsnorm_columns: weight {tuple(weight.shape)} for {n} columns")
        out = torch.empty((x.shape[0], n), dtype=self.act_dtype, device=x.device)
        lib = self.lib("embed_norm")
        library.check(lib, lib.mie_rmsnorm_columns(xp, x.stride(0), _ptr(weight), _code(weight.dtype), _ptr(out),
                                                   _code(out.dtype), x.shape[0], n, float(eps), self._stream()))
        return out

    # ---- many small products in one launch
    def _grouped(self, A, lda, a_group, a_mod, W, ldw, w_group, C, ldc, c_group, M, N, K, G, bias=None, gate=None, ldg=0,
                 offs=None, gather=None, gather_div=1, act="none"):
        lib = self.lib("grouped_gemm")
        if self._zeros is None:
            self._zeros = torch.zeros(64, dtype=torch.int32, device=W.device)
        library.check(lib, lib.mie_grouped_linear(
            _ptr(A), _code(A.dtype), lda, a_group, a_mod, _ptr(W), _code(W.dtype), ldw, w_group, _ptr(C), _code(C.dtype), ldc,
            c_group, _ptr(bias), gate, ldg, _ptr(offs), _ptr(gather), gather_div, M, N, K, G, self.ACT_CODES[act],
            _ptr(self._zeros), self._stream()))

    def grouped_linear(self, x, w, bias=None, x_groups=None):
        self._on_device(x, w, bias)
        _rows_ok(x, "grouped_linear: x")
        if w.dim() != 3 or not w.is_contiguous():
            raise ValueError("grouped_linear: w must be contiguous [groups, out, in]")
        G, N, K = w.shape
        gx = int(x_groups or G)
        if x.shape[1] != gx * K:
            raise ValueError(f"grouped_linear: x {tuple(x.shape)} for {gx} blocks of {K}")
        if bias is not None:
            self._f32_vector(bias, G * N, "grouped_linear: bias")
        out = torch.empty((x.shape[0], G * N), dtype=torch.float32, device=x.device)
        self._grouped(x, x.stride(0), K, gx, w, K, N * K, out, G * N, N, x.shape[0], N, K, G, bias=bias)
        return out

    # ---- attention through a cached latent
    def _check_latent_cache(self, what, k_cache, v_cache, kv_rank, rot_dim):
        pages, one, page, P = k_cache.shape
        if one != 1 or tuple(v_cache.shape) != (pages, 1, P, page) or P < kv_rank + rot_dim:
            raise ValueError(f"{what}: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} for a latent of {kv_rank} + {rot_dim}")
        if k_cache.dtype != v_cache.dtype or not (k_cache.is_contiguous() and v_cache.is_contiguous()):
            raise ValueError(f"{what}: caches must be contiguous and of one dtype")
        return page, P

    def latent_kv_store(self, sums, col, kv_rank, rot_dim, norm_weight, eps, positions, inv_freq, k_cache, v_cache,
                        slot_mapping, also_norm=None, layout="interleaved"):
        self._on_device(sums, norm_weight, positions, inv_freq, k_cache, v_cache, slot_mapping)
        if layout not in self.LAYOUTS:
            raise ValueError(f"latent_kv_store: layout {layout!r} (interleaved or half)")
        if also_norm is not None and (k_cache.dtype != self.act_dtype or also_norm[2].dtype != norm_weight.dtype):
            # the kernel writes both in one dtype and reads both weights in one: otherwise two calls
            self.latent_kv_store(sums, col, kv_rank, rot_dim, norm_weight, eps, positions, inv_freq, k_cache, v_cache, slot_mapping,
                                 layout=layout)
            return self.rmsnorm_columns(sums, also_norm[0], also_norm[1], also_norm[2], eps)
        sp = self._f32_columns(sums, col, kv_rank + rot_dim, "latent_kv_store")
        T = sums.shape[0]
        page, P = self._check_latent_cache("latent_kv_store", k_cache, v_cache, kv_rank, rot_dim)
        if tuple(norm_weight.shape) != (kv_rank,) or not norm_weight.is_contiguous():
            raise ValueError(f"latent_kv_store: norm weight {tuple(norm_weight.shape)} for a latent of {kv_rank}")
        n_freq = inv_freq.numel()
        self._f32_vector(inv_freq, n_freq, "latent_kv_store: inv_freq")
        for name, t in (("positions", positions), ("slot_mapping", slot_mapping)):
            if t.dtype != torch.int32 or t.shape[0] != T or not t.is_contiguous():
                raise ValueError(f"latent_kv_store: {name} must be contiguous int32 [{T}]")
        qp, qw, q_out, qn = None, None, None, 0
        if also_norm is not None:
            qcol, qn, qweight = also_norm
            qp = self._f32_columns(sums, qcol, qn, "latent_kv_store: query latent")
            if tuple(qweight.shape) != (qn,) or not qweight.is_contiguous():
                raise ValueError(f"latent_kv_store: query norm weight {tuple(qweight.shape)} for {qn} columns")
            self._on_device(qweight)
            qw = _ptr(qweight)
            q_out = torch.empty((T, qn), dtype=self.act_dtype, device=sums.device)
        lib = self.lib("latent_attention")
        library.check(lib, lib.mie_latent_kv_store(
            sp, sums.stride(0), _ptr(norm_weight), _code(norm_weight.dtype), float(eps), _ptr(positions), _ptr(inv_freq), n_freq,
            _ptr(k_cache), _ptr(v_cache), _code(k_cache.dtype), _ptr(slot_mapping), T, kv_rank, rot_dim, P, page,
            qp, qw, _ptr(q_out), qn, self.LAYOUTS[layout], self._stream()))
        return q_out

    def latent_query_rotate_(self, q, num_heads, kv_rank, padded_dim, positions, inv_freq, layout="interleaved"):
        self._on_device(q, positions, inv_freq)
        if layout not in self.LAYOUTS:
            raise ValueError(f"latent_query_rotate_: layout {layout!r} (interleaved or half)")
        _rows_ok(q, "latent_query_rotate_: q")
        H, P, T = num_heads, padded_dim, q.shape[0]
        n_freq = inv_freq.numel()
        if q.shape[1] != H * P or P < kv_rank + 2 * n_freq:
            raise ValueError(f"latent_query_rotate_: q {tuple(q.shape)} for {H} heads of {P}, latent {kv_rank}, {n_freq} turned pairs")
        if positions.dtype != torch.int32 or positions.shape[0] != T or not positions.is_contiguous():
            raise ValueError(f"latent_query_rotate_: positions must be contiguous int32 [{T}]")
        self._f32_vector(inv_freq, n_freq, "latent_query_rotate_: inv_freq")
        lib = self.lib("latent_attention")
        library.check(lib, lib.mie_latent_query_rotate(_ptr(q), q.stride(0), _code(q.dtype), _ptr(positions), _ptr(inv_freq),
                                                       n_freq, T, H, kv_rank, P, self.LAYOUTS[layout], self._stream()))
        return q

    def latent_value_gate(self, o, w_uv, gate, gate_col, num_heads, vdim, kv_rank, padded_dim):
        self._on_device(o, w_uv, gate)
        H, P, T = num_heads, padded_dim, o.shape[0]
        if tuple(o.shape) != (T, H * P) or not o.is_contiguous() or tuple(w_uv.shape) != (H * vdim, kv_rank) or not w_uv.is_contiguous():
            raise ValueError(f"latent_value_gate: o {tuple(o.shape)}, w {tuple(w_uv.shape)} for {H} heads of {vdim}, latent {kv_rank}")
        gp, ldg = None, 0
        if gate is not None:
            gp, ldg = self._f32_columns(gate, gate_col, H * vdim, "latent_value_gate: gate"), gate.stride(0)
            if gate.shape[0] != T:
                raise ValueError("latent_value_gate: one gate row a token")
        out = torch.empty((T, H * vdim), dtype=o.dtype, device=o.device)
        self._grouped(o, H * P, P, H, w_uv, kv_rank, vdim * kv_rank, out, H * vdim, vdim, T, vdim, kv_rank, H, gate=gp, ldg=ldg)
        return out

    # ---- gated linear recurrence
    SCAN_CHUNK = 32          # tokens a chunk of the recurrence's scan; rows up to this long run in one pass

    def _check_rows(self, what, step, T):
        for name, t, n in (("token_row", step.token_row, T), ("row_start", step.row_start, step.num_rows + 1),
                           ("state_slots", step.state_slots, step.num_rows)):
            if t is None or t.dtype != torch.int32 or t.shape[0] < n or not t.is_contiguous():
                raise ValueError(f"{what}: {name} must be contiguous int32 [{n}]")
        if step.num_tokens != T:
            raise ValueError(f"{what}: {T} tokens for a step of {step.num_tokens}")

    def causal_conv(self, x, col, channels, in_bias, taps, conv_bias, tail, step):
        self._on_device(x, in_bias, taps, conv_bias, tail)
        C, T = channels, x.shape[0]
        xp = self._f32_columns(x, col, C, "causal_conv")
        if taps.dim() != 2 or taps.shape[0] != C:
            raise ValueError(f"causal_conv: taps {tuple(taps.shape)} for {C} channels")
        K = taps.shape[1]
        self._f32_vector(taps, C * K, "causal_conv: taps")
        self._f32_vector(in_bias, C, "causal_conv: input bias")
        self._f32_vector(conv_bias, C, "causal_conv: bias")
        if tail.dtype != torch.float32 or tuple(tail.shape[1:]) != (max(1, K - 1), C) or not tail.is_contiguous():
            raise ValueError(f"causal_conv: tail {tuple(tail.shape)} for {K} taps of {C} channels")
        self._check_rows("causal_conv", step, T)
        if int(step.host["state_slots"].max()) >= tail.shape[0]:
            raise ValueError("causal_conv: a state slot beyond the tail's slots")
        u = torch.empty((T, C), dtype=torch.float32, device=x.device)
        lib = self.lib("recurrence")
        library.check(lib, lib.mie_causal_conv(xp, x.stride(0), _ptr(in_bias), _ptr(taps), _ptr(conv_bias), _ptr(tail),
                                               _ptr(step.token_row), _ptr(step.row_start), _ptr(step.state_slots), _ptr(u),
                                               T, C, K, self._stream()))
        return u

    def rglru_scan(self, u, gates, lam, y, y_col, y_bias, x, x_col, x_bias, state, tail, step, taps, decay_scale=8.0):
        self._on_device(u, gates, lam, y, y_bias, x, x_bias, state, tail)
        T, C = u.shape
        if u.dtype != torch.float32 or not u.is_contiguous() or gates.dtype != torch.float32 or tuple(gates.shape) != (T, 2 * C) \
                or not gates.is_contiguous():
            raise ValueError(f"rglru_scan: u {tuple(u.shape)} and gates {tuple(gates.shape)} must be contiguous float32 [T, C], [T, 2 C]")
        yp = self._f32_columns(y, y_col, C, "rglru_scan: y")
        xp = self._f32_columns(x, x_col, C, "rglru_scan: x")
        if y.shape[0] != T or x.shape[0] != T:
            raise ValueError("rglru_scan: one row of y and x a token")
        for name, t in (("lam", lam), ("y_bias", y_bias), ("x_bias", x_bias)):
            self._f32_vector(t, C, f"rglru_scan: {name}")
        K = int(taps)
        if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] != C or not state.is_contiguous() \
                or tail.dtype != torch.float32 or tuple(tail.shape) != (state.shape[0], max(1, K - 1), C) \
                or not tail.is_contiguous():
            raise ValueError(f"rglru_scan: state {tuple(state.shape)}, tail {tuple(tail.shape)} for {C} channels")
        self._check_rows("rglru_scan", step, T)
        if int(step.host["state_slots"].max()) >= state.shape[0]:
            raise ValueError("rglru_scan: a state slot beyond the state's slots")
        out = torch.empty((T, C), dtype=self.act_dtype, device=u.device)
        lib = self.lib("recurrence")
        longest = int(getattr(step, "max_row_tokens", 0) or (step.host["row_start"][1:] - step.host["row_start"][:-1]).max())
        if longest > self.SCAN_CHUNK:
            # rows of many tokens: chunks side by side (whether a step takes this path depends on its longest row
            # alone; the two paths differ by the rounding of the fold over whole chunks)
            chunks = -(-longest // self.SCAN_CHUNK)
            scratch = torch.empty((2 * step.num_rows * chunks + step.num_rows, C), dtype=torch.float32, device=u.device)
            n = step.num_rows * chunks
            library.check(lib, lib.mie_rglru_scan_chunked(
                _ptr(u), _ptr(gates), _ptr(lam), yp, y.stride(0), _ptr(y_bias), xp, x.stride(0), _ptr(x_bias), _ptr(state),
                _ptr(tail), _ptr(step.row_start), _ptr(step.state_slots), _ptr(out), _code(out.dtype), step.num_rows, C, K,
                float(decay_scale), self.SCAN_CHUNK, chunks, _ptr(scratch[:n]), _ptr(scratch[n:2 * n]), _ptr(scratch[2 * n:]),
                self._stream()))
            return out
        library.check(lib, lib.mie_rglru_scan(_ptr(u), _ptr(gates), _ptr(lam), yp, y.stride(0), _ptr(y_bias), xp, x.stride(0),
                                              _ptr(x_bias), _ptr(state), _ptr(tail), _ptr(step.row_start), _ptr(step.state_slots),
                                              _ptr(out), _code(out.dtype), step.num_rows, C, K, float(decay_scale), self._stream()))
        return out

    # ---- routed experts
    def route_topk(self, logits, bias, top, over="chosen", choice_bias=None, renormalise=False):
        self._on_device(logits, bias, choice_bias)
        if over not in ("chosen", "all") or ((choice_bias is not None or renormalise) and over != "all"):
            raise ValueError(f"route_topk: shares over {over!r} (chosen or all; a choice bias or renormalised shares go with all)")
        if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
            raise ValueError("route_topk: logits must be float32 [T, experts] with unit inner stride")
        T, E = logits.shape
        if bias is not None:
            self._f32_vector(bias, E, "route_topk: bias")
        if not 1 <= top <= min(E, 16):
            raise ValueError(f"route_topk: top {top} of {E} experts (at most 16)")
        experts = torch.empty((T, top), dtype=torch.int32, device=logits.device)
        shares = torch.empty((T, top), dtype=torch.float32, device=logits.device)
        lib = self.lib("grouped_gemm")
        if over == "all":
            if choice_bias is not None:
                self._f32_vector(choice_bias, E, "route_topk: choice bias")
            library.check(lib, lib.mie_route_topk_all(_ptr(logits), logits.stride(0), _ptr(bias), _ptr(choice_bias), _ptr(experts),
                                                      _ptr(shares), T, E, top, int(bool(renormalise)), self._stream()))
            return experts, shares
        library.check(lib, lib.mie_route_topk(_ptr(logits), logits.stride(0), _ptr(bias), _ptr(experts), _ptr(shares), T, E, top,
                                              self._stream()))
        return experts, shares

    GLU_BLOCK = 16      # the matrix-core kernel's tiles are 16 columns wide: a lane holds columns c and c + 16 of its row

    def glu_rows_block(self, inner):
        return self.GLU_BLOCK if self.act_dtype == torch.bfloat16 and inner % self.GLU_BLOCK == 0 else 0

    def routed_experts(self, x, experts, shares, w_up, w_down, activation="relu2", gated=None, identity_from=None,
                       glu_block=0):
        self._on_device(x, experts, shares, w_up, w_down)
        _rows_ok(x, "routed_experts: x")
        T, W = x.shape
        top = experts.shape[1]
        if experts.dtype != torch.int32 or tuple(experts.shape) != (T, top) or not experts.is_contiguous() \
                or shares.dtype != torch.float32 or tuple(shares.shape) != (T, top) or not shares.is_contiguous():
            raise ValueError("routed_experts: experts int32 [T, top] and shares float32 [T, top], contiguous")
        dev = x.device
        lib = self.lib("grouped_gemm")
        out = torch.empty((T, W), dtype=torch.float32, device=dev)
        n = T * top
        if w_up is None:            # every choice stands for the token's own input
            if identity_from != 0 or w_down is not None:
                raise ValueError("routed_experts: experts without matrices must all be identity experts (identity_from 0)")
            library.check(lib, lib.mie_moe_combine_identity(None, _ptr(experts), _ptr(shares), _ptr(out), T, W, top, _ptr(experts),
                                                            0, _ptr(x), _code(x.dtype), x.stride(0), self._stream()))
            return out
        if w_up.dim() != 3 or w_down.dim() != 3 or not (w_up.is_contiguous() and w_down.is_contiguous()):
            raise ValueError("routed_experts: contiguous [experts, ff, width] and [experts, width, ff]")
        E, up_rows, _ = w_up.shape
        ff = up_rows if gated is None else up_rows // 2
        if w_up.shape[2] != W or tuple(w_down.shape) != (E, W, ff) or (gated is not None and up_rows != 2 * ff):
            raise ValueError(f"routed_experts: w_up {tuple(w_up.shape)}, w_down {tuple(w_down.shape)} for width {W}")
        if identity_from is not None and identity_from != E:
            raise ValueError(f"routed_experts: identity experts from {identity_from} on, but {E} experts have matrices")
        if gated is None and activation not in self.ACT_CODES:
            raise ValueError(f"routed_experts: activation {activation!r}")
        if gated is not None:
            gated = (float(gated[0]), float(gated[1]), float(gated[2]) if len(gated) > 2 else 1.0)
            if not gated[0] > 0:
                raise ValueError(f"routed_experts: the gate's limit {gated[0]} must be positive (infinite: no clamp)")
        groups = E if identity_from is None else E + 1      # one more group behind the experts holds every identity choice
        offs = torch.empty(groups + 1, dtype=torch.int32, device=dev)
        order = torch.empty(n, dtype=torch.int32, device=dev)
        place = torch.empty(n, dtype=torch.int32, device=dev)
        # identity choices are sorted behind the experts' (the sort clamps every choice >= the last group into it), so
        # the grouped products, which walk the first E groups, never see them
        library.check(lib, lib.mie_moe_align(_ptr(experts), n, groups, _ptr(offs), _ptr(order), _ptr(place), self._stream()))
        hidden = torch.empty((n, ff), dtype=self.act_dtype, device=dev)
        if gated is None:
            self._grouped(x, x.stride(0), 0, 1, w_up, W, ff * W, hidden, ff, 0, n, ff, W, E, offs=offs, gather=order,
                          gather_div=top, act=activation)
        elif (glu_block == self.GLU_BLOCK and x.dtype == torch.bfloat16 and w_up.dtype == torch.bfloat16 and W % 8 == 0
              and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w_up.data_ptr() % 16 == 0):
            # gate and up sums meet in the product's own epilogue: the hidden activation is written once, rounded once
            if self._zeros is None:
                self._zeros = torch.zeros(64, dtype=torch.int32, device=dev)
            limit, alpha, shift = gated
            library.check(lib, lib.mie_grouped_glu(_ptr(x), _code(x.dtype), x.stride(0), _ptr(w_up), _code(w_up.dtype), W,
                                                   2 * ff * W, _ptr(hidden), _code(hidden.dtype), ff, _ptr(offs), _ptr(order),
                                                   top, n, 2 * ff, W, E, limit, alpha, shift, _ptr(self._zeros),
                                                   self._stream()))
        else:
            if glu_block and ff % glu_block:
                raise ValueError(f"routed_experts: blocks of {glu_block} rows in experts of inner size {ff}")
            limit, alpha, shift = gated
            gu = torch.empty((n, 2 * ff), dtype=torch.float32, device=dev)
            self._grouped(x, x.stride(0), 0, 1, w_up, W, 2 * ff * W, gu, 2 * ff, 0, n, 2 * ff, W, E, offs=offs, gather=order,
                          gather_div=top)
            glib = self.lib("gemm")
            # rows of identity choices hold whatever was there: the function of it is never read
            library.check(glib, glib.mie_clamped_glu(_ptr(gu), gu.stride(0), _ptr(hidden), hidden.stride(0), _code(hidden.dtype),
                                                     n, ff, limit, alpha, shift, int(glu_block), self._stream()))
        y = torch.empty((n, W), dtype=torch.float32, device=dev)
        self._grouped(hidden, ff, 0, 1, w_down, ff, W * ff, y, W, 0, n, W, ff, E, offs=offs)
        if identity_from is None:
            library.check(lib, lib.mie_moe_combine(_ptr(y), _ptr(place), _ptr(shares), _ptr(out), T, W, top, self._stream()))
        else:
            library.check(lib, lib.mie_moe_combine_identity(_ptr(y), _ptr(place), _ptr(shares), _ptr(out), T, W, top,
                                                            _ptr(experts), E, _ptr(x), _code(x.dtype), x.stride(0),
                                                            self._stream()))
        return out

    # ---- a short convolution on a mixer's input, attention from one product's sums, the delta rule
    def residual_conv(self, h, taps, tail, step, out_dtype=None):
        self._on_device(h, taps, tail)
        out_dtype = out_dtype or self.act_dtype
        if h.dtype != torch.float32 or h.dim() != 2 or not h.is_contiguous():
            raise ValueError("residual_conv: h must be contiguous float32 [T, channels]")
        T, C = h.shape
        if taps.dim() != 2 or taps.shape[0] != C:
            raise ValueError(f"residual_conv: taps {tuple(taps.shape)} for {C} channels")
        K = taps.shape[1]
        self._f32_vector(taps, C * K, "residual_conv: taps")
        if tail.dtype != torch.float32 or tuple(tail.shape[1:]) != (max(1, K - 1), C) or not tail.is_contiguous():
            raise ValueError(f"residual_conv: tail {tuple(tail.shape)} for {K} taps of {C} channels")
        self._check_rows("residual_conv", step, T)
        if int(step.host["state_slots"].max()) >= tail.shape[0]:
            raise ValueError("residual_conv: a state slot beyond the tail's slots")
        y = torch.empty((T, C), dtype=out_dtype, device=h.device)
        lib = self.lib("recurrence")
        library.check(lib, lib.mie_residual_conv(_ptr(h), _ptr(taps), _ptr(tail), _ptr(step.token_row), _ptr(step.row_start),
                                                 _ptr(step.state_slots), _ptr(y), _code(out_dtype), T, step.num_rows, C, K,
                                                 self._stream()))
        return y

    NORM_CONV_MAX_TAPS = 8

    def norm_pair_conv(self, stream, w_first, w_second, eps, taps, tail, step):
        self._on_device(stream, w_first, w_second, taps, tail)
        K = taps.shape[1] if taps.dim() == 2 else 0
        plain = lambda t: t is None or (t.dtype == torch.float32 and t.is_contiguous())      # noqa: E731
        if not 1 <= K <= self.NORM_CONV_MAX_TAPS or not (plain(w_first) and plain(w_second)):
            return super().norm_pair_conv(stream, w_first, w_second, eps, taps, tail, step)
        if stream.dtype != torch.float32 or stream.dim() != 2 or not stream.is_contiguous():
            raise ValueError("norm_pair_conv: the stream must be contiguous float32 [T, width]")
        T, W = stream.shape
        self._f32_vector(w_first, W, "norm_pair_conv: first weight")
        if w_second is not None:
            self._f32_vector(w_second, W, "norm_pair_conv: second weight")
        if taps.shape[0] != W:
            raise ValueError(f"norm_pair_conv: taps {tuple(taps.shape)} for width {W}")
        self._f32_vector(taps, W * K, "norm_pair_conv: taps")
        if tail.dtype != torch.float32 or tuple(tail.shape[1:]) != (max(1, K - 1), W) or not tail.is_contiguous():
            raise ValueError(f"norm_pair_conv: tail {tuple(tail.shape)} for {K} taps of width {W}")
        self._check_rows("norm_pair_conv", step, T)
        if int(step.host["state_slots"].max()) >= tail.shape[0]:
            raise ValueError("norm_pair_conv: a state slot beyond the tail's slots")
        x = torch.empty((T, W), dtype=self.act_dtype, device=stream.device)
        y = torch.empty((T, W), dtype=self.act_dtype, device=stream.device) if w_second is not None else None
        rstd = torch.empty(T, dtype=torch.float32, device=stream.device)
        lib = self.lib("embed_norm")
        library.check(lib, lib.mie_norm_pair_conv(_ptr(stream), _ptr(w_first), _ptr(w_second), _ptr(taps), _ptr(tail),
                                                  _ptr(step.token_row), _ptr(step.row_start), _ptr(step.state_slots), _ptr(x),
                                                  _ptr(y), _code(self.act_dtype), _ptr(rstd), T, step.num_rows, W, K, float(eps),
                                                  self._stream()))
        return x, y

    def branch_norm_conv(self, y, stream, w_out, eps_out, w_next, eps_next, taps, tail, step):
        K = taps.shape[1] if taps.dim() == 2 else 0
        T, W = stream.shape
        f32 = lambda t: t.dtype == torch.float32 and t.is_contiguous() and t.data_ptr() % 16 == 0      # noqa: E731
        # steps whose rows are single tokens: one kernel adds the branch and makes the next input
        if (step.num_rows != T or not 1 <= K <= self.NORM_CONV_MAX_TAPS or W % 4 or W > 8192
                or not all(f32(t) for t in (y, stream, w_out, w_next, taps, tail))):
            return super().branch_norm_conv(y, stream, w_out, eps_out, w_next, eps_next, taps, tail, step)
        self._on_device(y, stream, w_out, w_next, taps, tail)
        if tuple(y.shape) != (T, W) or tuple(taps.shape) != (W, K) or tuple(tail.shape[1:]) != (max(1, K - 1), W):
            raise ValueError(f"branch_norm_conv: y {tuple(y.shape)}, taps {tuple(taps.shape)}, tail {tuple(tail.shape)} "
                             f"for a stream of {(T, W)}")
        self._f32_vector(w_out, W, "branch_norm_conv: the branch's norm weight")
        self._f32_vector(w_next, W, "branch_norm_conv: the next norm's weight")
        if int(step.host["state_slots"].max()) >= tail.shape[0]:
            raise ValueError("branch_norm_conv: a state slot beyond the tail's slots")
        x = torch.empty((T, W), dtype=self.act_dtype, device=stream.device)
        lib = self.lib("embed_norm")
        library.check(lib, lib.mie_branch_norm_conv_single(_ptr(y), _ptr(stream), _ptr(w_out), float(eps_out), _ptr(w_next),
                                                           _ptr(taps), _ptr(tail), _ptr(step.state_slots), _ptr(x),
                                                           _code(self.act_dtype), T, W, K, float(eps_next), self._stream()))
        return x

    LAYOUTS = {"interleaved": 0, "half": 1}
    DELTA_CHUNK = 64         # tokens a chunk of the delta rule's scan; rows up to this long run whole
    DELTA_CHUNKED_MAX_DIM = 128   # wider heads always run whole (the fold keeps a chunk's d x d matrix in the LDS)

    def qkv_finish(self, sums, q_col, k_col, v_col, num_q_heads, num_kv_heads, dim, vdim, padded_dim, positions, inv_freq,
                   layout, k_cache, v_cache, slot_mapping, q_norm=None, k_norm=None, eps=0.0, q_head_scale=None,
                   norm_per_head=False, col_bias=None, position_temperature=None):
        self._on_device(sums, positions, inv_freq, k_cache, v_cache, slot_mapping, q_norm, k_norm, q_head_scale, col_bias)
        coef, every = 0.0, 0
        if position_temperature is not None:
            coef, every = float(position_temperature[0]), int(position_temperature[1])
            if every < 1 or every != position_temperature[1]:
                raise ValueError(f"qkv_finish: a query temperature every {position_temperature[1]} positions (a whole number >= 1)")
        if col_bias is not None:
            self._f32_vector(col_bias, sums.shape[1], "qkv_finish: col_bias (a number a column of the sums)")
        Hq, Hkv, P, T = num_q_heads, num_kv_heads, padded_dim, sums.shape[0]
        if layout not in self.LAYOUTS:
            raise ValueError(f"qkv_finish: layout {layout!r} (interleaved or half)")
        self._f32_columns(sums, q_col, Hq * dim, "qkv_finish: queries")
        self._f32_columns(sums, k_col, Hkv * dim, "qkv_finish: keys")
        if v_col is not None:
            self._f32_columns(sums, v_col, Hkv * vdim, "qkv_finish: values")
        elif vdim != dim:
            raise ValueError("qkv_finish: values that are the keys have the keys' size")
        pages, hk, page, d = k_cache.shape
        if (hk, d) != (Hkv, P) or tuple(v_cache.shape) != (pages, Hkv, P, page) or P < max(dim, vdim):
            raise ValueError(f"qkv_finish: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} for {Hkv} kv heads of {P}")
        if k_cache.dtype != self.act_dtype or v_cache.dtype != self.act_dtype or not (k_cache.is_contiguous() and v_cache.is_contiguous()):
            raise ValueError("qkv_finish: caches must be contiguous and of the activation dtype")
        nf = 0 if inv_freq is None else inv_freq.numel()
        if nf:
            self._f32_vector(inv_freq, nf, "qkv_finish: inv_freq")
        if 2 * nf > dim:
            raise ValueError(f"qkv_finish: {nf} turned pairs in heads of {dim}")
        for name, t, n in (("q_norm", q_norm, dim if norm_per_head else Hq * dim),
                           ("k_norm", k_norm, dim if norm_per_head else Hkv * dim), ("q_head_scale", q_head_scale, Hq)):
            if t is not None:
                self._f32_vector(t, n, f"qkv_finish: {name}")
        for name, t in (("positions", positions), ("slot_mapping", slot_mapping)):
            if t.dtype != torch.int32 or t.shape[0] != T or not t.is_contiguous():
                raise ValueError(f"qkv_finish: {name} must be contiguous int32 [{T}]")
        # rows 64 bytes apart from a multiple of their length, as the attention kernels like their q rows
        q = torch.empty((T, Hq * P), dtype=self.act_dtype, device=sums.device)
        lib = self.lib("attention_prep")
        library.check(lib, lib.mie_qkv_finish(
            _ptr(sums), sums.stride(0), q_col, k_col, -1 if v_col is None else v_col, _ptr(q_norm), _ptr(k_norm), float(eps),
            int(bool(norm_per_head)), _ptr(inv_freq), nf, self.LAYOUTS[layout], _ptr(q_head_scale), _ptr(positions), _ptr(slot_mapping), _ptr(q),
            _ptr(k_cache), _ptr(v_cache), _code(self.act_dtype), T, Hq, Hkv, dim, vdim, P, page, _ptr(col_bias), coef, every,
            self._stream()))
        return q

    def head_gate_(self, o, gate, gate_col, num_heads, head_dim):
        self._on_device(o, gate)
        T = o.shape[0]
        if tuple(o.shape) != (T, num_heads * head_dim) or not o.is_contiguous():
            raise ValueError(f"head_gate_: o {tuple(o.shape)} for {num_heads} heads of {head_dim}")
        gp = self._f32_columns(gate, gate_col, num_heads, "head_gate_: gate")
        if gate.shape[0] != T:
            raise ValueError("head_gate_: one gate row a token")
        lib = self.lib("attention_prep")
        library.check(lib, lib.mie_head_gate(_ptr(o), _code(o.dtype), gp, gate.stride(0), T, num_heads, head_dim, self._stream()))
        return o

    def delta_rule(self, sums, cols, num_heads, dim, w_decay, decay_bias, decay_scale, removal_bias, norm_weight, eps,
                   state, step):
        self._on_device(sums, w_decay, decay_bias, removal_bias, norm_weight, state)
        H, d, T = num_heads, dim, sums.shape[0]
        n = H * d
        if w_decay.dim() != 2 or w_decay.shape[0] != n:
            raise ValueError(f"delta_rule: decay matrix {tuple(w_decay.shape)} for {H} heads of {d}")
        rank = w_decay.shape[1]
        self._f32_vector(w_decay, n * rank, "delta_rule: decay matrix")
        for name in ("r", "k", "v", "g", "a"):
            self._f32_columns(sums, cols[name], n, f"delta_rule: {name}")
        self._f32_columns(sums, cols["w"], rank, "delta_rule: the decay's inner activations")
        for name, t in (("decay_bias", decay_bias), ("removal_bias", removal_bias), ("norm_weight", norm_weight)):
            self._f32_vector(t, n, f"delta_rule: {name}")
        if state.dtype != torch.float32 or tuple(state.shape[1:]) != (H, d, d) or not state.is_contiguous():
            raise ValueError(f"delta_rule: state {tuple(state.shape)} for {H} heads of {d} x {d}")
        self._check_rows("delta_rule", step, T)
        if int(step.host["state_slots"].max()) >= state.shape[0]:
            raise ValueError("delta_rule: a state slot beyond the state's slots")
        out = torch.empty((T, n), dtype=self.act_dtype, device=sums.device)
        prep = torch.empty((T, 3 * n), dtype=torch.float32, device=sums.device)
        longest = int(getattr(step, "max_row_tokens", 0) or (step.host["row_start"][1:] - step.host["row_start"][:-1]).max())
        chunk, chunks, summaries, starts = 0, 0, None, None
        if longest > self.DELTA_CHUNK and not self.true_fp32 and d <= self.DELTA_CHUNKED_MAX_DIM:
            # rows of many tokens: chunks side by side (whether a step takes this path depends on its longest row alone;
            # the two paths differ by the rounding of the fold over whole chunks, so the 32-bit mode keeps to one)
            chunk, chunks = self.DELTA_CHUNK, -(-longest // self.DELTA_CHUNK)
            scratch = torch.empty((3, step.num_rows * chunks * H, d, d), dtype=torch.float32, device=sums.device)
            summaries, starts = scratch[:2], scratch[2]
        lib = self.lib("delta_rule")
        library.check(lib, lib.mie_delta_rule(
            _ptr(sums), sums.stride(0), cols["r"], cols["k"], cols["v"], cols["g"], cols["a"], cols["w"], _ptr(w_decay), rank,
            _ptr(decay_bias), float(decay_scale), _ptr(removal_bias), _ptr(norm_weight), float(eps), _ptr(state),
            _ptr(step.row_start), _ptr(step.state_slots), _ptr(prep), _ptr(out), _code(out.dtype), T, step.num_rows, H, d,
            chunk, chunks, _ptr(summaries), _ptr(starts), self._stream()))
        return out

    GLA_CHUNK = 64           # tokens a chunk of the gated linear attention's scan; rows up to this long run whole

    def gla(self, sums, cols, num_heads, dim, vdim, w_decay, decay_bias, tau, q_scale, norm_weight, eps, state, step):
        self._on_device(sums, w_decay, decay_bias, norm_weight, state)
        H, d, dv, T = num_heads, dim, vdim, sums.shape[0]
        if w_decay.dim() != 2 or w_decay.shape[0] != H * d:
            raise ValueError(f"gla: decay matrix {tuple(w_decay.shape)} for {H} heads of {d}")
        rank = w_decay.shape[1]
        self._f32_vector(w_decay, H * d * rank, "gla: decay matrix")
        for name, n in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv), ("a", rank)):
            self._f32_columns(sums, cols[name], n, f"gla: {name}")
        if decay_bias is not None:
            self._f32_vector(decay_bias, H * d, "gla: decay_bias")
        self._f32_vector(norm_weight, dv, "gla: norm_weight")
        if state.dtype != torch.float32 or tuple(state.shape[1:]) != (H, d, dv) or not state.is_contiguous():
            raise ValueError(f"gla: state {tuple(state.shape)} for {H} heads of {d} x {dv}")
        if d > 256 or dv > 256:
            raise ValueError(f"gla: heads of {d} x {dv} are beyond the 256 x 256 the kernel takes")
        self._check_rows("gla", step, T)
        if int(step.host["state_slots"].max()) >= state.shape[0]:
            raise ValueError("gla: a state slot beyond the state's slots")
        out = torch.empty((T, H * dv), dtype=self.act_dtype, device=sums.device)
        decay = torch.empty((T, H * d), dtype=torch.float32, device=sums.device)
        longest = int(getattr(step, "max_row_tokens", 0) or (step.host["row_start"][1:] - step.host["row_start"][:-1]).max())
        chunk, chunks, sum_a, sum_b, starts = 0, 0, None, None, None
        if longest > self.GLA_CHUNK and not self.true_fp32:
            # rows of many tokens: chunks side by side (whether a step takes this path depends on its longest row alone;
            # the two paths differ by the rounding of the fold over whole chunks, so the 32-bit mode keeps to one)
            chunk, chunks = self.GLA_CHUNK, -(-longest // self.GLA_CHUNK)
            units = step.num_rows * chunks * H
            sum_a = torch.empty((units, d), dtype=torch.float32, device=sums.device)
            scratch = torch.empty((2, units, d, dv), dtype=torch.float32, device=sums.device)
            sum_b, starts = scratch[0], scratch[1]
        lib = self.lib("gla")
        library.check(lib, lib.mie_gla(
            _ptr(sums), sums.stride(0), cols["q"], cols["k"], cols["v"], cols["g"], cols["a"], _ptr(w_decay), rank,
            _ptr(decay_bias), float(tau), float(q_scale), _ptr(norm_weight), float(eps), _ptr(state), _ptr(step.row_start),
            _ptr(step.state_slots), _ptr(decay), _ptr(out), _code(out.dtype), T, step.num_rows, H, d, dv, chunk, chunks,
            _ptr(sum_a), _ptr(sum_b), _ptr(starts), self._stream()))
        return out

    def normed_sum_add(self, stream, ys, weights, eps, scale):
        self._on_device(stream, *ys, *weights)
        if stream.dtype != torch.float32 or stream.dim() != 2 or not stream.is_contiguous():
            raise ValueError("normed_sum_add: the stream must be contiguous float32 [T, width]")
        T, W = stream.shape
        if not 1 <= len(ys) <= 2 or len(weights) != len(ys):
            raise ValueError("normed_sum_add: one or two branch outputs, a weight each")
        for y, w in zip(ys, weights):
            if y.dtype != torch.float32 or tuple(y.shape) != (T, W) or not y.is_contiguous():
                raise ValueError(f"normed_sum_add: a branch output {tuple(y.shape)} {y.dtype}; contiguous float32 {(T, W)} expected")
            self._f32_vector(w, W, "normed_sum_add: weight")
        lib = self.lib("embed_norm")
        library.check(lib, lib.mie_normed_sum_add(_ptr(stream), _ptr(ys[0]), _ptr(weights[0]), _ptr(ys[1]) if len(ys) > 1 else None,
                                                  _ptr(weights[1]) if len(ys) > 1 else None, T, W, float(eps), float(scale),
                                                  self._stream()))
        return stream

    def linear_rotary_kv_store(self, x, w_qkv, positions, cos, sin, rotary_dim, num_q_heads, num_kv_heads, head_dim,
                               k_cache, v_cache, slot_mapping, for_attention: bool = False):
        Hq, Hkv, D = num_q_heads, num_kv_heads, head_dim
        can_rope = (Hkv > 0 and rotary_dim == D and D % 16 == 0 and k_cache is not None
                    and k_cache.dtype == torch.bfloat16)
        prepared = self._prepared(x, w_qkv, None) if can_rope and getattr(x, "rows", None) is None else None
        eps = x.eps if prepared is not None else 0.0
        if prepared is not None:
            x = prepared["x"]
        elif isinstance(x, Normed):
            x = x.materialize()
        fused = can_rope and self._skinny_ok(x, w_qkv, None)
        if not fused and can_rope and self._mid_ok(x, w_qkv, None) and self.act_dtype == torch.bfloat16:
            return self._mid_rotary_kv_store(x, w_qkv, positions, cos, sin, Hq, Hkv, D, k_cache, v_cache, slot_mapping,
                                             for_attention)
        if (not fused and can_rope and not self.true_fp32 and self.act_dtype == torch.bfloat16
                and x.dtype == torch.bfloat16 and w_qkv.dtype == torch.bfloat16):
            # many rows: library product with float32 sums, then rotary and cache write from those sums (q and k
            # are rounded to bfloat16 once, after the rotation)
            self._on_device(x, w_qkv)
            self._on_device(positions, cos, sin, k_cache, v_cache, slot_mapping)
            M, K = x.shape
            page = self._check_rope_operands("linear_rotary_kv_store", M, K, w_qkv, positions, cos, sin, Hq, Hkv, D,
                                             k_cache, v_cache, slot_mapping)
            if self._lt_ok(x, w_qkv):
                sums = self._lt_product(x, w_qkv, self.LT_F32, torch.empty((M, w_qkv.shape[0]), dtype=torch.float32, device=x.device))
            else:
                sums = torch.mm(x, w_qkv.t(), out_dtype=torch.float32)
            pending = ProjectionSums(self, sums[None], positions, cos, sin, slot_mapping, k_cache, v_cache, Hq, Hkv, D, page)
            return pending if for_attention else pending.finish()
        if not fused:
            return super().linear_rotary_kv_store(x, w_qkv, positions, cos, sin, rotary_dim, Hq, Hkv, D, k_cache,
                                                  v_cache, slot_mapping)
        self._on_device(x, w_qkv, positions, cos, sin, k_cache, v_cache, slot_mapping)
        M, K = x.shape
        page = self._check_rope_operands("linear_rotary_kv_store", M, K, w_qkv, positions, cos, sin, Hq, Hkv, D,
                                         k_cache, v_cache, slot_mapping)
        q = torch.empty((M, Hq * D), dtype=torch.bfloat16, device=x.device)
        lib = self.lib("gemm_bf16")
        library.check(lib, lib.mie_skinny_qkv_rope(
            _ptr(x), x.stride(0), _ptr(w_qkv), w_qkv.stride(0), _ptr(q), q.stride(0), _ptr(positions), _ptr(cos),
            _ptr(sin), _ptr(slot_mapping), _ptr(k_cache), _ptr(v_cache), M, Hq, Hkv, D, page, K,
            _ptr(prepared["ss"]) if prepared else None, prepared["tiles"] if prepared else 0, float(eps),
            self._stream()))
        return q

    def _check_rope_operands(self, what, M, K, w_qkv, positions, cos, sin, Hq, Hkv, D, k_cache, v_cache, slot_mapping):
        if tuple(w_qkv.shape) != ((Hq + 2 * Hkv) * D, K):
            raise ValueError(f"{what}: w {tuple(w_qkv.shape)} for {Hq}+2x{Hkv} heads of {D}, K {K}")
        page = k_cache.shape[2]
        for name, t, want in (("k_cache", k_cache, (k_cache.shape[0], Hkv, page, D)),
                              ("v_cache", v_cache, (k_cache.shape[0], Hkv, D, page))):
            if tuple(t.shape) != want or t.dtype != torch.bfloat16 or not t.is_contiguous():
                raise ValueError(f"{what}: {name} {tuple(t.shape)} {t.dtype}, expected {want}")
        for name, t in (("cos", cos), ("sin", sin)):
            if t.dtype != torch.float32 or t.dim() != 2 or t.shape[1] != D // 2 or not t.is_contiguous():
                raise ValueError(f"{what}: {name} must be contiguous float32 [positions, {D // 2}]")
        for name, t in (("positions", positions), ("slot_mapping", slot_mapping)):
            if t.dtype != torch.int32 or t.shape[0] != M or not t.is_contiguous():
                raise ValueError(f"{what}: {name} must be contiguous int32 [{M}]")
        return page

    def _mid_rotary_kv_store(self, x, w_qkv, positions, cos, sin, Hq, Hkv, D, k_cache, v_cache, slot_mapping,
                             for_attention=False):
        """The q/k/v projection of 17 to 128 rows: split product, then one kernel that adds the partial
        results, rotates q and k and writes k and v to the cache.  Returns q [M, Hq * D] (for_attention: the
        partial results, for paged_attention to finish)."""
        self._on_device(x, w_qkv, positions, cos, sin, k_cache, v_cache, slot_mapping)
        M, K = x.shape
        page = self._check_rope_operands("linear_rotary_kv_store", M, K, w_qkv, positions, cos, sin, Hq, Hkv, D,
                                         k_cache, v_cache, slot_mapping)
        pending = ProjectionSums(self, self._mid_partials(x, w_qkv), positions, cos, sin, slot_mapping, k_cache, v_cache,
                                 Hq, Hkv, D, page)
        return pending if for_attention else pending.finish()

    def rotary_kv_store(self, qkv, positions, cos, sin, rotary_dim, num_q_heads, num_kv_heads, head_dim,
                        k_cache, v_cache, slot_mapping):
        self._on_device(qkv, positions, cos, sin, k_cache, v_cache, slot_mapping)
        _rows_ok(qkv, "rotary_kv_store: qkv")
        T = qkv.shape[0]
        Hq, Hkv, D = num_q_heads, num_kv_heads, head_dim
        if qkv.shape[1] != (Hq + 2 * Hkv) * D:
            raise ValueError(f"rotary_kv_store: qkv has {qkv.shape[1]} columns, expected {(Hq + 2 * Hkv) * D}")
        page = 0
        if rotary_dim:
            half = rotary_dim // 2
            for name, t in (("cos", cos), ("sin", sin)):
                if t is None or t.dtype != torch.float32 or t.dim() != 2 or t.shape[1] != half or not t.is_contiguous():
                    raise ValueError(f"rotary_kv_store: {name} must be contiguous float32 [positions, {half}]")
            if positions.dtype != torch.int32 or positions.shape[0] != T or not positions.is_contiguous():
                raise ValueError("rotary_kv_store: positions must be contiguous int32 [T]")
        if Hkv:
            page = k_cache.shape[2]
            for name, t, want in (("k_cache", k_cache, (k_cache.shape[0], Hkv, page, D)),
                                  ("v_cache", v_cache, (k_cache.shape[0], Hkv, D, page))):
                if tuple(t.shape) != want or t.dtype != qkv.dtype or not t.is_contiguous():
                    raise ValueError(f"rotary_kv_store: {name} {tuple(t.shape)} {t.dtype}, expected {want} {qkv.dtype}")
            if slot_mapping.dtype != torch.int32 or slot_mapping.shape[0] != T or not slot_mapping.is_contiguous():
                raise ValueError("rotary_kv_store: slot_mapping must be contiguous int32 [T]")
        lib = self.lib("rope_kv")
        library.check(lib, lib.mie_rotary_kv_store(
            _ptr(qkv), _code(qkv.dtype), qkv.stride(0), _ptr(positions), _ptr(cos), _ptr(sin), rotary_dim, Hq, Hkv, D,
            _ptr(k_cache), _ptr(v_cache), _ptr(slot_mapping), page, T, self._stream()))

    def _check_attention(self, qkv, Hq, Hkv, D, k_cache, v_cache, group, step):
        _rows_ok(qkv, "paged_attention: qkv")
        if qkv.shape[1] < Hq * D:
            raise ValueError(f"paged_attention: qkv has {qkv.shape[1]} columns, fewer than {Hq * D}")
        return self._check_attention_cache(qkv.shape[0], qkv.dtype, Hkv, D, k_cache, v_cache, group, step)

    def _check_attention_cache(self, T, dtype, Hkv, D, k_cache, v_cache, group, step):
        pages, hk, page, d = k_cache.shape
        if (hk, d) != (Hkv, D) or tuple(v_cache.shape) != (pages, Hkv, D, page):
            raise ValueError(f"paged_attention: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} for "
                             f"{Hkv} kv heads of {D}")
        if k_cache.dtype != dtype or v_cache.dtype != dtype or not (k_cache.is_contiguous() and v_cache.is_contiguous()):
            raise ValueError("paged_attention: caches must be contiguous and of the activation dtype")
        bt = group.block_tables
        if bt.dtype != torch.int32 or bt.dim() != 2 or bt.stride(1) != 1 or bt.stride(0) != bt.shape[1]:
            raise ValueError("paged_attention: block tables must be contiguous int32 [rows, max_blocks]")
        if bt.shape[0] < step.num_rows:
            raise ValueError(f"paged_attention: {bt.shape[0]} block-table rows for {step.num_rows} rows")
        for name, t in (("token_row", step.token_row), ("positions", step.positions)):
            if t.dtype != torch.int32 or t.shape[0] != T or not t.is_contiguous():
                raise ValueError(f"paged_attention: {name} must be contiguous int32 [T]")
        if step.max_context > bt.shape[1] * page:
            raise ValueError(f"paged_attention: context {step.max_context} exceeds the block tables "
                             f"({bt.shape[1]} pages of {page})")
        return T, page, bt

    # workgroups the decode attention kernel should at least be spread over (two per compute unit)
    DECODE_TARGET_WORKGROUPS = 512
    DECODE_WHOLE_WORKGROUPS = 256

    def decode_splits(self, rows: int, Hq: int, Hkv: int, context_bound: int, window, block_keys: int,
                      head_dim: int = 64):
        """(keys per split, number of splits) for single-token rows: split the context only as far
        as the rows and heads alone do not fill the GPU (inference_engine/kernels/decode_attention.py:117-125
        follows the same idea), in whole blocks of the kernel.

        Not split at all (no partial results, no merge kernel): always when rows and heads give every compute unit
        a workgroup; and with fewer workgroups where the contexts are short, because a workgroup then reads its
        whole context in less time than the merge kernel takes.  Measured at head size 64 (keys of 256 bytes a kv
        head): the unsplit kernel wins from 64 workgroups on at 512 keys, from 96 at 1,024, from 144 at 2,048:
        about 32 + keys / 18.  At head size 128 (8 and 32 kv heads, 1 to 16 rows, 512 to 8,192 keys) whole decode
        steps with half the target, or unsplit at 512 keys, are within 3 % of this rule's, faster or slower by the
        case: the rule holds there."""
        if window:
            context_bound = min(context_bound, window + 32)
        base = rows * Hkv * -(-(Hq // Hkv) // 16)
        most = max(1, -(-context_bound // block_keys))
        whole_from = min(self.DECODE_WHOLE_WORKGROUPS, 32 + context_bound * head_dim // (64 * 18))
        target = self.DECODE_TARGET_WORKGROUPS if base < whole_from else base
        splits = max(1, min(-(-target // base), most))
        partition = -(-(-(-context_bound // splits)) // block_keys) * block_keys
        return partition, max(1, -(-context_bound // partition))

    def _decode_attention_from_sums(self, pending, Hq, Hkv, D, k_cache, v_cache, group, step, scale, window, forced):
        """A step of single-token rows whose rows and kv heads alone fill the GPU: the decode kernel finishes the
        projection itself (no kernel between product and attention).  None: not such a step."""
        T = pending.part.shape[1]
        # The kernel rotates with the step's positions, takes the row's own key from its LDS and writes it to
        # pending.slots: that is the same result as finish() only if the projection was made for this very step
        # and this page group (same position and slot arrays, same caches).  Anything else takes finish().
        if (forced or step.num_decode_rows != T or step.num_tokens != T or Hq // Hkv > 16
                or pending.k_cache is not k_cache or pending.v_cache is not v_cache
                or pending.positions.data_ptr() != step.positions.data_ptr()
                or pending.slots.data_ptr() != group.slot_mapping.data_ptr()
                or (pending.Hq, pending.Hkv, pending.D) != (Hq, Hkv, D)):
            return None
        lib = self.lib("attention_bf16", (f"-DHEAD_DIM={D}",))
        block_keys = lib.mie_decode_block_keys()
        partition, splits = self.decode_splits(T, Hq, Hkv, step.max_context, window, block_keys, D)
        if splits != 1:
            return None
        bound = min(step.max_context, window + 32) if window else step.max_context
        if partition < bound:
            raise AssertionError(f"decode attention from sums: one split of {partition} keys for contexts up to {bound}")
        part = pending.part
        self._on_device(k_cache, v_cache)
        _, _, bt = self._check_attention_cache(T, torch.bfloat16, Hkv, D, k_cache, v_cache, group, step)
        out = torch.empty((T, Hq * D), dtype=torch.bfloat16, device=part.device)
        library.check(lib, lib.mie_decode_attention_from_sums(
            _ptr(part), part.shape[0], part.stride(0), part.stride(1), _ptr(pending.cos), _ptr(pending.sin),
            _ptr(pending.slots), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(bt), bt.shape[1], _ptr(step.positions), T,
            Hq, Hkv, D, pending.page, float(scale), int(window or 0), partition, self._stream()))
        return out

    def paged_attention(self, qkv, num_q_heads, num_kv_heads, head_dim, k_cache, v_cache, group, step, scale,
                        window, sink=None, weights="softmax", softcap=None, chunk=None, head_bias=None,
                        distance_bias=None, force_generic: bool = False, num_splits: int | None = None):
        Hq, Hkv, D = num_q_heads, num_kv_heads, head_dim
        dist_n = 0
        if distance_bias is not None:
            self._on_device(distance_bias)
            if distance_bias.dim() != 2 or distance_bias.shape[0] != Hq or distance_bias.shape[1] < 1:
                raise ValueError(f"paged_attention: distance_bias {tuple(distance_bias.shape)} for {Hq} query heads")
            dist_n = distance_bias.shape[1]
            self._f32_vector(distance_bias, Hq * dist_n, "paged_attention: distance_bias")
        has_sink, sink = int(sink is not None), float(sink or 0.0)
        if weights not in ("softmax", "sigmoid"):
            raise ValueError(f"paged_attention: weights {weights!r} (softmax or sigmoid)")
        sigmoid = weights == "sigmoid"
        if sigmoid and has_sink:
            raise ValueError("paged_attention: a sink belongs to a softmax")
        if (chunk is not None and chunk < 1) or (softcap is not None and not softcap > 0):
            raise ValueError(f"paged_attention: chunk {chunk}, score cap {softcap}")
        if head_bias is not None:
            if not sigmoid:
                raise ValueError("paged_attention: a bias per head goes with sigmoid weights")
            self._on_device(head_bias)
            self._f32_vector(head_bias, Hq, "paged_attention: head_bias")
        scored = sigmoid or softcap is not None or chunk is not None or distance_bias is not None
        biased = distance_bias is not None and not sigmoid and softcap is None and chunk is None and not has_sink
        if scored and not sigmoid and not biased:
            force_generic = True            # a capped or chunked softmax: the 32-bit kernel computes it
        table2 = None
        if biased and qkv.dtype == torch.bfloat16 and not force_generic and D <= 256:
            # the matrix-core kernels work in units of log2 e: the table in those units, made once a table
            key = distance_bias.data_ptr()
            held = self._log2_tables.get(key)
            if held is None or held[0] is not distance_bias:
                held = self._log2_tables[key] = (distance_bias, (distance_bias * 1.4426950408889634).contiguous())
            table2 = held[1]
        if isinstance(qkv, ProjectionSums):
            out = self._decode_attention_from_sums(qkv, Hq, Hkv, D, k_cache, v_cache, group, step, scale, window,
                                                   force_generic or num_splits is not None or bool(has_sink))
            if out is not None:
                return out
            qkv = qkv.finish()
        self._on_device(qkv, k_cache, v_cache)
        T, page, bt = self._check_attention(qkv, Hq, Hkv, D, k_cache, v_cache, group, step)
        out = torch.empty((T, Hq * D), dtype=qkv.dtype, device=qkv.device)
        done = 0
        if D > 256:
            force_generic = True            # beyond the matrix-core kernels' head sizes: the 32-bit kernel takes up to 1,024
        if qkv.dtype == torch.bfloat16 and not force_generic and step.num_decode_rows > 0:
            done = step.num_decode_rows        # single-token rows lead the batch: token t is row t
            lib = self.lib("attention_bf16", (f"-DHEAD_DIM={D}",))
            block_keys = lib.mie_decode_block_keys()
            # a row sees at most a chunk's keys: the splits are planned as for a window of that many
            reach = min(window or chunk, chunk or window) if (window or chunk) else None
            partition, splits = self.decode_splits(done, Hq, Hkv, step.max_context, reach, block_keys, D)
            if num_splits is not None:
                bound = min(step.max_context, reach + 32) if reach else step.max_context
                partition = -(-(-(-bound // num_splits)) // block_keys) * block_keys
                splits = max(1, -(-bound // partition))
            o_part = lse_part = None
            if splits > 1:
                o_part = torch.empty((done, Hq, splits, D), dtype=torch.float32, device=qkv.device)
                lse_part = torch.empty((done, Hq, splits), dtype=torch.float32, device=qkv.device)
            args = (_ptr(qkv), qkv.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(o_part), _ptr(lse_part),
                    _ptr(bt), bt.shape[1], _ptr(step.positions), done, Hq, Hkv, D, page, float(scale), int(window or 0),
                    partition, splits)
            if sigmoid:
                library.check(lib, lib.mie_decode_attention_sigmoid(*args, int(chunk or 0), float(softcap or 0.0),
                                                                    _ptr(head_bias), self._stream()))
            elif table2 is not None:
                library.check(lib, lib.mie_decode_attention_biased(*args, _ptr(table2), dist_n, self._stream()))
            elif has_sink:
                library.check(lib, lib.mie_decode_attention_sink(*args, sink, self._stream()))
            else:
                library.check(lib, lib.mie_decode_attention(*args, self._stream()))
        end = T                                # tokens [done, end) are left to the 32-bit kernel
        if step.num_decode_rows < T and qkv.dtype == torch.bfloat16 and not force_generic:
            # rows of several tokens: matrix-core kernel over their own and earlier portions' keys
            for name, t, n in (("row_start", step.row_start, step.num_rows + 1),
                               ("row_position", step.row_position, step.num_rows)):
                if t is None or t.dtype != torch.int32 or t.shape[0] < n or not t.is_contiguous():
                    raise ValueError(f"paged_attention: {name} must be contiguous int32 [{n}]")
            lib = self.lib("prefill_attention_bf16", (f"-DHEAD_DIM={D}",))
            args = (_ptr(qkv), qkv.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(bt), bt.shape[1],
                    _ptr(step.row_start), _ptr(step.row_position), step.num_decode_rows,
                    step.num_rows - step.num_decode_rows, step.max_row_tokens, Hq, Hkv, D, page, float(scale),
                    int(window or 0))
            if sigmoid:
                library.check(lib, lib.mie_prefill_attention_sigmoid(*args, int(chunk or 0), float(softcap or 0.0),
                                                                     _ptr(head_bias), self._stream()))
            elif table2 is not None:
                library.check(lib, lib.mie_prefill_attention_biased(*args, _ptr(table2), dist_n, self._stream()))
            elif has_sink:
                library.check(lib, lib.mie_prefill_attention_sink(*args, sink, self._stream()))
            else:
                library.check(lib, lib.mie_prefill_attention(*args, self._stream()))
            end = step.num_decode_rows
        if done < end:
            lib = self.lib("attention")
            esz = qkv.element_size()
            args = (c_void_p(qkv.data_ptr() + done * qkv.stride(0) * esz), qkv.stride(0), _ptr(k_cache), _ptr(v_cache),
                    c_void_p(out.data_ptr() + done * Hq * D * esz), _code(qkv.dtype), _ptr(bt), bt.shape[1],
                    c_void_p(step.token_row.data_ptr() + done * 4), c_void_p(step.positions.data_ptr() + done * 4),
                    end - done, Hq, Hkv, D, page, float(scale), int(window or 0), has_sink, sink)
            if scored:
                library.check(lib, lib.mie_paged_attention_scored(*args, int(chunk or 0), float(softcap or 0.0), int(sigmoid),
                                                                  _ptr(head_bias), _ptr(distance_bias), dist_n, self._stream()))
            else:
                library.check(lib, lib.mie_paged_attention(*args, self._stream()))
        return out

    def sample(self, logits, temperatures, seeds, counters, out=None):
        self._on_device(logits, temperatures, seeds, counters, out)
        if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
            raise ValueError("sample: logits must be float32 [rows, vocab] with unit inner stride")
        R, V = logits.shape
        if (temperatures.dtype, seeds.dtype, counters.dtype) != (torch.float32, torch.int64, torch.int32):
            raise ValueError("sample: temperatures float32, seeds int64, counters int32")
        if not (temperatures.shape[0] == seeds.shape[0] == counters.shape[0] == R):
            raise ValueError("sample: one temperature, seed and counter per row")
        if out is None:
            out = torch.empty(R, dtype=torch.int32, device=logits.device)
        elif out.dtype != torch.int32 or tuple(out.shape) != (R,) or not out.is_contiguous():
            raise ValueError(f"sample: out must be contiguous int32 [{R}]")
        lib = self.lib("sampling")
        library.check(lib, lib.mie_sample(_ptr(logits), logits.stride(0), _ptr(temperatures), _ptr(seeds),
                                          _ptr(counters), _ptr(out), R, V, self._stream()))
        return out
