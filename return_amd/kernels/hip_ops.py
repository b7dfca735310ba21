"""The kernel set of the engine: thin, checked bindings of the HIP library.

Every method checks on the host that shapes, dtypes and contiguity are what the
kernel and its grid assume, and raises before anything is launched otherwise.
There is no other implementation behind these names: if the library cannot be
built or loaded, constructing HipOps raises.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..parts.runtime import ScaledRows, Slabs
from . import build as _build

_F32, _BF16 = 0, 1
_c_int, _c_ll, _c_float, _c_ptr = ctypes.c_int, ctypes.c_longlong, ctypes.c_float, ctypes.c_void_p


class KernelError(RuntimeError):
    pass


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _F32
    if dtype == torch.bfloat16:
        return _BF16
    raise KernelError(f"kernels take float32 or bfloat16 tensors, got {dtype}")


_LIB = None


def load_library():
    """The HIP library, built first if it is not there. Raises if that is impossible."""
    global _LIB
    if _LIB is None:
        path = _build.ensure_built()
        try:
            _LIB = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"cannot load the HIP library {path}: {e}") from e
        _declare(_LIB)
    return _LIB


def _declare(lib):
    P, I, L, F = _c_ptr, _c_int, _c_ll, _c_float
    sigs = {
        "ra_embed": [P, P, P, I, I, I, I, P],
        "ra_add_rmsnorm": [P, P, P, F, P, P, I, I, I, P],
        "ra_add_slabs_rmsnorm": [P, P, I, L, P, F, P, P, I, I, I, P],
        "ra_residual_add": [P, P, L, I, P],
        "ra_head_rmsnorm": [P, P, F, L, I, I, P],
        "ra_rope": [P, P, P, P, I, I, I, I, I, P],
        "ra_split_heads": [P, P, P, P, I, I, I, I, P],
        "ra_kv_write": [P, P, P, P, P, I, I, I, I, L, I, P],
        "ra_qkv_prepare": [P, I, I, I, I, P, P, F, P, P, P, I, P, P, P, P, I, L, I, P],
        "ra_silu_mul": [P, P, I, I, I, P],
        "ra_gemm_nt": [P, P, P, I, I, I, I, I, P],
        "ra_gemm_skinny_bf16": [P, P, P, I, I, I, I, I, P],
        "ra_gemm_skinny_gated_bf16": [P, P, P, I, I, I, P],
        "ra_gemm_mfma_bf16": [P, P, P, I, I, I, I, P],
        "ra_gemm_resident_bf16": [P, P, P, I, I, I, I, I, I, P],
        "ra_gemm_resident_fits": [I, I, I],
        "ra_gemm_sweep_bf16": [P, P, P, I, I, I, I, I, I, P],
        "ra_gemm_sweep_fits": [I, I],
        "ra_gemm_sweep_workgroups": [I, I],
        "ra_gemm_sweep_norm_bf16": [P, P, P, I, I, I, I, I, I, P, I, I, F, P, P, P, P],
        "ra_attention_plain": [P, P, P, P, P, P, P, P, P, P, I, I, I, I, I, I, F, I, I, P],
        "ra_attention_decode_bf16": [P, P, P, P, P, P, P, P, P, P, P, P, I, I, I, I, I, F, I, I, I, I, P],
        "ra_attention_decode_fused_bf16": [P, P, P, P, P, P, P, P, P, P, P, P, I, I, I, I, I, F, I, I, I, P, P, F, P, P, I, P],
        "ra_attention_decode_static_bf16": [P, P, P, P, P, P, P, P, P, P, I, I, I, I, I, F, I, I, I, I, P],
        "ra_attention_decode_merge_waves": [I],
        "ra_attention_prefill_bf16": [P, P, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, F, I, P],
        "ra_attention_prefill_tile_rows": [I],
        "ra_sample": [P, I, I, P, P, P, P, P, P],
        "ra_sample_traced": [P, I, I, P, P, P, P, P, P, P],
        "ra_stream_read": [P, L, P, I, P],
    }
    for name, args in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = _c_int


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


# What tune_products has measured in this process: (row step, N, K, gated, result dtype) -> the way that
# beat the rule's, or None where the rule stands. Every kernel set that tunes gets the same answers.
_PRODUCTS_MEASURED = {}
_PRODUCT_TIMES = {}        # the same keys -> {way: seconds}, as measured
_NORM_PAIRS_MEASURED = {}  # (row step, shape of the product before a norm, of the one after, gated) -> the norm inside them is faster


class HipOps:
    def __init__(self, device="cuda:0"):
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise KernelError(f"the HIP kernels run on a GPU, not on {self.device}")
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible to this process")
        self.lib = load_library()
        # float32 products must be true 32-bit wherever a library routine is used
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        self.decode_split_tokens = 0         # keys per split of the decode attention; 0: by batch size
        # a request's splits as one workgroup that merges them itself: one such workgroup fills a CU
        # (LDS), so it pays when the (request, kv head) pairs come to whole rounds over the CUs
        self.cu_count = torch.cuda.get_device_properties(self.device).multi_processor_count
        self.decode_merge_round = self.cu_count
        self.decode_merge_waves = 0          # waves of such a workgroup; 0: by the number of pairs and the context
        self.prefill_key_split = 0           # groups of waves that share a q tile's keys (1 or 2); 0: by the number of tiles
        self.prefill_small_tiles = True      # q tiles of 64 rows instead of 128 while those would not fill the chip
        self.overlap_attention = True        # mixed steps: the decode and the prefill attention side by side on two streams
        self._side_stream = None
        self.skinny_max_grid = 0             # 0: one workgroup per 16 weight rows
        self.gated_skinny_rows = 8           # up to this many rows gate-up and SiLU-mul are one kernel
        self.own_gemm = False                # True: bf16 products of many rows use the hand-written MFMA kernel
        self.defer_norms = True              # finish RMSNorms inside the products around them where the sweep takes both
        try:                                 # whether the library multiplies bf16 operands into fp32 results
            a = torch.ones(1, 8, dtype=torch.bfloat16, device=self.device)
            self._library_fp32_out = torch.mm(a, a.t(), out_dtype=torch.float32).dtype == torch.float32
        except (TypeError, RuntimeError):
            self._library_fp32_out = False
        try:                                 # and the same for a batch of products
            a = torch.ones(2, 1, 8, dtype=torch.bfloat16, device=self.device)
            self._library_bmm_fp32 = torch.bmm(a, a.transpose(1, 2), out_dtype=torch.float32).dtype == torch.float32
        except (TypeError, RuntimeError):
            self._library_bmm_fp32 = False
        # whether the library's float32 product is a true 32-bit one (against a 64-bit product; operands
        # rounded to a shorter mantissa would be off by 1e-3)
        g = torch.Generator(device="cpu").manual_seed(0)
        a = torch.randn(32, 512, generator=g).to(self.device)
        b = torch.randn(48, 512, generator=g).to(self.device)
        want = a.double() @ b.double().t()
        self._library_fp32_exact = bool(((torch.matmul(a, b.t()).double() - want).abs().max()
                                         <= 2e-5 * want.abs().max()).item())
        self.product_plan = {}               # (row step, N, K, gated, result dtype) -> way, where measured faster than the rule
        self._measured = _PRODUCTS_MEASURED
        self._times = _PRODUCT_TIMES
        self._defer = {}                     # as _NORM_PAIRS_MEASURED, for the pairs this kernel set has been shown

    def use_skinny(self, M, N, K, out_dtype):
        """Whether the hand-written skinny product beats the library for x [M, K] @ W[N, K]^T
        (measured on MI355X: it wins for one to four rows, up to 16 rows on small weights and up
        to 32 rows on the smallest)."""
        if K % 8 or M > 64:
            return False
        if out_dtype == torch.float32:
            return M <= 16                   # more rows: the library, or the tiled MFMA product
        return M <= 4 or (M <= 16 and N * K <= (32 << 20)) or (M <= 32 and N * K <= (16 << 20))

    def use_sweep(self, M, N, K, gated):
        """Whether the product that reads W as one sweep through memory (one workgroup per CU, column
        c with workgroup c % CUs) is the rule's choice for x [M, K] and N result columns. Measured on
        MI355X at 1 to 16 rows: 12 against 15 µs (q/k/v of the 8B shape), 10 against 11 (o), 36 against
        41 (gate-up), 100 against 118 (gate-up of the 32B shape, K = 5,120) for the x-resident and
        skinny products; on the output head's 152 thousand rows the x-resident product is ahead (two
        workgroups per CU hide each other's tile ends), and on few rows of many columns (down: one tile
        a workgroup, K = 12,288) the library."""
        if not self.lib.ra_gemm_sweep_fits(M, K):
            return False
        if M > 16 and not gated:             # 17 to 32 rows: 41 to 44 µs against the library's 49 and the SiLU-mul's 5
            return False                     # for gate-up, but q/k/v 17 to 19 against 15, o 14 to 16 against 13
        rows = N * (2 if gated else 1)
        least = 8 if K <= 4096 or M <= 2 else 32         # rows a workgroup, at least (down at 1 and 2 rows: 20 against 21 to 23 µs)
        return least * self.cu_count <= rows <= 256 * self.cu_count

    def use_resident(self, M, N, K, gated):
        """Whether the product with x resident in LDS beats the skinny product for x [M, K] and
        N result columns (measured on MI355X): when there are tiles of 16 columns enough for
        every workgroup (two per CU); few tiles are the skinny product's."""
        if not self.lib.ra_gemm_resident_fits(M, K, 1 if gated else 0):
            return False
        tiles = -(-N // 16)
        if 1 <= M <= 8:
            return tiles >= 384
        return M > 8 and tiles >= 2048

    # ------------------------------------------------------------------ helpers
    def _stream(self):
        return torch.cuda.current_stream(self.device).cuda_stream

    def _check(self, status: int, name: str):
        if status != 0:
            why = {1: "arguments outside what the kernel takes", 2: "launch failed",
                   3: "more partial results than the library's own buffer holds",
                   4: "the library's own buffer was not found on this device"}.get(status, "?")
            raise KernelError(f"{name}: {why} (status {status})")

    def _want(self, t, name, dtype=None, dims=None):
        if t.device != self.device:
            raise KernelError(f"{name} is on {t.device}, kernels run on {self.device}")
        if not t.is_contiguous():
            raise KernelError(f"{name} must be contiguous")
        if dtype is not None and t.dtype != dtype:
            raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
        if dims is not None and t.dim() != dims:
            raise KernelError(f"{name} must have {dims} dimensions, got shape {tuple(t.shape)}")

    # ------------------------------------------------------------------ rows
    def embed(self, table, ids, out):
        self._want(table, "embedding table", dims=2)
        self._want(ids, "token ids", torch.int32, 1)
        self._want(out, "embedding output", torch.float32, 2)
        T, H = out.shape
        if ids.shape[0] != T or table.shape[1] != H:
            raise KernelError(f"embed: ids {tuple(ids.shape)}, table {tuple(table.shape)}, out {tuple(out.shape)}")
        self._check(self.lib.ra_embed(_ptr(table), _ptr(ids), _ptr(out), T, H, table.shape[0],
                                      _code(table.dtype), self._stream()), "embed")

    def add_rmsnorm(self, h, delta, weight, eps, out, rows=None):
        self._want(h, "residual stream", torch.float32, 2)
        self._want(weight, "norm weight", torch.float32, 1)
        self._want(out, "norm output", dims=2)
        R, H = h.shape
        if weight.shape[0] != H or out.shape[1] != H:
            raise KernelError(f"add_rmsnorm: h {tuple(h.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
        if isinstance(delta, Slabs):
            self._want(delta.tensor, "shares of the product", torch.float32, 3)
            if tuple(delta.tensor.shape[1:]) != (R, H):
                raise KernelError(f"add_rmsnorm: shares {tuple(delta.tensor.shape)} do not match h {tuple(h.shape)}")
            if rows is not None:
                self._want(rows, "row list", torch.int32, 1)
            M = R if rows is None else rows.shape[0]
            if out.shape[0] != M:
                raise KernelError(f"add_rmsnorm: out has {out.shape[0]} rows, {M} wanted")
            self._check(self.lib.ra_add_slabs_rmsnorm(_ptr(h), _ptr(delta.tensor), delta.tensor.shape[0], R, _ptr(weight),
                                                      float(eps), _ptr(out), _ptr(rows), M, H, _code(out.dtype),
                                                      self._stream()), "add_slabs_rmsnorm")
            return
        if delta is not None:
            self._want(delta, "delta", out.dtype, 2)
            if tuple(delta.shape) != (R, H):
                raise KernelError(f"add_rmsnorm: delta {tuple(delta.shape)} does not match h {tuple(h.shape)}")
        if rows is not None:
            self._want(rows, "row list", torch.int32, 1)
            M = rows.shape[0]
        else:
            M = R
        if out.shape[0] != M:
            raise KernelError(f"add_rmsnorm: out has {out.shape[0]} rows, {M} wanted")
        self._check(self.lib.ra_add_rmsnorm(_ptr(h), _ptr(delta), _ptr(weight), float(eps), _ptr(out),
                                            _ptr(rows), M, H, _code(out.dtype), self._stream()),
                    "add_rmsnorm")

    def residual_add(self, h, delta):
        self._want(h, "residual stream", torch.float32)
        self._want(delta, "delta")
        if h.shape != delta.shape:
            raise KernelError(f"residual_add: {tuple(h.shape)} += {tuple(delta.shape)}")
        self._check(self.lib.ra_residual_add(_ptr(h), _ptr(delta), h.numel(), _code(delta.dtype),
                                             self._stream()), "residual_add")

    def head_rmsnorm(self, x, weight, eps):
        self._want(x, "heads", dims=3)
        self._want(weight, "head norm weight", torch.float32, 1)
        if weight.shape[0] != x.shape[2]:
            raise KernelError(f"head_rmsnorm: weight {tuple(weight.shape)} for heads {tuple(x.shape)}")
        self._check(self.lib.ra_head_rmsnorm(_ptr(x), _ptr(weight), float(eps), x.shape[0] * x.shape[1],
                                             x.shape[2], _code(x.dtype), self._stream()), "head_rmsnorm")

    def rope(self, x, positions, cos, sin, rotary_dim):
        self._want(x, "heads", dims=3)
        self._want(positions, "positions", torch.int32, 1)
        self._want(cos, "cos table", torch.float32, 2)
        self._want(sin, "sin table", torch.float32, 2)
        T, heads, D = x.shape
        R = int(rotary_dim)
        if positions.shape[0] != T or R % 2 or R > D or cos.shape[1] != R // 2 or sin.shape != cos.shape:
            raise KernelError(f"rope: x {tuple(x.shape)}, rotary_dim {R}, tables {tuple(cos.shape)}")
        self._check(self.lib.ra_rope(_ptr(x), _ptr(positions), _ptr(cos), _ptr(sin), T, heads, D, R,
                                     _code(x.dtype), self._stream()), "rope")

    def split_heads(self, qkv, n_q, n_kv, D, q, k, v):
        self._want(qkv, "qkv", dims=2)
        T = qkv.shape[0]
        for t, name, heads in ((q, "q", n_q), (k, "k", n_kv), (v, "v", n_kv)):
            self._want(t, name, qkv.dtype, 3)
            if tuple(t.shape) != (T, heads, D):
                raise KernelError(f"split_heads: {name} is {tuple(t.shape)}, wanted {(T, heads, D)}")
        if qkv.shape[1] != (n_q + 2 * n_kv) * D:
            raise KernelError(f"split_heads: qkv width {qkv.shape[1]} is not {(n_q + 2 * n_kv) * D}")
        self._check(self.lib.ra_split_heads(_ptr(qkv), _ptr(q), _ptr(k), _ptr(v), T, n_q * D, n_kv * D,
                                            _code(qkv.dtype), self._stream()), "split_heads")

    def _pool_rows(self, k_pool, v_pool, n_kv, D, dtype):
        """Checks the pools of one cache layer, [pages, kv heads, rows in a page, D], and returns the
        number of token rows they hold (pages x page size)."""
        for t, name in ((k_pool, "k pool"), (v_pool, "v pool")):
            self._want(t, name, dtype, 4)
            if t.shape[1] != n_kv or t.shape[3] != D:
                raise KernelError(f"{name} {tuple(t.shape)} does not hold {n_kv} heads of {D}")
        if k_pool.shape != v_pool.shape:
            raise KernelError("k pool and v pool differ in shape")
        if k_pool.shape[0] * k_pool.shape[1] * k_pool.shape[2] >= 2 ** 31:
            raise KernelError(f"k pool {tuple(k_pool.shape)}: the kernels count head rows in 32 bits")
        return k_pool.shape[0] * k_pool.shape[2]

    def kv_write(self, k, v, k_pool, v_pool, slot_mapping):
        self._want(k, "k", dims=3)
        self._want(v, "v", k.dtype, 3)
        self._want(slot_mapping, "slot mapping", torch.int32, 1)
        T, n_kv, D = k.shape
        rows = self._pool_rows(k_pool, v_pool, n_kv, D, k.dtype)
        if v.shape != k.shape or slot_mapping.shape[0] != T:
            raise KernelError(f"kv_write: k {tuple(k.shape)}, v {tuple(v.shape)}, slots {tuple(slot_mapping.shape)}")
        self._check(self.lib.ra_kv_write(_ptr(k), _ptr(v), _ptr(k_pool), _ptr(v_pool), _ptr(slot_mapping),
                                         T, n_kv, D, k_pool.shape[2], rows, _code(k.dtype), self._stream()), "kv_write")

    def qkv_prepare(self, qkv, n_q, n_kv, D, w_q, w_k, eps, positions, cos, sin, rotary_dim, q_out,
                    k_pool, v_pool, slot_mapping):
        self._want(qkv, "qkv", dims=2)
        self._want(q_out, "q", qkv.dtype, 3)
        self._want(positions, "positions", torch.int32, 1)
        self._want(slot_mapping, "slot mapping", torch.int32, 1)
        T = qkv.shape[0]
        R = int(rotary_dim)
        if qkv.shape[1] != (n_q + 2 * n_kv) * D or tuple(q_out.shape) != (T, n_q, D):
            raise KernelError(f"qkv_prepare: qkv {tuple(qkv.shape)}, q {tuple(q_out.shape)}")
        if positions.shape[0] != T or slot_mapping.shape[0] != T:
            raise KernelError("qkv_prepare: positions/slot mapping do not match the token count")
        if (w_q is None) != (w_k is None):
            raise KernelError("qkv_prepare: q and k norm weights come together")
        if w_q is not None:
            for w in (w_q, w_k):
                self._want(w, "head norm weight", torch.float32, 1)
                if w.shape[0] != D:
                    raise KernelError(f"qkv_prepare: norm weight {tuple(w.shape)} for head size {D}")
        if R:
            self._want(cos, "cos table", torch.float32, 2)
            self._want(sin, "sin table", torch.float32, 2)
            if R % 2 or R > D or cos.shape[1] != R // 2 or sin.shape != cos.shape:
                raise KernelError(f"qkv_prepare: rotary_dim {R}, tables {tuple(cos.shape)}, head size {D}")
        if D > 512 or R // 2 > 256 or D - R > 256:
            raise KernelError(f"qkv_prepare: head size {D} (rotary {R}) is beyond the kernel's 512")
        rows = 0
        if k_pool is not None:
            rows = self._pool_rows(k_pool, v_pool, n_kv, D, qkv.dtype)
        self._check(self.lib.ra_qkv_prepare(
            _ptr(qkv), T, n_q, n_kv, D, _ptr(w_q), _ptr(w_k), float(eps), _ptr(positions),
            _ptr(cos) if R else None, _ptr(sin) if R else None, R, _ptr(q_out), _ptr(k_pool),
            _ptr(v_pool), _ptr(slot_mapping), k_pool.shape[2] if k_pool is not None else 0, rows, _code(qkv.dtype),
            self._stream()), "qkv_prepare")

    def silu_mul(self, gu, out):
        self._want(gu, "gate-up", dims=2)
        self._want(out, "silu-mul output", gu.dtype, 2)
        T, I = out.shape
        if tuple(gu.shape) != (T, 2 * I):
            raise KernelError(f"silu_mul: gate-up {tuple(gu.shape)}, out {tuple(out.shape)}")
        self._check(self.lib.ra_silu_mul(_ptr(gu), _ptr(out), T, I, _code(gu.dtype), self._stream()),
                    "silu_mul")

    # ------------------------------------------------------------------ matrix products
    # Ways to form y = x @ w^T from bfloat16 operands. Which is fastest depends on the shape in ways no
    # rule captures (the library streams one weight at 5.6 TB/s and the next at 2): route_* give the
    # rule's choice, tune_products replaces it where a measurement at load time says otherwise.
    ROW_STEPS = (1, 2, 4, 8, 12, 16, 24, 32, 48, 64)     # row counts at which products are measured
    # ... and beyond them the products for the residual stream only: with a few hundred rows (portions of
    # prompts beside decoded tokens) the library gives a product with few result columns and many of K too
    # few workgroups, and a batch over pieces of K is up to twice as fast (measured on MI355X, 512 rows:
    # 8B down 84 -> 55 µs, 32B down 272 -> 122 µs)
    ROW_STEPS_RESIDUAL = (96, 128, 192, 256, 384, 512, 640, 768, 1024, 1536, 2048, 3072, 4096)

    def _rows_step(self, M, residual=False):
        for r in self.ROW_STEPS + (self.ROW_STEPS_RESIDUAL if residual else ()):
            if M <= r:
                return r
        return 0                                          # more rows than are ever measured: the library

    SPLITS = (2, 4, 8)            # pieces of K that a product for the residual stream may be cut into

    def route_linear(self, M, N, K, out_dtype):
        """How linear() forms a bfloat16 product of M rows: the measured choice if there is one, else the rule.
        out_dtype "residual": the product whose result goes into the residual stream (linear_residual), bfloat16
        rows or, "split<n>", n shares of 32-bit sums from the library's batched product over n pieces of K."""
        hit = self.product_plan.get((self._rows_step(M, out_dtype == "residual"), N, K, False, out_dtype))
        if hit is not None:
            return hit
        if out_dtype == "residual":
            # measured on MI355X (8B shape, down: N 4,096, K 12,288): at 17 to 64 rows the library gives one
            # workgroup to each tile of the result and leaves half the chip idle; four pieces of K as a
            # batch take 24 µs against 29 to 38
            if 16 < M <= 64 and K >= 8192 and N * 2 <= K and K % 32 == 0 and self._library_bmm_fp32:
                return "split4"
            out_dtype = torch.bfloat16
        if out_dtype in (torch.bfloat16, torch.float32) and self.use_sweep(M, N, K, False):
            return "sweep"
        if out_dtype in (torch.bfloat16, torch.float32) and self.use_resident(M, N, K, False):
            return "resident512" if M <= 8 else "resident256"
        if self.use_skinny(M, N, K, out_dtype):
            return "skinny"
        if not self.own_gemm and (out_dtype == torch.bfloat16 or self._library_fp32_out):
            return "library"
        return "mfma" if K % 8 == 0 else "plain"

    def route_gated(self, M, I, K):
        hit = self.product_plan.get((self._rows_step(M), I, K, True, torch.bfloat16))
        if hit is not None:
            return hit
        if self.use_sweep(M, I, K, True):
            return "sweep"
        if self.use_resident(M, I, K, True):
            return "resident512" if M <= 8 else "resident256"
        if 0 < M <= self.gated_skinny_rows and K % 8 == 0:
            return "skinny"
        return "two"

    def _linear_by(self, how, x, w, out_dtype):
        M, K = x.shape
        N = w.shape[0]
        if how == "library":
            if out_dtype == torch.bfloat16:
                return torch.matmul(x, w.t())          # library product, as the reference's F.linear
            return torch.mm(x, w.t(), out_dtype=torch.float32)   # bf16 operands, 32-bit sums and results
        y = torch.empty(M, N, dtype=out_dtype, device=self.device)
        if how == "sweep":
            self._check(self.lib.ra_gemm_sweep_bf16(_ptr(x), _ptr(w), _ptr(y), M, N, K, 0, _code(out_dtype),
                                                    self.cu_count, self._stream()), "gemm_sweep")
        elif how.startswith("resident"):
            self._check(self.lib.ra_gemm_resident_bf16(_ptr(x), _ptr(w), _ptr(y), M, N, K, 0, _code(out_dtype),
                                                       int(how[8:]), self._stream()), "gemm_resident")
        elif how == "skinny":
            self._check(self.lib.ra_gemm_skinny_bf16(_ptr(x), _ptr(w), _ptr(y), M, N, K, _code(out_dtype),
                                                     self.skinny_max_grid, self._stream()), "gemm_skinny")
        elif how == "mfma":
            self._check(self.lib.ra_gemm_mfma_bf16(_ptr(x), _ptr(w), _ptr(y), M, N, K, _code(out_dtype),
                                                   self._stream()), "gemm_mfma")
        else:
            self._check(self.lib.ra_gemm_nt(_ptr(x), _ptr(w), _ptr(y), M, N, K, _code(x.dtype),
                                            _code(out_dtype), self._stream()), "gemm_nt")
        return y

    # ---- a norm finished inside the products around it (ScaledRows)
    def can_defer_norm(self, M, w_last, w_first, gated_first):
        """Whether, for M rows, the product by w_last [H, K1] can add its result into the residual stream
        and leave the rows of the norm that follows unfinished (linear_add_norm), and the product by
        w_first ([N, H], or [2N, H] gated) can finish them: both must be products that the sweep forms."""
        if not self.defer_norms or M < 1 or M > 16:
            return False
        for w in (w_last, w_first):
            if w.dtype != torch.bfloat16 or w.dim() != 2 or w.device != self.device:
                return False
        H = w_last.shape[0]
        if w_first.shape[1] != H or H < self.cu_count or (gated_first and w_first.shape[0] % 2):
            return False
        if self.lib.ra_gemm_sweep_workgroups(H, self.cu_count) > 256:      # shares of a row's sum that the next product adds up
            return False
        if not (self.lib.ra_gemm_sweep_fits(M, w_last.shape[1]) and self.lib.ra_gemm_sweep_fits(M, H)):
            return False
        # measured at load (tune_norm_pairs) where it was; else yes
        hit = self._defer.get((self._rows_step(M), tuple(w_last.shape), tuple(w_first.shape), bool(gated_first)))
        return True if hit is None else hit

    def tune_norm_pairs(self, pairs, max_rows=16):
        """Measures, for every shape among ``pairs`` and every row count of ROW_STEPS up to 16, whether the
        norm between two products is faster finished inside them (which ties both to the sweep) or as a
        kernel of its own between the fastest ways to form them, and notes it for can_defer_norm.
        pairs: (w_last [H, K1], norm weight [H] fp32, eps, w_first, gated) as the model has them."""
        groups = {}
        for w_last, wn, eps, w_first, gated in pairs:
            if w_last.dtype != torch.bfloat16 or w_first.dtype != torch.bfloat16 or w_last.device != self.device:
                continue
            groups.setdefault((tuple(w_last.shape), tuple(w_first.shape), bool(gated)), []).append((w_last, wn, eps, w_first))
        for (s_last, s_first, gated), members in groups.items():
            for rows in self.ROW_STEPS:
                if rows > 16 or (rows > max(1, max_rows) and rows != self._rows_step(max_rows)):
                    continue
                key = (rows, s_last, s_first, gated)
                if key in _NORM_PAIRS_MEASURED:
                    self._defer[key] = _NORM_PAIRS_MEASURED[key]
                    continue
                self._defer.pop(key, None)
                if not self.can_defer_norm(rows, members[0][0], members[0][3], gated):
                    continue
                _NORM_PAIRS_MEASURED[key] = self._defer[key] = self._measure_norm_pair(rows, members[:16], gated)

    def _measure_norm_pair(self, rows, members, gated):
        H, K1 = members[0][0].shape
        x = torch.randn(rows, K1, device=self.device, dtype=torch.float32).to(torch.bfloat16)
        h = torch.randn(rows, H, device=self.device, dtype=torch.float32)
        out = torch.empty(rows, H, dtype=torch.bfloat16, device=self.device)
        finish = self.linear_silu_mul if gated else self.linear

        def inside(m):
            w_last, wn, eps, w_first = m
            return finish(self.linear_add_norm(x, w_last, h, wn, eps), w_first)

        def apart(m):
            w_last, wn, eps, w_first = m
            self.add_rmsnorm(h, self.linear_residual(x, w_last), wn, eps, out)
            return finish(out, w_first)
        launches = max(4, min(16, len(members)))
        t_in = self._time_over(inside, members, launches)
        h.normal_()
        t_out = self._time_over(apart, members, launches)
        return t_in <= t_out

    def _sweep_norm(self, x, w, gated, out_dtype, rows_in=None, h=None, w_next=None):
        """The sweeping product with a row scale from rows_in (ScaledRows) and, with h, the residual epilogue."""
        M, K = x.shape
        N = w.shape[0] // 2 if gated else w.shape[0]
        if not self.lib.ra_gemm_sweep_fits(M, K) or M > 32:
            raise KernelError(f"rows with an unfinished norm need the sweeping product, which does not take {M} x {K}")
        out = torch.empty(M, N, dtype=out_dtype, device=self.device)
        psq_in = n_in = cols = None
        eps = 0.0
        if rows_in is not None:
            self._want(rows_in.partials, "partial sums of squares", torch.float32, 2)
            if rows_in.partials.shape[0] != M:
                raise KernelError(f"partial sums for {rows_in.partials.shape[0]} rows, x has {M}")
            psq_in, n_in, cols, eps = rows_in.partials, rows_in.partials.shape[1], rows_in.size, rows_in.eps
        psq_out = None
        if h is not None:
            self._want(h, "residual stream", torch.float32, 2)
            self._want(w_next, "norm weight", torch.float32, 1)
            if tuple(h.shape) != (M, N) or w_next.shape[0] != N or gated or out_dtype != torch.bfloat16 or M > 16:
                raise KernelError(f"linear_add_norm: x {tuple(x.shape)}, weight {tuple(w.shape)}, h {tuple(h.shape)}")
            psq_out = torch.empty(M, self.lib.ra_gemm_sweep_workgroups(N, self.cu_count), dtype=torch.float32,
                                  device=self.device)
        self._check(self.lib.ra_gemm_sweep_norm_bf16(
            _ptr(x), _ptr(w), _ptr(out), M, N, K, 1 if gated else 0, _code(out_dtype), self.cu_count,
            _ptr(psq_in), n_in or 0, cols or 0, float(eps), _ptr(h), _ptr(w_next), _ptr(psq_out), self._stream()),
            "gemm_sweep_norm")
        return out, psq_out

    def linear_add_norm(self, x, w, h, norm_weight, eps):
        """h += x @ w^T (the result rounded to the compute dtype first, as a stored result would be), and
        the rows of RMSNorm(h) with this weight and eps left unfinished: ScaledRows for linear() or
        linear_silu_mul(). x: plain rows or ScaledRows."""
        rows_in = x if isinstance(x, ScaledRows) else None
        xt = x.tensor if rows_in is not None else x
        self._want(xt, "x", torch.bfloat16, 2)
        self._want(w, "weight", torch.bfloat16, 2)
        if w.shape[1] != xt.shape[1]:
            raise KernelError(f"linear_add_norm: x {tuple(xt.shape)} times weight {tuple(w.shape)}^T")
        xw, psq = self._sweep_norm(xt, w, False, torch.bfloat16, rows_in, h, norm_weight)
        return ScaledRows(xw, psq, w.shape[0], eps)

    def _split_product(self, x, w, pieces):
        """x @ w^T as `pieces` shares [pieces, M, N] fp32, share i from columns i*K/pieces .. of K: one batched
        library product over strided views of x and w (nothing is copied)."""
        M, K = x.shape
        N = w.shape[0]
        xs = x.view(M, pieces, K // pieces).transpose(0, 1)
        wv = w.view(N, pieces, K // pieces).permute(1, 2, 0)
        return Slabs(torch.bmm(xs, wv, out_dtype=torch.float32))

    def linear_residual(self, x, w):
        """x @ w^T for the residual stream: bfloat16 (or float32) rows as linear() gives them, or Slabs
        where cutting K into pieces is faster; what takes the result must take both (the norm part does)."""
        if isinstance(x, ScaledRows) or x.dtype != torch.bfloat16:
            return self.linear(x, w)
        self._want(x, "x", dims=2)
        self._want(w, "weight", x.dtype, 2)
        M, K = x.shape
        if w.shape[1] != K:
            raise KernelError(f"linear: x {tuple(x.shape)} times weight {tuple(w.shape)}^T")
        if M == 0:
            return self.linear(x, w)
        how = self.route_linear(M, w.shape[0], K, "residual")
        if how.startswith("split"):
            return self._split_product(x, w, int(how[5:]))
        return self._linear_by(how, x, w, torch.bfloat16)

    def linear(self, x, w, out_dtype=None):
        """y = x @ w^T, x [M, K] (or ScaledRows: rows whose norm this product finishes), w [N, K]."""
        if isinstance(x, ScaledRows):
            self._want(x.tensor, "x", torch.bfloat16, 2)
            self._want(w, "weight", torch.bfloat16, 2)
            if w.shape[1] != x.tensor.shape[1]:
                raise KernelError(f"linear: x {tuple(x.tensor.shape)} times weight {tuple(w.shape)}^T")
            return self._sweep_norm(x.tensor, w, False, out_dtype or torch.bfloat16, x)[0]
        self._want(x, "x", dims=2)
        self._want(w, "weight", x.dtype, 2)
        M, K = x.shape
        N = w.shape[0]
        if w.shape[1] != K:
            raise KernelError(f"linear: x {tuple(x.shape)} times weight {tuple(w.shape)}^T")
        out_dtype = out_dtype or x.dtype
        if x.dtype == torch.float32 and out_dtype == torch.float32 and M > 16 and self._library_fp32_exact \
                and not self.own_gemm:
            return torch.matmul(x, w.t())          # the library's float32 product: checked above to be 32-bit
        if M == 0 or x.dtype != torch.bfloat16:
            return self._linear_by("plain", x, w, out_dtype)      # float32: 32-bit FMA products, W streamed once
        return self._linear_by(self.route_linear(M, N, K, out_dtype), x, w, out_dtype)

    def _gated_by(self, how, x, w_gate_up):
        M, K = x.shape
        I = w_gate_up.shape[0] // 2
        out = torch.empty(M, I, dtype=x.dtype, device=self.device)
        if how == "sweep":
            self._check(self.lib.ra_gemm_sweep_bf16(_ptr(x), _ptr(w_gate_up), _ptr(out), M, I, K, 1, _code(x.dtype),
                                                    self.cu_count, self._stream()), "gemm_sweep_gated")
        elif how.startswith("resident"):
            self._check(self.lib.ra_gemm_resident_bf16(_ptr(x), _ptr(w_gate_up), _ptr(out), M, I, K, 1,
                                                       _code(x.dtype), int(how[8:]), self._stream()),
                        "gemm_resident_gated")
        elif how == "skinny":
            self._check(self.lib.ra_gemm_skinny_gated_bf16(_ptr(x), _ptr(w_gate_up), _ptr(out), M, I, K,
                                                           self._stream()), "gemm_skinny_gated")
        else:
            self.silu_mul(self.linear(x, w_gate_up), out)
        return out

    def linear_silu_mul(self, x, w_gate_up):
        """silu(x @ Wg^T) * (x @ Wu^T) for w_gate_up = [Wg; Wu]: one kernel for few rows, else two."""
        if isinstance(x, ScaledRows):
            self._want(x.tensor, "x", torch.bfloat16, 2)
            self._want(w_gate_up, "gate-up weight", torch.bfloat16, 2)
            if w_gate_up.shape[1] != x.tensor.shape[1] or w_gate_up.shape[0] % 2:
                raise KernelError(f"linear_silu_mul: x {tuple(x.tensor.shape)}, weight {tuple(w_gate_up.shape)}")
            return self._sweep_norm(x.tensor, w_gate_up, True, torch.bfloat16, x)[0]
        self._want(x, "x", dims=2)
        self._want(w_gate_up, "gate-up weight", x.dtype, 2)
        M, K = x.shape
        I = w_gate_up.shape[0] // 2
        if w_gate_up.shape[1] != K or w_gate_up.shape[0] != 2 * I:
            raise KernelError(f"linear_silu_mul: x {tuple(x.shape)}, weight {tuple(w_gate_up.shape)}")
        how = self.route_gated(M, I, K) if x.dtype == torch.bfloat16 and M > 0 else "two"
        return self._gated_by(how, x, w_gate_up)

    def _candidates(self, M, N, K, gated, out_dtype):
        """The ways that can form this product at all."""
        residual = out_dtype == "residual"
        if residual:
            out_dtype = torch.bfloat16
        if gated:
            c = ["two"]
            if M <= 16 and K % 8 == 0:
                c.append("skinny")
        else:
            c = ["library"] if out_dtype == torch.bfloat16 or self._library_fp32_out else []
            if M <= 64 and K % 8 == 0:
                c.append("skinny")
        if self.lib.ra_gemm_resident_fits(M, K, 1 if gated else 0):
            c += ["resident256", "resident512"]
        if self.lib.ra_gemm_sweep_fits(M, K):
            c.append("sweep")
        if residual and self._library_bmm_fp32 and M > 16:
            c += [f"split{n}" for n in self.SPLITS if K % (8 * n) == 0]
        return c

    def tune_products(self, products, max_rows=64, margin=0.93, max_rows_residual=0):
        """Measures, for every shape among ``products`` and every row count of ROW_STEPS up to max_rows,
        the ways to form the product, and notes the fastest in product_plan where it beats the rule's
        choice by more than the margin (so that noise does not move a choice to and fro).

        products: (weight [N, K] bfloat16, gated, out_dtype) of the model's projections. The weights
        of one shape are taken in turn, as a decode step reads them: from memory, not from a cache
        that a repeated product on one weight would sit in. A few milliseconds per shape and row count."""
        groups = {}
        for w, gated, out_dtype in products:
            if w.dtype != torch.bfloat16 or w.dim() != 2 or w.device != self.device:
                continue
            N = w.shape[0] // 2 if gated else w.shape[0]
            groups.setdefault((N, w.shape[1], bool(gated), out_dtype or torch.bfloat16), []).append(w)
        for (N, K, gated, out_dtype), ws in groups.items():
            seen, uniq = set(), []
            for w in ws:                                  # tied weights are listed once
                if w.data_ptr() not in seen:
                    seen.add(w.data_ptr())
                    uniq.append(w)
            launches = max(4, min(16, len(uniq)))
            steps = self.ROW_STEPS
            if out_dtype == "residual" and max_rows_residual > self.ROW_STEPS[-1]:
                top = self._rows_step(max_rows_residual, True) or self.ROW_STEPS_RESIDUAL[-1]
                steps = steps + tuple(r for r in self.ROW_STEPS_RESIDUAL if r <= top)
            for rows in steps:
                if rows <= self.ROW_STEPS[-1] and rows > max(1, max_rows) and rows != self._rows_step(max_rows):
                    continue
                key = (rows, N, K, gated, out_dtype)
                if key not in self._measured:
                    # (products of many rows take long enough to be timed over a few launches)
                    few = launches if rows <= self.ROW_STEPS[-1] else max(4, min(launches, 4096 // rows))
                    self._measured[key] = self._measure(key, uniq, few, margin)
                if self._measured[key] is not None:
                    self.product_plan[key] = self._measured[key]

    def _measure(self, key, weights, launches, margin):
        """The way that forms this product clearly faster than the rule's, or None."""
        rows, N, K, gated, out_dtype = key
        cands = self._candidates(rows, N, K, gated, out_dtype)
        saved, self.product_plan = self.product_plan, {}          # the rule's choice, and "two" by the rule's product
        try:
            rule = self.route_gated(rows, N, K) if gated else self.route_linear(rows, N, K, out_dtype)
            if len(cands) < 2 or rule not in cands:
                return None
            x = torch.randn(rows, K, device=self.device, dtype=torch.float32).to(torch.bfloat16)
            if out_dtype == "residual":
                # with the residual add and norm that takes the result: shares cost it more than one result does
                h = torch.zeros(rows, N, device=self.device, dtype=torch.float32)
                wn = torch.ones(N, device=self.device, dtype=torch.float32)
                normed = torch.empty(rows, N, device=self.device, dtype=torch.bfloat16)
            runs = {}
            for how in cands:
                if gated:
                    runs[how] = lambda w, how=how: self._gated_by(how, x, w)
                elif how.startswith("split"):
                    runs[how] = lambda w, how=how: self.add_rmsnorm(h, self._split_product(x, w, int(how[5:])), wn, 1e-6, normed)
                elif out_dtype == "residual":
                    runs[how] = lambda w, how=how: self.add_rmsnorm(h, self._linear_by(how, x, w, torch.bfloat16), wn, 1e-6, normed)
                else:
                    runs[how] = lambda w, how=how: self._linear_by(how, x, w, out_dtype)
            times = self._time_ways(runs, weights, launches)
        finally:
            self.product_plan = saved
        self._times[key] = dict(times)
        best = min(times, key=times.get)
        return best if best != rule and times[best] < margin * times[rule] else None

    def _time_ways(self, runs, weights, launches, rounds=3):
        """Seconds per call of every way in ``runs`` (name -> run(w)), the weights taken in turn: one captured
        graph per way, and the ways timed in turn, round after round, each way's fastest round counting. So a
        clock that is still rising, or falls under load, meets every way alike, and the choice between two
        ways that are close does not follow the order in which they were measured."""
        import time
        graphs = {}
        for how, run in runs.items():
            run(weights[0])
            torch.cuda.synchronize(self.device)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for i in range(launches):
                    run(weights[i % len(weights)])
            graph.replay()
            graphs[how] = graph
        torch.cuda.synchronize(self.device)
        best = {how: float("inf") for how in runs}
        for _ in range(rounds):
            for how, graph in graphs.items():
                t0 = time.perf_counter()
                graph.replay()
                torch.cuda.synchronize(self.device)
                best[how] = min(best[how], time.perf_counter() - t0)
        return {how: t / launches for how, t in best.items()}

    def _time_over(self, run, weights, launches):
        """Seconds per call of run(w), the weights taken in turn, launched from one captured graph."""
        import time
        run(weights[0])
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(launches):
                run(weights[i % len(weights)])
        graph.replay()
        torch.cuda.synchronize(self.device)
        best = float("inf")
        for _ in range(3):
            t0 = time.perf_counter()
            graph.replay()
            torch.cuda.synchronize(self.device)
            best = min(best, time.perf_counter() - t0)
        return best / launches

    # ------------------------------------------------------------------ attention
    MAX_HEAD_DIM = 512

    def check_attention_sizes(self, n_q, n_kv, D, dtype):
        """Raises for head counts and sizes that no attention kernel here takes (asked when a model is built)."""
        if D > self.MAX_HEAD_DIM or D < 1:
            raise KernelError(f"attention: head size {D} is beyond the kernels' {self.MAX_HEAD_DIM}")
        if n_kv < 1 or n_q % n_kv:
            raise KernelError(f"attention: {n_q} query heads over {n_kv} kv heads")
        _code(dtype)

    def prefill_tile_rows(self, D, dtype):
        """Rows per q tile of the lists that attention() reads from step.prefill_tiles for requests with
        more than one token (a tuple; the first is the one it needs, the others it uses when they are
        there), or None where the kernel that serves this head size takes no list."""
        if dtype == torch.bfloat16 and D % 16 == 0 and D <= 256:
            rows = int(self.lib.ra_attention_prefill_tile_rows(D))
            return (rows,) if rows == 64 else (rows, 64)
        return None

    def attention(self, q, out, k_pool, v_pool, step, group, scale, window=0):
        self._want(q, "q", dims=3)
        self._want(out, "attention output", q.dtype, 3)
        T, n_q, D = q.shape
        g = step.groups[group]
        n_kv = k_pool.shape[1]
        self._pool_rows(k_pool, v_pool, n_kv, D, q.dtype)
        if out.shape != q.shape or T != step.n_tokens:
            raise KernelError(f"attention: q {tuple(q.shape)}, out {tuple(out.shape)}, step of {step.n_tokens}")
        if n_q % n_kv:
            raise KernelError(f"attention: {n_q} query heads over {n_kv} kv heads")
        self.check_attention_sizes(n_q, n_kv, D, q.dtype)
        P = k_pool.shape[2]
        window = int(window)
        tabs = (_ptr(g.page_table), _ptr(g.cu_pages), _ptr(g.kv_start), _ptr(step.cu_q), _ptr(step.q_start))
        fast_decode = q.dtype == torch.bfloat16 and step.n_decode > 0 and D % 16 == 0 and D <= 256
        fast_prefill = q.dtype == torch.bfloat16 and bool(step.prefill_tiles) and D % 16 == 0 and D <= 256 and \
            (fast_decode or step.n_decode == 0)

        def decode_part():
            S, max_splits, merge = self._decode_splits(step, n_q, n_kv, D, window)
            nd = step.n_decode
            part_acc = part_ml = None
            if not merge:
                part_acc = torch.empty(nd, n_q, max_splits, D, dtype=torch.float32, device=self.device)
                part_ml = torch.empty(nd, n_q, max_splits, 2, dtype=torch.float32, device=self.device)
            self._check(self.lib.ra_attention_decode_bf16(
                _ptr(q), _ptr(out), _ptr(part_acc), _ptr(part_ml), _ptr(k_pool), _ptr(v_pool), *tabs,
                _ptr(step.decode_segs), nd, n_q, n_kv, D, P, float(scale), window, S, max_splits,
                1 if merge else 0, self._stream()), "attention_decode_bf16")

        def prefill_part():
            rows = self.lib.ra_attention_prefill_tile_rows(D)
            tiles = step.prefill_tiles.get(rows)
            if tiles is None:
                raise KernelError(f"attention: the step lists no q tiles of {rows} rows (head size {D})")
            # Few tiles (a portion of 512 rows is four or five of 128 rows: 128 to 160 workgroups with 32
            # heads) leave CUs idle: tiles of 64 rows, one group of rows per wave and two groups of waves a
            # tile, make twice the workgroups of less than half the work each (measured at 32 heads of 128:
            # 512 rows over 4,096 keys 78 µs against 109, 300 rows at 1,500 beside 212 from scratch 36
            # against 50; from 1,024 rows on slower)
            small = step.prefill_tiles.get(64) if rows == 128 else None
            small_split = 0
            if small is not None and self.prefill_small_tiles and 2 * small.shape[0] * n_q <= 3 * self.cu_count:
                rows, tiles, small_split = 64, small, 2
            split = self.prefill_key_split or small_split or self._prefill_key_split(step, rows, tiles.shape[0] * n_q)
            self._check(self.lib.ra_attention_prefill_bf16(
                _ptr(q), _ptr(out), _ptr(k_pool), _ptr(v_pool), *tabs, _ptr(tiles), tiles.shape[0], rows,
                split, n_q, n_kv, D, P, float(scale), window, self._stream()),
                "attention_prefill_bf16")

        if fast_decode and fast_prefill and step.n_prefill_tokens > 0:
            # A step of prompt portions beside decoded tokens: the two kernels work on different rows of q and
            # out, one is bound by memory and the other by the matrix cores and the latency inside its waves,
            # so they run side by side on two streams (never while a graph is being captured: such steps are
            # not captured anyway, and a fork and join inside a graph costs more than it gives).
            if self.overlap_attention and not torch.cuda.is_current_stream_capturing():
                main = torch.cuda.current_stream(self.device)
                if self._side_stream is None:
                    self._side_stream = torch.cuda.Stream(self.device)      # (default priority, like every stream here)
                side = self._side_stream
                side.wait_stream(main)               # q and the new keys and values are written
                with torch.cuda.stream(side):
                    prefill_part()
                decode_part()
                main.wait_stream(side)               # what follows reads both kernels' rows of out
            else:
                decode_part()
                prefill_part()
            return
        if fast_decode:
            decode_part()
            if step.n_prefill_tokens == 0:
                return
            toks, n_tok = step.prefill_toks, step.n_prefill_tokens
        else:
            toks, n_tok = None, T
        if fast_prefill:
            prefill_part()
            return
        self._check(self.lib.ra_attention_plain(
            _ptr(q), _ptr(out), _ptr(k_pool), _ptr(v_pool), *tabs, _ptr(toks), step.n_seqs, n_tok,
            n_q, n_kv, D, P, float(scale), window, _code(q.dtype), self._stream()), "attention_plain")

    def _decode_splits(self, step, n_q, n_kv, D, window):
        """Keys per split of the decode attention, the most splits a request has, and whether a
        request's splits are the waves of one workgroup that merges them itself (no partial sums
        in memory, no merge kernel). Measured on MI355X: that is 3 to 11 % faster when the
        (request, kv head) pairs are a whole number of rounds over the CUs (batch 32, 64, 96, 128 with
        8 kv heads) or at least three rounds (batch 100 of uneven lengths: 208 against 221 µs), and
        slower otherwise (batch 40, 48, 72: 5 to 15 %): a workgroup of eight waves fills a CU's LDS, and
        a last round that is far from full leaves most of the chip idle."""
        longest = step.max_decode_seq_len
        # what the choice is based on: the step's own numbers, or the class its runner names (then a step run
        # eagerly and its replay from a graph choose alike and sum in the same order)
        rule = getattr(step, "decode_rule", None)
        n_rule, l_rule = rule if rule else (step.n_decode, longest)
        S = self.decode_split_tokens
        groups = n_rule * n_kv * -(-(n_q // n_kv) // 16)
        waves = self.lib.ra_attention_decode_merge_waves(D)
        if S <= 0 and window == 0 and waves >= 2 and l_rule > 64 and self.decode_merge_round > 0 \
                and (groups % self.decode_merge_round == 0 or groups >= 3 * self.decode_merge_round):
            # (the kernel cuts every request into W even splits of its own length)
            # Waves of such a workgroup (measured, 8 kv heads of 128, batch 32 to 128, contexts of 2,048 and
            # 8,192, even and uneven lengths): with fewer waves more workgroups share a CU and one's start and
            # merge run while another reads. Two are 3 to 9 % faster from two rounds of pairs on with contexts
            # up to 4,096 (and 2 % slower with longer, uneven ones), four up to 5 % faster below two rounds.
            want = self.decode_merge_waves
            if want <= 0:
                want = 4 if groups < 2 * self.decode_merge_round else (2 if l_rule <= 4096 else 8)
            W = min(want, waves, -(-l_rule // 64))
            return 64, max(W, 2), True
        if S <= 0:
            # about two thousand waves in all (eight per CU) fill the chip; fewer, longer
            # splits spend less on starting up and on the merge (measured from 1 to 128 requests)
            # (a few hundred waves do not fill it: then a wave takes one pass of 64 keys and all of a
            # request's loads are on their way at once; batch 1 over 2,048 keys 10.0 against 10.8 µs, batch 2
            # 11.8 against 12.4, from about a thousand waves on 15.4 against 14.8)
            chunks = n_rule * n_kv * ((l_rule + 63) // 64)
            S = 64 * max(1 if chunks <= 640 else 2, -(-chunks // 2048), -(-l_rule // 4096))     # and at most 64 splits a request
            if rule or getattr(step, "decode_len_is_bound", False):
                # the lengths lie somewhere below the bound (a graph's context bucket): splits
                # of at most an eighth of it keep the work of a request even
                S = min(S, max(128 if S > 64 else 64, l_rule // 8 // 64 * 64))
        max_splits = (longest - 1) // S + 1
        if window > 0:                       # a window spans at most this many splits
            max_splits = min(max_splits, (window + S - 2) // S + 1)
        return S, max_splits, False

    def attention_qkv(self, qkv, out, k_pool, v_pool, step, group, scale, window, n_q, n_kv, D,
                      w_q, w_k, eps, cos, sin, rotary_dim):
        """Attention of a step in which every request brings one token, straight from the q/k/v
        projection: the decode kernel norms and rotates q and k itself and writes k and v into
        the cache, which saves the preparation kernel. Returns False, having done nothing, when
        the step or the sizes are not such (then qkv_prepare and attention do the work)."""
        if qkv.dtype != torch.bfloat16 or step.n_decode != step.n_seqs or step.n_prefill_tokens != 0:
            return False
        R = int(rotary_dim)
        if D % 64 or D > 256 or R not in (0, D) or (w_q is None) != (w_k is None):
            return False
        self._want(qkv, "qkv", torch.bfloat16, 2)
        self._want(out, "attention output", torch.bfloat16, 3)
        T = qkv.shape[0]
        g = step.groups[group]
        self._pool_rows(k_pool, v_pool, n_kv, D, torch.bfloat16)
        if qkv.shape[1] != (n_q + 2 * n_kv) * D or tuple(out.shape) != (T, n_q, D) or T != step.n_tokens or n_q % n_kv:
            raise KernelError(f"attention_qkv: qkv {tuple(qkv.shape)}, out {tuple(out.shape)}, "
                              f"{n_q} heads over {n_kv} of {D}, step of {step.n_tokens}")
        if w_q is not None:
            for w in (w_q, w_k):
                self._want(w, "head norm weight", torch.float32, 1)
                if w.shape[0] != D:
                    raise KernelError(f"attention_qkv: norm weight {tuple(w.shape)} for head size {D}")
        if R:
            self._want(cos, "cos table", torch.float32, 2)
            self._want(sin, "sin table", torch.float32, 2)
            if cos.shape[1] != D // 2 or sin.shape != cos.shape:
                raise KernelError(f"attention_qkv: tables {tuple(cos.shape)} for head size {D}")
        P = k_pool.shape[2]
        window = int(window)
        S, max_splits, merge = self._decode_splits(step, n_q, n_kv, D, window)
        nd = step.n_decode
        part_acc = part_ml = None
        if not merge:
            part_acc = torch.empty(nd, n_q, max_splits, D, dtype=torch.float32, device=self.device)
            part_ml = torch.empty(nd, n_q, max_splits, 2, dtype=torch.float32, device=self.device)
        self._check(self.lib.ra_attention_decode_fused_bf16(
            _ptr(qkv), _ptr(out), _ptr(part_acc), _ptr(part_ml), _ptr(k_pool), _ptr(v_pool),
            # (no cu_q: every request brings one token, checked above, so request i is row i)
            _ptr(g.page_table), _ptr(g.cu_pages), _ptr(g.kv_start), None, _ptr(step.q_start),
            None, nd, n_q, n_kv, D, P, float(scale), window, S, max_splits,
            _ptr(w_q), _ptr(w_k), float(eps), _ptr(cos) if R else None, _ptr(sin) if R else None,
            1 if merge else 0, self._stream()), "attention_decode_fused_bf16")
        return True

    @staticmethod
    def _prefill_key_split(step, rows, n_workgroups):
        """Whether two groups of waves should share each q tile's keys (measured on MI355X): yes
        while the workgroups do not fill the chip, and up to three per CU when the longest tile
        reads far more keys than the average one, since then the longest tile decides the time."""
        if n_workgroups <= 256:
            return 2
        if n_workgroups > 768:
            return 1
        ends = [s + min(off + rows, q) for q, s in zip(step.q_lens, step.q_starts) if q != 1
                for off in range(0, q, rows)]
        return 2 if max(ends) * len(ends) >= 1.4 * sum(ends) else 1

    # ------------------------------------------------------------------ measurement
    def stream_read(self, t, workgroups=0):
        """Reads every byte of tensor t once with a plain read-only kernel (one workgroup per CU unless
        given); returns the words it folded them into. For measuring the machine's read rate."""
        self._want(t, "tensor to read")
        n = t.numel() * t.element_size()
        if n == 0 or n % 16 or t.data_ptr() % 16:
            raise KernelError(f"stream_read: {n} bytes at {t.data_ptr():#x} are no whole 16-byte pieces")
        g = int(workgroups) or self.cu_count
        out = torch.empty(g, dtype=torch.int32, device=self.device)
        self._check(self.lib.ra_stream_read(_ptr(t), n, _ptr(out), g, self._stream()), "stream_read")
        return out

    # ------------------------------------------------------------------ sampling
    def sample(self, logits, temperature, top_k, top_p, u, path=None):
        """Tokens and their raw log-probabilities: int32 [m, 2] (token, float bits of logprob).
        path (int32 [m], optional) is told how each row's thresholds were found: 0 none were needed,
        1 from the list of the row's largest logits, 2 by passes over the whole row."""
        self._want(logits, "logits", torch.float32, 2)
        M, V = logits.shape
        for t, name, dt in ((temperature, "temperature", torch.float32), (top_k, "top_k", torch.int32),
                            (top_p, "top_p", torch.float32), (u, "uniforms", torch.float32)):
            self._want(t, name, dt, 1)
            if t.shape[0] != M:
                raise KernelError(f"sample: {name} has {t.shape[0]} entries for {M} rows")
        out = torch.empty(M, 2, dtype=torch.int32, device=self.device)
        if path is not None:
            self._want(path, "path", torch.int32, 1)
            if path.shape[0] != M:
                raise KernelError(f"sample: path has {path.shape[0]} entries for {M} rows")
        self._check(self.lib.ra_sample_traced(_ptr(logits), M, V, _ptr(temperature), _ptr(top_k), _ptr(top_p),
                                              _ptr(u), _ptr(out), _ptr(path), self._stream()), "sample")
        return out
