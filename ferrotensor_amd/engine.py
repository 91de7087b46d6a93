"""Python mirror of the reference's kernel boundary over libferrotensor_hip.so.

Same names, argument order and error behaviour as
`ferrotensor_backend::{WgpuContext, UnifiedTensor, ComputeEngine, AdamParams,
AttentionOptions, DType}` (ferrotensor-backend/src/lib.rs:38-46), so tests read
like the reference's `tests/gpu_kernels.rs`. Where the reference panics on a
shape or dtype violation, these raise (AssertionError for shape checks done
here, FtError for errors the library reports). All compute happens in the HIP
library; numpy only carries host data in and out.
"""
import atexit
import ctypes as C
import weakref
from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np

from . import _lib
from ._lib import FtError, check

MASKED_CE_SKIP = 0xFFFFFFFF   # engine/training.rs:7
SUM_SQUARES_CHUNK = 4096      # engine/training.rs (sum_squares_partial)


class DType:
    """tensor.rs:18-40 (Q4 is out of scope)."""
    FP32 = 0
    FP16 = 1

    @staticmethod
    def size_bytes(dtype):
        return 4 if dtype == DType.FP32 else 2


# Contexts still open when the interpreter shuts down are closed from an atexit hook, i.e. while
# the HIP runtime is still alive: finalisers that run during module teardown may come after it.
_live_contexts = weakref.WeakSet()


def _close_live_contexts():
    for ctx in list(_live_contexts):
        try:
            ctx.close()
        except Exception:
            pass


atexit.register(_close_live_contexts)


class HipContext:
    """`WgpuContext` (context.rs): one device, one in-order stream, the buffer pool."""

    def __init__(self, device: int = 0, stream: Optional[int] = None):
        self._lib = _lib.load()
        h = C.c_void_p()
        if stream is None:
            check(self._lib.ft_context_create(device, C.byref(h)))
        else:
            check(self._lib.ft_context_create_on_stream(device, C.c_void_p(stream), C.byref(h)))
        self.handle = h
        # Objects that hold device memory of this context (models, trainers):
        # closed first, so no handle outlives the context it allocates from.
        self._children = weakref.WeakSet()
        _live_contexts.add(self)

    def _adopt(self, child):
        self._children.add(child)

    def synchronize(self):
        check(self._lib.ft_synchronize(self.handle))

    def flush(self):
        check(self._lib.ft_flush(self.handle))

    @property
    def stream(self) -> int:
        return int(self._lib.ft_context_stream(self.handle) or 0)

    def mfma_probe(self, rounds, waves_per_simd=2, chains=4, random_operands=True):
        """(seconds, flops) of one launch of the register-only FP32 MFMA loop."""
        s, f = C.c_double(), C.c_double()
        check(self._lib.ft_mfma_probe(self.handle, rounds, waves_per_simd, chains, 1 if random_operands else 0,
                                      C.byref(s), C.byref(f)))
        return s.value, f.value

    def pool_stats(self):
        live, idle = C.c_size_t(), C.c_size_t()
        check(self._lib.ft_pool_stats(self.handle, C.byref(live), C.byref(idle)))
        return live.value, idle.value

    def pool_trim(self):
        """Returns every idle pooled buffer to the device (`BufferPool::clear`, pool.rs)."""
        check(self._lib.ft_pool_trim(self.handle))

    def close(self):
        if self.handle is not None and self.handle.value:
            for child in list(self._children):
                child.close()
            self._lib.ft_context_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class _Storage:
    """The Arc<TensorData> of tensor.rs:53-65: returns its buffer to the pool on last drop."""

    def __init__(self, ctx: HipContext, nbytes: int):
        self.ctx = ctx
        p = C.c_void_p()
        check(ctx._lib.ft_alloc(ctx.handle, nbytes, C.byref(p)))
        self.ptr = p.value
        self.nbytes = nbytes

    def __del__(self):
        try:
            if self.ptr and self.ctx.handle is not None:
                self.ctx._lib.ft_free(self.ctx.handle, C.c_void_p(self.ptr))
        except Exception:
            pass


def _numel(shape):
    n = 1
    for s in shape:
        n *= int(s)
    return n


class UnifiedTensor:
    """`UnifiedTensor` (tensor.rs:53-65): device buffer + shape + dtype; views share storage."""

    def __init__(self, storage: _Storage, shape: Sequence[int], dtype: int):
        self._storage = storage
        self.shape = [int(s) for s in shape]
        self.dtype = dtype

    # -- constructors (tensor.rs:146-406) --
    @staticmethod
    def _bytes_for(shape, dtype):
        n = _numel(shape) * DType.size_bytes(dtype)
        return max(4, (n + 3) // 4 * 4)

    @classmethod
    def empty_with_dtype(cls, ctx, shape, dtype):
        return cls(_Storage(ctx, cls._bytes_for(shape, dtype)), shape, dtype)

    @classmethod
    def empty(cls, ctx, shape):
        return cls.empty_with_dtype(ctx, shape, DType.FP32)

    @classmethod
    def zeros(cls, ctx, shape):
        t = cls.empty(ctx, shape)
        check(ctx._lib.ft_zero(ctx.handle, C.c_void_p(t.ptr), t._storage.nbytes))
        return t

    @classmethod
    def new(cls, ctx, data, shape):
        data = np.ascontiguousarray(data, np.float32)
        assert data.size == _numel(shape), "UnifiedTensor::new: %d values for shape %s" % (data.size, list(shape))
        t = cls.empty(ctx, shape)
        t.write_data(ctx, data)
        return t

    @classmethod
    def from_bytes(cls, ctx, data, shape):
        """tensor.rs:220-223: raw words (e.g. u32 targets) as an FP32-typed buffer."""
        raw = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        t = cls.empty(ctx, shape)
        assert raw.size <= t._storage.nbytes
        t.write_data(ctx, raw)
        return t

    @classmethod
    def from_f32_as_f16(cls, ctx, data, shape):
        data = np.ascontiguousarray(data, np.float32)
        assert data.size == _numel(shape)
        t = cls.empty_with_dtype(ctx, shape, DType.FP16)
        check(ctx._lib.ft_upload_f32_as_f16(ctx.handle, C.c_void_p(t.ptr), data.ctypes.data_as(C.c_void_p), data.size))
        return t

    @classmethod
    def from_f32_transposed(cls, ctx, data, rows, cols, dtype):
        data = np.ascontiguousarray(data, np.float32)
        assert data.size == rows * cols, \
            "from_f32_transposed: %d values for a [%d, %d] matrix" % (data.size, rows, cols)
        t = cls.empty_with_dtype(ctx, [cols, rows], dtype)
        check(ctx._lib.ft_upload_f32_transposed(ctx.handle, C.c_void_p(t.ptr), data.ctypes.data_as(C.c_void_p),
                                                rows, cols, dtype))
        return t

    # -- accessors --
    @property
    def ptr(self) -> int:
        return self._storage.ptr

    @property
    def ctx(self) -> HipContext:
        return self._storage.ctx

    def numel(self):
        return _numel(self.shape)

    def size_in_bytes(self):
        return self._storage.nbytes

    def reshaped(self, new_shape):
        """tensor.rs:307-330: a view with the same element count."""
        assert _numel(new_shape) == self.numel(), \
            "reshaped: %s does not hold %d elements" % (list(new_shape), self.numel())
        return UnifiedTensor(self._storage, new_shape, self.dtype)

    def write_data(self, ctx, data):
        raw = np.ascontiguousarray(data)
        assert raw.nbytes <= self._storage.nbytes
        check(ctx._lib.ft_upload(ctx.handle, C.c_void_p(self.ptr), raw.ctypes.data_as(C.c_void_p), raw.nbytes))

    def to_vec(self, ctx=None, dtype=np.float32):
        """tensor.rs:333-369: waits for queued work, then copies to the host."""
        ctx = ctx or self.ctx
        n = self.numel() * DType.size_bytes(self.dtype)
        out = np.empty(n // np.dtype(dtype).itemsize, dtype=dtype)
        check(ctx._lib.ft_download(ctx.handle, out.ctypes.data_as(C.c_void_p), C.c_void_p(self.ptr), out.nbytes))
        return out

    def to_numpy(self, ctx=None):
        if self.dtype == DType.FP16:
            return self.to_vec(ctx, np.float16).astype(np.float32).reshape(self.shape)
        return self.to_vec(ctx).reshape(self.shape)


@dataclass
class AdamParams:
    """engine/training.rs:13-32."""
    lr: float
    beta1: float = 0.9
    beta2: float = 0.999
    eps: float = 1e-8
    weight_decay: float = 0.01
    t: float = 1.0

    def c(self):
        return _lib.AdamParamsC(self.lr, self.beta1, self.beta2, self.eps, self.weight_decay, self.t)


@dataclass
class AttentionOptions:
    """engine/attention.rs:575-594."""
    causal: bool = False
    causal_offset: int = 0
    window: int = 0
    dropout_prob: float = 0.0
    seed: int = 0

    def c(self):
        return _lib.AttentionOptionsC(1 if self.causal else 0, self.causal_offset, self.window,
                                      self.dropout_prob, self.seed)


def _p(t):
    return C.c_void_p(t.ptr) if t is not None else C.c_void_p(0)


def _v(t):
    return t.ptr if t is not None else None


class ComputeEngine:
    """`ComputeEngine` (engine/mod.rs:215-274): the hot subset of its methods."""

    def __init__(self, ctx: HipContext):
        self._lib = ctx._lib

    # -- matmul (engine/matmul.rs:94-156) --
    def matmul(self, ctx, a, b, out):
        assert a.dtype == DType.FP32 and b.dtype == DType.FP32
        M, K = a.shape
        K2, N = b.shape
        assert K == K2 and out.numel() == M * N, (a.shape, b.shape, out.shape)
        check(self._lib.ft_matmul(ctx.handle, _p(a), _p(b), _p(out), M, K, N))

    def matmul_bt(self, ctx, a, b, out):
        assert a.dtype == DType.FP32 and b.dtype == DType.FP32
        M, K = a.shape
        N, K2 = b.shape
        assert K == K2 and out.numel() == M * N, (a.shape, b.shape, out.shape)
        check(self._lib.ft_matmul_bt(ctx.handle, _p(a), _p(b), _p(out), M, K, N))

    def matmul_at(self, ctx, a, b, out):
        assert a.dtype == DType.FP32 and b.dtype == DType.FP32
        K, M = a.shape
        K2, N = b.shape
        assert K == K2 and out.numel() == M * N, (a.shape, b.shape, out.shape)
        check(self._lib.ft_matmul_at(ctx.handle, _p(a), _p(b), _p(out), M, K, N))

    def matmul_f16b(self, ctx, a, b, out):
        assert b.dtype == DType.FP16, "matmul_f16b: b must be FP16"
        M, K = a.shape
        K2, N = b.shape
        assert K == K2 and out.numel() == M * N, (a.shape, b.shape, out.shape)
        check(self._lib.ft_matmul_f16b(ctx.handle, _p(a), _p(b), _p(out), M, K, N))

    def matmul_bt_f16b(self, ctx, a, b, out):
        assert b.dtype == DType.FP16, "matmul_bt_f16b: b must be FP16"
        M, K = a.shape
        N, K2 = b.shape
        assert K == K2 and out.numel() == M * N, (a.shape, b.shape, out.shape)
        check(self._lib.ft_matmul_bt_f16b(ctx.handle, _p(a), _p(b), _p(out), M, K, N))

    # -- fused LoRA linear (no single counterpart: Linear::project_2d, graph/src/lib.rs:112-126) --
    def lora_down(self, ctx, x, a, t, scale):
        M, K = x.shape
        K2, r = a.shape
        assert K == K2 and t.numel() == M * r
        check(self._lib.ft_lora_down(ctx.handle, _p(x), _p(a), _p(t), M, K, r, scale))

    def lora_linear(self, ctx, x, w, t, b, y, residual=None):
        M, K = x.shape
        K2, N = w.shape
        r = b.shape[0] if b is not None else 0
        assert K == K2 and y.numel() == M * N
        check(self._lib.ft_lora_linear(ctx.handle, _p(x), _p(w), w.dtype, _p(t), _p(b), _p(residual), _p(y), M, K, N, r))

    def rope_table(self, ctx, seq, head_dim, pos, theta):
        """(cos, sin) pairs of `rope_theta` for `seq` positions from `pos`: [seq, head_dim/2, 2] f32."""
        table = UnifiedTensor.empty(ctx, [seq, head_dim // 2, 2])
        check(self._lib.ft_rope_table(ctx.handle, _p(table), seq, head_dim, pos, theta))
        return table

    def rope_apply(self, ctx, x, out, head_dim, table, inverse=False):
        batch, seq, hidden = x.shape
        check(self._lib.ft_rope_apply(ctx.handle, _p(x), _p(out), batch, seq, hidden, head_dim, _p(table),
                                      1 if inverse else 0))

    def lora_linear_group(self, ctx, x, linears, rope_table=None, rope_seq=0, n_rope=0):
        """linears: [(w, t, b, y, residual)] sharing the input x; one launch when all can be batched.
        The first `n_rope` outputs are rotated through RoPE (heads of 64, rows of `rope_seq` tokens)."""
        from ._lib import LoraLinearDescC
        M, K = x.shape
        descs = (LoraLinearDescC * len(linears))()
        for i, (d, (w, t, b, y, residual)) in enumerate(zip(descs, linears)):
            assert w.shape[0] == K and y.numel() == M * w.shape[1]
            d.w, d.w_dtype, d.t, d.b, d.residual, d.y = _v(w), w.dtype, _v(t), _v(b), _v(residual), _v(y)
            d.N, d.r = w.shape[1], (b.shape[0] if b is not None else 0)
            if i < n_rope and rope_table is not None:
                d.rope_table, d.rope_seq = _v(rope_table), rope_seq
        check(self._lib.ft_lora_linear_group(ctx.handle, _p(x), descs, len(linears), M, K))

    def lora_linear_dx_group(self, ctx, linears, dx, residual=None):
        """linears: [(dy, w, dt, a)] of linears that shared their input; dx = (residual +) sum of their dx."""
        from ._lib import LoraDxDescC
        M = linears[0][0].shape[0]
        K = linears[0][1].shape[0]
        descs = (LoraDxDescC * len(linears))()
        for d, (dy, w, dt, a) in zip(descs, linears):
            assert list(dy.shape) == [M, w.shape[1]]
            assert w.shape[0] == K
            d.dy, d.w, d.w_dtype, d.dt, d.a = _v(dy), _v(w), w.dtype, _v(dt), _v(a)
            d.N, d.r = w.shape[1], (a.shape[1] if a is not None else 0)
        assert dx.numel() == M * K
        check(self._lib.ft_lora_linear_dx_group(ctx.handle, descs, len(linears), _p(residual), _p(dx), M, K))

    def mlp_gate_up(self, ctx, x, w_gate, w_up, gate, up, act):
        """gate = x@w_gate, up = x@w_up, act = silu(gate) * up in one launch."""
        M, K = x.shape
        K2, N = w_up.shape
        assert K == K2 and list(w_gate.shape) == [K, N] and w_gate.dtype == w_up.dtype
        assert gate.numel() == up.numel() == act.numel() == M * N
        check(self._lib.ft_mlp_gate_up(ctx.handle, _p(x), _p(w_gate), _p(w_up), w_up.dtype, _p(gate), _p(up), _p(act),
                                       M, K, N))

    def mlp_down_backward(self, ctx, dy, w_down, gate, up, d_gate, d_up, scratch=None):
        """d_gate, d_up from dy through the down projection and the gated activation, in one launch."""
        M, H = dy.shape
        F, H2 = w_down.shape
        assert H == H2 and gate.numel() == up.numel() == d_gate.numel() == d_up.numel() == M * F
        check(self._lib.ft_mlp_down_backward(ctx.handle, _p(dy), _p(w_down), w_down.dtype, _p(gate), _p(up),
                                             _p(d_gate), _p(d_up), _p(scratch), M, F, H))

    def lora_grad_down(self, ctx, dy, b, dt, scale):
        M, N = dy.shape
        r, N2 = b.shape
        assert N == N2 and dt.numel() == M * r
        check(self._lib.ft_lora_grad_down(ctx.handle, _p(dy), _p(b), _p(dt), M, N, r, scale))

    def lora_linear_dx(self, ctx, dy, w, dt, a, dx, residual=None):
        M, N = dy.shape
        K, N2 = w.shape
        r = a.shape[1] if a is not None else 0
        assert N == N2 and dx.numel() == M * K
        check(self._lib.ft_lora_linear_dx(ctx.handle, _p(dy), _p(w), w.dtype, _p(dt), _p(a), _p(residual), _p(dx), M, K, N, r))

    def lora_grad_b(self, ctx, t, dy, db):
        M, r = t.shape
        M2, N = dy.shape
        assert M == M2 and db.numel() == r * N
        check(self._lib.ft_lora_grad_b(ctx.handle, _p(t), _p(dy), _p(db), M, N, r))

    def lora_grad_a(self, ctx, x, dt, da):
        M, K = x.shape
        M2, r = dt.shape
        assert M == M2 and da.numel() == K * r
        check(self._lib.ft_lora_grad_a(ctx.handle, _p(x), _p(dt), _p(da), M, K, r))

    # -- norm (engine/norm.rs:20-99) --
    def rms_norm_eps(self, ctx, x, w, out, eps):
        size = x.shape[-1]
        assert w.numel() == size and out.numel() == x.numel()
        check(self._lib.ft_rms_norm_eps(ctx.handle, _p(x), _p(w), _p(out), x.numel() // size, size, eps))

    def rms_norm(self, ctx, x, w, out):
        self.rms_norm_eps(ctx, x, w, out, 1e-5)

    def rms_norm_backward(self, ctx, x, w, g, gx, gw, eps):
        size = x.shape[-1]
        assert g.numel() == x.numel() and gx.numel() == x.numel() and (gw is None or gw.numel() == size)
        check(self._lib.ft_rms_norm_backward(ctx.handle, _p(x), _p(w), _p(g), _p(gx), _p(gw),
                                             x.numel() // size, size, eps))

    def rms_norm_backward_noalloc(self, ctx, x, w, g, gx, gw, eps):
        """`rms_norm_backward` for callers that cannot allocate: partial sums in the library's fixed
        device array (size <= 2048, a multiple of 4; gw required)."""
        size = x.shape[-1]
        assert g.numel() == x.numel() and gx.numel() == x.numel() and gw is not None and gw.numel() == size
        check(self._lib.ft_rms_norm_backward_noalloc(ctx.handle, _p(x), _p(w), _p(g), _p(gx), _p(gw),
                                                     x.numel() // size, size, eps))

    # -- rope (engine/attention.rs:15-83) --
    @staticmethod
    def _rope_dims(t):
        if len(t.shape) == 3:
            return t.shape
        assert len(t.shape) == 2, "RoPE expects 2D or 3D tensor, got %s" % t.shape
        return [1, t.shape[0], t.shape[1]]

    def rope_theta(self, ctx, t, head_dim, pos, theta):
        b, s, h = self._rope_dims(t)
        check(self._lib.ft_rope_theta(ctx.handle, _p(t), b, s, h, head_dim, pos, theta))

    def rope(self, ctx, t, head_dim, pos):
        self.rope_theta(ctx, t, head_dim, pos, 10000.0)

    def rope_theta_inverse(self, ctx, t, head_dim, pos, theta):
        b, s, h = self._rope_dims(t)
        check(self._lib.ft_rope_theta_inverse(ctx.handle, _p(t), b, s, h, head_dim, pos, theta))

    def rope_theta_to(self, ctx, src, dst, head_dim, pos, theta, inverse=False):
        """Out-of-place `rope_theta` / `rope_theta_inverse`: dst = rotation of src, src untouched."""
        b, s, h = self._rope_dims(src)
        assert dst.numel() == src.numel()
        check(self._lib.ft_rope_theta_to(ctx.handle, _p(src), _p(dst), b, s, h, head_dim, pos, theta,
                                         1 if inverse else 0))

    # -- attention (engine/attention.rs:165-177, 341-358) --
    @staticmethod
    def _attn_dims(q, k):
        assert len(q.shape) == 4, "q must be [batch, seq, heads, head_dim]"
        assert len(k.shape) == 4, "k must be [batch, seq, kv_heads, head_dim]"
        B, Sq, H, D = q.shape
        _, Sk, Hkv, _ = k.shape
        assert D <= 128, "flash attention supports head_dim <= 128, got %d" % D
        assert Hkv > 0 and H % Hkv == 0, "num_heads (%d) must be a multiple of num_kv_heads (%d)" % (H, Hkv)
        return B, Sq, Sk, H, Hkv, D

    def flash_attention_v2_with_stats(self, ctx, q, k, v, out, stats, opts, mask=None):
        assert mask is None, "additive masks are not supported"
        B, Sq, Sk, H, Hkv, D = self._attn_dims(q, k)
        if stats is not None:
            assert stats.numel() == B * H * Sq * 2, "attention stats must be %d f32 values" % (B * H * Sq * 2)
        o = opts.c()
        check(self._lib.ft_flash_attention_v2_with_stats(ctx.handle, _p(q), _p(k), _p(v), _p(out), _p(stats),
                                                         B, Sq, Sk, H, Hkv, D, C.byref(o)))

    def flash_attention_v2_with(self, ctx, q, k, v, out, opts, mask=None):
        self.flash_attention_v2_with_stats(ctx, q, k, v, out, None, opts, mask)

    def flash_attention_v2_backward_with_stats(self, ctx, q, k, v, out, grad_out, grad_q, grad_k, grad_v, stats,
                                               opts, mask=None):
        assert mask is None, "additive masks are not supported"
        B, Sq, Sk, H, Hkv, D = self._attn_dims(q, k)
        assert stats.numel() == B * H * Sq * 2
        o = opts.c()
        check(self._lib.ft_flash_attention_v2_backward_with_stats(
            ctx.handle, _p(q), _p(k), _p(v), _p(out), _p(grad_out), _p(grad_q), _p(grad_k), _p(grad_v), _p(stats),
            B, Sq, Sk, H, Hkv, D, C.byref(o)))

    # -- elementwise (engine/elementwise.rs) --
    def add(self, ctx, a, b, out):
        assert a.numel() == b.numel() == out.numel()
        check(self._lib.ft_add(ctx.handle, _p(a), _p(b), _p(out), a.numel()))

    def add_backward(self, ctx, g, ga, gb):
        check(self._lib.ft_add_backward(ctx.handle, _p(g), _p(ga), _p(gb), g.numel()))

    def silu_gate_fused(self, ctx, up, gate, out):
        """out = silu(first) * second (engine/elementwise.rs:183-192 names them up, gate)."""
        check(self._lib.ft_silu_gate_fused(ctx.handle, _p(up), _p(gate), _p(out), out.numel()))

    def silu_gate_backward(self, ctx, up, gate, g, g_up, g_gate):
        check(self._lib.ft_silu_gate_backward(ctx.handle, _p(up), _p(gate), _p(g), _p(g_up), _p(g_gate), g.numel()))

    # -- training (engine/training.rs) --
    def gradient_scale(self, ctx, grad, scale):
        check(self._lib.ft_gradient_scale(ctx.handle, _p(grad), grad.numel(), scale))

    def clip_grad_by_norm(self, ctx, grad, scale):
        check(self._lib.ft_clip_grad_by_norm(ctx.handle, _p(grad), grad.numel(), scale))

    def gradient_accumulate(self, ctx, acc, g):
        check(self._lib.ft_gradient_accumulate(ctx.handle, _p(acc), _p(g), acc.numel()))

    def sum_squares_partial(self, ctx, x, out, offset) -> int:
        chunks = C.c_size_t()
        check(self._lib.ft_sum_squares_partial(ctx.handle, _p(x), x.numel(), _p(out), offset, C.byref(chunks)))
        return chunks.value

    def masked_cross_entropy_weighted(self, ctx, logits, targets, weights, grad, row_loss, grad_scale=1.0):
        vocab = logits.shape[-1]
        rows = logits.numel() // vocab
        assert targets.numel() == rows and weights.numel() == rows and row_loss.numel() == rows
        check(self._lib.ft_masked_cross_entropy_weighted(ctx.handle, _p(logits), _p(targets), _p(weights), _p(grad),
                                                         _p(row_loss), rows, vocab, grad_scale))

    def masked_cross_entropy(self, ctx, logits, targets, inv_tokens, grad, row_loss):
        """engine/training.rs:207-225: one weight for every row."""
        rows = logits.numel() // logits.shape[-1]
        w = UnifiedTensor.new(ctx, np.full(rows, inv_tokens, np.float32), [rows])
        self.masked_cross_entropy_weighted(ctx, logits, targets, w, grad, row_loss)

    def adamw_update(self, ctx, w, g, m, v, p: AdamParams):
        pc = p.c()
        check(self._lib.ft_adamw_update(ctx.handle, _p(w), _p(g), _p(m), _p(v), w.numel(), C.byref(pc)))

    def adamw_update_multi(self, ctx, ws, gs, ms, vs, p: AdamParams, grad_scale=1.0):
        n = len(ws)
        arr = lambda ts: (C.c_void_p * n)(*[t.ptr for t in ts])
        sizes = (C.c_size_t * n)(*[t.numel() for t in ws])
        pc = p.c()
        check(self._lib.ft_adamw_update_multi(ctx.handle, arr(ws), arr(gs), arr(ms), arr(vs), sizes, n,
                                              C.byref(pc), grad_scale))

    def copy_tensor(self, ctx, src, dst, dst_byte_offset=0):
        check(self._lib.ft_copy_tensor(ctx.handle, _p(src), src.numel() * DType.size_bytes(src.dtype), _p(dst),
                                       dst_byte_offset))

    def embedding(self, ctx, table, ids, out):
        vocab, hidden = table.shape
        check(self._lib.ft_embedding(ctx.handle, _p(table), vocab, hidden, _p(ids), ids.numel(), _p(out)))
