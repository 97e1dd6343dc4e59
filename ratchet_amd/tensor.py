"""Host-side mirror of the reference's operator interface for the Matmul path.

Same names, argument meaning and error behaviour as ratchet-core
(crates/ratchet-core/src/tensor.rs, ops/matmul.rs, quant.rs, dtype/mod.rs,
device.rs), so tests read like the reference's own:

    a_gpu = a.to(device); b_gpu = b.to(device)
    c = a_gpu.gemm(b_gpu, bias_gpu, trans_lhs, trans_rhs, trans_out).resolve()
    ours = c.to(Device.CPU)
    ground.all_close(ours, 1e-4, 1e-4)

All shape / dtype rules and all arithmetic live in libratchet_hip.so; this
module only moves bytes (torch supplies device memory and the stream) and
translates rt_status codes into exceptions.  Where the reference panics, an
InvariantError is raised; where it returns Err, an OperationError.
"""
from __future__ import annotations

import ctypes
import enum
import os
from typing import Optional, Sequence

import numpy as np

from . import _ffi


class DType(enum.IntEnum):
    """crates/ratchet-core/src/dtype/mod.rs:10-20 (Matmul subset) + Q4_K."""
    F32 = _ffi.RT_F32
    F16 = _ffi.RT_F16
    Q8_0F = _ffi.RT_Q8_0F
    Q8_0H = _ffi.RT_Q8_0H
    Q4_K = _ffi.RT_Q4_K

    def is_quantized(self) -> bool:
        return self in (DType.Q8_0F, DType.Q8_0H, DType.Q4_K)

    def activation_dt(self) -> "DType":
        return {DType.Q8_0F: DType.F32, DType.Q8_0H: DType.F16, DType.Q4_K: DType.F16}.get(self, self)

    def numpy(self):
        return {DType.F32: np.float32, DType.F16: np.float16}[self]


class OperationError(RuntimeError):
    """An Err(...) of the reference (anyhow / OperationError / TensorError)."""

    def __init__(self, status: int, msg: str = ""):
        self.status = status
        super().__init__(f"{_ffi.status_string(status)}{': ' + msg if msg else ''}")


class InvariantError(OperationError):
    """A panic of the reference (Matmul::new, OpGuards, GEMMSpec::new)."""


class DeviceRequest(enum.Enum):
    CPU = "cpu"
    GPU = "gpu"


class Device:
    """crates/ratchet-core/src/device.rs:25-56.  A GPU device owns an rt_ctx."""

    CPU: "Device"

    def __init__(self, kind: str, ordinal: int = 0):
        self.kind, self.ordinal, self._ctx = kind, ordinal, None

    @staticmethod
    def request_device(req: DeviceRequest, ordinal: int = 0) -> "Device":
        if req == DeviceRequest.CPU:
            return Device.CPU
        dev = Device("gpu", ordinal)
        ctx = ctypes.c_void_p()
        st = _ffi.lib().rt_ctx_create(ordinal, ctypes.byref(ctx))
        if st != _ffi.RT_OK:
            raise OperationError(st, "Device::request_device(GPU)")
        dev._ctx = ctx
        return dev

    @property
    def ctx(self):
        if self._ctx is None:
            raise OperationError(_ffi.RT_ERR_NO_DEVICE, "not a GPU device")
        return self._ctx

    def is_gpu(self) -> bool:
        return self.kind == "gpu"

    def __del__(self):
        if getattr(self, "_ctx", None) is not None:
            try:
                _ffi.lib().rt_ctx_destroy(self._ctx)
            except Exception:
                pass
            self._ctx = None

    def __repr__(self):
        return "Device::CPU" if self.kind == "cpu" else f"Device::GPU({self.ordinal})"


Device.CPU = Device("cpu")


def _torch():
    import torch
    return torch


def _stream_ptr() -> ctypes.c_void_p:
    return ctypes.c_void_p(_torch().cuda.current_stream().cuda_stream)


def _check(st: int, device: Optional[Device] = None, panic: bool = False):
    if st == _ffi.RT_OK:
        return
    msg = ""
    if device is not None and device._ctx is not None:
        msg = _ffi.lib().rt_last_error(device._ctx).decode()
    raise (InvariantError if panic else OperationError)(st, msg)


def tensor_nbytes(dt: DType, numel: int) -> int:
    n = ctypes.c_uint64()
    _check(_ffi.lib().rt_tensor_nbytes(int(dt), numel, ctypes.byref(n)))
    return n.value


class Matmul:
    """ops/matmul.rs:247-282: the op node; construction applies the panics of
    Matmul::new and the OpGuards."""

    def __init__(self, lhs: "Tensor", rhs: "Tensor", bias: Optional["Tensor"], trans_lhs: bool, trans_rhs: bool,
                 trans_out: bool):
        self.lhs, self.rhs, self.bias = lhs, rhs, bias
        self.trans_lhs, self.trans_rhs, self.trans_out = trans_lhs, trans_rhs, trans_out
        self.desc = _ffi.make_desc(lhs.dt, lhs.shape, rhs.dt, rhs.shape, trans_lhs, trans_rhs, trans_out,
                                   None if bias is None else bias.dt, None if bias is None else bias.shape)

    @staticmethod
    def compute_c_shape(a: "Tensor", b: "Tensor", trans_lhs: bool, trans_rhs: bool, trans_out: bool):
        d = _ffi.make_desc(a.dt, a.shape, b.dt, b.shape, trans_lhs, trans_rhs, trans_out)
        shape = (ctypes.c_int64 * _ffi.RT_MAX_RANK)()
        rank, dt = ctypes.c_int32(), ctypes.c_int32()
        _check(_ffi.lib().rt_matmul_infer(ctypes.byref(d), shape, ctypes.byref(rank), ctypes.byref(dt)))
        return tuple(shape[i] for i in range(rank.value))

    def compute_view(self):
        shape = (ctypes.c_int64 * _ffi.RT_MAX_RANK)()
        rank, dt = ctypes.c_int32(), ctypes.c_int32()
        _check(_ffi.lib().rt_matmul_infer(ctypes.byref(self.desc), shape, ctypes.byref(rank), ctypes.byref(dt)))
        return tuple(shape[i] for i in range(rank.value)), DType(dt.value)

    def check_invariants(self):
        st = _ffi.lib().rt_matmul_validate(ctypes.byref(self.desc))
        # a rank-1 operand passes graph construction in the reference and only
        # panics in GEMMSpec::new at compile time; resolve() reports it
        if st == _ffi.RT_ERR_INVALID_SHAPE and (len(self.lhs.shape) < 2 or len(self.rhs.shape) < 2):
            return
        _check(st, panic=True)

    def compute_spec(self) -> _ffi.GemmSpec:
        spec = _ffi.GemmSpec()
        _check(_ffi.lib().rt_matmul_spec(ctypes.byref(self.desc), ctypes.byref(spec)), panic=True)
        return spec

    def srcs(self):
        return [self.lhs, self.rhs] + ([self.bias] if self.bias is not None else [])


class Softmax:
    """ops/softmax.rs:15-49: the op node.  The guards (rank >= 2, dim < rank, float input) are the
    reference's panics."""

    def __init__(self, input: "Tensor", dim: int):
        self.input, self.dim = input, int(dim)
        self.shape_arr = (ctypes.c_int64 * _ffi.RT_MAX_RANK)(*input.shape) if len(input.shape) <= _ffi.RT_MAX_RANK \
            else None

    def check_invariants(self):
        if self.shape_arr is None:
            raise InvariantError(_ffi.RT_ERR_INVALID_SHAPE, "rank above RT_MAX_RANK")
        st = _ffi.lib().rt_softmax_validate(int(self.input.dt), len(self.input.shape), self.shape_arr, self.dim)
        if st in (_ffi.RT_ERR_INVALID_SHAPE, _ffi.RT_ERR_DTYPE_MISMATCH):
            _check(st, panic=True)
        _check(st)

    def srcs(self):
        return [self.input]


class Unary:
    """ops/unary.rs:71-83: the op node, for the two activations the models put behind a Linear
    (Gelu: whisper/mlp.rs:18-22, phi2/mlp.rs:13-15; Silu: phi3/mlp.rs:31-39)."""

    ACTS = {"gelu": _ffi.RT_ACT_GELU, "silu": _ffi.RT_ACT_SILU}

    def __init__(self, input: "Tensor", op: str):
        self.input, self.op, self.act = input, op, Unary.ACTS[op]

    def check_invariants(self):
        if self.input.dt not in (DType.F32, DType.F16):
            raise InvariantError(_ffi.RT_ERR_DTYPE_MISMATCH, f"{self.op} needs a float tensor")

    def srcs(self):
        return [self.input]


class Cast:
    """ops/cast.rs:15-18: the op node; F32 <-> F16."""

    def __init__(self, input: "Tensor", dst_dt: DType):
        self.input, self.dst_dt = input, DType(dst_dt)

    def check_invariants(self):
        if {self.input.dt, self.dst_dt} != {DType.F32, DType.F16}:
            raise InvariantError(_ffi.RT_ERR_DTYPE_MISMATCH, f"cast {self.input.dt.name} -> {self.dst_dt.name}")

    def srcs(self):
        return [self.input]


class Attention:
    """The attention modules' operator chain as one node (phi3/attn.rs:142-158, phi2/attn.rs:138-152,
    whisper/mha.rs:105-124): softmax(scale * q k^T + mask) v on F16 tensors [batch, heads, len, head_dim].
    `kv_len` uses the first kv_len rows of k and v, which may be a longer key/value cache; `merge_heads`
    writes the result as [batch, q_len, heads * head_dim], the callers' permute + view."""

    def __init__(self, q: "Tensor", k: "Tensor", v: "Tensor", mask: Optional["Tensor"], scale: Optional[float],
                 causal: bool, kv_len: Optional[int], merge_heads: bool):
        self.q, self.k, self.v, self.mask = q, k, v, mask
        self.causal, self.merge_heads = bool(causal), bool(merge_heads)
        self.use_workspace = True   # let a decode-shaped launch share the keys among workgroups
        if len(k.shape) != 4 or k.shape != v.shape:
            raise OperationError(_ffi.RT_ERR_INVALID_SHAPE, f"attention: k {k.shape}, v {v.shape}")
        # q is [batch, heads, len, head_dim], or [batch, len, heads * head_dim] as a projection leaves it
        # (the callers' view + permute, phi2/attn.rs:113-127, becomes a choice of strides)
        q_rows_interleaved = len(q.shape) == 3
        if q_rows_interleaved:
            if q.shape[0] != k.shape[0] or q.shape[2] != k.shape[1] * k.shape[3]:
                raise OperationError(_ffi.RT_ERR_INVALID_SHAPE, f"attention: q {q.shape}, k {k.shape}")
            B, Lq, H, D = q.shape[0], q.shape[1], k.shape[1], k.shape[3]
        else:
            if len(q.shape) != 4 or q.shape[:2] != k.shape[:2] or q.shape[3] != k.shape[3]:
                raise OperationError(_ffi.RT_ERR_INVALID_SHAPE, f"attention: q {q.shape}, k {k.shape}, v {v.shape}")
            B, H, Lq, D = q.shape
        cap = k.shape[2]
        self.kv_len = cap if kv_len is None else int(kv_len)
        if not 0 <= self.kv_len <= cap:
            raise OperationError(_ffi.RT_ERR_INVALID_SHAPE, f"attention: kv_len {self.kv_len} of a cache of {cap}")
        if mask is not None and tuple(mask.shape[-2:]) != (Lq, self.kv_len):
            raise OperationError(_ffi.RT_ERR_INVALID_SHAPE, f"attention: mask {mask.shape} for [{Lq}, {self.kv_len}] scores")
        if mask is not None and int(np.prod(mask.shape[:-2], dtype=np.int64)) != 1:
            # the kernel applies ONE [q_len, kv_len] mask to every batch and head (rt_attention_desc has a row stride only)
            raise OperationError(_ffi.RT_ERR_UNSUPPORTED, f"attention: a mask per batch or head ({mask.shape}) is not supported")
        d = _ffi.AttentionDesc()
        d.dtype, d.batch, d.heads, d.q_len, d.kv_len, d.head_dim = int(q.dt), B, H, Lq, self.kv_len, D
        d.q_strides[:] = [Lq * H * D, D, H * D] if q_rows_interleaved else [H * Lq * D, Lq * D, D]
        d.k_strides[:] = [H * cap * D, cap * D, D]
        d.v_strides[:] = [H * cap * D, cap * D, D]
        d.o_strides[:] = [Lq * H * D, D, H * D] if merge_heads else [H * Lq * D, Lq * D, D]
        d.scale = float(1.0 / np.sqrt(D)) if scale is None else float(scale)
        d.causal = int(self.causal)
        d.mask_dtype = int(mask.dt) if mask is not None else int(DType.F32)
        d.mask_row_stride = self.kv_len
        self.desc = d
        self.out_shape = (B, Lq, H * D) if merge_heads else (B, H, Lq, D)

    def check_invariants(self):
        for x in (self.k, self.v):
            if x.dt != self.q.dt:
                raise InvariantError(_ffi.RT_ERR_DTYPE_MISMATCH, "attention: q, k, v share a dtype")
        if self.mask is not None and self.mask.dt not in (DType.F32, DType.F16):
            raise InvariantError(_ffi.RT_ERR_DTYPE_MISMATCH, "attention: the mask is F32 or F16")
        st = _ffi.lib().rt_attention_validate(ctypes.byref(self.desc))
        _check(st, panic=st in (_ffi.RT_ERR_DTYPE_MISMATCH, _ffi.RT_ERR_INVALID_SHAPE))

    def srcs(self):
        return [self.q, self.k, self.v] + ([self.mask] if self.mask is not None else [])


class Cache:
    """ops/cache.rs:20-30 with dim = 2: writes `source` into rows offset .. of `cache`
    [batch, heads, capacity, head_dim].  `fresh` selects the reference's result, a new contiguous tensor
    [batch, heads, offset + len, head_dim]; otherwise the node's value is the cache itself (same storage),
    to be read in place by attention with kv_len = offset + len.  `source` is [batch, heads, len, head_dim]
    or [batch, len, heads * head_dim] as a projection leaves it."""

    def __init__(self, cache: "Tensor", source: "Tensor", offset: int, fresh: bool):
        self.cache, self.source, self.offset, self.fresh = cache, source, int(offset), bool(fresh)
        if len(cache.shape) != 4:
            raise InvariantError(_ffi.RT_ERR_INVALID_SHAPE, "cache: rank 4 expected")       # cache.rs:113 asserts rank >= 3
        B, H, cap, D = cache.shape
        if len(source.shape) == 3 and source.shape[0] == B and source.shape[2] == H * D:
            self.len, self.src_strides = source.shape[1], [source.shape[1] * H * D, D, H * D]
        elif len(source.shape) == 4 and (source.shape[0], source.shape[1], source.shape[3]) == (B, H, D):
            self.len, self.src_strides = source.shape[2], [H * source.shape[2] * D, source.shape[2] * D, D]
        else:
            raise OperationError(_ffi.RT_ERR_INVALID_SHAPE, f"cache {cache.shape} <- source {source.shape}")
        if self.offset > cap:
            raise InvariantError(_ffi.RT_ERR_INVALID_SHAPE, "cache: offset beyond the capacity")   # cache.rs:114
        self.out_shape = (B, H, self.offset + self.len, D) if fresh else cache.shape

    def check_invariants(self):
        if self.cache.dt != self.source.dt:
            raise InvariantError(_ffi.RT_ERR_DTYPE_MISMATCH, "cache and source dtypes differ")     # cache.rs:118-120

    def srcs(self):
        return [self.cache, self.source]


# An activation whose input is a Matmul node nobody has resolved yet runs in that product's
# epilogue (one kernel, one rounding) instead of as a second pass over the output.
FUSE_ACTIVATIONS = True

# A product the library would cut along K (few output tiles, long contraction) gets the workspace
# it asks for; False keeps every product in one pass.
SPLIT_K = True

# Checked mode (the role of the reference's RATCHET_CHECKED, gpu/pools/kernel_module_pool.rs:62-67): every
# output buffer is filled with 0xFF bytes (NaN as f16 and as f32) before the operator that writes it is
# enqueued, so an element a kernel fails to write cannot pass for a number.  The GPU tests switch it on.
POISON_OUTPUTS = False


class Tensor:
    """Lazy tensor: either resolved storage, or an operator node awaiting resolve()."""

    def __init__(self, shape: Sequence[int], dt: DType, device: Device, storage=None, op: Optional[Matmul] = None):
        self.shape = tuple(int(s) for s in shape)
        self.dt, self.device, self.storage, self.op = DType(dt), device, storage, op
        self.consumers = 0   # operator nodes built on this tensor
        if op is not None:
            for src in op.srcs():
                src.consumers += 1

    # -- construction -------------------------------------------------------
    @staticmethod
    def from_data(data, shape: Optional[Sequence[int]] = None, device: Device = Device.CPU) -> "Tensor":
        arr = np.ascontiguousarray(data)
        if arr.dtype not in (np.float32, np.float16):
            arr = arr.astype(np.float32)
        if shape is not None:
            arr = arr.reshape(shape)
        dt = DType.F32 if arr.dtype == np.float32 else DType.F16
        return Tensor(arr.shape, dt, Device.CPU, arr.copy())._moved(device)

    @staticmethod
    def from_quantized(data, dt: DType, shape: Sequence[int], device: Device = Device.CPU) -> "Tensor":
        raw = np.frombuffer(np.ascontiguousarray(data).tobytes(), dtype=np.uint8).copy()
        want = tensor_nbytes(dt, int(np.prod(shape, dtype=np.int64)))
        if raw.size != want:
            raise OperationError(_ffi.RT_ERR_INVALID_ARG, f"{dt.name} {tuple(shape)} needs {want} bytes, got {raw.size}")
        return Tensor(shape, dt, Device.CPU, raw)._moved(device)

    @staticmethod
    def randn(shape: Sequence[int], device: Device = Device.CPU, dt: DType = DType.F32) -> "Tensor":
        """tensor.rs:515-532: N(0,1); RATCHET_SEED seeds the generator."""
        seed = os.environ.get("RATCHET_SEED")
        rng = np.random.default_rng(int(seed) if seed is not None else None)
        return Tensor.from_data(rng.standard_normal(tuple(shape)).astype(dt.numpy()), None, device)

    # -- storage movement ---------------------------------------------------
    def _moved(self, device: Device) -> "Tensor":
        return self if device.kind == "cpu" else self.to(device)

    def resolved(self) -> bool:
        return self.storage is not None

    def to(self, device: Device) -> "Tensor":
        """tensor.rs:864-870."""
        if not self.resolved():
            raise OperationError(_ffi.RT_ERR_INVALID_ARG, "tensor is not resolved")
        if device.kind == self.device.kind:
            return self
        torch = _torch()
        if device.is_gpu():
            host = self.storage.view(np.uint8).reshape(-1)
            dev_t = torch.empty(max(host.size, 16), dtype=torch.uint8, device=f"cuda:{device.ordinal}")
            dev_t[: host.size].copy_(torch.from_numpy(host))
            return Tensor(self.shape, self.dt, device, dev_t)
        raw = self.storage.cpu().numpy()
        if self.dt.is_quantized():
            return Tensor(self.shape, self.dt, Device.CPU, raw[: tensor_nbytes(self.dt, self.numel())].copy())
        nbytes = self.numel() * (4 if self.dt == DType.F32 else 2)
        return Tensor(self.shape, self.dt, Device.CPU, raw[:nbytes].view(self.dt.numpy()).reshape(self.shape).copy())

    def numel(self) -> int:
        return int(np.prod(self.shape, dtype=np.int64))

    def data_ptr(self) -> ctypes.c_void_p:
        if not (self.resolved() and self.device.is_gpu()):
            raise OperationError(_ffi.RT_ERR_INVALID_ARG, "not a resolved GPU tensor")
        return ctypes.c_void_p(self.storage.data_ptr())

    # -- the operator -------------------------------------------------------
    def matmul(self, rhs: "Tensor", trans_lhs: bool, trans_rhs: bool) -> "Tensor":
        """tensor.rs:381-386."""
        return self.gemm(rhs, None, trans_lhs, trans_rhs, False)

    def gemm(self, rhs: "Tensor", bias: Optional["Tensor"], trans_lhs: bool, trans_rhs: bool,
             trans_out: bool) -> "Tensor":
        """tensor.rs:388-400: builds the lazy Matmul node."""
        op = Matmul(self, rhs, bias, trans_lhs, trans_rhs, trans_out)
        shape, dt = op.compute_view()   # Err on shape failure
        op.check_invariants()           # panics of Matmul::new and the OpGuards
        return Tensor(shape, dt, self.device, None, op)

    def softmax(self, dim: int) -> "Tensor":
        """tensor.rs `softmax(dim)`: the lazy Softmax node (ops/softmax.rs); same shape and dtype."""
        op = Softmax(self, dim)
        op.check_invariants()
        return Tensor(self.shape, self.dt, self.device, None, op)

    def attention(self, k: "Tensor", v: "Tensor", mask: Optional["Tensor"] = None, scale: Optional[float] = None,
                  causal: bool = False, kv_len: Optional[int] = None, merge_heads: bool = False) -> "Tensor":
        """softmax(scale * self k^T + mask) v as one lazy node; see Attention."""
        op = Attention(self, k, v, mask, scale, causal, kv_len, merge_heads)
        op.check_invariants()
        return Tensor(op.out_shape, self.dt, self.device, None, op)

    def cache(self, source: "Tensor", dim: int, offset: int) -> "Tensor":
        """tensor.rs `cache(source, dim, offset)` (ops/cache.rs): self is the cache; the result is the fresh
        tensor cache[.., :offset, :] ++ source, and the cache holds the new rows too."""
        if dim != 2:
            raise OperationError(_ffi.RT_ERR_UNSUPPORTED, "cache: dim 2 (the sequence axis of [b, h, s, d])")
        op = Cache(self, source, offset, fresh=True)
        op.check_invariants()
        return Tensor(op.out_shape, self.dt, self.device, None, op)

    def cache_write(self, source: "Tensor", offset: int) -> "Tensor":
        """The same write without the copy: the result is the cache itself (same storage), to be passed to
        attention(kv_len = offset + len)."""
        op = Cache(self, source, offset, fresh=False)
        op.check_invariants()
        return Tensor(op.out_shape, self.dt, self.device, None, op)

    def gelu(self) -> "Tensor":
        """tensor.rs `gelu()` (impl_unary_op): the lazy Unary node; same shape and dtype."""
        return self._unary("gelu")

    def silu(self) -> "Tensor":
        """tensor.rs `silu()` (impl_unary_op)."""
        return self._unary("silu")

    def _unary(self, name: str) -> "Tensor":
        op = Unary(self, name)
        op.check_invariants()
        return Tensor(self.shape, self.dt, self.device, None, op)

    def cast(self, dst_dt: DType) -> "Tensor":
        """tensor.rs `cast(dst_dt)`: a no-op for the same dtype, the lazy Cast node otherwise."""
        if DType(dst_dt) == self.dt:
            return self
        op = Cast(self, dst_dt)
        op.check_invariants()
        return Tensor(self.shape, DType(dst_dt), self.device, None, op)

    def full(self) -> "Tensor":
        """tensor.rs `full()`: cast to F32."""
        return self.cast(DType.F32)

    def half(self) -> "Tensor":
        """tensor.rs `half()`: cast to F16."""
        return self.cast(DType.F16)

    def resolve(self) -> "Tensor":
        """tensor.rs:738-787: run every unresolved node below this one, then wait."""
        if self.resolved():
            return self
        dev = self.device
        if not dev.is_gpu():
            raise OperationError(_ffi.RT_ERR_NO_DEVICE, "resolve() needs a GPU tensor (try_gpu)")
        self._execute()
        _check(_ffi.lib().rt_sync(dev.ctx, _stream_ptr()), dev)
        return self

    def _execute(self):
        if self.resolved():
            return
        op, dev, torch = self.op, self.device, _torch()
        act = _ffi.RT_ACT_NONE
        # an activation behind a product nobody else reads runs in that product's epilogue; a product with a second
        # consumer is computed once, rounded, and the activation reads it (as the reference's two operators do)
        if (isinstance(op, Unary) and FUSE_ACTIVATIONS and isinstance(op.input.op, Matmul) and not op.input.resolved()
                and op.input.consumers <= 1):
            act, op = op.act, op.input.op
        for src in op.srcs():
            src._execute()
            if not src.device.is_gpu():
                raise OperationError(_ffi.RT_ERR_NO_DEVICE, "operand is not on the GPU")
        if isinstance(op, Softmax):
            # the kernel works in place (softmax.rs:47-49); the source tensor keeps its own storage
            out = op.input.storage.clone()
            st = _ffi.lib().rt_softmax_enqueue(dev.ctx, int(self.dt), ctypes.c_void_p(out.data_ptr()), len(self.shape),
                                               op.shape_arr, op.dim, _stream_ptr())
            _check(st, dev)
            self.storage = out
            return
        esz = 4 if self.dt == DType.F32 else 2
        out = torch.empty(max(self.numel() * esz, 16), dtype=torch.uint8, device=f"cuda:{dev.ordinal}")
        if POISON_OUTPUTS:
            out.fill_(0xFF)
        if isinstance(op, Cache):
            B, H, cap, D = op.cache.shape
            strides = (ctypes.c_int64 * 3)(*op.src_strides)
            dst = ctypes.c_void_p(out.data_ptr()) if op.fresh else None
            st = _ffi.lib().rt_cache_write_enqueue(dev.ctx, int(self.dt), op.cache.data_ptr(), op.source.data_ptr(), strides,
                                                   dst, B, H, cap, op.offset, op.len, D, _stream_ptr())
            _check(st, dev)
            self.storage = out if op.fresh else op.cache.storage
            return
        if isinstance(op, Attention):
            need = ctypes.c_uint64()
            _check(_ffi.lib().rt_attention_workspace_bytes(ctypes.byref(op.desc), ctypes.byref(need)), dev)
            ws = torch.empty(need.value, dtype=torch.uint8, device=f"cuda:{dev.ordinal}") if need.value and op.use_workspace else None
            st = _ffi.lib().rt_attention_enqueue(
                dev.ctx, ctypes.byref(op.desc), op.q.data_ptr(), op.k.data_ptr(), op.v.data_ptr(),
                op.mask.data_ptr() if op.mask is not None else None, ctypes.c_void_p(out.data_ptr()),
                ctypes.c_void_p(ws.data_ptr()) if ws is not None else None, need.value if ws is not None else 0, _stream_ptr())
            _check(st, dev)
            self.storage = out
            return
        if isinstance(op, Unary):
            st = _ffi.lib().rt_unary_enqueue(dev.ctx, op.act, int(self.dt), op.input.data_ptr(),
                                             ctypes.c_void_p(out.data_ptr()), self.numel(), _stream_ptr())
            _check(st, dev)
            self.storage = out
            return
        if isinstance(op, Cast):
            st = _ffi.lib().rt_cast_enqueue(dev.ctx, int(op.input.dt), int(op.dst_dt), op.input.data_ptr(),
                                            ctypes.c_void_p(out.data_ptr()), self.numel(), _stream_ptr())
            _check(st, dev)
            self.storage = out
            return
        op.compute_spec()  # GEMMSpec::new asserts (rank >= 2, stacks)
        need = ctypes.c_uint64()
        _check(_ffi.lib().rt_matmul_workspace_bytes(dev.ctx, ctypes.byref(op.desc), ctypes.byref(need)), dev)
        ws = torch.empty(need.value, dtype=torch.uint8, device=f"cuda:{dev.ordinal}") if need.value and SPLIT_K else None
        st = _ffi.lib().rt_matmul_enqueue_ws(
            dev.ctx, ctypes.byref(op.desc), op.lhs.data_ptr(), op.rhs.data_ptr(),
            op.bias.data_ptr() if op.bias is not None else None, ctypes.c_void_p(out.data_ptr()), act,
            ctypes.c_void_p(ws.data_ptr()) if ws is not None else None, need.value if ws is not None else 0, _stream_ptr())
        _check(st, dev)
        self.storage = out

    # -- inspection ---------------------------------------------------------
    def to_ndarray(self) -> np.ndarray:
        t = self.to(Device.CPU)
        if t.dt.is_quantized():
            raise OperationError(_ffi.RT_ERR_DTYPE_MISMATCH, "quantized tensor has no ndarray view")
        return t.storage

    def all_close(self, other: "Tensor", atol: float, rtol: float) -> None:
        """tensor.rs:1035-1082 with CloseStats::is_close (tensor.rs:954-958):
        |a - b| <= atol + rtol * |b|, NaN == NaN, same-signed infinities equal."""
        if self.shape != other.shape:
            raise OperationError(_ffi.RT_ERR_INVALID_SHAPE, f"Shape mismatch {self.shape} != {other.shape}")
        assert self.dt == other.dt, f"DType mismatch {self.dt} != {other.dt}"
        a = self.to_ndarray().astype(np.float64)
        b = other.to_ndarray().astype(np.float64)
        diff = np.abs(a - b)
        ok = (np.isnan(a) & np.isnan(b)) | (np.isinf(a) & np.isinf(b) & (np.sign(a) == np.sign(b))) | (
            diff <= atol + rtol * np.abs(b))
        if not ok.all():
            bad = int((~ok).sum())
            idx = np.unravel_index(np.nanargmax(np.where(np.isfinite(diff), diff, -1)), diff.shape)
            raise AssertionError(f"{bad} samples not close - MAE={np.nanmax(diff)} at {idx}")

    def __repr__(self):
        state = "resolved" if self.resolved() else "lazy"
        return f"Tensor({self.dt.name}{list(self.shape)}, {self.device}, {state})"


class Quantization(enum.Enum):
    """quant.rs:173-196."""
    NONE = (1, 1)
    SInt8 = (4, 32)

    def pack_size(self) -> int:
        return self.value[0]

    def group_size(self) -> int:
        return self.value[1]


class Quantizer:
    """quant.rs:8-124.  The arithmetic runs on the GPU (rt_quantize_q8_0 /
    rt_dequantize); a CPU tensor is staged through `device` and returned on
    the CPU, as in the reference."""

    def __init__(self, format: Quantization, device: Optional[Device] = None):
        self.format, self.device = format, device

    def _dev(self, t: Tensor) -> Device:
        if t.device.is_gpu():
            return t.device
        if self.device is None:
            self.device = Device.request_device(DeviceRequest.GPU)
        return self.device

    def quantize(self, tensor: Tensor) -> Tensor:
        return tensor if self.format == Quantization.NONE else self.sint8_quantize(tensor)

    def sint8_quantize(self, tensor: Tensor) -> Tensor:
        numel = tensor.numel()
        assert numel % self.format.pack_size() == 0 and numel % self.format.group_size() == 0
        assert tensor.dt == DType.F32
        dev, torch = self._dev(tensor), _torch()
        src = tensor.to(dev)
        out = torch.empty(tensor_nbytes(DType.Q8_0F, numel), dtype=torch.uint8, device=f"cuda:{dev.ordinal}")
        _check(_ffi.lib().rt_quantize_q8_0(dev.ctx, src.data_ptr(), numel, ctypes.c_void_p(out.data_ptr()),
                                           _stream_ptr()), dev)
        _check(_ffi.lib().rt_sync(dev.ctx, _stream_ptr()), dev)
        q = Tensor(tensor.shape, DType.Q8_0F, dev, out)
        return q if tensor.device.is_gpu() else q.to(Device.CPU)

    def sint8_dequantize(self, quantized: Tensor) -> Tensor:
        assert quantized.dt == DType.Q8_0F
        return dequantize(quantized, self._dev(quantized))


def dequantize(quantized: Tensor, device: Optional[Device] = None) -> Tensor:
    """Quantized tensor -> f32 tensor on the tensor's own device kind."""
    assert quantized.dt.is_quantized()
    dev = quantized.device if quantized.device.is_gpu() else (device or Device.request_device(DeviceRequest.GPU))
    torch = _torch()
    src = quantized.to(dev)
    out = torch.empty(max(quantized.numel() * 4, 16), dtype=torch.uint8, device=f"cuda:{dev.ordinal}")
    _check(_ffi.lib().rt_dequantize(dev.ctx, int(quantized.dt), src.data_ptr(), quantized.numel(),
                                    ctypes.c_void_p(out.data_ptr()), _stream_ptr()), dev)
    _check(_ffi.lib().rt_sync(dev.ctx, _stream_ptr()), dev)
    t = Tensor(quantized.shape, DType.F32, dev, out)
    return t if quantized.device.is_gpu() else t.to(Device.CPU)


def transcode_gguf_q8_0(blocks, shape: Sequence[int], dt: DType, device: Device) -> Tensor:
    """GGUFInterop::transcode (crates/ratchet-loader/src/gguf/dtype.rs:40-110):
    raw GGUF Q8_0 blocks (host bytes) -> Q8_0F / Q8_0H tensor on `device`."""
    torch = _torch()
    raw = np.frombuffer(np.ascontiguousarray(blocks).tobytes(), dtype=np.uint8)
    numel = int(np.prod(shape, dtype=np.int64))
    assert raw.size == (numel // 32) * 34
    src = torch.from_numpy(raw.copy()).to(f"cuda:{device.ordinal}")
    out = torch.empty(tensor_nbytes(dt, numel), dtype=torch.uint8, device=f"cuda:{device.ordinal}")
    _check(_ffi.lib().rt_transcode_gguf_q8_0(device.ctx, ctypes.c_void_p(src.data_ptr()), numel // 32, int(dt),
                                             ctypes.c_void_p(out.data_ptr()), _stream_ptr()), device)
    _check(_ffi.lib().rt_sync(device.ctx, _stream_ptr()), device)
    return Tensor(shape, dt, device, out)
