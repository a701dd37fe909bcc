"""Run-side API of the MI355X path, in the shape of ``pypto.runtime``.

Mirrors, for the HIP target, the reference's run-side surface so that a test written for the
reference reads the same here:

* ``RunConfig``          python/pypto/runtime/runner.py:155-384  (platform whitelist, rtol/atol)
* ``DeviceTensor``       python/pypto/runtime/device_tensor.py:43-110
* ``ChipWorker``         python/pypto/runtime/worker.py:118-673  (init/close, malloc/free,
                         copy_to/copy_from, alloc_tensor/free_tensor, run, register)
* ``RegistrationHandle`` python/pypto/runtime/worker.py:675-773
* ``run``                python/pypto/runtime/runner.py:628-682
* ``benchmark``          python/pypto/runtime/bench.py:1267
* ``validate_golden``    python/pypto/runtime/device_runner.py:850-899

Everything executes through libpto_hip.so (``pypto_amd._lib``); there is no CPU path.
Host tensors must be CPU and contiguous (runner.py:930-939); outputs are written back in
place into the caller's tensors and nothing is returned (device_runner.py:751-755).
"""

from __future__ import annotations

import contextvars
import ctypes as C
import math
import struct
from dataclasses import dataclass
from typing import Any, Sequence

import torch

from . import _lib

PLATFORMS = ("mi355x",)

# torch dtype -> DataType code (include/pypto/core/dtype.h:48-96)
_DTYPE_CODES = {
    torch.int8: 0x11,
    torch.int32: 0x13,
    torch.int64: 0x14,
    torch.float8_e4m3fn: 0x31,
    torch.float16: 0x33,
    torch.float32: 0x34,
    torch.bfloat16: 0x40,
}

IN, OUT, INOUT = "IN", "OUT", "INOUT"
HOST = "HOST"  # read on the host by the launcher; never copied to the device


@dataclass(frozen=True)
class HipProgram:
    """A tile program the HIP target has a kernel for, with its tensor signature.

    The counterpart of a ``CompiledProgram`` whose manifest lists per-tensor IN/OUT/INOUT
    directions (python/pypto/backend/pto_backend.py:933-1045).
    """

    name: str
    signature: tuple[str, ...]
    optional: int = 0  # trailing tensors that may be omitted
    scalars: tuple[str, ...] = ()

    def __call__(self, *args: Any, config: "RunConfig | None" = None) -> None:
        run(self, *args, config=config)


paged_attention = HipProgram("paged_attention", (IN, IN, IN, IN, IN, OUT, HOST, IN, IN), optional=2)
# the same attention through the reference's other orchestration signatures
# 05_paged_attention_batch.py:373-386: ... config, size_query, size_key_cache, size_value_cache (never read)
paged_attention_batch = HipProgram("paged_attention_batch", (IN, IN, IN, IN, IN, OUT, HOST, HOST, HOST, HOST))
# 06_paged_attention_dynamic.py:262-270: no config, the tensors' shapes are the configuration
paged_attention_dynamic = HipProgram("paged_attention_dynamic", (IN, IN, IN, IN, IN, OUT))
# 09_paged_attention_spmd.py:445-456: scale as an FP32[1] tensor before out; config[6] = active_block_num
paged_attention_spmd = HipProgram("paged_attention_spmd", (IN, IN, IN, IN, IN, HOST, OUT, HOST))
paged_gather = HipProgram("paged_gather", (IN, IN, IN, OUT), scalars=("block_size", "col_offset"))
rms_norm = HipProgram("rms_norm", (IN, IN, OUT), scalars=("eps",))
rms_norm_unweighted = HipProgram("rms_norm", (IN, OUT), scalars=("eps",))  # 08_llama_mini.py:93-118
ffn_swiglu = HipProgram("ffn_swiglu", (IN, IN, IN, IN, OUT))
# the example's two other FFNs: act(x Wg) Wd with GELU (x * sigmoid(1.702 x)) or ReLU (01_ffn.py:90-108, :133-151)
ffn_gelu = HipProgram("ffn_gelu", (IN, IN, IN, OUT))
ffn_relu = HipProgram("ffn_relu", (IN, IN, IN, OUT))
ffn_block = HipProgram("ffn_block", (IN, IN, IN, IN, IN, OUT), scalars=("eps",))
# the block on e4m3 operands: x, gamma, then (codes [out, in], scale [out]) for gate, up and down
ffn_block_fp8 = HipProgram("ffn_block_fp8", (IN,) * 8 + (OUT,), scalars=("eps",))

# the reference's minimal single-head LLaMA forward: hidden, causal_mask, cos, sin, 7 x [D,D], w_lm, logits
llama_mini = HipProgram("llama_mini", (IN,) * 12 + (OUT,))

projection = HipProgram("projection", (IN, IN, OUT))
projection_residual = HipProgram("projection", (IN, IN, IN, OUT))
gate_up_swiglu = HipProgram("gate_up_swiglu", (IN, IN, IN, OUT))
w8a16_matmul = HipProgram("w8a16_matmul", (IN, IN, IN, OUT))
w8a16_matmul_residual = HipProgram("w8a16_matmul", (IN, IN, IN, IN, OUT))
w8a16_swiglu = HipProgram("w8a16_swiglu", (IN, IN, IN, IN, IN, OUT))
rope_kv_cache_update = HipProgram(
    "rope_kv_cache_update", (IN, IN, IN, IN, IN, INOUT, INOUT, OUT),
    scalars=("num_heads", "kv_head_num", "head_dim", "block_size"))
rope_kv_cache_update_fp8 = HipProgram(
    "rope_kv_cache_update_fp8", (IN, IN, IN, IN, IN, INOUT, INOUT, INOUT, INOUT, OUT),
    scalars=("num_heads", "kv_head_num", "head_dim", "block_size"))
decoder_layer_decode = HipProgram(
    "decoder_layer_decode", (IN, IN, IN, INOUT, INOUT) + (IN,) * 14 + (OUT,),
    scalars=("num_heads", "kv_head_num", "head_dim", "block_size", "eps"))

# the same layer over FP8E4M3FN caches: k_scale, v_scale follow value_cache
decoder_layer_decode_fp8kv = HipProgram(
    "decoder_layer_decode", (IN, IN, IN, INOUT, INOUT, INOUT, INOUT) + (IN,) * 14 + (OUT,),
    scalars=("num_heads", "kv_head_num", "head_dim", "block_size", "eps"))

# the reference's own layer: 16-bit weights, no scale tensors
decoder_layer_decode_w16 = HipProgram(
    "decoder_layer_decode", (IN, IN, IN, INOUT, INOUT) + (IN,) * 9 + (OUT,),
    scalars=("num_heads", "kv_head_num", "head_dim", "block_size", "eps"))
decoder_layer_decode_w16_fp8kv = HipProgram(
    "decoder_layer_decode", (IN, IN, IN, INOUT, INOUT, INOUT, INOUT) + (IN,) * 9 + (OUT,),
    scalars=("num_heads", "kv_head_num", "head_dim", "block_size", "eps"))

PROGRAMS = {p.name: p for p in (paged_attention, paged_attention_batch, paged_attention_dynamic, paged_attention_spmd,
                                paged_gather, rms_norm, ffn_swiglu, ffn_gelu, ffn_relu, ffn_block, ffn_block_fp8, llama_mini,
                                projection, gate_up_swiglu,
                                w8a16_matmul,
                                w8a16_swiglu, rope_kv_cache_update, rope_kv_cache_update_fp8,
                                decoder_layer_decode)}


@dataclass
class RunConfig:
    """Configuration of one run (subset of runner.py:155-365 that applies to the HIP target)."""

    platform: str = "mi355x"
    device_id: int = 0
    rtol: float = 1e-5
    atol: float = 1e-5

    def __post_init__(self) -> None:
        if self.platform not in PLATFORMS:
            raise ValueError(f"Invalid platform {self.platform!r}. Expected 'mi355x'.")
        if isinstance(self.device_id, bool) or not isinstance(self.device_id, int) or self.device_id < 0:
            raise ValueError(f"device_id must be a non-negative int, got {self.device_id!r}")


def _element_size(dtype: torch.dtype) -> int:
    return torch.empty(0, dtype=dtype).element_size()


def _require_plain_int(value: Any) -> bool:
    """True for an int that is not a bool (bool is an int subclass and never a size or an address)."""
    return isinstance(value, int) and not isinstance(value, bool)


class DeviceTensor:
    """Handle to a buffer already resident on a worker: address, shape and element type.

    The contract is the reference's (device_tensor.py:43-110): the address is a positive integer,
    the shape a non-empty sequence of positive integers, the dtype a ``torch.dtype``; the memory
    belongs to whoever allocated it.
    """

    __slots__ = ("data_ptr", "shape", "dtype")

    def __init__(self, data_ptr: int, shape: Sequence[int], dtype: torch.dtype) -> None:
        dims = tuple(shape)
        problem: Exception | None = None
        if not _require_plain_int(data_ptr) or data_ptr <= 0:
            problem = ValueError(f"DeviceTensor.data_ptr must be a positive int, got {data_ptr!r}")
        elif not all(_require_plain_int(d) for d in dims):
            problem = TypeError(f"DeviceTensor.shape must contain ints, got {dims!r}")
        elif len(dims) == 0:
            problem = ValueError("DeviceTensor.shape must be non-empty")
        elif min(dims) <= 0:
            problem = ValueError(f"DeviceTensor.shape must be all positive, got {dims}")
        elif not isinstance(dtype, torch.dtype):
            problem = TypeError(f"DeviceTensor.dtype must be torch.dtype, got {type(dtype).__name__}")
        if problem is not None:
            raise problem
        self.data_ptr, self.shape, self.dtype = data_ptr, dims, dtype

    @property
    def numel(self) -> int:
        return math.prod(self.shape)

    @property
    def nbytes(self) -> int:
        return self.numel * _element_size(self.dtype)

    def __repr__(self) -> str:
        return f"DeviceTensor(data_ptr={self.data_ptr:#x}, shape={self.shape}, dtype={self.dtype})"


def scalar_to_uint64(value: Any) -> int:
    """Raw 64-bit pattern of a scalar argument; floats travel as fp32 bits (runner.py:948-953)."""
    if isinstance(value, bool):
        return int(value)
    if isinstance(value, int):
        return value & 0xFFFFFFFFFFFFFFFF
    if isinstance(value, float):
        return struct.unpack("I", struct.pack("f", value))[0]
    raise TypeError(f"unsupported scalar type {type(value).__name__}")


def _dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODES[dtype]
    except KeyError:
        raise ValueError(f"dtype {dtype} has no DataType code on the HIP target") from None


def _descriptor(ptr: int, shape: Sequence[int], dtype: torch.dtype, nbytes: int) -> _lib.ChipTensor:
    if len(shape) > _lib.MAX_DIMS:
        raise ValueError(f"tensors of more than {_lib.MAX_DIMS} dims are not supported, got {tuple(shape)}")
    t = _lib.ChipTensor()
    t.buffer.addr = ptr
    t.buffer.size = nbytes
    t.start_offset = 0
    for i, d in enumerate(shape):
        t.shapes[i] = d
    t.ndims = len(shape)
    t.dtype = _dtype_code(dtype)
    return t


_active_worker: contextvars.ContextVar["ChipWorker | None"] = contextvars.ContextVar(
    "pypto_amd_active_worker", default=None
)


class ChipWorker:
    """Single-GPU execution handle bound to one ``(platform, device_id)`` (worker.py:118-673).

    Inside ``with ChipWorker(...)`` the module-level :func:`run` reuses this worker instead of
    creating a one-shot one.
    """

    def __init__(self, config: RunConfig | None = None, *, level: int = 2, auto_init: bool = True) -> None:
        if level != 2:
            # one GPU is the reference's level 2 (a single chip); higher levels are its multi-chip workers
            raise ValueError(f"ChipWorker only supports level=2 (one device), got level={level}")
        self._config = config or RunConfig()
        self._lib = _lib.load()
        self._initialized = False
        self._owned: dict[int, int] = {}  # device ptr -> nbytes (alloc_tensor / malloc)
        self._handles: list[RegistrationHandle] = []
        self._token = None
        if auto_init:
            self.init()

    # ---- lifecycle -------------------------------------------------------------------
    def init(self) -> None:
        if self._initialized:
            return
        _lib.check(self._lib.pto_hip_init(self._config.device_id))
        self._initialized = True

    def close(self) -> None:
        if not self._initialized:
            return
        for h in self._handles:
            h._mark_closed()
        self._handles.clear()
        for ptr in list(self._owned):
            _lib.check(self._lib.pto_hip_free(ptr))
        self._owned.clear()
        _lib.check(self._lib.pto_hip_close())
        self._initialized = False

    def __enter__(self) -> "ChipWorker":
        self.init()
        self._token = _active_worker.set(self)
        return self

    def __exit__(self, *_exc: Any) -> None:
        if self._token is not None:
            _active_worker.reset(self._token)
            self._token = None
        self.close()

    @staticmethod
    def current() -> "ChipWorker | None":
        return _active_worker.get()

    @property
    def initialized(self) -> bool:
        return self._initialized

    @property
    def platform(self) -> str:
        return self._config.platform

    @property
    def device_id(self) -> int:
        return self._config.device_id

    @property
    def level(self) -> int:
        return 2

    def _require_ready(self, op: str) -> None:
        if not self._initialized:
            raise RuntimeError(f"ChipWorker.{op}() called on a worker that is not initialized")

    def device_info(self) -> dict:
        self._require_ready("device_info")
        info = _lib.DeviceInfo()
        _lib.check(self._lib.pto_hip_device_info(C.byref(info)))
        return {
            "device_id": info.device_id,
            "compute_units": info.compute_units,
            "wavefront_size": info.wavefront_size,
            "lds_bytes_per_cu": info.lds_bytes_per_cu,
            "hbm_bytes": info.hbm_bytes,
            "arch": info.arch.decode(),
        }

    def set_option(self, name: str, value: int) -> None:
        _lib.check(self._lib.pto_hip_set_option(name.encode(), int(value)))

    def get_option(self, name: str) -> int:
        value = C.c_int64(0)
        _lib.check(self._lib.pto_hip_get_option(name.encode(), C.byref(value)))
        return value.value

    # ---- raw memory (runtime_base.py:106-118) -------------------------------------------
    def malloc(self, nbytes: int) -> int:
        self._require_ready("malloc")
        ptr = C.c_uint64(0)
        _lib.check(self._lib.pto_hip_malloc(int(nbytes), C.byref(ptr)))
        self._owned[ptr.value] = int(nbytes)
        return ptr.value

    def free(self, ptr: int) -> None:
        self._require_ready("free")
        if ptr not in self._owned:
            raise ValueError(f"pointer 0x{ptr:x} was not allocated by this worker")
        _lib.check(self._lib.pto_hip_free(ptr))
        del self._owned[ptr]

    def copy_to(self, dst_dev_ptr: int, src_host_ptr: int, nbytes: int) -> None:
        self._require_ready("copy_to")
        _lib.check(self._lib.pto_hip_copy_to(dst_dev_ptr, src_host_ptr, int(nbytes)))

    def copy_from(self, dst_host_ptr: int, src_dev_ptr: int, nbytes: int) -> None:
        self._require_ready("copy_from")
        _lib.check(self._lib.pto_hip_copy_from(dst_host_ptr, src_dev_ptr, int(nbytes)))

    def sync(self, stream: int = 0) -> None:
        self._require_ready("sync")
        _lib.check(self._lib.pto_hip_sync(stream))

    # ---- resident tensors (runtime_base.py:228-314) -------------------------------------
    def alloc_tensor(self, shape: Sequence[int], dtype: torch.dtype, *, init: torch.Tensor | None = None) -> DeviceTensor:
        self._require_ready("alloc_tensor")
        shape = tuple(int(d) for d in shape)
        nbytes = torch.tensor([], dtype=dtype).element_size()
        for d in shape:
            nbytes *= d
        ptr = self.malloc(nbytes)
        t = DeviceTensor(ptr, shape, dtype)
        if init is not None:
            _check_host_tensor(init, "init")
            if tuple(init.shape) != shape or init.dtype != dtype:
                raise ValueError(f"init has shape {tuple(init.shape)}/{init.dtype}, expected {shape}/{dtype}")
            self.copy_to(ptr, init.data_ptr(), nbytes)
        return t

    def free_tensor(self, t: DeviceTensor) -> None:
        self.free(t.data_ptr)

    def to_host(self, t: DeviceTensor) -> torch.Tensor:
        out = torch.empty(t.shape, dtype=t.dtype)
        self.copy_from(out.data_ptr(), t.data_ptr, t.nbytes)
        return out

    # ---- dispatch -------------------------------------------------------------------
    def register(self, program: HipProgram) -> "RegistrationHandle":
        self._require_ready("register")
        if not isinstance(program, HipProgram):
            raise TypeError(f"register() expects a HipProgram, got {type(program).__name__}")
        cid = C.c_int(-1)
        _lib.check(self._lib.pto_hip_register(program.name.encode(), C.byref(cid)))
        h = RegistrationHandle(self, cid.value, program)
        self._handles.append(h)
        return h

    def run(self, program: HipProgram, *args: Any, config: RunConfig | None = None, stream: int = 0) -> None:
        with self.register(program) as h:
            h(*args, config=config, stream=stream)

    def _dispatch(self, cid: int, program: HipProgram, args: Sequence[Any], stream: int) -> None:
        tensors, scalars = _split_args(program, args)
        staged: list[tuple[torch.Tensor, int, int]] = []  # (host tensor, dev ptr, nbytes) to copy back
        temps: list[int] = []
        descs = (_lib.ChipTensor * len(tensors))()
        try:
            for i, (arg, direction) in enumerate(zip(tensors, program.signature)):
                if isinstance(arg, DeviceTensor):
                    descs[i] = _descriptor(arg.data_ptr, arg.shape, arg.dtype, arg.nbytes)
                elif isinstance(arg, torch.Tensor) and arg.is_cuda:
                    if not arg.is_contiguous():
                        raise ValueError(f"tensor argument {i} must be contiguous")
                    nbytes = arg.numel() * arg.element_size()
                    descs[i] = _descriptor(arg.data_ptr() or 1, tuple(arg.shape), arg.dtype, nbytes)
                elif isinstance(arg, torch.Tensor):
                    _check_host_tensor(arg, f"argument {i}")
                    nbytes = arg.numel() * arg.element_size()
                    if direction == HOST:
                        descs[i] = _descriptor(arg.data_ptr(), tuple(arg.shape), arg.dtype, nbytes)
                        continue
                    ptr = self.malloc(max(nbytes, 1))
                    temps.append(ptr)
                    if direction in (IN, INOUT) and nbytes:
                        self.copy_to(ptr, arg.data_ptr(), nbytes)
                    if direction in (OUT, INOUT):
                        staged.append((arg, ptr, nbytes))
                    descs[i] = _descriptor(ptr, tuple(arg.shape), arg.dtype, nbytes)
                else:
                    raise TypeError(
                        f"tensor argument {i} must be a torch.Tensor or DeviceTensor, got {type(arg).__name__}"
                    )
            sc = (C.c_uint64 * max(len(scalars), 1))(*[scalar_to_uint64(s) for s in scalars])
            _lib.check(self._lib.pto_hip_run(cid, descs, len(tensors), sc, len(scalars), stream))
            if staged or temps:
                self.sync(stream)
            for host, ptr, nbytes in staged:
                if nbytes:
                    self.copy_from(host.data_ptr(), ptr, nbytes)
        finally:
            for ptr in temps:
                self.free(ptr)


class RegistrationHandle:
    """A program registered once on a worker, callable many times (worker.py:675-773)."""

    def __init__(self, worker: ChipWorker, cid: int, program: HipProgram) -> None:
        self._worker = worker
        self._cid = cid
        self._program = program
        self._closed = False

    @property
    def cid(self) -> int:
        return self._cid

    @property
    def compiled(self) -> HipProgram:
        return self._program

    @property
    def closed(self) -> bool:
        return self._closed

    def __call__(self, *args: Any, config: RunConfig | None = None, stream: int = 0) -> None:
        if self._closed:
            raise RuntimeError("RegistrationHandle is closed")
        self._worker._dispatch(self._cid, self._program, args, stream)

    def unregister(self) -> None:
        if self._closed:
            return
        _lib.check(self._worker._lib.pto_hip_unregister(self._cid))
        self._closed = True

    def _mark_closed(self) -> None:
        self._closed = True

    def __enter__(self) -> "RegistrationHandle":
        return self

    def __exit__(self, *_exc: Any) -> None:
        self.unregister()


def _check_host_tensor(t: torch.Tensor, what: str) -> None:
    if t.device.type != "cpu":
        raise ValueError(f"{what} must be a CPU tensor, got device {t.device}")
    if not t.is_contiguous():
        raise ValueError(f"{what} must be contiguous")


def _split_args(program: HipProgram, args: Sequence[Any]) -> tuple[list[Any], list[Any]]:
    n_t_max = len(program.signature)
    n_t_min = n_t_max - program.optional
    n_s = len(program.scalars)
    n = len(args)
    if not (n_t_min + n_s <= n <= n_t_max + n_s):
        raise ValueError(
            f"{program.name} takes {n_t_min}..{n_t_max} tensors followed by {n_s} scalar(s) "
            f"{program.scalars}, got {n} argument(s)"
        )
    n_t = n - n_s
    return list(args[:n_t]), list(args[n_t:])


def run(program: HipProgram, *tensors: Any, config: RunConfig | None = None) -> HipProgram:
    """Execute *program* with *tensors* (then scalars) on the device; outputs are updated in place.

    Counterpart of ``pypto.runtime.run`` (runner.py:628-682).  Reuses the worker of an
    enclosing ``with ChipWorker(...)``; otherwise opens a one-shot worker.
    """
    if isinstance(program, str):
        program = PROGRAMS[program]
    config = config or RunConfig()
    worker = ChipWorker.current()
    if worker is not None and worker.initialized and worker.device_id == config.device_id:
        worker.run(program, *tensors, config=config)
    else:
        w = ChipWorker(config)
        try:
            w.run(program, *tensors, config=config)
        finally:
            w.close()
    return program


@dataclass
class BenchmarkStats:
    rounds: int
    warmup: int
    device_wall_us: float  # mean device time per launch

    @property
    def avg_us(self) -> float:
        return self.device_wall_us


class PreparedBenchmark:
    """Descriptors of one or more argument sets, built once; ``run(rounds)`` is then a single call into
    the library's register-once loop, so a caller's own clock around it sees launches only."""

    def __init__(self, handle: RegistrationHandle, arg_sets: Sequence[Sequence[Any]], stream: int = 0) -> None:
        program = handle.compiled
        flat: list[_lib.ChipTensor] = []
        scalars: list[Any] = []
        n_t = None
        for args in arg_sets:
            tensors, scalars = _split_args(program, args)
            if n_t is None:
                n_t = len(tensors)
            elif n_t != len(tensors):
                raise ValueError("all argument sets must have the same number of tensors")
            for arg, direction in zip(tensors, program.signature):
                if isinstance(arg, DeviceTensor):
                    flat.append(_descriptor(arg.data_ptr, arg.shape, arg.dtype, arg.nbytes))
                elif isinstance(arg, torch.Tensor) and (arg.is_cuda or direction == HOST):
                    flat.append(_descriptor(arg.data_ptr(), tuple(arg.shape), arg.dtype,
                                            arg.numel() * arg.element_size()))
                else:
                    raise ValueError("benchmark() needs device-resident tensors (DeviceTensor or CUDA torch tensors)")
        if n_t is None:
            raise ValueError("benchmark() needs at least one argument set")
        self._keep = list(arg_sets)  # the descriptors hold bare addresses
        self._handle, self._stream, self._n_sets, self._n_t = handle, stream, len(arg_sets), n_t
        self._descs = (_lib.ChipTensor * len(flat))(*flat)
        self._n_scalars = len(scalars)
        self._scalars = (C.c_uint64 * max(len(scalars), 1))(*[scalar_to_uint64(x) for x in scalars])

    def run(self, rounds: int, warmup: int = 0) -> "BenchmarkStats":
        if rounds <= 0:
            raise ValueError(f"rounds must be positive, got {rounds}")
        avg = C.c_float(0.0)
        _lib.check(self._handle._worker._lib.pto_hip_benchmark(
            self._handle.cid, self._descs, self._n_sets, self._n_t, self._scalars, self._n_scalars, rounds, warmup,
            self._stream, C.byref(avg)))
        return BenchmarkStats(rounds=rounds, warmup=warmup, device_wall_us=float(avg.value))


def autotune_attention(worker: ChipWorker, handle: RegistrationHandle, arg_sets: Sequence[Sequence[Any]], *,
                       rounds: int = 30,
                       candidates: Sequence[tuple[int, int]] | None = None) -> dict:
    """Picks the launch shape of the partition-grid attention kernel for a workload by measurement.

    Two knobs decide how a launch spreads over the CUs: ``attn_tokens_per_partition`` (how finely a
    context is cut) and ``attn_waves_per_cu`` (how many wavefronts a CU may hold at once).  Their best
    values depend on how ragged the context lengths are, which the host launcher cannot see; a
    serving engine that keeps its batch composition for many steps can measure instead.  Each
    candidate ``(tokens_per_partition, waves_per_cu)`` (``0`` = the library's own choice) runs
    ``rounds`` launches of ``handle`` over ``arg_sets``; the fastest is left set on the worker and
    returned with the table of timings.  Works for any program that contains the attention kernel
    (``paged_attention``, ``decoder_layer_decode``).
    """
    if candidates is None:
        candidates = [(0, 0), (0, 2), (0, 3), (0, 4), (512, 3), (768, 2), (768, 3), (1024, 3), (2048, 0), (2048, 2)]
    prepared = PreparedBenchmark(handle, arg_sets)
    timings = {}
    for tpp, cap in candidates:
        worker.set_option("attn_tokens_per_partition", tpp)
        worker.set_option("attn_waves_per_cu", cap)
        # (0, 0) leaves the choice to the library, whose own first calls of a launch signature time
        # a few shapes: the warm-up is long enough for it to have settled
        prepared.run(max(rounds, 40))
        timings[(tpp, cap)] = prepared.run(rounds).device_wall_us
    best = min(timings, key=timings.get)
    # the library's own choice stays unless a candidate beats it by more than measurement noise
    if (0, 0) in timings and timings[best] > 0.99 * timings[(0, 0)]:
        best = (0, 0)
    worker.set_option("attn_tokens_per_partition", best[0])
    worker.set_option("attn_waves_per_cu", best[1])
    return {"tokens_per_partition": best[0], "waves_per_cu": best[1], "us": timings[best],
            "default_us": timings.get((0, 0)), "timings": timings}


def attention_stream_probe(worker: ChipWorker, key_cache: torch.Tensor, value_cache: torch.Tensor,
                           block_table: torch.Tensor, context_lens: torch.Tensor, config: torch.Tensor, *,
                           q_dtype: torch.dtype = torch.bfloat16, rounds: int = 50, stream: int = 0) -> float:
    """Microseconds the memory system needs to deliver the cache bytes of one ``paged_attention`` launch.

    Runs the library's load-only twin of the partition-grid attention kernel (same grid, block-table
    walk and loads under the worker's current ``attn_tokens_per_partition`` / ``attn_waves_per_cu``;
    nothing computed, nothing written) ``rounds`` times on device-resident tensors and returns the
    mean duration of one launch.  The attention kernel's time over this figure is what the kernel
    itself loses; this figure over bytes / 8 TB/s is what the launch shape and access pattern lose.
    """
    worker._require_ready("attention_stream_probe")
    for name, t in (("key_cache", key_cache), ("value_cache", value_cache), ("block_table", block_table),
                    ("context_lens", context_lens)):
        if not t.is_cuda or not t.is_contiguous():
            raise ValueError(f"attention_stream_probe: {name} must be a contiguous device tensor")
    cfg = config.to("cpu", torch.int64).contiguous()
    mean_ns = C.c_double(0.0)
    _lib.check(worker._lib.pto_hip_paged_attention_stream_probe(
        key_cache.data_ptr(), value_cache.data_ptr(), block_table.data_ptr(), context_lens.data_ptr(),
        C.cast(cfg.data_ptr(), C.POINTER(C.c_int64)), _dtype_code(q_dtype), _dtype_code(key_cache.dtype), int(rounds),
        stream, C.byref(mean_ns)))
    return mean_ns.value / 1e3


def mfma_only_probe(worker: ChipWorker, a: torch.Tensor, b: torch.Tensor, *, iters: int = 1500, warm_rounds: int = 100,
                    rounds: int = 60, stream: int = 0) -> dict:
    """Rate of the MFMA pipes on the values of ``a`` and ``b`` with nothing else in the loop.

    Runs the library's register-only MFMA kernel (the FFN GEMM's instruction, accumulator tiles and
    wavefronts per CU; operand fragments loaded once from the two tensors) and returns
    ``{"us": mean time per launch, "tflops": rate}``.  The shader clock under MFMA load depends on the
    operand bits, so this figure for a workload's own tensors is the ceiling its GEMM can approach.
    """
    worker._require_ready("mfma_only_probe")
    for name, t in (("a", a), ("b", b)):
        if not t.is_cuda or not t.is_contiguous() or t.dtype not in (torch.bfloat16, torch.float16):
            raise ValueError(f"mfma_only_probe: {name} must be a contiguous 16-bit device tensor")
    if a.dtype != b.dtype:
        raise ValueError("mfma_only_probe: a and b must have the same dtype")
    us, flops = C.c_double(0.0), C.c_double(0.0)
    _lib.check(worker._lib.pto_hip_mfma_probe(a.data_ptr(), a.numel(), b.data_ptr(), b.numel(), _dtype_code(a.dtype),
                                              int(iters), int(warm_rounds), int(rounds), stream, C.byref(us), C.byref(flops)))
    return {"us": us.value, "tflops": flops.value / us.value / 1e6}


def hbm_read_probe(worker: ChipWorker, buf: torch.Tensor, *, streams: bool = False, waves_per_cu: int = 8,
                   warm_rounds: int = 3, rounds: int = 10, stream: int = 0) -> dict:
    """Rate at which the GPU's compute units read ``buf`` (a contiguous device tensor, larger than the
    last-level cache if memory is to be measured) when they do nothing else.  ``streams=False``: all
    wavefronts sweep the buffer together (the most the memory system gives); ``streams=True``: every
    wavefront streams its own contiguous share, as the (sequence, head) streams of paged attention do.
    Returns ``{"us": mean time per pass, "gbps": rate}``."""
    worker._require_ready("hbm_read_probe")
    if not buf.is_cuda or not buf.is_contiguous():
        raise ValueError("hbm_read_probe: buf must be a contiguous device tensor")
    nbytes = buf.numel() * buf.element_size()
    us = C.c_double(0.0)
    _lib.check(worker._lib.pto_hip_hbm_read_probe(buf.data_ptr(), nbytes, 1 if streams else 0, int(waves_per_cu),
                                                  int(warm_rounds), int(rounds), stream, C.byref(us)))
    return {"us": us.value, "gbps": nbytes / us.value / 1e3}


def benchmark(
    handle: RegistrationHandle,
    arg_sets: Sequence[Sequence[Any]],
    *,
    rounds: int = 100,
    warmup: int = 3,
    stream: int = 0,
) -> BenchmarkStats:
    """Register-once, launch-many timing with HIP events (bench.py:1251-1267).

    ``arg_sets`` holds one or more complete argument lists of device-resident tensors; the
    rounds cycle through them so a caller can keep the working set larger than the
    last-level cache.
    """
    if rounds <= 0:
        raise ValueError(f"rounds must be positive, got {rounds}")
    return PreparedBenchmark(handle, arg_sets, stream).run(rounds, warmup)


def validate_golden(
    outputs: dict[str, torch.Tensor],
    golden: dict[str, torch.Tensor],
    rtol: float = 1e-5,
    atol: float = 1e-5,
) -> None:
    """Compares every tensor of ``outputs`` with its namesake in ``golden``.

    The rule is the reference's (device_runner.py:850-899): an element passes when
    ``|actual - expected| <= atol + rtol * |expected|``; a NaN in the golden marks an element nobody
    cares about and always passes.  The first failing tensor raises AssertionError with the count
    of mismatches and up to 20 of them.
    """
    limit = 20
    for name, produced in outputs.items():
        got, want = produced.detach().cpu(), golden[name].detach().cpu()
        # torch.isclose on the tensors as they are fails a shape that does not broadcast (as the
        # reference's comparison does); two shapes with the same element count must not pass by
        # being compared in memory order either
        if got.shape != want.shape:
            raise AssertionError(f"Output '{name}' has shape {tuple(got.shape)}, golden has {tuple(want.shape)}.")
        got, want = got.reshape(-1), want.reshape(-1)
        ignored = want.isnan()
        wrong = ~(torch.isclose(got, want, rtol=rtol, atol=atol) | ignored)
        n_wrong = int(wrong.sum())
        if n_wrong == 0:
            continue
        where = wrong.nonzero().flatten()[:limit].tolist()
        report = [f"Output '{name}' does not match golden.",
                  f"Mismatched elements: {n_wrong}/{got.numel()}"
                  + (f" ({int(ignored.sum())} don't-care skipped)" if bool(ignored.any()) else ""),
                  f"rtol={rtol}, atol={atol}",
                  f"First {len(where)} mismatches:"]
        report += [f"    [{i}] actual={got[i].item()}, expected={want[i].item()}" for i in where]
        raise AssertionError("\n".join(report))
