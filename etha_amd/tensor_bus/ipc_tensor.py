"""Tensors across the worker -> agent process boundary, as hipIPC handles.

The reference pickles ``tensor.detach()`` with ``ForkingPickler`` (torch's CUDA-IPC reductions,
``src/etha/tensor_bus/client.py:314``) and rebuilds it in the agent with a patched
``rebuild_cuda_tensor`` (``tensor_bus/utils.py:14-69``).  Here the worker exports the allocation with
``hipIpcGetMemHandle`` through the library (base handle + byte offset, because the caching allocator
sub-allocates) and the agent maps it with ``hipIpcOpenMemHandle``.  The agent never needs a
``torch.Tensor``: the planner and the descriptor builder only ask for shape, strides, dtype, device
and addresses, which :class:`IpcTensor` provides.

When worker and agent share a process (the in-process agent used by tests and single-process
tools), a handle cannot be opened in its own process, so the tensor object itself is passed through
a process-local registry.
"""

from __future__ import annotations

import os
import pickle
import threading

import torch

from .. import _native as nat

_DTYPE_NAMES = {str(d): d for d in (
    torch.float16, torch.bfloat16, torch.float32, torch.float64, torch.int8, torch.uint8, torch.int16,
    torch.int32, torch.int64, torch.bool, torch.complex64, torch.float8_e4m3fn, torch.float8_e5m2)}

_local_registry: dict[int, torch.Tensor] = {}
_local_lock = threading.Lock()
_local_next = [0]


class _Storage:
    def __init__(self, lo: int, nbytes: int):
        self._lo, self._n = lo, nbytes

    def data_ptr(self) -> int:
        return self._lo

    def nbytes(self) -> int:
        return self._n


class IpcTensor:
    """A device tensor that exists here only as a mapped pointer plus its metadata."""

    def __init__(self, ptr: int, shape, stride, dtype: torch.dtype, device: torch.device, storage_lo: int,
                 storage_nbytes: int):
        self._ptr = ptr
        self.shape = torch.Size(shape)
        self._stride = tuple(int(s) for s in stride)
        self.dtype = dtype
        self.device = device
        self._storage = _Storage(storage_lo, storage_nbytes)
        self._open = True

    def data_ptr(self) -> int:
        return self._ptr

    def stride(self) -> tuple[int, ...]:
        return self._stride

    def dim(self) -> int:
        return len(self.shape)

    def element_size(self) -> int:
        return self.dtype.itemsize

    def numel(self) -> int:
        n = 1
        for s in self.shape:
            n *= int(s)
        return n

    def untyped_storage(self) -> _Storage:
        return self._storage

    def close(self) -> None:
        if self._open:
            self._open = False
            nat.ipc_close(self._ptr)

    def __repr__(self) -> str:
        return f"IpcTensor(shape={tuple(self.shape)}, dtype={self.dtype}, ptr={self._ptr:#x})"


def export_tensor(tensor: torch.Tensor) -> bytes:
    """Worker side: describe ``tensor`` so that the agent can address its memory."""
    tensor = tensor.detach()
    meta = {
        "pid": os.getpid(),
        "shape": tuple(tensor.shape),
        "stride": tuple(tensor.stride()),
        "dtype": str(tensor.dtype),
        "device": str(tensor.device),
    }
    if tensor.device.type != "cuda":
        # host tensors can only be handed to an agent in the same process
        with _local_lock:
            token = _local_next[0]
            _local_next[0] += 1
            _local_registry[token] = tensor
        meta["local_token"] = token
        return pickle.dumps(meta)
    st = tensor.untyped_storage()
    meta["storage_offset_bytes"] = tensor.data_ptr() - st.data_ptr()
    meta["storage_nbytes"] = st.nbytes()
    with _local_lock:
        token = _local_next[0]
        _local_next[0] += 1
        _local_registry[token] = tensor
    meta["local_token"] = token
    if tensor.numel() > 0:
        with torch.cuda.device(tensor.device):
            meta["ipc"] = nat.ipc_export(tensor.data_ptr())
    return pickle.dumps(meta)


def import_tensor(payload: bytes, device_index: int | None = None):
    """Agent side: the tensor itself when it lives in this process, else an :class:`IpcTensor`."""
    meta = pickle.loads(payload)
    if meta["pid"] == os.getpid():
        with _local_lock:
            return _local_registry[meta["local_token"]]
    if "ipc" not in meta and meta["device"].startswith("cuda"):
        dev = torch.device(meta["device"])
        return IpcTensor(0, meta["shape"], meta["stride"], _DTYPE_NAMES[meta["dtype"]], dev, 0, 0)
    if not meta["device"].startswith("cuda"):
        raise RuntimeError("a host tensor cannot be registered with an agent in another process")
    dev = torch.device(meta["device"]) if device_index is None else torch.device("cuda", device_index)
    with torch.cuda.device(dev):
        ptr = nat.ipc_open(meta["ipc"])
    return IpcTensor(ptr, meta["shape"], meta["stride"], _DTYPE_NAMES[meta["dtype"]], dev,
                     ptr - meta["storage_offset_bytes"], meta["storage_nbytes"])


def release_local(payload: bytes) -> None:
    meta = pickle.loads(payload)
    if meta["pid"] == os.getpid():
        with _local_lock:
            _local_registry.pop(meta.get("local_token"), None)
