"""ROCArray: the boundary data type of the path (reference: src/array.jl:19-39).

A dense COLUMN-MAJOR device array: a device buffer, Julia ``dims`` and a byte ``offset``; the device
pointer handed to the kernels is ``buffer + offset`` exactly like
``Base.unsafe_convert(Ptr{T}, ::ROCArray)`` (src/array.jl:353-354).  PyTorch supplies the device
memory and the stream, nothing else: no torch kernel runs on the path.
"""
from __future__ import annotations

import numpy as np
import torch

from . import _lib as L

_DTYPE_CODE = {
    np.dtype(np.float32): L.RK_F32, np.dtype(np.float64): L.RK_F64,
    np.dtype(np.int32): L.RK_I32, np.dtype(np.int64): L.RK_I64,
    np.dtype(np.bool_): L.RK_U8, np.dtype(np.uint8): L.RK_U8,
    np.dtype(np.uint32): L.RK_U32, np.dtype(np.uint64): L.RK_U64,
    np.dtype(np.float16): L.RK_F16, np.dtype(np.int16): L.RK_I16,
    np.dtype(np.int8): L.RK_I8, np.dtype(np.uint16): L.RK_U16,
}


def dtype_code(dt) -> int:
    try:
        return _DTYPE_CODE[np.dtype(dt)]
    except KeyError:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, f"eltype {np.dtype(dt)}") from None


def device() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU visible: ROCArray needs a HIP device (there is no CPU path)")
    return torch.device("cuda", torch.cuda.current_device())


def stream_ptr() -> int:
    """The current (task-local, in the reference: src/tls.jl:71-86) stream as a hipStream_t."""
    return int(torch.cuda.current_stream().cuda_stream)


class ROCArray:
    """Column-major device array with Julia's logical ``dims`` (1-based API at the op level)."""

    __slots__ = ("buf", "dims", "dtype", "offset")

    def __init__(self, data=None, *, dims=None, dtype=None, buf=None, offset=0):
        if buf is not None:                      # wrap existing storage (views, reshape)
            self.buf = buf
            self.dims = tuple(int(d) for d in dims)
            self.dtype = np.dtype(dtype)
            self.offset = int(offset)
            return
        if data is None:                         # ROCArray{T}(undef, dims)
            self.dims = tuple(int(d) for d in dims)
            self.dtype = np.dtype(dtype)
            self.offset = 0
            nbytes = int(np.prod(self.dims, dtype=np.int64)) * self.dtype.itemsize
            self.buf = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device())
            return
        host = np.asarray(data)
        if dtype is not None:
            host = host.astype(dtype)
        self.dims = tuple(host.shape)
        self.dtype = host.dtype
        self.offset = 0
        flat = np.ascontiguousarray(host.reshape(-1, order="F"))
        raw = torch.from_numpy(flat.view(np.uint8).copy()) if flat.size else torch.empty(1, dtype=torch.uint8)
        self.buf = raw.to(device(), non_blocking=False)

    # -- Julia-like queries ---------------------------------------------------------------------
    @property
    def ndim(self) -> int:
        return len(self.dims)

    def size(self, d=None):
        if d is None:
            return self.dims
        return self.dims[d - 1] if d <= len(self.dims) else 1

    def __len__(self) -> int:
        return int(np.prod(self.dims, dtype=np.int64))

    length = __len__

    @property
    def ptr(self) -> int:
        return int(self.buf.data_ptr()) + self.offset

    @property
    def code(self) -> int:
        return dtype_code(self.dtype)

    def __repr__(self):
        return f"ROCArray{{{self.dtype}}}{self.dims}"

    # -- host transfer (src/array.jl:215-249) ------------------------------------------------------
    def to_host(self) -> np.ndarray:
        """``Array(x)``: synchronises the stream and copies to the host (Julia-shaped NumPy array)."""
        n = len(self)
        nbytes = n * self.dtype.itemsize
        check_waits()                       # the host waits here anyway: the place to learn of a give-up
        torch.cuda.current_stream().synchronize()
        raw = self.buf[self.offset:self.offset + nbytes].cpu().numpy()
        return raw.view(self.dtype)[:n].reshape(self.dims, order="F").copy()

    def item(self):
        """The first element as a host scalar (the scalar fetch behind ``sum(x)``, ``findmax(x)``, the count of
        ``findall``): one small copy into a pinned staging buffer kept per stream, then one stream synchronisation."""
        if len(self) == 0:
            raise IndexError("item() of an empty array")
        check_waits()                       # the host waits here anyway: the place to learn of a give-up
        n = self.dtype.itemsize
        key = (torch.cuda.current_device(), stream_ptr())
        pin = _staging.get(key)
        if pin is None:
            pin = _staging[key] = torch.empty(16, dtype=torch.uint8, pin_memory=True)
        pin[:n].copy_(self.buf[self.offset:self.offset + n], non_blocking=True)
        torch.cuda.current_stream().synchronize()
        return pin.numpy()[:n].view(self.dtype)[0].copy()

    # -- wrappers that keep the storage ----------------------------------------------------------
    def reshape(self, *dims):
        if len(dims) == 1 and isinstance(dims[0], (tuple, list)):
            dims = tuple(dims[0])
        if int(np.prod(dims, dtype=np.int64)) != len(self):
            raise L.DimensionMismatch(L.RK_ERR_DIMENSION, "reshape")
        return ROCArray(buf=self.buf, dims=dims, dtype=self.dtype, offset=self.offset)

    def view_range(self, first: int, last: int):
        """``view(x, first:last)`` of a vector (1-based, inclusive): contiguous, possibly unaligned."""
        if self.ndim != 1 or not (1 <= first and last <= self.dims[0]):
            raise IndexError("view_range needs a vector and an in-bounds range")
        return ROCArray(buf=self.buf, dims=(max(last - first + 1, 0),), dtype=self.dtype,
                        offset=self.offset + (first - 1) * self.dtype.itemsize)

    def copy(self):
        out = similar(self)
        n = len(self) * self.dtype.itemsize
        out.buf[:n].copy_(self.buf[self.offset:self.offset + n])
        return out


def similar(x: ROCArray, dtype=None, dims=None) -> ROCArray:
    """``similar(x, T, dims)`` (src/broadcast.jl:26-30 for broadcast outputs)."""
    return ROCArray(dims=x.dims if dims is None else dims, dtype=x.dtype if dtype is None else dtype)


def zeros(dtype, *dims) -> ROCArray:
    out = ROCArray(dims=dims, dtype=dtype)
    out.buf.zero_()
    return out


def Array(x) -> np.ndarray:
    """``Array(x)`` of a ROCArray, or of a strided wrapper (copied to a dense array on the device first)."""
    if not isinstance(x, ROCArray):
        from .views import copy
        x = copy(x)
    return x.to_host()


# ---- per-(device, stream) workspace: the analogue of the reference's per-task library state --------
_workspaces: dict = {}
_retired: list = []


def workspace(min_bytes: int = 0):
    """(pointer, bytes) of the initialised workspace bound to the current device and stream.

    A workspace that is too small is replaced by one of at least twice its size.  The outgrown buffers stay
    allocated -- a prepared launch or a captured graph may hold their address -- which costs less than the size of
    the live one in total, since sizes double.  No growth happens on a stream that is being captured: the
    allocation would not belong to the graph's memory.  Run the call once before the capture (as a warm-up
    does anyway) or ask for the size up front with ``workspace(rk_workspace_bytes(...))``.
    """
    key = (torch.cuda.current_device(), stream_ptr())
    need = max(int(min_bytes), 16 << 20)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        if torch.cuda.is_current_stream_capturing():
            raise L.RKError(L.RK_ERR_WORKSPACE, f"workspace of {need} bytes requested while the stream is being captured; "
                            "run the call once before the capture")
        size = max(need, 2 * ws.numel() if ws is not None else 0)
        if ws is not None:
            _retired.append(ws)
        ws = torch.empty(size, dtype=torch.uint8, device=device())
        assert ws.data_ptr() % 256 == 0
        L.check(L.lib.rk_workspace_init(ws.data_ptr(), ws.numel(), stream_ptr()), "rk_workspace_init")
        _workspaces[key] = ws
    return ws.data_ptr(), ws.numel()


# ---- give-ups of bounded waits -------------------------------------------------------------------------
# The single-pass scans, the one-pass findall and the small sorts wait on other workgroups with a budget; a kernel that
# runs out of it records that in the workspace (the sort: in its temporary) and finishes with meaningless results.
# The mirror reads those records where it synchronises anyway -- Array(x), item() -- for every workspace and sort
# temporary that such a kernel has used on the current stream since the last look, and raises.
_staging: dict = {}            # (device, stream) -> pinned bytes for scalar fetches (item())
_waiting: set = set()          # (device, stream) keys whose workspace has been handed to a kernel with bounded waits
_sort_tmps: dict = {}          # (device, stream) -> temporaries of sorts whose record has not been read


def note_waiting_call() -> None:
    """The call being issued on the current stream polls other workgroups through the stream's workspace."""
    _waiting.add((torch.cuda.current_device(), stream_ptr()))


def note_sort(tmp: "torch.Tensor") -> None:
    """Keeps a sort's temporary until its record has been read (instead of freeing it at once)."""
    pending = _sort_tmps.setdefault((torch.cuda.current_device(), stream_ptr()), [])
    pending.append(tmp)
    if len(pending) > 16:                   # a long run of sorts without a fetch: read the records rather than hoard memory
        check_waits()


def check_waits() -> None:
    """Reads the give-up records of the current stream (synchronises it when there are any to read); raises
    ``WaitError`` after preparing the workspace again."""
    if torch.cuda.is_current_stream_capturing():
        return
    key = (torch.cuda.current_device(), stream_ptr())
    failed = None
    if key in _waiting:
        _waiting.discard(key)
        ws = _workspaces.get(key)
        if ws is not None:
            st = L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr())
            if st == L.RK_ERR_WAIT:
                L.check(L.lib.rk_workspace_init(ws.data_ptr(), ws.numel(), stream_ptr()), "rk_workspace_init")
                failed = "a scan or findall on this stream"
            elif st != L.RK_SUCCESS:
                L.check(st, "rk_workspace_status")
    for tmp in _sort_tmps.pop(key, ()):
        st = L.lib.rk_sort_status(tmp.data_ptr(), tmp.numel(), stream_ptr())
        if st == L.RK_ERR_WAIT:
            failed = "a sort on this stream"
        elif st != L.RK_SUCCESS:
            L.check(st, "rk_sort_status")
    if failed is not None:
        raise L.WaitError(L.RK_ERR_WAIT, failed)
