"""ctypes loader for libmccnn_hip.so and helpers to pass torch tensors through
its C ABI (include/mccnn_hip.h).  There is no fallback: if the library is not
built, or a tensor is not a contiguous GPU tensor of the right dtype, the call
raises."""
import ctypes
import os
import threading
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
# MCCNN_HIP_LIBRARY selects another build of the same library (e.g. an experiment).
LIB_PATH = os.environ.get("MCCNN_HIP_LIBRARY") or os.path.join(_HERE, "libmccnn_hip.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

_lib = None

i64 = ctypes.c_int64
cint = ctypes.c_int
cfloat = ctypes.c_float
csize = ctypes.c_size_t
vptr = ctypes.c_void_p


class InvalidArgumentError(ValueError):
    """Shape or attribute violation reported by an op (the reference raises
    tf.errors.InvalidArgumentError for the same conditions)."""


def build(jobs=8):
    """Compile every HIP source for gfx950 into libmccnn_hip.so (in-tree)."""
    subprocess.run(["make", "-C", CSRC_DIR, "-B", "-j%d" % jobs], check=True,
                   stdout=subprocess.DEVNULL)
    global _lib
    _lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libmccnn_hip.so is not built (expected at %s); run "
                "`make -C %s` or __graft_entry__.build()" % (LIB_PATH, CSRC_DIR))
        handle = ctypes.CDLL(LIB_PATH)
        handle.mccnn_last_error.restype = ctypes.c_char_p
        for name in ("mccnn_build_grid_workspace_bytes",
                     "mccnn_find_neighbors_workspace_bytes",
                     "mccnn_mc_basis_grads_workspace_bytes",
                     "mccnn_mc_conv_project_grads_workspace_bytes",
                     "mccnn_pair_dense_grads_workspace_bytes",
                     "mccnn_pointconv_density_grads_workspace_bytes",
                     "mccnn_reorder_neighbors_workspace_bytes",
                     "mccnn_sampling_workspace_bytes",
                     "mccnn_sort_keys_workspace_bytes",
                     "mccnn_transpose_neighbors_workspace_bytes",
                     "mccnn_weight_grad_product_workspace_bytes"):
            getattr(handle, name).restype = csize
        _lib = handle
    return _lib


def check(rc):
    if rc == 0:
        return
    msg = lib().mccnn_last_error().decode("utf-8", "replace")
    if rc == 1:
        raise InvalidArgumentError(msg)
    raise RuntimeError("HIP error in libmccnn_hip: " + msg)


def stream():
    """torch's current stream on the current device as a raw hipStream_t."""
    import torch
    try:        # the raw accessors skip the Stream object and its device bookkeeping
        return vptr(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))
    except AttributeError:
        return vptr(torch.cuda.current_stream().cuda_stream)


def ptr(t, dtype=None):
    """Device pointer of a contiguous GPU tensor (None -> NULL)."""
    if t is None:
        return vptr(0)
    if not t.is_cuda:
        raise TypeError("expected a GPU tensor, got one on %s" % t.device)
    if dtype is not None and t.dtype != dtype:
        raise TypeError("expected dtype %s, got %s" % (dtype, t.dtype))
    if not t.is_contiguous():
        raise TypeError("expected a contiguous tensor")
    return vptr(t.data_ptr())


_host_counts = threading.local()


def host_count():
    """One int64 in pinned host memory per thread: the `_count` halves of the
    dynamic-size ops copy their total there, and a device-to-host copy into pinned
    memory completes without the staging a pageable destination needs.
    -> (tensor [1], pointer)."""
    import torch
    t = getattr(_host_counts, "tensor", None)
    if t is None:
        # [0] the count; [1], [2] the two facts mccnn_find_neighbors_count_facts reports
        t = torch.zeros(4, dtype=torch.int64, pin_memory=True)
        _host_counts.tensor = t
    return t, vptr(t.data_ptr())


def workspace(nbytes, device):
    import torch
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


# ------------------------------------------------------------------ timing ----
# When a dict is installed with start_timing(), every op call made through
# region() records a pair of events on torch's current stream, the stream the
# kernels are launched on.  collect_timing() synchronises and returns, per op
# name, the list of elapsed milliseconds.

_timing = None


def start_timing():
    global _timing
    _timing = {}


class region:
    def __init__(self, name):
        self.name = name

    def __enter__(self):
        if _timing is not None:
            import torch
            self.start = torch.cuda.Event(enable_timing=True)
            self.end = torch.cuda.Event(enable_timing=True)
            self.start.record()
        return self

    def __exit__(self, *exc):
        if _timing is not None:
            self.end.record()
            _timing.setdefault(self.name, []).append((self.start, self.end))
        return False


def collect_timing():
    global _timing
    import torch
    torch.cuda.synchronize()
    out = {k: [a.elapsed_time(b) for a, b in v] for k, v in (_timing or {}).items()}
    _timing = None
    return out


def call(name, *args, timed_as=None):
    """Invoke entry point mccnn_<name>, raise on a non-zero status, and time it
    when timing is active (under `timed_as` if given)."""
    fn = getattr(lib(), "mccnn_" + name)
    with region(timed_as or name):
        check(fn(*args))
