"""ctypes binding of libgq_hip.so, the HIP (gfx950) library behind the group-quantization path.

Stands where the reference imports its JIT-compiled pybind11 module
(popxl_addons/ops/group_quantize_decompress/group_quantize_decompress.py:4-6).  There is no
CPU fallback: a missing library or a non-zero return code raises.
"""
import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
_DEFAULT_LIB = os.path.join(os.path.dirname(_PKG_DIR), "lib", "libgq_hip.so")

GQ_ABI_VERSION = 4
GQ_ERR_NULL_POINTER = -1
GQ_ERR_BAD_SHAPE = -2
GQ_ERR_MISALIGNED = -3
GQ_ERR_UNSUPPORTED = -4
GQ_ERR_NO_DEVICE = -5
GQ_ACT_NONE, GQ_ACT_RELU, GQ_ACT_GELU_TANH = 0, 1, 2
GQ_DESC_KN_LAYOUT = 0x100  # or-ed into a sequence entry's activation: weight grouped along the output features
ACTIVATIONS = {None: GQ_ACT_NONE, "none": GQ_ACT_NONE, "relu": GQ_ACT_RELU, "gelu_tanh": GQ_ACT_GELU_TANH}


def activation_code(activation):
    """GQ_ACT_* of an activation given by name (None, "relu", "gelu_tanh") or by code."""
    if isinstance(activation, int) and activation in ACTIVATIONS.values():
        return activation
    try:
        return ACTIVATIONS[activation]
    except (KeyError, TypeError):
        raise ValueError(f"unknown activation {activation!r}; expected one of {sorted(k for k in ACTIVATIONS if k)}") from None

# every symbol declared in include/gq_hip.h
EXPORTS = (
    "gq_abi_version",
    "gq_last_error",
    "gq_decompress_f16",
    "gq_decompress_f16_transposed",
    "gq_gemv_f16",
    "gq_gemm_f16",
    "gq_linear_f16",
    "gq_linear_act_f16",
    "gq_gemm_workspace_bytes",
    "gq_linear_act_ws_f16",
    "gq_linear_p_act_f16",
    "gq_linear_p_strided_f16",
    "gq_linear_kn_workspace_bytes",
    "gq_linear_kn_act_f16",
    "gq_linear_kn_act_noalloc_f16",
    "gq_gemv_sequence_f16",
    "gq_gemv_sequence_workspace_bytes",
    "gq_gemv_sequence_ws_f16",
    "gq_gemv_prepacked_bytes",
    "gq_gemv_prepack_f16",
    "gq_gemv_kn_prepacked_bytes",
    "gq_gemv_kn_prepack_f16",
    "gq_linear_knp_act_f16",
    "gq_linear_knp_strided_f16",
    "gq_compress_f16",
    "gq_compress_f32",
)


class GQHipError(RuntimeError):
    """A libgq_hip entry point returned a non-zero code."""

    def __init__(self, function, code, message):
        super().__init__(f"{function} failed with code {code}: {message}")
        self.function = function
        self.code = code


_lib = None


def library_path():
    return os.environ.get("GQ_HIP_LIBRARY", _DEFAULT_LIB)


def load():
    """Load the shared library once; raise if it is not built (python popxl-addons_amd/build.py)."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise ImportError(
            f"libgq_hip.so not found at {path}: build it with `python popxl-addons_amd/build.py` "
            "(there is no CPU fallback for the device ops)"
        )
    lib = ctypes.CDLL(path)
    p, i64 = ctypes.c_void_p, ctypes.c_int64
    lib.gq_abi_version.argtypes = []
    lib.gq_abi_version.restype = ctypes.c_int
    lib.gq_last_error.argtypes = []
    lib.gq_last_error.restype = ctypes.c_char_p
    for name in ("gq_decompress_f16", "gq_decompress_f16_transposed"):
        fn = getattr(lib, name)
        fn.argtypes = [p, p, p, p, i64, i64, i64, p]
        fn.restype = ctypes.c_int
    for name in ("gq_gemv_f16", "gq_gemm_f16", "gq_linear_f16"):
        fn = getattr(lib, name)
        fn.argtypes = [p, i64, p, p, p, p, p, i64, i64, i64, p]
        fn.restype = ctypes.c_int
    lib.gq_linear_act_f16.argtypes = [p, i64, p, p, p, p, p, i64, i64, i64, ctypes.c_int32, p]
    lib.gq_linear_act_f16.restype = ctypes.c_int
    lib.gq_gemm_workspace_bytes.argtypes = [i64, i64, i64, i64]
    lib.gq_gemm_workspace_bytes.restype = i64
    lib.gq_linear_act_ws_f16.argtypes = [p, i64, p, p, p, p, p, i64, i64, i64, ctypes.c_int32, p, i64, p]
    lib.gq_linear_act_ws_f16.restype = ctypes.c_int
    lib.gq_linear_p_act_f16.argtypes = [p, i64, p, p, p, p, p, p, i64, i64, i64, ctypes.c_int32, p, i64, p]
    lib.gq_linear_p_act_f16.restype = ctypes.c_int
    lib.gq_linear_p_strided_f16.argtypes = [p, i64, i64, p, p, p, p, p, p, i64, i64, i64, ctypes.c_int32, p]
    lib.gq_linear_p_strided_f16.restype = ctypes.c_int
    lib.gq_linear_kn_workspace_bytes.argtypes = [i64, i64, i64, i64]
    lib.gq_linear_kn_workspace_bytes.restype = i64
    lib.gq_linear_kn_act_f16.argtypes = [p, i64, p, p, p, p, p, i64, i64, i64, ctypes.c_int32, p, i64, p]
    lib.gq_linear_kn_act_f16.restype = ctypes.c_int
    lib.gq_linear_kn_act_noalloc_f16.argtypes = [p, i64, p, p, p, p, p, i64, i64, i64, ctypes.c_int32, p]
    lib.gq_linear_kn_act_noalloc_f16.restype = ctypes.c_int
    lib.gq_gemv_sequence_f16.argtypes = [p, p, i64, p, p]
    lib.gq_gemv_sequence_f16.restype = ctypes.c_int
    lib.gq_gemv_sequence_workspace_bytes.argtypes = []
    lib.gq_gemv_sequence_workspace_bytes.restype = i64
    lib.gq_gemv_sequence_ws_f16.argtypes = [p, p, i64, p, p, i64, i64, p]
    lib.gq_gemv_sequence_ws_f16.restype = ctypes.c_int
    lib.gq_gemv_prepacked_bytes.argtypes = [i64, i64, i64]
    lib.gq_gemv_prepacked_bytes.restype = i64
    lib.gq_gemv_prepack_f16.argtypes = [p, p, p, p, i64, i64, i64, p]
    lib.gq_gemv_prepack_f16.restype = ctypes.c_int
    lib.gq_gemv_kn_prepacked_bytes.argtypes = [i64, i64, i64]
    lib.gq_gemv_kn_prepacked_bytes.restype = i64
    lib.gq_gemv_kn_prepack_f16.argtypes = [p, p, p, p, i64, i64, i64, p]
    lib.gq_gemv_kn_prepack_f16.restype = ctypes.c_int
    lib.gq_linear_knp_act_f16.argtypes = [p, i64, p, p, p, i64, i64, i64, ctypes.c_int32, p]
    lib.gq_linear_knp_act_f16.restype = ctypes.c_int
    lib.gq_linear_knp_strided_f16.argtypes = [p, i64, i64, p, p, p, i64, i64, i64, ctypes.c_int32, p]
    lib.gq_linear_knp_strided_f16.restype = ctypes.c_int
    for name in ("gq_compress_f16", "gq_compress_f32"):
        fn = getattr(lib, name)
        fn.argtypes = [p, p, p, p, p, i64, i64, i64, p]
        fn.restype = ctypes.c_int
    if lib.gq_abi_version() != GQ_ABI_VERSION:
        raise ImportError(f"{path}: ABI version {lib.gq_abi_version()} != expected {GQ_ABI_VERSION}")
    _lib = lib
    return lib


def last_error():
    return load().gq_last_error().decode("utf-8", "replace")


def call(name, *args):
    """Call an entry point; raise GQHipError on a non-zero return."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise GQHipError(name, rc, lib.gq_last_error().decode("utf-8", "replace"))


_kn_workspaces = {}


def linear_kn_workspace(device, nbytes):
    """The scratch buffer of gq_linear_kn_act_f16 and gq_linear_act_ws_f16 for calls enqueued on the
    CURRENT stream of `device`: one buffer per (device, stream), grown on demand; its arrival counters
    start at zero and every call leaves them zero.  Calls that share a buffer are on the same stream
    and therefore ordered; layers built on different streams get different buffers and may overlap."""
    import torch

    device = torch.device(device)
    if device.index is None:
        device = torch.device(device.type, torch.cuda.current_device())
    key = (device, torch.cuda.current_stream(device).cuda_stream)
    ws = _kn_workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        with torch.cuda.device(device):
            # (a buffer that is being replaced stays alive until the work enqueued on it has run:
            # the caching allocator hands its memory out again on the same stream only)
            ws = torch.zeros(max(int(nbytes), 1 << 20), dtype=torch.uint8, device=device)
        _kn_workspaces[key] = ws
    return ws


class PrepackedWeight:
    """One weight in a streaming layout: a device blob derived from the three LinearGQ variables.
    layout "nk": groups along the input features (LinearGQ dim=0), made by prepack_gemv(), read by
    GemvSequence entries and, beside the variables, by gq_linear_p_act_f16's GEMM kernel; layout "kn":
    groups along the output features (dim=-1 / 1, the
    default), made by prepack_gemv_kn(), read by GemvSequence entries and by linear_knp()."""

    def __init__(self, blob, n_out, k_in, group_size, layout="nk"):
        self.blob, self.n_out, self.k_in, self.group_size, self.layout = blob, n_out, k_in, group_size, layout


def prepack_gemv(packed, scale, bias):
    """packed uint16 [n_out, G, I], scale / bias float16 [n_out, G, 1] on the GPU -> PrepackedWeight."""
    import torch

    n_out, n_groups, n_ids = packed.shape
    k_in, group_size = n_groups * n_ids * 4, n_ids * 4
    for t in (packed, scale, bias):
        assert t.is_cuda and t.is_contiguous()
    lib = load()
    nbytes = lib.gq_gemv_prepacked_bytes(n_out, k_in, group_size)
    if nbytes < 0:
        raise GQHipError("gq_gemv_prepacked_bytes", nbytes, lib.gq_last_error().decode("utf-8", "replace"))
    with torch.cuda.device(packed.device):
        blob = torch.empty(nbytes, dtype=torch.uint8, device=packed.device)
        call("gq_gemv_prepack_f16", packed.data_ptr(), scale.data_ptr(), bias.data_ptr(), blob.data_ptr(), n_out, k_in,
             group_size, torch.cuda.current_stream(packed.device).cuda_stream)
    return PrepackedWeight(blob, n_out, k_in, group_size)


def prepack_gemv_kn(packed, scale, bias):
    """The variables of a layer grouped along the OUTPUT features -- packed uint16 [k_in, n_out / 64, 16],
    scale / bias float16 [k_in, n_out / 64, 1] on the GPU -> PrepackedWeight in the kn streaming layout."""
    import torch

    k_in, n_groups, n_ids = packed.shape
    n_out, group_size = n_groups * n_ids * 4, n_ids * 4
    for t in (packed, scale, bias):
        assert t.is_cuda and t.is_contiguous()
    lib = load()
    nbytes = lib.gq_gemv_kn_prepacked_bytes(n_out, k_in, group_size)
    if nbytes < 0:
        raise GQHipError("gq_gemv_kn_prepacked_bytes", nbytes, lib.gq_last_error().decode("utf-8", "replace"))
    with torch.cuda.device(packed.device):
        blob = torch.empty(nbytes, dtype=torch.uint8, device=packed.device)
        call("gq_gemv_kn_prepack_f16", packed.data_ptr(), scale.data_ptr(), bias.data_ptr(), blob.data_ptr(), n_out, k_in,
             group_size, torch.cuda.current_stream(packed.device).cuda_stream)
    return PrepackedWeight(blob, n_out, k_in, group_size, layout="kn")


def linear_knp(x, weight, out_bias=None, activation=None, y=None):
    """y = act(x @ w + out_bias) for x float16 [m_rows, k_in] on the GPU and a PrepackedWeight in the kn
    streaming layout (gq_linear_knp_act_f16: the decode kernel up to 16 rows, the MFMA pipeline above).
    A decode batch (up to 16 rows) may be a column slice of a wider matrix -- unit stride along the features,
    rows a multiple of 8 elements apart: it is read where it lies (gq_linear_knp_strided_f16)."""
    import torch

    assert weight.layout == "kn" and x.is_cuda and x.dim() == 2 and x.shape[-1] == weight.k_in
    m_rows = x.shape[0]
    strided = not x.is_contiguous()
    assert not strided or (x.stride(1) == 1 and x.stride(0) >= weight.k_in and x.stride(0) % 8 == 0 and m_rows <= 16)
    with torch.cuda.device(x.device):
        if y is None:
            y = torch.empty((m_rows, weight.n_out), dtype=torch.float16, device=x.device)
        tail = (weight.blob.data_ptr(), 0 if out_bias is None else out_bias.data_ptr(), y.data_ptr(), weight.n_out, weight.k_in,
                weight.group_size, activation_code(activation), torch.cuda.current_stream(x.device).cuda_stream)
        if strided:
            call("gq_linear_knp_strided_f16", x.data_ptr(), x.stride(0), m_rows, *tail)
        else:
            call("gq_linear_knp_act_f16", x.data_ptr(), m_rows, *tail)
    return y


class GemvSequence:
    """A list of decode GEMVs run by one `gq_gemv_sequence_f16` call (see include/gq_hip.h).

    add(x, packed, scale, bias, y, out_bias=None, wait_previous=False, wait_for=None, activation=None) appends an
    entry from torch tensors on the GPU (kept alive by this object) and returns its index; the entry
    starts after every earlier entry (wait_previous) or after entries 0..wait_for have completed.
    run() enqueues the whole list on the current stream.  `status` is a device int32 the kernel
    sets to 1 if it gave up waiting (some workgroup of the persistent kernel was not resident:
    another kernel held compute units); the results of that run are then invalid.  A give-up does
    not pass silently: run() raises GQHipError as soon as it finds that an earlier run() of this
    object ended that way (it looks at a host copy of `status` that earlier runs left behind, without
    waiting for the GPU), and check() waits for the GPU and raises for every run so far.  After the
    error has been raised once the object is usable again.
    """

    def __init__(self, device, own_workspace=False, spin_limit=0):
        """own_workspace: keep the kernel's progress words in a buffer of this object
        (gq_gemv_sequence_ws_f16) instead of the block the library holds per device.  Sequences
        with buffers of their own may be enqueued on different streams, but the caller must still
        ORDER them (events): each persistent kernel needs every compute unit, and two that really
        overlap give up (status 1).  Without it, all sequences of a device share the library's block
        and must be enqueued on one stream (the library refuses a second stream while the first is
        busy).  spin_limit: polls without progress after which a wait gives up (0: the library's
        default)."""
        import numpy as np

        self.device = device
        self.own_workspace = own_workspace or spin_limit > 0
        self.spin_limit = int(spin_limit)
        self._workspace = None
        self.dtype = np.dtype(
            [("x", "<u8"), ("packed", "<u8"), ("scale", "<u8"), ("bias", "<u8"), ("out_bias", "<u8"), ("y", "<u8"),
             ("m_rows", "<i4"), ("n_out", "<i4"), ("k_in", "<i4"), ("group_size", "<i4"), ("wait_entries", "<i4"),
             ("activation", "<i4")]
        )
        assert self.dtype.itemsize == 72  # sizeof(gq_gemv_desc)
        self.entries = []
        self.keep = []
        self._host = None
        self._dev = None
        self.status = None
        self._status_host = None   # pinned int32: the last copy of `status` that reached the host
        self._status_event = None  # recorded behind that copy; None: no copy under way

    def add(self, x, packed, scale, bias, y, out_bias=None, wait_previous=False, wait_for=None, activation=None):
        """`packed` may be a PrepackedWeight of either layout (then scale and bias are None)."""
        m_rows, k_in = x.shape
        layout_flag = 0
        if isinstance(packed, PrepackedWeight):
            assert scale is None and bias is None and packed.k_in == k_in
            n_out, group_size = packed.n_out, packed.group_size
            pointers = (packed.blob.data_ptr(), 0, 0)
            tensors = (x, packed.blob, y)
            layout_flag = GQ_DESC_KN_LAYOUT if packed.layout == "kn" else 0
        else:
            n_out, n_groups, n_ids = packed.shape
            assert n_groups * n_ids * 4 == k_in
            group_size = n_ids * 4
            pointers = (packed.data_ptr(), scale.data_ptr(), bias.data_ptr())
            tensors = (x, packed, scale, bias, y)
        assert y.shape == (m_rows, n_out)
        for t in tensors:
            assert t.is_cuda and t.is_contiguous()
        index = len(self.entries)
        wait_entries = index if wait_previous else (0 if wait_for is None else int(wait_for) + 1)
        if not 0 <= wait_entries <= index:
            raise ValueError(f"entry {index} cannot wait for entry {wait_for}")
        self.entries.append(
            (x.data_ptr(), *pointers,
             0 if out_bias is None else out_bias.data_ptr(), y.data_ptr(), m_rows, n_out, k_in, group_size,
             wait_entries, activation_code(activation) | layout_flag)
        )
        self.keep.append((x, packed, scale, bias, y, out_bias))
        self._host = None
        return index

    def _finalise(self):
        import numpy as np
        import torch

        self._host = np.array(self.entries, dtype=self.dtype)
        self._dev = torch.from_numpy(self._host.view(np.uint8).copy()).to(self.device)
        self.status = torch.zeros(1, dtype=torch.int32, device=self.device)
        self._status_host = torch.zeros(1, dtype=torch.int32, pin_memory=True)
        self._status_event = None
        if self.own_workspace and self._workspace is None:
            self._workspace = torch.zeros(load().gq_gemv_sequence_workspace_bytes(), dtype=torch.uint8, device=self.device)

    def run(self):
        import torch

        if self._host is None:
            self._finalise()
        capturing = torch.cuda.is_current_stream_capturing()
        if not capturing:
            self._raise_if_gave_up(wait=False)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        if self.own_workspace:
            call("gq_gemv_sequence_ws_f16", self._host.ctypes.data, self._dev.data_ptr(), len(self.entries),
                 self.status.data_ptr(), self._workspace.data_ptr(), self._workspace.numel(), self.spin_limit, stream)
        else:
            call("gq_gemv_sequence_f16", self._host.ctypes.data, self._dev.data_ptr(), len(self.entries),
                 self.status.data_ptr(), stream)
        # `status` only ever goes from 0 to 1 on the device, so any later copy also tells of this run.  One
        # copy at a time: a loop that enqueues runs faster than the GPU executes them adds no copies.
        if not capturing and self._status_event is None:
            self._status_host.copy_(self.status, non_blocking=True)
            self._status_event = torch.cuda.Event()
            self._status_event.record(torch.cuda.current_stream(self.device))

    _GAVE_UP = ("a wait for earlier entries gave up, the results of that run are invalid: some workgroup was not "
                "resident (is another kernel occupying the compute units?)")

    def _raise_if_gave_up(self, wait):
        import torch

        if self.status is None:
            return
        if wait:
            torch.cuda.synchronize(self.device)
            gave_up = int(self.status.item()) != 0
            self._status_event = None
        else:
            if self._status_event is None or not self._status_event.query():
                return
            self._status_event = None
            gave_up = int(self._status_host[0]) != 0
        if gave_up:
            torch.cuda.synchronize(self.device)
            self.status.zero_()
            self._status_host.zero_()
            torch.cuda.synchronize(self.device)
            raise GQHipError("gq_gemv_sequence_f16", 1, self._GAVE_UP)

    def check(self):
        """Wait for the GPU and raise if a wait of any run() so far gave up (results are then invalid)."""
        self._raise_if_gave_up(wait=True)
