"""Thin ctypes binding of libbitsknn.so (the C ABI declared in include/bitsknn.h).

Used by the parity tests and the benchmark to call the HIP kernels on torch-allocated device
memory.  torch is plumbing here (device buffers, the current stream); every computation goes
through the C ABI.  There is no CPU fallback: a missing library raises ImportError-like
RuntimeError on first use, and every non-zero status raises BitsKnnError with the library's
message.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "libbitsknn.so")

OK, ERR_UNSUPPORTED, ERR_INVALID, ERR_HIP, ERR_INTERNAL = 0, 1, 2, 3, 4
DIST_L2, DIST_PARTIAL_L2, DIST_EXPANDED, DIST_PARTIAL_L2_BF16X3 = 0, 1, 2, 3

# every symbol include/bitsknn.h declares
EXPORTS = (
    "bitsknn_last_error",
    "bitsknn_version",
    "bitsknn_topk_bits_f32",
    "bitsknn_topk_bits_parts_f32",
    "bitsknn_topk_partial_bitonic_f32",
    "bitsknn_label_offsets",
    "bitsknn_fill_f32",
    "bitsknn_stream_read_f32",
    "bitsknn_dist_f32",
    "bitsknn_dist_layout_workspace_bytes",
    "bitsknn_dist_layout_f32",
    "bitsknn_fused_l2_topk_f32",
    "bitsknn_fused_workspace_bytes",
    "bitsknn_fused_image_bytes",
    "bitsknn_fused_l2_topk_f32_ws",
    "bitsknn_fused_l2_topk_f32_ex",
    "bitsknn_fused_l2_topk_f32_tuned",
    "bitsknn_fused_static_scratch_bytes",
    "bitsknn_fused_l2_topk_f32_static",
    "bitsknn_fused_status",
)


class FusedTuning(ctypes.Structure):
    """bitsknn_fused_tuning of include/bitsknn.h"""
    _fields_ = [("ranges", ctypes.c_int32), ("first_radius", ctypes.c_int32), ("image", ctypes.c_int32),
                ("workgroup", ctypes.c_int32), ("reserved", ctypes.c_int32 * 4)]


class BitsKnnError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(message)
        self.code = code


_lib = None


def lib():
    """Load libbitsknn.so (built in-tree by `make -C bits-knn-jpdc2024_amd lib`)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.dirname(_HERE)} lib` "
                "(there is no fallback path)")
        # torch bundles its own HIP runtime under the same soname as the system one; it has to be
        # loaded first so that this library binds to the runtime that owns torch's device memory
        # and streams instead of bringing up a second runtime in the process
        import torch  # noqa: F401
        L = ctypes.CDLL(LIB_PATH)
        vp, sz, i32, u32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int32, ctypes.c_uint32
        L.bitsknn_last_error.restype = ctypes.c_char_p
        L.bitsknn_last_error.argtypes = []
        L.bitsknn_version.restype = ctypes.c_char_p
        L.bitsknn_version.argtypes = []
        L.bitsknn_topk_bits_f32.restype = ctypes.c_int
        L.bitsknn_topk_bits_f32.argtypes = [vp, sz, vp, sz, vp, sz, sz, vp, vp, sz, u32, u32, u32,
                                            ctypes.c_int, vp]
        L.bitsknn_topk_bits_parts_f32.restype = ctypes.c_int
        L.bitsknn_topk_bits_parts_f32.argtypes = [vp, sz, sz, u32, vp, vp, vp, vp, vp, sz, u32, u32, u32, vp]
        L.bitsknn_topk_partial_bitonic_f32.restype = ctypes.c_int
        L.bitsknn_topk_partial_bitonic_f32.argtypes = [vp, sz, sz, sz, vp, vp, sz, u32, u32, vp]
        L.bitsknn_label_offsets.restype = ctypes.c_int
        L.bitsknn_label_offsets.argtypes = [vp, sz, sz, sz, vp]
        L.bitsknn_fill_f32.restype = ctypes.c_int
        L.bitsknn_fill_f32.argtypes = [vp, sz, ctypes.c_float, vp]
        L.bitsknn_stream_read_f32.restype = ctypes.c_int
        L.bitsknn_stream_read_f32.argtypes = [vp, sz, sz, sz, vp, vp]
        L.bitsknn_dist_f32.restype = ctypes.c_int
        L.bitsknn_dist_f32.argtypes = [ctypes.c_int, ctypes.c_int, sz, sz, vp, sz, vp, sz, vp, sz, vp]
        L.bitsknn_dist_layout_workspace_bytes.restype = ctypes.c_size_t
        L.bitsknn_dist_layout_workspace_bytes.argtypes = [ctypes.c_int, sz, sz, ctypes.c_int, ctypes.c_int]
        L.bitsknn_dist_layout_f32.restype = ctypes.c_int
        L.bitsknn_dist_layout_f32.argtypes = [ctypes.c_int, ctypes.c_int, sz, sz, vp, ctypes.c_int, sz, vp,
                                              ctypes.c_int, sz, vp, sz, vp, sz, vp]
        L.bitsknn_fused_l2_topk_f32.restype = ctypes.c_int
        L.bitsknn_fused_l2_topk_f32.argtypes = [vp, vp, ctypes.c_int, i32, i32, vp, vp, ctypes.c_int,
                                                ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                ctypes.c_int, ctypes.c_int, vp]
        L.bitsknn_fused_l2_topk_f32_ex.restype = ctypes.c_int
        L.bitsknn_fused_l2_topk_f32_ex.argtypes = [vp, vp, ctypes.c_int, i32, i32, vp, vp, ctypes.c_int,
                                                   ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                   ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, sz, vp]
        L.bitsknn_fused_workspace_bytes.restype = ctypes.c_size_t
        L.bitsknn_fused_workspace_bytes.argtypes = [i32, i32, ctypes.c_int]
        L.bitsknn_fused_image_bytes.restype = ctypes.c_size_t
        L.bitsknn_fused_image_bytes.argtypes = [ctypes.c_int, i32]
        L.bitsknn_fused_l2_topk_f32_ws.restype = ctypes.c_int
        L.bitsknn_fused_l2_topk_f32_ws.argtypes = [vp, vp, ctypes.c_int, i32, i32, vp, vp, ctypes.c_int,
                                                   ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                   ctypes.c_int, ctypes.c_int, vp, sz, vp]
        L.bitsknn_fused_static_scratch_bytes.restype = ctypes.c_size_t
        L.bitsknn_fused_static_scratch_bytes.argtypes = []
        L.bitsknn_fused_l2_topk_f32_static.restype = ctypes.c_int
        L.bitsknn_fused_l2_topk_f32_static.argtypes = L.bitsknn_fused_l2_topk_f32.argtypes
        L.bitsknn_fused_l2_topk_f32_tuned.restype = ctypes.c_int
        L.bitsknn_fused_l2_topk_f32_tuned.argtypes = [vp, vp, ctypes.c_int, i32, i32, vp, vp, ctypes.c_int,
                                                      ctypes.c_int, ctypes.POINTER(FusedTuning), vp, sz, vp]
        L.bitsknn_fused_status.restype = ctypes.c_int
        L.bitsknn_fused_status.argtypes = [vp]
        _lib = L
    return _lib


def _check(status):
    if status != OK:
        raise BitsKnnError(status, lib().bitsknn_last_error().decode())


def _stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _row_stride(t):
    # torch reports arbitrary strides for dimensions of extent 1
    rows, cols = t.shape
    return max(t.stride(0), cols) if rows > 1 else cols


def version():
    return lib().bitsknn_version().decode()


def topk_bits(dist, k, block_size=256, items_per_thread=16, prefetch=False, in_label=None,
              label_offsets=None, out_dist=None, out_label=None):
    """bits top-k of every row of a 2-D float32 device tensor (last dim contiguous).
    Returns (values, labels), each rows x k."""
    import torch
    assert dist.is_cuda and dist.dtype == torch.float32 and dist.dim() == 2
    assert dist.shape[1] == 1 or dist.stride(1) == 1
    rows, cols = dist.shape
    if out_dist is None:
        out_dist = torch.empty((rows, k), dtype=torch.float32, device=dist.device)
    if out_label is None:
        out_label = torch.empty((rows, k), dtype=torch.int32, device=dist.device)
    label_stride = 0
    if in_label is not None:
        assert in_label.dtype == torch.int32 and in_label.shape == dist.shape and (cols == 1 or in_label.stride(1) == 1)
        label_stride = _row_stride(in_label)
    if label_offsets is not None:
        assert label_offsets.dtype == torch.int32 and label_offsets.numel() == rows
    _check(lib().bitsknn_topk_bits_f32(_ptr(dist), _row_stride(dist),
                                       _ptr(in_label), label_stride, _ptr(label_offsets), rows, cols,
                                       _ptr(out_dist), _ptr(out_label), _row_stride(out_dist), k,
                                       block_size, items_per_thread, 1 if prefetch else 0, _stream()))
    return out_dist, out_label


def topk_bits_parts(dist, k, parts, block_size=256, items_per_thread=16, scratch=None, out_dist=None,
                    out_label=None):
    """bits-sq: bits top-k of every row of a contiguous 2-D float32 device tensor with the rows cut
    into `parts` parts (bitsknn_topk_bits_parts_f32).  scratch: a dict that keeps the device memory
    for the parts' results and the counters between calls.  Returns (values, labels), rows x k."""
    import torch
    assert dist.is_cuda and dist.dtype == torch.float32 and dist.dim() == 2 and dist.is_contiguous()
    rows, cols = dist.shape
    if out_dist is None:
        out_dist = torch.empty((rows, k), dtype=torch.float32, device=dist.device)
    if out_label is None:
        out_label = torch.empty((rows, k), dtype=torch.int32, device=dist.device)
    key = (rows, parts, k, str(dist.device))
    scratch = scratch if scratch is not None else {}
    if key not in scratch:
        scratch[key] = (torch.empty(rows * parts * k, dtype=torch.float32, device=dist.device),
                        torch.empty(rows * parts * k, dtype=torch.int32, device=dist.device),
                        torch.zeros(rows, dtype=torch.int32, device=dist.device))
    part_d, part_l, counters = scratch[key]
    _check(lib().bitsknn_topk_bits_parts_f32(_ptr(dist), rows, cols, parts, _ptr(part_d), _ptr(part_l),
                                             _ptr(counters), _ptr(out_dist), _ptr(out_label),
                                             _row_stride(out_dist), k, block_size, items_per_thread, _stream()))
    return out_dist, out_label


def topk_partial_bitonic(dist, k, block_size=256, out_dist=None, out_label=None):
    """partial-bitonic-regs top-k (no filtering) of every row of a 2-D float32 device tensor."""
    import torch
    assert dist.is_cuda and dist.dtype == torch.float32 and dist.dim() == 2
    assert dist.shape[1] == 1 or dist.stride(1) == 1
    rows, cols = dist.shape
    if out_dist is None:
        out_dist = torch.empty((rows, k), dtype=torch.float32, device=dist.device)
    if out_label is None:
        out_label = torch.empty((rows, k), dtype=torch.int32, device=dist.device)
    _check(lib().bitsknn_topk_partial_bitonic_f32(_ptr(dist), _row_stride(dist), rows, cols,
                                                  _ptr(out_dist), _ptr(out_label),
                                                  _row_stride(out_dist), k, block_size, _stream()))
    return out_dist, out_label


def label_offsets(rows, parts, cols_per_part, device="cuda"):
    import torch
    out = torch.empty(rows * parts, dtype=torch.int32, device=device)
    _check(lib().bitsknn_label_offsets(_ptr(out), rows, parts, cols_per_part, _stream()))
    return out


def fill(t, value):
    _check(lib().bitsknn_fill_f32(_ptr(t), t.numel(), float(value), _stream()))
    return t


def stream_read(matrix, out=None):
    """Row minima by a plain streaming read (calibration of the achievable read rate)."""
    import torch
    rows, cols = matrix.shape
    if out is None:
        out = torch.empty(rows, dtype=torch.float32, device=matrix.device)
    _check(lib().bitsknn_stream_read_f32(_ptr(matrix), _row_stride(matrix), rows, cols, _ptr(out), _stream()))
    return out


def distances(queries_dm, points_dm, op=DIST_L2, out=None):
    """Distance matrix q x n from dim-major inputs (d x q and d x n float32 device tensors)."""
    import torch
    d, q = queries_dm.shape
    d2, n = points_dm.shape
    assert d == d2 and (q == 1 or queries_dm.stride(1) == 1) and (n == 1 or points_dm.stride(1) == 1)
    if out is None:
        out = torch.empty((q, n), dtype=torch.float32, device=queries_dm.device)
    _check(lib().bitsknn_dist_f32(op, d, q, n, _ptr(queries_dm), _row_stride(queries_dm),
                                  _ptr(points_dm), _row_stride(points_dm), _ptr(out),
                                  _row_stride(out), _stream()))
    return out


LAYOUT_ROW_MAJOR, LAYOUT_COLUMN_MAJOR = 0, 1


def distances_layout(queries, queries_layout, points, points_layout, op=DIST_L2, out=None):
    """Distance matrix q x n from 2-D float32 device tensors in the caller's layout: LAYOUT_ROW_MAJOR
    (count x dim, the vectors one after the other) or LAYOUT_COLUMN_MAJOR (dim x count)."""
    import torch
    q, d = queries.shape if queries_layout == LAYOUT_ROW_MAJOR else queries.shape[::-1]
    n, d2 = points.shape if points_layout == LAYOUT_ROW_MAJOR else points.shape[::-1]
    assert d == d2
    if out is None:
        out = torch.empty((q, n), dtype=torch.float32, device=queries.device)
    need = int(lib().bitsknn_dist_layout_workspace_bytes(d, q, n, queries_layout, points_layout))
    workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=queries.device)
    _check(lib().bitsknn_dist_layout_f32(op, d, q, n, _ptr(queries), queries_layout, _row_stride(queries),
                                         _ptr(points), points_layout, _row_stride(points), _ptr(out),
                                         _row_stride(out), _ptr(workspace), need, _stream()))
    return out


FUSED_FP32, FUSED_BF16X3, FUSED_EXACT = 0, 1, 2


def fused_l2_topk(queries_dm, points_dm, k, params=(8, 4, 2), block_query_dim=1, dim_mult=1,
                  out_dist=None, out_label=None, workspace=None, arithmetic=None, tuning=None):
    """bits-fused: top-k of ||p||^2 - 2 q.p without materialising the distance matrix.
    workspace: None -> the plain entry point; "auto" -> allocate what
    bitsknn_fused_workspace_bytes asks for; "image" -> that plus room for the stage image
    (fused_workspace_with_image_bytes); "static" -> the entry point that uses the library's own
    scratch memory and allocates nothing; or a uint8 device tensor.
    arithmetic: None -> the plain entry points (FUSED_EXACT); FUSED_FP32 / FUSED_BF16X3 /
    FUSED_EXACT -> bitsknn_fused_l2_topk_f32_ex with that arithmetic.
    tuning: None, or (ranges, first_radius[, image[, workgroup]]) -> bitsknn_fused_l2_topk_f32_tuned."""
    import torch
    d, q = queries_dm.shape
    d2, n = points_dm.shape
    assert d == d2 and queries_dm.is_contiguous() and points_dm.is_contiguous()
    if out_dist is None:
        out_dist = torch.empty((q, k), dtype=torch.float32, device=queries_dm.device)
    if out_label is None:
        out_label = torch.empty((q, k), dtype=torch.int32, device=queries_dm.device)
    if isinstance(workspace, str) and workspace == "auto":
        workspace = torch.empty(max(1, fused_workspace_bytes(q, n, k)), dtype=torch.uint8,
                                device=queries_dm.device)
    if isinstance(workspace, str) and workspace == "image":
        workspace = torch.empty(max(1, fused_workspace_with_image_bytes(d, q, n, k)), dtype=torch.uint8,
                                device=queries_dm.device)
    head = (_ptr(queries_dm), _ptr(points_dm), d, q, n, _ptr(out_dist), _ptr(out_label), k,
            params[0], params[1], params[2], block_query_dim, dim_mult)
    if tuning is not None:
        assert not isinstance(workspace, str)
        knobs = FusedTuning(int(tuning[0]), int(tuning[1]), int(tuning[2]) if len(tuning) > 2 else 0,
                            int(tuning[3]) if len(tuning) > 3 else 0, (ctypes.c_int32 * 4)())
        _check(lib().bitsknn_fused_l2_topk_f32_tuned(*head[:8], FUSED_EXACT if arithmetic is None else int(arithmetic),
                                                     ctypes.byref(knobs), _ptr(workspace),
                                                     workspace.numel() if workspace is not None else 0, _stream()))
    elif isinstance(workspace, str) and workspace == "static":
        assert arithmetic is None
        _check(lib().bitsknn_fused_l2_topk_f32_static(*head, _stream()))
    elif arithmetic is not None:
        _check(lib().bitsknn_fused_l2_topk_f32_ex(*head, int(arithmetic), _ptr(workspace),
                                                  workspace.numel() if workspace is not None else 0,
                                                  _stream()))
    elif workspace is None:
        _check(lib().bitsknn_fused_l2_topk_f32(*head, _stream()))
    else:
        _check(lib().bitsknn_fused_l2_topk_f32_ws(*head, _ptr(workspace), workspace.numel(), _stream()))
    return out_dist, out_label


def fused_workspace_bytes(q, n, k):
    return int(lib().bitsknn_fused_workspace_bytes(q, n, k))


def fused_image_bytes(dim, n):
    return int(lib().bitsknn_fused_image_bytes(dim, n))


def fused_workspace_with_image_bytes(dim, q, n, k):
    """Partial lists, rounded up to a multiple of 256 bytes, then the stage image."""
    return (fused_workspace_bytes(q, n, k) + 255) // 256 * 256 + fused_image_bytes(dim, n)


def fused_static_scratch_bytes():
    return int(lib().bitsknn_fused_static_scratch_bytes())


def fused_status():
    """Synchronises the current stream and raises BitsKnnError(ERR_INTERNAL) if a fused kernel has
    reported a wait that ran out of polls since the last check."""
    _check(lib().bitsknn_fused_status(_stream()))
