"""ctypes binding of libmi355fp8.so (the C ABI declared in include/mi355_fp8.h)."""
import ctypes
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmi355fp8.so")

GEMM_AUTO, GEMM_TILE256, GEMM_TILE128, GEMM_SKINNY, GEMM_GENERIC, GEMM_TILE256x128 = 0, 1, 2, 3, 4, 5
GEMM_TILE256_RING, GEMM_TILE256_ONCE, GEMM_TILE256_STREAMK, GEMM_SKINNY_XSHARE = 6, 7, 8, 9
GEMM_ROWS128 = 10
GEMM_SKINNY_CU = 11
GEMM_ROWS_MTILED = 12
WS_COUNTER_BYTES = 65536
DTYPE_CODES = {torch.bfloat16: 0, torch.float32: 1, torch.float16: 2}

_c = ctypes
_vp, _i64, _i32, _f32, _sz = _c.c_void_p, _c.c_int64, _c.c_int32, _c.c_float, _c.c_size_t

# name -> (restype, argtypes); must list every symbol of include/mi355_fp8.h
SIGNATURES = {
    "mi355_error_string": (_c.c_char_p, [_c.c_int]),
    "mi355_device_info": (_c.c_int, [_c.c_int, _c.POINTER(_i64)]),
    "mi355_group_quant_fp8": (_c.c_int, [_vp, _i32, _vp, _vp, _i64, _i64, _i32, _f32, _i64, _i64, _vp]),
    "mi355_block_weight_quant_fp8": (_c.c_int, [_vp, _i32, _vp, _vp, _i64, _i64, _i32, _vp]),
    "mi355_block_fp8_gemm_variant": (_i32, [_i64, _i64, _i64]),
    "mi355_block_fp8_gemm_plan": (_i32, [_i64, _i64, _i64, _sz, _i32]),
    "mi355_block_fp8_gemm_workspace_bytes": (_sz, [_i64, _i64, _i64, _i32]),
    "mi355_block_fp8_gemm_noalloc": (
        _c.c_int,
        [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32,
         _i32, _vp],
    ),
    "mi355_reset_workspace": (_c.c_int, [_vp, _sz, _vp]),
    "mi355_block_fp8_gemm": (
        _c.c_int,
        [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32,
         _vp, _sz, _i32, _vp],
    ),
    "mi355_block_fp8_gemm_dtype": (
        _c.c_int,
        [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32,
         _vp, _sz, _i32, _i32, _vp],
    ),
    "mi355_moe_align_fused": (_c.c_int, [_vp, _vp, _i64, _i32, _vp, _vp, _vp, _vp]),
    "mi355_moe_align": (_c.c_int, [_vp, _i64, _i32, _vp, _i64, _vp]),
    "mi355_moe_align1": (_c.c_int, [_vp, _i64, _vp, _i64, _i32, _vp, _i64, _vp, _vp]),
    "mi355_moe_align2_rows": (_i64, [_i64, _i32, _i32]),
    "mi355_moe_align2": (_c.c_int, [_vp, _i32, _i32, _i64, _vp, _vp]),
    "mi355_grouped_block_m": (_i32, [_i64, _i32, _i64, _i64]),
    "mi355_grouped_workspace_bytes": (_sz, [_i64]),
    "mi355_grouped_block_fp8_gemm": (
        _c.c_int,
        [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i64, _i64, _i32, _i32, _i64, _i64, _i32, _vp, _vp,
         _c.c_size_t, _vp],
    ),
    "mi355_grouped_block_fp8_gemm_dtype": (
        _c.c_int,
        [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i64, _i64, _i32, _i32, _i64, _i64, _i32, _vp, _vp,
         _c.c_size_t, _i32, _vp],
    ),
    "mi355_grouped_block_fp8_gemm_bias": (
        _c.c_int,
        [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i64, _i64, _i32, _i32, _i64, _i64, _i32, _vp, _vp,
         _c.c_size_t, _i32, _vp, _i32, _i64, _vp],
    ),
    "mi355_silu_and_mul": (_c.c_int, [_vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "mi355_silu_and_mul_ex": (_c.c_int, [_vp, _vp, _i64, _i64, _i64, _i64, _i32, _i32, _f32, _f32, _vp]),
    "mi355_silu_and_mul_group_quant_fp8": (
        _c.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i32, _i64, _i64, _vp, _i64, _vp]
    ),
    "mi355_moe_sum_reduce": (_c.c_int, [_vp, _vp, _i64, _i32, _i64, _vp]),
    "mi355_block_weight_dequant": (_c.c_int, [_vp, _vp, _vp, _i64, _i64, _i32, _vp]),
    "mi355_probe_mfma": (_c.c_int, [_vp, _vp, _i32, _i32, _i32, _vp]),
}

_lib = None
_lock = threading.Lock()


class Mi355Error(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """Loads the HIP library; there is no fallback path when it is missing."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise Mi355Error(
                        f"{LIB_PATH} is missing: build it with `python -m lightllm_amd.build` "
                        "(hipcc, gfx950). lightllm_amd has no CPU or eager fallback."
                    )
                handle = ctypes.CDLL(LIB_PATH)
                for name, (res, args) in SIGNATURES.items():
                    fn = getattr(handle, name)
                    fn.restype = res
                    fn.argtypes = args
                _lib = handle
    return _lib


def check(code: int, what: str) -> None:
    """Re-raise a negative C-ABI status as the Python error the reference would raise."""
    if code == 0:
        return
    msg = lib().mi355_error_string(code).decode()
    if code in (-2,):
        raise AssertionError(f"{what}: {msg}")
    if code in (-1, -3, -4, -6, -7):
        raise ValueError(f"{what}: {msg}")
    raise Mi355Error(f"{what}: {msg}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device: torch.device) -> int:
    """The HIP stream torch would launch on for `device`, as an integer handle."""
    if _raw_stream is not None:   # a fifth of the cost of building a Stream object per call
        return _raw_stream(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


def require_cuda(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise Mi355Error("lightllm_amd operators run on the GPU only; got a CPU tensor")


_workspaces = {}  # (device index, stream handle or _GRAPH) -> buffer
_retired = []  # outgrown workspaces: kept alive, a captured HIP graph may still hold their address


_GRAPH = "graph"  # key of a device's workspace for launches recorded into HIP graphs


def workspace(device: torch.device, nbytes: int, stream: int = None) -> torch.Tensor:
    """Scratch for split-K and persistent launches: zero-initialised once, grown on demand.

    Eager launches use one buffer per (device, stream).  Launches recorded under HIP graph capture use one buffer
    per device that every eager call sizes along with its own: the capture stream is not the stream of the warm-up
    run (``torch.cuda.graph`` captures on a side stream), so a buffer looked up by stream would be missed there and
    allocated - and zero-filled on every replay - inside the graph.  After the shape has run once outside a
    capture, capturing it allocates nothing.  A capture of a shape that never ran eagerly still works: it gets a
    buffer from the graph's own pool, zero-filled by a node of the graph.

    The kernels leave the counter words zero, so a buffer is never cleared again.  A buffer that has been handed
    out is never freed: when a later call needs more, a larger one takes its place for new launches and the old
    one stays allocated, because a graph captured earlier has its address baked in and keeps using it on replay.
    Graphs of one device share that device's buffer: replay them one at a time (launches that overlap in time on
    one workspace race).
    """
    dev = device.index if device.index is not None else torch.cuda.current_device()
    capturing = torch.cuda.is_current_stream_capturing()
    key = (dev, _GRAPH) if capturing else (dev, stream_ptr(device) if stream is None else stream)
    buf = _workspaces.get(key)
    if buf is not None and buf.numel() >= nbytes:
        return buf
    if capturing:
        return torch.zeros(max(nbytes, WS_COUNTER_BYTES), dtype=torch.uint8, device=device)
    size = max(nbytes, WS_COUNTER_BYTES + (32 << 20))
    with _lock:
        for k in (key, (dev, _GRAPH)):
            old = _workspaces.get(k)
            if old is None or old.numel() < nbytes:
                if old is not None:
                    _retired.append(old)
                _workspaces[k] = torch.zeros(size, dtype=torch.uint8, device=device)
        buf = _workspaces[key]
    return buf


def reset_workspace(device: torch.device) -> None:
    """Re-zero the counter words of the current stream's workspace (after an aborted launch)."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_ptr(device))
    with _lock:
        buf = _workspaces.get(key)
    if buf is not None:
        check(lib().mi355_reset_workspace(buf.data_ptr(), buf.numel(), stream_ptr(device)), "mi355_reset_workspace")


def device_info(device: int = -1) -> dict:
    out = (_i64 * 8)()
    check(lib().mi355_device_info(device, out), "mi355_device_info")
    keys = ["compute_units", "clock_khz", "lds_bytes", "l2_bytes", "mem_clock_khz", "mem_bus_bits", "is_gfx950", "hbm_bytes"]
    return dict(zip(keys, [int(v) for v in out]))
