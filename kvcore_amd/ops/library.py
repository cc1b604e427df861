"""Python face of the gfx950 kernel library: loads it, checks operands on the host,
launches on torch's current stream.

There is no other compute path.  If the library cannot be loaded or built, the first
use raises; nothing falls back to the CPU or to torch's operators (library matrix
products for bfloat16 excepted, which is where the reference uses a library too:
``nn.Linear`` at kvcore/model/layer/linear.py:6-11).
"""

from __future__ import annotations

import os

import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p
from dataclasses import dataclass

import torch

from . import build as _build

_LIB: ctypes.CDLL | None = None
_LIB_PATH: str | None = None

DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}


class KernelError(RuntimeError):
    """The kernel library refused its arguments or could not launch."""


def _declare(lib: ctypes.CDLL) -> None:
    P, I, L, F = c_void_p, c_int, c_int64, c_float
    sigs = {
        "kvc_embed": [P, P, P, I, I, I, I, F, P],
        "kvc_logits_finish": [P, I, I, L, P, I, F, F, P],
        "kvc_fill_pages": [P, P, I, I, I, I, L, I, ctypes.c_uint32, P],
        "kvc_fill_normal": [P, L, I, ctypes.c_uint32, ctypes.c_uint32, F, F, P],
        "kvc_add_rmsnorm": [P, P, P, P, F, I, I, I, P],
        "kvc_add_slices_rmsnorm": [P, P, P, I, P, P, F, I, I, I, P],
        "kvc_rmsnorm": [P, P, P, F, I, I, L, L, I, P],
        "kvc_residual_add": [P, P, I, I, I, P],
        "kvc_silu_mul": [P, P, I, I, I, P],
        "kvc_gather_rows": [P, P, P, I, I, I, I, P],
        "kvc_to_float": [P, P, L, I, P],
        "kvc_rope_table": [P, P, P, P, I, I, P],
        "kvc_kv_slots": [P, P, P, P, P, I, I, I, I, P],
        "kvc_rope_kv_write": [P, P, P, P, P, I, I, P, I, I, I, I, I, I, I, I, P],
        "kvc_paged_attention": [P, P, L, P, P, P, I, P, P, P, I, I, I, I, I, I, F, I, I, P],
        "kvc_decode_attention": [P, P, P, P, L, P, P, P, I, P, P, P, P, P, P, I, I, I, I, I, I, I, I, I,
                                 F, I, I, P],
        "kvc_decode_attention_waves": [I, I, I],
        "kvc_decode_attention_max_table": [I, I, I],
        "kvc_decode_attention_supported": [I, I, I, I, I],
        "kvc_prefill_attention": [P, P, L, P, P, P, I, P, P, P, I, I, I, I, I, I, I, F, I, P, P, I,
                                  P, P, I, I, P],
        "kvc_prefill_attention_supported": [I, I, I, I, I],
        "kvc_gemm_mid_slices": [I, I],
        "kvc_gemm_mid_bf16": [P, P, P, P, P, I, I, I, L, L, I, I, I, P],
        "kvc_gemm_f32": [P, P, P, P, I, I, I, L, L, P],
        "kvc_gemm_skinny_bf16": [P, P, P, P, I, I, I, L, L, I, I, P],
        "kvc_gemm_skinny_silu_mul_bf16": [P, P, P, P, I, I, I, L, L, I, P],
        "kvc_pack_weight": [P, P, I, I, P],
        "kvc_gemm_skinny_blocks": [I, I, I, I],
        "kvc_gemm_skinny_fused_bf16": [P, P, P, P, I, I, I, L, L, I, P, I, I, F, P, L, P, P, I, P],
        "kvc_table_update": [P, I, I, P, I, P],
        "kvc_argmax": [P, P, I, I, L, P, P, I, P],
        "kvc_argmax_static": [P, P, I, I, L, P],
        "kvc_sample": [P, P, I, I, L, P, P, P, P, P, P, P, L, I, P],
        "kvc_sample_workspace_words": [I, I],
        "kvc_peak_read": [P, L, I, P, P],
        "kvc_peak_mfma_bf16": [P, I, I, P],
    }
    for name, argtypes in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = c_int
    lib.kvc_last_error.restype = ctypes.c_char_p
    lib.kvc_last_error.argtypes = []
    lib.kvc_version.restype = c_int
    lib.kvc_compute_units.restype = c_int
    lib.kvc_compute_units.argtypes = []
    lib.kvc_last_variant.restype = ctypes.c_char_p
    lib.kvc_last_variant.argtypes = [c_int]
    lib.kvc_argmax_static_capacity.restype = c_int
    lib.kvc_argmax_static_capacity.argtypes = []


def load(build_if_missing: bool = True) -> ctypes.CDLL:
    """The loaded library; built first when no matching build is found."""
    global _LIB, _LIB_PATH
    if _LIB is not None:
        return _LIB
    path = _build.find_library()
    if path is None:
        if not build_if_missing:
            raise KernelError("kvcore_amd: the gfx950 kernel library is not built")
        path = _build.build()
    try:
        lib = ctypes.CDLL(str(path))
    except OSError as exc:
        raise KernelError(f"kvcore_amd: cannot load the kernel library {path}: {exc}") from exc
    _declare(lib)
    _LIB, _LIB_PATH = lib, str(path)
    return lib


def library_path() -> str | None:
    return _LIB_PATH


def _check(code: int, name: str) -> None:
    if code != 0:
        msg = load().kvc_last_error().decode("utf-8", "replace")
        raise KernelError(f"{name} failed ({code}): {msg}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current stream's handle (asked of torch at every launch: a stream context or a
    graph capture may have changed it)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, name: str, dtype: torch.dtype | None = None) -> int:
    if not t.is_cuda:
        raise KernelError(f"{name} must be a GPU tensor (this engine has no CPU path)")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    return t.data_ptr()


def _code(t: torch.Tensor, name: str) -> int:
    try:
        return DTYPE_CODE[t.dtype]
    except KeyError:
        raise KernelError(f"{name}: unsupported dtype {t.dtype}") from None


# ------------------------------------------------------------------------ wrappers
def embed(residual: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0) -> None:
    """``residual[t] = float(table[ids[t]]) * scale``; an id outside the table gives a NaN row."""
    T, H = residual.shape
    V = table.shape[0]
    if table.shape[1] != H or ids.numel() != T:
        raise KernelError("embed: shapes do not match")
    _check(load().kvc_embed(_dev(residual, "residual", torch.float32), _dev(table, "table"),
                            _dev(ids, "ids", torch.int32), T, H, V, _code(table, "table"), float(scale),
                            _stream()), "kvc_embed")


def logits_finish(logits: torch.Tensor, bias: torch.Tensor | None = None, soft_cap: float = 0.0,
                  scale: float = 1.0) -> None:
    """In place on float32 ``logits [S, V]``: ``+ bias``, then ``soft_cap * tanh(x / soft_cap)``
    when ``soft_cap > 0``, then ``* scale`` (the order of kvcore/sample/logits_processor.py:50-54)."""
    S, V = logits.shape
    if logits.dtype != torch.float32 or not logits.is_cuda or logits.stride(1) != 1:
        raise KernelError("logits_finish: expects float32 GPU logits [S, V]")
    if bias is not None and bias.shape != (V,):
        raise KernelError("logits_finish: bias must be [V]")
    _check(load().kvc_logits_finish(logits.data_ptr(), S, V, logits.stride(0),
                                    None if bias is None else _dev(bias, "bias"),
                                    0 if bias is None else _code(bias, "bias"), float(soft_cap),
                                    float(scale), _stream()), "kvc_logits_finish")


def fill_pages(storage: torch.Tensor, pages: torch.Tensor, n: int, value: float, stride: int = 1,
               page_axis: int = -4) -> None:
    """``storage`` is cache memory whose axis ``page_axis`` counts pages, everything behind it
    being one page and everything before it planes (a cache group's ``[entries, pages, elements
    a page]`` with ``page_axis=1``; by default ``[..., pages, kv_heads, page_size, head_dim]``);
    contiguous, float32 or bfloat16.  Every element of the pages ``pages[i * stride]``,
    ``i < n`` (int32 on the device), in all planes becomes ``value`` (0 or NaN as a
    rule); the null page is skipped."""
    axis = page_axis if page_axis >= 0 else storage.dim() + page_axis
    if not 0 <= axis < storage.dim() - 1 or not storage.is_contiguous():
        raise KernelError("fill_pages: storage must be contiguous [..., pages, a page...]")
    if n > 0 and pages.numel() < (n - 1) * stride + 1:
        raise KernelError("fill_pages: page list too short")
    num_pages = storage.shape[axis]
    page_elems = 1
    for size in storage.shape[axis + 1:]:
        page_elems *= size
    outer = storage.numel() // (num_pages * page_elems)
    esize = storage.element_size()
    probe = torch.tensor([value], dtype=storage.dtype)
    bits = int(probe.view(torch.int16 if esize == 2 else torch.int32)[0]) & (0xFFFF if esize == 2 else 0xFFFFFFFF)
    if pages.dtype != torch.int32 or not pages.is_cuda:
        raise KernelError("fill_pages: pages must be int32 on the GPU")
    _check(load().kvc_fill_pages(_dev(storage, "storage"), pages.data_ptr(), stride, n, outer,
                                 num_pages, page_elems, esize, bits, _stream()), "kvc_fill_pages")


def fill_normal(out: torch.Tensor, seed_lo: int, seed_hi: int, mean: float, std: float) -> None:
    """``out`` (contiguous float32 or bfloat16 on the GPU) gets ``mean + std * z_i``, ``z_i`` the
    normal variate of (seed_lo, seed_hi, i): the same bits as ``weights/random_normal.py``."""
    _check(load().kvc_fill_normal(_dev(out, "out"), out.numel(), _code(out, "out"),
                                  seed_lo & 0xFFFFFFFF, seed_hi & 0xFFFFFFFF, float(mean), float(std),
                                  _stream()), "kvc_fill_normal")


def add_rmsnorm(out: torch.Tensor, residual: torch.Tensor, delta: torch.Tensor | None,
                weight: torch.Tensor, eps: float) -> None:
    T, H = residual.shape
    if out.shape != (T, H) or weight.shape != (H,) or (delta is not None and delta.shape != (T, H)):
        raise KernelError("add_rmsnorm: shapes do not match")
    if delta is not None and delta.dtype != out.dtype:
        raise KernelError("add_rmsnorm: delta and out must share a dtype")
    _check(load().kvc_add_rmsnorm(_dev(out, "out"), _dev(residual, "residual", torch.float32),
                                  None if delta is None else _dev(delta, "delta"),
                                  _dev(weight, "weight", torch.float32), float(eps), T, H,
                                  _code(out, "out"), _stream()), "kvc_add_rmsnorm")


def rmsnorm(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float) -> None:
    """Rows of ``x`` (last dim contiguous, any row stride) normalised into ``out``."""
    if x.dim() != 2 or out.shape != x.shape or x.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("rmsnorm: expects 2-D tensors with a contiguous last dim")
    if x.dtype != out.dtype or not x.is_cuda or not out.is_cuda:
        raise KernelError("rmsnorm: x and out must be GPU tensors of one dtype")
    T, H = x.shape
    if weight.shape != (H,):
        raise KernelError("rmsnorm: weight shape")
    _check(load().kvc_rmsnorm(out.data_ptr(), x.data_ptr(), _dev(weight, "weight", torch.float32),
                              float(eps), T, H, x.stride(0), out.stride(0), _code(x, "x"), _stream()),
           "kvc_rmsnorm")


def residual_add(residual: torch.Tensor, delta: torch.Tensor) -> None:
    T, H = residual.shape
    if delta.shape != (T, H):
        raise KernelError("residual_add: shapes do not match")
    _check(load().kvc_residual_add(_dev(residual, "residual", torch.float32), _dev(delta, "delta"),
                                   T, H, _code(delta, "delta"), _stream()), "kvc_residual_add")


def silu_mul(out: torch.Tensor, gate_up: torch.Tensor) -> None:
    T, I2 = gate_up.shape
    if I2 % 2 or out.shape != (T, I2 // 2) or out.dtype != gate_up.dtype:
        raise KernelError("silu_mul: shapes or dtypes do not match")
    _check(load().kvc_silu_mul(_dev(out, "out"), _dev(gate_up, "gate_up"), T, I2 // 2,
                               _code(out, "out"), _stream()), "kvc_silu_mul")


def gather_rows(out: torch.Tensor, src: torch.Tensor, rows: torch.Tensor) -> None:
    S, H = out.shape
    if src.shape[1] != H or rows.numel() != S:
        raise KernelError("gather_rows: shapes do not match")
    _check(load().kvc_gather_rows(_dev(out, "out"), _dev(src, "src"), _dev(rows, "rows", torch.int32),
                                  S, H, _code(src, "src"), _code(out, "out"), _stream()),
           "kvc_gather_rows")


def to_float(out: torch.Tensor, src: torch.Tensor) -> None:
    if out.numel() != src.numel():
        raise KernelError("to_float: sizes do not match")
    _check(load().kvc_to_float(_dev(out, "out", torch.float32), _dev(src, "src"), src.numel(),
                               _code(src, "src"), _stream()), "kvc_to_float")


def rope_table(cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
               inv_freq: torch.Tensor) -> None:
    T, half = cos.shape
    if sin.shape != (T, half) or positions.numel() < T or inv_freq.numel() != half:
        raise KernelError("rope_table: shapes do not match")
    _check(load().kvc_rope_table(_dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32),
                                 _dev(positions, "positions", torch.int32),
                                 _dev(inv_freq, "inv_freq", torch.float32), T, half, _stream()),
           "kvc_rope_table")


def kv_slots(out: torch.Tensor, *, positions: torch.Tensor, token_req: torch.Tensor,
             slots: torch.Tensor, table: torch.Tensor, page_size: int, num_pages: int) -> None:
    """``out[t]`` = cache slot of token ``t`` (page * page_size + offset), -1 without a page,
    -2 for a padding token.  Reference: kvcore/kv/block_table.py:215-227 computes the same
    mapping per layer in Python."""
    T = out.numel()
    if positions.numel() < T or token_req.numel() < T:
        raise KernelError("kv_slots: per-token arrays too short")
    _check(load().kvc_kv_slots(_dev(out, "out", torch.int32), _dev(positions, "positions", torch.int32),
                               _dev(token_req, "token_req", torch.int32),
                               _dev(slots, "slots", torch.int32), _dev(table, "table", torch.int32),
                               table.shape[1], T, page_size, num_pages, _stream()), "kvc_kv_slots")


def rope_kv_write(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  cos: torch.Tensor, sin: torch.Tensor, *, rot_dim: int, interleaved: bool,
                  kv_slot: torch.Tensor, nh: int, nkv: int, d: int, write_kv: bool = True,
                  rotate_q: bool = True) -> None:
    """``k_cache`` is ``[pages, nkv, page_size, d]``, ``v_cache`` ``[pages, nkv, d, page_size]``,
    both of the dtype of ``qkv``; ``kv_slot`` comes from ``kv_slots``.  Without ``rotate_q``
    the query heads are left as they are, for an attention kernel that rotates them itself."""
    T = qkv.shape[0]
    if qkv.shape != (T, (nh + 2 * nkv) * d):
        raise KernelError(f"rope_kv_write: qkv shape {tuple(qkv.shape)} does not fit heads")
    num_pages, page_size = _check_cache(k_cache, v_cache, nkv, d, "rope_kv_write")
    if k_cache.dtype != qkv.dtype or v_cache.dtype != qkv.dtype:
        raise KernelError("rope_kv_write: cache dtype differs from qkv")
    if cos.shape[0] < T or cos.shape[1] != rot_dim // 2 or sin.shape != cos.shape:
        raise KernelError("rope_kv_write: rotary tables do not fit")
    if kv_slot.numel() < T:
        raise KernelError("rope_kv_write: kv_slot too short")
    _check(load().kvc_rope_kv_write(
        _dev(qkv, "qkv"), _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"),
        _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32), rot_dim, int(interleaved),
        _dev(kv_slot, "kv_slot", torch.int32), T, nh, nkv, d, page_size, int(write_kv),
        int(rotate_q), _code(qkv, "qkv"), _stream()), "kvc_rope_kv_write")


def paged_attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    *, table: torch.Tensor, positions: torch.Tensor, token_req: torch.Tensor,
                    slots: torch.Tensor, nh: int, nkv: int, d: int, scale: float,
                    window: int = 0) -> None:
    """``q`` is a ``[T, >= nh*d]`` view whose rows hold the query heads first."""
    T = out.shape[0]
    if out.shape != (T, nh * d) or not out.is_contiguous():
        raise KernelError("paged_attention: out must be contiguous [T, nh*d]")
    if q.shape[0] != T or q.stride(1) != 1 or q.shape[1] < nh * d or q.dtype != out.dtype:
        raise KernelError("paged_attention: q does not fit")
    num_pages, page_size = _check_cache(k_cache, v_cache, nkv, d, "paged_attention")
    if k_cache.dtype != out.dtype:
        raise KernelError("paged_attention: cache dtype differs from the queries'")
    if positions.numel() < T or token_req.numel() < T:
        raise KernelError("paged_attention: per-token arrays too short")
    _check(load().kvc_paged_attention(
        out.data_ptr(), q.data_ptr(), q.stride(0), _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"),
        _dev(table, "table", torch.int32), table.shape[1],
        _dev(positions, "positions", torch.int32), _dev(token_req, "token_req", torch.int32),
        _dev(slots, "slots", torch.int32), T, nh, nkv, d, page_size, num_pages, float(scale),
        int(window), _code(out, "out"), _stream()), "kvc_paged_attention")


def decode_attention_supported(nh: int, nkv: int, d: int, page_size: int, dtype: torch.dtype) -> bool:
    return bool(load().kvc_decode_attention_supported(nh, nkv, d, page_size, DTYPE_CODE.get(dtype, -1)))


KERNEL_FAMILIES = {"prefill_attention": 0, "rope_kv_write": 1}


def last_variant(family: str) -> str:
    """Which variant of a kernel family this thread's last launch took (see the C header): for
    tests that must know which code ran."""
    return load().kvc_last_variant(KERNEL_FAMILIES[family]).decode()


def measure_peaks(device: str | torch.device = "cuda:0") -> dict[str, float]:
    """What this chip gives a kernel that does nothing but read (bytes a second: 16-byte loads
    over 1 GiB pieces of a 3 GiB buffer, so that no cache serves them, two blocks a compute
    unit) and nothing but multiply on the matrix cores (bfloat16 flops a second, operands in
    registers, four waves a SIMD).  Some 0.1 s.  The data sheet says 8 TB/s and 2.5 PFLOP/s."""
    lib = load()
    device = torch.device(device)
    cus = compute_units()
    piece = 1 << 30
    buf = torch.empty(3 * piece, dtype=torch.uint8, device=device)
    buf.fill_(1)
    sink = torch.zeros(4, dtype=torch.int32, device=device)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def read(i: int) -> None:
        _check(lib.kvc_peak_read(buf.data_ptr() + (i % 3) * piece, piece, 2 * cus, sink.data_ptr(), _stream()),
               "kvc_peak_read")

    for i in range(3):
        read(i)
    start.record()
    for i in range(12):
        read(i)
    end.record()
    end.synchronize()
    read_rate = 12 * piece / (start.elapsed_time(end) * 1e-3)
    del buf
    blocks, rounds = 4 * cus, 8000
    out = torch.empty(blocks * 256, dtype=torch.float32, device=device)
    for _ in range(2):
        _check(lib.kvc_peak_mfma_bf16(out.data_ptr(), blocks, 200, _stream()), "kvc_peak_mfma_bf16")
    flops = blocks * 4 * rounds * 4 * 2.0 * 32 * 32 * 16
    best = 0.0
    for _ in range(4):  # the clock takes a few milliseconds to rise: the fastest run is the peak
        start.record()
        _check(lib.kvc_peak_mfma_bf16(out.data_ptr(), blocks, rounds, _stream()), "kvc_peak_mfma_bf16")
        end.record()
        end.synchronize()
        best = max(best, flops / (start.elapsed_time(end) * 1e-3))
    return {"read_bytes_per_s": read_rate, "mfma_bf16_flops_per_s": best}


_COMPUTE_UNITS: int | None = None


def compute_units() -> int:
    """Compute units of the current GPU, which launch plans count their blocks against (256, an
    MI355X's, where no GPU is visible: plans are also worked out on a host without one)."""
    global _COMPUTE_UNITS
    if _COMPUTE_UNITS is None:
        _COMPUTE_UNITS = int(load().kvc_compute_units()) if torch.cuda.is_available() else 256
    return _COMPUTE_UNITS


def decode_attention_max_table(nh: int, nkv: int, d: int) -> int:
    """The widest block table (entries per request) that :func:`decode_attention` serves."""
    return int(load().kvc_decode_attention_max_table(nh, nkv, d))


def decode_attention_waves(nh: int, nkv: int, d: int) -> int:
    """How many waves of a block share its range of keys in :func:`decode_attention`."""
    return int(load().kvc_decode_attention_waves(nh, nkv, d))


def decode_attention(out: torch.Tensor, qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     *, table: torch.Tensor, positions: torch.Tensor, token_req: torch.Tensor,
                     slots: torch.Tensor, nh: int, nkv: int, d: int, scale: float, window: int = 0,
                     nsplit: int = 1, part_o: torch.Tensor | None = None,
                     part_ml: torch.Tensor | None = None, cos: torch.Tensor | None = None,
                     sin: torch.Tensor | None = None, rot_dim: int = 0, interleaved: bool = False,
                     write_kv: bool = False, token_rows: torch.Tensor | None = None) -> None:
    """bfloat16 attention of single tokens on the matrix cores (see the C header), with the
    rotation of each token's query and key and the write of its key and value into the cache
    (``write_kv``) in the same kernel; ``qkv`` is not changed.  With ``rot_dim = 0`` and
    ``write_kv = False`` it is the attention alone over queries as they are.  ``token_rows``
    (``slots[token_req]``, -1 for padding) may be given to save the kernel a lookup.  ``part_o`` and
    ``part_ml`` are float32 workspaces of at least ``T*nh*nsplit*d`` and ``T*nh*nsplit*2``
    elements when ``nsplit > 1``."""
    T = out.shape[0]
    if out.shape != (T, nh * d) or not out.is_contiguous() or out.dtype != torch.bfloat16:
        raise KernelError("decode_attention: out must be contiguous bfloat16 [T, nh*d]")
    need = (nh + 2 * nkv) * d if write_kv else nh * d
    if qkv.shape[0] != T or qkv.stride(1) != 1 or qkv.shape[1] < need or qkv.dtype != out.dtype:
        raise KernelError("decode_attention: qkv does not fit")
    num_pages, page_size = _check_cache(k_cache, v_cache, nkv, d, "decode_attention")
    if k_cache.dtype != out.dtype:
        raise KernelError("decode_attention: cache dtype differs from the queries'")
    if positions.numel() < T or token_req.numel() < T:
        raise KernelError("decode_attention: per-token arrays too short")
    c = s_ = None
    if rot_dim:
        if cos is None or sin is None or cos.shape[0] < T or cos.shape[1] != rot_dim // 2 \
                or sin.shape != cos.shape or not cos.is_contiguous() or not sin.is_contiguous():
            raise KernelError("decode_attention: cos and sin must be contiguous [>= T, rot_dim/2]")
        c, s_ = _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32)
    po = pm = None
    if nsplit > 1:
        if part_o is None or part_ml is None or part_o.numel() < T * nh * nsplit * d \
                or part_ml.numel() < T * nh * nsplit * 2:
            raise KernelError("decode_attention: workspace missing or too small")
        po, pm = _dev(part_o, "part_o", torch.float32), _dev(part_ml, "part_ml", torch.float32)
    _check(load().kvc_decode_attention(
        out.data_ptr(), po, pm, qkv.data_ptr(), qkv.stride(0), _dev(k_cache, "k_cache"),
        _dev(v_cache, "v_cache"), _dev(table, "table", torch.int32), table.shape[1],
        _dev(positions, "positions", torch.int32), _dev(token_req, "token_req", torch.int32),
        _dev(slots, "slots", torch.int32),
        None if token_rows is None else _dev(token_rows, "token_rows", torch.int32),
        c, s_, int(rot_dim), int(bool(interleaved)),
        int(bool(write_kv)), T, nh, nkv, d, page_size, num_pages, float(scale),
        int(window), int(nsplit), _stream()), "kvc_decode_attention")


def prefill_attention_supported(nh: int, nkv: int, d: int, page_size: int, dtype: torch.dtype) -> bool:
    return bool(load().kvc_prefill_attention_supported(nh, nkv, d, page_size, DTYPE_CODE.get(dtype, -1)))


def prefill_attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      *, table: torch.Tensor, positions: torch.Tensor, q_start: torch.Tensor,
                      slots: torch.Tensor, num_reqs: int, nh: int, nkv: int, d: int, scale: float,
                      window: int = 0, nsplit: int = 1, part_o: torch.Tensor | None = None,
                      part_ml: torch.Tensor | None = None, cos: torch.Tensor | None = None,
                      sin: torch.Tensor | None = None, rot_dim: int = 0, interleaved: bool = False) -> None:
    """bfloat16 attention of portions of prompts on the matrix cores (see the C header).
    ``nsplit > 1`` deals every tile's keys to that many blocks; ``part_o`` (float32,
    ``T*nh*nsplit*d`` values) and ``part_ml`` (``T*nh*nsplit*2``) are then the workspace.
    With ``cos`` and ``sin`` (``[T, rot_dim / 2]`` float32) the queries come unrotated and
    the kernel rotates them (``prefill_attention_rotates`` says for which shapes)."""
    T = out.shape[0]
    if out.shape != (T, nh * d) or not out.is_contiguous() or out.dtype != torch.bfloat16:
        raise KernelError("prefill_attention: out must be contiguous bfloat16 [T, nh*d]")
    if q.shape[0] != T or q.stride(1) != 1 or q.shape[1] < nh * d or q.dtype != out.dtype:
        raise KernelError("prefill_attention: q does not fit")
    num_pages, page_size = _check_cache(k_cache, v_cache, nkv, d, "prefill_attention")
    if k_cache.dtype != out.dtype:
        raise KernelError("prefill_attention: cache dtype differs from the queries'")
    if positions.numel() < T or q_start.numel() < num_reqs + 1 or slots.numel() < num_reqs:
        raise KernelError("prefill_attention: index arrays too short")
    po = pml = None
    if nsplit > 1:
        if part_o is None or part_ml is None or part_o.numel() < T * nh * nsplit * d or \
                part_ml.numel() < T * nh * nsplit * 2:
            raise KernelError("prefill_attention: the workspace for splits is missing or too small")
        po, pml = _dev(part_o, "part_o", torch.float32), _dev(part_ml, "part_ml", torch.float32)
    cs = sn = None
    if cos is not None:
        if sin is None or cos.shape[0] < T or cos.shape[1] != rot_dim // 2 or sin.shape != cos.shape \
                or not prefill_attention_rotates(rot_dim, interleaved):
            raise KernelError("prefill_attention: rotary tables do not fit")
        cs, sn = _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32)
    _check(load().kvc_prefill_attention(
        out.data_ptr(), q.data_ptr(), q.stride(0), _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"),
        _dev(table, "table", torch.int32), table.shape[1], _dev(positions, "positions", torch.int32),
        _dev(q_start, "q_start", torch.int32), _dev(slots, "slots", torch.int32), T, num_reqs,
        nh, nkv, d, page_size, num_pages, float(scale), int(window), po, pml, int(nsplit),
        cs, sn, int(rot_dim) if cs is not None else 0, int(interleaved), _stream()),
        "kvc_prefill_attention")


def prefill_attention_rotates(rot_dim: int, interleaved: bool) -> bool:
    """Whether ``prefill_attention`` can rotate the queries itself: a lane of the kernel
    must hold both elements of every rotary pair."""
    return rot_dim > 0 and rot_dim % (32 if interleaved else 64) == 0


def _check_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, nkv: int, d: int, who: str) -> tuple[int, int]:
    """K pages are ``[pages, nkv, page_size, d]``, V pages ``[pages, nkv, d, page_size]``."""
    if k_cache.dim() != 4 or v_cache.dim() != 4:
        raise KernelError(f"{who}: cache planes must be 4-D")
    num_pages, ckv, page_size, cd = k_cache.shape
    if (ckv, cd) != (nkv, d) or tuple(v_cache.shape) != (num_pages, nkv, d, page_size):
        raise KernelError(f"{who}: cache shapes {tuple(k_cache.shape)} / {tuple(v_cache.shape)} do not fit "
                          f"{nkv} kv heads of {d}")
    if k_cache.dtype != v_cache.dtype:
        raise KernelError(f"{who}: K and V planes differ in dtype")
    return num_pages, page_size


def gemm_f32(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None) -> None:
    M, K = a.shape
    N = w.shape[0]
    if w.shape != (N, K) or out.shape != (M, N) or a.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm_f32: shapes do not match")
    for t, name in ((a, "a"), (out, "out")):
        if t.dtype != torch.float32 or not t.is_cuda:
            raise KernelError(f"gemm_f32: {name} must be a float32 GPU tensor")
    _check(load().kvc_gemm_f32(out.data_ptr(), a.data_ptr(), _dev(w, "w", torch.float32),
                               None if bias is None else _dev(bias, "bias", torch.float32),
                               M, N, K, a.stride(0), out.stride(0), _stream()), "kvc_gemm_f32")


SKINNY_MAX_ROWS = 64
SKINNY_PREFERRED_ROWS = 16


def can_pack_weight(w: torch.Tensor) -> bool:
    return (w.dim() == 2 and w.dtype == torch.bfloat16 and w.is_cuda and w.is_contiguous()
            and w.shape[0] % 16 == 0 and w.shape[1] % 64 == 0)


def pack_weight(w: torch.Tensor) -> torch.Tensor:
    """A copy of the bfloat16 matrix ``w [N, K]`` in tiles of 16 rows x 32 columns, each 1 KB in
    one piece, the tiles of 16 rows one after the other along K: the order in which the
    weight-streaming products for few rows read a matrix, so that a load of theirs is one
    contiguous kilobyte instead of 64 bytes from each of 16 rows (some 8% more bandwidth on
    this chip).  The copy is kept as ``w.kvc_packed``; the products find it there and give
    the same bits with it as without."""
    if not can_pack_weight(w):
        raise KernelError("pack_weight: a contiguous bfloat16 GPU matrix of a multiple of 16 rows "
                          "and a multiple of 64 columns")
    packed = torch.empty_like(w)
    _check(load().kvc_pack_weight(packed.data_ptr(), w.data_ptr(), w.shape[0], w.shape[1], _stream()),
           "kvc_pack_weight")
    w.kvc_packed = packed
    return packed


def _streamed(w: torch.Tensor, rows: int | None = None) -> tuple[int, int]:
    """(pointer, packed flag) of the matrix a weight-streaming product should read: the packed
    twin of ``w`` where there is one (``rows``: the product's own row count, a multiple of 16
    for a packed matrix, which the gated product's half must be too)."""
    packed = getattr(w, "kvc_packed", None)
    if packed is not None and (rows is None or rows % 16 == 0):
        return packed.data_ptr(), 1
    return _dev(w, "w"), 0


def gemm_skinny_bf16(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor,
                     bias: torch.Tensor | None = None) -> None:
    """``out = a @ w.T (+ bias)`` for up to 64 rows of bfloat16; ``out`` is bfloat16 or
    float32 (the sums are float32 either way)."""
    M, K = a.shape
    N = w.shape[0]
    if w.shape != (N, K) or out.shape != (M, N) or a.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm_skinny_bf16: shapes do not match")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or not a.is_cuda or not out.is_cuda:
        raise KernelError("gemm_skinny_bf16: operands must be bfloat16 GPU tensors")
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.shape != (N,)):
        raise KernelError("gemm_skinny_bf16: bias must be bfloat16 [N]")
    w_ptr, packed = _streamed(w)
    _check(load().kvc_gemm_skinny_bf16(out.data_ptr(), a.data_ptr(), w_ptr,
                                       None if bias is None else _dev(bias, "bias"), M, N, K,
                                       a.stride(0), out.stride(0), _code(out, "out"), packed, _stream()),
           "kvc_gemm_skinny_bf16")


@dataclass
class ScaledRows:
    """Activation rows ``[T, H]`` that carry an RMS norm still to be finished: ``data`` holds
    ``residual * gain`` in bfloat16, ``ss_parts`` ``[T, parts]`` float32 partial sums of the
    residual's squares.  ``linear`` and ``linear_silu_mul`` take it in place of ``x`` and
    multiply row ``t``'s sums by ``rsqrt(sum(ss_parts[t]) / width + eps)``, which equals
    the product of the normalised row.  Made by ``linear`` into a :class:`ResidualSink`."""

    data: torch.Tensor
    ss_parts: torch.Tensor
    width: int
    eps: float

    @property
    def shape(self) -> torch.Size:
        return self.data.shape

    @property
    def dtype(self) -> torch.dtype:
        return self.data.dtype


@dataclass
class ResidualSink:
    """Where a product's result may go instead of a plain tensor: added into the float32
    ``residual`` rows, with ``out`` receiving ``bfloat16(residual * gain)`` and ``ss_parts``
    (room for ``[T, parts]`` float32) the new rows' partial sums of squares: the next norm,
    done but for the scale factor that the consuming product applies."""

    residual: torch.Tensor
    gain: torch.Tensor
    eps: float
    out: torch.Tensor
    ss_parts: torch.Tensor | None
    # for steps of 17 to 192 rows: float32 room for the partial sums of a product cut along K
    # (``mid_slices_bound(N) * T * N`` values); the sink then finishes the norm itself and
    # ``out`` receives the normalised rows
    slices: torch.Tensor | None = None


@dataclass
class NormedRows:
    """Rows that a :class:`ResidualSink` has already added into the residual and normalised:
    what ``linear`` returns for a sink that carries a workspace (steps of 17 to 192 rows)."""

    data: torch.Tensor


# The most rows the kernel that shares its rows through LDS takes (twelve tiles of 16 a wave).
# Measured on the 8B shape against the vendor's products with a norm kernel between them, a
# whole decode step: 72 rows 5.93 against 6.66 ms, 96 rows 6.53 against 7.72, 128 rows 7.57
# against 8.63, 160 rows 9.37 against 9.79, 192 rows 10.12 against 11.35; with sixteen tiles a
# wave 256 rows took 12.86 against 11.11, so the vendor's product has them.
MID_ROWS = 192
# Which products gain beyond 64 rows, one by one against the vendor's (us at 96 / 128 / 192 rows,
# packed weights): the narrow ones that are cut along K do (4096 x 14336: 33 / 45 / 64 against
# 64 / 76 / 104; 4096 x 4096: 13 / 15 / 21 against 23 / 25 / 34; 8192 x 28672: 109 / 136 / 209
# against 123 / 201 / 232); the gated one up to 128 rows (28672 x 4096: 54 / 67 / 83 against 53 /
# 54 / 61 and an activation kernel of 8 to 12; in a whole step of 128 rows 7.64 against 7.74 ms,
# of 192 rows 10.19 against 9.96); the head does not (128256 x 4096: 224 / 256 / 324 against
# 226 / 233 / 254; no difference in a whole step).  Matrices without a packed copy are read row by row, which
# the vendor's product does better from 65 rows on (a step of the 70B shape at 96 requests:
# 40.8 ms against 43.6) and up to 32 (24 requests: 30.4 against 32.7 ms, 32: 31.2 against 32.8;
# 48: 39.2 against 36.3, 64: the same).
MID_ROWS_UNPACKED = 64
MID_ROWS_UNPACKED_FROM = 33
MID_ROWS_GATED = 128
MID_ROWS_WIDE = 64


# Up to here the few-row kernel with the norms folded in is the fastest.  Measured at 16 rows
# against the kernels that share their rows through LDS: the 8B shape 4.13 against 4.45 ms a
# step, the 70B shape 30.4 against 32.6, the 1B shape 1.13 against 1.11.
FOLD_ROWS = 16


def mid_rows_ok(num_rows: int, packed: bool, most: int) -> bool:
    """Whether a product of ``num_rows`` rows by a matrix with or without a packed copy runs in
    the kernel that shares its rows through LDS (``most``: the kind of product's own limit)."""
    if packed:
        return FOLD_ROWS < num_rows <= most
    return MID_ROWS_UNPACKED_FROM <= num_rows <= min(most, MID_ROWS_UNPACKED)


def rows_fusable(num_rows: int, dtype: torch.dtype) -> bool:
    """Whether a step of ``num_rows`` tokens hands its norms to the products around them: up
    to 16 rows of bfloat16."""
    return dtype == torch.bfloat16 and 0 < num_rows <= FOLD_ROWS


def rows_sinkable(num_rows: int, dtype: torch.dtype) -> bool:
    """Whether a step of ``num_rows`` tokens sends the products before its norms into a
    :class:`ResidualSink` that finishes the norm itself: 17 to 192 rows."""
    return dtype == torch.bfloat16 and FOLD_ROWS < num_rows <= MID_ROWS


def skinny_blocks(N: int, K: int, gated: bool = False, packed: bool = False) -> int:
    """How many blocks of columns the weight-streaming kernel cuts ``N`` outputs into."""
    return int(load().kvc_gemm_skinny_blocks(N, K, int(gated), int(packed)))


def _fused_skinny(out: torch.Tensor | ResidualSink, x: torch.Tensor | ScaledRows, w: torch.Tensor,
                  bias: torch.Tensor | None, gated: bool) -> ScaledRows | None:
    """The weight-streaming product with a norm on either side folded in (see the C header)."""
    data = x.data if isinstance(x, ScaledRows) else x
    M, K = data.shape
    N = w.shape[0] // 2 if gated else w.shape[0]
    if data.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.shape[1] != K:
        raise KernelError("fused product: operands must be bfloat16 of matching width")
    if not _skinny_operands_ok(data, w):
        raise KernelError("fused product: at most 64 rows, K a multiple of 8, 16-byte aligned operands")
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != w.shape[0]):
        raise KernelError("fused product: bias must be bfloat16, one per weight row")
    in_ss = in_parts = in_width = 0
    in_eps = 0.0
    if isinstance(x, ScaledRows):
        in_parts = x.ss_parts.shape[1]
        if x.ss_parts.shape[0] < M or x.ss_parts.dtype != torch.float32 or not x.ss_parts.is_contiguous():
            raise KernelError("fused product: ss_parts must be contiguous float32 [>= T, parts]")
        in_ss, in_width, in_eps = x.ss_parts.data_ptr(), x.width, x.eps
    result = None
    if isinstance(out, ResidualSink):
        parts = skinny_blocks(N, K, packed=bool(_streamed(w, N)[1]))
        if out.residual.shape != (M, N) or out.residual.dtype != torch.float32 or out.residual.stride(1) != 1:
            raise KernelError("fused product: the residual must be float32 [T, N]")
        if out.gain.shape != (N,) or out.gain.dtype != torch.float32:
            raise KernelError("fused product: the gain must be float32 [N]")
        if out.out.shape != (M, N) or out.out.dtype != torch.bfloat16 or out.out.stride(1) != 1:
            raise KernelError("fused product: the sink's rows must be bfloat16 [T, N]")
        if out.ss_parts.numel() < M * parts or out.ss_parts.dtype != torch.float32 \
                or not out.ss_parts.is_contiguous():
            raise KernelError("fused product: the sink's ss_parts is too small")
        ss_view = out.ss_parts.view(-1)[: M * parts].view(M, parts)
        c_ptr, ldc = out.out.data_ptr(), out.out.stride(0)
        residual, ldr, gain, out_ss = (out.residual.data_ptr(), out.residual.stride(0),
                                       out.gain.data_ptr(), ss_view.data_ptr())
        result = ScaledRows(out.out, ss_view, N, out.eps)
    else:
        if out.shape != (M, N) or out.dtype != torch.bfloat16 or out.stride(1) != 1:
            raise KernelError("fused product: out must be bfloat16 [T, N]")
        c_ptr, ldc = out.data_ptr(), out.stride(0)
        residual = gain = out_ss = None
        ldr = 0
    if M:
        w_ptr, packed = _streamed(w, N)
        _check(load().kvc_gemm_skinny_fused_bf16(
            c_ptr, data.data_ptr(), w_ptr, None if bias is None else _dev(bias, "bias"), M, N, K,
            data.stride(0), ldc, int(gated), in_ss or None, in_parts, in_width, float(in_eps),
            residual, ldr, gain, out_ss, packed, _stream()), "kvc_gemm_skinny_fused_bf16")
    return result


def skinny_operands_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the weight-streaming product for few rows takes these operands."""
    return (x.shape[0] <= SKINNY_MAX_ROWS and x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


_skinny_operands_ok = skinny_operands_ok


def mid_slices_bound(N: int) -> int:
    """The most slices along K that ``gemm_mid`` cuts a weight with ``N`` rows into: blocks
    enough for 256 compute units, a block owning 64 weight rows, or 128 from 16,384 rows on
    (``plan_mid`` in csrc/gemm_mid.hip)."""
    rows_a_block = 128 if N >= 16384 else 64
    return min(64, -(-256 // -(-N // rows_a_block)))


def mid_slices(N: int, K: int) -> int:
    """Slices along K that ``gemm_mid`` cuts an [N, K] weight into when it may (see mode 2)."""
    return int(load().kvc_gemm_mid_slices(N, K))


def mid_operands_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``gemm_mid`` takes these operands (K a multiple of 512, aligned rows)."""
    return (x.shape[1] % 512 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0 and w.is_contiguous()
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def gemm_mid(out: torch.Tensor | None, x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None,
             *, mode: int = 0, partial: torch.Tensor | None = None) -> None:
    """The weight-streaming product for up to 192 rows of bfloat16 whose waves share the rows
    through LDS, the faster one from 9 rows on (see the C header for the
    modes: 0 plain, 1 ``silu(gate) * up``, 2 partial sums of slices along K only, 3 plain
    with slices and a kernel that sums them)."""
    M, K = x.shape
    N = w.shape[0] // 2 if mode == 1 else w.shape[0]
    if w.shape[1] != K or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or not x.is_cuda:
        raise KernelError("gemm_mid: operands must be bfloat16 GPU tensors with matching K")
    if not mid_operands_ok(x, w):
        raise KernelError("gemm_mid: K must be a multiple of 512 and the operands aligned")
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != w.shape[0]):
        raise KernelError("gemm_mid: bias must be bfloat16, one value per weight row")
    out_ptr, ldc, code = None, N, 1
    if mode != 2:
        if out is None or out.shape != (M, N) or out.stride(1) != 1 or not out.is_cuda:
            raise KernelError("gemm_mid: out does not fit")
        out_ptr, ldc, code = out.data_ptr(), out.stride(0), _code(out, "out")
    part_ptr = None
    if partial is not None:
        if partial.dtype != torch.float32 or partial.numel() < mid_slices(N, K) * M * N:
            raise KernelError("gemm_mid: the buffer for partial sums is too small")
        part_ptr = _dev(partial, "partial", torch.float32)
    w_ptr, packed = _streamed(w, N)
    _check(load().kvc_gemm_mid_bf16(out_ptr, part_ptr, x.data_ptr(), w_ptr,
                                    None if bias is None else _dev(bias, "bias"), M, N, K, x.stride(0),
                                    ldc, code, mode, packed, _stream()), "kvc_gemm_mid_bf16")


def add_slices_rmsnorm(out: torch.Tensor, residual: torch.Tensor, partial: torch.Tensor, slices: int,
                       bias: torch.Tensor | None, weight: torch.Tensor, eps: float) -> None:
    """``residual += sum_s partial[s] (+ bias)``; ``out = rmsnorm(residual) * weight`` (see the
    C header); ``partial`` holds ``[slices, T, H]`` float32."""
    T, H = residual.shape
    if out.shape != (T, H) or not out.is_contiguous() or not residual.is_contiguous():
        raise KernelError("add_slices_rmsnorm: out and residual must be contiguous [T, H]")
    if partial.dtype != torch.float32 or partial.numel() < slices * T * H:
        raise KernelError("add_slices_rmsnorm: the partial sums do not fit")
    _check(load().kvc_add_slices_rmsnorm(
        _dev(out, "out"), _dev(residual, "residual", torch.float32), _dev(partial, "partial"), slices,
        None if bias is None else _dev(bias, "bias", torch.bfloat16), _dev(weight, "weight", torch.float32),
        float(eps), T, H, _code(out, "out"), _stream()), "kvc_add_slices_rmsnorm")


def _sink_mid(sink: ResidualSink, x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None) -> NormedRows:
    """A product of 17 to 192 rows into a sink: partial sums of slices along K, then one kernel
    that adds them into the residual and normalises.  Shapes the weight-streaming kernel does
    not take run the vendor product into the same workspace first."""
    M, K = x.shape
    N = w.shape[0]
    if sink.slices is None or sink.slices.dtype != torch.float32:
        raise KernelError("linear: this sink needs its float32 workspace")
    if sink.residual.shape != (M, N) or sink.residual.dtype != torch.float32 or not sink.residual.is_contiguous():
        raise KernelError("linear: the sink's residual must be contiguous float32 [T, N]")
    if sink.out.shape != (M, N) or not sink.out.is_contiguous():
        raise KernelError("linear: the sink's rows must be contiguous [T, N]")
    # measured: the vendor product is as fast or faster once the output is wide and K is not
    # long (8192 x 8192), and slower for narrow outputs and long K (8192 x 28672: 139 against
    # 107 us at 64 rows; 4096 x 4096: 19 against 12)
    ours = (N < 8192 or K > 8192) and mid_rows_ok(M, bool(_streamed(w, N)[1]), MID_ROWS)
    if ours and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and mid_operands_ok(x, w) and N % 8 == 0:
        slices = mid_slices(N, K)
        if sink.slices.numel() < slices * M * N:
            raise KernelError("linear: the sink's workspace is too small")
        gemm_mid(None, x, w, mode=2, partial=sink.slices)
        add_slices_rmsnorm(sink.out, sink.residual, sink.slices, slices, bias, sink.gain, sink.eps)
    else:
        if sink.slices.numel() * 2 < M * N:
            raise KernelError("linear: the sink's workspace is too small")
        tmp = sink.slices.view(-1).view(x.dtype)[: M * N].view(M, N)
        linear(tmp, x, w, bias)
        add_rmsnorm(sink.out, sink.residual, tmp, sink.gain, sink.eps)
    return NormedRows(sink.out)


def linear_silu_mul(out: torch.Tensor, x: torch.Tensor | ScaledRows, w: torch.Tensor,
                    bias: torch.Tensor | None, scratch) -> None:
    """``out = silu(x @ wg.T) * (x @ wu.T)`` with ``wg`` the first half of ``w``'s rows and
    ``wu`` the second (biases likewise).  Few rows of bfloat16 run as one weight-streaming
    kernel; otherwise ``scratch()`` gives the ``[M, 2I]`` buffer for the two-kernel form."""
    if isinstance(x, ScaledRows):
        _fused_skinny(out, x, w, bias, gated=True)
        return
    M, K = x.shape
    I = w.shape[0] // 2
    if w.shape != (2 * I, K) or out.shape != (M, I):
        raise KernelError("linear_silu_mul: shapes do not match")
    if (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
            and x.is_cuda and _skinny_operands_ok(x, w)
            and M <= FOLD_ROWS):
        if M == 0:
            return
        if bias is not None and (bias.dtype != torch.bfloat16 or bias.shape != (2 * I,)):
            raise KernelError("linear_silu_mul: bias must be bfloat16 [2I]")
        w_ptr, packed = _streamed(w, I)
        _check(load().kvc_gemm_skinny_silu_mul_bf16(
            out.data_ptr(), x.data_ptr(), w_ptr, None if bias is None else _dev(bias, "bias"),
            M, I, K, x.stride(0), out.stride(0), packed, _stream()), "kvc_gemm_skinny_silu_mul_bf16")
        return
    if (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
            and x.is_cuda and mid_operands_ok(x, w) and out.stride(1) == 1
            and mid_rows_ok(M, bool(_streamed(w, I)[1]), MID_ROWS_GATED)):
        # 17 to 128 rows: the waves of a block share the rows through LDS
        gemm_mid(out, x, w, bias, mode=1)
        return
    gate_up = scratch()
    linear(gate_up, x, w, bias)
    silu_mul(out, gate_up)


def linear(out: torch.Tensor | ResidualSink, x: torch.Tensor | ScaledRows, w: torch.Tensor,
           bias: torch.Tensor | None = None) -> ScaledRows | None:
    """``out = x @ w.T (+ bias)``.  float32 runs the library's own true-float32 kernel.
    bfloat16 with few rows runs the weight-streaming matrix-core kernel; more rows run the
    vendor matrix product through torch.  All sum in float32, and a float32 ``out`` receives
    the sums unrounded on either path.  With a :class:`ScaledRows` for ``x`` or a :class:`ResidualSink` for ``out``
    (few rows of bfloat16 only) the norm before or after the product is folded into it; a
    sink returns the :class:`ScaledRows` it made, or, in a step of 17 to 192 rows, where it
    finishes the norm itself, :class:`NormedRows`."""
    if isinstance(out, ResidualSink) and out.slices is not None:
        if isinstance(x, ScaledRows):
            raise KernelError("linear: a sink that finishes the norm itself takes plain rows")
        return _sink_mid(out, x, w, bias)
    if isinstance(x, ScaledRows) or isinstance(out, ResidualSink):
        return _fused_skinny(out, x, w, bias, gated=False)
    if x.dtype == torch.float32:
        gemm_f32(out, x, w, bias)
        return
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or not x.is_cuda:
        raise KernelError(f"linear: unsupported operands {x.dtype}/{w.dtype} on {x.device}")
    if x.shape[0] == 0:
        return
    M, K = x.shape
    N = w.shape[0]
    kernel = choose_product(M, N, K, few_rows_ok=_skinny_operands_ok(x, w),
                            shared_rows_ok=mid_operands_ok(x, w) and out.stride(1) == 1)
    if kernel == "few rows":
        gemm_skinny_bf16(out, x, w, bias)
        return
    if kernel == "shared rows":
        gemm_mid(out, x, w, bias, mode=0)
        return
    if out.dtype == torch.float32:
        # the vendor product with float32 sums stored as they are (no rounding to bfloat16)
        if out.stride(1) != 1 or not out.is_contiguous():
            raise KernelError("linear: a float32 result of bfloat16 operands must be contiguous")
        torch.mm(x, w.t(), out_dtype=torch.float32, out=out)
        if bias is not None:
            out.add_(bias.to(torch.float32))
        return
    if out.dtype != torch.bfloat16:
        raise KernelError(f"linear: unsupported result type {out.dtype}")
    if bias is None:
        torch.mm(x, w.t(), out=out)
    else:
        torch.addmm(bias, x, w.t(), out=out)


def choose_product(M: int, N: int, K: int, *, few_rows_ok: bool = True, shared_rows_ok: bool = True) -> str:
    """Which kernel multiplies ``M`` rows of bfloat16 by an ``[N, K]`` matrix when nothing is
    folded into the product: ``"few rows"`` (``gemm_skinny_bf16``: every wave streams its own
    weight rows), ``"shared rows"`` (``gemm_mid``: the waves of a block share the rows through
    LDS) or ``"vendor"`` (the vendor's product through torch).  The one place where row counts
    and matrix sizes decide this; parts do not.  Measured on an MI355X with N x K from 4096 x
    4096 to 128256 x 4096 and 8192 x 28672: the few-row kernel wins up to 8 rows everywhere,
    up to 12 rows unless K is very long, up to 16 rows unless the output is as wide as a
    vocabulary, and up to 32 rows for small matrices; from 17 to 64 rows the shared-row
    kernel wins for outputs as wide as a vocabulary (215 against 231 us at 64 rows of 128256
    x 4096) and the vendor's product is as fast or faster otherwise, as it is beyond 64 rows.
    The flags say whether the operands' alignment and strides allow each kernel."""
    if few_rows_ok and M <= SKINNY_MAX_ROWS and (
            M <= 8 or (M <= 12 and K <= 8192) or (M <= SKINNY_PREFERRED_ROWS and K <= 8192 and N < 65536)
            or (M <= 32 and K <= 4096 and N <= 4096)):
        return "few rows"
    if shared_rows_ok and SKINNY_PREFERRED_ROWS < M <= MID_ROWS_WIDE and N >= 65536:
        return "shared rows"
    return "vendor"


def table_update(table: torch.Tensor, triples: torch.Tensor, n: int) -> None:
    if triples.numel() < 3 * n:
        raise KernelError("table_update: triples too short")
    _check(load().kvc_table_update(_dev(table, "table", torch.int32), table.shape[1], table.shape[0],
                                   _dev(triples, "triples", torch.int32), n, _stream()),
           "kvc_table_update")


def argmax(out: torch.Tensor, logits: torch.Tensor, part_val: torch.Tensor | None = None,
           part_idx: torch.Tensor | None = None) -> None:
    """``part_val`` (float32) and ``part_idx`` (int32) of equal length are an optional
    workspace that lets several blocks search one long row."""
    S, V = logits.shape
    if out.numel() < S or logits.stride(1) != 1 or logits.dtype != torch.float32 or not logits.is_cuda:
        raise KernelError("argmax: expects float32 GPU logits [S, V] and S outputs")
    pv = pi = None
    cap = 0
    if part_val is not None and part_idx is not None:
        pv, pi = _dev(part_val, "part_val", torch.float32), _dev(part_idx, "part_idx", torch.int32)
        cap = min(part_val.numel(), part_idx.numel())
    _check(load().kvc_argmax(_dev(out, "out", torch.int32), logits.data_ptr(), S, V,
                             logits.stride(0), pv, pi, cap, _stream()), "kvc_argmax")


def sample_workspace_words(S: int, V: int) -> int:
    """64-bit words of workspace with which ``sample`` deals each row to several blocks
    (0 for rows too short to gain from it)."""
    return int(load().kvc_sample_workspace_words(S, V))


def sample(out: torch.Tensor, logits: torch.Tensor, *, temperature: torch.Tensor,
           top_k: torch.Tensor, top_p: torch.Tensor, seed_lo: torch.Tensor, seed_hi: torch.Tensor,
           index: torch.Tensor, workspace: torch.Tensor | None = None, filters: int = 3) -> None:
    """``workspace``: int64, ``sample_workspace_words(S, V)`` values or more, lets several
    blocks work on a row (the same draws, sooner); ``filters`` says which of top-k (1) and
    top-p (2) some row uses."""
    S, V = logits.shape
    if logits.stride(1) != 1 or logits.dtype != torch.float32 or not logits.is_cuda:
        raise KernelError("sample: expects float32 GPU logits [S, V]")
    for t, name in ((out, "out"), (temperature, "temperature"), (top_k, "top_k"), (top_p, "top_p"),
                    (seed_lo, "seed_lo"), (seed_hi, "seed_hi"), (index, "index")):
        if t.numel() < S or t.element_size() != 4:
            raise KernelError(f"sample: {name} must hold {S} 32-bit values")
    _check(load().kvc_sample(_dev(out, "out", torch.int32), logits.data_ptr(), S, V, logits.stride(0),
                             _dev(temperature, "temperature", torch.float32),
                             _dev(top_k, "top_k", torch.int32), _dev(top_p, "top_p", torch.float32),
                             _dev(seed_lo, "seed_lo"), _dev(seed_hi, "seed_hi"), _dev(index, "index"),
                             None if workspace is None else _dev(workspace, "workspace", torch.int64),
                             0 if workspace is None else workspace.numel(), int(filters),
                             _stream()), "kvc_sample")
