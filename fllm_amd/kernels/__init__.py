"""The kernel library seen from Python: `Ops` wraps the C ABI of csrc/api.h.

Every method checks on the host that tensors are on the GPU, dense, of the element type and the
shape the kernel assumes, before anything is launched.  There is no other implementation: if the
library cannot be loaded or built, constructing `Ops` raises.
"""
from __future__ import annotations

import ctypes
import weakref
from typing import Dict, NamedTuple, Optional, Sequence, Tuple

import torch

from . import build as _build

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}
OUT_STORE, OUT_STORE_F32, OUT_ADD_F32 = 0, 1, 2


class KernelError(RuntimeError):
    pass


class SampleRow(ctypes.Structure):
    _fields_ = [("temperature", ctypes.c_float), ("top_p", ctypes.c_float), ("top_k", ctypes.c_int32),
                ("min_p", ctypes.c_float), ("seed", ctypes.c_uint64), ("draw", ctypes.c_uint64)]


class PreparedNorm(NamedTuple):
    """What `Ops.linear_add_prepare` leaves for the RMSNorm that reads the residual stream next: the rows times the
    norm's weight in bfloat16, and every row's sum of squares in `parts` parts a row."""
    x: torch.Tensor
    ssq: torch.Tensor
    parts: int


class AdjustLists(ctypes.Structure):
    """FllmAdjustLists: device addresses of the lists that the row records of `adjust_logits` point into."""
    _fields_ = [(name, ctypes.c_void_p) for name in ("seen_ids", "seen_counts", "bias_ids", "bias_values", "blocked_ids",
                                                     "allowed_ids", "if_last", "then_blocked")]


SAMPLE_ROW_BYTES = ctypes.sizeof(SampleRow)
ADJUST_ROW_WORDS = 14         # int32 words of one FllmAdjustRow
assert SAMPLE_ROW_BYTES == 32

_lib = None


ABI_VERSION = 17


def load_library(build_if_missing: bool = True):
    """The loaded library; builds it first when there is none that matches the sources."""
    global _lib
    if _lib is not None:
        return _lib
    path = _build.find_library()
    if path is None:
        if not build_if_missing:
            raise KernelError("the HIP kernel library is not built (run `python -m fllm_amd.kernels.build`)")
        path = _build.build()
    try:
        lib = ctypes.CDLL(path)
    except OSError as exc:
        raise KernelError(f"cannot load the HIP kernel library {path}: {exc}") from None
    c_int, c_void, c_float, c_size = ctypes.c_int, ctypes.c_void_p, ctypes.c_float, ctypes.c_size_t
    lib.fllm_last_error.restype = ctypes.c_char_p
    lib.fllm_abi_version.restype = c_int
    if lib.fllm_abi_version() != ABI_VERSION:
        raise KernelError(f"the HIP kernel library {path} has interface version {lib.fllm_abi_version()}, this package needs "
                          f"{ABI_VERSION}: build it again (python -m fllm_amd.kernels.build)")
    sig = {
        "fllm_embed": [c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_float, c_void],
        "fllm_rmsnorm": [c_void, c_void, c_void, c_void, c_int, c_int, c_float, c_int, c_void],
        "fllm_linear": [c_void, c_int, c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_void],
        "fllm_swiglu": [c_void, c_void, c_int, c_int, c_int, c_void],
        "fllm_add_residual": [c_void, c_void, c_int, c_int, c_int, c_void],
        "fllm_add_rmsnorm": [c_void, c_void, c_int, c_void, c_void, c_int, c_int, c_float, c_int, c_void],
        "fllm_rope_kv_store": [c_void, c_void, c_void, c_void, c_int, c_void, c_void, c_int, c_void, c_void, c_int,
                               c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void],
        "fllm_attention": [c_void, c_int, c_void, c_void, c_void, c_int, c_void, c_void, c_void, c_int, c_void, c_int,
                           c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_void, c_int, c_int, c_int, c_void, c_size,
                           c_void],
        "fllm_postnorm_add": [c_void, c_void, c_int, c_int, c_void, c_void, c_float, c_int, c_void, c_float, c_void, c_int, c_int, c_int, c_void],
        "fllm_route_topk": [c_void, c_int, c_void, c_int, c_int, c_int, c_int, c_void, c_void, c_int, c_int, c_float, c_int, c_void],
        "fllm_short_conv": [c_void, c_void, c_void, c_void, c_void, c_void, c_int, c_void, c_int, c_int, c_int, c_int, c_void],
        "fllm_norm_short_conv": [c_void, c_void, c_float, c_void, c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_void],
        "fllm_linear_attention": [c_void, c_void, c_void, c_int, c_void, c_void, c_void, c_void, c_void, c_void, c_int, c_void, c_int,
                                  c_int, c_int, c_int, c_int, c_int, c_int, c_void, c_void],
        "fllm_gated_norm": [c_void, c_int, c_void, c_float, c_void, c_int, c_void, c_int, c_int, c_int, c_void],
        "fllm_polynorm": [c_void, c_int, c_void, c_float, c_void, c_int, c_int, c_int, c_void],
        "fllm_head_norm_kv_store": [c_void, c_int, c_float, c_int, c_void, c_void, c_void, c_int, c_void, c_void, c_int, c_int, c_int,
                                    c_int, c_int, c_int, c_int, c_int, c_int, c_void],
        "fllm_experts_gate_up": [c_void, c_int, c_void, c_void, c_int, c_int, c_void, c_int, c_int, c_int, c_void, c_float, c_float,
                                 c_float, c_int, c_void],
        "fllm_experts_down": [c_void, c_void, c_int, c_void, c_int, c_int, c_int, c_void, c_int, c_void],
        "fllm_experts_grouped": [c_void, c_int, c_void, c_void, c_int, c_int, c_void, c_void, c_int, c_int, c_int, c_int, c_void, c_void,
                                 c_void, c_void, c_void, c_float, c_float, c_float, c_void],
        "fllm_attention_sloped": [c_void, c_int, c_void, c_void, c_void, c_int, c_void, c_void, c_void, c_int, c_void, c_int,
                                  c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_void, c_void],
        "fllm_norm_linear": [c_void, c_void, c_float, c_void, c_void, c_void, c_int, c_int, c_int, c_void],
        "fllm_norm_gate_up_swiglu": [c_void, c_void, c_float, c_void, c_void, c_void, c_int, c_int, c_int, c_void],
        "fllm_norm_gate_up_glu": [c_void, c_void, c_float, c_void, c_void, c_void, c_int, c_int, c_int, c_float, c_float, c_float,
                                  c_void],
        "fllm_gate_up_glu": [c_void, c_int, c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_float, c_float, c_float, c_void],
        "fllm_norm_qkv_rope_store": [c_void, c_void, c_float, c_void, c_void, c_void, c_void, c_void, c_void, c_int, c_void,
                                     c_void, c_int, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void],
        "fllm_argmax": [c_void, c_void, c_int, c_int, c_void],
        "fllm_gate_up_swiglu": [c_void, c_int, c_void, c_void, c_void, c_int, c_int, c_int, c_void],
        "fllm_linear_add_normed": [c_void, c_int, c_void, c_void, c_void, c_int, c_int, c_int, c_void, c_void, c_void, c_void, c_void, c_void],
        "fllm_tile_weights": [c_void, c_void, c_int, c_int, c_void],
        "fllm_tile_weights_gate_up": [c_void, c_void, c_int, c_int, c_void],
        "fllm_gate_up_swiglu_tiled": [c_void, c_int, c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_void],
        "fllm_linear_add_tiled": [c_void, c_int, c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_void],
        "fllm_linear_f32_tiled": [c_void, c_int, c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_void],
        "fllm_scaled_gate_up_swiglu": [c_void, c_void, c_int, c_float, c_void, c_void, c_void, c_int, c_int, c_int, c_void, c_void],
        "fllm_scaled_qkv_rope_store": [c_void, c_void, c_int, c_float, c_void, c_void, c_void, c_void, c_void, c_void, c_int, c_void,
                                       c_void, c_int, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void, c_void],
        "fllm_prepare_norm": [c_void, c_void, c_void, c_void, c_int, c_int, c_void],
        "fllm_carry_ids": [c_void, c_void, c_void, c_int, c_int, c_void],
        "fllm_sample": [c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_void],
        "fllm_adjust_logits": [c_void, c_int, c_int, c_void, c_void, c_void, c_void],
        "fllm_logprobs": [c_void, c_int, c_int, c_void, c_int, c_void, c_int, c_void, c_void, c_void],
        "fllm_logprobs_processed": [c_void, c_int, c_int, c_void, c_int, c_void, c_void, c_int, c_void, c_void, c_void],
        "fllm_rmsnorm_pair": [c_void, c_void, c_void, c_void, c_void, c_int, c_int, c_float, c_float, c_int, c_void],
        "fllm_glu_clamped": [c_void, c_void, c_int, c_int, c_float, c_float, c_float, c_int, c_void],
        "fllm_scale_f32": [c_void, c_size, c_float, c_void],
        "fllm_stream_add": [c_void, c_void, c_void, c_int, c_int, c_float, c_void, c_int, c_int, c_void],
        "fllm_qk_norm_rope_store": [c_void, c_int, c_void, c_void, c_float, c_void, c_void, c_void, c_void, c_int, c_void, c_void,
                                    c_int, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_void],
        "fllm_talking_attention": [c_void, c_void, c_int, c_void, c_void, c_void, c_int, c_void, c_void, c_void, c_int, c_void,
                                   c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_int,
                                   c_int, c_void, ctypes.c_size_t, c_int, c_void],
        "fllm_normed_rope_store": [c_void, c_int, c_int, c_void, c_void, c_float, c_void, c_void, c_void, c_void, c_int, c_void, c_void,
                                   c_int, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                   c_void],
        "fllm_pool_blocks": [c_void, c_void, c_void, c_void, c_void, c_int, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int,
                             c_int, c_int, c_void],
        "fllm_pooled_window_attention": [c_void, c_int, c_void, c_void, c_void, c_void, c_void, c_int, c_void, c_void, c_void, c_int, c_void,
                                         c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_int, c_int, c_void],
        "fllm_sigmoid_attention": [c_void, c_int, c_void, c_void, c_void, c_int, c_void, c_void, c_void, c_int, c_void, c_int, c_int,
                                   c_int, c_int, c_int, c_int, c_float, c_float, c_void, c_void, c_void, c_float, c_int, c_int, c_int,
                                   c_int, c_void],
        "fllm_rotate_scale": [c_void, c_int, c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
                              c_void],
        "fllm_group_norm_gate": [c_void, c_int, c_float, c_int, c_void, c_int, c_void, c_int, c_int, c_int, c_int, c_void],
        "fllm_weighted_sum": [c_void, c_void, c_float, c_void, c_float, c_size, c_int, c_void],
        "fllm_stream_concat": [c_void, c_void, c_void, c_int, c_float, c_void, c_int, c_int, c_int, c_void],
        "fllm_relu_squared": [c_void, c_void, c_size, c_int, c_void],
        "fllm_route_grouped": [c_void, c_int, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_void, c_void, c_float, c_int,
                               c_void],
        "fllm_experts_grouped_ungated": [c_void, c_int, c_void, c_int, c_int, c_void, c_void, c_int, c_int, c_int, c_int, c_void, c_void,
                                         c_void, c_void, c_void],
        "fllm_experts_up": [c_void, c_int, c_void, c_int, c_int, c_void, c_int, c_int, c_int, c_void, c_int, c_void],
    }
    for name, args in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = c_int
    lib.fllm_fused_decode_supported.argtypes = [c_int, c_int]
    lib.fllm_fused_decode_supported.restype = c_int
    lib.fllm_set_option.argtypes = [ctypes.c_char_p, c_int]
    lib.fllm_set_option.restype = c_int
    lib.fllm_set_device_workspace.argtypes = [c_void, c_size]
    lib.fllm_set_device_workspace.restype = c_int
    lib.fllm_probe_read.argtypes = [c_void, c_size, c_void, c_int, c_void]
    lib.fllm_probe_read.restype = c_int
    lib.fllm_probe_mfma_bf16.argtypes = [c_void, c_int, c_int, c_void]
    lib.fllm_probe_mfma_bf16.restype = ctypes.c_double
    lib.fllm_random_fill.argtypes = [c_void, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint32, c_int, c_int, c_void]
    lib.fllm_random_fill.restype = c_int
    lib.fllm_weight_tiles_supported.argtypes = [c_int, c_int]
    lib.fllm_weight_tiles_supported.restype = c_int
    lib.fllm_weight_tiles_elements.argtypes = [c_int, c_int]
    lib.fllm_weight_tiles_elements.restype = c_size
    lib.fllm_weight_tiles_elements_gate_up.argtypes = [c_int, c_int]
    lib.fllm_weight_tiles_elements_gate_up.restype = c_size
    lib.fllm_set_fast_kernels.argtypes = [c_int]
    lib.fllm_set_fast_kernels.restype = None
    lib.fllm_experts_grouped_plane_floats.argtypes = [c_int, c_int, c_int, c_int]
    lib.fllm_experts_grouped_plane_floats.restype = c_size
    lib.fllm_linear_attention_carried_floats.argtypes = [c_int, c_int, c_int, c_int, c_int]
    lib.fllm_linear_attention_carried_floats.restype = c_size
    lib.fllm_experts_grouped_work_ints.argtypes = [c_int, c_int]
    lib.fllm_experts_grouped_work_ints.restype = c_size
    lib.fllm_attention_workspace_bytes.argtypes = [c_int, c_int, c_int, c_int, c_int]
    lib.fllm_attention_workspace_bytes.restype = c_size
    _lib = lib
    return lib


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dense(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    # (every launch checks its operands: the messages are put together only when a check fails)
    if not t.is_cuda:
        raise KernelError(f"{name} must be on the GPU")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, is {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name} must have shape {tuple(shape)}, has {tuple(t.shape)}")


class Ops:
    """Launches kernels on the current torch stream of the tensors' device.

    `library_gemm_from`: bfloat16 products of at least this many rows (prompt portions, large decode batches) go
    to the vendor's GEMM library through `torch.matmul`, as the reference sends its prompt-sized dense products
    to a library (rust/engine/cuda/cublaslt_gemm.cu:1-20).  None: every product runs the hand-written kernels.
    `fused_decode_rows`: up to this many rows a step uses the kernels that fold the norm, rotary, cache store and
    activation into the product (the kernels take up to 64 rows; beyond 16 the library products with separate small
    kernels are faster at the sizes measured)."""

    def __init__(self, library_gemm_from: Optional[int] = 17, fused_decode_rows: int = 16):
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: the engine runs on gfx950 only")
        self.lib = load_library()
        self.library_gemm_from = library_gemm_from
        self.fused_decode_rows = int(fused_decode_rows)
        self._device_workspace(torch.cuda.current_device())

    _WORKSPACE_BYTES = 192 << 20
    _workspaces = {}         # device index -> tensor; lives as long as the process: the library keeps its address

    def _device_workspace(self, device: int) -> None:
        """Hands the library the memory in which workgroups of one kernel meet (counters, partial sums): once per device."""
        if device in Ops._workspaces:
            return
        with torch.cuda.device(device):
            buf = torch.zeros(Ops._WORKSPACE_BYTES, dtype=torch.uint8, device=f"cuda:{device}")
            torch.cuda.synchronize()
            self._check(self.lib.fllm_set_device_workspace(_ptr(buf), buf.numel()))
        Ops._workspaces[device] = buf

    # ---- tile-major copies of weights for decode steps --------------------------------------------------
    _tiles: Dict[int, Tuple[tuple, torch.Tensor]] = {}     # address of a weight matrix -> (its shape, its tile-major copy)

    def tile_for_decode(self, w: torch.Tensor, gate_up: bool = False) -> bool:
        """Keeps beside `w` (bfloat16 [N, K] on the GPU) a copy in the order in which the products of decode steps read
        it (`fllm_tile_weights`): `linear(..., accumulate=True)`, `linear_add_prepare`, the forms behind a prepared norm
        and `linear` with float32 logits find it by the matrix's address and use it for steps of up to 64 rows (sums into a
        float32 `out` and `gate_up_swiglu`: up to 128).  `gate_up`: w is [gate; up] and the copy holds 8 gate rows and the
        same 8 up rows a tile (`fllm_tile_weights_gate_up`), for `norm_gate_up_swiglu` and `gate_up_swiglu`.  The copy is
        given up with `w`.  False: nothing was made (another type or place, a shape the kernels do not take tiles of)."""
        if not (w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_contiguous()):
            return False
        N, K = w.shape
        if not self.lib.fllm_weight_tiles_supported(N, K) or (gate_up and N % 2 != 0):
            return False
        key = w.data_ptr()
        kind = (N, K, bool(gate_up))
        if key in Ops._tiles and Ops._tiles[key][0] == kind:
            return True
        with torch.cuda.device(w.device):
            if gate_up:
                tiles = torch.empty(int(self.lib.fllm_weight_tiles_elements_gate_up(N // 2, K)), dtype=torch.bfloat16, device=w.device)
                self._check(self.lib.fllm_tile_weights_gate_up(_ptr(w), _ptr(tiles), N // 2, K, self._stream()))
            else:
                tiles = torch.empty(int(self.lib.fllm_weight_tiles_elements(N, K)), dtype=torch.bfloat16, device=w.device)
                self._check(self.lib.fllm_tile_weights(_ptr(w), _ptr(tiles), N, K, self._stream()))
        Ops._tiles[key] = (kind, tiles)
        weakref.finalize(w, Ops._tiles.pop, key, None)
        return True

    def _tiles_of(self, w: torch.Tensor, gate_up: bool = False) -> Optional[torch.Tensor]:
        held = Ops._tiles.get(w.data_ptr())
        return held[1] if held is not None and held[0] == (w.shape[0], w.shape[1], bool(gate_up)) else None

    # 17 to 128 rows beside the GEMM library: with the tile-major copies the own products of the feed-forward (gate/up
    # with its SwiGLU epilogue, down with the residual sum) are faster than the library's products and the SwiGLU kernel
    # (measured at the 8B sizes, 64 / 32 rows: gate/up 48 / 44 us against 55 / 53, down 34 / 28 against 40 / 31; at the 1B
    # sizes, 67 MB of gate and up weights, the library is 3 % of a 64-row step ahead, hence the same floor on the bytes
    # as for `prefers_own_gate_up`)
    def own_feed_forward(self, rows: int, w_gate_up: torch.Tensor, w_down: torch.Tensor) -> bool:
        """Whether a bfloat16 step of 17 to 128 rows whose products would go to the GEMM library should take
        `gate_up_swiglu` and `linear(..., accumulate=True)` for its feed-forward instead: when both matrices have their
        tile-major copies."""
        return (self.library_gemm_from is not None and self.library_gemm_from <= rows <= self.GATE_UP_SWIGLU_TILED_ROWS and bool(Ops._tiles)
                and (rows <= 64 or (w_gate_up.shape[1] % 256 == 0 and w_down.shape[1] % 256 == 0))
                and w_gate_up.numel() * w_gate_up.element_size() >= self.OWN_GATE_UP_BYTES
                and self._tiles_of(w_gate_up, gate_up=True) is not None and self._tiles_of(w_down) is not None)

    def set_fast_kernels(self, on: bool) -> None:
        """Off: bfloat16 calls run the plain kernels (tests compare the two)."""
        self.lib.fllm_set_fast_kernels(1 if on else 0)

    def set_option(self, name: str, value: int) -> None:
        """Switches a kernel variant, for measurements and for tests that compare variants."""
        self._check(self.lib.fllm_set_option(name.encode(), int(value)))

    def _check(self, code: int) -> None:
        if code != 0:
            raise KernelError(self.lib.fllm_last_error().decode("utf-8", "replace"))

    _streams = {}            # device index -> the stream on which this process launches the kernels of that device

    @staticmethod
    def _stream() -> int:
        """The current stream.  Kernels of one device meet in that device's workspace (counters that each launch leaves
        at zero, partial results behind them), so launches on one device must not overlap: all of them go to one stream
        (a stream that is capturing a graph stands for the stream the graph will be replayed on).  A launch on a second
        stream of the same device is refused."""
        raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        if raw is not None:               # the handle without a Stream object around it (a launch asks for it every time)
            device = torch.cuda.current_device()
            handle = raw(device)
        else:
            stream = torch.cuda.current_stream()
            handle, device = stream.cuda_stream, stream.device_index
        seen = Ops._streams.get(device)
        if seen is None:
            if not torch.cuda.is_current_stream_capturing():
                Ops._streams[device] = handle
        elif handle != seen and not torch.cuda.is_current_stream_capturing():
            raise KernelError(f"kernels of device {device} were launched on stream {seen:#x} before and are now asked for on "
                              f"stream {handle:#x}: they share the device workspace and must stay on one stream")
        return handle

    def random_fill(self, out: torch.Tensor, key, kind: int) -> torch.Tensor:
        """Fills `out` with the random tensor of `key` (two 32-bit words): kind 0 normal numbers of deviation 0.02, kind 1
        norm weights; the generator of `fllm_amd.weights.random_init`."""
        _dense(out, "out")
        _need(out.dtype in _DTYPE_CODE, f"out dtype {out.dtype} unsupported")
        with torch.cuda.device(out.device):
            self._check(self.lib.fllm_random_fill(_ptr(out), out.numel(), int(key[0]), int(key[1]), int(kind),
                                                  _DTYPE_CODE[out.dtype], self._stream()))
        return out

    def embed(self, ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
        rows = ids.numel()
        vocab, width = table.shape
        _dense(ids, "ids", torch.int32)
        _dense(table, "table")
        _need(table.dtype in _DTYPE_CODE, f"table dtype {table.dtype} unsupported")
        _dense(out, "out", torch.float32, (rows, width))
        self._check(self.lib.fllm_embed(_ptr(ids), _ptr(table), _ptr(out), rows, width, vocab, _DTYPE_CODE[table.dtype],
                                        float(scale), self._stream()))
        return out

    def rmsnorm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        width = x.shape[-1]
        _dense(x, "x", torch.float32)
        _dense(weight, "weight", torch.float32, (width,))
        count = x.shape[0] if rows is None else rows.numel()
        if rows is not None:
            _dense(rows, "rows", torch.int32)
        _dense(out, "out", None, (count, width))
        _need(out.dtype in _DTYPE_CODE, f"out dtype {out.dtype} unsupported")
        self._check(self.lib.fllm_rmsnorm(_ptr(x), _ptr(rows), _ptr(weight), _ptr(out), count, width, float(eps),
                                          _DTYPE_CODE[out.dtype], self._stream()))
        return out

    def add_rmsnorm(self, x: torch.Tensor, branch: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor) -> torch.Tensor:
        """x += branch (float32 sum, in place), out = rmsnorm(x): the residual add and the norm after it in one pass."""
        rows, width = x.shape
        _dense(x, "x", torch.float32)
        _dense(branch, "branch", None, (rows, width))
        _need(branch.dtype in _DTYPE_CODE, f"branch dtype {branch.dtype} unsupported")
        _dense(weight, "weight", torch.float32, (width,))
        _dense(out, "out", None, (rows, width))
        _need(out.dtype in _DTYPE_CODE, f"out dtype {out.dtype} unsupported")
        self._check(self.lib.fllm_add_rmsnorm(_ptr(x), _ptr(branch), _DTYPE_CODE[branch.dtype], _ptr(weight), _ptr(out), rows,
                                              width, float(eps), _DTYPE_CODE[out.dtype], self._stream()))
        return out

    def linear(self, x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None,
               accumulate: bool = False) -> torch.Tensor:
        """out = x @ w.T (+ bias); `accumulate` adds into a float32 `out` instead of storing."""
        _need(x.dim() == 2 and w.dim() == 2 and out.dim() == 2, "linear takes matrices")
        M, K = x.shape
        N = w.shape[0]
        _need(w.shape[1] == K, f"w has {w.shape[1]} columns, x has {K}")
        _need(x.is_cuda and w.is_cuda and out.is_cuda, "linear operands must be on the GPU")
        _need(x.dtype == w.dtype and x.dtype in _DTYPE_CODE, f"x is {x.dtype}, w is {w.dtype}")
        _need(x.stride(1) == 1 and out.stride(1) == 1 and w.is_contiguous(), "linear operands must be row-major")
        _need(tuple(out.shape) == (M, N), f"out must have shape {(M, N)}, has {tuple(out.shape)}")
        if accumulate:
            _need(out.dtype == torch.float32, "accumulate needs a float32 out")
            mode = OUT_ADD_F32
        elif out.dtype == x.dtype:
            mode = OUT_STORE
        else:
            _need(out.dtype == torch.float32, f"out must be {x.dtype} or float32")
            mode = OUT_STORE_F32
        if bias is not None:
            _dense(bias, "bias", torch.float32, (N,))
        ldx = x.stride(0) if M > 1 else K
        ldo = out.stride(0) if M > 1 else N
        tiles = (self._tiles_of(w) if Ops._tiles and ((mode == OUT_ADD_F32 and M <= self.ADD_KERNEL_ROWS) or (mode == OUT_STORE_F32 and M <= 64))
                 else None)
        if tiles is not None and ldx % 8 == 0 and K % 8 == 0 and (M <= 64 or K % 256 == 0):
            entry = self.lib.fllm_linear_add_tiled if mode == OUT_ADD_F32 else self.lib.fllm_linear_f32_tiled
            self._check(entry(_ptr(x), ldx, _ptr(w), _ptr(tiles), _ptr(bias), _ptr(out), ldo, M, N, K, self._stream()))
            return out
        if (self.library_gemm_from is not None and M >= self.library_gemm_from and x.dtype == torch.bfloat16
                and bias is None):
            if mode == OUT_STORE:
                torch.matmul(x, w.t(), out=out)
            elif mode == OUT_STORE_F32:
                torch.mm(x, w.t(), out_dtype=torch.float32, out=out)     # bfloat16 operands, float32 sums stored as they are
            else:
                self.add_residual(out, torch.matmul(x, w.t()))
            return out
        self._check(self.lib.fllm_linear(_ptr(x), ldx, _ptr(w), _ptr(bias), _ptr(out), ldo, M, N, K, _DTYPE_CODE[x.dtype],
                                         mode, self._stream()))
        return out

    # ---- fused forms of decode steps (bfloat16, at most 64 rows) ---------------------------------
    def fused_decode_supported(self, rows: int, width: int) -> bool:
        """Whether a step of `rows` rows should take the fused forms: the kernels can (1..64 rows, widths in steps of 8)
        and `fused_decode_rows` lets them."""
        return rows <= self.fused_decode_rows and self._fused_kernels_take(rows, width)

    def _fused_kernels_take(self, rows: int, width: int) -> bool:
        return bool(self.lib.fllm_fused_decode_supported(int(rows), int(width)))

    def _fused_operands(self, x, norm_weight, w, bias, n_rows_w):
        M, K = x.shape
        _dense(x, "x", torch.float32)
        _dense(norm_weight, "norm_weight", torch.float32, (K,))
        _dense(w, "w", torch.bfloat16, (n_rows_w, K))
        if bias is not None:
            _dense(bias, "bias", torch.float32, (n_rows_w,))
        _need(self._fused_kernels_take(M, K), f"the fused decode kernels take 1..64 rows and widths in steps of 8, not {M} x {K}")
        return M, K

    def norm_linear(self, x, norm_weight, eps, w, out, bias=None):
        """out = rmsnorm(x) @ w.T (+ bias); x float32 [M, K], w bfloat16 [N, K], out bfloat16 [M, N]."""
        N = w.shape[0]
        M, K = self._fused_operands(x, norm_weight, w, bias, N)
        _dense(out, "out", torch.bfloat16, (M, N))
        self._check(self.lib.fllm_norm_linear(_ptr(x), _ptr(norm_weight), float(eps), _ptr(w), _ptr(bias), _ptr(out), M, N, K,
                                              self._stream()))
        return out

    PREPARED_NORM_ROWS = 16
    CHUNK_KERNEL_ROWS = 64   # what those kernels take behind a prepared norm
    ADD_KERNEL_ROWS = 128    # and as sums into the residual stream or with the SwiGLU epilogue (beyond 64 rows from the tile-major
                             # copies only): the feed-forward of steps of up to 128 rows, whose down projection the GEMM library
                             # runs on half of the device (96 / 128 rows of the 8B sizes: 39 / 53 us against 63 / 75)
    CHUNK_ROWS = 48          # steps of 17 to this many rows take the fused forms of the kernels that pass the activations through
                             # LDS in chunks (measured at the 8B sizes: 4 to 5 % of a step at 17 and 32 rows, 1 % at 48; from 49
                             # rows on the library's q/k/v and output products beside the own feed-forward are 1 % faster)

    def fused_form(self, rows: int, width: int, w: torch.Tensor, gate_up: bool = False) -> Optional[str]:
        """Which fused kernels serve a product of `rows` rows with the matrix `w` behind an RMSNorm of `width`:
        "resident" (up to `fused_decode_rows` rows), "chunks" (17 to 64 rows: they need the norm prepared, by
        `linear_add_prepare` or `prepare_norm`, and the tile-major copy of `w`) or None."""
        if self.fused_decode_supported(rows, width):
            return "resident"
        if (self.fused_decode_rows < rows <= self.CHUNK_ROWS and (self.library_gemm_from is None or rows >= self.library_gemm_from)
                and self.fused_decode_rows >= self.PREPARED_NORM_ROWS and width % 256 == 0 and Ops._tiles
                and self._tiles_of(w, gate_up=gate_up) is not None):
            return "chunks"
        return None

    def prepares_norm(self, rows: int, width: int, w: Optional[torch.Tensor] = None) -> bool:
        """Whether `linear_add_prepare` serves a sum into a residual stream of this size: the fused forms are in use,
        up to 16 rows, or up to 64 with the tile-major copy of the matrix `w`; widths in steps of 16."""
        if width % 16 != 0:
            return False
        if rows <= self.PREPARED_NORM_ROWS:
            return self.fused_decode_supported(rows, width)
        return w is not None and self.fused_form(rows, w.shape[1], w) == "chunks"      # the product's own width counts

    def prepare_norm(self, x: torch.Tensor, norm_weight: torch.Tensor) -> PreparedNorm:
        """What `linear_add_prepare` leaves for an RMSNorm, from float32 rows that no such product wrote (a model's first
        layer): the rows times the norm's weight in bfloat16 and each row's sum of squares as one part."""
        M, K = x.shape
        _dense(x, "x", torch.float32)
        _dense(norm_weight, "norm_weight", torch.float32, (K,))
        xn = torch.empty((M, K), dtype=torch.bfloat16, device=x.device)
        ssq = torch.empty((M,), dtype=torch.float32, device=x.device)
        self._check(self.lib.fllm_prepare_norm(_ptr(x), _ptr(norm_weight), _ptr(xn), _ptr(ssq), M, K, self._stream()))
        return PreparedNorm(xn, ssq, 1)

    def linear_add_prepare(self, x, w, residual, next_norm_weight, bias=None) -> PreparedNorm:
        """residual += x @ w.T (+ bias) as `linear(..., accumulate=True)` does, and in the same kernel what the RMSNorm
        with weight `next_norm_weight` that reads `residual` next would compute first (fllm_linear_add_normed): hand the
        result to `norm_gate_up_swiglu` / `norm_qkv_rope_store` as `prepared`.  x bfloat16 [M <= 64, K], w bfloat16 [N, K],
        residual float32 [M, N], N a multiple of 16."""
        M, K = x.shape
        N = w.shape[0]
        _need(x.is_cuda and x.dtype == torch.bfloat16 and x.dim() == 2 and x.stride(1) == 1, "x must be bfloat16 rows on the GPU")
        _dense(w, "w", torch.bfloat16, (N, K))
        _dense(residual, "residual", torch.float32, (M, N))
        _dense(next_norm_weight, "next_norm_weight", torch.float32, (N,))
        if bias is not None:
            _dense(bias, "bias", torch.float32, (N,))
        _need(1 <= M <= self.ADD_KERNEL_ROWS and N % 16 == 0 and K % 8 == 0,
              f"linear_add_prepare takes 1..128 rows, N in steps of 16 and K in steps of 8, not {M} x {N} x {K}")
        xn = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
        ssq = torch.empty((M * (N // 8),), dtype=torch.float32, device=x.device)
        parts = ctypes.c_int(0)
        self._check(self.lib.fllm_linear_add_normed(_ptr(x), x.stride(0) if M > 1 else K, _ptr(w), _ptr(bias), _ptr(residual), M, N,
                                                    K, _ptr(next_norm_weight), _ptr(xn), _ptr(ssq), ctypes.addressof(parts),
                                                    _ptr(self._tiles_of(w)) if Ops._tiles else None, self._stream()))
        return PreparedNorm(xn, ssq, int(parts.value))

    def _prepared_operands(self, prepared: PreparedNorm, w, bias, n_rows_w):
        M, K = prepared.x.shape
        _dense(prepared.x, "prepared.x", torch.bfloat16)
        _dense(prepared.ssq, "prepared.ssq", torch.float32)
        _need(prepared.parts >= 1 and prepared.ssq.numel() >= M * prepared.parts, "prepared.ssq is shorter than rows x parts")
        _dense(w, "w", torch.bfloat16, (n_rows_w, K))
        if bias is not None:
            _dense(bias, "bias", torch.float32, (n_rows_w,))
        _need(1 <= M <= self.CHUNK_KERNEL_ROWS and K % 8 == 0, f"a prepared norm serves 1..64 rows and widths in steps of 8, not {M} x {K}")
        return M, K

    def _chunk_tiles(self, M: int, K: int, w: torch.Tensor, gate_up: bool = False) -> Optional[torch.Tensor]:
        """The tile-major copy that a prepared norm of more than 16 rows needs; up to 16 rows the kernel streams it
        where there is one and the launch it chooses can."""
        tiles = self._tiles_of(w, gate_up=gate_up) if Ops._tiles else None
        if M <= self.PREPARED_NORM_ROWS:
            return tiles
        _need(tiles is not None and K % 256 == 0,
              f"a prepared norm of {M} rows needs the tile-major copy of the matrix (tile_for_decode) and a width in steps of 256, not {K}")
        return tiles

    def norm_gate_up_swiglu(self, x, norm_weight, eps, w_gate_up, out, bias=None, prepared: Optional[PreparedNorm] = None):
        """out = silu(rmsnorm(x) @ gate.T) * (rmsnorm(x) @ up.T); w_gate_up = [gate; up], out bfloat16 [M, I].
        `prepared`: what `linear_add_prepare` left for this norm, in place of x and norm_weight."""
        two_i = w_gate_up.shape[0]
        _need(two_i % 2 == 0, "w_gate_up needs an even number of rows")
        if prepared is not None:
            M, K = self._prepared_operands(prepared, w_gate_up, bias, two_i)
            _dense(out, "out", torch.bfloat16, (M, two_i // 2))
            self._check(self.lib.fllm_scaled_gate_up_swiglu(_ptr(prepared.x), _ptr(prepared.ssq), prepared.parts, float(eps),
                                                            _ptr(w_gate_up), _ptr(bias), _ptr(out), M, two_i // 2, K,
                                                            _ptr(self._chunk_tiles(M, K, w_gate_up, gate_up=True)), self._stream()))
            return out
        M, K = self._fused_operands(x, norm_weight, w_gate_up, bias, two_i)
        _dense(out, "out", torch.bfloat16, (M, two_i // 2))
        self._check(self.lib.fllm_norm_gate_up_swiglu(_ptr(x), _ptr(norm_weight), float(eps), _ptr(w_gate_up), _ptr(bias),
                                                      _ptr(out), M, two_i // 2, K, self._stream()))
        return out

    GATE_UP_SWIGLU_ROWS = 64          # from the matrix as the checkpoint has it
    GATE_UP_SWIGLU_TILED_ROWS = 128   # from its tile-major copy, widths in steps of 256
    # Beside the GEMM library: up to this many rows, and from this many bytes of gate and up weights on, the own
    # product with the SwiGLU epilogue is faster than the library's product and a SwiGLU kernel behind it (measured at
    # 17 and 32 rows: 6.5 and 4.6 us a layer at 235 MB of weights; slower at 64 rows, and at 67 MB of weights).
    OWN_GATE_UP_ROWS = 32
    OWN_GATE_UP_BYTES = 128 << 20

    def prefers_own_gate_up(self, rows: int, w_gate_up: torch.Tensor) -> bool:
        """Whether a bfloat16 step of `rows` rows whose products go to the GEMM library should still take
        `gate_up_swiglu` for its gate/up product."""
        return (self.library_gemm_from is not None and self.library_gemm_from <= rows <= self.OWN_GATE_UP_ROWS
                and w_gate_up.numel() * w_gate_up.element_size() >= self.OWN_GATE_UP_BYTES)

    def gate_up_swiglu(self, x, w_gate_up, out, bias=None):
        """out = silu(x @ gate.T) * (x @ up.T) for up to 64 bfloat16 rows, up to 128 with the tile-major copy of w_gate_up
        ([gate; up]); out bfloat16 [M, I]."""
        M, K = x.shape
        two_i = w_gate_up.shape[0]
        _need(two_i % 2 == 0, "w_gate_up needs an even number of rows")
        _need(x.dtype == torch.bfloat16 and x.is_cuda and x.stride(1) == 1, "x must be bfloat16 rows on the GPU")
        _dense(w_gate_up, "w_gate_up", torch.bfloat16, (two_i, K))
        if bias is not None:
            _dense(bias, "bias", torch.float32, (two_i,))
        _dense(out, "out", torch.bfloat16, (M, two_i // 2))
        _need(1 <= M <= self.GATE_UP_SWIGLU_TILED_ROWS and K % 8 == 0, f"gate_up_swiglu takes 1..128 rows and widths in steps of 8, not {M} x {K}")
        tiles = self._tiles_of(w_gate_up, gate_up=True) if M >= 17 and Ops._tiles else None
        _need(M <= 64 or (tiles is not None and K % 256 == 0 and x.stride(0) % 8 == 0),
              f"gate_up_swiglu takes more than 64 rows only with the tile-major copy of the matrix and widths in steps of 256, not {M} x {K}")
        if tiles is not None and x.stride(0) % 8 == 0:
            self._check(self.lib.fllm_gate_up_swiglu_tiled(_ptr(x), x.stride(0), _ptr(w_gate_up), _ptr(tiles), _ptr(bias), _ptr(out), M,
                                                           two_i // 2, K, self._stream()))
            return out
        self._check(self.lib.fllm_gate_up_swiglu(_ptr(x), x.stride(0) if M > 1 else K, _ptr(w_gate_up), _ptr(bias), _ptr(out), M,
                                                 two_i // 2, K, self._stream()))
        return out

    def norm_gate_up_glu(self, x, norm_weight, eps, w_gate_up, out, limit: float, alpha: float, up_offset: float, bias=None):
        """`norm_gate_up_swiglu` with the activation's constants as arguments: out = a(g') * (u' + up_offset) with
        a(g) = g * sigmoid(alpha * g), g' = min(gate, limit), u' = clamp(up, -limit, limit) (limit <= 0: nothing is
        clamped), gate and up the two halves of rmsnorm(x) @ w_gate_up.T; x float32 [M <= 64, K], out bfloat16 [M, I]."""
        two_i = w_gate_up.shape[0]
        _need(two_i % 2 == 0, "w_gate_up needs an even number of rows")
        M, K = self._fused_operands(x, norm_weight, w_gate_up, bias, two_i)
        _dense(out, "out", torch.bfloat16, (M, two_i // 2))
        self._check(self.lib.fllm_norm_gate_up_glu(_ptr(x), _ptr(norm_weight), float(eps), _ptr(w_gate_up), _ptr(bias), _ptr(out), M,
                                                   two_i // 2, K, float(limit), float(alpha), float(up_offset), self._stream()))
        return out

    def gate_up_glu(self, x, w_gate_up, out, limit: float, alpha: float, up_offset: float, bias=None):
        """`gate_up_swiglu` with the activation's constants as arguments (see `norm_gate_up_glu`): up to 64 bfloat16 rows,
        up to 128 with the tile-major copy of w_gate_up."""
        M, K = x.shape
        two_i = w_gate_up.shape[0]
        _need(two_i % 2 == 0, "w_gate_up needs an even number of rows")
        _need(x.dtype == torch.bfloat16 and x.is_cuda and x.stride(1) == 1, "x must be bfloat16 rows on the GPU")
        _need(M == 1 or x.stride(0) % 8 == 0, "rows of x must begin on 16 bytes")
        _dense(w_gate_up, "w_gate_up", torch.bfloat16, (two_i, K))
        if bias is not None:
            _dense(bias, "bias", torch.float32, (two_i,))
        _dense(out, "out", torch.bfloat16, (M, two_i // 2))
        _need(1 <= M <= self.GATE_UP_SWIGLU_TILED_ROWS and K % 8 == 0, f"gate_up_glu takes 1..128 rows and widths in steps of 8, not {M} x {K}")
        tiles = self._tiles_of(w_gate_up, gate_up=True) if M >= 17 and Ops._tiles else None
        _need(M <= 64 or (tiles is not None and K % 256 == 0),
              f"gate_up_glu takes more than 64 rows only with the tile-major copy of the matrix and widths in steps of 256, not {M} x {K}")
        self._check(self.lib.fllm_gate_up_glu(_ptr(x), x.stride(0) if M > 1 else K, _ptr(w_gate_up), _ptr(tiles), _ptr(bias), _ptr(out),
                                              M, two_i // 2, K, float(limit), float(alpha), float(up_offset), self._stream()))
        return out

    def norm_qkv_rope_store(self, x, norm_weight, eps, w_qkv, q_out, row_pos, row_seg, tables, cos, sin, k_pages, v_pages,
                            heads, kv_heads, head_dim, rope_dims, page_size, bias=None, prepared: Optional[PreparedNorm] = None):
        """q, k, v = rmsnorm(x) @ w_qkv.T; rotary on pairs (2l, 2l+1) of q and k; q to `q_out`
        (bfloat16 [M, heads * head_dim]), k and v into the pages (None: not stored).
        `prepared`: what `linear_add_prepare` left for this norm, in place of x and norm_weight."""
        if prepared is not None:
            M, K = self._prepared_operands(prepared, w_qkv, bias, (heads + 2 * kv_heads) * head_dim)
        else:
            M, K = self._fused_operands(x, norm_weight, w_qkv, bias, (heads + 2 * kv_heads) * head_dim)
        _dense(q_out, "q_out", torch.bfloat16, (M, heads * head_dim))
        _dense(row_pos, "row_pos", torch.int32, (M,))
        _dense(row_seg, "row_seg", torch.int32, (M,))
        _dense(tables, "tables", torch.int32)
        _need(tables.dim() == 2, "tables must be [segments, pages]")
        _dense(cos, "cos", torch.float32)
        _dense(sin, "sin", torch.float32, tuple(cos.shape))
        _need(cos.dim() == 2 and cos.shape[1] == rope_dims // 2, f"rotary tables must be [positions, {rope_dims // 2}]")
        store = k_pages is not None
        if store:
            pages = k_pages.shape[0]
            _dense(k_pages, "k_pages", torch.bfloat16, (pages, kv_heads, head_dim // 8, page_size, 8))
            _dense(v_pages, "v_pages", torch.bfloat16, (pages, kv_heads, head_dim, page_size))
        if prepared is not None:
            self._check(self.lib.fllm_scaled_qkv_rope_store(
                _ptr(prepared.x), _ptr(prepared.ssq), prepared.parts, float(eps), _ptr(w_qkv), _ptr(bias), _ptr(q_out), _ptr(row_pos),
                _ptr(row_seg), _ptr(tables), tables.shape[1], _ptr(cos), _ptr(sin), rope_dims, _ptr(k_pages), _ptr(v_pages), M, heads,
                kv_heads, head_dim, K, page_size, 1 if store else 0, _ptr(self._chunk_tiles(M, K, w_qkv)), self._stream()))
            return q_out
        self._check(self.lib.fllm_norm_qkv_rope_store(
            _ptr(x), _ptr(norm_weight), float(eps), _ptr(w_qkv), _ptr(bias), _ptr(q_out), _ptr(row_pos), _ptr(row_seg),
            _ptr(tables), tables.shape[1], _ptr(cos), _ptr(sin), rope_dims, _ptr(k_pages), _ptr(v_pages), M, heads, kv_heads,
            head_dim, K, page_size, 1 if store else 0, self._stream()))
        return q_out

    def add_residual(self, residual: torch.Tensor, branch: torch.Tensor) -> torch.Tensor:
        """residual += branch, summed in float32."""
        _dense(residual, "residual", torch.float32)
        _dense(branch, "branch", None, tuple(residual.shape))
        _need(branch.dtype in _DTYPE_CODE and residual.dim() == 2, "add_residual takes matrices of float32 / bfloat16")
        self._check(self.lib.fllm_add_residual(_ptr(residual), _ptr(branch), residual.shape[0], residual.shape[1],
                                               _DTYPE_CODE[branch.dtype], self._stream()))
        return residual

    def swiglu(self, gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        rows, two_i = gate_up.shape
        _need(two_i % 2 == 0, "gate_up needs an even width")
        _dense(gate_up, "gate_up")
        _need(gate_up.dtype in _DTYPE_CODE, f"dtype {gate_up.dtype} unsupported")
        _dense(out, "out", gate_up.dtype, (rows, two_i // 2))
        self._check(self.lib.fllm_swiglu(_ptr(gate_up), _ptr(out), rows, two_i // 2, _DTYPE_CODE[gate_up.dtype],
                                         self._stream()))
        return out

    def rope_kv_store(self, qkv: torch.Tensor, row_pos: torch.Tensor, row_seg: torch.Tensor, tables: torch.Tensor,
                      cos: torch.Tensor, sin: torch.Tensor, k_pages: Optional[torch.Tensor],
                      v_pages: Optional[torch.Tensor], heads: int, kv_heads: int, head_dim: int, rope_dims: int,
                      pairing: int, page_size: int, v_dim: Optional[int] = None, key_chunk: int = 8) -> None:
        """`v_dim`: lanes of a value head where they differ from the keys'; `key_chunk`: values of a key that lie together
        in a page (8; 1 for head sizes that are no multiple of 8)."""
        rows = qkv.shape[0]
        v_dim = head_dim if v_dim is None else int(v_dim)
        _dense(qkv, "qkv", None, (rows, (heads + kv_heads) * head_dim + kv_heads * v_dim))
        _need(qkv.dtype in _DTYPE_CODE, f"dtype {qkv.dtype} unsupported")
        _dense(row_pos, "row_pos", torch.int32, (rows,))
        _dense(row_seg, "row_seg", torch.int32, (rows,))
        _dense(tables, "tables", torch.int32)
        _need(tables.dim() == 2, "tables must be [segments, pages]")
        half = rope_dims // 2
        _dense(cos, "cos", torch.float32)
        _dense(sin, "sin", torch.float32, tuple(cos.shape))
        _need(cos.dim() == 2 and cos.shape[1] == half, f"rotary tables must be [positions, {half}]")
        store = k_pages is not None
        num_pages = 0
        _need(key_chunk > 0 and head_dim % key_chunk == 0, f"head size {head_dim}: keys cannot be stored in chunks of {key_chunk} values")
        if store:
            num_pages = k_pages.shape[0]
            _dense(k_pages, "k_pages", qkv.dtype, (num_pages, kv_heads, head_dim // key_chunk, page_size, key_chunk))
            _dense(v_pages, "v_pages", qkv.dtype, (num_pages, kv_heads, v_dim, page_size))
        self._check(self.lib.fllm_rope_kv_store(
            _ptr(qkv), _ptr(row_pos), _ptr(row_seg), _ptr(tables), tables.shape[1], _ptr(cos), _ptr(sin), cos.shape[0],
            _ptr(k_pages), _ptr(v_pages), num_pages, rows, heads, kv_heads, head_dim, v_dim, rope_dims, pairing, page_size,
            key_chunk, _DTYPE_CODE[qkv.dtype], 1 if store else 0, self._stream()))

    def attention_workspace_bytes(self, rows: int, heads: int, kv_heads: int, head_dim: int, max_context: int) -> int:
        return int(self.lib.fllm_attention_workspace_bytes(rows, heads, kv_heads, head_dim, max_context))

    def attention(self, q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, tables: torch.Tensor,
                  row_pos: torch.Tensor, row_seg: torch.Tensor, seg_start: torch.Tensor, out: torch.Tensor, heads: int, kv_heads: int,
                  head_dim: int, page_size: int, scale: float, window: Optional[int], max_context: int,
                  uniform_rows: int = 0, workspace: Optional[torch.Tensor] = None, single_from: Optional[int] = None,
                  head_slopes: Optional[torch.Tensor] = None, v_dim: Optional[int] = None, chunk: Optional[int] = None,
                  key_chunk: int = 8, sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
        """`q` may be a column slice of a wider row-major matrix (the fused qkv buffer).
        `max_context` bounds pos + 1 over the rows; the segments from `single_from` on have one row each
        (`uniform_rows` = 1 is `single_from` = 0: a decode step; by default no segment is known to).
        `head_slopes` (float32 [heads]): every score gets head_slopes[head] * (key position - row position) added, for
        position encodings that bias scores; such a call runs the plain kernel in both precisions.
        `v_dim`: lanes of a value head where they differ from the keys' (`out` is [rows, heads * v_dim]); `chunk`: a row sees
        no key before the start of its own chunk of that many positions (chunks counted from position 0); `key_chunk`: values
        of a key that lie together in a page.  The matrix-core kernels take v_dim == head_dim and key chunks of 8.
        `sinks` (float32 [heads]): the softmax's denominator also holds exp(sinks[head]), a term without key or value."""
        rows = q.shape[0]
        v_dim = head_dim if v_dim is None else int(v_dim)
        chunk = int(chunk) if chunk else 0
        _need(chunk >= 0 and key_chunk > 0 and head_dim % key_chunk == 0, "attention: bad chunk of positions or of key values")
        _need(q.is_cuda and q.dim() == 2 and q.stride(1) == 1 and q.shape[1] == heads * head_dim,
              f"q must be [rows, {heads * head_dim}] with unit column stride")
        _need(q.dtype in _DTYPE_CODE, f"dtype {q.dtype} unsupported")
        num_pages = k_pages.shape[0]
        _dense(k_pages, "k_pages", q.dtype, (num_pages, kv_heads, head_dim // key_chunk, page_size, key_chunk))
        _dense(v_pages, "v_pages", q.dtype, (num_pages, kv_heads, v_dim, page_size))
        _dense(tables, "tables", torch.int32)
        _need(tables.dim() == 2, "tables must be [segments, pages]")
        _dense(row_pos, "row_pos", torch.int32, (rows,))
        _dense(row_seg, "row_seg", torch.int32, (rows,))
        _dense(seg_start, "seg_start", torch.int32)
        _need(seg_start.numel() >= 2, "seg_start must hold at least one segment")
        _need(tables.shape[0] >= seg_start.numel() - 1, "tables must have a row per segment")
        _dense(out, "out", q.dtype, (rows, heads * v_dim))
        ws_ptr, ws_bytes = None, 0
        if workspace is not None:
            _need(workspace.is_cuda and workspace.is_contiguous(), "workspace must be a dense GPU tensor")
            ws_ptr, ws_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
        q_stride = q.stride(0) if rows > 1 else heads * head_dim
        num_segs = seg_start.numel() - 1
        if sinks is not None:
            _dense(sinks, "sinks", torch.float32, (heads,))
        if head_slopes is not None:
            _need(sinks is None, "biased scores come without a sink")
            _need(v_dim == head_dim and not chunk and key_chunk == 8, "biased scores come with one width of keys and values and no chunks")
            _dense(head_slopes, "head_slopes", torch.float32, (heads,))
            self._check(self.lib.fllm_attention_sloped(
                _ptr(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(tables), tables.shape[1], _ptr(row_pos), _ptr(row_seg),
                _ptr(seg_start), num_segs, _ptr(out), rows, heads, kv_heads, head_dim, page_size, num_pages, float(scale),
                int(window) if window else 0, _DTYPE_CODE[q.dtype], int(max_context), _ptr(head_slopes), self._stream()))
            return out
        if single_from is None:
            single_from = 0 if uniform_rows else num_segs
        _need(0 <= single_from <= num_segs and num_segs - single_from <= rows, f"single_from {single_from} does not fit {num_segs} segments of {rows} rows")
        self._check(self.lib.fllm_attention(
            _ptr(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(tables), tables.shape[1], _ptr(row_pos), _ptr(row_seg),
            _ptr(seg_start), seg_start.numel() - 1, _ptr(out), rows, heads, kv_heads, head_dim, v_dim, page_size, num_pages,
            float(scale), int(window) if window else 0, chunk, key_chunk, _ptr(sinks), _DTYPE_CODE[q.dtype], int(max_context), int(single_from),
            ws_ptr, ws_bytes, self._stream()))
        return out

    # ---- parts of other layer designs ----------------------------------------------------------------------
    def rmsnorm_pair(self, x: torch.Tensor, w1: torch.Tensor, eps1: float, out1: torch.Tensor,
                     w2: Optional[torch.Tensor] = None, eps2: Optional[float] = None, out2: Optional[torch.Tensor] = None):
        """Two RMSNorms of the same float32 rows in one pass over them (w2 and out2 None: one)."""
        rows, width = x.shape
        _dense(x, "x", torch.float32)
        _dense(w1, "w1", torch.float32, (width,))
        _dense(out1, "out1", None, (rows, width))
        _need(out1.dtype in _DTYPE_CODE, f"out dtype {out1.dtype} unsupported")
        _need((w2 is None) == (out2 is None), "the second norm needs a weight and an output")
        if w2 is not None:
            _dense(w2, "w2", torch.float32, (width,))
            _dense(out2, "out2", out1.dtype, (rows, width))
        self._check(self.lib.fllm_rmsnorm_pair(_ptr(x), _ptr(w1), _ptr(w2), _ptr(out1), _ptr(out2), rows, width, float(eps1),
                                               float(eps1 if eps2 is None else eps2), _DTYPE_CODE[out1.dtype], self._stream()))
        return out1, out2

    def glu_clamped(self, gate_up: torch.Tensor, out: torch.Tensor, limit: float, alpha: float, up_offset: float) -> torch.Tensor:
        """out = g * sigmoid(alpha * g) * (u + up_offset), g = min(gate, limit), u = clamp(up, -limit, limit) (limit <= 0:
        nothing is clamped); gate_up = [gate | up] side by side in every row."""
        rows, two_i = gate_up.shape
        _need(two_i % 2 == 0, "gate_up needs an even width")
        _dense(gate_up, "gate_up")
        _need(gate_up.dtype in _DTYPE_CODE, f"dtype {gate_up.dtype} unsupported")
        _dense(out, "out", gate_up.dtype, (rows, two_i // 2))
        self._check(self.lib.fllm_glu_clamped(_ptr(gate_up), _ptr(out), rows, two_i // 2, float(limit), float(alpha),
                                              float(up_offset), _DTYPE_CODE[gate_up.dtype], self._stream()))
        return out

    def scale_(self, x: torch.Tensor, scale: float) -> torch.Tensor:
        """x *= scale, float32, in place."""
        _dense(x, "x", torch.float32)
        self._check(self.lib.fllm_scale_f32(_ptr(x), x.numel(), float(scale), self._stream()))
        return x

    def stream_add(self, x: torch.Tensor, ids: Optional[torch.Tensor] = None, table: Optional[torch.Tensor] = None,
                   scale: float = 1.0, vec: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x[r] = (x[r] + scale * table[ids[r]]) + vec: the embedding of the rows' tokens and / or one vector added to the
        float32 residual stream."""
        rows, width = x.shape
        _dense(x, "x", torch.float32)
        vocab, code = 0, F32
        if table is not None:
            _need(ids is not None, "a table needs ids")
            _dense(ids, "ids", torch.int32, (rows,))
            _dense(table, "table")
            _need(table.dtype in _DTYPE_CODE and table.dim() == 2 and table.shape[1] == width, f"table must be [vocab, {width}]")
            vocab, code = table.shape[0], _DTYPE_CODE[table.dtype]
        if vec is not None:
            _dense(vec, "vec", torch.float32, (width,))
        self._check(self.lib.fllm_stream_add(_ptr(x), _ptr(ids) if table is not None else None, _ptr(table), code, vocab,
                                             float(scale), _ptr(vec), rows, width, self._stream()))
        return x

    def postnorm_add(self, x: torch.Tensor, branch: torch.Tensor, gain: torch.Tensor, eps: Optional[float], parts: int = 1,
                     next_weight: Optional[torch.Tensor] = None, next_eps: float = 0.0,
                     next_out: Optional[torch.Tensor] = None, part_weights: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x[r] += v * rsqrt(mean(v^2) + eps) * gain with v = the sum of the row's `parts` partial branches (`branch` is
        [rows * parts, width], a row's parts one after the other); eps None: x[r] += v * gain.  With `next_weight`, the
        RMSNorm of the new rows (`next_eps`) goes to `next_out`.  `part_weights` (float32 [rows, parts]): part k of row r is
        multiplied by part_weights[r, k] as it is summed."""
        rows, width = x.shape
        _dense(x, "x", torch.float32)
        _dense(branch, "branch", None, (rows * parts, width))
        _need(branch.dtype in _DTYPE_CODE, f"branch dtype {branch.dtype} unsupported")
        _dense(gain, "gain", torch.float32, (width,))
        _need((next_weight is None) == (next_out is None), "the norm behind the sum needs a weight and an output")
        code = F32
        if next_weight is not None:
            _dense(next_weight, "next_weight", torch.float32, (width,))
            _dense(next_out, "next_out", None, (rows, width))
            _need(next_out.dtype in _DTYPE_CODE, f"next_out dtype {next_out.dtype} unsupported")
            code = _DTYPE_CODE[next_out.dtype]
        if part_weights is not None:
            _dense(part_weights, "part_weights", torch.float32, (rows, parts))
        self._check(self.lib.fllm_postnorm_add(_ptr(x), _ptr(branch), _DTYPE_CODE[branch.dtype], int(parts), _ptr(part_weights), _ptr(gain),
                                               float(eps or 0.0), 0 if eps is None else 1, _ptr(next_weight), float(next_eps),
                                               _ptr(next_out), code, rows, width, self._stream()))
        return x

    def route_topk(self, h: torch.Tensor, w_router: torch.Tensor, top: int, ids: torch.Tensor, weights: torch.Tensor,
                   score: str = "sigmoid", renormalize: bool = False, route_scale: float = 1.0):
        """score = sigmoid(h @ w_router.T) in float32, or with `score` "softmax" the softmax of those logits over all experts;
        ids[r, k] / weights[r, k]: the expert with the k-th largest score of row r (the lower index among equals) and that
        score, with `renormalize` divided by the sum of the row's picked scores (+ 1e-20), times `route_scale`."""
        _need(score in ("sigmoid", "softmax"), f"router score {score!r} unknown")
        rows, K = h.shape
        E = w_router.shape[0]
        _need(h.is_cuda and h.dim() == 2 and h.stride(1) == 1 and h.dtype in _DTYPE_CODE, "h must be a row-major GPU matrix")
        _dense(w_router, "w_router", h.dtype, (E, K))
        _dense(ids, "ids", torch.int32, (rows, top))
        _dense(weights, "weights", torch.float32, (rows, top))
        self._check(self.lib.fllm_route_topk(_ptr(h), h.stride(0) if rows > 1 else K, _ptr(w_router), rows, K, E, int(top), _ptr(ids),
                                             _ptr(weights), 1 if score == "softmax" else 0, 1 if renormalize else 0, float(route_scale),
                                             _DTYPE_CODE[h.dtype], self._stream()))
        return ids, weights

    def experts_gate_up(self, h: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, w_gate_up: torch.Tensor, act: torch.Tensor,
                        limit: float = 0.0, alpha: float = 1.0, up_offset: float = 0.0) -> torch.Tensor:
        """act[r * top + k] = a(g) * (u + up_offset), g and u the gate and up rows of expert ids[r, k] times (h[r] *
        weights[r, k]); w_gate_up [experts, 2 * inter, width] (gate rows, then up rows); the activation as in `glu_clamped`."""
        rows, K = h.shape
        top = ids.shape[1]
        E, two_i = w_gate_up.shape[0], w_gate_up.shape[1]
        _need(h.is_cuda and h.dim() == 2 and h.stride(1) == 1 and h.dtype in _DTYPE_CODE, "h must be a row-major GPU matrix")
        _dense(w_gate_up, "w_gate_up", h.dtype, (E, two_i, K))
        _need(two_i % 2 == 0, "w_gate_up holds gate rows and as many up rows")
        _dense(ids, "ids", torch.int32, (rows, top))
        _dense(weights, "weights", torch.float32, (rows, top))
        _dense(act, "act", h.dtype, (rows * top, two_i // 2))
        self._check(self.lib.fllm_experts_gate_up(_ptr(h), h.stride(0) if rows > 1 else K, _ptr(ids), _ptr(weights), rows, top,
                                                  _ptr(w_gate_up), E, two_i // 2, K, _ptr(act), float(limit), float(alpha),
                                                  float(up_offset), _DTYPE_CODE[h.dtype], self._stream()))
        return act

    def experts_down(self, act: torch.Tensor, ids: torch.Tensor, w_down: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """out[p] = w_down[ids[p]] @ act[p] for every (row, pick) pair p, float32; w_down [experts, width, inter]."""
        pairs, inter = act.shape
        E, N = w_down.shape[0], w_down.shape[1]
        _dense(act, "act")
        _need(act.dtype in _DTYPE_CODE, f"dtype {act.dtype} unsupported")
        _dense(w_down, "w_down", act.dtype, (E, N, inter))
        _need(ids.is_cuda and ids.is_contiguous() and ids.dtype == torch.int32 and ids.numel() == pairs, "ids must name an expert a pair")
        _dense(out, "out", torch.float32, (pairs, N))
        self._check(self.lib.fllm_experts_down(_ptr(act), _ptr(ids), pairs, _ptr(w_down), E, N, inter, _ptr(out),
                                               _DTYPE_CODE[act.dtype], self._stream()))
        return out

    GROUPED_EXPERTS_ROWS = 17      # steps of this many rows and more group their (row, pick) pairs by expert,
    GROUPED_EXPERTS_SHARE = 2      # and smaller ones that have this many pairs an expert: the plain kernels read an expert's
                                   # matrices once a pair, the grouped ones once a step

    def experts_grouped(self, h: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor,
                        out: torch.Tensor, limit: float = 0.0, alpha: float = 1.0, up_offset: float = 0.0) -> bool:
        """`experts_gate_up` and `experts_down` in one call on the matrix cores (bfloat16, prompt portions): the pairs are
        grouped by expert on the device, and an expert multiplies the rows that picked it as tiles.  out float32
        [rows * top, width].  False: not taken (few rows, float32, sizes that are no multiples of 8), nothing was written."""
        rows, K = h.shape
        top = ids.shape[1]
        E, two_i = w_gate_up.shape[0], w_gate_up.shape[1]
        if h.dtype != torch.bfloat16 or not h.is_cuda:
            return False
        if rows < self.GROUPED_EXPERTS_ROWS and rows * top < self.GROUPED_EXPERTS_SHARE * E:
            return False
        N = w_down.shape[1]
        _need(h.dim() == 2 and h.stride(1) == 1, "h must be a row-major matrix")
        _dense(w_gate_up, "w_gate_up", h.dtype, (E, two_i, K))
        _dense(w_down, "w_down", h.dtype, (E, N, two_i // 2))
        _dense(ids, "ids", torch.int32, (rows, top))
        _dense(weights, "weights", torch.float32, (rows, top))
        _dense(out, "out", torch.float32, (rows * top, N))
        act = torch.empty((rows * top, two_i // 2), dtype=h.dtype, device=h.device)
        xs = torch.empty((rows * top, K), dtype=h.dtype, device=h.device)      # the rows times their picks' weights
        work = torch.empty((int(self.lib.fllm_experts_grouped_work_ints(rows * top, E)),), dtype=torch.int32, device=h.device)
        need = int(self.lib.fllm_experts_grouped_plane_floats(rows * top, E, N, two_i // 2))     # a down product cut along K
        planes = torch.empty((need,), dtype=torch.float32, device=h.device) if need else None
        code = self.lib.fllm_experts_grouped(_ptr(h), h.stride(0), _ptr(ids), _ptr(weights), rows, top, _ptr(w_gate_up), _ptr(w_down), E,
                                             two_i // 2, K, N, _ptr(act), _ptr(xs), _ptr(out), _ptr(work), _ptr(planes), float(limit), float(alpha),
                                             float(up_offset), self._stream())
        if code == 1:
            return False
        self._check(code)
        return True

    # ---- what a sequence carries outside the pages, and the small kernels around it ---------------------------------------
    def short_conv(self, x: torch.Tensor, w: torch.Tensor, state: Optional[torch.Tensor], row_seg: torch.Tensor,
                   seg_start: torch.Tensor, slots: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """out[t] = x[t] + sum_j w[:, j] x[t - taps + 1 + j] over the rows of each segment, the inputs before the step's first
        row from `state` [slots, taps - 1, width] (of x's type), which then takes the sequence's last taps - 1 inputs."""
        rows, width = x.shape
        taps = w.shape[1]
        _dense(x, "x")
        _need(x.dtype in _DTYPE_CODE, f"dtype {x.dtype} unsupported")
        _dense(w, "w", torch.float32, (width, taps))
        _dense(out, "out", x.dtype, (rows, width))
        _need(out.data_ptr() != x.data_ptr(), "short_conv: rows read their neighbours, out cannot be x")
        _dense(row_seg, "row_seg", torch.int32, (rows,))
        _dense(seg_start, "seg_start", torch.int32)
        _dense(slots, "slots", torch.int32)
        num_segs = seg_start.numel() - 1
        _need(num_segs >= 1 and slots.numel() >= num_segs, "short_conv: a slot a segment")
        if taps > 1:
            _need(state is not None, "short_conv: the taps before a step need a state")
            _dense(state, "state", x.dtype, (state.shape[0], taps - 1, width))
        self._check(self.lib.fllm_short_conv(_ptr(x), _ptr(w), _ptr(state), _ptr(row_seg), _ptr(seg_start), _ptr(slots), num_segs,
                                             _ptr(out), rows, width, taps, _DTYPE_CODE[x.dtype], self._stream()))
        return out

    def norm_short_conv(self, x: torch.Tensor, norm_weight: torch.Tensor, eps: float, w: torch.Tensor, state: Optional[torch.Tensor],
                        row_seg: torch.Tensor, slots: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """`short_conv` of the RMSNorm of the float32 rows x in one kernel, for steps of ONE row a segment (segment s is row s)."""
        rows, width = x.shape
        taps = w.shape[1]
        _dense(x, "x", torch.float32)
        _dense(norm_weight, "norm_weight", torch.float32, (width,))
        _dense(w, "w", torch.float32, (width, taps))
        _dense(out, "out", None, (rows, width))
        _need(out.dtype in _DTYPE_CODE, f"dtype {out.dtype} unsupported")
        _dense(row_seg, "row_seg", torch.int32, (rows,))
        _dense(slots, "slots", torch.int32)
        _need(slots.numel() >= rows, "norm_short_conv: a slot a row")
        if taps > 1:
            _need(state is not None, "norm_short_conv: the taps before a step need a state")
            _dense(state, "state", out.dtype, (state.shape[0], taps - 1, width))
        self._check(self.lib.fllm_norm_short_conv(_ptr(x), _ptr(norm_weight), float(eps), _ptr(w), _ptr(state), _ptr(row_seg), _ptr(slots),
                                                  _ptr(out), rows, width, taps, _DTYPE_CODE[out.dtype], self._stream()))
        return out

    LINEAR_ATTENTION_PARTS_ROWS = 512      # steps of this many rows and more cut their segments into parts

    def linear_attention(self, qkv: torch.Tensor, decay_hi: torch.Tensor, decay_lo: torch.Tensor, state: torch.Tensor,
                         row_seg: torch.Tensor, seg_start: torch.Tensor, slots: torch.Tensor, out: torch.Tensor, heads: int,
                         dim: int, vdim: int, activation: str = "silu", form: str = "auto", parts: bool = True) -> torch.Tensor:
        """Per head S <- decay S + k v^T, o = S^T q over each segment's rows; rows of `qkv` hold [q | k | v | ..] (heads * dim,
        heads * dim, heads * vdim); S float32 state[slots, heads, dim, vdim]; out float32 [rows, heads * vdim].  `form`:
        "tokens" runs token after token, "chunks" 32 tokens at a time on the matrix cores in float32 (dim a multiple of 16 up
        to 128, vdim a multiple of 16), "auto" chunks where a step holds portions of prompts and the sizes allow.  With `parts`
        the chunked form cuts the segments of a step of 512 rows or more into parts of 256 tokens that run side by side, each
        from zeros, and a second kernel hands the states from part to part and adds what the tokens of a part lack."""
        rows = qkv.shape[0]
        _need(qkv.is_cuda and qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.dtype in _DTYPE_CODE, "qkv must be a row-major GPU matrix")
        ld = qkv.stride(0) if rows > 1 else qkv.shape[1]
        _need(qkv.shape[1] >= heads * (2 * dim + vdim), "qkv rows are too short")
        _need(activation in ("silu", "none"), f"activation {activation!r} unknown")
        _need(form in ("auto", "tokens", "chunks"), f"form {form!r} unknown")
        _dense(decay_hi, "decay_hi", torch.float32, (heads,))
        _dense(decay_lo, "decay_lo", torch.float32, (heads,))
        _dense(state, "state", torch.float32, (state.shape[0], heads, dim, vdim))
        _dense(out, "out", torch.float32, (rows, heads * vdim))
        _dense(row_seg, "row_seg", torch.int32, (rows,))
        _dense(seg_start, "seg_start", torch.int32)
        _dense(slots, "slots", torch.int32)
        num_segs = seg_start.numel() - 1
        _need(num_segs >= 1 and slots.numel() >= num_segs, "linear_attention: a slot a segment")
        elem = qkv.element_size()
        base = qkv.data_ptr()
        carried = None
        if parts and form != "tokens" and rows >= self.LINEAR_ATTENTION_PARTS_ROWS and rows > num_segs:
            need = int(self.lib.fllm_linear_attention_carried_floats(rows, num_segs, heads, dim, vdim))
            carried = torch.empty((need,), dtype=torch.float32, device=qkv.device)
        self._check(self.lib.fllm_linear_attention(base, base + heads * dim * elem, base + 2 * heads * dim * elem, ld, _ptr(decay_hi),
                                                   _ptr(decay_lo), _ptr(state), _ptr(row_seg), _ptr(seg_start), _ptr(slots), num_segs,
                                                   _ptr(out), rows, heads, dim, vdim, 1 if activation == "silu" else 0,
                                                   {"auto": 0, "tokens": 1, "chunks": 2}[form], _DTYPE_CODE[qkv.dtype], _ptr(carried),
                                                   self._stream()))
        return out

    def gated_norm(self, x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, gate: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """out = x * rsqrt(mean x^2 + eps) * weight * sigmoid(gate) (weight None: out = x * sigmoid(gate)); `gate` may be a
        column slice of a wider matrix."""
        rows, width = x.shape
        _dense(x, "x")
        _need(x.dtype in _DTYPE_CODE, f"dtype {x.dtype} unsupported")
        _need(gate.is_cuda and gate.dim() == 2 and gate.stride(1) == 1 and tuple(gate.shape) == (rows, width) and gate.dtype == out.dtype,
              "gate must be [rows, width] of out's type with unit column stride")
        _dense(out, "out", None, (rows, width))
        _need(out.dtype in _DTYPE_CODE and (x.dtype == torch.float32 or x.dtype == out.dtype), "gated_norm: x is float32 or of out's type")
        if weight is not None:
            _dense(weight, "weight", torch.float32, (width,))
        self._check(self.lib.fllm_gated_norm(_ptr(x), _DTYPE_CODE[x.dtype], _ptr(weight), float(eps), _ptr(gate),
                                             gate.stride(0) if rows > 1 else width, _ptr(out), rows, width, _DTYPE_CODE[out.dtype],
                                             self._stream()))
        return out

    def polynorm(self, z: torch.Tensor, coeffs: torch.Tensor, eps: float, out: torch.Tensor) -> torch.Tensor:
        """out = c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3, N the division of a row by its root mean square; coeffs float32 [4]."""
        rows, width = z.shape
        _need(z.is_cuda and z.stride(1) == 1 and z.dtype in _DTYPE_CODE, "z must be a row-major GPU matrix")
        _dense(coeffs, "coeffs", torch.float32, (4,))
        _dense(out, "out", z.dtype, (rows, width))
        self._check(self.lib.fllm_polynorm(_ptr(z), z.stride(0) if rows > 1 else width, _ptr(coeffs), float(eps), _ptr(out), rows, width,
                                           _DTYPE_CODE[z.dtype], self._stream()))
        return out

    def head_norm_kv_store(self, qkv: torch.Tensor, eps: float, norm_dim: int, row_pos: torch.Tensor, row_seg: torch.Tensor,
                           tables: torch.Tensor, k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], heads: int,
                           kv_heads: int, head_dim: int, page_size: int, v_dim: Optional[int] = None, key_chunk: int = 8) -> None:
        """Every head of q and k in the rows [q | k | v | ..] is divided by its root mean square over `norm_dim` lanes (q in
        place); k and v go into the pages of the row's request (pages None: q alone is normed)."""
        rows = qkv.shape[0]
        v_dim = head_dim if v_dim is None else int(v_dim)
        _dense(qkv, "qkv")
        _need(qkv.dtype in _DTYPE_CODE and qkv.shape[1] >= (heads + kv_heads) * head_dim + kv_heads * v_dim, "qkv rows are too short")
        _dense(row_pos, "row_pos", torch.int32, (rows,))
        _dense(row_seg, "row_seg", torch.int32, (rows,))
        _dense(tables, "tables", torch.int32)
        _need(tables.dim() == 2, "tables must be [segments, pages]")
        store = k_pages is not None
        if store:
            num_pages = k_pages.shape[0]
            _dense(k_pages, "k_pages", qkv.dtype, (num_pages, kv_heads, head_dim // key_chunk, page_size, key_chunk))
            _dense(v_pages, "v_pages", qkv.dtype, (num_pages, kv_heads, v_dim, page_size))
        self._check(self.lib.fllm_head_norm_kv_store(_ptr(qkv), qkv.shape[1], float(eps), int(norm_dim), _ptr(row_pos), _ptr(row_seg),
                                                     _ptr(tables), tables.shape[1], _ptr(k_pages), _ptr(v_pages), rows, heads, kv_heads,
                                                     head_dim, v_dim, page_size, key_chunk, _DTYPE_CODE[qkv.dtype], 1 if store else 0,
                                                     self._stream()))

    def _talking_pages(self, k_pages, v_pages, dtype, kv_heads, k_dim, v_dim, page_size, key_chunk):
        _need(key_chunk > 0 and k_dim % key_chunk == 0, f"keys of {k_dim} values cannot lie in chunks of {key_chunk}")
        num_pages = k_pages.shape[0]
        _dense(k_pages, "k_pages", dtype, (num_pages, kv_heads, k_dim // key_chunk, page_size, key_chunk))
        _dense(v_pages, "v_pages", dtype, (num_pages, kv_heads, v_dim, page_size))

    def qk_norm_rope_store(self, qkv: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor, eps: float, q_out: torch.Tensor,
                           row_pos: torch.Tensor, row_seg: torch.Tensor, tables: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                           k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], heads: int, kv_heads: int, k_dim: int,
                           v_dim: int, rope_dims: int, page_size: int, key_chunk: int) -> torch.Tensor:
        """Rows of a joint product [q | k | v | ...]: RMSNorm over the whole query projection and over the whole key
        projection, rotary on the first `rope_dims` lanes of every head (lane i with lane i + rope_dims / 2), queries to
        `q_out`, keys and values into the pages (None: nothing is stored)."""
        rows = qkv.shape[0]
        _need(qkv.is_cuda and qkv.dim() == 2 and qkv.is_contiguous() and qkv.dtype in _DTYPE_CODE, "qkv must be dense rows on the GPU")
        _need(qkv.shape[1] >= heads * k_dim + kv_heads * (k_dim + v_dim), "qkv rows are too short for q, k and v")
        _dense(q_weight, "q_weight", torch.float32, (heads * k_dim,))
        _dense(k_weight, "k_weight", torch.float32, (kv_heads * k_dim,))
        _dense(q_out, "q_out", qkv.dtype, (rows, heads * k_dim))
        _dense(row_pos, "row_pos", torch.int32, (rows,))
        _dense(row_seg, "row_seg", torch.int32, (rows,))
        _dense(tables, "tables", torch.int32)
        _need(tables.dim() == 2, "tables must be [segments, pages]")
        _dense(cos, "cos", torch.float32)
        _dense(sin, "sin", torch.float32, tuple(cos.shape))
        _need(cos.dim() == 2 and cos.shape[1] == rope_dims // 2, f"rotary tables must be [positions, {rope_dims // 2}]")
        store = k_pages is not None
        if store:
            self._talking_pages(k_pages, v_pages, qkv.dtype, kv_heads, k_dim, v_dim, page_size, key_chunk)
        self._check(self.lib.fllm_qk_norm_rope_store(
            _ptr(qkv), qkv.shape[1], _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(q_out), _ptr(row_pos), _ptr(row_seg),
            _ptr(tables), tables.shape[1], _ptr(cos), _ptr(sin), cos.shape[0], _ptr(k_pages), _ptr(v_pages), rows, heads, kv_heads,
            k_dim, v_dim, rope_dims, page_size, key_chunk, _DTYPE_CODE[qkv.dtype], 1 if store else 0, self._stream()))
        return q_out

    TALKING_TILE_ROWS = 16          # rows of one request that a workgroup of the matrix-core kernel takes
    TALKING_KEY_BLOCK = 64          # keys it walks at a time
    TALKING_WORKGROUPS = 512        # what a launch should come to: two a compute unit

    def talking_attention_splits(self, rows: int, num_segs: int, chunk: Optional[int], max_context: int) -> int:
        """How many workgroups should share the keys of a row tile of `talking_attention` (1: none): enough to fill the
        device when the step has few tiles (a decode step has one a request), at most one a block of keys."""
        tiles = rows // self.TALKING_TILE_ROWS + num_segs
        span = max_context if not chunk else min(max_context, chunk + self.TALKING_TILE_ROWS)
        blocks = -(-(span + self.TALKING_TILE_ROWS) // self.TALKING_KEY_BLOCK)
        return max(1, min(self.TALKING_WORKGROUPS // max(tiles, 1), blocks, 64))

    def talking_attention_workspace(self, rows: int, num_segs: int, heads: int, v_dim: int, splits: int) -> int:
        """float32 elements of workspace that `splits` workgroups a tile need."""
        if splits <= 1:
            return 0
        return (rows // self.TALKING_TILE_ROWS + num_segs) * splits * self.TALKING_TILE_ROWS * heads * (2 + v_dim)

    def talking_attention(self, q: torch.Tensor, gate: Optional[torch.Tensor], k_pages: torch.Tensor, v_pages: torch.Tensor,
                          tables: torch.Tensor, row_pos: torch.Tensor, row_seg: torch.Tensor, seg_start: torch.Tensor,
                          talk: torch.Tensor, temp: torch.Tensor, out: torch.Tensor, heads: int, kv_heads: int, k_dim: int,
                          v_dim: int, page_size: int, scale: float, chunk: Optional[int], key_chunk: int, max_context: int,
                          splits: int = 1, workspace: Optional[torch.Tensor] = None, single_rows: bool = False) -> torch.Tensor:
        """Attention whose scores are mixed across heads before the softmax (score[h] = sum_g talk[h, g] * q_g . k * scale *
        temp[g]) over the keys of the row's own chunk of `chunk` positions up to the row (None: all keys up to the row);
        head h's output times sigmoid(gate[row, h]) (`gate` may be a column slice of a wider matrix; None: no gate)."""
        rows = q.shape[0]
        _dense(q, "q", None, (rows, heads * k_dim))
        _need(q.dtype in _DTYPE_CODE, f"dtype {q.dtype} unsupported")
        gate_stride = 0
        if gate is not None:
            _need(gate.is_cuda and gate.dtype == q.dtype and tuple(gate.shape) == (rows, heads) and gate.stride(1) == 1,
                  f"gate must be [rows, {heads}] of {q.dtype} with unit column stride")
            gate_stride = gate.stride(0) if rows > 1 else heads
        self._talking_pages(k_pages, v_pages, q.dtype, kv_heads, k_dim, v_dim, page_size, key_chunk)
        _dense(tables, "tables", torch.int32)
        _need(tables.dim() == 2, "tables must be [segments, pages]")
        _dense(row_pos, "row_pos", torch.int32, (rows,))
        _dense(row_seg, "row_seg", torch.int32, (rows,))
        _dense(seg_start, "seg_start", torch.int32)
        _need(seg_start.numel() >= 2 and tables.shape[0] >= seg_start.numel() - 1, "tables must have a row per segment")
        _dense(talk, "talk", torch.float32, (heads, heads))
        _dense(temp, "temp", torch.float32, (heads,))
        _dense(out, "out", q.dtype, (rows, heads * v_dim))
        ws_floats = 0
        if splits > 1:
            _need(workspace is not None, "workgroups that share a tile need a workspace")
            _dense(workspace, "workspace", torch.float32)
            ws_floats = workspace.numel()
        self._check(self.lib.fllm_talking_attention(
            _ptr(q), _ptr(gate), gate_stride, _ptr(k_pages), _ptr(v_pages), _ptr(tables), tables.shape[1], _ptr(row_pos),
            _ptr(row_seg), _ptr(seg_start), seg_start.numel() - 1, _ptr(talk), _ptr(temp), _ptr(out), rows, heads, kv_heads, k_dim,
            v_dim, page_size, float(scale), int(chunk) if chunk else 0, key_chunk, _DTYPE_CODE[q.dtype], int(max_context),
            int(splits), _ptr(workspace), ws_floats, 1 if single_rows and rows == seg_start.numel() - 1 else 0, self._stream()))
        return out

    # ---- mixers beside the softmax attention over all keys ----------------------------------------------------------------
    def _paged(self, q, k_pages, v_pages, tables, row_pos, row_seg, out, heads, kv_heads, k_dim, v_dim, page_size, key_chunk):
        rows = q.shape[0]
        _need(q.is_cuda and q.dim() == 2 and q.stride(1) == 1 and q.shape[1] == heads * k_dim and q.dtype in _DTYPE_CODE,
              f"q must be [rows, {heads * k_dim}] of float32 or bfloat16 with unit column stride")
        _need(heads % kv_heads == 0, f"{heads} heads are not a multiple of {kv_heads} key/value heads")
        self._talking_pages(k_pages, v_pages, q.dtype, kv_heads, k_dim, v_dim, page_size, key_chunk)
        _dense(tables, "tables", torch.int32)
        _need(tables.dim() == 2, "tables must be [segments, pages]")
        _dense(row_pos, "row_pos", torch.int32, (rows,))
        _dense(row_seg, "row_seg", torch.int32, (rows,))
        _dense(out, "out", q.dtype, (rows, heads * v_dim))
        return rows, (q.stride(0) if rows > 1 else heads * k_dim)

    @staticmethod
    def _segments(seg_start, tables, rows):
        _dense(seg_start, "seg_start", torch.int32)
        _need(seg_start.numel() >= 2 and tables.shape[0] >= seg_start.numel() - 1, "seg_start must hold a segment's first row and the end; tables a row a segment")

    def normed_rope_store(self, qkv: torch.Tensor, norm_mode: int, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                          eps: float, q_out: torch.Tensor, row_pos: torch.Tensor, row_seg: torch.Tensor, tables: torch.Tensor,
                          cos: torch.Tensor, sin: torch.Tensor, k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor],
                          heads: int, kv_heads: int, k_dim: int, v_dim: int, rope_dims: int, page_size: int, key_chunk: int,
                          values_from_keys: bool = False) -> torch.Tensor:
        """Rows of a joint product [q | k | v | ...]: `norm_mode` 0 none, 1 an RMS norm of every head of q and of k with one weight
        vector [k_dim] for all heads, 2 an RMS norm over the whole query projection and the whole key projection; rotary on the
        first `rope_dims` lanes of every head (lane i with lane i + rope_dims / 2); queries to `q_out`, keys and values into the
        pages (None: nothing is stored).  `values_from_keys`: the values are the keys as projected; the rows hold no values."""
        rows = qkv.shape[0]
        _need(qkv.is_cuda and qkv.dim() == 2 and qkv.is_contiguous() and qkv.dtype in _DTYPE_CODE, "qkv must be dense rows on the GPU")
        _need(norm_mode in (0, 1, 2), f"norm mode {norm_mode} unknown")
        _need(not values_from_keys or v_dim == k_dim, "keys that double as values have one width")
        _need(qkv.shape[1] >= heads * k_dim + kv_heads * k_dim + (0 if values_from_keys else kv_heads * v_dim), "qkv rows are too short")
        if norm_mode:
            _dense(q_weight, "q_weight", torch.float32, (heads * k_dim if norm_mode == 2 else k_dim,))
            _dense(k_weight, "k_weight", torch.float32, (kv_heads * k_dim if norm_mode == 2 else k_dim,))
        _dense(q_out, "q_out", qkv.dtype, (rows, heads * k_dim))
        _dense(row_pos, "row_pos", torch.int32, (rows,))
        _dense(row_seg, "row_seg", torch.int32, (rows,))
        _dense(tables, "tables", torch.int32)
        _need(tables.dim() == 2, "tables must be [segments, pages]")
        _dense(cos, "cos", torch.float32)
        _dense(sin, "sin", torch.float32, tuple(cos.shape))
        _need(cos.dim() == 2 and cos.shape[1] == rope_dims // 2, f"rotary tables must be [positions, {rope_dims // 2}]")
        store = k_pages is not None
        if store:
            self._talking_pages(k_pages, v_pages, qkv.dtype, kv_heads, k_dim, v_dim, page_size, key_chunk)
        self._check(self.lib.fllm_normed_rope_store(
            _ptr(qkv), qkv.shape[1], int(norm_mode), _ptr(q_weight) if norm_mode else None, _ptr(k_weight) if norm_mode else None,
            float(eps), _ptr(q_out), _ptr(row_pos), _ptr(row_seg), _ptr(tables), tables.shape[1], _ptr(cos), _ptr(sin), cos.shape[0],
            _ptr(k_pages), _ptr(v_pages), rows, heads, kv_heads, k_dim, v_dim, rope_dims, page_size, key_chunk, _DTYPE_CODE[qkv.dtype],
            1 if store else 0, 1 if values_from_keys else 0, self._stream()))
        return q_out

    def _pools(self, pool_k, pool_v, num_pages, kv_heads, k_dim, v_dim, page_size, pool):
        slots = -(-page_size // pool)
        _dense(pool_k, "pool_k", torch.float32, (num_pages, kv_heads, slots, k_dim))
        _dense(pool_v, "pool_v", torch.float32, (num_pages, kv_heads, slots, v_dim))

    def pool_blocks(self, k_pages: torch.Tensor, v_pages: torch.Tensor, pool_k: torch.Tensor, pool_v: torch.Tensor, tables: torch.Tensor,
                    row_pos: torch.Tensor, row_seg: torch.Tensor, kv_heads: int, k_dim: int, v_dim: int, page_size: int,
                    key_chunk: int, pool: int) -> None:
        """For every row whose position ends a block of `pool` positions: the float32 means of the block's keys and values as the
        pages hold them, into pool_k / pool_v [pages, kv_heads, ceil(page_size / pool), k_dim or v_dim] at the page of the block's
        last token, slot (the token's place in the page) // pool.  Runs behind the store of the step's keys."""
        rows = row_pos.numel()
        _need(pool > 0, "a block holds at least one position")
        self._talking_pages(k_pages, v_pages, k_pages.dtype, kv_heads, k_dim, v_dim, page_size, key_chunk)
        _need(k_pages.dtype in _DTYPE_CODE, f"dtype {k_pages.dtype} unsupported")
        self._pools(pool_k, pool_v, k_pages.shape[0], kv_heads, k_dim, v_dim, page_size, pool)
        _dense(tables, "tables", torch.int32)
        _need(tables.dim() == 2, "tables must be [segments, pages]")
        _dense(row_pos, "row_pos", torch.int32, (rows,))
        _dense(row_seg, "row_seg", torch.int32, (rows,))
        self._check(self.lib.fllm_pool_blocks(_ptr(k_pages), _ptr(v_pages), _ptr(pool_k), _ptr(pool_v), _ptr(tables), tables.shape[1],
                                              _ptr(row_pos), _ptr(row_seg), rows, kv_heads, k_dim, v_dim, page_size, key_chunk, int(pool),
                                              _DTYPE_CODE[k_pages.dtype], self._stream()))

    def pooled_window_attention(self, q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, pool_k: torch.Tensor,
                                pool_v: torch.Tensor, tables: torch.Tensor, row_pos: torch.Tensor, row_seg: torch.Tensor,
                                seg_start: torch.Tensor, out: torch.Tensor, heads: int, kv_heads: int, k_dim: int, v_dim: int,
                                page_size: int, scale: float, window: int, pool: int, key_chunk: int, max_context: int = 0) -> torch.Tensor:
        """A row at position p attends to the tokens max(0, p - window + 1) .. p and to one mean key and value (`pool_blocks`) for
        every block b of `pool` positions with b * pool + pool - 1 <= p - window, in one softmax."""
        rows, q_stride = self._paged(q, k_pages, v_pages, tables, row_pos, row_seg, out, heads, kv_heads, k_dim, v_dim, page_size, key_chunk)
        self._segments(seg_start, tables, rows)
        _need(window > 0 and pool > 0, "window and pool must be positive")
        self._pools(pool_k, pool_v, k_pages.shape[0], kv_heads, k_dim, v_dim, page_size, pool)
        self._check(self.lib.fllm_pooled_window_attention(
            _ptr(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(pool_k), _ptr(pool_v), _ptr(tables), tables.shape[1], _ptr(row_pos),
            _ptr(row_seg), _ptr(seg_start), seg_start.numel() - 1, _ptr(out), rows, heads, kv_heads, k_dim, v_dim, page_size,
            float(scale), int(window), int(pool), key_chunk,
            _DTYPE_CODE[q.dtype], int(max_context), self._stream()))
        return out

    def sigmoid_attention(self, q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, tables: torch.Tensor, row_pos: torch.Tensor,
                          row_seg: torch.Tensor, seg_start: torch.Tensor, out: torch.Tensor, heads: int, kv_heads: int, k_dim: int,
                          v_dim: int, page_size: int, scale: float, softcap: float, r1: torch.Tensor, r2: torch.Tensor, pb: torch.Tensor,
                          temp_coef: float, temp_every: int, key_chunk: int, max_context: int = 0) -> torch.Tensor:
        """out[h] = sum over the keys j <= p of sigmoid(softcap * tanh(s / softcap) - r1[h] * ln(1 + r2[h] * (p - j)) + pb[h]) * v_j,
        s = q . k_j * scale * (1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)); `q` may be a column slice of a wider matrix."""
        rows, q_stride = self._paged(q, k_pages, v_pages, tables, row_pos, row_seg, out, heads, kv_heads, k_dim, v_dim, page_size, key_chunk)
        self._segments(seg_start, tables, rows)
        for name, t in (("r1", r1), ("r2", r2), ("pb", pb)):
            _dense(t, name, torch.float32, (heads,))
        _need(softcap > 0 and temp_every > 0, "softcap and temp_every must be positive")
        self._check(self.lib.fllm_sigmoid_attention(
            _ptr(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(tables), tables.shape[1], _ptr(row_pos), _ptr(row_seg), _ptr(seg_start),
            seg_start.numel() - 1, _ptr(out), rows, heads, kv_heads, k_dim, v_dim, page_size, float(scale), float(softcap), _ptr(r1), _ptr(r2), _ptr(pb), float(temp_coef),
            int(temp_every), key_chunk, _DTYPE_CODE[q.dtype], int(max_context), self._stream()))
        return out

    def rotate_scale(self, qkv: torch.Tensor, out: torch.Tensor, row_pos: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, heads: int,
                     dim: int, vdim: int, rope_dims: int, key_scale: float) -> torch.Tensor:
        """Rows [q | k | v | ..] (heads * dim, heads * dim, heads * vdim) -> float32 rows [q | k | v]: q and k rotated on the first
        `rope_dims` lanes of every head at the row's position (lane i with lane i + rope_dims / 2), k times `key_scale`."""
        rows = qkv.shape[0]
        _need(qkv.is_cuda and qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.dtype in _DTYPE_CODE, "qkv must be a row-major GPU matrix")
        _need(qkv.shape[1] >= heads * (2 * dim + vdim), "qkv rows are too short")
        _dense(out, "out", torch.float32, (rows, heads * (2 * dim + vdim)))
        _dense(row_pos, "row_pos", torch.int32, (rows,))
        _dense(cos, "cos", torch.float32)
        _dense(sin, "sin", torch.float32, tuple(cos.shape))
        _need(cos.dim() == 2 and cos.shape[1] == rope_dims // 2, f"rotary tables must be [positions, {rope_dims // 2}]")
        self._check(self.lib.fllm_rotate_scale(_ptr(qkv), qkv.stride(0) if rows > 1 else qkv.shape[1], _ptr(out), _ptr(row_pos), _ptr(cos),
                                               _ptr(sin), cos.shape[0], rows, heads, dim, vdim, rope_dims, float(key_scale),
                                               _DTYPE_CODE[qkv.dtype], self._stream()))
        return out

    def group_norm_gate(self, x: torch.Tensor, eps: float, group: int, gate: torch.Tensor, out: torch.Tensor,
                        activation: str = "silu") -> torch.Tensor:
        """out = x / sqrt(mean over each group of `group` lanes of x^2 + eps) * act(gate), act "silu" or "sigmoid"; `gate` may be a
        column slice of a wider matrix."""
        rows, width = x.shape
        _dense(x, "x")
        _need(activation in ("silu", "sigmoid"), f"activation {activation!r} unknown")
        _need(x.dtype in _DTYPE_CODE and group > 0 and width % group == 0, f"groups of {group} lanes in rows of {width}")
        _need(gate.is_cuda and gate.dim() == 2 and gate.stride(1) == 1 and tuple(gate.shape) == (rows, width) and gate.dtype == out.dtype,
              "gate must be [rows, width] of out's type with unit column stride")
        _dense(out, "out", None, (rows, width))
        _need(out.dtype in _DTYPE_CODE and (x.dtype == torch.float32 or x.dtype == out.dtype), "group_norm_gate: x is float32 or of out's type")
        self._check(self.lib.fllm_group_norm_gate(_ptr(x), _DTYPE_CODE[x.dtype], float(eps), int(group), _ptr(gate),
                                                  gate.stride(0) if rows > 1 else width, _ptr(out), rows, width,
                                                  1 if activation == "silu" else 0, _DTYPE_CODE[out.dtype], self._stream()))
        return out

    def weighted_sum(self, out: torch.Tensor, x: torch.Tensor, a: float, y: torch.Tensor, b: float, accumulate: bool = False) -> torch.Tensor:
        """out = a * x + b * y, or with `accumulate` out += a * x + b * y; float32."""
        _dense(out, "out", torch.float32)
        _dense(x, "x", torch.float32, tuple(out.shape))
        _dense(y, "y", torch.float32, tuple(out.shape))
        self._check(self.lib.fllm_weighted_sum(_ptr(out), _ptr(x), float(a), _ptr(y), float(b), out.numel(), 1 if accumulate else 0,
                                               self._stream()))
        return out

    def stream_concat(self, x: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, scale: float, out: torch.Tensor) -> torch.Tensor:
        """out[r] = [x[r] | scale * table[ids[r]]] in the table's type: the float32 stream beside the rows' embeddings."""
        rows, width = x.shape
        _dense(x, "x", torch.float32)
        _dense(ids, "ids", torch.int32, (rows,))
        _dense(table, "table")
        _need(table.dtype in _DTYPE_CODE and table.dim() == 2 and table.shape[1] == width, f"table must be [vocab, {width}]")
        _dense(out, "out", table.dtype, (rows, 2 * width))
        self._check(self.lib.fllm_stream_concat(_ptr(x), _ptr(ids), _ptr(table), table.shape[0], float(scale), _ptr(out), rows, width,
                                                _DTYPE_CODE[table.dtype], self._stream()))
        return out

    def activation(self, x: torch.Tensor, out: torch.Tensor, kind: str = "relu2") -> torch.Tensor:
        """out = relu(x)^2 element by element (`out` may be `x`)."""
        _need(kind == "relu2", f"activation {kind!r} unknown")
        _dense(x, "x")
        _need(x.dtype in _DTYPE_CODE, f"dtype {x.dtype} unsupported")
        _dense(out, "out", x.dtype, tuple(x.shape))
        self._check(self.lib.fllm_relu_squared(_ptr(x), _ptr(out), x.numel(), _DTYPE_CODE[x.dtype], self._stream()))
        return out

    def route_grouped(self, h: torch.Tensor, w_router: torch.Tensor, correction: torch.Tensor, top: int, groups: int, groups_kept: int,
                      ids: torch.Tensor, weights: torch.Tensor, route_scale: float = 1.0):
        """score = sigmoid(h @ w_router.T) in float32; the picks are the `top` largest of score + correction among the experts of
        the `groups_kept` groups (of `groups` equal groups of neighbours) whose two largest corrected scores sum highest (the lower
        index among equals, for groups and experts); weights = the picks' plain scores / (their sum + 1e-20) * route_scale."""
        rows, K = h.shape
        E = w_router.shape[0]
        _need(h.is_cuda and h.dim() == 2 and h.stride(1) == 1 and h.dtype in _DTYPE_CODE, "h must be a row-major GPU matrix")
        _dense(w_router, "w_router", h.dtype, (E, K))
        _dense(correction, "correction", torch.float32, (E,))
        _need(groups > 0 and E % groups == 0 and 0 < groups_kept <= groups and 0 < top <= groups_kept * (E // groups),
              f"{E} experts in {groups} groups, {groups_kept} kept, {top} picked")
        _dense(ids, "ids", torch.int32, (rows, top))
        _dense(weights, "weights", torch.float32, (rows, top))
        self._check(self.lib.fllm_route_grouped(_ptr(h), h.stride(0) if rows > 1 else K, _ptr(w_router), _ptr(correction), rows, K, E,
                                                int(top), int(groups), int(groups_kept), _ptr(ids), _ptr(weights), float(route_scale),
                                                _DTYPE_CODE[h.dtype], self._stream()))
        return ids, weights

    def experts_up(self, h: torch.Tensor, ids: torch.Tensor, w_up: torch.Tensor, act: torch.Tensor, activation: str = "relu2") -> torch.Tensor:
        """act[r * top + k] = relu(w_up[ids[r, k]] @ h[r])^2: the up product of experts without a gate; w_up [experts, inter, width]."""
        rows, K = h.shape
        top = ids.shape[1]
        E, inter = w_up.shape[0], w_up.shape[1]
        _need(activation == "relu2", f"activation {activation!r} unknown")
        _need(h.is_cuda and h.dim() == 2 and h.stride(1) == 1 and h.dtype in _DTYPE_CODE, "h must be a row-major GPU matrix")
        _dense(w_up, "w_up", h.dtype, (E, inter, K))
        _dense(ids, "ids", torch.int32, (rows, top))
        _dense(act, "act", h.dtype, (rows * top, inter))
        self._check(self.lib.fllm_experts_up(_ptr(h), h.stride(0) if rows > 1 else K, _ptr(ids), rows, top, _ptr(w_up), E, inter, K,
                                             _ptr(act), _DTYPE_CODE[h.dtype], self._stream()))
        return act

    def experts_grouped_ungated(self, h: torch.Tensor, ids: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, out: torch.Tensor) -> bool:
        """`experts_up` and `experts_down` in one call on the matrix cores (bfloat16, steps with enough pairs an expert): the
        pairs are grouped by expert on the device.  out float32 [rows * top, width].  False: not taken, nothing was written."""
        rows, K = h.shape
        top = ids.shape[1]
        E, inter = w_up.shape[0], w_up.shape[1]
        if h.dtype != torch.bfloat16 or not h.is_cuda:
            return False
        if rows < self.GROUPED_EXPERTS_ROWS and rows * top < self.GROUPED_EXPERTS_SHARE * E:
            return False
        N = w_down.shape[1]
        _need(h.dim() == 2 and h.stride(1) == 1, "h must be a row-major matrix")
        _dense(w_up, "w_up", h.dtype, (E, inter, K))
        _dense(w_down, "w_down", h.dtype, (E, N, inter))
        _dense(ids, "ids", torch.int32, (rows, top))
        _dense(out, "out", torch.float32, (rows * top, N))
        act = torch.empty((rows * top, inter), dtype=h.dtype, device=h.device)
        work = torch.empty((int(self.lib.fllm_experts_grouped_work_ints(rows * top, E)),), dtype=torch.int32, device=h.device)
        need = int(self.lib.fllm_experts_grouped_plane_floats(rows * top, E, N, inter))
        planes = torch.empty((need,), dtype=torch.float32, device=h.device) if need else None
        code = self.lib.fllm_experts_grouped_ungated(_ptr(h), h.stride(0), _ptr(ids), rows, top, _ptr(w_up), _ptr(w_down), E, inter, K, N,
                                                     _ptr(act), _ptr(out), _ptr(work), _ptr(planes), self._stream())
        if code == 1:
            return False
        self._check(code)
        return True

    def measured_ceilings(self, read_bytes: int = 4 << 30, repeats: int = 5) -> dict:
        """What the device delivers to kernels that do nothing else: GB/s of a kernel that only reads a buffer much larger
        than the caches, TFLOP/s of a kernel that only issues bfloat16 MFMA products.  The best of `repeats` timings."""
        dev = torch.device("cuda", torch.cuda.current_device())
        props = torch.cuda.get_device_properties(dev)
        blocks = props.multi_processor_count * 8
        buf = torch.zeros(read_bytes, dtype=torch.uint8, device=dev)
        sink = torch.zeros(max(blocks, 2 * props.multi_processor_count * 512), dtype=torch.float32, device=dev)
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        best_read, best_mfma = 0.0, 0.0
        iters, mfma_blocks = 4096, 2 * props.multi_processor_count
        for _ in range(repeats + 1):
            start.record()
            self._check(self.lib.fllm_probe_read(_ptr(buf), buf.numel(), _ptr(sink), blocks, self._stream()))
            end.record()
            end.synchronize()
            best_read = max(best_read, buf.numel() / (start.elapsed_time(end) * 1e-3) / 1e9)
            start.record()
            flops = self.lib.fllm_probe_mfma_bf16(_ptr(sink), mfma_blocks, iters, self._stream())
            end.record()
            end.synchronize()
            if flops < 0:
                raise KernelError(self.lib.fllm_last_error().decode("utf-8", "replace"))
            best_mfma = max(best_mfma, flops / (start.elapsed_time(end) * 1e-3) / 1e12)
        return {"hbm_read_gbs": best_read, "mfma_bf16_tflops": best_mfma}

    def carry_ids(self, ids: torch.Tensor, source: torch.Tensor, previous: torch.Tensor) -> torch.Tensor:
        """ids[r] = previous[source[r]] where source[r] >= 0 (int32 device tensors): tokens an earlier step chose
        become this step's input without passing through the host."""
        rows = ids.numel()
        _dense(ids, "ids", torch.int32)
        _dense(source, "source", torch.int32, (rows,))
        _dense(previous, "previous", torch.int32)
        self._check(self.lib.fllm_carry_ids(_ptr(ids), _ptr(source), _ptr(previous), rows, previous.numel(), self._stream()))
        return ids

    def argmax(self, logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        rows, vocab = logits.shape
        _dense(logits, "logits", torch.float32)
        _dense(out, "out", torch.int32, (rows,))
        self._check(self.lib.fllm_argmax(_ptr(logits), _ptr(out), rows, vocab, self._stream()))
        return out

    def adjust_logits(self, logits: torch.Tensor, packed: torch.Tensor, sections: Sequence[int],
                      last_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Penalties, biases, blocked and allowed ids on float32 logits [rows, vocab], in place (fllm_adjust_logits).
        `packed`: one int32 device tensor holding, one behind the other, the row records (14 words a row: the three
        penalties as float bits, then seen_off, seen_len, bias_off, bias_len, blocked_off, blocked_len, last_row,
        allowed_off, allowed_len, pairs_off, pairs_len), the seen ids, the seen counts, the bias ids, the bias values
        (float bits), the blocked ids, the allowed ids (rising within a row) and the pairs (first all "if the newest
        token is" ids, then all "block" ids); `sections`: (entries of the seen lists, of the bias lists, blocked ids,
        allowed ids, pairs), each over all rows.
        `last_tokens`: int32 device tensor that the records' last_row points into."""
        rows, vocab = logits.shape
        seen, bias, blocked, allowed, pairs = (int(n) for n in sections)
        _dense(logits, "logits", torch.float32)
        _dense(packed, "packed", torch.int32, (rows * ADJUST_ROW_WORDS + 2 * seen + 2 * bias + blocked + allowed + 2 * pairs,))
        if last_tokens is not None:
            _dense(last_tokens, "last_tokens", torch.int32)
        base = packed.data_ptr()
        at = rows * ADJUST_ROW_WORDS
        lists = AdjustLists()
        for name, count in (("seen_ids", seen), ("seen_counts", seen), ("bias_ids", bias), ("bias_values", bias),
                            ("blocked_ids", blocked), ("allowed_ids", allowed), ("if_last", pairs), ("then_blocked", pairs)):
            setattr(lists, name, base + 4 * at)
            at += count
        self._check(self.lib.fllm_adjust_logits(_ptr(logits), rows, vocab, base, ctypes.byref(lists), _ptr(last_tokens), self._stream()))
        return logits

    def logprobs(self, logits: torch.Tensor, wanted_rows: torch.Tensor, tokens: torch.Tensor, top: int,
                 values: torch.Tensor, ids: torch.Tensor) -> None:
        """Log-probabilities in the softmax of float32 logits [rows, vocab] (fllm_logprobs): for each row named in
        `wanted_rows` (int32 on the device, every one inside [0, rows): the caller's word), `values[w, 0]` is that of
        `tokens[row]` and `values[w, 1:]`, `ids[w, 1:]` are the `top` likeliest tokens, the lower id first among equals;
        `ids[w, 0]` repeats the chosen token.  A row with a NaN or +inf, or without a finite value, gives NaN."""
        rows, vocab = logits.shape
        wanted = wanted_rows.numel()
        _dense(logits, "logits", torch.float32)
        _dense(wanted_rows, "wanted_rows", torch.int32, (wanted,))
        _dense(tokens, "tokens", torch.int32, (rows,))
        _dense(values, "values", torch.float32, (wanted, 1 + top))
        _dense(ids, "ids", torch.int32, (wanted, 1 + top))
        self._check(self.lib.fllm_logprobs(_ptr(logits), rows, vocab, _ptr(wanted_rows), wanted, _ptr(tokens), int(top),
                                           _ptr(values), _ptr(ids), self._stream()))

    def logprobs_processed(self, logits: torch.Tensor, wanted_rows: torch.Tensor, tokens: torch.Tensor, params: torch.Tensor,
                           top: int, values: torch.Tensor, ids: torch.Tensor) -> None:
        """As `logprobs`, in the distribution each token was drawn from (fllm_logprobs_processed): `logits` are what the
        sampler saw (penalties and biases applied), `params` the `SampleRow` records `sample` took (uint8 [rows, 32]):
        temperature, then top-k, min-p and top-p with the sampler's ties; a greedy row is a point mass.  A chosen token
        that the filters leave out gives -inf; where fewer than `top` tokens are left, the rest of `ids` is -1."""
        rows, vocab = logits.shape
        wanted = wanted_rows.numel()
        _dense(logits, "logits", torch.float32)
        _dense(wanted_rows, "wanted_rows", torch.int32, (wanted,))
        _dense(tokens, "tokens", torch.int32, (rows,))
        _dense(params, "params", torch.uint8, (rows, SAMPLE_ROW_BYTES))
        _dense(values, "values", torch.float32, (wanted, 1 + top))
        _dense(ids, "ids", torch.int32, (wanted, 1 + top))
        self._check(self.lib.fllm_logprobs_processed(_ptr(logits), rows, vocab, _ptr(wanted_rows), wanted, _ptr(tokens), _ptr(params),
                                                     int(top), _ptr(values), _ptr(ids), self._stream()))

    def sample(self, logits: torch.Tensor, work: torch.Tensor, params: torch.Tensor, out: torch.Tensor,
               kinds: int = 7) -> torch.Tensor:
        """`params`: uint8 GPU tensor [rows, 32] holding `SampleRow` records.  `kinds`: what the caller knows of the rows,
        a sum of 1 (some have a temperature and no filter: their draw looks at every token, and several workgroups
        share such a row), 2 (some are of another kind) and 4 (some of those have a top-k of at most 64: several
        workgroups share such a row as well); 7 when nothing is known."""
        rows, vocab = logits.shape
        _dense(logits, "logits", torch.float32)
        _dense(work, "work", torch.float32, (rows, vocab))
        _dense(params, "params", torch.uint8, (rows, SAMPLE_ROW_BYTES))
        _dense(out, "out", torch.int32, (rows,))
        self._check(self.lib.fllm_sample(_ptr(logits), _ptr(work), _ptr(params), _ptr(out), rows, vocab, int(kinds), self._stream()))
        return out
