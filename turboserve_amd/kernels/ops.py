"""Python face of the HIP kernels: shape checks on the host, then one C call per op.

Every op runs on the current torch stream of the tensors' device.  There is no fallback: if
the library cannot be built or loaded, or a tensor is not on a GPU, the op raises.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p
from dataclasses import dataclass

import torch

from turboserve_amd.kernels import build

TS_F32 = 0
TS_BF16 = 1

_ERRORS = {
    1: "unsupported dtype code",
    2: "a size the kernel does not take",
    3: "the kernel launch failed",
    4: "null pointer or inconsistent arguments",
}


class KernelError(RuntimeError):
    """A kernel refused its arguments or failed to launch."""


def glu_rule(rule) -> tuple[float, float, float, float]:
    """``(steepness, limit, up_shift, cubic)`` of a gated unit ``g' * sigmoid(steepness * (g' + cubic *
    g'^3)) * (u' + up_shift)`` with ``g' = min(g, limit)``, ``u' = clamp(u, -limit, limit)`` where
    ``limit > 0``; a rule of three numbers has no cubic term."""
    values = tuple(float(v) for v in rule)
    if len(values) == 3:
        values = (*values, 0.0)
    if len(values) != 4:
        raise KernelError(f"a gated unit's rule is (steepness, limit, up_shift[, cubic]), not {rule!r}")
    return values


#: ``silu(gate) * up``.
SWIGLU_RULE = (1.0, 0.0, 0.0, 0.0)
#: The tanh form of GELU on the gate: ``0.5 g (1 + tanh(c (g + a g^3))) = g sigmoid(2 c (g + a g^3))``.
GELU_TANH_RULE = (2.0 * (2.0 / 3.141592653589793) ** 0.5, 0.0, 0.0, 0.044715)


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return TS_F32
    if dtype == torch.bfloat16:
        return TS_BF16
    raise KernelError(f"kernels take float32 or bfloat16, not {dtype}")


_SIGNATURES: dict[str, dict[str, list]] = {
    "core": {
        "ts_embed": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "ts_rmsnorm": [c_void_p, c_void_p, c_void_p, c_float, c_int, c_int, c_float, c_int, c_int, c_void_p],
        "ts_add_rmsnorm": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p, c_float,
                           c_int, c_int, c_float, c_int, c_int, c_void_p, c_int, c_long, c_void_p, c_float, c_float, c_void_p],
        "ts_swiglu": [c_void_p, c_void_p, c_int, c_int, c_long, c_int, c_int, c_int, c_float, c_float, c_float, c_float, c_int,
                      c_void_p],
        "ts_activate": [c_void_p, c_void_p, c_int, c_int, c_long, c_int, c_int, c_int, c_int, c_void_p],
        "ts_rope_store": [c_void_p, c_long, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p, c_void_p, c_void_p,
                          c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "ts_gather_rows": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
        "ts_patch_tokens": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
        "ts_paged_attention_generic": [c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int,
                                       c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                       c_float, c_float, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p, c_int, c_int, c_int,
                                       c_void_p],
        "ts_attention_tiles": [c_void_p, c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                               c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_int,
                               c_int, c_float, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p],
        "ts_attention_tiles_combine": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float,
                                       c_void_p, c_void_p],
        "ts_head_norm_store": [c_void_p, c_long, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                               c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_int, c_int, c_int, c_int, c_float, c_int,
                               c_int, c_void_p],
        "ts_span_norm_store": [c_void_p, c_long, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_float, c_float, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "ts_latent_store": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p, c_float, c_void_p,
                            c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                            c_void_p],
        "ts_head_gate": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_long, c_int, c_int, c_int, c_int, c_int, c_int,
                         c_float, c_long, c_void_p],
        "ts_scaled_pair": [c_void_p, c_void_p, c_int, c_int, c_long, c_float, c_void_p, c_int, c_int, c_long, c_float, c_long,
                           c_int, c_void_p],
        "ts_add_tanh_norm": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p, c_float, c_void_p, c_int,
                             c_int, c_int, c_void_p, c_int, c_long, c_void_p],
        "ts_tanh_cap": [c_void_p, c_long, c_float, c_void_p],
        "ts_short_conv": [c_void_p, c_int, c_void_p, c_int, c_int, c_long, c_int, c_int, c_int, c_void_p, c_int, c_void_p,
                          c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "ts_short_conv_carry": [c_void_p, c_void_p, c_int, c_int, c_long, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                                c_int, c_int, c_void_p],
        "ts_delta_prepare": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_int, c_int,
                             c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "ts_delta_scan": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                          c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "ts_delta_finish": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_int, c_int, c_int, c_void_p, c_void_p,
                            c_float, c_int, c_int, c_int, c_int, c_float, c_long, c_void_p],
        "ts_stream_fold": [c_void_p, c_void_p, c_int, c_int, c_long, c_long, c_int, c_int, c_void_p],
        "ts_stream_pair": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
        "ts_linear_state_scan": [c_void_p, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p, c_float, c_void_p, c_void_p,
                                 c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                 c_int, c_void_p],
        "ts_linear_state_carry": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "ts_linear_state_finish": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p, c_float, c_int, c_int, c_int,
                                   c_int, c_int, c_int, c_void_p],
        "ts_embed_positions": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "ts_copy_f32": [c_void_p, c_void_p, c_long, c_void_p],
        "ts_stream_offset": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
        "ts_moe_select": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float,
                          c_int, c_void_p, c_int, c_int, c_void_p],
        "ts_moe_pair_rows": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float,
                             c_float, c_float, c_float, c_int, c_void_p],
        "ts_moe_group": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
        "ts_moe_grouped_rows": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                c_int, c_float, c_float, c_float, c_float, c_void_p],
        "ts_moe_combine": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p, c_int, c_int, c_int,
                           c_int, c_void_p, c_int, c_void_p, c_void_p],
        "ts_gemm_plain": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long,
                          c_int, c_int, c_void_p],
        "ts_gemm_tiled": [c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                          c_int, c_float, c_float, c_float, c_float, c_void_p],
        "ts_gemm_wide": [c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                         c_int, c_int, c_int, c_int, c_float, c_float, c_float, c_float, c_void_p],
        "ts_gemm_skinny_resident": [c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                    c_int, c_int, c_int, c_void_p],
        "ts_argmax": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
        "ts_hbm_read": [c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_long, c_long, c_int, c_long, c_long, c_int,
                        c_void_p],
        "ts_sample": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p,
                      c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    },
}

def _attention_signatures(head_dim: int) -> dict[str, list]:
    return {
        f"ts_attention_decode_d{head_dim}": [c_void_p, c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_void_p,
                                             c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                             c_int, c_float, c_float, c_int, c_int, c_int, c_void_p, c_void_p],
        f"ts_attention_prefill_d{head_dim}": [c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int,
                                              c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float,
                                              c_float, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
        f"ts_attention_prefill_rows_d{head_dim}": [c_int, c_int],
        f"ts_attention_prefill_shape_d{head_dim}": [c_int, c_int, c_int, c_void_p, c_void_p],
    }


_LIBRARIES: dict[str, ctypes.CDLL] = {}


def load_module(module: str) -> ctypes.CDLL:
    """The loaded library of a kernel module, compiled first if nothing is built."""
    lib = _LIBRARIES.get(module)
    if lib is not None:
        return lib
    path = build.ensure_module(module)
    try:
        lib = ctypes.CDLL(str(path))
    except OSError as exc:  # pragma: no cover - depends on the machine
        raise KernelError(f"cannot load the kernel library {path}: {exc}") from exc
    signatures = _SIGNATURES.get(module, {})
    if module.startswith("attn_d"):
        signatures = _attention_signatures(int(module[6:]))
    for name, argtypes in signatures.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = c_int
    _LIBRARIES[module] = lib
    return lib


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _check(status: int, name: str) -> None:
    if status != 0:
        raise KernelError(f"{name}: {_ERRORS.get(status, f'error {status}')}")


def _need(cond: bool, message: str) -> None:
    if not cond:
        raise KernelError(message)


def _gpu(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernels run on the GPU only; got a tensor on " + str(t.device))


def _i32(t: torch.Tensor | None, name: str) -> None:
    if t is not None:
        _need(t.dtype == torch.int32 and t.is_contiguous(), f"{name} must be contiguous int32")


def _check_pages(k_pages: torch.Tensor, v_pages: torch.Tensor, dtype: torch.dtype, *, any_value_width: bool = False) -> None:
    """Key pages ``[NB, Hkv, BS, D]`` and transposed value pages ``[NB, Hkv, D, BS]`` (with
    ``any_value_width``: ``[NB, Hkv, Dv, BS]``)."""
    _need(k_pages.dim() == 4 and v_pages.dim() == 4 and k_pages.is_contiguous() and v_pages.is_contiguous()
          and k_pages.dtype == dtype and v_pages.dtype == dtype,
          "pages must be contiguous 4-d tensors of the queries' dtype")
    nb, kv_heads, block_size, head_dim = k_pages.shape
    if any_value_width:
        _need(v_pages.shape[0] == nb and v_pages.shape[1] == kv_heads and v_pages.shape[3] == block_size and v_pages.shape[2] >= 1,
              "value pages must be [NB, Hkv, Dv, BS] for key pages [NB, Hkv, BS, D]")
        return
    _need(tuple(v_pages.shape) == (nb, kv_heads, head_dim, block_size),
          "value pages must be [NB, Hkv, D, BS] for key pages [NB, Hkv, BS, D]")


#: Largest head size the attention parts take (the store that norms heads holds one; the matrix-core kernels stop at 256).
ATTENTION_MAX_HEAD_DIM = 512
#: Longest key row and widest value the generic attention kernel takes (a layer that caches one row for all heads).
ATTENTION_MAX_ROW = 1024


def attention_geometry_error(num_heads: int, num_kv_heads: int, head_dim: int) -> str | None:
    """Why no attention kernel of this library takes a geometry, or ``None`` if one does.  A pure
    function of the sizes, so a part can refuse at construction, before any weight is read."""
    if num_heads < 1 or num_kv_heads < 1 or num_heads % num_kv_heads != 0:
        return f"{num_heads} query heads are not a multiple of {num_kv_heads} KV heads"
    if num_heads > 65535:
        return f"{num_heads} query heads are more than a launch's 65,535"
    if head_dim < 2 or head_dim % 2 != 0:
        return f"a head size of {head_dim} is not even (keys and values are written in pairs)"
    if head_dim > ATTENTION_MAX_HEAD_DIM:
        return f"a head size of {head_dim} is above the {ATTENTION_MAX_HEAD_DIM} the attention kernels take"
    return None


def prefill_block_list(query_lens, context_lens, rows: int) -> list[list[int]]:
    """``[request index, first row]`` of every block of ``rows`` consecutive rows of requests that
    bring ``query_lens`` tokens and hold ``context_lens`` afterwards, rows numbered through the
    requests in order; blocks whose last row sees the most keys come first."""
    blocks, first_row = [], 0
    for index, (count, context) in enumerate(zip(query_lens, context_lens)):
        for offset in range(0, count, rows):
            blocks.append((context - count + min(offset + rows, count), index, first_row + offset))
        first_row += count
    blocks.sort(key=lambda b: -b[0])
    return [[block[1], block[2]] for block in blocks]


#: Keys a round of the prefill attention kernel for blocks of 32 rows takes (its "window").
PREFILL_WINDOW_KEYS = 32
#: Most workgroups that share the keys of one block.
PREFILL_MAX_SHARES = 16


def prefill_block_windows(first_position: int, rows: int, window: int) -> int:
    """Windows of 32 keys that a block of ``rows`` rows, the first at ``first_position``, runs
    over: from the window that holds the lowest key its first row sees to its last row's own."""
    lowest = max(0, first_position - window + 1) if window > 0 else 0
    begin = lowest - lowest % PREFILL_WINDOW_KEYS
    return -(-(first_position + rows - begin) // PREFILL_WINDOW_KEYS)


def prefill_share_list(query_lens, context_lens, rows: int, window: int, per_block: int, places: int,
                       min_windows: int, *, combine_cost: int = 20):
    """The work list of the prefill attention with the keys of long blocks shared out over several
    workgroups, where that shortens the launch: ``(blocks, ranges, combine)`` as lists of
    ``[request, first row]``, ``[first window, windows, slot]`` (slot -1, windows 0: a whole block) and
    ``[first row, rows, first slot, shares]``; ``ranges`` and ``combine`` are empty where nothing
    is shared out and the list is :func:`prefill_block_list`'s.

    An entry becomes ``per_block`` workgroups, ``places`` of which run at a time.  Sharing pays
    where whole blocks leave places idle (a short portion at the end of a long context: 512
    tokens behind 7,680 take 84 us instead of 187 on an MI355X), and only as far as every
    workgroup still has a place at once: a second workgroup's start on a compute unit costs
    about what ten windows take, so a prompt of 2,048 tokens alone, whose whole blocks fill the
    device, is slower with its long blocks in two (77 against 66 us).  So the smallest share
    size (from ``min_windows`` up; a block's windows are spread evenly over its shares) is taken
    at which all workgroups run at once, if the longest entry gets shorter by more than putting
    the shares together costs (``combine_cost`` windows: the second kernel and the sums' way
    through memory)."""
    whole, first_row = [], 0
    for index, (count, context) in enumerate(zip(query_lens, context_lens)):
        for offset in range(0, count, rows):
            here = min(rows, count - offset)
            whole.append((prefill_block_windows(context - count + offset, here, window), index, first_row + offset, here))
        first_row += count
    plain = prefill_block_list(query_lens, context_lens, rows)
    longest = max((block[0] for block in whole), default=0)
    if (rows != PREFILL_WINDOW_KEYS or per_block < 1 or longest < 2 * min_windows
            or (len(whole) + 1) * per_block > places):
        return plain, [], []

    def shares_of(windows: int, size: int) -> int:
        return 1 if windows <= size else min(PREFILL_MAX_SHARES, -(-windows // size))

    def fits(size: int) -> bool:
        return sum(shares_of(block[0], size) for block in whole) * per_block <= places

    low, high = min_windows, longest  # whole blocks (size = longest) fit
    while low < high:
        size = (low + high) // 2
        if fits(size):
            high = size
        else:
            low = size + 1
    size = low
    if max(-(-block[0] // shares_of(block[0], size)) for block in whole) + combine_cost >= longest:
        return plain, [], []
    entries, combine, slot = [], [], 0
    for windows, index, row, here in whole:
        shares = shares_of(windows, size)
        if shares == 1:
            entries.append((windows, index, row, 0, 0, -1))
            continue
        each = -(-windows // shares)
        shares = -(-windows // each)  # no empty share
        combine.append([row, here, slot, shares])
        for share in range(shares):
            entries.append((min(each, windows - share * each), index, row, share * each, min(each, windows - share * each), slot))
            slot += 1
    entries.sort(key=lambda entry: -entry[0])
    return [[e[1], e[2]] for e in entries], [[e[3], e[4], e[5]] for e in entries], combine


@dataclass
class PrefillWork:
    """The work list of one prefill attention launch on the device (see :meth:`Ops.prefill_blocks`)."""

    blocks: torch.Tensor                 # int32 [n, 2]: request index, first row
    ranges: torch.Tensor | None = None   # int32 [n, 3]: first window, windows, slot; None: whole blocks only
    combine: torch.Tensor | None = None  # int32 [c, 4]: first row, rows, first slot, shares
    slots: int = 0


class Ops:
    """The kernel library bound to one device."""

    def __init__(self, device: torch.device | str = "cuda:0", modules: tuple[str, ...] = ("core",)) -> None:
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise KernelError(f"the kernels need a GPU device, not {self.device}")
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible to torch; this engine has no CPU path")
        self.core = load_module("core")
        for module in modules:
            load_module(module)
        self._device_index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        self._raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        self._tiled_plans: dict[tuple, tuple[int, int, int]] = {}  # (m, n, k, max_splits) -> grid of the tiled product
        self._wide_plans: dict[tuple, tuple[int, int, int, int, int]] = {}  # (m, n, k, one range) -> grid of the wide product
        #: (rows a step's products run at, N, K, kind) -> whether this engine's own product was the
        #: faster one when both were timed (``time_wide_choices``).
        self.wide_choices: dict[tuple, bool] = {}
        #: The same keys -> (milliseconds of the own product, of the library's) as timed.
        self.wide_timings: dict[tuple, tuple[float, float]] = {}
        #: While true, a product of many rows whose choice is not known yet runs both ways, timed.
        self.time_wide_choices = False
        #: Compute units of the device (256 on an MI355X): the launch plans below size their grids by it.
        self.compute_units = int(torch.cuda.get_device_properties(self.device).multi_processor_count)
        #: Wavefronts a decode attention launch aims for (each keeps two windows of loads in
        #: flight): two per compute unit while the step has few requests x KV heads, one per SIMD
        #: from half as many of those as there are compute units.  Measured through the engine at
        #: the 7B shape (4 KV heads), context 8,192, two per unit against four: 3.78 against 3.83
        #: ms a step with 4 requests, 4.11 against 4.15 with 8, 4.19 against 4.23 with 16 (context
        #: 4,096), 6.27 against 6.28 with 32, 9.43 against 9.29 with 64.
        self.decode_waves_few_pairs = 2 * self.compute_units
        self.decode_waves_many_pairs = 4 * self.compute_units
        #: Wavefronts (16 weight rows x one range of K each) the resident product aims for: 16 per compute unit.
        self.skinny_resident_waves = 16 * self.compute_units

    def device_ints(self, values) -> torch.Tensor:
        """A list (or nested list) of integers as an int32 tensor on the device, copied from pinned
        memory behind the work already launched: a copy from pageable memory would make the host
        wait until the stream has drained, and the device then waits for the host in turn."""
        host = torch.tensor(values, dtype=torch.int32).pin_memory()
        return host.to(self.device, non_blocking=True)

    def stream(self) -> int:
        """The handle of torch's current stream on this device (what every launch goes to)."""
        if self._raw_stream is not None:
            return self._raw_stream(self._device_index)  # 0.06 us; the public way below takes 2 us, a step has 260 launches
        return torch.cuda.current_stream(self.device).cuda_stream

    # -- rows ---------------------------------------------------------------------------------

    def embed(self, table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """``float32 [T, H]`` rows of ``table [V, H]`` at ``ids [T]`` (the start of the 32-bit
        residual stream)."""
        _gpu(table, ids)
        _i32(ids, "ids")
        _need(table.dim() == 2 and table.is_contiguous(), "table must be contiguous [V, H]")
        tokens, (vocab, hidden) = ids.numel(), table.shape
        if out is None:
            out = torch.empty((tokens, hidden), dtype=torch.float32, device=table.device)
        _need(out.shape == (tokens, hidden) and out.dtype == torch.float32 and out.is_contiguous(),
              "out must be contiguous float32 [T, H]")
        _check(self.core.ts_embed(_ptr(out), _ptr(table), _ptr(ids), tokens, hidden, vocab,
                                  dtype_code(table.dtype), self.stream()), "ts_embed")
        return out

    def rmsnorm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, *, gain_offset: float = 0.0,
                one_rounding: bool = False) -> torch.Tensor:
        """``weight * round(x * rsqrt(mean(x^2) + eps))`` or, with ``one_rounding``,
        ``round(x * rsqrt(mean(x^2) + eps) * (gain_offset + weight))`` computed in 32-bit."""
        _gpu(x, weight)
        _need(x.dim() == 2 and x.is_contiguous(), "x must be contiguous [T, H]")
        _need(weight.shape == (x.shape[1],) and weight.dtype == x.dtype and weight.is_contiguous(),
              "weight must be [H] of x's dtype")
        y = torch.empty_like(x)
        _check(self.core.ts_rmsnorm(_ptr(y), _ptr(x), _ptr(weight), float(eps), x.shape[0], x.shape[1],
                                    float(gain_offset), 1 if one_rounding else 0, dtype_code(x.dtype), self.stream()),
               "ts_rmsnorm")
        return y

    @staticmethod
    def _partials(t: torch.Tensor, rows: int, width: int, dtype: torch.dtype, what: str) -> tuple[int, int, int]:
        """``(is_float32_partials, splits, split_stride)`` of a projection output: either
        ``[rows, width]`` of the run dtype, or ``[S, rows, width]`` 32-bit partial sums (what the
        skinny product leaves for its consumer to add up)."""
        _need(t.is_contiguous(), f"{what} must be contiguous")
        if t.dim() == 3:
            _need(t.dtype == torch.float32 and t.shape[1:] == (rows, width),
                  f"{what}: partial sums must be float32 [S, {rows}, {width}]")
            return 1, t.shape[0], rows * width
        _need(t.shape == (rows, width) and t.dtype == dtype, f"{what} must be [{rows}, {width}] of {dtype}")
        return 0, 1, 0

    def dense(self, t: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
        """A projection output as one ``[rows, width]`` tensor of ``dtype`` (partial sums added
        up), for consumers that have no fused form."""
        return t.sum(dim=0).to(dtype) if t.dim() == 3 else t

    def add_rmsnorm(
        self,
        residual: torch.Tensor,
        pending: torch.Tensor | None,
        weight: torch.Tensor,
        eps: float,
        rows: torch.Tensor | None = None,
        *,
        gain_offset: float = 0.0,
        one_rounding: bool = False,
        also: torch.Tensor | None = None,
        pending_norm: tuple[torch.Tensor, float, float] | None = None,
    ) -> torch.Tensor:
        """``residual += pending`` in 32-bit (in place) and the normalised sum in ``weight``'s
        dtype; with ``rows`` only those rows, and ``residual`` is left alone.  ``pending`` is a
        ``[T, H]`` tensor of the run dtype or ``[S, T, H]`` 32-bit partial sums.  ``also``: a second
        addend, ``[S, T, H]`` 32-bit partial sums.  The gain is applied as in :meth:`rmsnorm`.
        ``pending_norm = (gain [H], eps, scale)``: the pending output is first divided by its own
        root mean square (``eps`` inside the root) and multiplied by ``gain`` and ``scale``, in
        32-bit, so what is added is ``scale * norm(pending)``."""
        _gpu(residual, pending, weight, rows)
        _i32(rows, "rows")
        _need(residual.dim() == 2 and residual.dtype == torch.float32 and residual.is_contiguous(),
              "residual must be contiguous float32 [T, H]")
        tokens, hidden = residual.shape
        _need(weight.shape == (hidden,) and weight.is_contiguous(), "weight must be [H]")
        is_f32, splits, stride = (0, 1, 0)
        if pending is not None:
            is_f32, splits, stride = self._partials(pending, tokens, hidden, weight.dtype, "pending")
        also_splits, also_stride = 0, 0
        if also is not None:
            _gpu(also)
            _need(also.dim() == 3 and also.dtype == torch.float32 and also.is_contiguous() and also.shape[1:] == (tokens, hidden),
                  "a second addend must be float32 partial sums [S, T, H]")
            also_splits, also_stride = also.shape[0], tokens * hidden
        post_gain, post_eps, post_scale = None, 0.0, 1.0
        if pending_norm is not None:
            post_gain, post_eps, post_scale = pending_norm
            _gpu(post_gain)
            _need(pending is not None and also is None, "a norm on the pending output needs one, and no second addend")
            _need(post_gain.shape == (hidden,) and post_gain.dtype == weight.dtype and post_gain.is_contiguous(),
                  "the pending output's gain must be [H] of the run dtype")
        out_rows = tokens if rows is None else rows.numel()
        y = self.rows_buffer(out_rows, hidden, weight.dtype, residual.device)
        _check(self.core.ts_add_rmsnorm(_ptr(y), _ptr(residual), _ptr(pending), is_f32, splits, stride, _ptr(weight),
                                        _ptr(rows), float(eps), out_rows, hidden, float(gain_offset),
                                        1 if one_rounding else 0, dtype_code(weight.dtype), _ptr(also), also_splits,
                                        also_stride, _ptr(post_gain), float(post_eps), float(post_scale), self.stream()),
               "ts_add_rmsnorm")
        return y

    def swiglu(self, gate_up: torch.Tensor, dtype: torch.dtype | None = None, *, paired: bool = False,
               rule: tuple[float, float, float] = (1.0, 0.0, 0.0)) -> torch.Tensor:
        """``silu(gate) * up`` of the fused ``[T, 2 I]`` projection (or its ``[S, T, 2 I]`` 32-bit
        partial sums) -> ``[T, I]`` of ``dtype`` (the projection's own if it is not partial).
        Gate fills the first ``I`` columns and up the last, or, with ``paired``, they alternate
        (gate ``i`` in column ``2 i``, up ``i`` in column ``2 i + 1``).  ``rule = (steepness,
        limit, up_shift)`` is the gated unit's: with ``g' = min(g, limit)`` and ``u' = clamp(u,
        -limit, limit)`` where ``limit > 0``, ``g' * sigmoid(steepness * g') * (u' + up_shift)``."""
        _gpu(gate_up)
        tokens, width = gate_up.shape[-2], gate_up.shape[-1]
        _need(width % 2 == 0, "gate_up must be [T, 2 I]")
        out_dtype = dtype or gate_up.dtype
        if gate_up.dim() == 3:
            _need(dtype is not None, "partial sums need the output dtype")
        is_f32, splits, stride = self._partials(gate_up, tokens, width, out_dtype, "gate_up")
        inter = width // 2
        out = self.rows_buffer(tokens, inter, out_dtype, gate_up.device)
        _check(self.core.ts_swiglu(_ptr(out), _ptr(gate_up), is_f32, splits, stride, tokens, inter,
                                   1 if paired else 0, *glu_rule(rule),
                                   dtype_code(out_dtype), self.stream()), "ts_swiglu")
        return out

    #: The activations :meth:`activate` knows, by name.
    ACTIVATIONS = {"relu_squared": 0, "relu": 1, "silu": 2, "gelu_tanh": 3}

    def activate(self, proj: torch.Tensor, kind: str, dtype: torch.dtype | None = None) -> torch.Tensor:
        """``act(proj)`` element by element, in 32-bit with one rounding: ``proj`` is a projection
        ``[T, I]`` of the run dtype or its ``[S, T, I]`` 32-bit partial sums, the result ``[T, I]`` of
        ``dtype``.  ``kind``: ``relu_squared`` (``max(x, 0)^2``), ``relu``, ``silu``, ``gelu_tanh``."""
        _gpu(proj)
        _need(kind in self.ACTIVATIONS, f"activation {kind!r} is not one of {sorted(self.ACTIVATIONS)}")
        tokens, inter = proj.shape[-2], proj.shape[-1]
        out_dtype = dtype or proj.dtype
        if proj.dim() == 3:
            _need(dtype is not None, "partial sums need the output dtype")
        is_f32, splits, stride = self._partials(proj, tokens, inter, out_dtype, "projection")
        out = self.rows_buffer(tokens, inter, out_dtype, proj.device)
        _check(self.core.ts_activate(_ptr(out), _ptr(proj), is_f32, splits, stride, tokens, inter, self.ACTIVATIONS[kind],
                                     dtype_code(out_dtype), self.stream()), "ts_activate")
        return out

    def gather_rows(self, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        _gpu(x, rows)
        _i32(rows, "rows")
        _need(x.dim() == 2 and x.is_contiguous(), "x must be contiguous [T, W]")
        out = torch.empty((rows.numel(), x.shape[1]), dtype=x.dtype, device=x.device)
        _check(self.core.ts_gather_rows(_ptr(out), _ptr(x), _ptr(rows), rows.numel(), x.shape[1],
                                        dtype_code(x.dtype), self.stream()), "ts_gather_rows")
        return out

    def patch_tokens(self, token_ids: torch.Tensor, patch: torch.Tensor, source: torch.Tensor) -> None:
        """``token_ids[i] = source[patch[i]]`` where ``patch[i] >= 0``, in place: a step's token
        ids taken from what the step before sampled, without the host having seen them."""
        _gpu(token_ids, patch, source)
        _i32(token_ids, "token_ids")
        _i32(patch, "patch")
        _i32(source, "source")
        _need(token_ids.dim() == 1 and patch.shape == token_ids.shape and source.dim() == 1 and source.numel() >= 1,
              "token_ids and patch must be [n], source [m >= 1]")
        _check(self.core.ts_patch_tokens(_ptr(token_ids), _ptr(patch), _ptr(source), token_ids.numel(), source.numel(),
                                         self.stream()), "ts_patch_tokens")

    def rope_store(
        self,
        proj: torch.Tensor,
        k_pages: torch.Tensor | None,
        v_pages: torch.Tensor | None,
        cos: torch.Tensor | None,
        sin: torch.Tensor | None,
        positions: torch.Tensor,
        slots: torch.Tensor | None,
        heads: int,
        kv_heads: int,
        head_dim: int,
        block_size: int,
        max_position: int,
        dtype: torch.dtype | None = None,
    ) -> tuple[torch.Tensor, int]:
        """Rotate q and k of the fused projection ``[T, (Hq + 2 Hkv) D]`` (skipped when ``cos`` is
        ``None``) and store k, v at ``slots`` into key pages ``[NB, Hkv, BS, D]`` and value pages
        ``[NB, Hkv, D, BS]`` (skipped when ``slots`` is ``None``).  Returns the tensor that holds
        the encoded queries and its row stride: the projection itself (rotated in place) when it
        is a tensor of the run dtype, a new ``[T, Hq D]`` tensor of ``dtype`` when it is 32-bit
        partial sums.  ``max_position`` is the largest position of the step, known on the host,
        and must lie inside the tables."""
        _gpu(proj, k_pages, v_pages, cos, sin, positions, slots)
        _i32(positions, "positions")
        _i32(slots, "slots")
        tokens = positions.numel()
        width = (heads + 2 * kv_heads) * head_dim
        run_dtype = dtype or proj.dtype
        if proj.dim() == 3:
            _need(dtype is not None, "partial sums need the run dtype")
        is_f32, splits, stride = self._partials(proj, tokens, width, run_dtype, "projection")
        _need(head_dim % 2 == 0, "head_dim must be even")
        if cos is not None:
            half = head_dim // 2
            _need(sin is not None and cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] == half
                  and cos.dtype == torch.float32 and sin.dtype == torch.float32
                  and cos.is_contiguous() and sin.is_contiguous(), "cos/sin must be float32 [capacity, D/2]")
            _need(max_position < cos.shape[0], f"position {max_position} is beyond the rotary tables ({cos.shape[0]})")
        if slots is not None:
            _need(slots.numel() == tokens, "one slot per token")
            _need(k_pages is not None and v_pages is not None, "slots given without pages")
            _check_pages(k_pages, v_pages, run_dtype)
            _need(k_pages.shape[1:] == (kv_heads, block_size, head_dim), "pages do not match the heads' geometry")
        if proj.dim() == 3:
            q_out = torch.empty((tokens, heads * head_dim), dtype=run_dtype, device=proj.device)
            q_stride = heads * head_dim
        else:
            q_out, q_stride = proj, width
        _check(self.core.ts_rope_store(_ptr(q_out), q_stride, _ptr(proj), is_f32, splits, stride, _ptr(k_pages),
                                       _ptr(v_pages), _ptr(cos), _ptr(sin), _ptr(positions), _ptr(slots), tokens,
                                       heads, kv_heads, head_dim, block_size, 0 if cos is None else 1,
                                       dtype_code(run_dtype), self.stream()), "ts_rope_store")
        return q_out, q_stride

    def embed_positions(self, table: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor,
                        at: torch.Tensor) -> torch.Tensor:
        """``float32 [T, H]``: row ``ids[t]`` of ``table [V, H]`` plus row ``positions[t]`` of the 32-bit
        position table ``at [capacity, H]`` (the host keeps every position below its capacity)."""
        _gpu(table, ids, positions, at)
        _i32(ids, "ids")
        _i32(positions, "positions")
        _need(table.dim() == 2 and table.is_contiguous(), "table must be contiguous [V, H]")
        tokens, (vocab, hidden) = ids.numel(), table.shape
        _need(positions.numel() == tokens, "one position per token")
        _need(at.dim() == 2 and at.shape[1] == hidden and at.dtype == torch.float32 and at.is_contiguous(),
              "the position table must be contiguous float32 [capacity, H]")
        out = torch.empty((tokens, hidden), dtype=torch.float32, device=table.device)
        _check(self.core.ts_embed_positions(_ptr(out), _ptr(table), _ptr(ids), _ptr(positions), _ptr(at), tokens, hidden,
                                            vocab, dtype_code(table.dtype), self.stream()), "ts_embed_positions")
        return out

    def copy_float32(self, x: torch.Tensor) -> torch.Tensor:
        """A copy of a contiguous 32-bit tensor made by a kernel: a step that is recorded holds
        kernels only, and torch's ``clone`` would record a copy node."""
        _gpu(x)
        _need(x.dtype == torch.float32 and x.is_contiguous(), "x must be contiguous float32")
        out = torch.empty_like(x)
        _check(self.core.ts_copy_f32(_ptr(out), _ptr(x), x.numel(), self.stream()), "ts_copy_f32")
        return out

    def stream_offset(self, residual: torch.Tensor, origin: torch.Tensor | None, offset: torch.Tensor | None) -> None:
        """``residual [T, H] += origin [T, H] + offset [H]`` in 32-bit, in place (either addend may
        be absent)."""
        _gpu(residual, origin, offset)
        _need(residual.dim() == 2 and residual.dtype == torch.float32 and residual.is_contiguous(),
              "residual must be contiguous float32 [T, H]")
        tokens, hidden = residual.shape
        if origin is not None:
            _need(origin.shape == residual.shape and origin.dtype == torch.float32 and origin.is_contiguous(),
                  "origin must be float32 like the residual")
        code = TS_F32
        if offset is not None:
            _need(offset.shape == (hidden,) and offset.is_contiguous(), "offset must be contiguous [H]")
            code = dtype_code(offset.dtype)
        _check(self.core.ts_stream_offset(_ptr(residual), _ptr(origin), _ptr(offset), tokens, hidden, code, self.stream()),
               "ts_stream_offset")

    def head_norm_store(
        self,
        proj: torch.Tensor,
        k_pages: torch.Tensor | None,
        v_pages: torch.Tensor | None,
        q_gain: torch.Tensor | None,
        k_gain: torch.Tensor | None,
        eps: float,
        positions: torch.Tensor,
        slots: torch.Tensor | None,
        heads: int,
        kv_heads: int,
        head_dim: int,
        value_dim: int,
        block_size: int,
        dtype: torch.dtype | None = None,
        *,
        gain_offset: float = 0.0,
        cos: torch.Tensor | None = None,
        sin: torch.Tensor | None = None,
        max_position: int = 0,
        keep_values: torch.Tensor | None = None,
        blend_values: tuple[torch.Tensor, float] | None = None,
        normed: bool = False,
        norm_after: bool = False,
        values_are_keys: bool = False,
        query_temperature: tuple[float, int] | None = None,
        tail: int = 0,
    ) -> tuple[torch.Tensor, int]:
        """Per-head norm of the q and k heads of the fused projection ``[T, Hq D + Hkv D + Hkv Dv]``
        (``x * rsqrt(mean(x^2) + eps) * (gain_offset + gain)`` in 32-bit, the gain ``[D]`` shared by
        the heads; no norm without gains), then the rotation by ``cos``/``sin [capacity, D/2]`` where
        given, one rounding, and the store of k and v at ``slots`` into key pages ``[NB, Hkv, BS,
        D]`` and value pages ``[NB, Hkv, Dv, BS]`` (skipped when ``slots`` is ``None``).  Returns
        the tensor that holds the queries and its row stride, as :meth:`rope_store` does.
        ``keep_values [T, Hkv Dv]`` 32-bit receives the step's values as projected;
        ``blend_values = (other [T, Hkv Dv] 32-bit, w)`` stores ``(1 - w) v + w other`` instead of ``v``
        (another layer's values of the same tokens mixed in, in 32-bit).  ``normed``: the heads are divided
        by their root mean square also without gains; ``norm_after``: the norm follows the rotation; tables
        ``[capacity, R/2]`` with ``R < D`` turn the first ``R`` elements of a head only; ``values_are_keys``:
        the projection is ``[T, Hq D + Hkv D]`` and the values are the key heads as projected;
        ``query_temperature = (coef, every)``: a query at position ``p`` is multiplied by ``1 + coef ln(floor((p
        + 1) / every) + 1)``; ``tail``: a row of the projection holds that many columns more behind the heads."""
        _gpu(proj, k_pages, v_pages, q_gain, k_gain, positions, slots, cos, sin, keep_values)
        _i32(positions, "positions")
        _i32(slots, "slots")
        tokens = positions.numel()
        width = (heads + kv_heads) * head_dim + (0 if values_are_keys else kv_heads * value_dim) + int(tail)
        _need(not values_are_keys or value_dim == head_dim, "values that are the keys have the keys' size")
        run_dtype = dtype or proj.dtype
        if proj.dim() == 3:
            _need(dtype is not None, "partial sums need the run dtype")
        is_f32, splits, stride = self._partials(proj, tokens, width, run_dtype, "projection")
        _need(1 <= head_dim <= ATTENTION_MAX_HEAD_DIM and value_dim >= 1, "head sizes outside what the kernel takes")
        _need((q_gain is None) == (k_gain is None), "both gains or none")
        for gain in (q_gain, k_gain):
            if gain is not None:
                _need(gain.shape == (head_dim,) and gain.dtype == run_dtype and gain.is_contiguous(),
                      "a gain must be [D] of the run dtype")
        if cos is not None:
            _need(sin is not None and cos.shape == sin.shape and cos.dim() == 2 and 1 <= cos.shape[1] <= head_dim // 2
                  and cos.dtype == torch.float32 and sin.dtype == torch.float32
                  and cos.is_contiguous() and sin.is_contiguous(), "cos/sin must be float32 [capacity, R/2], R <= D")
            _need(max_position < cos.shape[0], f"position {max_position} is beyond the rotary tables ({cos.shape[0]})")
        if slots is not None:
            _need(slots.numel() == tokens, "one slot per token")
            _need(k_pages is not None and v_pages is not None, "slots need pages")
            _check_pages(k_pages, v_pages, run_dtype, any_value_width=True)
            _need(k_pages.shape[1] == kv_heads and k_pages.shape[2] == block_size and k_pages.shape[3] == head_dim
                  and v_pages.shape[2] == value_dim, "pages do not fit the heads")
        if is_f32:
            q_out = self.rows_buffer(tokens, heads * head_dim, run_dtype, proj.device)
            q_stride = heads * head_dim
        else:
            q_out, q_stride = proj, width
        other, weight = (None, 0.0) if blend_values is None else blend_values
        coef, every = (0.0, 1) if query_temperature is None else query_temperature
        _need(every >= 1, "the query temperature counts positions in stretches of at least one")
        for held in (keep_values, other):
            if held is not None:
                _gpu(held)
                _need(slots is not None and held.dtype == torch.float32 and held.is_contiguous()
                      and held.shape == (tokens, kv_heads * value_dim), "values kept or mixed in are float32 [T, Hkv Dv], with slots")
        _check(self.core.ts_head_norm_store(
            _ptr(q_out), q_stride, _ptr(proj), is_f32, splits, stride, _ptr(k_pages), _ptr(v_pages), _ptr(q_gain),
            _ptr(k_gain), float(eps), float(gain_offset), _ptr(cos), _ptr(sin), _ptr(positions), _ptr(slots), tokens,
            heads, kv_heads, head_dim, value_dim, block_size, dtype_code(run_dtype), _ptr(keep_values), _ptr(other),
            float(weight), 1 if normed else 0, 1 if norm_after else 0, 0 if cos is None else 2 * cos.shape[1],
            1 if values_are_keys else 0, float(coef), int(every), int(tail), self.stream()), "ts_head_norm_store")
        return q_out, q_stride

    # -- stores and stream steps of other mixers ------------------------------------------------

    def span_norm_store(self, proj: torch.Tensor, k_pages: torch.Tensor | None, v_pages: torch.Tensor | None,
                        q_gain: torch.Tensor, k_gain: torch.Tensor, eps: float, slots: torch.Tensor | None, tokens: int,
                        heads: int, kv_heads: int, head_dim: int, value_dim: int, block_size: int,
                        dtype: torch.dtype | None = None, *, gain_offset: float = 0.0) -> tuple[torch.Tensor, int]:
        """The store of a mixer whose queries and keys are normalised over their whole projection:
        of the fused projection ``[T, Hq D + Hkv D + Hkv Dv]`` the ``Hq D`` query elements of a token
        become ``x * rsqrt(mean(x^2) + eps) * (gain_offset + q_gain)`` (statistics over all heads at
        once, ``q_gain [Hq D]``), its ``Hkv D`` key elements likewise with ``k_gain [Hkv D]``, in
        32-bit with one rounding; keys and values go to their pages at ``slots`` (skipped when
        ``None``).  Returns the tensor that holds the queries and its row stride, as
        :meth:`rope_store` does."""
        _gpu(proj, k_pages, v_pages, q_gain, k_gain, slots)
        _i32(slots, "slots")
        width = (heads + kv_heads) * head_dim + kv_heads * value_dim
        run_dtype = dtype or proj.dtype
        if proj.dim() == 3:
            _need(dtype is not None, "partial sums need the run dtype")
        is_f32, splits, stride = self._partials(proj, tokens, width, run_dtype, "projection")
        _need(q_gain.shape == (heads * head_dim,) and k_gain.shape == (kv_heads * head_dim,) and q_gain.dtype == run_dtype
              and k_gain.dtype == run_dtype and q_gain.is_contiguous() and k_gain.is_contiguous(),
              "the gains must be [Hq D] and [Hkv D] of the run dtype")
        if slots is not None:
            _need(slots.numel() == tokens, "one slot per token")
            _need(k_pages is not None and v_pages is not None, "slots need pages")
            _check_pages(k_pages, v_pages, run_dtype, any_value_width=True)
            _need(k_pages.shape[1] == kv_heads and k_pages.shape[2] == block_size and k_pages.shape[3] == head_dim
                  and v_pages.shape[2] == value_dim, "pages do not fit the heads")
        if is_f32:
            q_out = self.rows_buffer(tokens, heads * head_dim, run_dtype, proj.device)
            q_stride = heads * head_dim
        else:
            q_out, q_stride = proj, width
        _check(self.core.ts_span_norm_store(
            _ptr(q_out), q_stride, _ptr(proj), is_f32, splits, stride, _ptr(k_pages), _ptr(v_pages), _ptr(q_gain),
            _ptr(k_gain), float(eps), float(gain_offset), _ptr(slots), tokens, heads, kv_heads, head_dim, value_dim,
            block_size, dtype_code(run_dtype), self.stream()), "ts_span_norm_store")
        return q_out, q_stride

    def latent_store(self, proj: torch.Tensor, k_pages: torch.Tensor | None, gain: torch.Tensor, eps: float,
                     cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor | None,
                     heads: int, head_dim: int, rot_dim: int, rank: int, block_size: int, max_position: int,
                     dtype: torch.dtype | None = None, *, neighbours: bool = False, tail: int = 0) -> tuple[torch.Tensor, torch.Tensor]:
        """A latent-attention layer's pass over its fused projection ``[T, H (D + R) + C + R]`` (per
        head ``D`` plain and ``R`` rotated query elements, then the latent of ``C`` and the shared
        rotated key part of ``R``): the latent is divided by its root mean square and multiplied by
        ``gain [C]``; of the rotated parts the first ``2 * cos.shape[1]`` elements are turned by the
        position's angles; ``[latent | rotated key]`` goes to the key pages ``[NB, 1, BS, C + R]`` at
        ``slots``.  Returns ``(q_plain [T H, D], q_wide [T, H, C + R])``; of ``q_wide`` only the last
        ``R`` elements of every head are written (the turned query parts).  ``neighbours``: the pairs
        turned together are ``(2 i, 2 i + 1)`` instead of ``(i, i + turned / 2)``.  ``tail``: columns
        behind the rotated key part in every row of the projection that this pass does not read."""
        _gpu(proj, k_pages, gain, cos, sin, positions, slots)
        _i32(positions, "positions")
        _i32(slots, "slots")
        tokens = positions.numel()
        width = heads * (head_dim + rot_dim) + rank + rot_dim + int(tail)
        run_dtype = dtype or proj.dtype
        if proj.dim() == 3:
            _need(dtype is not None, "partial sums need the run dtype")
        is_f32, splits, stride = self._partials(proj, tokens, width, run_dtype, "projection")
        _need(gain.shape == (rank,) and gain.dtype == run_dtype and gain.is_contiguous(), "the gain must be [C] of the run dtype")
        _need(cos.shape == sin.shape and cos.dim() == 2 and cos.dtype == torch.float32 and sin.dtype == torch.float32
              and cos.is_contiguous() and sin.is_contiguous() and 1 <= cos.shape[1] and 2 * cos.shape[1] <= rot_dim,
              "cos/sin must be float32 [capacity, turned / 2] with turned <= R")
        _need(max_position < cos.shape[0], f"position {max_position} is beyond the rotary tables ({cos.shape[0]})")
        if slots is not None:
            _need(slots.numel() == tokens and k_pages is not None, "one slot per token, and pages")
            _need(k_pages.dim() == 4 and k_pages.is_contiguous() and k_pages.dtype == run_dtype
                  and tuple(k_pages.shape[1:]) == (1, block_size, rank + rot_dim), "key pages must be [NB, 1, BS, C + R]")
        q_plain = torch.empty((tokens * heads, head_dim), dtype=run_dtype, device=proj.device)
        q_wide = torch.empty((tokens, heads, rank + rot_dim), dtype=run_dtype, device=proj.device)
        _check(self.core.ts_latent_store(
            _ptr(q_plain), _ptr(q_wide), _ptr(proj), is_f32, splits, stride, _ptr(k_pages), _ptr(gain), float(eps),
            _ptr(cos), _ptr(sin), _ptr(positions), _ptr(slots), tokens, heads, head_dim, rot_dim, rank, 2 * cos.shape[1],
            block_size, 1 if neighbours else 0, int(tail), dtype_code(run_dtype), self.stream()), "ts_latent_store")
        return q_plain, q_wide

    def _columns_of(self, out: tuple[torch.Tensor, int] | None, tokens: int, width: int, dtype: torch.dtype, device):
        """Where a kernel writes ``[tokens, width]`` of ``dtype``: a buffer of its own, or the columns ``col0 .. col0 +
        width - 1`` of a wider ``[tokens, W]`` buffer handed in as ``(buffer, col0)``.  Returns ``(result, pointer, row
        stride)``."""
        if out is None:
            made = self.rows_buffer(tokens, width, dtype, device)
            return made, _ptr(made), width
        buffer, col0 = out
        _gpu(buffer)
        _need(buffer.dim() == 2 and buffer.is_contiguous() and buffer.dtype == dtype and buffer.shape[0] == tokens
              and 0 <= col0 and col0 + width <= buffer.shape[1], "the columns must lie inside a contiguous [T, W] buffer of the run dtype")
        return buffer, buffer.data_ptr() + col0 * buffer.element_size(), buffer.shape[1]

    def head_gate(self, values: torch.Tensor, proj: torch.Tensor, gate_at: int, heads: int, dtype: torch.dtype, *,
                  scale: float = 1.0, out: tuple[torch.Tensor, int] | None = None) -> torch.Tensor:
        """``[T, H Dv]`` of ``dtype``: head ``h``'s ``Dv`` elements of ``values [T, H Dv]`` (32-bit, or of ``dtype``) times
        ``sigmoid`` of column ``gate_at + h`` of the token's row of ``proj`` (a projection of the run
        dtype or its 32-bit partial sums) and times ``scale``, in 32-bit with one rounding.  ``out = (buffer, col0)``:
        the result is written into those columns of a wider buffer, which is returned."""
        _gpu(values, proj)
        tokens, width = proj.shape[-2], proj.shape[-1]
        is_f32, splits, stride = self._partials(proj, tokens, width, dtype, "projection")
        _need(values.dtype in (torch.float32, dtype) and values.is_contiguous() and values.dim() == 2 and values.shape[0] == tokens
              and values.shape[1] % heads == 0 and 0 <= gate_at and gate_at + heads <= width,
              "values must be [T, H Dv], 32-bit or of the run dtype, and the gates' columns inside the projection")
        result, pointer, out_stride = self._columns_of(out, tokens, values.shape[1], dtype, values.device)
        _check(self.core.ts_head_gate(pointer, _ptr(values), 1 if values.dtype == torch.float32 else 0, _ptr(proj), is_f32, splits,
                                      stride, tokens, width, gate_at, heads, values.shape[1] // heads, dtype_code(dtype),
                                      float(scale), out_stride, self.stream()), "ts_head_gate")
        return result

    def stream_fold(self, residual: torch.Tensor, part: torch.Tensor, dtype: torch.dtype, *, assign: bool = False) -> None:
        """``residual [T, H] += part`` in 32-bit, in place (``assign``: ``residual = part``); ``part`` is a
        ``[T, H]`` tensor of the run dtype or ``[S, T, H]`` 32-bit partial sums."""
        _gpu(residual, part)
        _need(residual.dim() == 2 and residual.dtype == torch.float32 and residual.is_contiguous(),
              "residual must be contiguous float32 [T, H]")
        tokens, hidden = residual.shape
        is_f32, splits, stride = self._partials(part, tokens, hidden, dtype, "part")
        _check(self.core.ts_stream_fold(_ptr(residual), _ptr(part), is_f32, splits, stride, tokens * hidden,
                                        1 if assign else 0, dtype_code(dtype), self.stream()), "ts_stream_fold")

    def stream_pair(self, x: torch.Tensor, origin: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
        """``[T, 2 H]`` of ``dtype``: every row of the 32-bit ``x`` followed by the same row of ``origin``."""
        _gpu(x, origin)
        _need(x.dim() == 2 and x.dtype == torch.float32 and x.is_contiguous() and origin.shape == x.shape
              and origin.dtype == torch.float32 and origin.is_contiguous(), "x and origin must be contiguous float32 [T, H]")
        tokens, hidden = x.shape
        out = self.rows_buffer(tokens, 2 * hidden, dtype, x.device)
        _check(self.core.ts_stream_pair(_ptr(out), _ptr(x), _ptr(origin), tokens, hidden, dtype_code(dtype), self.stream()),
               "ts_stream_pair")
        return out

    # -- a state matrix per head instead of cached keys ------------------------------------------

    #: Tokens of a piece when long portions are cut up to run side by side.
    linear_state_piece = 64

    @staticmethod
    def linear_state_pieces(query_lens, piece: int) -> tuple[list[list[int]], list[list[int]]]:
        """For the requests ``0 .. len(query_lens) - 1`` at the front of a step: ``(pieces, carries)``,
        ``pieces[i] = [request, first row, rows, 0]`` cutting every request's rows into runs of at
        most ``piece``, ``carries[r] = [request, first piece, pieces, 0]``."""
        pieces: list[list[int]] = []
        carries: list[list[int]] = []
        row = 0
        for request, count in enumerate(query_lens):
            carries.append([request, len(pieces), -(-count // piece), 0])
            for first in range(0, count, piece):
                pieces.append([request, row + first, min(piece, count - first), 0])
            row += count
        return pieces, carries

    def linear_state(self, proj: torch.Tensor, a2: torch.Tensor, a2_bias: torch.Tensor, tau: float, state: torch.Tensor,
                     state_slots: torch.Tensor, query_start_loc: torch.Tensor, *, tokens: int, first_seq: int,
                     num_seqs: int, heads: int, head_dim: int, value_dim: int, dtype: torch.dtype,
                     out: torch.Tensor, plan: tuple | None = None) -> None:
        """The recurrence ``S <- diag(a_t) S + k_t v_t^T``, ``o_t = S^T q_t`` of a gated-linear-attention
        layer over the fused projection ``[T, 2 H D + 2 H Dv + R]`` (q, k, v, output gate, the decay's
        low-rank input ``y``), for the requests ``first_seq .. first_seq + num_seqs - 1`` of the step:
        ``a_t = sigmoid(a2 y_t + a2_bias)^(1 / tau)`` per key channel, ``q`` scaled by ``D^-0.5``, all
        in 32-bit; ``state [slots, H, D, Dv]`` 32-bit is read at the requests' ``state_slots`` and left
        updated; ``o`` goes to the requests' rows of ``out [T, H Dv]`` 32-bit.  Without a ``plan`` each
        request is walked whole; ``plan = (pieces, carries, n_pieces, n_requests)`` (int32 device
        tensors from :meth:`linear_state_pieces`, for the requests from 0 on) cuts them into pieces
        that run side by side."""
        _gpu(proj, a2, a2_bias, state, state_slots, query_start_loc, out)
        _i32(state_slots, "state_slots")
        _i32(query_start_loc, "query_start_loc")
        low = a2.shape[1]
        width = 2 * heads * head_dim + 2 * heads * value_dim + low
        is_f32, splits, stride = self._partials(proj, tokens, width, dtype, "projection")
        _need(a2.shape == (heads * head_dim, low) and a2.dtype == dtype and a2.is_contiguous()
              and a2_bias.shape == (heads * head_dim,) and a2_bias.dtype == dtype and a2_bias.is_contiguous(),
              "a2 [H D, R] and its bias [H D] of the run dtype")
        _need(head_dim <= 256 and low <= 128, "up to 256 key channels a head and a decay input of up to 128")
        _need(state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (heads, head_dim, value_dim),
              "state must be contiguous float32 [slots, H, D, Dv]")
        _need(out.dtype == torch.float32 and out.is_contiguous() and out.shape == (tokens, heads * value_dim),
              "out must be contiguous float32 [T, H Dv]")
        _need(query_start_loc.numel() >= first_seq + num_seqs + 1 and state_slots.numel() >= first_seq + num_seqs,
              "the step's row ranges and state slots do not cover the requests")
        code = dtype_code(dtype)

        def scan(mode: int, items: int, pieces, piece_state, piece_decay) -> None:
            _check(self.core.ts_linear_state_scan(
                _ptr(out), _ptr(proj), is_f32, splits, stride, _ptr(a2), _ptr(a2_bias), float(tau), _ptr(state),
                _ptr(state_slots), _ptr(query_start_loc), first_seq, _ptr(pieces), _ptr(piece_state), _ptr(piece_decay),
                items, heads, head_dim, value_dim, low, mode, code, self.stream()), "ts_linear_state_scan")

        if plan is None:
            scan(0, num_seqs, None, None, None)
            return
        pieces, carries, n_pieces, n_requests = plan
        _need(first_seq == 0 and n_requests == num_seqs, "a plan of pieces covers the requests from the first on")
        _i32(pieces, "pieces")
        _i32(carries, "carries")
        piece_state = torch.empty((n_pieces, heads, head_dim, value_dim), dtype=torch.float32, device=proj.device)
        piece_decay = torch.empty((n_pieces, heads, head_dim), dtype=torch.float32, device=proj.device)
        scan(1, n_pieces, pieces, piece_state, piece_decay)
        _check(self.core.ts_linear_state_carry(_ptr(state), _ptr(state_slots), _ptr(carries), _ptr(piece_state),
                                               _ptr(piece_decay), n_requests, heads, head_dim, value_dim, self.stream()),
               "ts_linear_state_carry")
        scan(2, n_pieces, pieces, piece_state, piece_decay)

    def linear_state_finish(self, o: torch.Tensor, proj: torch.Tensor, gain: torch.Tensor, eps: float, *, heads: int,
                            head_dim: int, value_dim: int, low: int, dtype: torch.dtype) -> torch.Tensor:
        """``[T, H Dv]`` of ``dtype``: every head's ``o`` divided by its root mean square (``eps``
        inside the root), times ``gain [Dv]``, times ``silu`` of the head's output gate, which lies in
        the projection's rows (see :meth:`linear_state`)."""
        _gpu(o, proj, gain)
        tokens = o.shape[0]
        width = 2 * heads * head_dim + 2 * heads * value_dim + low
        is_f32, splits, stride = self._partials(proj, tokens, width, dtype, "projection")
        _need(o.dtype == torch.float32 and o.is_contiguous() and o.shape == (tokens, heads * value_dim), "o must be float32 [T, H Dv]")
        _need(gain.shape == (value_dim,) and gain.dtype == dtype and gain.is_contiguous(), "gain must be [Dv] of the run dtype")
        y = self.rows_buffer(tokens, heads * value_dim, dtype, o.device)
        _check(self.core.ts_linear_state_finish(_ptr(y), _ptr(o), _ptr(proj), is_f32, splits, stride, _ptr(gain), float(eps),
                                                tokens, heads, head_dim, value_dim, low, dtype_code(dtype), self.stream()),
               "ts_linear_state_finish")
        return y

    def scaled_pair(self, a: torch.Tensor, a_scale: float, b: torch.Tensor, b_scale: float, dtype: torch.dtype) -> torch.Tensor:
        """``a_scale * a + b_scale * b`` in 32-bit as one partial sum ``[1, T, H]``: two parts' outputs (each
        ``[T, H]`` of the run dtype or ``[S, T, H]`` 32-bit partial sums) as one addend of the residual stream."""
        _gpu(a, b)
        tokens, hidden = a.shape[-2], a.shape[-1]
        a_f32, a_splits, a_stride = self._partials(a, tokens, hidden, dtype, "the first output")
        b_f32, b_splits, b_stride = self._partials(b, tokens, hidden, dtype, "the second output")
        out = torch.empty((1, tokens, hidden), dtype=torch.float32, device=a.device)
        _check(self.core.ts_scaled_pair(_ptr(out), _ptr(a), a_f32, a_splits, a_stride, float(a_scale), _ptr(b), b_f32, b_splits,
                                        b_stride, float(b_scale), tokens * hidden, dtype_code(dtype), self.stream()), "ts_scaled_pair")
        return out

    def add_tanh_norm(self, residual: torch.Tensor, pending: torch.Tensor | None, weight: torch.Tensor, bias: torch.Tensor,
                      alpha: float, rows: torch.Tensor | None = None, *, also: torch.Tensor | None = None) -> torch.Tensor:
        """``residual += pending (+ also)`` in 32-bit (in place) and ``tanh(alpha s) * weight + bias`` of the sum
        ``s`` in ``weight``'s dtype, rounded once; with ``rows`` only those rows, and ``residual`` is left alone.
        ``pending`` is ``[T, H]`` of the run dtype or ``[S, T, H]`` 32-bit partial sums, ``also`` partial sums."""
        _gpu(residual, pending, weight, bias, rows, also)
        _i32(rows, "rows")
        _need(residual.dim() == 2 and residual.dtype == torch.float32 and residual.is_contiguous(),
              "residual must be contiguous float32 [T, H]")
        tokens, hidden = residual.shape
        _need(weight.shape == (hidden,) and weight.is_contiguous() and bias.shape == (hidden,) and bias.is_contiguous()
              and bias.dtype == weight.dtype, "weight and bias must be [H] of one dtype")
        is_f32, splits, stride = (0, 1, 0)
        if pending is not None:
            is_f32, splits, stride = self._partials(pending, tokens, hidden, weight.dtype, "pending")
        also_splits, also_stride = 0, 0
        if also is not None:
            _need(also.dim() == 3 and also.dtype == torch.float32 and also.is_contiguous() and also.shape[1:] == (tokens, hidden),
                  "a second addend must be float32 partial sums [S, T, H]")
            also_splits, also_stride = also.shape[0], tokens * hidden
        out_rows = tokens if rows is None else rows.numel()
        y = self.rows_buffer(out_rows, hidden, weight.dtype, residual.device)
        _check(self.core.ts_add_tanh_norm(_ptr(y), _ptr(residual), _ptr(pending), is_f32, splits, stride, _ptr(weight), _ptr(bias),
                                          float(alpha), _ptr(rows), out_rows, hidden, dtype_code(weight.dtype), _ptr(also),
                                          also_splits, also_stride, self.stream()), "ts_add_tanh_norm")
        return y

    def tanh_cap(self, x: torch.Tensor, cap: float) -> torch.Tensor:
        """``x <- cap * tanh(x / cap)`` in place over a contiguous 32-bit tensor."""
        _gpu(x)
        _need(x.dtype == torch.float32 and x.is_contiguous() and cap > 0.0, "a positive cap on contiguous float32 values")
        _check(self.core.ts_tanh_cap(_ptr(x), x.numel(), float(cap), self.stream()), "ts_tanh_cap")
        return x

    def short_conv(self, proj: torch.Tensor, first_col: int, taps: torch.Tensor, state: torch.Tensor, state_slots: torch.Tensor,
                   token_seq: torch.Tensor, query_start_loc: torch.Tensor, *, tokens: int, num_seqs: int, dtype: torch.dtype,
                   silu: bool = False, out_float32: bool = False) -> torch.Tensor:
        """A short causal convolution over time on the ``C`` columns of ``proj`` from ``first_col`` on (``taps [C,
        K]``: ``y_t = sum_j taps[:, j] u_(t - K + 1 + j)``), continuing every request from the ``K - 1`` inputs its
        state slot holds (``state [slots, max(K - 1, 1), C]`` 32-bit, oldest first) and leaving its last ``K - 1``
        inputs there (by a second launch; in a step whose requests all bring one token the first launch does it).
        ``proj`` is ``[T, W]`` of the run dtype or 32-bit partial sums.  Returns ``[T, C]`` of the run dtype (32-bit
        with ``out_float32``), through ``silu`` if asked."""
        _gpu(proj, taps, state, state_slots, token_seq, query_start_loc)
        _i32(state_slots, "state_slots")
        _i32(token_seq, "token_seq")
        _i32(query_start_loc, "query_start_loc")
        width = proj.shape[-1]
        is_f32, splits, stride = self._partials(proj, tokens, width, dtype, "projection")
        channels, k = taps.shape
        _need(taps.dtype == dtype and taps.is_contiguous() and 1 <= k <= 8 and 0 <= first_col and first_col + channels <= width,
              "taps must be [C, K] of the run dtype, K up to 8, over columns of the projection")
        _need(state.dtype == torch.float32 and state.is_contiguous() and state.dim() == 3
              and state.shape[1:] == (max(k - 1, 1), channels), "the state must be float32 [slots, K - 1, C]")
        _need(token_seq.numel() >= tokens and query_start_loc.numel() >= num_seqs + 1 and state_slots.numel() >= num_seqs,
              "row ranges and slots of every request")
        wide = out_float32 or dtype == torch.float32
        out = torch.empty((tokens, channels), dtype=torch.float32, device=proj.device) if wide \
            else self.rows_buffer(tokens, channels, dtype, proj.device)
        code = dtype_code(dtype)
        # Every request brings one token: the launch that convolves also moves the state on.
        single = tokens == num_seqs
        _check(self.core.ts_short_conv(_ptr(out), 1 if wide else 0, _ptr(proj), is_f32, splits, stride, width, first_col, channels,
                                       _ptr(taps), k, _ptr(state), _ptr(state_slots), _ptr(token_seq), _ptr(query_start_loc),
                                       tokens, 1 if silu else 0, 1 if single else 0, code, self.stream()), "ts_short_conv")
        if single:
            return out
        _check(self.core.ts_short_conv_carry(_ptr(state), _ptr(proj), is_f32, splits, stride, width, first_col, channels, k,
                                             _ptr(state_slots), _ptr(query_start_loc), num_seqs, code, self.stream()),
               "ts_short_conv_carry")
        return out

    def delta_rule(self, u: torch.Tensor, proj: torch.Tensor, *, beta_at: int, decay_at: int, gate_at: int, a2: torch.Tensor,
                   dt_bias: torch.Tensor, a_log: torch.Tensor, g2: torch.Tensor, gain: torch.Tensor, eps: float,
                   state: torch.Tensor, state_slots: torch.Tensor, query_start_loc: torch.Tensor, tokens: int, num_seqs: int,
                   heads: int, kv_heads: int, head_dim: int, value_dim: int, dtype: torch.dtype,
                   num_long_seqs: int = 0, scale: float = 1.0, out: tuple[torch.Tensor, int] | None = None) -> torch.Tensor:
        """The gated delta rule over a step: per head and request a 32-bit state ``S [D, Dv]`` (``state [slots, H,
        D, Dv]``) that every token decays, corrects and reads: ``S <- diag(g) S; w = beta (v - S^T k); S <- S + k
        w^T; o = S^T q``.  ``u [T, 2 G D + H Dv]`` (32-bit) holds the step's convolved ``q | k | v``; ``q`` and ``k``
        are made unit vectors per head (``q`` also times ``D^-1/2``), ``g = exp(-exp(a_log) softplus(a2 . low +
        dt_bias))`` with ``low`` the ``a2.shape[1]`` columns of ``proj`` from ``decay_at`` on, ``beta`` the sigmoid of
        the ``H`` columns from ``beta_at`` on.  Every head's ``o`` is divided by its root mean square, multiplied
        by ``gain [Dv]`` and by ``sigmoid(g2 . low')``, ``low'`` the ``g2.shape[1]`` columns from ``gate_at`` on.
        The first ``num_long_seqs`` requests (those that bring several tokens) are walked with the state spread
        thinly over many workgroups, the others with whole cache lines of the state a workgroup.  Returns ``[T, H
        Dv]`` of ``dtype``, times ``scale``; with ``out = (buffer, col0)`` written into those columns of a wider buffer,
        which is returned."""
        _gpu(u, proj, a2, dt_bias, a_log, g2, gain, state, state_slots, query_start_loc)
        _i32(state_slots, "state_slots")
        _i32(query_start_loc, "query_start_loc")
        width = proj.shape[-1]
        is_f32, splits, stride = self._partials(proj, tokens, width, dtype, "projection")
        keys, values = kv_heads * head_dim, heads * value_dim
        _need(u.dtype == torch.float32 and u.is_contiguous() and u.shape == (tokens, 2 * keys + values),
              "the convolved q | k | v must be float32 [T, 2 G D + H Dv]")
        _need(heads % kv_heads == 0 and 1 <= head_dim <= 256, "heads in equal shares of the key heads, up to 256 key channels")
        _need(a2.dim() == 2 and a2.shape[0] == heads * head_dim and 1 <= a2.shape[1] <= 256 and a2.dtype == dtype and a2.is_contiguous()
              and dt_bias.shape == (heads * head_dim,) and dt_bias.dtype == dtype and dt_bias.is_contiguous(),
              "the decay's matrix must be [H D, R] with R up to 256 and its bias [H D], of the run dtype")
        _need(g2.dim() == 2 and g2.shape[0] == values and 1 <= g2.shape[1] <= 256 and g2.dtype == dtype and g2.is_contiguous()
              and gain.shape == (value_dim,) and gain.dtype == dtype and gain.is_contiguous(),
              "the gate's matrix must be [H Dv, R] with R up to 256 and the gain [Dv], of the run dtype")
        _need(a_log.shape == (heads,) and a_log.dtype == torch.float32 and a_log.is_contiguous(), "a_log must be float32 [H]")
        _need(state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (heads, head_dim, value_dim),
              "the state must be float32 [slots, H, D, Dv]")
        device = u.device
        qn = torch.empty((tokens, keys), dtype=torch.float32, device=device)
        kn = torch.empty((tokens, keys), dtype=torch.float32, device=device)
        kq = torch.empty((tokens, kv_heads), dtype=torch.float32, device=device)
        decay = torch.empty((tokens, heads * head_dim), dtype=torch.float32, device=device)
        beta = torch.empty((tokens, heads), dtype=torch.float32, device=device)
        o = torch.empty((tokens, values), dtype=torch.float32, device=device)
        code = dtype_code(dtype)
        _check(self.core.ts_delta_prepare(_ptr(qn), _ptr(kn), _ptr(kq), _ptr(decay), _ptr(beta), _ptr(u), _ptr(proj), is_f32, splits, stride,
                                          width, beta_at, decay_at, a2.shape[1], _ptr(a2), _ptr(dt_bias), _ptr(a_log), tokens,
                                          heads, kv_heads, head_dim, value_dim, code, self.stream()), "ts_delta_prepare")
        for first, count, spread in ((0, num_long_seqs, 1), (num_long_seqs, num_seqs - num_long_seqs, 0)):
            _check(self.core.ts_delta_scan(_ptr(o), _ptr(state), _ptr(qn), _ptr(kn), _ptr(kq), _ptr(decay), _ptr(beta), _ptr(u),
                                           _ptr(state_slots), _ptr(query_start_loc), first, count, heads, kv_heads, head_dim,
                                           value_dim, spread, self.stream()), "ts_delta_scan")
        y, pointer, out_stride = self._columns_of(out, tokens, values, dtype, device)
        _check(self.core.ts_delta_finish(pointer, _ptr(o), _ptr(proj), is_f32, splits, stride, width, gate_at, g2.shape[1], _ptr(g2),
                                         _ptr(gain), float(eps), tokens, heads, value_dim, code, float(scale), out_stride,
                                         self.stream()), "ts_delta_finish")
        return y

    # -- routed feed-forward --------------------------------------------------------------------

    def moe_route(self, x: torch.Tensor, router: torch.Tensor, *, top: int, groups: int, keep: int, scale: float,
                  experts: int | None = None, softmax: bool = False, correction: torch.Tensor | None = None,
                  normalise: bool = True, mark_top: int = 2) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor | None]:
        """The router of a routed feed-forward: ``z = x router^T`` by the engine's product with a
        32-bit result, then in 32-bit ``s = sigmoid(z)`` or, with ``softmax``, the softmax over the
        ``experts`` outputs; experts are chosen by ``c = s + correction`` (``correction [experts]``
        32-bit; none: ``c = s``): they form ``groups`` equal groups of neighbours, a group's mark is
        the sum of its two largest ``c`` (``mark_top = 1``: its largest alone), only the ``keep`` best groups' experts can be taken, the
        ``top`` of them with the largest ``c`` are.  Returns ``(taken [T, top] int32, weights [T, top]
        float32, gate)``: weights are ``s / (sum of the taken s + 1e-20) * scale``, or ``s * scale``
        where ``normalise`` is off.  With ``experts`` one less than the rows of ``router``, the last
        row is a gate's vector and ``gate [T]`` the sigmoid of its product (else ``None``)."""
        _gpu(x, router, correction)
        _need(x.dim() == 2 and x.is_contiguous() and router.dim() == 2 and router.is_contiguous()
              and router.shape[1] == x.shape[1] and router.dtype == x.dtype, "x [T, H] and router [E, H] of one dtype")
        tokens = x.shape[0]
        experts = router.shape[0] if experts is None else int(experts)
        _need(router.shape[0] - experts in (0, 1), "the router holds the experts' rows and at most a gate's")
        _need(1 <= experts <= 1024 and 1 <= top <= 32 and groups >= 1 and experts % groups == 0 and 1 <= keep <= groups
              and top <= (experts // groups) * keep, "a routing rule the kernel does not take")
        if correction is not None:
            _need(correction.shape == (experts,) and correction.dtype == torch.float32 and correction.is_contiguous(),
                  "the correction must be contiguous float32 [experts]")
        z = self.linear_float32_out(x, router)
        _need(z.dtype == torch.float32 and z.stride(1) == 1, "the router's outputs must be 32-bit rows")
        taken = torch.empty((tokens, top), dtype=torch.int32, device=x.device)
        weights = torch.empty((tokens, top), dtype=torch.float32, device=x.device)
        gate = torch.empty((tokens,), dtype=torch.float32, device=x.device) if router.shape[0] > experts else None
        _check(self.core.ts_moe_select(_ptr(taken), _ptr(weights), _ptr(gate), _ptr(z), tokens, z.stride(0), experts, top,
                                       groups, keep, float(scale), 1 if softmax else 0, _ptr(correction),
                                       1 if normalise else 0, int(mark_top), self.stream()), "ts_moe_select")
        return taken, weights, gate

    def moe_pair_rows(self, rows: torch.Tensor, weight: torch.Tensor, taken: torch.Tensor | None, *, share: int,
                      rule: tuple[float, float, float] | None = None, pairs: int | None = None) -> torch.Tensor:
        """The product of every (token, taken expert) pair with its expert's matrix out of the
        stack ``weight [E, N, K]``: pair ``p`` (``taken.view(-1)[p]`` its expert) reads row ``p //
        share`` of ``rows [*, K]``.  With ``rule`` the ``N = 2 I`` rows alternate gate, up and the
        result is the gated unit, ``[P, I]`` of the run dtype; else ``[P, N]`` float32.  Without
        ``taken``, pair ``p`` of ``pairs`` is with expert ``p % E`` (a product per head over rows laid
        out head by head)."""
        _gpu(rows, weight, taken)
        _i32(taken, "taken")
        _need(taken is not None or pairs is not None, "pairs are counted from the taken experts, or given")
        pairs = taken.numel() if taken is not None else int(pairs)
        _need(weight.dim() == 3 and weight.is_contiguous() and rows.dim() == 2 and rows.is_contiguous()
              and rows.dtype == weight.dtype and rows.shape[1] == weight.shape[2], "rows [*, K] and weight [E, N, K] of one dtype")
        experts, n, k = weight.shape
        _need(share >= 1 and rows.shape[0] * share >= pairs and k <= 12288, "rows do not cover the pairs")
        if rule is not None:
            _need(n % 2 == 0, "a gated stack has an even number of rows")
            out = torch.empty((pairs, n // 2), dtype=rows.dtype, device=rows.device)
        else:
            out = torch.empty((pairs, n), dtype=torch.float32, device=rows.device)
        r = rule or (1.0, 0.0, 0.0)
        _check(self.core.ts_moe_pair_rows(_ptr(out), _ptr(rows), _ptr(weight), _ptr(taken), pairs, share, n, k, experts,
                                          0 if rule is None else 1, *glu_rule(r),
                                          dtype_code(rows.dtype), self.stream()), "ts_moe_pair_rows")
        return out

    #: From this many tokens on, a bfloat16 step's pairs are grouped by expert and go through the
    #: matrix cores (below it every pair streams its expert's matrices, which is what few tokens cost anyway).
    moe_grouped_min_tokens = 33

    def moe_grouping(self, taken: torch.Tensor | None, experts: int, dtype: torch.dtype, *widths: int,
                     pairs: int | None = None):
        """``(order, tile_first, row_first)`` for :meth:`moe_grouped_rows` where a step's pairs are
        worth grouping by expert (bfloat16, many tokens, every inner width a multiple of 8), else
        ``None``.  All on the device: the host never sees who took which expert.  Without ``taken``,
        pair ``p`` of ``pairs`` is with expert ``p % experts``."""
        _gpu(taken)
        _i32(taken, "taken")
        tokens = taken.shape[0] if taken is not None else int(pairs) // experts
        if (dtype != torch.bfloat16 or tokens < self.moe_grouped_min_tokens or experts > 1024
                or any(w % 8 != 0 for w in widths)):
            return None
        pairs = taken.numel() if taken is not None else int(pairs)
        device = taken.device if taken is not None else self.device
        order = torch.empty((pairs,), dtype=torch.int32, device=device)
        tile_first = torch.empty((experts + 1,), dtype=torch.int32, device=device)
        row_first = torch.empty((experts + 1,), dtype=torch.int32, device=device)
        _check(self.core.ts_moe_group(_ptr(order), _ptr(tile_first), _ptr(row_first), _ptr(taken), pairs, experts,
                                      self.stream()), "ts_moe_group")
        return order, tile_first, row_first

    def per_head_rows(self, rows: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
        """``[T H, N]`` float32: row ``t H + h`` of ``rows [T H, K]`` against head ``h``'s matrix of the
        stack ``weight [H, N, K]``.  The heads are the experts of a routed product that every token
        takes in turn, so the same kernels run it: head by head for few tokens, grouped through the
        matrix cores for many."""
        heads, n, k = weight.shape
        pairs = rows.shape[0]
        _need(pairs % heads == 0, "rows are laid out head by head")
        grouping = self.moe_grouping(None, heads, rows.dtype, k, pairs=pairs)
        if grouping is not None:
            return self.moe_grouped_rows(rows, weight, grouping, pairs, share=1)
        return self.moe_pair_rows(rows, weight, None, share=1, pairs=pairs)

    def moe_grouped_rows(self, rows: torch.Tensor, weight: torch.Tensor, grouping: tuple, pairs: int, *, share: int,
                         rule: tuple[float, float, float] | None = None) -> torch.Tensor:
        """What :meth:`moe_pair_rows` computes, for bfloat16 pairs grouped by expert
        (:meth:`moe_grouping`), on the matrix cores."""
        _gpu(rows, weight)
        order, tile_first, row_first = grouping
        _need(weight.dim() == 3 and weight.is_contiguous() and rows.dim() == 2 and rows.is_contiguous()
              and rows.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and rows.shape[1] == weight.shape[2],
              "rows [*, K] and weight [E, N, K] must be bfloat16")
        experts, n, k = weight.shape
        _need(k % 8 == 0 and share >= 1 and rows.shape[0] * share >= pairs and order.numel() == pairs
              and tile_first.numel() == experts + 1, "grouping and sizes do not fit")
        if rule is not None:
            _need(n % 2 == 0, "a gated stack has an even number of rows")
            out = torch.empty((pairs, n // 2), dtype=torch.bfloat16, device=rows.device)
        else:
            out = torch.empty((pairs, n), dtype=torch.float32, device=rows.device)
        r = rule or (1.0, 0.0, 0.0)
        _check(self.core.ts_moe_grouped_rows(_ptr(out), _ptr(rows), _ptr(weight), _ptr(order), _ptr(tile_first),
                                             _ptr(row_first), pairs, share, n, k, experts, 0 if rule is None else 1,
                                             *glu_rule(r), self.stream()), "ts_moe_grouped_rows")
        return out

    def moe_expert_units(self, x: torch.Tensor, gate_up: torch.Tensor, taken: torch.Tensor,
                         rule: tuple[float, float, float], grouping: tuple | None = None) -> torch.Tensor:
        """The gated units ``[T * top, I]`` of every (token, taken expert) pair: ``x [T, H]`` against
        the pair's expert's matrix of the stack ``gate_up [E, 2 I, H]`` (rows alternate gate, up)."""
        if grouping is not None:
            return self.moe_grouped_rows(x, gate_up, grouping, taken.numel(), share=taken.shape[1], rule=rule)
        return self.moe_pair_rows(x, gate_up, taken, share=taken.shape[1], rule=rule)

    def moe_expert_outputs(self, units: torch.Tensor, down: torch.Tensor, taken: torch.Tensor,
                           grouping: tuple | None = None) -> torch.Tensor:
        """``[T * top, H]`` float32: every pair's units against its expert's matrix of ``down [E, H, I]``."""
        if grouping is not None:
            return self.moe_grouped_rows(units, down, grouping, taken.numel(), share=1)
        return self.moe_pair_rows(units, down, taken, share=1)

    def moe_combine(self, pair_out: torch.Tensor, weights: torch.Tensor, extra: torch.Tensor | None = None,
                    extra_gate: torch.Tensor | None = None, dtype: torch.dtype | None = None, *,
                    taken: torch.Tensor | None = None, experts: int = 0, rows: torch.Tensor | None = None) -> torch.Tensor:
        """``[1, T, H]`` float32 (one partial sum for the residual stream): the pairs' outputs
        ``[T * top, H]`` weighted by ``weights [T, top]`` and summed per token, plus ``extra_gate [T]``
        times ``extra`` (``[T, H]`` of ``dtype`` or ``[S, T, H]`` 32-bit partial sums) where given.
        With ``taken [T, top]``, ``experts`` and ``rows [T, H]`` (the feed-forward's input), a pair
        whose index is ``>= experts`` is the identity: it contributes its token's row of ``rows``,
        and its row of ``pair_out`` is not read."""
        _gpu(pair_out, weights, extra, extra_gate, taken, rows)
        tokens, top = weights.shape
        _need(pair_out.dtype == torch.float32 and pair_out.is_contiguous() and pair_out.dim() == 2
              and pair_out.shape[0] == tokens * top and weights.dtype == torch.float32 and weights.is_contiguous(),
              "pair_out [T * top, H] and weights [T, top] must be float32")
        hidden = pair_out.shape[1]
        is_f32, splits, stride, code = 0, 1, 0, TS_F32
        if extra is not None:
            run = dtype or extra.dtype
            is_f32, splits, stride = self._partials(extra, tokens, hidden, run, "extra")
            code = dtype_code(run)
        if extra_gate is not None:
            _need(extra_gate.shape == (tokens,) and extra_gate.dtype == torch.float32, "extra_gate must be float32 [T]")
        _need((taken is None) == (rows is None), "identity pairs need both the taken experts and the input rows")
        if taken is not None:
            _i32(taken, "taken")
            _need(taken.shape == (tokens, top) and rows.shape == (tokens, hidden) and rows.is_contiguous(),
                  "taken [T, top] and rows [T, H]")
            _need(extra is None or is_f32 or rows.dtype == (dtype or extra.dtype), "rows and extra must share the run dtype")
            code = dtype_code(rows.dtype)
        out = torch.empty((1, tokens, hidden), dtype=torch.float32, device=pair_out.device)
        _check(self.core.ts_moe_combine(_ptr(out), _ptr(pair_out), _ptr(weights), _ptr(extra), is_f32, splits, stride,
                                        _ptr(extra_gate), tokens, top, hidden, code, _ptr(taken), int(experts), _ptr(rows),
                                        self.stream()), "ts_moe_combine")
        return out

    # -- attention ----------------------------------------------------------------------------

    def paged_attention_generic(
        self,
        q: torch.Tensor,
        q_stride: int,
        k_pages: torch.Tensor,
        v_pages: torch.Tensor | None,
        block_table: torch.Tensor,
        token_seq: torch.Tensor,
        positions: torch.Tensor,
        heads: int,
        scale: float,
        window: int | None,
        slopes: torch.Tensor | None = None,
        softcap: float = 0.0,
        *,
        chunk: int | None = None,
        sinks: float = 0.0,
        value_dim: int | None = None,
        sink_scores: torch.Tensor | None = None,
        distance_bias: torch.Tensor | None = None,
        keep_first: int = 0,
    ) -> torch.Tensor:
        """Attention of every token over the keys ``lo..position`` of its request (behind a window
        also over the request's first ``keep_first`` keys).  With
        ``softcap = c > 0`` a scaled score ``s`` becomes ``c * tanh(s / c)``.  Values may have a
        width of their own (value pages ``[NB, Hkv, Dv, BS]``); the result is ``[T, heads * Dv]``.

        ``q`` is the tensor whose first ``heads * D`` elements of each ``q_stride``-long row
        are the (already encoded) queries.  ``slopes [heads]`` (32-bit), if given, biases the
        score of key ``j`` for a query at position ``p`` by ``slopes[h] * (j - p)``.  ``chunk = C``:
        a query at ``p`` sees no key below ``(p // C) * C``.  ``sinks = n``: the softmax's denominator
        counts ``n`` more keys of score 0 that have no value.  ``v_pages = None`` with ``value_dim =
        Dv <= D``: a key's value is its own first ``Dv`` elements.  ``sink_scores [heads]`` (32-bit):
        the sinks' score per head instead of 0.  ``distance_bias [heads, L]`` (32-bit): the score of
        the key ``n`` positions back gets ``distance_bias[h, min(n, L - 1)]`` added."""
        _gpu(q, k_pages, v_pages, block_table, token_seq, positions)
        self._score_tables(heads, sinks, sink_scores, distance_bias)
        if slopes is not None:
            _gpu(slopes)
            _need(slopes.dtype == torch.float32 and slopes.is_contiguous() and slopes.numel() == heads,
                  "slopes must be contiguous float32 [heads]")
        _i32(block_table, "block_table")
        _i32(token_seq, "token_seq")
        _i32(positions, "positions")
        if v_pages is not None:
            _check_pages(k_pages, v_pages, q.dtype, any_value_width=True)
            value_dim = v_pages.shape[2]
        else:
            _need(k_pages.dim() == 4 and k_pages.is_contiguous() and k_pages.dtype == q.dtype,
                  "key pages must be a contiguous [NB, Hkv, BS, D] tensor of the queries' dtype")
            _need(value_dim is not None and 1 <= value_dim <= k_pages.shape[3],
                  "values inside the keys are their first value_dim elements")
        _, kv_heads, block_size, head_dim = k_pages.shape
        _need(value_dim <= ATTENTION_MAX_ROW, f"values of {value_dim} elements are wider than the kernel takes")
        _need((chunk is None or chunk >= 1) and sinks >= 0.0, "a chunk is at least one position, sinks are not negative")
        tokens = positions.numel()
        _need(q.is_contiguous() and q.numel() >= tokens * q_stride and q_stride >= heads * head_dim,
              "q does not hold [T, q_stride] rows")
        _need(block_table.dim() == 2 and token_seq.numel() == tokens, "block_table [S, MB], token_seq [T]")
        _need(1 <= kv_heads and heads % kv_heads == 0 and heads <= 65535 and 1 <= head_dim <= ATTENTION_MAX_ROW,
              f"{heads} query heads on {kv_heads} KV heads of {head_dim} elements are outside what the kernel takes")
        out = self.rows_buffer(tokens, heads * value_dim, q.dtype, q.device)
        _check(self.core.ts_paged_attention_generic(
            _ptr(out), _ptr(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
            block_table.shape[1], _ptr(token_seq), _ptr(positions), tokens, heads, kv_heads, head_dim, value_dim,
            block_size, float(scale), float(softcap), int(window or 0), _ptr(slopes) if slopes is not None else None,
            int(chunk or 0), float(sinks), _ptr(sink_scores), _ptr(distance_bias),
            0 if distance_bias is None else distance_bias.shape[1], int(keep_first), dtype_code(q.dtype), self.stream()),
            "ts_paged_attention_generic")
        return out

    @staticmethod
    def _score_tables(heads: int, sinks: float, sink_scores: torch.Tensor | None, distance_bias: torch.Tensor | None) -> None:
        if sink_scores is not None:
            _gpu(sink_scores)
            _need(sinks > 0.0 and sink_scores.dtype == torch.float32 and sink_scores.is_contiguous()
                  and sink_scores.shape == (heads,), "sink scores are float32 [heads] and go with a count of sinks")
        if distance_bias is not None:
            _gpu(distance_bias)
            _need(distance_bias.dtype == torch.float32 and distance_bias.is_contiguous() and distance_bias.dim() == 2
                  and distance_bias.shape[0] == heads and distance_bias.shape[1] >= 1, "a distance bias is float32 [heads, L]")

    @staticmethod
    def tiled_attention_supported(dtype: torch.dtype, head_dim: int, value_dim: int, block_size: int, q_stride: int,
                                  values_in_keys: bool = False) -> bool:
        """Whether :meth:`attention_tiles` takes this geometry: bfloat16, key rows of up to 384 and
        values of up to 256 elements (448 and 384 where the values lie inside the key rows), both
        multiples of 8 (16-byte accesses), pages of a multiple of 8 tokens, query rows 16 bytes apart
        or a multiple of that."""
        widest = (448, 384) if values_in_keys else (384, 256)
        return (dtype == torch.bfloat16 and head_dim % 8 == 0 and 8 <= head_dim <= widest[0] and value_dim % 8 == 0
                and 8 <= value_dim <= widest[1] and block_size % 8 == 0 and block_size & (block_size - 1) == 0 and q_stride % 8 == 0)

    @staticmethod
    def attention_tile_list(query_lens, context_lens=None, rows: int = 64, *, window: int | None = None,
                            chunk: int | None = None) -> list[list[int]]:
        """``[request, first row]`` of every tile of ``rows`` consecutive tokens of the requests
        ``0 .. len(query_lens) - 1`` at the front of a step; with the requests' ``context_lens``, the
        tiles that see the most keys (under the layer's ``window`` and ``chunk``) come first, so that
        the longest walks start first."""
        tiles, row = [], 0
        for request, count in enumerate(query_lens):
            start = 0 if context_lens is None else context_lens[request] - count
            for first in range(0, count, rows):
                lowest = start + first
                lowest = max(0 if window is None else lowest - window + 1, 0 if chunk is None else (lowest // chunk) * chunk)
                tiles.append((start + first + min(rows, count - first) - lowest, request, row + first))
            row += count
        if context_lens is not None:
            tiles.sort(key=lambda tile: -tile[0])
        return [[request, first] for _, request, first in tiles]

    def attention_tiles(self, q: torch.Tensor, q_stride: int, k_pages: torch.Tensor, v_pages: torch.Tensor | None,
                        block_table: torch.Tensor, query_start_loc: torch.Tensor, context_lens: torch.Tensor, *,
                        tokens: int, heads: int, scale: float, prefill_tiles: torch.Tensor | None, num_prefill_seqs: int,
                        num_decode_seqs: int, max_decode_context: int, window: int | None = None, chunk: int | None = None,
                        sinks: float = 0.0, slopes: torch.Tensor | None = None, softcap: float = 0.0,
                        value_dim: int | None = None, sink_scores: torch.Tensor | None = None,
                        distance_bias: torch.Tensor | None = None, keep_first: int = 0) -> torch.Tensor:
        """What :meth:`paged_attention_generic` computes, for bfloat16, on the matrix cores: the
        requests that bring several tokens (the first ``num_prefill_seqs``) in tiles of 64 tokens by
        one head (``prefill_tiles``: int32 ``[n, 2]`` from :meth:`attention_tile_list`), the
        ``num_decode_seqs`` single tokens behind them with the heads of a KV head as one tile and
        their keys (at most ``max_decode_context``, a bound the step's shape gives) shared out over
        several workgroups.  Returns ``[T, heads * Dv]``."""
        _gpu(q, k_pages, v_pages, block_table, query_start_loc, context_lens, prefill_tiles, slopes)
        self._score_tables(heads, sinks, sink_scores, distance_bias)
        tables = (_ptr(sink_scores), _ptr(distance_bias), 0 if distance_bias is None else distance_bias.shape[1], int(keep_first))
        _i32(block_table, "block_table")
        _i32(query_start_loc, "query_start_loc")
        _i32(context_lens, "context_lens")
        _i32(prefill_tiles, "prefill_tiles")
        _need(q.dtype == torch.bfloat16 and k_pages.dtype == torch.bfloat16 and k_pages.dim() == 4 and k_pages.is_contiguous(),
              "queries and key pages [NB, Hkv, BS, D] must be bfloat16")
        _, kv_heads, block_size, head_dim = k_pages.shape
        if v_pages is not None:
            _check_pages(k_pages, v_pages, q.dtype, any_value_width=True)
            value_dim = v_pages.shape[2]
        _need(value_dim is not None and (v_pages is not None or value_dim <= head_dim), "values inside the keys are their first value_dim elements")
        _need(distance_bias is None or v_pages is not None, "key rows that hold their values take no bias by distance")
        _need(self.tiled_attention_supported(q.dtype, head_dim, value_dim, block_size, q_stride, v_pages is None),
              "a geometry the tiled attention kernel does not take")
        _need(heads % kv_heads == 0 and q.is_contiguous() and q.numel() >= tokens * q_stride and q_stride >= heads * head_dim,
              "q does not hold [T, q_stride] rows of the heads")
        _need(block_table.dim() == 2 and query_start_loc.numel() >= num_prefill_seqs + num_decode_seqs + 1, "block_table [S, MB], row ranges [S + 1]")
        if slopes is not None:
            _need(slopes.dtype == torch.float32 and slopes.is_contiguous() and slopes.numel() == heads, "slopes must be float32 [heads]")
        out = self.rows_buffer(tokens, heads * value_dim, q.dtype, q.device)
        common = (_ptr(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(block_table), block_table.shape[1],
                  _ptr(query_start_loc), _ptr(context_lens))
        rule = (float(scale), float(softcap), int(window or 0), int(chunk or 0), float(sinks), _ptr(slopes))
        if num_prefill_seqs > 0:
            _need(prefill_tiles is not None and prefill_tiles.dim() == 2 and prefill_tiles.shape[1] == 2, "prefill_tiles [n, 2]")
            _check(self.core.ts_attention_tiles(_ptr(out), None, None, *common, _ptr(prefill_tiles), prefill_tiles.shape[0], 0,
                                                heads, kv_heads, head_dim, value_dim, block_size, *rule, 0, 1, *tables, self.stream()),
                   "ts_attention_tiles")
        if num_decode_seqs > 0:
            # Workgroups per (request, KV head): enough to fill the compute units (key rows of up to 128
            # elements leave room for four workgroups on each), no more than the keys have tiles of 64 (a
            # chunk or window bounds what a token sees; a window starts anywhere inside a tile).
            seen = max(1, min(max_decode_context, chunk or max_decode_context, window or max_decode_context))
            key_tiles = -(-seen // 64) + (1 if window and window < max_decode_context else 0)
            if window and window < max_decode_context:
                key_tiles += -(-int(keep_first) // 64)
            head_tiles = kv_heads * (-(-(heads // kv_heads) // 64))
            room = (4 if head_dim <= 128 else 1) * self.compute_units
            splits = max(1, min(key_tiles, -(-room // (num_decode_seqs * head_tiles)), 64))
            partial_o = partial_ml = None
            if splits > 1:
                partial_o = torch.empty((num_decode_seqs, heads, splits, value_dim), dtype=torch.float32, device=q.device)
                partial_ml = torch.empty((num_decode_seqs, heads, splits, 2), dtype=torch.float32, device=q.device)
            _check(self.core.ts_attention_tiles(_ptr(out), _ptr(partial_o), _ptr(partial_ml), *common, None, num_decode_seqs,
                                                num_prefill_seqs, heads, kv_heads, head_dim, value_dim, block_size, *rule, 1,
                                                splits, *tables, self.stream()), "ts_attention_tiles")
            if splits > 1:
                _check(self.core.ts_attention_tiles_combine(_ptr(out), _ptr(partial_o), _ptr(partial_ml), _ptr(query_start_loc),
                                                            num_decode_seqs, num_prefill_seqs, heads, value_dim, splits,
                                                            float(sinks), _ptr(sink_scores), self.stream()),
                       "ts_attention_tiles_combine")
        return out

    @staticmethod
    def mfma_attention_supported(dtype: torch.dtype, head_dim: int, block_size: int) -> bool:
        """Whether the matrix-core attention kernels take this geometry (bfloat16, head sizes
        16..256 in steps of 16, pages of at least 8 tokens); anything else runs the generic
        kernel."""
        return dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 256 and block_size >= 8

    def attention_decode(
        self,
        out: torch.Tensor,
        q: torch.Tensor,
        q_stride: int,
        k_pages: torch.Tensor,
        v_pages: torch.Tensor,
        block_table: torch.Tensor,
        query_start_loc: torch.Tensor,
        context_lens: torch.Tensor,
        seq_begin: int,
        requests: int,
        heads: int,
        scale: float,
        window: int | None,
        max_context: int,
        max_context_dev: torch.Tensor | None = None,
        softcap: float = 0.0,
    ) -> None:
        """Matrix-core attention for the single-token requests ``seq_begin .. seq_begin +
        requests - 1`` of the step; writes their rows of ``out [T, heads * D]``.  ``max_context``
        (host-known) bounds their context lengths and fixes the number of splits of the keys;
        ``max_context_dev`` (one int32 on the device, at most ``max_context``) is the step's
        true longest context, from which a recorded launch sizes each split."""
        _gpu(out, q, k_pages, v_pages, block_table, query_start_loc, context_lens, max_context_dev)
        _i32(max_context_dev, "max_context_dev")
        _i32(block_table, "block_table")
        _i32(query_start_loc, "query_start_loc")
        _i32(context_lens, "context_lens")
        _check_pages(k_pages, v_pages, torch.bfloat16)
        _, kv_heads, block_size, head_dim = k_pages.shape
        _need(self.mfma_attention_supported(q.dtype, head_dim, block_size), "geometry not taken by the matrix-core kernels")
        _need(out.dtype == torch.bfloat16 and out.is_contiguous() and out.shape[1] == heads * head_dim,
              "out must be contiguous bfloat16 [T, heads * D]")
        _need(q.is_contiguous() and q_stride >= heads * head_dim, "q does not hold [T, q_stride] rows")
        _need(heads % kv_heads == 0 and block_table.dim() == 2, "heads / block table do not fit")
        _need(seq_begin >= 0 and seq_begin + requests <= context_lens.numel() and requests <= block_table.shape[0],
              "request range outside the step")
        _need(max_context <= block_table.shape[1] * block_size, "block table does not cover the context")
        span = max_context if not window else min(max_context, window + 31)
        head_tiles = -(-(heads // kv_heads) // 16)
        pairs = requests * kv_heads * head_tiles
        waves = self.decode_waves_few_pairs if 2 * pairs <= self.compute_units else self.decode_waves_many_pairs
        splits = max(1, min(-(-waves // pairs), -(-span // self.decode_min_keys), 256))
        keys_per_split = -(-(-(-(span + 31) // splits)) // 32) * 32
        splits = -(-(span + 31) // keys_per_split)
        partial_acc = torch.empty((requests * heads * splits, head_dim), dtype=torch.float32, device=q.device)
        partial_ml = torch.empty((requests * heads * splits, 2), dtype=torch.float32, device=q.device)
        lib = load_module(build.attention_module(head_dim))
        fn = getattr(lib, f"ts_attention_decode_d{head_dim}")
        _check(fn(_ptr(out), _ptr(partial_acc), _ptr(partial_ml), _ptr(q), q_stride, _ptr(k_pages), _ptr(v_pages),
                  _ptr(block_table), block_table.shape[1], _ptr(query_start_loc), _ptr(context_lens), seq_begin,
                  requests, heads, kv_heads, block_size, float(scale), float(softcap), int(window or 0), keys_per_split, splits,
                  _ptr(max_context_dev), self.stream()), "ts_attention_decode")

    def prefill_block_rows(self, head_dim: int, heads: int, kv_heads: int) -> int:
        """Consecutive rows of one request that a wavefront of the prefill attention kernel
        handles for this geometry (16 or 32): the length of the blocks its work list is made of."""
        lib = load_module(build.attention_module(head_dim))
        return int(getattr(lib, f"ts_attention_prefill_rows_d{head_dim}")(heads, kv_heads))

    #: Fewest windows of 32 keys worth a workgroup of their own when a block's keys are shared out,
    #: and what putting the shares together costs, in windows (see :func:`prefill_share_list`).
    prefill_share_min_windows = 16
    prefill_share_combine_cost = 20

    def prefill_blocks(self, query_lens, context_lens, rows: int, *, heads: int = 0, kv_heads: int = 0,
                       head_dim: int = 0, block_size: int = 0, window: int | None = None) -> PrefillWork:
        """The work list of :meth:`attention_prefill` for the multi-token requests at the front
        of a step (their numbers of new tokens and their contexts after the step): (request
        index, first row) of every block of ``rows`` rows (:meth:`prefill_block_rows`), those
        that see the most keys first, so the long ones start early and the short ones fill the
        tail of the launch.  Given the geometry (and the layer's window), the keys of long
        blocks are shared out over several workgroups where whole blocks would leave compute
        units idle (:func:`prefill_share_list`): a short portion at the end of a long context."""
        ranges, combine = [], []
        if heads and kv_heads and head_dim and block_size and rows == PREFILL_WINDOW_KEYS:
            per_block, per_unit = c_int(0), c_int(0)
            lib = load_module(build.attention_module(head_dim))
            getattr(lib, f"ts_attention_prefill_shape_d{head_dim}")(heads, kv_heads, block_size, ctypes.byref(per_block),
                                                                   ctypes.byref(per_unit))
            blocks, ranges, combine = prefill_share_list(
                query_lens, context_lens, rows, int(window or 0), per_block.value, per_unit.value * self.compute_units,
                self.prefill_share_min_windows, combine_cost=self.prefill_share_combine_cost)
        else:
            blocks = prefill_block_list(query_lens, context_lens, rows)
        work = PrefillWork(torch.tensor(blocks, dtype=torch.int32).view(-1, 2).to(self.device))
        if ranges:
            work.ranges = torch.tensor(ranges, dtype=torch.int32).view(-1, 3).to(self.device)
            work.combine = torch.tensor(combine, dtype=torch.int32).view(-1, 4).to(self.device)
            work.slots = sum(entry[3] for entry in combine)
        return work

    def attention_prefill(
        self,
        out: torch.Tensor,
        q: torch.Tensor,
        q_stride: int,
        k_pages: torch.Tensor,
        v_pages: torch.Tensor,
        block_table: torch.Tensor,
        query_start_loc: torch.Tensor,
        context_lens: torch.Tensor,
        blocks: "torch.Tensor | PrefillWork",
        heads: int,
        scale: float,
        window: int | None,
        max_context: int,
        block_rows: int = 16,
        softcap: float = 0.0,
    ) -> None:
        """Matrix-core attention for blocks of ``block_rows`` consecutive rows of multi-token
        requests (what :meth:`prefill_block_rows` says for the geometry): ``blocks`` is the work
        list of :meth:`prefill_blocks` (made for this ``window``), or ``[n, 2]`` (request index,
        first row) of whole blocks; writes those rows of ``out [T, heads * D]``."""
        work = blocks if isinstance(blocks, PrefillWork) else PrefillWork(blocks)
        blocks = work.blocks
        _gpu(out, q, k_pages, v_pages, block_table, query_start_loc, context_lens, blocks, work.ranges, work.combine)
        _i32(block_table, "block_table")
        _i32(query_start_loc, "query_start_loc")
        _i32(context_lens, "context_lens")
        _i32(blocks, "blocks")
        _i32(work.ranges, "ranges")
        _i32(work.combine, "combine")
        _check_pages(k_pages, v_pages, torch.bfloat16)
        _, kv_heads, block_size, head_dim = k_pages.shape
        _need(self.mfma_attention_supported(q.dtype, head_dim, block_size), "geometry not taken by the matrix-core kernels")
        _need(out.dtype == torch.bfloat16 and out.is_contiguous() and out.shape[1] == heads * head_dim,
              "out must be contiguous bfloat16 [T, heads * D]")
        _need(q.is_contiguous() and q_stride >= heads * head_dim, "q does not hold [T, q_stride] rows")
        _need(heads % kv_heads == 0 and block_table.dim() == 2, "heads / block table do not fit")
        _need(blocks.dim() == 2 and blocks.shape[1] == 2, "blocks must be [n, 2]")
        _need(max_context <= block_table.shape[1] * block_size, "block table does not cover the context")
        _need(block_rows == self.prefill_block_rows(head_dim, heads, kv_heads),
              f"blocks of {block_rows} rows are not what the kernel for this geometry takes")
        partial_acc = partial_ml = None
        num_combine = 0
        if work.ranges is not None:
            _need(block_rows == PREFILL_WINDOW_KEYS, "only blocks of 32 rows are shared out")
            _need(tuple(work.ranges.shape) == (blocks.shape[0], 3), "ranges must be [n, 3] beside blocks [n, 2]")
            _need(work.combine is not None and work.combine.dim() == 2 and work.combine.shape[1] == 4 and work.slots >= 1,
                  "a work list with shares names the blocks to combine")
            num_combine = work.combine.shape[0]
            partial_acc = torch.empty((work.slots, heads, PREFILL_WINDOW_KEYS, head_dim), dtype=torch.float32, device=out.device)
            partial_ml = torch.empty((work.slots, heads, PREFILL_WINDOW_KEYS, 2), dtype=torch.float32, device=out.device)
        lib = load_module(build.attention_module(head_dim))
        fn = getattr(lib, f"ts_attention_prefill_d{head_dim}")
        _check(fn(_ptr(out), _ptr(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
                  block_table.shape[1], _ptr(query_start_loc), _ptr(context_lens), _ptr(blocks), blocks.shape[0],
                  block_rows, heads, kv_heads, block_size, float(scale), float(softcap), int(window or 0), int(max_context),
                  _ptr(work.ranges), _ptr(partial_acc), _ptr(partial_ml), _ptr(work.combine), num_combine,
                  self.stream()),
               "ts_attention_prefill")

    #: Fewest keys worth a wavefront of its own.
    decode_min_keys = 128

    # -- products -----------------------------------------------------------------------------

    def gemm_plain(
        self,
        x: torch.Tensor,
        weight: torch.Tensor,
        bias: torch.Tensor | None = None,
        *,
        out_float32: bool = False,
    ) -> torch.Tensor:
        """``x [M, K] @ weight [N, K]^T (+ bias)`` by 32-bit fused multiply-adds."""
        _gpu(x, weight, bias)
        _need(x.dim() == 2 and x.stride(1) == 1 and weight.dim() == 2 and weight.is_contiguous(),
              "x must be [M, K] with unit inner stride, weight contiguous [N, K]")
        _need(x.shape[1] == weight.shape[1] and x.dtype == weight.dtype, "x and weight disagree on K or dtype")
        m, k = x.shape
        n = weight.shape[0]
        if bias is not None:
            _need(bias.shape == (n,) and bias.dtype == x.dtype and bias.is_contiguous(), "bias must be [N]")
        out_dtype = torch.float32 if out_float32 else x.dtype
        y = torch.empty((m, n), dtype=out_dtype, device=x.device)
        _check(self.core.ts_gemm_plain(_ptr(y), _ptr(x), _ptr(weight), _ptr(bias), m, n, k,
                                       x.stride(0) if m > 1 else max(k, x.stride(0)), n,
                                       dtype_code(x.dtype), 1 if out_float32 else 0, self.stream()),
               "ts_gemm_plain")
        return y

    #: Most ranges of K the resident product is split into (its consumer adds them up).
    skinny_max_splits = 8
    #: Largest batch the weight-streaming products serve; above it the BLAS library is used.
    skinny_max_rows = 128
    #: Most rows the resident product takes (a split's activations stay in LDS).
    skinny_resident_rows = 16
    #: Wavefronts per workgroup of the resident variant (4 or 8); 0 chooses by the grid's size.
    skinny_resident_wg = 0
    #: Whether the resident product reads its weights with non-temporal loads.
    skinny_resident_once = False
    #: Chunks of 256 staged in LDS at a time for up to 8 rows and for up to 16 rows (even numbers).
    skinny_stage_chunks = (10, 4)

    @staticmethod
    def skinny_supported(x: torch.Tensor, weight: torch.Tensor) -> bool:
        """bfloat16, at most 128 rows, K a multiple of 8."""
        return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.shape[0] <= 128
                and x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0)

    @staticmethod
    def skinny_supported_any_rows(x: torch.Tensor, weight: torch.Tensor) -> bool:
        """bfloat16 and K a multiple of 8: what this engine's matrix-core products take, whatever the rows."""
        return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.shape[1] % 8 == 0
                and x.stride(0) % 8 == 0 and x.stride(1) == 1 and weight.is_contiguous())

    def _resident_plan(self, m: int, n: int, chunks: int, max_splits: int | None) -> tuple[int, int, int, int]:
        """(chunks per split, splits, wavefronts per workgroup, chunks staged at a time) of the
        skinny product with resident activations: splits sized for a number of wavefronts."""
        limit = min(chunks, max_splits or self.skinny_max_splits)
        want = max(1, min(limit, -(-self.skinny_resident_waves // -(-n // 16))))
        per_split = -(-chunks // want)
        splits = -(-chunks // per_split)
        waves = self.skinny_resident_wg or (8 if (splits == limit or -(-n // 128) * splits >= 4 * self.compute_units) else 4)
        return per_split, splits, waves, self.skinny_stage_chunks[0 if m <= 8 else 1]

    #: Matrices smaller than this many bytes stay with the resident kernel up to 16 rows: the product
    #: lasts a few microseconds and the resident kernel's many small workgroups start faster.
    resident_small_bytes = 64 << 20

    def _tiled_plan(self, m: int, n: int, k: int, max_splits: int | None) -> tuple[int, int, int]:
        """(iterations of 128 per split, splits, tile) of the tiled product: the cheapest by
        :meth:`_tiled_cost`."""
        key = (m, n, k, max_splits)
        known = self._tiled_plans.get(key)
        if known is not None:
            return known
        iters = -(-k // 128)
        limit = min(iters, max_splits or 32)
        best = None
        for tile in (8, 5, 4, 2):
            # Tiles of 256 weight rows leave LDS for 32 activation rows, and pay where one range
            # of K as one round of them replaces nearly two rounds of smaller tiles; in grids of
            # several rounds or ranges they measured slower than the others.
            if tile == 8 and (m > 32 or -(-n // 256) > self.compute_units):
                continue
            for want in range(1, (1 if tile == 8 else limit) + 1):
                per_split = -(-iters // want)
                splits = -(-iters // per_split)
                if splits != want:
                    continue  # the same grid as a smaller `want`
                cost = self._tiled_cost(m, n, k, per_split, splits, tile)
                if best is None or cost < best[0] * 0.999:
                    best = (cost, per_split, splits, tile)
        self._tiled_plans[key] = (best[1], best[2], best[3])
        return self._tiled_plans[key]

    def _tiled_cost(self, m: int, n: int, k: int, per_split: int, splits: int, tile: int) -> float:
        """What a grid of the tiled product costs, in weight rows x iterations streamed by a
        compute unit one after the other.  A compute unit holds one workgroup of the larger tiles
        (their LDS fills it) or, up to 64 activation rows, two of the smallest, and streams the
        faster the more weight rows it has in flight: 64 rows (one small workgroup) count as 1,
        two small workgroups as 1.25, a tile of 128 as 1.21, of 160 as 1.27, of 256 (one range of
        K in one round only) as 1.26 (the 72B shape's gate|up, 59,136 rows by 8,192, at eight rows:
        231 tiles of 256 rows 152 us, 462 of 128 169 us, 924 of 64 211 us; the 32B shape's, 55,296
        by 5,120: 216 of 256 93 us, 432 of 128 90 us).  With more than 32
        distinct activation rows two workgroups on a unit get in each other's way (at 64 rows the
        pair is slower than one after the other).  Workgroups beyond what the device holds at
        once wait for a later round, which starts on a busy device, unevenly.  Every workgroup
        pays one more iteration for starting up; partial sums are written here and read by the
        consumer.  Fitted to steps of the 7B and 14B shapes at 8, 32 and 64 rows, measured
        through the engine with each product's grid varied in turn, and to kernel traces of them;
        the 32B shape's widest matrix added the rule for a later round that is not full."""
        rows = 32 * tile
        units = self.compute_units
        workgroups = -(-n // rows) * splits
        stretch = rows * (per_split + 1)
        pairs = tile == 2 and m <= 64  # else the activation rows' LDS leaves room for one workgroup
        pair_extra = 0.6 if m <= 32 else 0.6 + 0.6 * (m - 32) / 32  # a pair costs 1 + this of a single one

        def round_cost(count: int) -> float:
            if tile == 2:
                doubled = max(0, count - units) / units if pairs else 0.0  # share of the units that hold two
                return stretch * (1.0 + pair_extra * doubled)
            return stretch / {4: 1.21, 5: 1.27, 8: 1.26}[tile]

        held = units * (2 if pairs else 1)
        full, rest = divmod(workgroups, held)
        cost = full * round_cost(held) + (round_cost(rest) if rest else 0.0)
        if tile != 2 and full >= 1 and rest:
            # A later round of the larger tiles that does not fill the device: its workgroups share
            # the memory among fewer and finish sooner, down to about 0.7 of the units busy, which
            # is what it takes to saturate the memory (the 32B shape's gate|up, 432 tiles of 128
            # rows: 90 us at eight rows, as if it were 1.7 rounds; 346 tiles of 160: 112 us).
            cost = full * round_cost(held) + round_cost(rest) * max(rest / held, 0.7)
        rounds = full + (1 if rest else 0)
        cost *= 1.0 + 0.1 * (rounds - 1)
        cost *= 1.0 + 3.0 * splits * m / k
        return cost

    def gemm_tiled(self, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
                   *, max_splits: int | None = None, plan: tuple[int, int, int] | None = None,
                   gated: bool = False, rule: tuple[float, float, float] = (1.0, 0.0, 0.0)) -> torch.Tensor:
        """``[S, M, N]`` 32-bit partial sums of ``x [M, K] @ weight [N, K]^T`` over ``S`` ranges of
        K (bias in the first) by the LDS-tiled kernel: M up to 128, K a multiple of 8.  ``plan``
        overrides the grid (iterations per split, splits, tile) for measurements.  ``gated``:
        the weight is a gate|up projection whose rows alternate gate, up, and the result is
        ``silu(gate) * up`` as bfloat16 ``[M, N / 2]`` (one range of K only)."""
        _gpu(x, weight, bias)
        _need(x.dim() == 2 and x.stride(1) == 1 and weight.dim() == 2 and weight.is_contiguous()
              and x.shape[1] == weight.shape[1], "x must be [M, K] with unit inner stride, weight contiguous [N, K]")
        _need(self.skinny_supported(x, weight), "the tiled product takes bfloat16, M <= 128 and K % 8 == 0")
        m, k = x.shape
        n = weight.shape[0]
        if bias is not None:
            _need(bias.shape == (n,) and bias.dtype == torch.bfloat16 and bias.is_contiguous(), "bias must be bfloat16 [N]")
        per_split, splits, tile = plan or self._tiled_plan(m, n, k, max_splits)
        x_stride = x.stride(0) if m > 1 else max(k, x.stride(0))
        if gated:
            _need(splits == 1 and bias is None and n % 2 == 0,
                  "the gated result needs one range of K, no bias and an even number of weight rows")
            out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
            _check(self.core.ts_gemm_tiled(None, _ptr(out), _ptr(x), x_stride, _ptr(weight), None, m, n, k,
                                           per_split, splits, tile, *glu_rule(rule), self.stream()),
                   "ts_gemm_tiled")
            return out
        partial = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
        _check(self.core.ts_gemm_tiled(_ptr(partial), None, _ptr(x), x_stride, _ptr(weight), _ptr(bias), m, n, k,
                                       per_split, splits, tile, *glu_rule(rule), self.stream()),
                   "ts_gemm_tiled")
        return partial

    #: Up to this many rows a product that was not timed against the BLAS library runs this
    #: engine's own kernel (more than ``skinny_max_rows``: ``gemm_wide``).  At the 7B shape the own
    #: kernel is the faster one up to about a thousand rows (down projection at 256 / 512 rows: 47 /
    #: 75 us against the library's best 75 / 116; gate|up with its SwiGLU 78 / 149 against 89 / 151),
    #: the library above (2,048 rows: gate|up 516 against 402 + 44 us, down 270 against 241).
    wide_default_rows = 640

    def _wide_plan(self, m: int, n: int, k: int, one_range: bool) -> tuple[int, int, int, int, int]:
        """(iterations of 64 per range of K, ranges, tile, activation rows, wavefronts) of the wide
        product for ``m`` rows: the cheapest grid by a small model of what a compute unit does.
        A workgroup's time is its iterations times its tile's area over how well that tile feeds
        the matrix cores (measured at 2,048 rows: tiles of 256 x 256, 160 x 256, 128 x 256,
        160 x 128 and 128 x 128 reach 1.06, 0.92, 0.87, 0.75 and 0.72 PFLOP/s) plus a start; the
        workgroups run in rounds of one per compute unit; partial sums of several ranges of K
        are written here and read by the consumer.  ``one_range``: the consumer wants one
        bfloat16 result."""
        key = (m, n, k, one_range)
        known = self._wide_plans.get(key)
        if known is not None:
            return known
        iters = -(-k // 64)
        units = self.compute_units
        unit_flops_per_us = 2.5e9 / units  # a compute unit's share of the matrix peak (2.5 PFLOP/s), per microsecond
        best = None
        for tile, x_rows, rate in ((8, 256, 1.06), (5, 256, 0.92), (4, 256, 0.87), (5, 128, 0.75), (4, 128, 0.72)):
            if x_rows == 256 and m <= 128:
                continue
            per_iteration = 2.0 * 32 * tile * x_rows * 64 / (rate / 2.5 * unit_flops_per_us)  # microseconds
            for want in range(1, (1 if one_range else min(iters, 24)) + 1):
                per_split = -(-iters // want)
                splits = -(-iters // per_split)
                if splits != want:
                    continue
                workgroups = -(-n // (32 * tile)) * -(-m // x_rows) * splits
                rounds = -(-workgroups // units)
                cost = rounds * (per_split + 3) * per_iteration
                if splits > 1:
                    cost += 2.0 * splits * m * n * 4 / 4e6  # the partial sums' way through memory, 4 TB/s
                if best is None or cost < best[0]:
                    best = (cost, per_split, splits, tile, x_rows, 8)
        self._wide_plans[key] = best[1:]
        return best[1:]

    def _wide_runs(self, rows: int, n: int, k: int, kind: str, plan, own, library) -> bool:
        """Whether this engine's own product (with the grid ``plan``), not the BLAS library's, runs
        a product of ``rows`` rows (more than the decode products take): what a timing found, or,
        untimed, up to ``wide_default_rows`` rows if the grid gives at least half of the compute
        units a workgroup.  With ``time_wide_choices`` an unknown product that is worth timing
        runs both ways here (``own()`` and ``library()``), four launches each behind a warm-up, each
        waited for, the best by device events that see the device's time alone."""
        key = (self.library_rows(rows), n, k, kind)
        known = self.wide_choices.get(key)
        if known is not None:
            return known
        if not self.time_wide_choices or rows * n * k < self.library_tuning_min_work:
            workgroups = -(-n // (32 * plan[2])) * -(-rows // plan[3]) * plan[1]
            return rows <= self.wide_default_rows and (2 * workgroups >= self.compute_units or rows * n * k < self.library_tuning_min_work)
        # One launch at a time, each waited for: launches that follow one another without a
        # dependency overlap where a grid leaves compute units idle, and would look faster than
        # they are inside a step.  Each timed launch follows a kernel that keeps the device busy
        # for longer than the host needs to issue it (reading 512 MB: some 80 us; reading, because
        # a kernel that writes leaves the caches full of lines that go back to memory under the
        # product), so that the events see the device's time alone: the host's own time per
        # launch differs between a library call and this engine's (by more than a short
        # product lasts) and is hidden inside a step, where the host runs ahead.
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        busy = torch.empty(1 << 27, dtype=torch.int32, device=self.device)
        chunk = 16 * 4 * 256  # bytes a workgroup of the read-only kernel takes per iteration
        count = busy.numel() * 4 // (1024 * chunk)
        times = []
        for run in (own, library):
            run()
            run()
            best = float("inf")
            for _ in range(4):
                torch.cuda.synchronize(self.device)
                self.hbm_read(busy, workgroups=1024, iters=count, pieces=4, ahead=2, wg_stride=count * chunk,
                              it_stride=chunk, blk_rows=64, blk_stride=0, row_stride=256)
                start.record()
                run()
                stop.record()
                stop.synchronize()
                best = min(best, start.elapsed_time(stop))
            times.append(best)
        del busy
        self.wide_choices[key] = times[0] <= times[1]
        self.wide_timings[key] = (times[0], times[1])
        return self.wide_choices[key]

    def gemm_wide(self, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None, *,
                  plan: tuple[int, int, int, int, int], gated: bool = False, sums: bool = False,
                  rule: tuple[float, float, float] = (1.0, 0.0, 0.0)) -> torch.Tensor:
        """``x [M, K] @ weight [N, K]^T (+ bias)`` by the LDS-tiled kernel for steps of many rows
        (``csrc/gemm_wide.hip``): any M, K a multiple of 8.  ``plan`` = (iterations per range
        of K, ranges, tile, activation rows a workgroup, wavefronts a workgroup[, k per iteration: 64 (the default) or 128]).  One range: bfloat16 ``[M, N]``; several
        (or, with ``sums``, one as well): 32-bit partial sums ``[S, M, N]`` (bias in the first).  ``gated``: the weight is a gate|up
        projection whose rows alternate gate, up, and the result is ``silu(gate) * up`` as
        bfloat16 ``[M, N / 2]`` (one range of K, no bias)."""
        _gpu(x, weight, bias)
        _need(x.dim() == 2 and x.stride(1) == 1 and weight.dim() == 2 and weight.is_contiguous()
              and x.shape[1] == weight.shape[1], "x must be [M, K] with unit inner stride, weight contiguous [N, K]")
        _need(x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0,
              "the wide product takes bfloat16 and K % 8 == 0")
        m, k = x.shape
        n = weight.shape[0]
        if bias is not None:
            _need(bias.shape == (n,) and bias.dtype == torch.bfloat16 and bias.is_contiguous(), "bias must be bfloat16 [N]")
        per_split, splits, tile, x_rows, waves = plan[:5]
        depth = plan[5] if len(plan) > 5 else 64
        x_stride = x.stride(0) if m > 1 else max(k, x.stride(0))
        if gated:
            _need(splits == 1 and bias is None and n % 2 == 0,
                  "the gated result needs one range of K, no bias and an even number of weight rows")
            out = self.rows_buffer(m, n // 2, torch.bfloat16, x.device)
            _check(self.core.ts_gemm_wide(None, _ptr(out), _ptr(x), x_stride, _ptr(weight), None, m, n, k, per_split, splits,
                                          tile, x_rows, waves, depth, 2, *glu_rule(rule),
                                          self.stream()), "ts_gemm_wide")
            return out
        if splits == 1 and not sums:
            out = self.rows_buffer(m, n, torch.bfloat16, x.device)
            _check(self.core.ts_gemm_wide(None, _ptr(out), _ptr(x), x_stride, _ptr(weight), _ptr(bias), m, n, k, per_split,
                                          splits, tile, x_rows, waves, depth, 0, 1.0, 0.0, 0.0, 0.0, self.stream()), "ts_gemm_wide")
            return out
        partial = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
        _check(self.core.ts_gemm_wide(_ptr(partial), None, _ptr(x), x_stride, _ptr(weight), _ptr(bias), m, n, k, per_split,
                                      splits, tile, x_rows, waves, depth, 1, 1.0, 0.0, 0.0, 0.0, self.stream()), "ts_gemm_wide")
        return partial

    def gemm_resident(self, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
                      *, max_splits: int | None = None) -> torch.Tensor:
        """The same partial sums by the kernel that keeps a split's activations resident in LDS and
        streams the weights through registers: M up to 16."""
        _gpu(x, weight, bias)
        _need(x.dim() == 2 and x.stride(1) == 1 and weight.dim() == 2 and weight.is_contiguous()
              and x.shape[1] == weight.shape[1], "x must be [M, K] with unit inner stride, weight contiguous [N, K]")
        _need(self.skinny_supported(x, weight) and x.shape[0] <= self.skinny_resident_rows,
              "the resident product takes bfloat16, M <= 16 and K % 8 == 0")
        m, k = x.shape
        n = weight.shape[0]
        if bias is not None:
            _need(bias.shape == (n,) and bias.dtype == torch.bfloat16 and bias.is_contiguous(), "bias must be bfloat16 [N]")
        x_stride = x.stride(0) if m > 1 else max(k, x.stride(0))
        per_split, splits, waves, stage = self._resident_plan(m, n, -(-k // 256), max_splits)
        partial = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
        _check(self.core.ts_gemm_skinny_resident(_ptr(partial), _ptr(x), x_stride, _ptr(weight), _ptr(bias),
                                                 m, n, k, per_split, splits, waves, stage,
                                                 1 if self.skinny_resident_once else 0, self.stream()),
               "ts_gemm_skinny_resident")
        return partial

    def gemm_skinny(self, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
                    *, max_splits: int | None = None) -> torch.Tensor:
        """``[S, M, N]`` 32-bit partial sums of ``x [M, K] @ weight [N, K]^T`` over ``S`` ranges of
        K (bias in the first); their sum over ``S`` is the product.  For decode-sized ``M``: the
        tiled kernel, except for up to 16 rows against a small matrix (the resident kernel's
        many small workgroups start faster)."""
        m, (n, k) = x.shape[0], weight.shape
        if self._resident_runs(m, n, k):
            return self.gemm_resident(x, weight, bias, max_splits=max_splits)
        if self._few_rows_wide(m, n, k, max_splits):
            return self.gemm_wide(x, weight, bias, plan=self._wide_plan_few_rows(m, n, k, max_splits), sums=True)
        return self.gemm_tiled(x, weight, bias, max_splits=max_splits)

    def _few_rows_wide(self, m: int, n: int, k: int, max_splits: int | None) -> bool:
        """Whether a decode-sized product runs the kernel of the steps of many rows
        (``gemm_wide``: eight wavefronts, an iteration's staging between the halves of the one
        before's products) instead of the tiled one: above 32 rows always (7B shape, alone, at 64
        rows: gate|up 46.7 against 50.1 us, down 27.6 against 29.3, q|k|v 10.7 against 14.4, o 9.5
        against 10.6, the head 209 against 221; at 128 rows: 59 against 72, 35 against 39, 14
        against 16, 246 against 282), from 17 rows for a matrix that runs as one range of K and
        whose best grid is at most two rounds of workgroups (gate|up at 24 to 32 rows, 7B / 14B /
        32B shape: 47.4 / 50.4 / 97.4 us against the tiled kernel's 48.7 / 51.7 / 99.9)."""
        if m > 32:
            return True
        if m <= 16 or max_splits != 1:
            return False
        tile = self._one_range_tile(n, 64)
        return 8 * self.compute_units <= 10 * -(-n // (32 * tile)) <= 20 * self.compute_units * (2 if tile == 2 else 1)

    #: Weight rows a compute unit streams per microsecond through the wide kernel at up to 128
    #: activation rows and K = 5,120, by tile (tiles of 64 rows: two workgroups a unit).  Larger
    #: tiles have more in flight and stream faster.  From the gate|up matrices of the 7B, 14B, 32B
    #: and 72B shapes at 64 rows, each timed with every tile.
    _ONE_RANGE_RATES = {2: 1.7, 4: 2.04, 5: 2.28, 8: 2.62}

    def _one_range_tile(self, n: int, x_rows: int) -> int:
        """The tile (in 32 weight rows) with which the wide kernel streams ``n`` weight rows as one
        range of K soonest: what a unit streams per round at that tile's rate, times the rounds
        of workgroups, a later round that is not full counting for what is in it but for no less
        than 0.7 (about that share of the units busy saturates the memory).  Measured against
        it at 64 rows (us, model / kernel): 7B shape, 37,888 rows: tile 5 49 / 49, tile 8 68 / 62,
        tile 4 75 / 67; 14B, 27,648: tile 4 63 / 54, 5 70 / 60, 8 98 / 99; 32B, 55,296: 8 98 / 98,
        4 107 / 106, 5 119 / 119, 2 128 / 126; 72B, 59,136 by 8,192: 8 156 / 157, 4 180 / 189, 5 191 / 196."""
        units = self.compute_units
        best = None
        for tile, rate in self._ONE_RANGE_RATES.items():
            held = units * (2 if tile == 2 else 1)
            full, rest = divmod(-(-n // (32 * tile)), held)
            rounds = 1.0 if full == 0 else full + (max(rest / held, 0.7) if rest else 0.0)
            cost = rounds * 32 * tile * (2 if tile == 2 else 1) / rate
            if best is None or cost < best[0]:
                best = (cost, tile)
        return best[1]

    def _wide_plan_few_rows(self, m: int, n: int, k: int, max_splits: int | None) -> tuple[int, int, int, int, int, int]:
        """The wide product's grid for up to 128 rows, where reading the weights sets the pace: one
        tile of 64 or 128 activation rows; as one range of K (a consumer that wants one result:
        the gated product, the head) the tile of weight rows that fills the device's rounds best
        (``_one_range_tile``), iterations 128 deep under the tiles of 64 activation rows (half as
        many barriers; the head, whose grid runs in several rounds, and tiles of 256 weight rows,
        whose LDS it would not fit, are 64 deep); else tiles of 128 and as many ranges of K as it
        takes to give every compute unit one."""
        x_rows = 64 if m <= 64 else 128
        if max_splits == 1 or 10 * -(-n // 160) >= 9 * self.compute_units:
            tile = self._one_range_tile(n, x_rows)
            depth = 128 if x_rows == 64 and tile != 8 and -(-n // 160) <= 2 * self.compute_units else 64
            return -(-k // depth), 1, tile, x_rows, 8, depth
        depth = 128 if x_rows == 64 else 64
        iters = -(-k // depth)
        want = max(1, min(iters, max_splits or iters, self.compute_units // -(-n // 128)))
        per_split = -(-iters // want)
        return per_split, -(-iters // per_split), 4, x_rows, 8, depth

    def _resident_runs(self, m: int, n: int, k: int) -> bool:
        """Whether the resident kernel, not the tiled one, runs a decode-sized product: small
        matrices up to 16 rows.  (Before the weights were read with non-temporal loads it also
        ran the widest matrices at up to eight rows; now the tiled kernel is faster there: the
        head of the 7B shape at eight rows in 173 against 189 us.)"""
        return m <= self.skinny_resident_rows and 2 * n * k < self.resident_small_bytes

    #: Row counts that steps of more rows than the decode products take are run at by the BLAS
    #: library (ascending; empty: every step at its own size).  The library's choice of kernel is
    #: only as good as its heuristic unless a shape has been timed, and a serving engine meets
    #: every row count; with a short list of sizes all of them can be timed at start-up
    #: (``LLMEngine`` sets the list when it is asked to time them).  A step runs at the next size
    #: up: its activation buffers are allocated that long (``rows_buffer``) and the rows beyond the
    #: step's own hold whatever was there; products are row by row, so nothing of it reaches a
    #: row that is read.
    library_buckets: tuple[int, ...] = ()

    @staticmethod
    def bucket_sizes(limit: int) -> tuple[int, ...]:
        """The sizes up to ``limit`` (which is one itself): multiples of 32 to 256, of 64 to 512,
        of 128 to 1,024, of 256 beyond, so that a step is at most a quarter longer than it had
        to be."""
        sizes = {limit}
        for step, end in ((32, 256), (64, 512), (128, 1024), (256, limit)):
            sizes.update(range(step, min(end, limit) + 1, step))
        return tuple(sorted(sizes))

    def library_rows(self, rows: int) -> int:
        """The row count a library product of ``rows`` rows is run at."""
        if rows <= self.skinny_max_rows:
            return rows
        for size in self.library_buckets:
            if size >= rows:
                return size
        return rows

    def rows_buffer(self, rows: int, width: int, dtype: torch.dtype, device) -> torch.Tensor:
        """``[rows, width]`` for a step's activations, with room behind it up to the size a
        library product of these rows is run at."""
        return torch.empty((self.library_rows(rows), width), dtype=dtype, device=device)[:rows]

    @staticmethod
    def _with_room(x: torch.Tensor, rows: int) -> torch.Tensor | None:
        """``x`` seen ``rows`` long, if its rows are dense and its storage reaches that far."""
        if rows == x.shape[0]:
            return x
        if x.dim() != 2 or x.stride(1) != 1 or x.stride(0) != x.shape[1]:
            return None
        needed = (x.storage_offset() + rows * x.shape[1]) * x.element_size()
        if needed > x.untyped_storage().nbytes():
            return None
        return x.as_strided((rows, x.shape[1]), (x.shape[1], 1))

    #: Products with fewer multiply-adds than this never use a timed choice of the BLAS library's
    #: kernels, only its default: timing them is noise, and the library's candidates for small,
    #: odd shapes are the ones that have misbehaved here (one for [200, 64] x [256, 64] returned
    #: garbage once in about eight processes).  The smallest product an engine times for the 7B
    #: shape, 160 rows of the output projection, has fifteen times as many.
    library_tuning_min_work = 1 << 27

    def _library_product(self, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None,
                         out_dtype: torch.dtype | None) -> torch.Tensor:
        """``x @ weight^T (+ bias)`` by the BLAS library behind torch, at the row count of
        :meth:`library_rows` when ``x`` has the room (see ``library_buckets``)."""
        rows = x.shape[0]
        roomy = self._with_room(x, self.library_rows(rows))
        if roomy is not None and roomy.shape[0] != rows:
            return self._library_product(roomy, weight, bias, out_dtype)[:rows]
        tunable = torch.cuda.tunable
        small = x.shape[0] * weight.shape[0] * weight.shape[1] < self.library_tuning_min_work
        paused = small and tunable.is_enabled()
        if paused:
            tunable.enable(False)
        try:
            if out_dtype is not None:
                return torch.mm(x, weight.t(), out_dtype=out_dtype)
            if bias is None:
                return torch.mm(x, weight.t())
            return torch.addmm(bias, x, weight.t())
        finally:
            if paused:
                tunable.enable(True)

    #: Whether a library product whose result goes into the residual stream leaves it in 32-bit.
    #: Off: the library's kernels with a 32-bit result are slower (a 2,048-token prompt of the 7B
    #: shape takes 29.1 ms against 26.2), and the exactness gained is small (140 short prompts in
    #: one step are off by 2.3% of a row's largest logit at most instead of 2.4%, the mean by
    #: 0.62% instead of 0.66%).
    library_residual_float32 = False

    def linear_swiglu(self, x: torch.Tensor, weight: torch.Tensor,
                      rule: tuple[float, float, float] | None = None) -> torch.Tensor:
        """The gated unit of the projection of ``x`` by a gate|up matrix ``[2 I, K]`` whose rows
        alternate gate, up -> ``[T, I]`` in the dtype of ``x``: ``silu(gate) * up``, or another
        unit by ``rule`` (see :meth:`swiglu`).  bfloat16 products that run as one range of K
        apply the unit in the product's own kernel; every other case is the projection followed
        by :meth:`swiglu`."""
        rule = (1.0, 0.0, 0.0) if rule is None else tuple(float(v) for v in rule)
        if x.dtype == torch.bfloat16 and self.skinny_supported(x, weight) and x.shape[0] <= self.skinny_max_rows:
            _gpu(x, weight)
            if (self._few_rows_wide(x.shape[0], weight.shape[0], weight.shape[1], 1) and weight.shape[0] % 2 == 0
                    and weight.is_contiguous() and x.stride(1) == 1):
                wide = self._wide_plan_few_rows(x.shape[0], weight.shape[0], weight.shape[1], 1)
                return self.gemm_wide(x, weight, plan=wide, gated=True, rule=rule)
            plan = self._tiled_plan(x.shape[0], weight.shape[0], weight.shape[1], None)
            if plan[1] == 1 and weight.shape[0] % 2 == 0 and weight.is_contiguous() and x.stride(1) == 1:
                return self.gemm_tiled(x, weight, plan=plan, gated=True, rule=rule)
        elif (x.dtype == torch.bfloat16 and self.skinny_supported_any_rows(x, weight) and weight.shape[0] % 2 == 0
              and weight.is_contiguous() and x.stride(1) == 1):
            _gpu(x, weight)
            m, (n, k) = x.shape[0], weight.shape
            plan = self._wide_plan(m, n, k, True)
            if self._wide_runs(m, n, k, "gated", plan, lambda: self.gemm_wide(x, weight, plan=plan, gated=True, rule=rule),
                               lambda: self.swiglu(self._library_product(x, weight, None, None), x.dtype, paired=True, rule=rule)):
                return self.gemm_wide(x, weight, plan=plan, gated=True, rule=rule)
            return self.swiglu(self._library_product(x, weight, None, None), x.dtype, paired=True, rule=rule)
        return self.swiglu(self.linear(x, weight), x.dtype, paired=True, rule=rule)

    def linear(self, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None, *,
               for_residual: bool = False) -> torch.Tensor:
        """The projection of the serving path.  32-bit runs use :meth:`gemm_plain` (no reduced
        matrix mode).  bfloat16 runs with decode-sized batches (up to ``skinny_max_rows`` rows) use
        :meth:`gemm_skinny` and return ``[S, M, N]`` 32-bit partial sums for the consumer to add
        up, or, where K is no multiple of 8 (the matrix-core kernels load 16 bytes at a time),
        :meth:`gemm_plain` on bfloat16 operands: slower, but a kernel of this engine, so a
        recorded step never holds a library call.  Larger batches use :meth:`gemm_wide` or the
        BLAS library behind torch (as the reference does for every linear layer,
        src/turboserve/engine/model/layers.py:142), whichever was the faster one when both were
        timed (``_wide_runs``).  ``for_residual``: the result is what a
        norm adds to the 32-bit residual stream, so the library leaves it in 32-bit too (as
        ``[1, M, N]``, one partial sum): the stream then gets the same unrounded addend from a
        prompt's step as from a decode step's partial sums."""
        if x.dtype == torch.float32:
            return self.gemm_plain(x, weight, bias)
        _gpu(x, weight, bias)
        if x.shape[0] <= self.skinny_max_rows:
            if self.skinny_supported(x, weight):
                return self.gemm_skinny(x, weight, bias)
            return self.gemm_plain(x, weight, bias)  # a K that 16-byte loads do not divide
        if self.skinny_supported_any_rows(x, weight):
            m, (n, k) = x.shape[0], weight.shape
            # What goes into the residual stream may stay partial sums (the norm adds them up);
            # any other consumer of a step this long wants one bfloat16 result.
            plan = self._wide_plan(m, n, k, not for_residual)
            if self._wide_runs(m, n, k, "sums" if for_residual else "one", plan,
                               lambda: self.gemm_wide(x, weight, bias, plan=plan),
                               lambda: self._library_product(x, weight, bias, None)):
                return self.gemm_wide(x, weight, bias, plan=plan)
        if for_residual and self.library_residual_float32:
            out = self._library_product(x, weight, None, torch.float32)
            if bias is not None:
                out += bias
            return out.unsqueeze(0)
        return self._library_product(x, weight, bias, None)

    def linear_float32_out(self, x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
        """``x @ weight^T`` with a 32-bit result (the head: logits are 32-bit,
        src/turboserve/engine/model/model.py:244)."""
        if x.dtype == torch.float32:
            return self.gemm_plain(x, weight)
        _gpu(x, weight)
        if x.shape[0] <= self.skinny_max_rows:
            if self.skinny_supported(x, weight):
                return self.gemm_skinny(x, weight, max_splits=1)[0]
            return self.gemm_plain(x, weight, out_float32=True)
        return self._library_product(x, weight, None, torch.float32)

    # -- measurement --------------------------------------------------------------------------

    def hbm_read(self, src: torch.Tensor, *, workgroups: int, iters: int, pieces: int, ahead: int, wg_stride: int,
                 it_stride: int, blk_rows: int, blk_stride: int, row_stride: int, non_temporal: bool = False) -> torch.Tensor:
        """Read ``src`` and nothing else, walking it as a weight-streaming product would (see
        ``csrc/probe.hip`` for the walk and the byte strides): what the memory gives that way of
        reading.  Returns one word per workgroup."""
        _gpu(src)
        _need(src.is_contiguous(), "src must be contiguous")
        out = torch.empty((workgroups,), dtype=torch.int32, device=src.device)
        _check(self.core.ts_hbm_read(_ptr(out), _ptr(src), src.numel() * src.element_size(), workgroups, iters, pieces,
                                     ahead, wg_stride, it_stride, blk_rows, blk_stride, row_stride, 1 if non_temporal else 0,
                                     self.stream()), "ts_hbm_read")
        return out

    # -- sampling -----------------------------------------------------------------------------

    def argmax(self, logits: torch.Tensor) -> torch.Tensor:
        _gpu(logits)
        _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.is_contiguous(),
              "logits must be contiguous float32 [n, V]")
        tokens = torch.empty((logits.shape[0],), dtype=torch.int32, device=logits.device)
        scratch = torch.empty((logits.shape[0], 128), dtype=torch.int32, device=logits.device)
        _check(self.core.ts_argmax(_ptr(tokens), _ptr(logits), _ptr(scratch), logits.shape[0], logits.shape[1],
                                   self.stream()), "ts_argmax")
        return tokens

    #: Most tokens the sampling kernel lists for its short way through a truncated row (the kernel
    #: holds 2,048); 0 sends every row the long way.
    sample_max_listed = 2048

    def sample(
        self,
        logits: torch.Tensor,
        temperature: torch.Tensor,
        top_k: torch.Tensor,
        top_p: torch.Tensor,
        penalty: torch.Tensor,
        seed_lo: torch.Tensor,
        seed_hi: torch.Tensor,
        draw_index: torch.Tensor,
        history: torch.Tensor,
        history_start: torch.Tensor,
        want_logprobs: bool,
        unread_tokens: torch.Tensor | None = None,
        unread_row: torch.Tensor | None = None,
    ) -> tuple[torch.Tensor, torch.Tensor | None]:
        """One token per row of ``logits [n, V]``; parameter tensors are per row (see
        ``csrc/sampling.hip``).  ``unread_tokens`` (int32, on the device) with ``unread_row [n]``
        (a place in it per row, or -1): one more token of a row's history that only the device
        knows yet.  Returns ``(tokens int32 [n], logprobs float32 [n] | None)``."""
        _gpu(logits, temperature, top_k, top_p, penalty, seed_lo, seed_hi, draw_index, history, history_start,
             unread_tokens, unread_row)
        _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.is_contiguous(),
              "logits must be contiguous float32 [n, V]")
        rows, vocab = logits.shape
        for name, t, dt in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                            ("top_p", top_p, torch.float32), ("penalty", penalty, torch.float32),
                            ("seed_lo", seed_lo, torch.int32), ("seed_hi", seed_hi, torch.int32),
                            ("draw_index", draw_index, torch.int32)):
            _need(t.shape == (rows,) and t.dtype == dt and t.is_contiguous(), f"{name} must be {dt} [n]")
        _i32(history, "history")
        _i32(history_start, "history_start")
        _need(history_start.numel() == rows + 1, "history_start must have n + 1 entries")
        _need((unread_tokens is None) == (unread_row is None), "unread_tokens and unread_row come together")
        if unread_row is not None:
            _i32(unread_tokens, "unread_tokens")
            _i32(unread_row, "unread_row")
            _need(unread_row.numel() == rows and unread_tokens.is_contiguous() and unread_row.is_contiguous(),
                  "unread_row must have n entries")
        tokens = torch.empty((rows,), dtype=torch.int32, device=logits.device)
        logprobs = torch.empty((rows,), dtype=torch.float32, device=logits.device) if want_logprobs else None
        work = torch.empty_like(logits)
        _check(self.core.ts_sample(_ptr(tokens), _ptr(logprobs), _ptr(logits), _ptr(work), rows, vocab,
                                   _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(penalty), _ptr(seed_lo),
                                   _ptr(seed_hi), _ptr(draw_index), _ptr(history), _ptr(history_start),
                                   _ptr(unread_tokens), _ptr(unread_row), int(self.sample_max_listed), self.stream()),
               "ts_sample")
        return tokens, logprobs
