"""The Python face of the kernel library's step program: a model's run order
as a list of operations that one native call issues, kernel after kernel,
instead of one call into the library per kernel (the launches of a step cost a
Python caller more time than most steps' kernels take).

Parts append themselves with `emit` methods; a part without one (a part
registered from outside, say) keeps the model on the path that calls the parts
one by one. The program owns no device memory: its scratch regions carry the
names of the workspace buffers the parts use when they run one by one, and the
engine binds those buffers to it.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, byref, c_float, c_int32, c_int64, c_void_p
from typing import Dict, List, Optional

import torch

from .library import library
from .ops import _CODES, KernelArgumentError

MAX_GROUPS = 8
SCRATCH_TOO_SMALL = 3


class LinearDesc(Structure):
    _fields_ = [("weight", c_void_p), ("bias", c_void_p), ("dtype", c_int32), ("n", c_int32), ("k", c_int32)]


class AttentionDesc(Structure):
    _fields_ = [("qkv", LinearDesc), ("out", LinearDesc), ("q_norm", c_void_p), ("k_norm", c_void_p),
                ("norm_eps", c_float), ("inv_freq", c_void_p), ("n_freq", c_int32), ("interleaved", c_int32),
                ("heads", c_int32), ("kv_heads", c_int32), ("head_dim", c_int32), ("scale", c_float),
                ("window", c_int32), ("k_cache", c_void_p), ("v_cache", c_void_p), ("n_pages", c_int32),
                ("v_transposed", c_int32), ("group", c_int32), ("owns_cache", c_int32)]


class ShortConvDesc(Structure):
    _fields_ = [("in_proj", LinearDesc), ("out_proj", LinearDesc), ("conv_weight", c_void_p), ("conv_bias", c_void_p),
                ("width", c_int32), ("taps", c_int32), ("state", c_void_p), ("n_slots", c_int32)]


class SwigluDesc(Structure):
    _fields_ = [("gate_up", LinearDesc), ("down", LinearDesc)]


class StepArgs(Structure):
    _fields_ = [("tokens", c_void_p), ("positions", c_void_p), ("row_of_token", c_void_p), ("seg_start", c_void_p),
                ("seg_len", c_void_p), ("slot", c_void_p), ("single_rows", c_void_p), ("portion_rows", c_void_p),
                ("want_rows", c_void_p), ("tables", c_void_p * MAX_GROUPS), ("n_groups", c_int32),
                ("table_width", c_int32), ("n_tokens", c_int32), ("n_rows", c_int32), ("n_want", c_int32),
                ("n_single", c_int32), ("n_portion", c_int32), ("max_seg_len", c_int32), ("max_context", c_int32),
                ("portion_tiles", c_int32)]


def _ptr(t: Optional[torch.Tensor], what: str, dtype=None) -> Optional[int]:
    if t is None:
        return None
    if t.device.type != "cuda" or not t.is_contiguous():
        raise KernelArgumentError(f"{what} must be a contiguous tensor on the GPU")
    if dtype is not None and t.dtype != dtype:
        raise KernelArgumentError(f"{what} has dtype {t.dtype}, expected {dtype}")
    return t.data_ptr()


class Program:
    """Built once per engine, after the cache's device memory exists (the
    operations hold its addresses). `sites` gives an operation its state:
    `paged[site]` the arrays by name, `fixed[site]` the slots' tensor,
    `group_of_site[site]` which block table of a step belongs to it."""

    def __init__(self, engine_dtype: torch.dtype, page_size: int, storage, group_of_site: Dict[int, int]):
        self._lib = library()
        self.engine_dtype = engine_dtype
        self.page_size = page_size
        self.storage = storage
        self.group_of_site = group_of_site
        self._h = self._lib.imparo_program_new(_CODES[engine_dtype], page_size)
        if not self._h:
            raise KernelArgumentError("the kernel library refused to make a step program")
        self._keep: List[torch.Tensor] = []          # every tensor whose address an operation holds
        n = self._lib.imparo_program_n_regions(self._h)
        self.region_names = [self._lib.imparo_program_region_name(self._h, i).decode() for i in range(n)]
        self._needs = (c_int64 * n)()
        self._logits = c_void_p()
        self.bound_version = -1                      # the workspace's version when it was last bound

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.imparo_program_delete(self._h)
            self._h = None

    def set_fold(self, mode: int) -> None:
        """Norms folded into the products around them in steps of at most 16 single tokens:
        0 never, 1 where the library's plan says it pays, 2 wherever the operations allow."""
        self._ok(self._lib.imparo_program_set_fold(self._h, int(mode)), "set_fold")

    def _ok(self, status: int, what: str) -> None:
        if status:
            raise KernelArgumentError(f"{what}: the step program refused the operation (sizes that do not fit)")

    def _hold(self, t: Optional[torch.Tensor], what: str, dtype=None) -> Optional[int]:
        if t is not None:
            self._keep.append(t)
        return _ptr(t, what, dtype)

    def linear(self, lin) -> LinearDesc:
        """The description of a parts.linear.Linear."""
        if lin.weight.dtype not in _CODES:
            raise KernelArgumentError(f"a projection weight of dtype {lin.weight.dtype}")
        return LinearDesc(self._hold(lin.weight, "projection weight"), self._hold(lin.bias, "projection bias", torch.float32),
                          _CODES[lin.weight.dtype], lin.out_features, lin.in_features)

    # ------------------------------------------------------------ operations, in run order
    def embedding(self, table: torch.Tensor, vocab: int, width: int) -> None:
        self._ok(self._lib.imparo_program_embedding(self._h, self._hold(table, "embedding table"), _CODES[table.dtype],
                                                    vocab, width), "embedding")

    def norm(self, weight: torch.Tensor, eps: float, width: int, out_dtype: torch.dtype) -> None:
        self._ok(self._lib.imparo_program_norm(self._h, self._hold(weight, "norm weight", torch.float32), float(eps),
                                               width, _CODES[out_dtype]), "norm")

    def attention(self, desc: AttentionDesc) -> None:
        self._ok(self._lib.imparo_program_attention(self._h, byref(desc)), "attention")

    def short_conv(self, desc: ShortConvDesc) -> None:
        self._ok(self._lib.imparo_program_short_conv(self._h, byref(desc)), "short conv")

    def swiglu(self, desc: SwigluDesc) -> None:
        self._ok(self._lib.imparo_program_swiglu(self._h, byref(desc)), "swiglu")

    def head(self, norm_weight: torch.Tensor, eps: float, width: int, head_linear) -> None:
        desc = self.linear(head_linear)
        self._ok(self._lib.imparo_program_head(self._h, self._hold(norm_weight, "norm weight", torch.float32), float(eps),
                                               width, byref(desc)), "head")

    # ------------------------------------------------------------ scratch
    def needs(self, args: StepArgs) -> Dict[str, int]:
        """Bytes of every region that a step of this shape uses."""
        self._ok(self._lib.imparo_program_needs(self._h, byref(args), self._needs), "needs")
        return {name: int(self._needs[i]) for i, name in enumerate(self.region_names) if self._needs[i]}

    def bind(self, workspace) -> None:
        """Binds every region to the workspace buffer of its name, as it is now."""
        for i, name in enumerate(self.region_names):
            buf = workspace.buffer(name)
            if buf is not None:
                self._ok(self._lib.imparo_program_bind(self._h, i, buf.data_ptr(), buf.numel()), f"bind {name}")
        self.bound_version = workspace.version

    # ------------------------------------------------------------ the step
    def run(self, args: StepArgs, workspace, stream: int) -> Optional[int]:
        """Issues the step's kernels on `stream`. Returns the address of the
        float32 [n_want, vocab] logits (in the workspace's "logits" buffer),
        or None when nothing is wanted. A region that is too small for the
        step grows first: nothing has been launched by then."""
        if self.bound_version != workspace.version:
            self.bind(workspace)
        status = self._lib.imparo_program_run(self._h, byref(args), byref(self._logits), stream)
        if status == SCRATCH_TOO_SMALL:
            for name, need in self.needs(args).items():
                workspace.reserve(name, need)
            self.bind(workspace)
            status = self._lib.imparo_program_run(self._h, byref(args), byref(self._logits), stream)
        if status:
            raise KernelArgumentError(f"the step program failed: {self._lib.imparo_program_error(self._h).decode()}")
        return self._logits.value
