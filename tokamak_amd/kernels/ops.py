"""Python face of the HIP kernels.

Every function checks on the host that shapes, dtypes and devices match what
the kernel and its grid assume, then launches on torch's current stream.  There
is no CPU path and no library fallback: without a GPU tensor or without the
compiled library the call raises.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_size_t, c_void_p

import torch

from tokamak_amd.kernels.build import load_library

_DT = {torch.float32: 0, torch.bfloat16: 1}


class KernelError(RuntimeError):
    pass


def _code(dtype: torch.dtype) -> int:
    try:
        return _DT[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16, not {dtype}") from None


def _p(t: torch.Tensor | None) -> c_void_p:
    if t is None:
        return c_void_p(0)
    if _recorder is not None:
        _recorder.keep.append(t)    # a replay launches on this memory again
    return c_void_p(t.data_ptr())


class LaunchRecorder:
    """The kernel launches of a stretch of host code: (library function, arguments, returned
    status) of every call that went through this module while the recorder was current, and
    the tensors whose addresses were passed.  The engine records one layer of a step and
    launches the layers of the same kind from the list, with their own weights and cache
    arrays in place of the recorded ones (engine/layer_replay.py): the checks, the choice of
    kernels and the allocations of the recorded layer hold for them too."""

    def __init__(self) -> None:
        self.calls: list[tuple] = []
        self.keep: list[torch.Tensor] = []
        self.valid = True

    def call(self, fn, args: tuple) -> int:
        status = fn(*args)
        self.calls.append((fn, args, status))
        return status


_recorder: LaunchRecorder | None = None


class recording:
    """``with recording() as rec``: launches inside the block are also listed in ``rec``."""

    def __enter__(self) -> LaunchRecorder:
        global _recorder
        self._before = _recorder
        _recorder = LaunchRecorder()
        return _recorder

    def __exit__(self, *exc):
        global _recorder
        _recorder = self._before
        return False


def slots_of(fn, args: tuple) -> list[int] | None:
    """The arguments of a recorded call as 64-bit slots (csrc/slots.h): integers and
    addresses as they are (negative ones in two's complement), a float by its bits.  None if
    the entry point has no slot form."""
    import struct

    if getattr(fn, "slots_address", None) is None or len(args) != len(fn.argtypes):
        return None
    out = []
    for kind, arg in zip(fn.argtypes, args):
        value = getattr(arg, "value", arg)
        if kind is c_float:
            out.append(struct.unpack("<I", struct.pack("<f", float(value)))[0])
        elif kind is c_void_p:
            out.append(int(value or 0))
        else:
            out.append(int(value) & 0xFFFFFFFFFFFFFFFF)
    return out


_replay_fn = None


def replay_calls(ncalls, fns, first_slot, slots, npatches, patch_slot, patch_key, patch_offset, addresses, expected, got) -> int:
    """Issue a packed list of recorded launches (csrc/replay.hip): every argument is the
    address of a host array.  Returns -1, or the index of the first call whose status
    differs from the recorded one."""
    global _replay_fn
    if _replay_fn is None:
        lib = load_library("replay")
        _replay_fn = lib.tk_replay_calls
        _replay_fn.argtypes = [c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_void_p, c_void_p]
        _replay_fn.restype = c_int
    return _replay_fn(ncalls, fns, first_slot, slots, npatches, patch_slot, patch_key, patch_offset, addresses, expected, got)


def not_replayable() -> None:
    """Called where work is launched past this module (a library routine of torch): a
    recording that is being made does not hold it and must not be replayed."""
    if _recorder is not None:
        _recorder.valid = False


def can_record() -> bool:
    return _recorder is None and _profile is None


_pinned_stream: c_void_p | None = None


def _stream() -> c_void_p:
    return _pinned_stream if _pinned_stream is not None else c_void_p(torch.cuda.current_stream().cuda_stream)


class pinned_stream:
    """Within the block every kernel of this module is launched on the stream that is
    current at entry, without asking torch for it launch by launch (that lookup costs
    more than the launch).  The caller must not switch streams inside the block."""

    def __enter__(self):
        global _pinned_stream
        self._before = _pinned_stream
        _pinned_stream = c_void_p(torch.cuda.current_stream().cuda_stream)
        return self

    def __exit__(self, *exc):
        global _pinned_stream
        _pinned_stream = self._before
        return False


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _gpu(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is None:
            continue
        _need(t.is_cuda, "kernel arguments must live on the GPU (there is no CPU path)")
        _need(t.is_contiguous(), "kernel arguments must be contiguous")


def _check(status: int, name: str) -> None:
    if status != 0:
        raise KernelError(f"{name} failed with status {status}")


_SIGS = {
    "elementwise": {
        "tk_embed_gather": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_int, c_void_p],
        "tk_feed_tokens": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
        "tk_add_rmsnorm": [c_int, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p,
                           c_void_p, c_int, c_int, c_float, c_int, c_void_p],
        "tk_add_norm2": [c_int, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p, c_int, c_int, c_long,
                         c_void_p, c_int, c_int, c_long, c_void_p, c_float, c_void_p,
                         c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_int, c_int, c_void_p],
        "tk_rope_tables": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p],
        "tk_qknorm_rope_store": [c_int, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                 c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p],
        "tk_rope_norm_store": [c_int, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                               c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float,
                               c_int, c_void_p, c_int, c_void_p, c_void_p],
        "tk_scale_softcap": [c_void_p, c_long, c_float, c_float, c_void_p],
        "tk_silu_mul": [c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p],
        "tk_add_bias": [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p],
        "tk_scaled_sum": [c_int, c_void_p, c_int, c_int, c_long, c_float, c_void_p, c_int, c_int, c_long, c_float,
                          c_void_p, c_void_p, c_int, c_int, c_void_p],
    },
    "attention_pooled": {
        "tk_bias_norm_store": [c_int, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                               c_int, c_float, c_int, c_void_p],
        "tk_pool_blocks": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                           c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "tk_pooled_window_attention": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                       c_void_p, c_void_p, c_void_p, c_void_p,
                                       c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                       c_int, c_int, c_int, c_int, c_float, c_void_p],
    },
    "attention_pooled_split": {
        "tk_pooled_window_attention_split": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                             c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                             c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                             c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p],
    },
    "recurrent": {
        "tk_token_shift": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                           c_int, c_int, c_void_p],
        "tk_tanh": [c_int, c_void_p, c_int, c_int, c_long, c_void_p, c_long, c_void_p],
        "tk_wkv_scan": [c_int, c_void_p, c_int, c_int, c_long, c_void_p, c_int, c_int, c_long, c_void_p, c_int, c_int,
                        c_long, c_void_p, c_int, c_int, c_long, c_void_p, c_int, c_int, c_long, c_void_p,
                        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float,
                        c_void_p],
        "tk_gla_scan": [c_int, c_void_p, c_int, c_int, c_long, c_void_p, c_int, c_int, c_long, c_void_p, c_int, c_int,
                        c_long, c_void_p, c_int, c_int, c_long, c_void_p, c_int, c_int, c_long, c_void_p,
                        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                        c_float, c_float, c_float, c_void_p],
    },
    "moe": {
        "tk_moe_route": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p,
                         c_int, c_int, c_int, c_float, c_void_p],
        "tk_moe_gate_up": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                           c_void_p],
        "tk_moe_down": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "tk_moe_sort": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
        "tk_moe_grouped": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                           c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    },
    "gemm_tiled": {
        "tk_gemm_tiled": [c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_long,
                          c_long, c_long, c_void_p],
        "tk_gemm_fewrows": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long,
                            c_long, c_void_p],
    },
    "gemm_mfma": {
        "tk_gemm_stream": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long,
                           c_long, c_int, c_long, c_int, c_void_p, c_int, c_float, c_void_p],
        "tk_gemm_stream_swiglu": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long, c_long,
                                  c_int, c_void_p, c_int, c_float, c_int, c_void_p],
        "tk_gemm_skinny": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long,
                           c_long, c_int, c_int, c_void_p],
    },
    "gemm_wholek": {
        "tk_gemm_wholek": [c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long, c_long,
                           c_void_p, c_int, c_float, c_int, c_void_p],
        "tk_gemm_wholek_slabs": [c_int],
        "tk_gemm_wholek_add": [c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long, c_void_p, c_long, c_void_p,
                               c_void_p, c_long, c_void_p, c_int, c_void_p],
    },
    "blas_lt": {
        "tk_lt_gemm": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long, c_long, c_void_p,
                       c_size_t, c_int, c_void_p],
    },
    "attention_generic": {
        "tk_paged_attention_generic": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                       c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                       c_float, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p,
                                       c_void_p],
    },
    "latent": {
        "tk_latent_prepare": [c_int, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                              c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                              c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
        "tk_head_linear": [c_int, c_void_p, c_long, c_long, c_void_p, c_void_p, c_long, c_long, c_int, c_int, c_int,
                           c_int, c_void_p],
    },
    "attention_mfma": {
        "tk_attention_mfma": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                              c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int,
                              c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_void_p],
    },
    "attention_tiles": {
        "tk_attention_tiles": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_void_p],
        "tk_attention_heads": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                               c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                               c_void_p, c_void_p],
    },
    "ssm": {
        "tk_conv_silu": [c_int, c_void_p, c_int, c_int, c_long, c_long, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                         c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "tk_ssd_scan": [c_int, c_void_p, c_void_p, c_int, c_int, c_long, c_long, c_int, c_void_p, c_void_p, c_void_p,
                        c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                        c_void_p, c_void_p, c_void_p],
        "tk_gated_group_norm": [c_int, c_void_p, c_void_p, c_int, c_int, c_long, c_long, c_int, c_void_p, c_void_p,
                                c_int, c_int, c_int, c_float, c_void_p],
    },
    "attention_fused": {
        "tk_attention_decode_fused": [c_void_p, c_int, c_int, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                      c_float, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                      c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                      c_int, c_int, c_float, c_void_p],
    },
    "sampling": {
        "tk_argmax": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p],
        "tk_argmax_masses": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                             c_int, c_int, c_long, c_void_p],
        "tk_argmax_segments": [],
        "tk_sample": [c_void_p, c_long, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                      c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    },
}
_LIBRARY_FILE = {"attention_fused": "attention_mfma", "attention_pooled_split": "attention_pooled"}   # signature group -> library that holds it
_fns: dict[str, ctypes._CFuncPtr] = {}
_profile: "KernelProfile | None" = None


class KernelProfile:
    """Times every kernel entry point called inside the ``with`` block with a pair
    of events on the current stream, and keeps what each call says about itself
    (shape, bytes it has to move, flops).  ``rows()`` gives one record per kind of
    call, summed.  Meant for one step at a time; the events add a few microseconds
    a launch, so the sum is above the step's time without them."""

    def __init__(self) -> None:
        self.calls: list[tuple[str, torch.cuda.Event, torch.cuda.Event, float, float]] = []
        self._note: tuple[str, float, float] | None = None

    def __enter__(self) -> "KernelProfile":
        global _profile
        self._before, _profile = _profile, self
        return self

    def __exit__(self, *exc) -> bool:
        global _profile
        _profile = self._before
        return False

    def note(self, shape: str, nbytes: float = 0.0, flops: float = 0.0) -> None:
        self._note = (shape, float(nbytes), float(flops))

    def timed(self, name: str, fn, args):
        shape, nbytes, flops = self._note or ("", 0.0, 0.0)
        self._note = None
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        status = fn(*args)
        e1.record()
        self.calls.append((f"{name[3:]} {shape}".strip(), e0, e1, nbytes, flops))
        return status

    def rows(self) -> list[dict]:
        """[{name, calls, us, bytes, flops}], longest first; synchronises."""
        torch.cuda.synchronize()
        merged: dict[str, dict] = {}
        for name, e0, e1, nbytes, flops in self.calls:
            row = merged.setdefault(name, {"name": name, "calls": 0, "us": 0.0, "bytes": 0.0, "flops": 0.0})
            row["calls"] += 1
            row["us"] += e0.elapsed_time(e1) * 1e3
            row["bytes"] += nbytes
            row["flops"] += flops
        return sorted(merged.values(), key=lambda r: -r["us"])


def _note(shape: str, nbytes: float = 0.0, flops: float = 0.0) -> None:
    """What the next kernel call is, for a running ``KernelProfile`` (else nothing)."""
    if _profile is not None:
        _profile.note(shape, nbytes, flops)


def _fn(library: str, name: str):
    fn = _fns.get(name)
    if fn is None:
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: tokamak_amd runs on an MI355X only")
        lib = load_library(_LIBRARY_FILE.get(library, library))
        fn = getattr(lib, name)
        fn.argtypes = _SIGS[library][name]
        fn.restype = c_int
        # the same entry point with its arguments as slots, if the library has it (csrc/slots.h)
        try:
            fn.slots_address = ctypes.cast(getattr(lib, name + "_slots"), c_void_p).value
        except AttributeError:
            fn.slots_address = None
        _fns[name] = fn
    if _profile is not None and name not in ("tk_argmax_segments",):
        profile = _profile
        return lambda *args: profile.timed(name, fn, args)
    if _recorder is not None:
        recorder = _recorder
        return lambda *args: recorder.call(fn, args)
    return fn


# ---------------------------------------------------------------------------
def embed_gather(table: torch.Tensor, ids: torch.Tensor, resid: torch.Tensor, scale: float = 1.0,
                 accumulate: bool = False) -> None:
    """resid[n] = float(table[ids[n]]) * scale (``accumulate``: added to what resid[n] holds);
    resid is float32 [N, H]."""
    _gpu(table, ids, resid)
    n = ids.numel()
    v, h = table.shape
    _need(ids.dtype == torch.int32, "token ids must be int32")
    _need(resid.dtype == torch.float32 and resid.shape[-1] == h and resid.numel() >= n * h,
          "residual buffer must be float32 [>=N, H]")
    _note(f"{n}x{h}", n * h * (table.element_size() + 4))
    _check(_fn("elementwise", "tk_embed_gather")(_code(table.dtype), _p(table), _p(ids), _p(resid),
                                                 n, h, v, float(scale), int(bool(accumulate)), _stream()),
           "embed_gather")


def feed_tokens(ids: torch.Tensor, sampled: torch.Tensor, slots: torch.Tensor, rows: torch.Tensor, count: int,
                num_sampled: int) -> None:
    """ids[slots[i]] = sampled[rows[i]] for i < count: token ids of a step that the sampler
    of the step before left on the GPU.  The host has checked slots and rows against the
    sizes (``num_sampled`` rows of ``sampled`` hold tokens)."""
    _gpu(ids, sampled, slots, rows)
    _need(ids.dtype == sampled.dtype == slots.dtype == rows.dtype == torch.int32, "token ids and indices are int32")
    _need(0 <= count <= slots.numel() and count <= rows.numel() and 0 <= num_sampled <= sampled.numel(),
          "more fed tokens than the index arrays hold")
    _check(_fn("elementwise", "tk_feed_tokens")(_p(ids), _p(sampled), _p(slots), _p(rows), count, _stream()), "feed_tokens")


def _partials(t: torch.Tensor | None, rows: int, width: int, dtype: torch.dtype, what: str):
    """(is_f32, parts, part_stride) of an input that is either [rows, width] in
    ``dtype`` or float32 partial sums [parts, rows, width] (a split-K product)."""
    if t is None:
        return 0, 1, 0
    if t.dim() == 3:
        _need(t.dtype == torch.float32 and t.shape[1] >= rows and t.shape[2] == width, f"{what}: partial sums must be float32 [parts, rows, {width}]")
        return 1, t.shape[0], t.stride(0)
    _need(t.dim() == 2 and t.shape[1] == width and t.shape[0] >= rows, f"{what} must be [rows, {width}]")
    if t.dtype == torch.float32:
        return 1, 1, 0
    _need(t.dtype == dtype, f"{what} must be float32 or the compute dtype")
    return 0, 1, 0


def add_rmsnorm(resid: torch.Tensor, delta: torch.Tensor | None, weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: torch.Tensor | None = None,
                write_resid: bool = True) -> None:
    """x = resid[row] (+ delta[row]); optionally stored back; out = rmsnorm(x) * weight.
    ``delta``: [M, H] in the compute dtype or float32, or float32 partial sums [P, M, H]."""
    _gpu(resid, delta, weight, out, rows)
    h = resid.shape[-1]
    m = out.shape[0] if rows is None else rows.numel()
    _need(resid.dtype == torch.float32 and weight.dtype == torch.float32, "residual and norm weight are float32")
    _need(weight.numel() == h and out.shape[-1] == h and out.shape[0] >= m, "rmsnorm shapes disagree")
    if rows is None:
        _need(resid.shape[0] >= m, "residual has fewer rows than the output")
    else:
        _need(rows.dtype == torch.int32 and not (write_resid and delta is not None),
              "row-indexed rmsnorm cannot write the residual")
        write_resid = False
    is_f32, parts, stride = _partials(delta, resid.shape[0], h, out.dtype, "delta")
    _note(f"{m}x{h}", m * h * (4 + (8 if write_resid else 0) + out.element_size())
          + (0 if delta is None else parts * m * h * delta.element_size()))
    _check(_fn("elementwise", "tk_add_rmsnorm")(_code(out.dtype), _p(resid), _p(delta), is_f32, parts, stride,
                                                _p(rows), _p(weight), _p(out), m, h, float(eps),
                                                int(bool(write_resid)), _stream()), "add_rmsnorm")


def add_norm2(resid: torch.Tensor, a: torch.Tensor | None, b: torch.Tensor | None, weight: torch.Tensor, eps: float,
              out: torch.Tensor, *, center: bool, rows: torch.Tensor | None = None, write_resid: bool = True,
              c: torch.Tensor | None = None, bias: torch.Tensor | None = None, scale: float = 1.0,
              weight2: torch.Tensor | None = None, out2: torch.Tensor | None = None) -> None:
    """x = resid[row] + scale * (a[row] + b[row] + c[row] + bias), optionally stored back; ``center``: out =
    (x - mean) / sqrt(mean((x - mean)^2) + eps) * weight (a layer norm without a bias), else the RMS norm.
    ``a``, ``b`` and ``c`` are each None, [M, H] in the compute dtype or float32, or float32 partial sums
    [P, M, H]; ``bias`` is None or float32 [H].  ``weight2`` and ``out2`` (both or neither): the same normalised
    row times a second weight, for two sub-layers that each norm the same stream."""
    _gpu(resid, a, b, c, bias, weight, out, rows, weight2, out2)
    h = resid.shape[-1]
    m = out.shape[0] if rows is None else rows.numel()
    _need(resid.dtype == torch.float32 and weight.dtype == torch.float32, "residual and norm weight are float32")
    _need(weight.numel() == h and out.shape[-1] == h and out.shape[0] >= m, "norm shapes disagree")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == h), "the bias is float32 [H]")
    _need((weight2 is None) == (out2 is None), "a second weight and a second output come together")
    if weight2 is not None:
        _need(weight2.dtype == torch.float32 and weight2.numel() == h and out2.dtype == out.dtype
              and out2.shape[-1] == h and out2.shape[0] >= m, "the second norm's shapes disagree")
    adds = a is not None or b is not None or c is not None or bias is not None
    if rows is None:
        _need(resid.shape[0] >= m, "residual has fewer rows than the output")
    else:
        _need(rows.dtype == torch.int32 and not (write_resid and adds), "a row-indexed norm cannot write the residual")
        write_resid = False
    pa, fa, na, sa = _branch(a, resid.shape[0], h, out.dtype, "a")
    pb, fb, nb, sb = _branch(b, resid.shape[0], h, out.dtype, "b")
    pc, fc, nc, sc = _branch(c, resid.shape[0], h, out.dtype, "c")
    _note(f"{m}x{h}", m * h * (4 + (8 if write_resid and adds else 0) + out.element_size() * (2 if out2 is not None else 1))
          + sum(t.element_size() * parts * m * h for t, parts in ((a, na), (b, nb), (c, nc)) if t is not None))
    _check(_fn("elementwise", "tk_add_norm2")(_code(out.dtype), _p(resid), pa, fa, na, sa, pb, fb, nb, sb, pc, fc, nc, sc,
                                              _p(bias), float(scale), _p(rows), _p(weight), _p(out), _p(weight2), _p(out2),
                                              m, h, float(eps), int(bool(write_resid)), int(bool(center)), _stream()),
           "add_norm2")


def rope_tables(positions: torch.Tensor, inv_freq: torch.Tensor, cos: torch.Tensor,
                sin: torch.Tensor, amplitude: float = 1.0) -> None:
    """cos and sin of float(position) * inv_freq[j], float32 [N, half], both times ``amplitude``."""
    _gpu(positions, inv_freq, cos, sin)
    n, half = positions.numel(), inv_freq.numel()
    _need(positions.dtype == torch.int32 and inv_freq.dtype == torch.float32, "positions int32, inv_freq float32")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.numel() >= n * half
          and sin.numel() >= n * half, "cos/sin tables must be float32 [N, half]")
    _check(_fn("elementwise", "tk_rope_tables")(_p(positions), _p(inv_freq), _p(cos), _p(sin), n,
                                                half, float(amplitude), _stream()), "rope_tables")


def qknorm_rope_store(qkv: torch.Tensor, q_weight: torch.Tensor | None,
                      k_weight: torch.Tensor | None, cos: torch.Tensor | None, sin: torch.Tensor | None,
                      positions: torch.Tensor, req_of_token: torch.Tensor,
                      block_tables: torch.Tensor, q_out: torch.Tensor,
                      k_cache: torch.Tensor | None, v_cache: torch.Tensor | None, *, num_heads: int,
                      num_kv_heads: int, head_dim: int, rotary_dim: int, page_size: int, eps: float,
                      store: bool = True) -> None:
    """Per-head norm + rotation of q (and k), q written to q_out, k/v into pages.
    ``rotary_dim`` 0 (then ``cos`` and ``sin`` may be None): no rotation."""
    _gpu(qkv, q_weight, k_weight, cos, sin, positions, req_of_token, block_tables, q_out, k_cache, v_cache)
    n = positions.numel()
    nkv_in = num_kv_heads if store else 0
    width = (num_heads + 2 * nkv_in) * head_dim
    in_f32, parts, stride = _partials(qkv, n, width, q_out.dtype, "qkv")
    _need(q_out.numel() >= n * num_heads * head_dim, "q_out too small")
    _need(head_dim % 16 == 0 and head_dim <= 512 and page_size % 8 == 0, "head_dim must be a multiple of 16 (at most 512), page_size a multiple of 8")
    _need(rotary_dim % 2 == 0 and rotary_dim <= head_dim, "rotary_dim must be even and <= head_dim")
    _need(rotary_dim == 0 or (cos is not None and sin is not None and cos.dtype == torch.float32
                               and sin.dtype == torch.float32 and cos.numel() >= n * (rotary_dim // 2)
                               and sin.numel() >= n * (rotary_dim // 2)), "rotary tables missing, not float32 or too small")
    for w in (q_weight, k_weight):
        _need(w is None or (w.dtype == torch.float32 and w.numel() == head_dim), "q/k norm weights are float32 [head_dim]")
    _need(positions.dtype == torch.int32 and req_of_token.dtype == torch.int32
          and block_tables.dtype == torch.int32 and block_tables.dim() == 2, "descriptor arrays are int32")
    _need(req_of_token.numel() >= n, "req_of_token shorter than positions")
    max_pages = block_tables.shape[1]
    if store:
        page_elems = num_kv_heads * head_dim * page_size
        _need(k_cache is not None and v_cache is not None and k_cache.dtype == q_out.dtype
              and v_cache.dtype == q_out.dtype, "cache dtype must match activations")
        _need(k_cache.numel() % page_elems == 0 and v_cache.numel() == k_cache.numel(), "cache size is not whole pages")
    _note(f"{n}x{width}", n * width * (qkv.element_size() * parts + q_out.element_size()))
    _check(_fn("elementwise", "tk_qknorm_rope_store")(
        _code(q_out.dtype), _p(qkv), in_f32, parts, stride, _p(q_weight), _p(k_weight), _p(cos), _p(sin), _p(positions),
        _p(req_of_token), _p(block_tables), _p(q_out), _p(k_cache), _p(v_cache), n, num_heads,
        nkv_in, num_kv_heads, head_dim, rotary_dim, page_size, max_pages, float(eps), _stream()),
        "qknorm_rope_store")


def rope_norm_store(qkv: torch.Tensor, q_weight: torch.Tensor | None, k_weight: torch.Tensor | None,
                    cos: torch.Tensor | None, sin: torch.Tensor | None, positions: torch.Tensor,
                    req_of_token: torch.Tensor, block_tables: torch.Tensor, q_out: torch.Tensor,
                    k_cache: torch.Tensor | None, v_cache: torch.Tensor | None, *, num_heads: int, num_kv_heads: int,
                    head_dim: int, value_dim: int, rotary_dim: int, page_size: int, unit_norm: bool, eps: float,
                    store: bool = True, interleaved: bool = False, value_keep: torch.Tensor | None = None,
                    value_mode: int = 0, value_lambda: torch.Tensor | None = None) -> None:
    """Rotation of the first ``rotary_dim`` dims of every q and k head, then (``unit_norm``) each
    head divided by its root mean square over ``head_dim`` (times a weight, if given); q written to
    q_out, k and v into pages.  Values are ``value_dim`` wide.  ``rotary_dim`` 0: no rotation.
    q_out and the pages are laid out for ``padded_sizes(head_dim, value_dim)``: the channels behind
    the true sizes hold zeros.  ``interleaved``: the rotation pairs dim 2j with 2j + 1 instead of j with
    j + rotary_dim / 2.  ``value_mode`` 1: the values, as projected, are also left in ``value_keep`` (float32
    [N, kv heads * value_dim]); 2: what is cached is (1 - lambda) v + lambda value_keep with lambda =
    ``value_lambda`` (one float32 number on the device)."""
    _gpu(qkv, q_weight, k_weight, cos, sin, positions, req_of_token, block_tables, q_out, k_cache, v_cache,
         value_keep, value_lambda)
    n = positions.numel()
    nkv_in = num_kv_heads if store else 0
    if not store:
        value_mode = 0
    _need(value_mode in (0, 1, 2), "value_mode is 0, 1 or 2")
    if value_mode:
        _need(value_keep is not None and value_keep.dtype == torch.float32
              and value_keep.numel() >= n * num_kv_heads * value_dim, "the kept values are float32 [N, kv heads * value_dim]")
    if value_mode == 2:
        _need(value_lambda is not None and value_lambda.dtype == torch.float32 and value_lambda.numel() == 1,
              "the mixing weight is one float32 number")
    width = (num_heads + nkv_in) * head_dim + nkv_in * value_dim
    in_f32, parts, stride = _partials(qkv, n, width, q_out.dtype, "qkv")
    hdp, vdp = padded_sizes(head_dim, value_dim)
    _need(q_out.numel() >= n * num_heads * hdp, "q_out too small")
    _need(min(head_dim, value_dim) >= 1 and max(hdp, vdp) <= 512 and page_size % 8 == 0,
          "head sizes are 1 to 512, page_size a multiple of 8")
    _need(rotary_dim % 2 == 0 and rotary_dim <= head_dim, "rotary_dim must be even and <= head_dim")
    _need(rotary_dim == 0 or (cos is not None and sin is not None and cos.dtype == torch.float32
                               and sin.dtype == torch.float32 and cos.numel() >= n * (rotary_dim // 2)
                               and sin.numel() >= n * (rotary_dim // 2)), "rotary tables missing, not float32 or too small")
    for w in (q_weight, k_weight):
        _need(w is None or (w.dtype == torch.float32 and w.numel() == head_dim), "q/k norm weights are float32 [head_dim]")
    _need(positions.dtype == torch.int32 and req_of_token.dtype == torch.int32
          and block_tables.dtype == torch.int32 and block_tables.dim() == 2, "descriptor arrays are int32")
    _need(req_of_token.numel() >= n, "req_of_token shorter than positions")
    if store:
        _need(k_cache is not None and v_cache is not None and k_cache.dtype == q_out.dtype
              and v_cache.dtype == q_out.dtype, "cache dtype must match activations")
        _need(k_cache.numel() % (num_kv_heads * hdp * page_size) == 0
              and v_cache.numel() % (num_kv_heads * vdp * page_size) == 0
              and k_cache.numel() // hdp == v_cache.numel() // vdp, "cache size is not whole pages")
    _note(f"{n}x{width}", n * width * (qkv.element_size() * parts + q_out.element_size()))
    _check(_fn("elementwise", "tk_rope_norm_store")(
        _code(q_out.dtype), _p(qkv), in_f32, parts, stride, _p(q_weight), _p(k_weight), _p(cos), _p(sin), _p(positions),
        _p(req_of_token), _p(block_tables), _p(q_out), _p(k_cache), _p(v_cache), n, num_heads,
        nkv_in, num_kv_heads, head_dim, value_dim, hdp, vdp, rotary_dim, page_size, block_tables.shape[1],
        int(bool(unit_norm)), float(eps), int(bool(interleaved)), _p(value_keep if value_mode else None), int(value_mode),
        _p(value_lambda if value_mode == 2 else None), _stream()), "rope_norm_store")


def padded_sizes(head_dim: int, value_dim: int) -> tuple[int, int]:
    """The sizes that cache pages are laid out for: keys in pieces of 8 channels, values in
    blocks of 16."""
    return -(-head_dim // 8) * 8, -(-value_dim // 16) * 16


def scale_softcap(logits: torch.Tensor, scale: float, cap: float | None) -> None:
    """In place on float32 logits: x <- x * scale, then with a ``cap`` x <- cap * tanh(x / cap)."""
    _gpu(logits)
    _need(logits.dtype == torch.float32, "logits are float32")
    _check(_fn("elementwise", "tk_scale_softcap")(_p(logits), logits.numel(), float(scale), float(cap or 0.0), _stream()),
           "scale_softcap")


GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor, activation: str = "silu", bias: torch.Tensor | None = None) -> None:
    """out[n, i] = act(gate_up[n, i]) * gate_up[n, I + i]; act is silu, or the tanh form of gelu.  ``bias``:
    float32 [2 I], added to both halves before the activation."""
    _gpu(gate_up, out, bias)
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == gate_up.shape[1]), "the bias is float32 [2 I]")
    n, two_i = gate_up.shape
    _need(two_i % 2 == 0 and out.shape == (n, two_i // 2) and out.dtype == gate_up.dtype, "silu_mul shapes disagree")
    _note(f"{n}x{two_i // 2}", n * two_i * out.element_size() * 1.5)
    _need(activation in GATE_ACTIVATIONS, f"the gate's activation is one of {sorted(GATE_ACTIVATIONS)}")
    _check(_fn("elementwise", "tk_silu_mul")(_code(out.dtype), _p(gate_up), _p(out), n, two_i // 2,
                                             GATE_ACTIVATIONS[activation], _p(bias), _stream()), "silu_mul")


def add_bias(x: torch.Tensor, bias: torch.Tensor) -> None:
    """x[n, c] += bias[c] in place; x [N, H] in the compute dtype or float32, bias float32 [H]."""
    _gpu(x, bias)
    n, h = x.shape
    _need(bias.dtype == torch.float32 and bias.numel() == h, "the bias is float32 [H]")
    _note(f"{n}x{h}", 2 * n * h * x.element_size())
    _check(_fn("elementwise", "tk_add_bias")(_code(x.dtype), _p(x), _p(bias), n, h, _stream()), "add_bias")


def _branch(t: torch.Tensor | None, rows: int, width: int, dtype: torch.dtype, what: str):
    """(pointer, is_f32, parts, part_stride) of a contiguous [rows, width] input in ``dtype`` or
    float32, or of float32 partial sums [parts, rows, width]."""
    if t is None:
        return _p(None), 0, 1, 0
    _need(t.is_contiguous() and t.shape[-2] == rows, f"{what} must be contiguous with {rows} rows")
    is_f32, parts, stride = _partials(t, rows, width, dtype, what)
    return _p(t), is_f32, parts, stride


def scaled_sum(a: torch.Tensor, weight_a: float, b: torch.Tensor | None, weight_b: float,
               scale: torch.Tensor | None, out: torch.Tensor, dtype: torch.dtype) -> None:
    """out = scale * (weight_a * a + weight_b * b), float32 [N, H].  ``a`` and ``b`` are each
    [N, H] in ``dtype`` or float32, or float32 partial sums [P, N, H]; ``b`` and ``scale`` [H]
    may be None."""
    _gpu(a, b, scale, out)
    n, h = out.shape
    _need(out.dtype == torch.float32, "the scaled sum is float32")
    _need(scale is None or (scale.dtype == torch.float32 and scale.numel() == h), "the scale is float32 [H]")
    pa, fa, na, sa = _branch(a, n, h, dtype, "a")
    pb, fb, nb, sb = _branch(b, n, h, dtype, "b")
    _note(f"{n}x{h}", n * h * (4 + a.element_size() * na + (0 if b is None else b.element_size() * nb)))
    _check(_fn("elementwise", "tk_scaled_sum")(_code(dtype), pa, fa, na, sa, float(weight_a), pb, fb, nb, sb,
                                               float(weight_b), _p(scale), _p(out), n, h, _stream()), "scaled_sum")


def bias_norm_store(qkv: torch.Tensor, bias: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor,
                    positions: torch.Tensor, req_of_token: torch.Tensor, tables: torch.Tensor, q_out: torch.Tensor,
                    k_cache: torch.Tensor, v_cache: torch.Tensor, *, q_width: int, k_width: int, v_width: int,
                    page_size: int, eps: float, store: bool = True) -> None:
    """q/k/v projection output plus ``bias``; q and k each divided by the root mean square of
    their whole row and multiplied by ``q_weight`` / ``k_weight``; q to ``q_out`` [N, q_width], k
    and v into the pages (``[page][token][width]``) of each token's request."""
    _gpu(qkv, bias, q_weight, k_weight, positions, req_of_token, tables, q_out, k_cache, v_cache)
    n = q_out.shape[0]
    total = q_width + k_width + v_width if store else q_width
    dtype = q_out.dtype
    _need(q_out.shape == (n, q_width) and k_cache.dtype == dtype and v_cache.dtype == dtype, "q/k/v outputs disagree")
    _need(bias.dtype == torch.float32 and bias.numel() == q_width + k_width + v_width, "one float32 bias per projected coordinate")
    _need(q_weight.dtype == torch.float32 and q_weight.numel() == q_width and k_weight.dtype == torch.float32
          and k_weight.numel() == k_width, "norm weights are float32 over the whole projection")
    _need(positions.numel() >= n and req_of_token.numel() >= n and tables.dim() == 2 and tables.dtype == torch.int32,
          "step descriptor arrays are too short")
    _need(k_cache.dim() == 2 and k_cache.shape[1] == k_width * page_size and v_cache.shape[1] == v_width * page_size
          and k_cache.shape[0] == v_cache.shape[0], "cache arrays do not have the page layout")
    p, is_f32, parts, stride = _branch(qkv, n, total, dtype, "qkv")
    _note(f"{n}x{total}", n * total * (qkv.element_size() * parts + dtype.itemsize))
    _check(_fn("attention_pooled", "tk_bias_norm_store")(
        _code(dtype), p, is_f32, parts, stride, _p(bias), _p(q_weight), _p(k_weight), _p(positions),
        _p(req_of_token), _p(tables), tables.shape[1], _p(q_out), _p(k_cache), _p(v_cache), n, q_width, k_width,
        v_width, page_size, float(eps), int(bool(store)), _stream()), "bias_norm_store")


def pooled_elems(width: int, pool: int) -> int:
    """Elements a position of a pooled array: block b's mean of ``width`` numbers is elements
    [b * width, (b + 1) * width) of the request's flat array, which therefore lies in pages the
    request owns once the block's ``pool`` positions are stored."""
    return -(-width // pool)


def _pooled_arrays(k_pool, v_pool, k_cache, k_width, v_width, pool, page_size):
    _need(k_pool.dtype == torch.float32 and v_pool.dtype == torch.float32, "pooled arrays are float32")
    _need(k_pool.shape[0] == k_cache.shape[0] == v_pool.shape[0] and k_pool.shape[1] % page_size == 0
          and v_pool.shape[1] % page_size == 0, "pooled arrays do not have the page layout")
    ke, ve = k_pool.shape[1] // page_size, v_pool.shape[1] // page_size
    _need(ke * pool >= k_width and ve * pool >= v_width, "pooled arrays are too narrow for a block's mean")
    return ke, ve


def pool_blocks(k_cache: torch.Tensor, v_cache: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                positions: torch.Tensor, req_of_token: torch.Tensor, tables: torch.Tensor, n: int, *,
                k_width: int, v_width: int, pool: int, page_size: int) -> None:
    """Every token of the step that completes a block of ``pool`` positions writes the means of
    the block's cached keys and values (summed in position order, float32) into the pooled arrays."""
    _gpu(k_cache, v_cache, k_pool, v_pool, positions, req_of_token, tables)
    _need(k_cache.dtype == v_cache.dtype and k_cache.shape[1] == k_width * page_size
          and v_cache.shape[1] == v_width * page_size, "cache arrays do not have the page layout")
    _need(positions.numel() >= n and req_of_token.numel() >= n and tables.dim() == 2, "step descriptor arrays are too short")
    ke, ve = _pooled_arrays(k_pool, v_pool, k_cache, k_width, v_width, pool, page_size)
    _check(_fn("attention_pooled", "tk_pool_blocks")(
        _code(k_cache.dtype), _p(k_cache), _p(v_cache), _p(k_pool), _p(v_pool), _p(positions), _p(req_of_token),
        _p(tables), tables.shape[1], n, k_width, v_width, ke, ve, pool, page_size, _stream()), "pool_blocks")


POOLED_LDS_BYTES = 144 * 1024      # of a CU's 160 KB
POOLED_ACC = 16                    # outputs a thread of the attention kernel accumulates


def pooled_window_plan(num_heads: int, num_kv_heads: int, dim: int, vdim: int, longest_span: int) -> tuple[int, int, int]:
    """(rows a block takes, entries a chunk, threads a block) for the pooled-window attention
    kernel: up to 8 consecutive rows of a portion share the keys and values a block stages;
    single tokens take a block each."""
    threads = 256
    while num_heads * vdim > POOLED_ACC * threads and threads < 1024:
        threads *= 2
    _need(num_heads * vdim <= POOLED_ACC * threads, f"{num_heads} heads of {vdim} values are more than the kernel accumulates")
    rows = 1 if longest_span <= 1 else max(1, min(8, POOLED_ACC * threads // (num_heads * vdim)))
    while True:
        fixed = rows * num_heads * dim + 2 * rows * num_heads + num_heads * num_heads
        per_entry = num_kv_heads * (dim + vdim) + 2 + 2 * rows * num_heads
        chunk = min(64, (POOLED_LDS_BYTES // 4 - fixed) // per_entry)
        if chunk >= 8 or rows == 1:
            break
        rows //= 2
    _need(chunk >= 1, "the heads of this attention do not fit the kernel's LDS")
    return rows, chunk, threads


POOLED_ONE_KERNEL_ONLY = False   # tests set this to run the one-kernel form on sizes the other form takes

POOLED_SPLIT_GROUP = 16      # query heads a kv head, value channels and rows times heads a block
POOLED_SPLIT_VDIM = 256      # that the four-kernel form of the attention takes
POOLED_SPLIT_PAIRS = 32
POOLED_SPLIT_HEADS = 64      # heads whose weights a thread of the mixing kernel holds
POOLED_SPLIT_BLOCKS = 512    # blocks wanted: two a CU run at once (some 200 registers a lane), a third waits for a whole turn
POOLED_SPLIT_LDS = 150 * 1024


def pooled_split_plan(num_heads: int, num_kv_heads: int, dim: int, vdim: int, window: int, pool: int, n: int,
                      longest_span: int, longest_context: int) -> tuple[int, int, int] | None:
    """(rows a block, shares of the entries, most entries a tile sees) for the four-kernel form of
    the pooled-window attention, or None where its sizes do not fit and the one-kernel form runs.
    Up to 8 consecutive rows of a portion share the rows a lane loads; single tokens take a
    block each; the entries are cut in shares until about a thousand blocks exist."""
    from tokamak_amd.kernels.attention import quarter_octave_at_least

    group = num_heads // num_kv_heads
    if group > POOLED_SPLIT_GROUP or vdim > POOLED_SPLIT_VDIM or num_heads > POOLED_SPLIT_HEADS or POOLED_ONE_KERNEL_ONLY:
        return None
    # the length rounded as recorded steps round it: a step computes the same bits recorded or not
    longest_context = quarter_octave_at_least(longest_context, 64)
    rows = 1 if longest_span <= 1 else max(1, min(8, POOLED_SPLIT_PAIRS // group))
    def values_lds(rows: int) -> int:
        return 4 * (rows * group * 256 + 64 * (vdim + 3))

    while rows > 1 and values_lds(rows) > POOLED_SPLIT_LDS:
        rows //= 2
    if (values_lds(rows) > POOLED_SPLIT_LDS or 4 * (rows * group * dim + 16 * POOLED_SPLIT_PAIRS) > POOLED_SPLIT_LDS
            or num_heads > 4096):
        return None
    most = min(longest_context, window + rows - 1) + longest_context // pool + 1
    blocks = -(-n // rows) * num_kv_heads
    # (a share of at least 32 entries; the shares' statistics of a row's heads fit the LDS they are merged in)
    shares = max(1, min(32, POOLED_SPLIT_BLOCKS // blocks, -(-most // 32), 2048 // num_heads))
    return rows, shares, most


def pooled_window_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, k_pool: torch.Tensor,
                            v_pool: torch.Tensor, tables: torch.Tensor, batch, talk: torch.Tensor, out: torch.Tensor, *, num_heads: int, num_kv_heads: int,
                            dim: int, vdim: int, window: int, pool: int, page_size: int, scale: float) -> None:
    """Attention of every row of the step over its request's pages: the last ``window``
    positions one by one, complete blocks of ``pool`` positions behind them by the means of
    their keys and values (``k_pool``, ``v_pool``, written by ``pool_blocks``), one softmax over
    both, the heads' weights mixed by ``talk`` [H, H]."""
    _gpu(q, k_cache, v_cache, k_pool, v_pool, tables, talk, out)
    ke, ve = _pooled_arrays(k_pool, v_pool, k_cache, num_kv_heads * dim, num_kv_heads * vdim, pool, page_size)
    n = q.shape[0]
    dtype = q.dtype
    _need(q.shape == (n, num_heads * dim) and out.shape == (n, num_heads * vdim) and out.dtype == dtype, "q/out shapes disagree")
    _need(k_cache.dtype == dtype and v_cache.dtype == dtype and k_cache.shape[1] == num_kv_heads * dim * page_size
          and v_cache.shape[1] == num_kv_heads * vdim * page_size, "cache arrays do not have the page layout")
    _need(talk.dtype == torch.float32 and talk.shape == (num_heads, num_heads), "the head-mixing matrix is float32 [H, H]")
    _need(num_heads % num_kv_heads == 0 and window >= 1 and pool >= 1, "bad attention sizes")
    _need(batch.num_tokens == n and tables.shape[0] == batch.num_requests and tables.dtype == torch.int32,
          "block tables do not match the step")
    _need(-(-batch.max_seq_len // page_size) <= tables.shape[1], "a block table is shorter than its request")
    if _profile is not None:
        # the least a step has to move: every cached position of every request once, queries in,
        # results out; and two multiply-adds per head, channel and visible entry
        elem = q.element_size()
        entries = 0
        for q_len, ctx in zip(batch.q_lens, batch.ctx_lens):
            for i in range(ctx, ctx + q_len):
                entries += min(i + 1, window) + max(0, (i - window - (pool - 1)) // pool + 1 if i - window >= pool - 1 else 0)
        # (a request's window of rows in the cache's type, its blocks' means in float32)
        cached = sum(min(c + ql, window + ql - 1) * elem + (c + ql) // pool * 4 for c, ql in zip(batch.ctx_lens, batch.q_lens))
        _note(f"{n}x{num_heads}x{dim}", cached * num_kv_heads * (dim + vdim) + n * num_heads * (dim + vdim) * elem,
              2.0 * num_heads * (dim + vdim) * entries)
    split = pooled_split_plan(num_heads, num_kv_heads, dim, vdim, window, pool, n, batch.max_q_len,
                              batch.facts.get("context.max_len", batch.max_seq_len))
    if split is not None:
        # the form that fills the GPU: a block a (tile of rows, kv head, share of the entries)
        rows, shares, most = split
        dev = q.device
        scores = torch.empty((n, most, num_heads), dtype=torch.float32, device=dev)
        part_m = torch.empty((n, num_heads, shares), dtype=torch.float32, device=dev)
        part_l = torch.empty((n, num_heads, shares), dtype=torch.float32, device=dev)
        part_o = torch.empty((shares, n, num_heads * vdim), dtype=torch.float32, device=dev) if shares > 1 else None
        _check(_fn("attention_pooled_split", "tk_pooled_window_attention_split")(
            _code(dtype), _p(q), _p(k_cache), _p(v_cache), _p(k_pool), _p(v_pool), ke, ve, _p(out), _p(batch.positions),
            _p(batch.req_of_token), _p(batch.q_start), _p(tables), tables.shape[1], _p(talk), _p(scores), _p(part_m),
            _p(part_l), _p(part_o), n, num_heads, num_kv_heads, dim, vdim, window, pool, page_size, rows, shares, most,
            float(scale), _stream()), "pooled_window_attention_split")
        return
    rows, chunk, threads = pooled_window_plan(num_heads, num_kv_heads, dim, vdim, batch.max_q_len)
    _check(_fn("attention_pooled", "tk_pooled_window_attention")(
        _code(dtype), _p(q), _p(k_cache), _p(v_cache), _p(k_pool), _p(v_pool), ke, ve, _p(out), _p(batch.positions),
        _p(batch.req_of_token), _p(batch.q_start), _p(tables), tables.shape[1], _p(talk), n, num_heads, num_kv_heads, dim, vdim, window, pool,
        page_size, rows, chunk, threads, float(scale), _stream()), "pooled_window_attention")


def token_shift(h: torch.Tensor, mu: torch.Tensor, last: torch.Tensor, out: torch.Tensor, batch) -> None:
    """out[s, n] = h[n] + (h[n - 1] - h[n]) * mu[s]; the row before a request's first token of
    the step is ``last[slot]`` (float32 [slots, W]), which then takes the request's last row."""
    _gpu(h, mu, last, out)
    n, w = h.shape
    s = mu.shape[0]
    _need(mu.dtype == torch.float32 and mu.shape == (s, w) and last.dtype == torch.float32 and last.shape[1] == w,
          "mix weights and the kept row are float32 of the input's width")
    _need(out.shape == (s, n, w) and out.dtype == h.dtype and batch.num_tokens == n, "token shift shapes disagree")
    _note(f"{n}x{w}x{s}", n * w * h.element_size() * (1 + s))
    _check(_fn("recurrent", "tk_token_shift")(_code(h.dtype), _p(h), _p(mu), _p(last), _p(out), _p(batch.req_of_token),
                                               _p(batch.q_start), _p(batch.state_slots), n, w, s, _stream()), "token_shift")


def tanh(x: torch.Tensor, out: torch.Tensor) -> None:
    """out = tanh(x); ``x`` [N, W] in out's dtype or float32, or float32 partial sums [P, N, W]."""
    _gpu(x, out)
    n, w = out.shape
    p, is_f32, parts, stride = _branch(x, n, w, out.dtype, "x")
    _check(_fn("recurrent", "tk_tanh")(_code(out.dtype), p, is_f32, parts, stride, _p(out), n * w, _stream()), "tanh")


WKV_MAX_DIM = 256


def wkv_scan(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gate: torch.Tensor, decay_in: torch.Tensor,
             w0: torch.Tensor, u: torch.Tensor, gain: torch.Tensor, state: torch.Tensor, out: torch.Tensor, batch,
             *, heads: int, dim: int, eps: float) -> None:
    """Per request and head, over the step's tokens in order: o = (S + diag(u) k v^T)^T r, then
    S <- diag(exp(-exp(decay_in + w0))) S + k v^T (S float32 [slots, heads, dim, dim], kept);
    out = o / rms(o) * gain * silu(gate).  r, k, v, gate, decay_in: [N, heads * dim] in out's dtype or
    float32, or float32 partial sums [P, N, heads * dim] of a split product."""
    _gpu(r, k, v, gate, decay_in, w0, u, gain, state, out)
    n, hd = out.shape
    dtype = out.dtype
    _need(hd == heads * dim and 1 <= dim <= WKV_MAX_DIM, f"the scan takes heads of up to {WKV_MAX_DIM} channels")
    for t in (w0, u, gain):
        _need(t.dtype == torch.float32 and t.numel() == hd, "decay offset, bonus and gain are float32 [heads * dim]")
    _need(state.dtype == torch.float32 and tuple(state.shape[1:]) == (heads, dim, dim), "the state is float32 [slots, heads, dim, dim]")
    _need(batch.num_tokens == n, "the step's descriptor does not match")
    operands = [x for t, what in ((r, "r"), (k, "k"), (v, "v"), (gate, "gate"), (decay_in, "decay_in"))
                for x in _branch(t, n, hd, dtype, what)]
    _note(f"{n}x{heads}x{dim}", n * hd * 6 * out.element_size(), 4.0 * n * heads * dim * dim)
    _check(_fn("recurrent", "tk_wkv_scan")(
        _code(dtype), *operands, _p(w0), _p(u), _p(gain), _p(state),
        _p(batch.q_start), _p(batch.state_slots), _p(out), batch.num_requests, heads, dim, float(eps), _stream()),
        "wkv_scan")


def gla_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gate: torch.Tensor, decay_in: torch.Tensor,
             bias: torch.Tensor, gain: torch.Tensor, state: torch.Tensor, out: torch.Tensor, batch, *, heads: int,
             dim: int, vdim: int, q_scale: float, tau: float, eps: float) -> None:
    """Per request and head, over the step's tokens in order: S <- diag(a) S + k v^T with
    a = sigmoid(decay_in + bias)^(1 / tau), then o = S^T (q * q_scale) (S float32 [slots, heads, dim, vdim],
    kept); out = o / rms(o) * gain * silu(gate).  q, k, decay_in: [N, heads * dim]; v, gate: [N, heads * vdim];
    each in out's dtype or float32, or float32 partial sums [P, N, width] of a split product."""
    _gpu(q, k, v, gate, decay_in, bias, gain, state, out)
    n = out.shape[0]
    dtype = out.dtype
    _need(out.shape[1] == heads * vdim and 1 <= dim <= WKV_MAX_DIM and 1 <= vdim <= WKV_MAX_DIM,
          f"the scan takes heads of up to {WKV_MAX_DIM} channels")
    _need(bias.dtype == torch.float32 and bias.numel() == heads * dim, "the decay's bias is float32 [heads * dim]")
    _need(gain.dtype == torch.float32 and gain.numel() == vdim, "the gain is float32 [vdim]")
    _need(state.dtype == torch.float32 and tuple(state.shape[1:]) == (heads, dim, vdim), "the state is float32 [slots, heads, dim, vdim]")
    _need(batch.num_tokens == n and tau > 0, "the step's descriptor does not match")
    operands = [x for t, what, w in ((q, "q", heads * dim), (k, "k", heads * dim), (v, "v", heads * vdim),
                                     (gate, "gate", heads * vdim), (decay_in, "decay_in", heads * dim))
                for x in _branch(t, n, w, dtype, what)]
    splits = gla_column_splits(batch.num_requests, heads, vdim, batch.max_q_len)
    # (scratch of a scan with shared columns: the raw outputs, and behind them the decays)
    raw = torch.empty((n, heads * (vdim + dim)), dtype=torch.float32, device=out.device) if splits > 1 else None
    _note(f"{n}x{heads}x{dim}x{vdim}", n * heads * (3 * dim + 3 * vdim) * out.element_size(), 4.0 * n * heads * dim * vdim)
    _check(_fn("recurrent", "tk_gla_scan")(
        _code(dtype), *operands, _p(bias), _p(gain), _p(state), _p(batch.q_start), _p(batch.state_slots), _p(out),
        _p(raw), n, splits, batch.num_requests, heads, dim, vdim, float(q_scale), 1.0 / float(tau), float(eps), _stream()),
        "gla_scan")


GLA_SPLIT_FROM_TOKENS = 64     # a request's tokens in a step from which its heads' value columns are shared out
GLA_SPLIT_MIN_COLUMNS = 8      # columns a block keeps at least
GLA_SPLIT_BLOCKS = 1024        # blocks wanted: four small ones a CU run side by side, each waiting for its own barriers


def gla_column_splits(requests: int, heads: int, vdim: int, longest: int) -> int:
    """Blocks that share a head's value columns in the scan: one in steps of few tokens a request
    (the scan then norms and gates by itself); in a long portion as many as give some 1,024 blocks,
    each with 8 columns or more (a second kernel then norms and gates)."""
    if longest < GLA_SPLIT_FROM_TOKENS:
        return 1
    splits = 1
    while (requests * heads * splits < GLA_SPLIT_BLOCKS and vdim // (2 * splits) >= GLA_SPLIT_MIN_COLUMNS
           and vdim % (2 * splits) == 0):
        splits *= 2
    return splits


SSM_MAX_TAPS = 8             # taps of the short convolution (csrc/ssm.hip: kMaxTaps)
SSM_SPLIT_FROM_TOKENS = 64   # a request's tokens in a step from which a head's value columns are shared out
SSM_SPLIT_MIN_COLUMNS = 8
SSM_SPLIT_BLOCKS = 1024
SSM_CHUNK_TOKENS = 64        # tokens of a chunk of a long portion; the chunks of a portion run side by side
SSM_CHUNKS_FROM_TOKENS = 128  # a request's tokens in a step from which the step's portions are cut into chunks


def _ssm_in(t: torch.Tensor, rows: int, dtype: torch.dtype, what: str):
    """(pointer, is_f32, parts, part_stride, row length) of a projection [rows, ld] in ``dtype`` or float32, or of
    float32 partial sums [parts, rows, ld]."""
    ld = t.shape[-1]
    pointer, is_f32, parts, stride = _branch(t, rows, ld, dtype, what)
    return pointer, is_f32, parts, stride, ld


def conv_silu(proj: torch.Tensor, col0: int, weight: torch.Tensor, bias: torch.Tensor, state: torch.Tensor | None,
              out: torch.Tensor, batch) -> None:
    """out[t, c] = silu(bias[c] + sum_j weight[c, j] x_(t - (taps - 1) + j)[c]) with x the columns col0 .. col0 + C of
    ``proj`` ([N, ld] in out's dtype or float32, or float32 partial sums [P, N, ld]): a causal convolution per
    channel whose last tap meets the token itself.  The inputs before a step's first token come from ``state``
    (float32 [slots, taps - 1, C], oldest first; zeros before a sequence's start), which then takes the step's last
    inputs.  weight float32 [C, taps], bias float32 [C]."""
    _gpu(proj, weight, bias, state, out)
    n, c = out.shape
    taps = weight.shape[1]
    _need(weight.dtype == torch.float32 and weight.shape == (c, taps) and bias.dtype == torch.float32 and bias.numel() == c,
          "the convolution's weight is float32 [channels, taps], its bias float32 [channels]")
    _need(1 <= taps <= SSM_MAX_TAPS, f"the convolution has 1 to {SSM_MAX_TAPS} taps")
    _need(taps == 1 or (state is not None and state.dtype == torch.float32 and tuple(state.shape[1:]) == (taps - 1, c)),
          "the convolution's state is float32 [slots, taps - 1, channels]")
    _need(batch.num_tokens == n, "the step's descriptor does not match")
    pointer, is_f32, parts, stride, ld = _ssm_in(proj, n, out.dtype, "projections")
    _need(0 <= col0 and col0 + c <= ld, "the convolution's channels lie outside the projections")
    _note(f"{n}x{c}x{taps}", n * c * (proj.element_size() * parts + out.element_size()))
    _check(_fn("ssm", "tk_conv_silu")(_code(out.dtype), pointer, is_f32, parts, stride, ld, int(col0), _p(weight), _p(bias),
                                      _p(state), _p(batch.q_start), _p(batch.state_slots), _p(out), batch.num_requests,
                                      c, taps, batch.max_q_len, _stream()), "conv_silu")


def ssd_column_splits(requests: int, heads: int, vdim: int, longest: int) -> int:
    """Blocks that share a head's value columns in the scan: one in steps of few tokens a request; in a long
    portion as many as give some 1,024 blocks, each with 8 columns or more (the columns never meet)."""
    if longest < SSM_SPLIT_FROM_TOKENS:
        return 1
    splits = 1
    while (requests * heads * splits < SSM_SPLIT_BLOCKS and vdim // (2 * splits) >= SSM_SPLIT_MIN_COLUMNS
           and vdim % (2 * splits) == 0):
        splits *= 2
    return splits


def ssd_scan(u: torch.Tensor, proj: torch.Tensor, dt_col: int, dt_bias: torch.Tensor, a_log: torch.Tensor,
             skip: torch.Tensor, state: torch.Tensor, y: torch.Tensor, batch, *, heads: int, groups: int, state_size: int,
             vdim: int) -> None:
    """Per request and head over the step's tokens in order: dt = softplus(proj[t, dt_col + head] + dt_bias),
    S <- exp(-exp(a_log) dt) S + dt B_t x_t^T, y_t = S^T C_t + skip x_t, with x, B, C the columns of ``u``
    ([N, heads * vdim + 2 groups * state_size], the convolution's output; head h reads group h // (heads / groups)),
    y float32 [N, heads * vdim] and the state S float32 [slots, heads, ceil(vdim / 4), state_size, 4] (kept; a head's
    value columns in groups of four, which is how the kernel's threads own them; columns behind vdim are zeros)."""
    _gpu(u, proj, dt_bias, a_log, skip, state, y)
    n = y.shape[0]
    c = heads * vdim + 2 * groups * state_size
    _need(heads % groups == 0 and u.shape == (n, c) and y.dtype == torch.float32 and y.shape == (n, heads * vdim),
          "the scan's operands do not match its sizes")
    _need(all(t.dtype == torch.float32 and t.numel() == heads for t in (dt_bias, a_log, skip)), "a head's constants are float32 [heads]")
    _need(state.dtype == torch.float32 and tuple(state.shape[1:]) == (heads, -(-vdim // 4), state_size, 4),
          "the state is float32 [slots, heads, ceil(vdim / 4), state, 4]")
    _need(1 <= vdim <= 1024 and 1 <= state_size <= 1024 and batch.num_tokens == n, "the scan takes sizes up to 1,024")
    pointer, is_f32, parts, stride, ld = _ssm_in(proj, n, u.dtype, "projections")
    _need(0 <= dt_col and dt_col + heads <= ld, "the step sizes lie outside the projections")
    # Long portions: chunks of SSM_CHUNK_TOKENS tokens side by side (a chunk acts on the state as S -> P S + L, with P
    # and L found from zeros; the chunks' start states follow from those in order; then every chunk runs again
    # from its own start and writes its outputs): twice the arithmetic of one walk, a thirtieth of its length.
    chunk = max_chunks = 0
    chunk_state = chunk_decay = None
    blocks = batch.num_requests
    if batch.max_q_len >= SSM_CHUNKS_FROM_TOKENS:
        chunk = SSM_CHUNK_TOKENS
        max_chunks = -(-batch.max_q_len // chunk)
        blocks = n // chunk + batch.num_requests        # (no step has more chunks than this)
        chunk_state = torch.empty((blocks, heads, -(-vdim // 4), state_size, 4), dtype=torch.float32, device=y.device)
        chunk_decay = torch.empty((blocks, heads), dtype=torch.float32, device=y.device)
    splits = ssd_column_splits(blocks, heads, vdim, batch.max_q_len)
    _note(f"{n}x{heads}x{state_size}x{vdim}", n * (c * u.element_size() + heads * vdim * 4), 6.0 * n * heads * state_size * vdim)
    _check(_fn("ssm", "tk_ssd_scan")(_code(u.dtype), _p(u), pointer, is_f32, parts, stride, ld, int(dt_col), _p(dt_bias),
                                     _p(a_log), _p(skip), _p(state), _p(batch.q_start), _p(batch.state_slots), _p(y),
                                     batch.num_requests, heads, groups, state_size, vdim, splits, chunk, max_chunks,
                                     _p(chunk_state), _p(chunk_decay), _stream()), "ssd_scan")


def gated_group_norm(y: torch.Tensor, proj: torch.Tensor, z_col: int, weight: torch.Tensor, out: torch.Tensor, *,
                     groups: int, eps: float) -> None:
    """g = y * silu(z) with z the columns z_col .. z_col + inner of ``proj``; out = g / rms(g) * weight, the root
    mean square taken over each of ``groups`` equal parts of the row.  y float32 [N, inner], weight float32 [inner]."""
    _gpu(y, proj, weight, out)
    n, inner = out.shape
    _need(y.dtype == torch.float32 and y.shape == (n, inner) and weight.dtype == torch.float32 and weight.numel() == inner
          and groups >= 1 and inner % groups == 0, "the gated norm's operands do not match")
    pointer, is_f32, parts, stride, ld = _ssm_in(proj, n, out.dtype, "projections")
    _need(0 <= z_col and z_col + inner <= ld, "the gate lies outside the projections")
    _note(f"{n}x{inner}/{groups}", n * inner * (4 + proj.element_size() * parts + out.element_size()))
    _check(_fn("ssm", "tk_gated_group_norm")(_code(out.dtype), _p(y), pointer, is_f32, parts, stride, ld, int(z_col),
                                             _p(weight), _p(out), n, inner, groups, float(eps), _stream()), "gated_group_norm")


MOE_LDS_BYTES = 96 * 1024      # of a row of activations in float32 that a block of the expert kernels stages


def moe_route(h: torch.Tensor, router: torch.Tensor, chosen: torch.Tensor, weight: torch.Tensor, top: int,
              scoring: str = "sigmoid", *, correction: torch.Tensor | None = None, groups: tuple[int, int] | None = None,
              normalise: bool = False, scale: float = 1.0) -> None:
    """Per token the ``top`` experts with the largest scores, float32 throughout: the scores are
    sigmoid(router . h), or with ``scoring="softmax"`` the softmax of router . h over all experts;
    chosen [N, top] int32 (largest first, the lower index on ties), weight [N, top] float32 their scores.
    ``correction`` (float32 [experts]): the choice goes by score + correction, the weights stay the scores.
    ``groups`` = (count, keep): the experts form ``count`` equal groups of neighbours, a group's score is the
    sum of its two largest choice scores, and only experts of the ``keep`` best groups can be chosen.
    ``normalise``: the chosen weights are divided by their sum (+ 1e-20); then all are multiplied by ``scale``."""
    _need(scoring in ("sigmoid", "softmax"), "the router's scores are sigmoids or a softmax")
    _gpu(h, router, chosen, weight, correction)
    n, w = h.shape
    e = router.shape[0]
    _need(router.dtype == torch.float32 and router.shape == (e, w), "the router is float32 [experts, width]")
    _need(1 <= top <= e and chosen.dtype == torch.int32 and weight.dtype == torch.float32
          and chosen.numel() >= n * top and weight.numel() >= n * top, "lists of chosen experts too small")
    _need(correction is None or (correction.dtype == torch.float32 and correction.numel() == e),
          "the correction is float32 [experts]")
    count, keep = groups or (0, 0)
    if groups:
        _need(count >= 1 and e % count == 0 and 1 <= keep <= count and keep * (e // count) >= top,
              "groups divide the experts evenly and the kept ones hold at least `top` experts")
    _check(_fn("moe", "tk_moe_route")(_code(h.dtype), _p(h), _p(router), _p(chosen), _p(weight), n, w, e, top,
                                      int(scoring == "softmax"), _p(correction), int(count), int(keep),
                                      int(bool(normalise)), float(scale), _stream()), "moe_route")


def moe_gate_up(h: torch.Tensor, gate_up: torch.Tensor, chosen: torch.Tensor, weight: torch.Tensor, act: torch.Tensor,
                top: int, weight_on_output: bool = False) -> None:
    """act[n * top + k] = silu(w gate_e h[n]) * (w up_e h[n]) for the token's k-th chosen expert e with
    weight w; gate_up [experts, 2 ff, width] holds an expert's gate rows, then its up rows.
    ``weight_on_output``: w * silu(gate_e h[n]) * (up_e h[n]) instead, so that the second product, which
    is linear, yields w times the expert's output."""
    _gpu(h, gate_up, chosen, weight, act)
    n, w = h.shape
    e, two_f, w2 = gate_up.shape
    f = two_f // 2
    _need(w2 == w and two_f % 2 == 0 and gate_up.dtype == h.dtype == act.dtype, "expert weights do not match the activations")
    _need(act.shape == (n * top, f) and chosen.numel() >= n * top and weight.numel() >= n * top, "expert activations too small")
    _need(w * 4 <= MOE_LDS_BYTES, "a row of activations must fit LDS")
    _note(f"{n}x{top} {two_f}x{w}", min(n * top, e) * two_f * w * h.element_size(), 2.0 * n * top * two_f * w)
    _check(_fn("moe", "tk_moe_gate_up")(_code(h.dtype), _p(h), _p(gate_up), _p(chosen), _p(weight), _p(act), n, w, f, top,
                                        int(bool(weight_on_output)), _stream()), "moe_gate_up")


def moe_down(act: torch.Tensor, down: torch.Tensor, chosen: torch.Tensor, out: torch.Tensor, top: int) -> None:
    """out[k, n] = down_e act[n * top + k] for the token's k-th chosen expert e; out float32 [top, N, width]:
    partial sums that the next kernel adds in order."""
    _gpu(act, down, chosen, out)
    e, w, f = down.shape
    n = out.shape[1]
    _need(act.shape == (n * top, f) and act.dtype == down.dtype and out.dtype == torch.float32 and out.shape == (top, n, w),
          "expert outputs do not match")
    _need(f * 4 <= MOE_LDS_BYTES, "a row of expert activations must fit LDS")
    _note(f"{n}x{top} {w}x{f}", min(n * top, e) * w * f * act.element_size(), 2.0 * n * top * w * f)
    _check(_fn("moe", "tk_moe_down")(_code(act.dtype), _p(act), _p(down), _p(chosen), _p(out), n, w, f, top, _stream()),
           "moe_down")


MOE_TILE_PAIRS = 64        # pairs of one expert that a block of the grouped products takes (csrc/moe.hip: kTilePairs)
MOE_GROUPED_FROM = 65      # pairs of a step from which the experts' products run grouped on the matrix cores


def moe_grouped_fits(h: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, pairs: int) -> bool:
    """Whether a step's expert products take the grouped form: bfloat16, enough pairs, rows that
    fill 16-byte pieces, and few enough experts for the one block that lists the pairs."""
    f = down.shape[2]
    return (h.dtype == torch.bfloat16 and pairs >= MOE_GROUPED_FROM and h.shape[1] % 8 == 0 and f % 8 == 0
            and gate_up.shape[0] <= 4096)


def moe_sort(chosen: torch.Tensor, num_experts: int, tile_pairs: int = MOE_TILE_PAIRS):
    """The step's (token, expert) pairs listed expert by expert and cut into tiles of up to
    ``tile_pairs``: (order, tile_expert, tile_start, tile_count, num_tiles, tile_pairs), int32 on the device."""
    _gpu(chosen)
    pairs = chosen.numel()
    _need(tile_pairs == MOE_TILE_PAIRS, "tiles hold 64 pairs")
    max_tiles = pairs // tile_pairs + num_experts
    lists = torch.empty(pairs + 3 * max_tiles + 1, dtype=torch.int32, device=chosen.device)
    order, rest = lists[:pairs], lists[pairs:]
    tile_expert, tile_start, tile_count = (rest[i * max_tiles:(i + 1) * max_tiles] for i in range(3))
    num_tiles = rest[3 * max_tiles:]
    _need(chosen.dtype == torch.int32, "lists of chosen experts are int32")
    _check(_fn("moe", "tk_moe_sort")(_p(chosen), pairs, num_experts, tile_pairs, _p(order), _p(tile_expert), _p(tile_start),
                                     _p(tile_count), _p(num_tiles), _stream()), "moe_sort")
    return order, tile_expert, tile_start, tile_count, num_tiles, tile_pairs


def moe_grouped(x: torch.Tensor, weights: torch.Tensor, lists: tuple, pair_weight: torch.Tensor | None,
                out: torch.Tensor, *, tokens: int, top: int, gated: bool, weight_on_output: bool = False) -> None:
    """One of the experts' two products over the tiles of ``lists`` (``moe_sort``), bfloat16 on the matrix
    cores.  ``gated``: x [tokens, K] the tokens' rows, weights [E, 2 R, K] (gate rows, then up rows), out
    bfloat16 [tokens * top, R] = silu(w g) * (w u) with the pairs' weights w (``weight_on_output``:
    w * silu(g) * u).  Else: x [tokens * top, K] the
    pairs' rows, weights [E, R, K], out float32 [top, tokens, R]."""
    order, tile_expert, tile_start, tile_count, num_tiles, tile_pairs = lists
    _gpu(x, weights, pair_weight, out)
    k = x.shape[1]
    e = weights.shape[0]
    r = weights.shape[1] // (2 if gated else 1)
    _need(x.dtype == weights.dtype == torch.bfloat16 and weights.shape[2] == k and k % 8 == 0, "grouped expert products are bfloat16 with rows of 16-byte pieces")
    _need(order.numel() == tokens * top and x.shape[0] == (tokens if gated else tokens * top), "the pairs' list does not match")
    if gated:
        _need(out.dtype == torch.bfloat16 and out.shape == (tokens * top, r) and pair_weight is not None
              and pair_weight.dtype == torch.float32 and pair_weight.numel() >= tokens * top, "gated output does not match")
    else:
        _need(out.dtype == torch.float32 and out.shape == (top, tokens, r), "the pairs' outputs are float32 [top, tokens, width]")
    _note(f"{tokens}x{top} {weights.shape[1]}x{k}", min(tokens * top, e) * weights.shape[1] * k * 2, 2.0 * tokens * top * weights.shape[1] * k)
    _check(_fn("moe", "tk_moe_grouped")(
        (2 if weight_on_output else 1) if gated else 0, _p(x), _p(weights), _p(order), _p(tile_expert), _p(tile_start), _p(tile_count), _p(num_tiles),
        _p(pair_weight), _p(out), tokens, top, r, k, tile_expert.numel(), tokens * top, tile_pairs, _stream()), "moe_grouped")


FEWROWS_MAX_ROWS = 64          # float32 products of up to this many rows stream the weights, a lane a weight row,
FEWROWS_GROUP = 16             # this many rows a pass over the weights
FEWROWS_SPLIT_BELOW = 65536    # weight rows below which every piece of 256 k gets a wave of its own


def fewrows_pays(m: int, n: int) -> bool:
    """Whether ``m`` rows stream the weights (one pass per FEWROWS_GROUP rows) rather than take
    the tiled kernel in tiles of 64 x 64, which reads the weights once but needs a block for
    every CU to be worth it: measured on the shapes of an 8B-shaped layer, the tiled kernel wins
    from 24 rows where it has a thousand tiles (the logits head at 64 rows: 4.7 -> 1.6 ms) and
    from 48 where it has one a CU (gate/up: 546 -> 303 us); a matrix of 4,096 rows never."""
    tiles = -(-n // 64)
    if m >= 48 and tiles >= 256:
        return False
    if m >= 24 and tiles >= 1024:
        return False
    return True


def gemm_tiled(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, fewrows_split: bool | None = None) -> None:
    """out[M, N] = a[M, K] @ w[N, K]^T, float32 multiply-add (rows may be strided).  float32
    operands of up to 64 rows go to the weight-streaming kernel where that pays
    (``fewrows_pays``), which gives the same bits (``fewrows_split``: that kernel with a wave
    per piece of K or not; None chooses the kernel and the split by the shape)."""
    for t in (a, w, out):
        _need(t.is_cuda and t.dim() == 2 and t.stride(1) == 1, "gemm operands are 2-D GPU tensors with unit inner stride")
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k and out.shape == (m, n), f"gemm shapes disagree: {tuple(a.shape)} x {tuple(w.shape)}^T -> {tuple(out.shape)}")
    _need(a.dtype == w.dtype, "gemm inputs must share a dtype")
    _need(m <= 64 * 65535, "too many rows for one launch")
    _note(f"{m}x{n}x{k}", (n * k + m * k) * a.element_size() + m * n * out.element_size(), 2.0 * m * n * k)
    if (m <= FEWROWS_MAX_ROWS and (fewrows_split is not None or fewrows_pays(m, n))
            and a.dtype == torch.float32 and out.dtype == torch.float32 and k % 4 == 0 and k >= 4
            and a.stride(0) % 4 == 0 and w.stride(0) % 4 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        # the same sums in the same order, by a kernel that streams the weights; a wave for every
        # piece of K where the matrix has too few rows to fill the GPU with a wave per 64 of them
        pieces = -(-k // 256)
        split = fewrows_split if fewrows_split is not None else (n < FEWROWS_SPLIT_BELOW and pieces > 1)
        for at in range(0, m, FEWROWS_GROUP):
            rows = min(FEWROWS_GROUP, m - at)
            partial = torch.empty((pieces, rows, n), dtype=torch.float32, device=a.device) if split else None
            _check(_fn("gemm_tiled", "tk_gemm_fewrows")(_p(a[at:]), _p(w), _p(out[at:]), _p(partial),
                                                        rows, n, k, a.stride(0), w.stride(0), out.stride(0), _stream()),
                   "gemm_fewrows")
        return
    _check(_fn("gemm_tiled", "tk_gemm_tiled")(_code(a.dtype), _code(out.dtype), _p(a), _p(w), _p(out),
                                              m, n, k, a.stride(0), w.stride(0), out.stride(0),
                                              _stream()), "gemm_tiled")


STREAM_MAX_ROWS = 128     # rows of activations the streaming product takes (more than 64: eight-wave blocks, not the gated form)
STREAM_SMALL_MATRIX_BYTES = 20 << 20   # below this a product's time is memory round trips, not bytes


def stream_waves(rows: int, k: int, gated: bool = False, n: int = 0) -> int:
    """Waves a block of the streaming product.  Eight waves share a chunk of the
    activations (the block then owns 128 weight rows, or 64 output columns of the gated
    product), which pays from 33 rows of activations on, where that chunk is as large as a
    block's weights, unless the matrix is small (blocks of four are spread over more CUs) or
    has so many rows (``n``: the logits head) that blocks of four already queue several deep
    on every CU.

    The gated product cannot split K, so the size of its blocks is all that spreads it over
    the GPU: two waves (16 output columns) with up to 16 rows of activations, and with more
    while the matrix is small; then four, then eight, as the activations' chunk that every
    block loads for itself grows against its weights.  Weight rows a multiple of 8 KB long
    take four waves where two would do: twice as many row tiles in flight at equal offsets
    meet the same memory channels (gate/up of an 8B-shaped layer, K = 4096, at 8 rows: 38 us
    with two waves, 34 with four; with K = 3840 or 4352 two waves are 9 % ahead).  Measured on
    the shapes of 0.6B to 32B models at 1 to 64 rows: two waves gain 5 to 20 % where chosen.

    Where eight waves are the rule, six (96 weight rows a block) are taken instead if the blocks
    then fill the CUs better: one block of either size runs on a CU at a time, so the gated
    product takes the size whose rounds of blocks times rows a block is smaller (gate/up of an
    8B-shaped layer: 192 blocks of eight leave a quarter of the CUs idle, 256 blocks of six none:
    44 -> 42 us at 64 rows; 4B 29.6 -> 26.9, 14B 107 -> 94; at 32B three rounds of six lose to two
    of eight), and the plain product six only if, with the best split of K for each, one round of
    them covers a tenth more of the CUs (q/k/v of 8B: 64 x 4 blocks against 48 x 4)."""
    if rows > 64:
        return 8        # five to eight tiles of 16 rows: only blocks of eight waves are built for them
    if gated:
        if rows <= 16:
            waves = 2
        elif rows <= 32:
            waves = 2 if n < 10240 else 4
        elif rows <= 48:
            waves = 2 if n < 8192 else 8
        else:
            waves = 2 if n < 4096 else 4 if n < 8192 else 8
        if waves == 2 and (2 * k) % 8192 == 0:
            waves = 4
        if waves == 8 and _rounds(n, 8 * 6) * 6 < _rounds(n, 8 * 8) * 8:
            waves = 6
        return waves
    if rows > 32 and n <= 256 * 128 and 2 * n * k >= STREAM_SMALL_MATRIX_BYTES:
        return 6 if stream_fill(n, k, 6)[0] >= 1.1 * stream_fill(n, k, 8)[0] else 8
    return 4


STREAM_CUS = 256    # blocks of six or eight waves that run at once: one a CU


def _rounds(n: int, columns: int) -> int:
    return -(-(-(-n // columns)) // STREAM_CUS)


def stream_fill(n: int, k: int, waves: int) -> tuple[float, int]:
    """(share of the CUs that one round of ``waves``-wave blocks covers, shares of K that do it):
    the split of K, of at least two chunks of 256 a share, whose blocks come closest to one a CU
    without exceeding it."""
    blocks = -(-n // (16 * waves))
    chunks = -(-k // 256)
    best, best_splits = min(blocks, STREAM_CUS), 1
    for per in range(2, chunks + 1):
        splits = -(-chunks // per)
        if best < blocks * splits <= STREAM_CUS:
            best, best_splits = blocks * splits, splits
    return best / STREAM_CUS, best_splits


def _row_scale(sumsq: torch.Tensor | None, m: int, what: str) -> int:
    """Checks the rows' sums of squares [slabs, M] that a product scales its result by; slabs."""
    if sumsq is None:
        return 0
    _gpu(sumsq)
    _need(sumsq.dtype == torch.float32 and sumsq.dim() == 2 and sumsq.shape[1] == m and sumsq.shape[0] >= 1
          and m <= ROW_SCALE_MAX_ROWS and sumsq.shape[0] <= ROW_SCALE_MAX_SLABS,
          f"{what}: the rows' sums of squares are float32 [slabs <= {ROW_SCALE_MAX_SLABS}, M <= {ROW_SCALE_MAX_ROWS}]")
    return sumsq.shape[0]


def gemm_stream(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, *, splits: int = 1, waves: int = 0,
                sumsq: torch.Tensor | None = None, eps: float = 0.0) -> int:
    """out = a[M, K] @ w[N, K]^T for M <= 64 with the LDS-staged weight-streaming
    MFMA kernel (``waves``: 4, 6 or 8 waves a block; 0 chooses by the shape).  ``splits == 1``: out is
    [M, N], bfloat16 or float32.  More:
    out is float32 [splits, M, N] and receives partial sums; returns how many of
    them were written (the reader adds out[:returned]).  ``sumsq`` [slabs, M] (M <= 16): row m
    of the result is multiplied by rsqrt(sum_s sumsq[s, m] / K + eps): ``a`` is then
    bf16(x * gamma) of an RMSNorm and ``sumsq`` the sums of squares of x's rows over slabs of
    columns (``gemm_wholek_add`` leaves both)."""
    for t in (a, w):
        _need(t.is_cuda and t.dim() == 2 and t.stride(1) == 1, "gemm operands are 2-D GPU tensors with unit inner stride")
    m, k = a.shape
    n = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "the streaming product takes bfloat16 inputs")
    _need(w.shape[1] == k, "gemm shapes disagree")
    waves = waves or stream_waves(m, k, False, n)
    _need(0 < m <= (STREAM_MAX_ROWS if waves == 8 else 64) and k >= 8 and k % 8 == 0 and a.stride(0) % 8 == 0
          and w.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0,
          "streaming product needs M <= 64 (128 with eight waves) and 16-byte aligned rows")
    _need(out.is_cuda and out.stride(-1) == 1, "output must be a GPU tensor with unit inner stride")
    if splits == 1:
        _need(out.shape == (m, n), "output must be [M, N]")
        ldc, stride = out.stride(0), 0
    else:
        _need(1 < splits <= 64 and out.dtype == torch.float32 and out.shape == (splits, m, n) and out.is_contiguous(),
              "with splits the output is contiguous float32 [splits, M, N]")
        ldc, stride = n, m * n
    slabs = _row_scale(sumsq, m, "gemm_stream")
    _note(f"{m}x{n}x{k}", (n * k + m * k) * 2 + splits * m * n * out.element_size(), 2.0 * m * n * k)
    used = _fn("gemm_mfma", "tk_gemm_stream")(_code(out.dtype), _p(a), _p(w), _p(out), m, n, k, a.stride(0),
                                              w.stride(0), ldc, splits, stride, waves,
                                              _p(sumsq), slabs, float(eps), _stream())
    if used < 1:
        raise KernelError(f"gemm_stream failed with status {used}")
    return used


def gemm_stream_swiglu(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, *, waves: int = 0,
                       sumsq: torch.Tensor | None = None, eps: float = 0.0, activation: str = "silu") -> None:
    """out[M, I] = act(a @ w[:I]^T) * (a @ w[I:]^T) for M <= 64: the gate and up
    projections and the gate product in one weight-streaming kernel (bfloat16); act is silu or the tanh
    form of gelu.  ``sumsq``, ``eps``: the rows' scale, applied to both products before the gate, as in
    ``gemm_stream``."""
    _need(activation in GATE_ACTIVATIONS, f"the gate's activation is one of {sorted(GATE_ACTIVATIONS)}")
    for t in (a, w, out):
        _need(t.is_cuda and t.dim() == 2 and t.stride(1) == 1, "gemm operands are 2-D GPU tensors with unit inner stride")
    m, k = a.shape
    _need(w.shape[0] % 2 == 0 and w.shape[1] == k and out.shape == (m, w.shape[0] // 2), "gated product shapes disagree")
    _need(a.dtype == w.dtype == out.dtype == torch.bfloat16, "the gated product is bfloat16")
    waves = waves or stream_waves(m, k, True, w.shape[0] // 2)
    _need(0 < m <= 64 and k >= 8 and k % 8 == 0 and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
          and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0, "gated product needs M <= 64 and 16-byte aligned rows")
    slabs = _row_scale(sumsq, m, "gemm_stream_swiglu")
    _note(f"{m}x{w.shape[0]}x{k}", (w.shape[0] * k + m * k) * 2 + m * w.shape[0], 2.0 * m * w.shape[0] * k)
    _check(_fn("gemm_mfma", "tk_gemm_stream_swiglu")(_p(a), _p(w), _p(out), m, w.shape[0] // 2, k, a.stride(0),
                                                     w.stride(0), out.stride(0), waves,
                                                     _p(sumsq), slabs, float(eps), GATE_ACTIVATIONS[activation],
                                                     _stream()), "gemm_stream_swiglu")


WHOLEK_MAX_ROWS = 16    # rows of activations that the whole-K product takes
ROW_SCALE_MAX_ROWS = 16  # rows up to which the streaming product applies a pending row scale
ROW_SCALE_MAX_SLABS = 512  # ... and slabs of sums of squares it takes (csrc/gemm_mfma.hip: 16 * kRowScaleLoads)


def wholek_waves(n: int, k: int, gated: bool = False) -> int:
    """Waves a block of the whole-K product: they split K in chunks of 256."""
    chunks = -(-k // 256)
    if gated:
        return 4 if chunks <= 16 else 8
    return 16 if chunks >= 16 else 8 if chunks >= 8 else 4


def _wholek_operands(a, w, what):
    for t in (a, w):
        _need(t.is_cuda and t.dim() == 2 and t.stride(1) == 1 and t.dtype == torch.bfloat16,
              f"{what}: operands are 2-D bfloat16 GPU tensors with unit inner stride")
    m, k = a.shape
    _need(w.shape[1] == k, f"{what}: shapes disagree")
    _need(0 < m <= WHOLEK_MAX_ROWS and k >= 8 and k % 8 == 0 and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
          and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0,
          f"{what} needs M <= {WHOLEK_MAX_ROWS}, K a multiple of 8 and 16-byte aligned rows")
    return m, k


def gemm_wholek(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, *, sumsq: torch.Tensor | None = None,
                eps: float = 0.0, gated: bool = False, waves: int = 0) -> None:
    """out[M, N] = (a[M, K] @ w[N, K]^T) * rstd for M <= 16, every block holding the whole of K
    for its 16 columns (no partial sums).  ``sumsq`` [slabs, M] float32: sums of squares of the
    rows of the stream that ``a`` was made from, over slabs of its columns; then
    rstd[m] = rsqrt(sum_s sumsq[s, m] / K + eps) (an RMSNorm whose weight is already in ``a``);
    without it rstd = 1.  ``gated``: w = [gate; up] of 2N rows and out = silu(.) * (.), bfloat16."""
    m, k = _wholek_operands(a, w, "gemm_wholek")
    n = w.shape[0] // 2 if gated else w.shape[0]
    _need(not gated or (w.shape[0] % 2 == 0 and out.dtype == torch.bfloat16), "the gated product has 2N weight rows and a bfloat16 result")
    _need(out.is_cuda and out.dim() == 2 and out.stride(1) == 1 and out.shape == (m, n), "output must be [M, N] on the GPU")
    if sumsq is not None:
        _gpu(sumsq)
        _need(sumsq.dtype == torch.float32 and sumsq.dim() == 2 and sumsq.shape[1] == m and sumsq.shape[0] >= 1,
              "the rows' sums of squares are float32 [slabs, M]")
    _note(f"{m}x{w.shape[0]}x{k}", (w.shape[0] * k + m * k) * 2 + m * n * out.element_size(), 2.0 * m * w.shape[0] * k)
    _check(_fn("gemm_wholek", "tk_gemm_wholek")(
        _code(out.dtype), int(gated), _p(a), _p(w), _p(out), m, n, k, a.stride(0), w.stride(0), out.stride(0),
        _p(sumsq), 0 if sumsq is None else sumsq.shape[0], float(eps), waves or wholek_waves(n, k, gated), _stream()),
        "gemm_wholek")


def gemm_wholek_add(a: torch.Tensor, w: torch.Tensor, resid: torch.Tensor, gamma: torch.Tensor | None = None,
                    *, waves: int = 0) -> tuple[torch.Tensor, torch.Tensor | None]:
    """resid[M, N] += a[M, K] @ w[N, K]^T (float32 stream, M <= 16) in the product's own kernel.
    Returns (sumsq, scaled): sumsq float32 [N/16, M], the sums of squares of every row of the new
    stream over slabs of 16 columns, and, given ``gamma`` [N] (the weight of the norm that reads
    the stream next), scaled = bf16(resid * gamma) [M, N]: what ``gemm_wholek`` takes."""
    m, k = _wholek_operands(a, w, "gemm_wholek_add")
    n = w.shape[0]
    _need(resid.is_cuda and resid.dtype == torch.float32 and resid.shape == (m, n) and resid.stride(1) == 1
          and n % 4 == 0 and resid.stride(0) % 4 == 0 and resid.data_ptr() % 16 == 0,
          "the stream is float32 [M, N], N a multiple of 4, rows 16-byte aligned")
    scaled = None
    if gamma is not None:
        _gpu(gamma)
        _need(gamma.dtype == torch.float32 and gamma.numel() == n and gamma.data_ptr() % 16 == 0, "the norm weight is float32 [N]")
        scaled = torch.empty((m, n), dtype=torch.bfloat16, device=a.device)
    sumsq = torch.empty((-(-n // 16), m), dtype=torch.float32, device=a.device)
    _note(f"{m}x{n}x{k}", (n * k + m * k) * 2 + m * n * 10, 2.0 * m * n * k)
    _check(_fn("gemm_wholek", "tk_gemm_wholek_add")(
        _p(a), _p(w), m, n, k, a.stride(0), w.stride(0), _p(resid), resid.stride(0), _p(gamma), _p(scaled),
        0 if scaled is None else scaled.stride(0), _p(sumsq), waves or wholek_waves(n, k), _stream()), "gemm_wholek_add")
    return sumsq, scaled


LT_WORKSPACE_BYTES = 128 << 20
LT_TUNE_CANDIDATES = 16     # of the library's candidates, timed once per shape class when tuning is on
_lt_workspace: dict[torch.device, torch.Tensor] = {}
_lt_tune = 1                # 1: take the library's first choice (the same in every process)


def set_library_tuning(on: bool) -> None:
    """Whether the library product times its candidate algorithms for each new shape
    class and keeps the fastest.  Off (the default) every process takes the library's
    first choice, so identical input gives identical bits from run to run; on, prompt
    portions run up to 2x faster on some shapes, the choice depends on timing noise, and
    the first step that meets a new shape class pays for some 60 extra products."""
    global _lt_tune
    _lt_tune = LT_TUNE_CANDIDATES if on else 1


if __import__("os").environ.get("TOKAMAK_AMD_LT_TUNE", "") not in ("", "0"):
    _lt_tune = LT_TUNE_CANDIDATES


def gemm_library(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> bool:
    """out[M, N] = a[M, K] @ w[N, K]^T through hipBLASLt (bf16 in and out, float32
    accumulation), for prompt portions too long for the weight-streaming kernels.
    The plan of each shape is kept; the algorithm is the library's first choice, or with
    ``set_library_tuning(True)`` the fastest of its candidates, timed once per shape class
    (csrc/blas_lt.hip; that synchronises, so the call must not be recorded into a graph).  All calls on a
    device share one workspace: launch them on one stream at a time (the engine has one).
    Returns False if the library has no algorithm for the shape (nothing was computed)."""
    for t in (a, w, out):
        _need(t.is_cuda and t.dim() == 2 and t.stride(1) == 1, "gemm operands are 2-D GPU tensors with unit inner stride")
        _need(t.dtype == torch.bfloat16 and t.data_ptr() % 16 == 0, "the library product is bfloat16 with 16-byte aligned operands")
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k and out.shape == (m, n), "gemm shapes disagree")
    ws = _lt_workspace.get(a.device)
    if ws is None:
        ws = _lt_workspace[a.device] = torch.empty(LT_WORKSPACE_BYTES, dtype=torch.uint8, device=a.device)
    _note(f"{m}x{n}x{k}", (n * k + m * k + m * n) * 2, 2.0 * m * n * k)
    status = _fn("blas_lt", "tk_lt_gemm")(_p(a), _p(w), _p(out), m, n, k, a.stride(0), w.stride(0), out.stride(0),
                                          _p(ws), ws.numel(), _lt_tune, _stream())
    if status == -2:
        return False
    _check(status, "gemm_library")
    return True


def gemm_skinny(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, *, row_tiles: int, waves: int) -> None:
    """out[M, N] = a[M, K] @ w[N, K]^T on the matrix cores for M <= 64 (bf16 in,
    float32 accumulation, bf16 or float32 out).  ``row_tiles`` (1 or 2) tiles of
    16 weight rows per block; ``waves`` (1..16) waves of a block split K."""
    for t in (a, w, out):
        _need(t.is_cuda and t.dim() == 2 and t.stride(1) == 1, "gemm operands are 2-D GPU tensors with unit inner stride")
    m, k = a.shape
    n = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "the skinny product takes bfloat16 inputs")
    _need(w.shape[1] == k and out.shape == (m, n), "gemm shapes disagree")
    _need(0 < m <= 64 and k >= 8 and k % 8 == 0 and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
          and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0, "skinny product needs M <= 64 and 16-byte aligned rows")
    _need(row_tiles in (1, 2, 4) and 1 <= waves <= 16, "row_tiles in (1, 2, 4), waves in 1..16")
    _note(f"{m}x{n}x{k}", (n * k + m * k) * 2 + m * n * out.element_size(), 2.0 * m * n * k)
    _check(_fn("gemm_mfma", "tk_gemm_skinny")(_code(out.dtype), _p(a), _p(w), _p(out), m, n, k, a.stride(0),
                                              w.stride(0), out.stride(0), row_tiles, waves, _stream()), "gemm_skinny")


def latent_prepare(proj: torch.Tensor, latent_weight: torch.Tensor | None, cos: torch.Tensor | None,
                   sin: torch.Tensor | None, positions: torch.Tensor, req_of_token: torch.Tensor,
                   block_tables: torch.Tensor, q_plain: torch.Tensor, q_full: torch.Tensor,
                   k_cache: torch.Tensor | None, v_cache: torch.Tensor | None, *, num_heads: int, head_dim: int,
                   rot_dim: int, rank: int, rotary_dim: int, interleaved: bool, page_size: int, eps: float,
                   store: bool = True, q_weight: torch.Tensor | None = None) -> None:
    """From a token's projections [q heads of (head_dim unrotated | rot_dim rotated) | latent of ``rank`` |
    one key part of rot_dim] (the last two only with ``store``): the unrotated query parts to q_plain
    [N, heads, head_dim]; the rotated ones into q_full[n, a, rank : rank + rot_dim] (q_full is [N, heads,
    padded key size]; its first ``rank`` channels are left for the query carried into the latent's space);
    the latent divided by its root mean square (``eps``) times ``latent_weight`` and the rotated key part
    into the K page as one key [latent | rotated part], the latent also into the V page.  ``q_weight``
    (float32 [head_dim]): the unrotated part of every query unit is divided by its root mean square (``eps``)
    and multiplied by it first (a query that is itself a normed latent); ``q_full`` may then be None if
    nothing is rotated."""
    _gpu(proj, latent_weight, cos, sin, positions, req_of_token, block_tables, q_plain, q_full, k_cache, v_cache, q_weight)
    _need(q_weight is None or (q_weight.dtype == torch.float32 and q_weight.numel() == head_dim),
          "the query norm's weight is float32 [head_dim]")
    _need(q_full is not None or (q_weight is not None and rot_dim == 0), "q_full may be absent only for a normed, unrotated query")
    n = positions.numel()
    qw = head_dim + rot_dim
    width = num_heads * qw + (rank + rot_dim if store else 0)
    in_f32, parts, stride = _partials(proj, n, width, q_plain.dtype, "projections")
    hdp, vdp = padded_sizes(rank + rot_dim, rank)
    _need(max(qw, rank + rot_dim) <= 1024 and max(hdp, vdp) <= 512, "heads of up to 1,024 and keys of up to 512 channels")
    _need(q_plain.numel() >= n * num_heads * head_dim
          and (q_full is None or (q_plain.dtype == q_full.dtype and q_full.numel() >= n * num_heads * hdp)),
          "q_plain / q_full too small")
    _need(rotary_dim % 2 == 0 and 0 <= rotary_dim <= rot_dim and page_size % 8 == 0, "rotary_dim is even and at most rot_dim")
    _need(rotary_dim == 0 or (cos is not None and sin is not None and cos.dtype == torch.float32
                               and sin.dtype == torch.float32 and cos.numel() >= n * (rotary_dim // 2)
                               and sin.numel() >= n * (rotary_dim // 2)), "rotary tables missing, not float32 or too small")
    _need(positions.dtype == torch.int32 and req_of_token.dtype == torch.int32 and req_of_token.numel() >= n
          and block_tables.dtype == torch.int32 and block_tables.dim() == 2, "descriptor arrays are int32")
    if store:
        _need(latent_weight is not None and latent_weight.dtype == torch.float32 and latent_weight.numel() == rank,
              "the latent's norm weight is float32 [rank]")
        _need(k_cache is not None and v_cache is not None and k_cache.dtype == q_plain.dtype == v_cache.dtype
              and k_cache.numel() % (hdp * page_size) == 0 and v_cache.numel() % (vdp * page_size) == 0
              and k_cache.numel() // hdp == v_cache.numel() // vdp, "cache size is not whole pages")
    _note(f"{n}x{width}", n * width * (proj.element_size() * parts + q_plain.element_size()))
    _check(_fn("latent", "tk_latent_prepare")(
        _code(q_plain.dtype), _p(proj), in_f32, parts, stride, _p(latent_weight), _p(q_weight), _p(cos), _p(sin), _p(positions),
        _p(req_of_token), _p(block_tables), _p(q_plain), _p(q_full), _p(k_cache if store else None),
        _p(v_cache if store else None), n, num_heads, head_dim, rot_dim, rank, hdp, vdp, rotary_dim,
        int(bool(interleaved)), page_size, block_tables.shape[1], float(eps), int(bool(store)), _stream()), "latent_prepare")


def head_linear(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor) -> None:
    """out[n, a, :] = weight[a] @ x[n, a, :]: a product per head.  x [N, heads, K] and out [N, heads, M] may
    be views with strides between rows and heads (the last dimension dense); weight [heads, M, K] is dense."""
    _need(x.is_cuda and weight.is_cuda and out.is_cuda, "kernel arguments must live on the GPU (there is no CPU path)")
    _need(x.dim() == 3 and out.dim() == 3 and weight.dim() == 3 and weight.is_contiguous(), "operands are [N, heads, K], [heads, M, K], [N, heads, M]")
    n, heads, k = x.shape
    m = weight.shape[1]
    _need(weight.shape == (heads, m, k) and out.shape == (n, heads, m), "head_linear shapes disagree")
    _need(x.dtype == weight.dtype == out.dtype and x.stride(2) == 1 and out.stride(2) == 1, "one dtype, dense last dimension")
    if n == 0:
        return
    _note(f"{n}x{heads} {m}x{k}", (weight.numel() + x.numel() + out.numel()) * x.element_size(), 2.0 * n * heads * m * k)
    _check(_fn("latent", "tk_head_linear")(_code(x.dtype), _p(x), x.stride(0), x.stride(1), _p(weight), _p(out),
                                           out.stride(0), out.stride(1), n, heads, m, k, _stream()), "head_linear")


def paged_attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            block_tables: torch.Tensor, positions: torch.Tensor,
                            req_of_token: torch.Tensor, out: torch.Tensor, *, num_heads: int,
                            num_kv_heads: int, head_dim: int, page_size: int, scale: float,
                            window: int | None = None, tiles: tuple | None = None,
                            share_heads: bool | None = None, value_dim: int | None = None,
                            chunk: int | None = None, only_single: bool = False,
                            sinks: torch.Tensor | None = None, keep_first: int = 0) -> None:
    """Causal attention of each query token over its request's pages.  ``tiles``:
    (tile_first, tile_count, num_tiles, single_tokens, num_single), the step's work lists (tiles
    of up to 16 consecutive tokens of one request, and token rows that run alone), which together
    name every token once; tokens of a tile share the keys and values they load.  Without it every
    token runs alone; the result is the same bit for bit.  ``share_heads``: whether the query heads
    of a group share a block (and the keys it loads) for the tokens that run alone; None chooses by
    how many there are; the same bits again.  ``value_dim``: size of a value head if it differs from
    ``head_dim``.  ``chunk``: a query sees only the keys of its own chunk of that many positions
    (counted from position 0); not together with ``window``.  ``only_single``: the tokens of the tiles
    are left to another kernel.  ``sinks``: float32 [num_heads]; head a's softmax has exp(sinks[a]) as one
    more term of its denominator, with no key and no value.  ``keep_first``: with a window, the first so many
    positions of a sequence stay visible whatever the distance."""
    _gpu(q, k_cache, v_cache, block_tables, positions, req_of_token, out, sinks)
    _need(keep_first >= 0 and (keep_first == 0 or window), "kept first positions go with a window")
    _need(sinks is None or (sinks.dtype == torch.float32 and sinks.numel() == num_heads), "sinks are float32 [num_heads]")
    n = positions.numel()
    vd = head_dim if value_dim is None else int(value_dim)
    _need(not (window and chunk), "a window or chunks, not both")
    span = int(window or 0) if not chunk else -int(chunk)
    _need(q.dtype == k_cache.dtype == v_cache.dtype == out.dtype, "attention tensors must share a dtype")
    _need(q.numel() >= n * num_heads * head_dim and out.numel() >= n * num_heads * vd, "q/out too small")
    _need(head_dim % 8 == 0 and vd % 16 == 0 and max(head_dim, vd) <= 512 and page_size % 8 == 0,
          "head_dim must be a multiple of 8, the value size of 16 (at most 512), page_size a multiple of 8")
    _need(num_heads % num_kv_heads == 0, "num_heads must be a multiple of num_kv_heads")
    page_elems = num_kv_heads * head_dim * page_size
    _need(k_cache.numel() % page_elems == 0 and v_cache.numel() * head_dim == k_cache.numel() * vd,
          "cache size is not whole pages")
    _need(positions.dtype == torch.int32 and req_of_token.dtype == torch.int32
          and block_tables.dtype == torch.int32 and block_tables.dim() == 2, "descriptor arrays are int32")
    tile_first = tile_count = single = None
    num_tiles = num_single = 0
    if tiles is not None and only_single:
        if tiles[4] == 0:
            return
        # (the list of tiles is there and empty: only the tokens of ``single`` run)
        tile_first, tile_count, num_tiles, single, num_single = tiles[3], tiles[3], 0, tiles[3], tiles[4]
        _need(single is not None and single.is_cuda and single.dtype == torch.int32 and single.numel() >= num_single,
              "bad list of single tokens")
    elif tiles is not None and tiles[2] > 0:
        tile_first, tile_count, num_tiles, single, num_single = tiles
        _gpu(tile_first, tile_count)
        _need(tile_first.dtype == torch.int32 and tile_count.dtype == torch.int32
              and tile_first.numel() >= num_tiles and tile_count.numel() >= num_tiles, "bad tile list")
        _need(num_single == 0 or (single is not None and single.is_cuda and single.dtype == torch.int32
                                  and single.numel() >= num_single), "bad list of single tokens")
    _check(_fn("attention_generic", "tk_paged_attention_generic")(
        _code(q.dtype), _p(q), _p(k_cache), _p(v_cache), _p(block_tables), _p(positions),
        _p(req_of_token), _p(out), n, num_heads, num_kv_heads, head_dim, vd, page_size,
        block_tables.shape[1], float(scale), span, int(keep_first), _p(tile_first), _p(tile_count), num_tiles,
        _p(single), num_single, -1 if share_heads is None else int(share_heads), _p(sinks), _stream()),
        "paged_attention_generic")


NOT_INSTANTIATED = -2


def attention_tiles(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                    positions: torch.Tensor, req_of_token: torch.Tensor, tile_first: torch.Tensor,
                    tile_count: torch.Tensor, num_tiles: int, out: torch.Tensor, *, num_heads: int, num_kv_heads: int,
                    head_dim: int, value_dim: int, page_size: int, scale: float, window: int | None = None,
                    chunk: int | None = None, sinks: torch.Tensor | None = None, keep_first: int = 0) -> bool:
    """bf16 attention of the tiles of prompt portions (up to 16 consecutive tokens of one request each) on
    the matrix cores, for keys and values of unlike sizes (up to 512; keys in pieces of 8, values in blocks
    of 16), any group, a window or chunks, sinks; pages of a multiple of 16 tokens.  Returns False
    (nothing launched) for a shape it does not take."""
    _gpu(q, k_cache, v_cache, block_tables, positions, req_of_token, tile_first, tile_count, out, sinks)
    n = positions.numel()
    if not (q.dtype == k_cache.dtype == v_cache.dtype == out.dtype == torch.bfloat16 and page_size % 16 == 0
            and head_dim % 8 == 0 and value_dim % 16 == 0 and max(head_dim, value_dim) <= 512):
        return False
    _need(not (window and chunk), "a window or chunks, not both")
    _need(q.numel() >= n * num_heads * head_dim and out.numel() >= n * num_heads * value_dim, "q/out too small")
    _need(num_heads % num_kv_heads == 0, "num_heads must be a multiple of num_kv_heads")
    _need(k_cache.numel() % (num_kv_heads * head_dim * page_size) == 0
          and v_cache.numel() * head_dim == k_cache.numel() * value_dim, "cache size is not whole pages")
    _need(positions.dtype == torch.int32 and req_of_token.dtype == torch.int32 and block_tables.dtype == torch.int32
          and block_tables.dim() == 2 and tile_first.dtype == torch.int32 and tile_count.dtype == torch.int32
          and tile_first.numel() >= num_tiles and tile_count.numel() >= num_tiles, "descriptor arrays are int32")
    _need(sinks is None or (sinks.dtype == torch.float32 and sinks.numel() == num_heads), "sinks are float32 [num_heads]")
    span = int(window or 0) if not chunk else -int(chunk)
    status = _fn("attention_tiles", "tk_attention_tiles")(
        _p(q), _p(k_cache), _p(v_cache), _p(block_tables), block_tables.shape[1], _p(positions), _p(req_of_token),
        _p(tile_first), _p(tile_count), num_tiles, _p(out), num_heads, num_kv_heads, head_dim, value_dim, page_size,
        float(scale), span, int(keep_first if window else 0), _p(sinks), _stream())
    if status == NOT_INSTANTIATED:
        return False
    _check(status, "attention_tiles")
    return True


def attention_mfma(mode: str, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                   block_tables: torch.Tensor, positions: torch.Tensor, req_of_token: torch.Tensor,
                   item_token: torch.Tensor, item_count: torch.Tensor | None, num_items: int,
                   out: torch.Tensor, *, num_heads: int, num_kv_heads: int, head_dim: int,
                   page_size: int, scale: float, split_keys: int = 256, num_splits: int = 1,
                   chunk: int | None = None, sinks: torch.Tensor | None = None) -> bool:
    """bf16 attention on the matrix cores.  ``mode`` "heads": every item is one
    decode token; "tokens": every item is up to 16 consecutive tokens of one
    request ("tokens_dense": the same, with the kernel variant for tiles that all
    walk a long context; "tokens_wide": items of up to 32 tokens, the 32x32 MFMA form;
    "tokens_group": the same items, a block of up to eight waves holding all query heads of
    a kv head and shares of the keys, any group size).  With ``num_splits`` > 1 the keys of an item are cut into pieces of
    ``split_keys`` (a multiple of 16; of 64 in "tokens" mode), each its own block, and a
    second kernel merges the pieces (in "heads" mode the sixteen waves of a block share a piece, so
    ``split_keys`` is a multiple of 256).  ``chunk`` ("tokens" and "tokens_dense" without splits): a
    query sees the keys of its own chunk of that many positions only.  ``sinks``: float32
    [num_heads], one more term exp(sinks[a]) of head a's denominator.  Returns False (nothing
    launched) if the shape is not instantiated."""
    _gpu(q, k_cache, v_cache, block_tables, positions, req_of_token, item_token, item_count, out, sinks)
    _need(sinks is None or (sinks.dtype == torch.float32 and sinks.numel() == num_heads), "sinks are float32 [num_heads]")
    n = positions.numel()
    _need(q.dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16
          and out.dtype == torch.bfloat16, "the MFMA attention kernel takes bfloat16")
    _need(q.numel() >= n * num_heads * head_dim and out.numel() >= n * num_heads * head_dim, "q/out too small")
    _need(num_heads % num_kv_heads == 0 and page_size >= 16 and page_size & (page_size - 1) == 0
          and split_keys % 16 == 0, "bad head counts, page size (a power of two >= 16) or split")
    page_elems = num_kv_heads * head_dim * page_size
    _need(k_cache.numel() % page_elems == 0 and v_cache.numel() == k_cache.numel(), "cache size is not whole pages")
    _need(positions.dtype == torch.int32 and req_of_token.dtype == torch.int32 and block_tables.dtype == torch.int32
          and item_token.dtype == torch.int32 and block_tables.dim() == 2, "descriptor arrays are int32")
    _need(item_token.numel() >= num_items and 0 < num_items <= 65535, "bad item list")
    _need(mode in ("heads", "tokens", "tokens_dense", "tokens_wide", "tokens_group"),
          "mode is heads, tokens, tokens_dense, tokens_wide or tokens_group")
    _need(mode not in ("tokens_wide", "tokens_group") or num_splits == 1, "the wide and group forms do not split keys over blocks")
    _need(mode != "heads" or num_splits == 1 or split_keys % 256 == 0, "heads mode splits keys in multiples of 256")
    _need(not chunk or (mode in ("tokens", "tokens_dense") and num_splits == 1 and chunk > 0),
          "chunked visibility: tiles of 16 tokens, keys not split")
    if mode != "heads":
        _need(item_count is not None and item_count.dtype == torch.int32 and item_count.numel() >= num_items,
              "tokens mode needs item counts")
        _need(num_splits == 1 or (split_keys % 64 == 0 and num_items * 16 <= 65535),
              "tokens mode splits keys in multiples of 64, for at most 4095 tiles")
    part_o = part_ml = None
    if num_splits > 1:
        rows = num_items * (16 if mode != "heads" else 1) * num_heads * num_splits
        part_o = torch.empty((rows, head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((rows, 2), dtype=torch.float32, device=q.device)
    status = _fn("attention_mfma", "tk_attention_mfma")(
        {"heads": 0, "tokens": 1, "tokens_dense": 2, "tokens_wide": 3, "tokens_group": 4}[mode], _p(q), _p(k_cache), _p(v_cache), _p(block_tables),
        block_tables.shape[1], _p(positions), _p(req_of_token), _p(item_token), _p(item_count),
        num_items, _p(out), _p(part_o), _p(part_ml), num_splits, split_keys, num_heads, num_kv_heads,
        head_dim, page_size, float(scale), int(chunk or 0), _p(sinks), _stream())
    if status == NOT_INSTANTIATED:
        return False
    _check(status, "attention_mfma")
    return True


def attention_tiles_fit(dtype: torch.dtype, head_dim: int, value_dim: int, page_size: int) -> bool:
    """Whether ``attention_tiles`` and ``attention_heads`` take the shape."""
    return (dtype == torch.bfloat16 and page_size % 16 == 0 and head_dim % 8 == 0 and value_dim % 16 == 0
            and 8 <= head_dim <= 512 and 16 <= value_dim <= 512)


def attention_heads(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                    positions: torch.Tensor, req_of_token: torch.Tensor, single: torch.Tensor, num_single: int,
                    out: torch.Tensor, *, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                    page_size: int, scale: float, num_splits: int, window: int | None = None,
                    chunk: int | None = None, sinks: torch.Tensor | None = None, keep_first: int = 0) -> None:
    """bf16 attention of tokens that run alone (``single``: their rows) on the matrix cores, the 16 columns of
    a product being 16 query heads of one kv head, for the shapes of ``attention_tiles``.  Each token's visible
    keys are dealt, 16 at a time, to the four waves of ``num_splits`` blocks; a second kernel merges the waves'
    partial results and adds the sinks."""
    _gpu(q, k_cache, v_cache, block_tables, positions, req_of_token, single, out, sinks)
    n = positions.numel()
    _need(attention_tiles_fit(q.dtype, head_dim, value_dim, page_size) and k_cache.dtype == v_cache.dtype == out.dtype == q.dtype,
          "attention_heads takes bfloat16, pages of a multiple of 16, keys in pieces of 8, values in blocks of 16")
    _need(not (window and chunk), "a window or chunks, not both")
    _need(q.numel() >= n * num_heads * head_dim and out.numel() >= n * num_heads * value_dim, "q/out too small")
    _need(num_heads % num_kv_heads == 0 and 1 <= num_splits <= 16, "bad head counts, or more than 16 splits")
    _need(k_cache.numel() % (num_kv_heads * head_dim * page_size) == 0
          and v_cache.numel() * head_dim == k_cache.numel() * value_dim, "cache size is not whole pages")
    _need(positions.dtype == torch.int32 and req_of_token.dtype == torch.int32 and block_tables.dtype == torch.int32
          and block_tables.dim() == 2 and single.dtype == torch.int32 and single.numel() >= num_single > 0,
          "descriptor arrays are int32")
    _need(sinks is None or (sinks.dtype == torch.float32 and sinks.numel() == num_heads), "sinks are float32 [num_heads]")
    rows = num_single * num_heads * num_splits * 4
    part_o = torch.empty((rows, value_dim), dtype=torch.float32, device=q.device)
    part_ml = torch.empty((rows, 2), dtype=torch.float32, device=q.device)
    span = int(window or 0) if not chunk else -int(chunk)
    _check(_fn("attention_tiles", "tk_attention_heads")(
        _p(q), _p(k_cache), _p(v_cache), _p(block_tables), block_tables.shape[1], _p(positions), _p(req_of_token),
        _p(single), num_single, _p(out), _p(part_o), _p(part_ml), num_splits, num_heads, num_kv_heads, head_dim,
        value_dim, page_size, float(scale), span, int(keep_first if window else 0), _p(sinks), _stream()), "attention_heads")


FUSED_DECODE_MAX_GROUP = 14   # query heads per kv head the fused decode kernel takes (two waves make the key and value)


def attention_decode_fused(qkv: torch.Tensor, q_weight: torch.Tensor | None, k_weight: torch.Tensor | None,
                           cos: torch.Tensor | None, sin: torch.Tensor | None, k_cache: torch.Tensor,
                           v_cache: torch.Tensor, block_tables: torch.Tensor, positions: torch.Tensor,
                           req_of_token: torch.Tensor, item_token: torch.Tensor, num_items: int,
                           out: torch.Tensor, *, num_heads: int, num_kv_heads: int, head_dim: int,
                           rotary_dim: int, page_size: int, eps: float, scale: float, store: bool,
                           split_keys: int, num_splits: int) -> bool:
    """Decode tokens from the q/k/v projection's output in one kernel: per-head norm and
    rotation of the queries (and, with ``store``, of the token's key, which is written to
    its page with the value), then attention over the pages as ``attention_mfma("heads")``.
    ``qkv``: [N, (nh + 2 nkv) hd] bfloat16, or float32 partial sums [P, N, ...] (without
    ``store`` the rows hold queries only).  Returns False (nothing launched) if the shape is
    not instantiated; the caller then runs the two kernels."""
    _gpu(qkv, q_weight, k_weight, cos, sin, k_cache, v_cache, block_tables, positions, req_of_token, item_token, out)
    n = positions.numel()
    nkv_in = num_kv_heads if store else 0
    width = (num_heads + 2 * nkv_in) * head_dim
    in_f32, parts, stride = _partials(qkv, n, width, out.dtype, "qkv")
    _need(qkv.shape[-2] == n, "the fused kernel reads qkv rows by token: one row per token")
    _need(out.dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16,
          "the fused decode kernel is bfloat16")
    _need(out.numel() >= n * num_heads * head_dim, "out too small")
    _need(num_heads % num_kv_heads == 0 and page_size >= 16 and page_size & (page_size - 1) == 0,
          "bad head counts or page size (a power of two >= 16)")
    _need(rotary_dim in (0, head_dim), "the fused decode kernel rotates whole heads or not at all")
    _need(rotary_dim == 0 or (cos is not None and sin is not None and cos.dtype == torch.float32 and sin.dtype == torch.float32
                              and cos.numel() >= n * (head_dim // 2) and sin.numel() >= n * (head_dim // 2)
                              and cos.data_ptr() % 8 == 0 and sin.data_ptr() % 8 == 0), "rotary tables missing or too small")
    for w in (q_weight, k_weight):
        _need(w is None or (w.dtype == torch.float32 and w.numel() == head_dim), "q/k norm weights are float32 [head_dim]")
    _need((q_weight is None) == (k_weight is None), "q and k are normed together or not at all")
    page_elems = num_kv_heads * head_dim * page_size
    _need(k_cache.numel() % page_elems == 0 and v_cache.numel() == k_cache.numel(), "cache size is not whole pages")
    _need(positions.dtype == torch.int32 and req_of_token.dtype == torch.int32 and block_tables.dtype == torch.int32
          and item_token.dtype == torch.int32 and block_tables.dim() == 2, "descriptor arrays are int32")
    _need(item_token.numel() >= num_items and 0 < num_items <= 65535, "bad item list")
    _need(split_keys % 256 == 0 and num_splits >= 1, "splits are multiples of 256 keys")
    part_o = part_ml = None
    if num_splits > 1:
        rows = num_items * num_heads * num_splits
        part_o = torch.empty((rows, head_dim), dtype=torch.float32, device=out.device)
        part_ml = torch.empty((rows, 2), dtype=torch.float32, device=out.device)
    status = _fn("attention_fused", "tk_attention_decode_fused")(
        _p(qkv), in_f32, parts, stride, _p(q_weight), _p(k_weight), _p(cos), _p(sin), rotary_dim, float(eps), nkv_in,
        _p(k_cache), _p(v_cache), _p(block_tables), block_tables.shape[1], _p(positions), _p(req_of_token),
        _p(item_token), num_items, _p(out), _p(part_o), _p(part_ml), num_splits, split_keys, num_heads, num_kv_heads,
        head_dim, page_size, float(scale), _stream())
    if status == NOT_INSTANTIATED:
        return False
    _check(status, "attention_decode_fused")
    return True


def argmax(logits: torch.Tensor, out: torch.Tensor, values: torch.Tensor | None = None) -> None:
    """out[m] = index of the first maximum of logits[m]; ``values`` (optional, float32
    [M]) receives the maxima."""
    _need(logits.is_cuda and logits.dim() == 2 and logits.stride(1) == 1 and logits.dtype == torch.float32,
          "logits are float32 [M, V] on the GPU")
    _gpu(out)
    m, v = logits.shape
    _need(out.dtype == torch.int32 and out.numel() >= m, "argmax output is int32 [M]")
    _need(m <= 65535, "at most 65535 rows")
    _need(values is None or (values.is_cuda and values.dtype == torch.float32 and values.numel() >= m
                             and values.is_contiguous()), "argmax values are float32 [M]")
    segments = _fn("sampling", "tk_argmax_segments")()
    part_v = torch.empty(m * segments, dtype=torch.float32, device=logits.device)
    part_i = torch.empty(m * segments, dtype=torch.int32, device=logits.device)
    _check(_fn("sampling", "tk_argmax")(_p(logits), _p(out), _p(values), _p(part_v), _p(part_i), m, v,
                                        logits.stride(0), _stream()), "argmax")


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
           top_p: torch.Tensor, seeds: torch.Tensor, counters: torch.Tensor, out: torch.Tensor,
           probs_out: torch.Tensor | None = None) -> None:
    """Temperature / top-k / top-p sampling, one row per request."""
    _need(logits.is_cuda and logits.dim() == 2 and logits.stride(1) == 1 and logits.dtype == torch.float32,
          "logits are float32 [M, V] on the GPU")
    _gpu(temperature, top_k, top_p, seeds, counters, out, probs_out)
    m, v = logits.shape
    _need(temperature.dtype == torch.float32 and top_p.dtype == torch.float32 and top_k.dtype == torch.int32,
          "temperature/top_p float32, top_k int32")
    _need(seeds.dtype == torch.int64 and counters.dtype == torch.int64, "seeds and counters are int64")
    for t in (temperature, top_k, top_p, seeds, counters, out):
        _need(t.numel() >= m, "one sampling parameter per row is required")
    _need(out.dtype == torch.int32, "sample output is int32")
    _need(probs_out is None or (probs_out.dtype == torch.float32 and probs_out.shape == (m, v)), "probs_out is float32 [M, V]")
    _need(m <= 65535, "at most 65535 rows")
    # the argmax pass: greedy rows are done with it, the others overwrite it; it also leaves every
    # row's maximum and, segment by segment, the maxima and the masses at the row's temperature,
    # from which a row without thresholds is drawn without another pass over its logits
    segments = _fn("sampling", "tk_argmax_segments")()
    floats = torch.empty((2 * segments + 1) * m, dtype=torch.float32, device=logits.device)
    row_max, seg_max, seg_mass = floats[:m], floats[m:m + segments * m], floats[m + segments * m:]
    seg_index = torch.empty(m * segments, dtype=torch.int32, device=logits.device)
    _check(_fn("sampling", "tk_argmax_masses")(_p(logits), _p(out), _p(row_max), _p(seg_max), _p(seg_index),
                                               _p(temperature), _p(top_k), _p(top_p), _p(seg_mass), m, v,
                                               logits.stride(0), _stream()),
           "argmax_masses")
    _check(_fn("sampling", "tk_sample")(_p(logits), logits.stride(0), m, v, _p(temperature), _p(top_k),
                                        _p(top_p), _p(seeds), _p(counters), _p(row_max), _p(seg_max), _p(seg_mass),
                                        _p(out), _p(probs_out), _stream()), "sample")
