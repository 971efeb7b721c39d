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
        "tk_embed_gather": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
        "tk_feed_tokens": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
        "tk_add_rmsnorm": [c_int, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p,
                           c_void_p, c_int, c_int, c_float, c_int, c_void_p],
        "tk_rope_tables": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
        "tk_qknorm_rope_store": [c_int, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                 c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p],
        "tk_silu_mul": [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p],
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
                                  c_int, c_void_p, c_int, c_float, c_void_p],
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
                                       c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                       c_float, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p],
    },
    "attention_mfma": {
        "tk_attention_mfma": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                              c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int,
                              c_int, c_int, c_int, c_int, c_float, c_void_p],
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
_LIBRARY_FILE = {"attention_fused": "attention_mfma"}   # signature group -> library that holds it
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
def embed_gather(table: torch.Tensor, ids: torch.Tensor, resid: torch.Tensor) -> None:
    """resid[n] = float(table[ids[n]]); resid is float32 [N, H]."""
    _gpu(table, ids, resid)
    n = ids.numel()
    v, h = table.shape
    _need(ids.dtype == torch.int32, "token ids must be int32")
    _need(resid.dtype == torch.float32 and resid.shape[-1] == h and resid.numel() >= n * h,
          "residual buffer must be float32 [>=N, H]")
    _note(f"{n}x{h}", n * h * (table.element_size() + 4))
    _check(_fn("elementwise", "tk_embed_gather")(_code(table.dtype), _p(table), _p(ids), _p(resid),
                                                 n, h, v, _stream()), "embed_gather")


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


def rope_tables(positions: torch.Tensor, inv_freq: torch.Tensor, cos: torch.Tensor,
                sin: torch.Tensor) -> None:
    _gpu(positions, inv_freq, cos, sin)
    n, half = positions.numel(), inv_freq.numel()
    _need(positions.dtype == torch.int32 and inv_freq.dtype == torch.float32, "positions int32, inv_freq float32")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.numel() >= n * half
          and sin.numel() >= n * half, "cos/sin tables must be float32 [N, half]")
    _check(_fn("elementwise", "tk_rope_tables")(_p(positions), _p(inv_freq), _p(cos), _p(sin), n,
                                                half, _stream()), "rope_tables")


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


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """out[n, i] = silu(gate_up[n, i]) * gate_up[n, I + i]."""
    _gpu(gate_up, out)
    n, two_i = gate_up.shape
    _need(two_i % 2 == 0 and out.shape == (n, two_i // 2) and out.dtype == gate_up.dtype, "silu_mul shapes disagree")
    _note(f"{n}x{two_i // 2}", n * two_i * out.element_size() * 1.5)
    _check(_fn("elementwise", "tk_silu_mul")(_code(out.dtype), _p(gate_up), _p(out), n, two_i // 2,
                                             _stream()), "silu_mul")


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
                       sumsq: torch.Tensor | None = None, eps: float = 0.0) -> None:
    """out[M, I] = silu(a @ w[:I]^T) * (a @ w[I:]^T) for M <= 64: the gate and up
    projections and the SiLU product in one weight-streaming kernel (bfloat16).  ``sumsq``,
    ``eps``: the rows' scale, applied to both products before the gate, as in ``gemm_stream``."""
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
                                                     _p(sumsq), slabs, float(eps), _stream()), "gemm_stream_swiglu")


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


def paged_attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            block_tables: torch.Tensor, positions: torch.Tensor,
                            req_of_token: torch.Tensor, out: torch.Tensor, *, num_heads: int,
                            num_kv_heads: int, head_dim: int, page_size: int, scale: float,
                            window: int | None = None, tiles: tuple | None = None,
                            share_heads: bool | None = None) -> None:
    """Causal attention of each query token over its request's pages.  ``tiles``:
    (tile_first, tile_count, num_tiles, single_tokens, num_single), the step's work lists (tiles
    of up to 16 consecutive tokens of one request, and token rows that run alone), which together
    name every token once; tokens of a tile share the keys and values they load.  Without it every
    token runs alone; the result is the same bit for bit.  ``share_heads``: whether the query heads
    of a group share a block (and the keys it loads) for the tokens that run alone; None chooses by
    how many there are; the same bits again."""
    _gpu(q, k_cache, v_cache, block_tables, positions, req_of_token, out)
    n = positions.numel()
    _need(q.dtype == k_cache.dtype == v_cache.dtype == out.dtype, "attention tensors must share a dtype")
    _need(q.numel() >= n * num_heads * head_dim and out.numel() >= n * num_heads * head_dim, "q/out too small")
    _need(head_dim % 16 == 0 and head_dim <= 512 and page_size % 8 == 0, "head_dim must be a multiple of 16 (at most 512), page_size a multiple of 8")
    _need(num_heads % num_kv_heads == 0, "num_heads must be a multiple of num_kv_heads")
    page_elems = num_kv_heads * head_dim * page_size
    _need(k_cache.numel() % page_elems == 0 and v_cache.numel() == k_cache.numel(), "cache size is not whole pages")
    _need(positions.dtype == torch.int32 and req_of_token.dtype == torch.int32
          and block_tables.dtype == torch.int32 and block_tables.dim() == 2, "descriptor arrays are int32")
    tile_first = tile_count = single = None
    num_tiles = num_single = 0
    if tiles is not None and tiles[2] > 0:
        tile_first, tile_count, num_tiles, single, num_single = tiles
        _gpu(tile_first, tile_count)
        _need(tile_first.dtype == torch.int32 and tile_count.dtype == torch.int32
              and tile_first.numel() >= num_tiles and tile_count.numel() >= num_tiles, "bad tile list")
        _need(num_single == 0 or (single is not None and single.is_cuda and single.dtype == torch.int32
                                  and single.numel() >= num_single), "bad list of single tokens")
    _check(_fn("attention_generic", "tk_paged_attention_generic")(
        _code(q.dtype), _p(q), _p(k_cache), _p(v_cache), _p(block_tables), _p(positions),
        _p(req_of_token), _p(out), n, num_heads, num_kv_heads, head_dim, page_size,
        block_tables.shape[1], float(scale), int(window or 0), _p(tile_first), _p(tile_count), num_tiles,
        _p(single), num_single, -1 if share_heads is None else int(share_heads), _stream()), "paged_attention_generic")


NOT_INSTANTIATED = -2


def attention_mfma(mode: str, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                   block_tables: torch.Tensor, positions: torch.Tensor, req_of_token: torch.Tensor,
                   item_token: torch.Tensor, item_count: torch.Tensor | None, num_items: int,
                   out: torch.Tensor, *, num_heads: int, num_kv_heads: int, head_dim: int,
                   page_size: int, scale: float, split_keys: int = 256, num_splits: int = 1) -> bool:
    """bf16 attention on the matrix cores.  ``mode`` "heads": every item is one
    decode token; "tokens": every item is up to 16 consecutive tokens of one
    request ("tokens_dense": the same, with the kernel variant for tiles that all
    walk a long context; "tokens_wide": items of up to 32 tokens, the 32x32 MFMA form;
    "tokens_group": the same items, a block of up to eight waves holding all query heads of
    a kv head and shares of the keys, any group size).  With ``num_splits`` > 1 the keys of an item are cut into pieces of
    ``split_keys`` (a multiple of 16; of 64 in "tokens" mode), each its own block, and a
    second kernel merges the pieces (in "heads" mode the sixteen waves of a block share a piece, so
    ``split_keys`` is a multiple of 256).  Returns False (nothing launched) if the shape
    is not instantiated."""
    _gpu(q, k_cache, v_cache, block_tables, positions, req_of_token, item_token, item_count, out)
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
        head_dim, page_size, float(scale), _stream())
    if status == NOT_INSTANTIATED:
        return False
    _check(status, "attention_mfma")
    return True


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
