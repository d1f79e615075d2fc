"""torch-tensor wrappers over the C ABI of libptv3_hip.so.

torch is used for device memory and the current stream only; every computation happens in
the HIP kernels. All tensors must live on the GPU; CPU tensors are rejected.
"""
import contextlib
import ctypes
import weakref

import numpy as np
import torch
from torch.optim.optimizer import register_optimizer_step_post_hook as _register_step_hook

from . import _lib

ORDER_IDS = {"z": 0, "z-trans": 1, "hilbert": 2, "hilbert-trans": 3}
_DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
DTYPE_CODES = _DTYPE_CODE   # the dtypes the mixed-dtype row kernels read and write
REDUCE_OPS = {"max": 0, "mean": 1, "sum": 2, "min": 3}


_LAUNCH_TIMER = None


def set_launch_timer(timer):
    """Install (or clear, with None) an object whose launch(name, work, fn) brackets selected
    kernel launches with device events; used by the benchmark, off by default."""
    global _LAUNCH_TIMER
    _LAUNCH_TIMER = timer


def _timed(name, work, call):
    """call(), between two events of the installed launch timer when there is one."""
    if _LAUNCH_TIMER is not None:
        _LAUNCH_TIMER.launch(name, work, call)
    else:
        call()


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_RAW_DEVICE = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """Handle of torch's current stream on the current device. One launch asks for it once; through the two C entry
    points that is a fraction of a microsecond, through torch.cuda.current_stream() (a Stream object per call) 2-3."""
    if _RAW_STREAM is not None and _RAW_DEVICE is not None:
        return _RAW_STREAM(_RAW_DEVICE())
    return torch.cuda.current_stream().cuda_stream


def _dev(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise _lib.Ptv3Error("ptv3 ops run on the GPU only; got a CPU tensor (there is no CPU fallback)")


def _ptr(t):
    return None if t is None else t.data_ptr()


def wants_grad(*tensors):
    """True when autograd is recording and one of the tensors (or parameters) takes a gradient: the fused
    inference kernels are then left for the operators that have a backward."""
    return torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in tensors)


_CAST_CACHE = {}     # (id(parameter), dtype, layout) -> _Cast
_CAST_EPOCH = [0]    # bumped by invalidate_casts()
_CAST_TABLES = {}    # (device, dtype) -> (table bytes, device table): optimizer steps ask for the same table again
_CAST_JOB = np.dtype([("src", "<u8"), ("dst", "<u8"), ("a", "<i4"), ("b", "<i4"), ("c", "<i4"), ("mirror", "<i4"),
                      ("first_block", "<i8")])   # ptv3_cast_job


class _Cast:
    __slots__ = ("stamp", "out", "ref", "shape", "mirror")


def _cast_shape(t, layout):
    """(a, b, c) of the parameter as the cast kernel sees it and the shape of the copy. layout "plain" keeps the
    element order; "transpose" swaps the axes of a matrix; "mirror" turns a convolution weight (Cout, taps..., Cin)
    into (Cin, mirrored taps, Cout), which is the weight of the input gradient."""
    if layout == "plain":
        return (1, 1, t.numel()), tuple(t.shape)
    a, c = t.shape[0], t.shape[-1]
    b = t.numel() // (a * c)
    return (a, b, c), ((c, a) if layout == "transpose" else (c, b, a))


def invalidate_casts():
    """Declare every remembered parameter copy stale. In-place updates through torch show in the parameter's
    version counter, which cast_cached checks by itself; fused optimizers (torch.optim.AdamW(fused=True)) write
    the parameters without touching it, and so does a write through .data: every optimizer step calls this through
    a global post-step hook, and so does the model at the start of every forward. Code that calls the operators
    without the model calls it after writing parameters some other way."""
    _CAST_EPOCH[0] += 1


def parameter_stamp(t):
    """What a derived copy of parameter t remembers to know when it is stale: storage, version counter and the
    count of invalidate_casts() calls."""
    return (t.data_ptr(), t._version, _CAST_EPOCH[0])


_cast_stamp = parameter_stamp
_register_step_hook(lambda *_: invalidate_casts())


def _refresh_stale_casts(dtype, device):
    """Every remembered copy in dtype whose parameter has been written since (an optimizer step touches all of them
    at once) is redone in place by one launch instead of a few small ones per parameter."""
    stale, blocks = [], 0
    for entry in _CAST_CACHE.values():
        t = entry.ref()
        if t is None or entry.out.dtype != dtype or t.device != device:
            continue
        now = _cast_stamp(t)
        if now != entry.stamp:
            a, b, c = entry.shape
            stale.append((entry, now, (t.data_ptr(), entry.out.data_ptr(), a, b, c, entry.mirror, blocks)))
            blocks += _lib.load().ptv3_cast_params_blocks(a, b, c, entry.mirror)
    if not stale:
        return
    table = np.array([row for _, _, row in stale], dtype=_CAST_JOB).tobytes()
    held = _CAST_TABLES.get((device, dtype))
    if held is None or held[0] != table:
        held = (table, torch.frombuffer(bytearray(table), dtype=torch.uint8).to(device))
        _CAST_TABLES[(device, dtype)] = held
    with torch.cuda.device(device):
        _lib.check(_lib.load().ptv3_cast_params(held[1].data_ptr(), len(stale), blocks, _DTYPE_CODE[dtype],
                                                _stream()), "ptv3_cast_params")
    for entry, now, _ in stale:
        entry.stamp = now


def cast_cached(t, dtype, layout="plain"):
    """The parameter t in dtype -- as it is ("plain"), transposed, or as the mirrored convolution weight of the
    input gradient (see _cast_shape) -- remembered until the parameter is written to or moved: training would
    otherwise cast every weight on every use, twice per step and layer. fp32 masters on the GPU are converted by
    ptv3_cast_params, all stale copies in one launch. The result must not be kept across optimizer steps: it is
    overwritten in place when the parameter changes."""
    if t.dtype == dtype and layout == "plain":
        return t
    if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and dtype in _DTYPE_CODE):
        with torch.no_grad():   # half-precision masters, CPU tensors: not worth remembering
            src = t.detach()
            if layout == "transpose":
                src = src.t()
            elif layout == "mirror":
                src = src.reshape(t.shape[0], -1, t.shape[-1]).flip(1).permute(2, 1, 0)
            return src.to(dtype).contiguous()
    key = (id(t), dtype, layout)
    entry = _CAST_CACHE.get(key)
    shape, out_shape = _cast_shape(t, layout)
    if entry is None or entry.ref() is not t or entry.shape != shape or entry.out.device != t.device:
        import weakref
        entry = _Cast()
        entry.stamp, entry.shape, entry.mirror = None, shape, int(layout != "plain")
        entry.out = torch.empty(out_shape, dtype=dtype, device=t.device)
        entry.ref = weakref.ref(t, lambda _r, k=key: _CAST_CACHE.pop(k, None))
        _CAST_CACHE[key] = entry
    if entry.stamp != _cast_stamp(t):
        _refresh_stale_casts(dtype, t.device)
    return entry.out


_IDLE_WORK = []        # callables that bring derived parameter copies up to date, see refresh_derived_copies
_IDLE_EPOCH = [-1]     # the invalidate_casts() count they last ran for
IDLE_WORK_ALLOWED = True   # off inside PrologueOverlap.scope(): what is allocated there is recycled two forwards on


def refresh_derived_copies():
    """Redo, once per invalidate_casts() epoch, the packed weight copies that the inference kernels will ask for
    (every convolution's and MLP's that has been used before), at a moment when the host has nothing better to do:
    Readback.get() calls this when its value is still on the way, the model before it queues an overlapped index
    prologue. Found stale at their first use instead, the copies cost the host its 0.2 ms of stamp comparisons right
    where the GPU waits for the launch behind them."""
    if _IDLE_EPOCH[0] == _CAST_EPOCH[0] or not IDLE_WORK_ALLOWED or torch.is_grad_enabled():
        return
    _IDLE_EPOCH[0] = _CAST_EPOCH[0]
    for fn in _IDLE_WORK:
        fn()


class Readback:
    """Device -> host read of a small tensor that does not drain the stream.

    A plain .tolist() / .item() waits for everything queued on the stream and leaves the GPU idle
    until the host has queued new work. Here the copy into pinned memory is queued right behind the
    producing kernels, followed by an event; get() waits for that event only, so whatever the host
    queued on the stream in between keeps the GPU busy while the value travels."""

    blocking = False   # True: plain stream-draining copy at get() (for comparison)

    def __init__(self, tensor):
        if Readback.blocking:
            self.tensor = tensor
            return
        self.host = torch.empty(tensor.shape, dtype=tensor.dtype, pin_memory=True)
        self.host.copy_(tensor, non_blocking=True)
        self.done = torch.cuda.Event()
        self.done.record(torch.cuda.current_stream(tensor.device))

    def get(self):
        """The values as a Python list (waits for the copy only)."""
        if Readback.blocking:
            return self.tensor.tolist()
        if not self.done.query():
            refresh_derived_copies()
        self.done.synchronize()
        return self.host.tolist()


def _ws(nbytes, device):
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


def _dtype_code(t):
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise _lib.Ptv3Error(f"unsupported dtype {t.dtype}") from None


def encode_orders(grid_coord, batch, depth, orders):
    """All requested curve codes in one pass: returns (k, N) int64."""
    _dev(grid_coord, batch)
    lib = _lib.load()
    g = grid_coord.to(torch.int32).contiguous()
    b = None if batch is None else batch.to(torch.int64).contiguous()
    n, k = g.shape[0], len(orders)
    ids = (ctypes.c_int32 * k)(*[ORDER_IDS[o] for o in orders])
    code = torch.empty((k, n), dtype=torch.int64, device=g.device)
    _timed("encode", (n, k), lambda: _lib.check(
        lib.ptv3_encode(_ptr(g), _ptr(b), n, int(depth), ids, k, _ptr(code), _stream()), "ptv3_encode"))
    return code


def decode_order(code, depth, order, with_batch=True):
    """Inverse of one row of encode_orders: (grid_coord (N,3) int64, batch (N,) int64 or None)."""
    _dev(code)
    lib = _lib.load()
    c = code.to(torch.int64).contiguous().reshape(-1)
    n = c.shape[0]
    grid = torch.empty((n, 3), dtype=torch.int64, device=c.device)
    batch = torch.empty((n,), dtype=torch.int64, device=c.device) if with_batch else None
    _lib.check(lib.ptv3_decode(_ptr(c), n, int(depth), ORDER_IDS[order], _ptr(grid), _ptr(batch), _stream()),
               "ptv3_decode")
    return grid, batch


def grid_max(grid_coord):
    """Per-axis maximum of (N,3) int32 coordinates as a (3,) int32 device tensor."""
    _dev(grid_coord)
    lib = _lib.load()
    g = grid_coord.to(torch.int32).contiguous()
    out = torch.empty(3, dtype=torch.int32, device=g.device)
    _lib.check(lib.ptv3_grid_max(_ptr(g), g.shape[0], _ptr(out), _stream()), "ptv3_grid_max")
    return out


def voxelize(coord, offset, grid_size, with_inverse=True, seed=0):
    """Per scene grid_coord = floor((coord - scene minimum) / grid_size), one point of every voxel kept: the first
    in input order when seed is 0, else a member drawn uniformly (another draw for another 32-bit seed).

    coord (N,3) float32 and offset (B,) cumulative scene ends on the device. Returns a dict:
    grid_coord (M,3) int32 and index (M,) int64 of the kept points in input order, offset (B,) int64
    scene ends of the kept points, inverse (N,) int64 voxel of every input point. One read-back (M)."""
    _dev(coord, offset)
    lib = _lib.load()
    coord = coord.to(torch.float32).contiguous()
    off = offset.to(torch.int64).contiguous()
    n, nb = coord.shape[0], off.shape[0]
    dev = coord.device
    grid = torch.empty((n, 3), dtype=torch.int32, device=dev)
    index = torch.empty(n, dtype=torch.int64, device=dev)
    inverse = torch.empty(n, dtype=torch.int64, device=dev) if with_inverse else None
    off_out = torch.empty(nb, dtype=torch.int64, device=dev)
    counts = torch.empty(2, dtype=torch.int64, device=dev)
    nbytes = lib.ptv3_voxelize_workspace_bytes(n, nb)
    ws = _ws(nbytes, dev)
    _lib.check(lib.ptv3_voxelize(_ptr(coord), n, _ptr(off), nb, float(grid_size), _ptr(grid), _ptr(index), _ptr(inverse),
                                 _ptr(off_out), _ptr(counts), int(seed) & 0xFFFFFFFF, _ptr(ws), nbytes, _stream()),
               "ptv3_voxelize")
    m, status = Readback(counts).get()
    if status:
        raise RuntimeError("voxelize: a grid coordinate does not fit 16 bits (grid_size too small for the scene extent)")
    out = dict(grid_coord=grid[:m], index=index[:m], offset=off_out)
    if with_inverse:
        out["inverse"] = inverse
    return out


def offset2batch(offset, n):
    """Scene id (int64) of each of n points from the cumulative scene ends on the device."""
    _dev(offset)
    lib = _lib.load()
    off = offset.to(torch.int64).contiguous()
    batch = torch.empty(int(n), dtype=torch.int64, device=off.device)
    _lib.check(lib.ptv3_offset2batch(_ptr(off), off.shape[0], int(n), _ptr(batch), _stream()), "ptv3_offset2batch")
    return batch


def argsort_rows(code, key_bits):
    """Row-wise ascending argsort of (k,N) int64 codes + inverse permutation."""
    _dev(code)
    lib = _lib.load()
    code = code.contiguous()
    k, n = code.shape
    order = torch.empty_like(code)
    inverse = torch.empty_like(code)
    nbytes = lib.ptv3_argsort_workspace_bytes(n, k)
    ws = _ws(nbytes, code.device)
    _timed("argsort", (n, k, int(key_bits)), lambda: _lib.check(
        lib.ptv3_argsort(_ptr(code), n, k, int(key_bits), _ptr(order), _ptr(inverse), _ptr(ws), nbytes, _stream()),
        "ptv3_argsort"))
    return order, inverse


def pad_sizes(offset_host, patch):
    """(n_pad, n_seq) from a host list of cumulative scene ends."""
    lib = _lib.load()
    nb = len(offset_host)
    arr = (ctypes.c_int64 * nb)(*[int(v) for v in offset_host])
    n_pad, n_seq = ctypes.c_int64(0), ctypes.c_int64(0)
    _lib.check(lib.ptv3_pad_sizes(arr, nb, int(patch), ctypes.byref(n_pad), ctypes.byref(n_seq)),
               "ptv3_pad_sizes")
    return n_pad.value, n_seq.value


def pad_index(offset, offset_host, patch):
    """pad (Npad,), unpad (N,), cu_seqlens (P+1,) int32 for the scenes in `offset`."""
    _dev(offset)
    lib = _lib.load()
    offset = offset.to(torch.int64).contiguous()
    nb = len(offset_host)
    n = int(offset_host[-1])
    n_pad, n_seq = pad_sizes(offset_host, patch)
    dev = offset.device
    pad = torch.empty(n_pad, dtype=torch.int64, device=dev)
    unpad = torch.empty(n, dtype=torch.int64, device=dev)
    cu = torch.empty(n_seq + 1, dtype=torch.int32, device=dev)
    nbytes = lib.ptv3_pad_index_workspace_bytes(nb)
    ws = _ws(nbytes, dev)
    _lib.check(lib.ptv3_pad_index(_ptr(offset), nb, int(patch), n, n_pad, n_seq, _ptr(pad), _ptr(unpad),
                                  _ptr(cu), _ptr(ws), nbytes, _stream()), "ptv3_pad_index")
    return pad, unpad, cu


def attn_slots(order_row, inverse_row, pad, unpad):
    """int32 gather (slot_src) and scatter (slot_dst, -1 for filler slots) tables."""
    _dev(order_row, inverse_row, pad, unpad)
    lib = _lib.load()
    n_pad = pad.shape[0]
    src = torch.empty(n_pad, dtype=torch.int32, device=pad.device)
    dst = torch.empty(n_pad, dtype=torch.int32, device=pad.device)
    _lib.check(lib.ptv3_attn_slots(_ptr(order_row.contiguous()), _ptr(inverse_row.contiguous()),
                                   _ptr(pad), _ptr(unpad), n_pad, _ptr(src), _ptr(dst), _stream()),
               "ptv3_attn_slots")
    return src, dst


def patch_attention(qkv, num_heads, slot_src, slot_dst, cu_seqlens, max_seqlen, scale):
    """softmax(q k^T * scale) v inside each sequence; qkv (N, 3C) in point order, result (N, C)
    in point order (gather and scatter fused into the kernel)."""
    _dev(qkv, slot_src, slot_dst, cu_seqlens)
    lib = _lib.load()
    qkv = qkv.contiguous()
    n, c3 = qkv.shape
    c = c3 // 3
    out = torch.empty((n, c), dtype=qkv.dtype, device=qkv.device)
    n_seq = cu_seqlens.shape[0] - 1

    def call():
        _lib.check(lib.ptv3_patch_attn_fwd(_ptr(qkv), _dtype_code(qkv), n, c, int(num_heads), _ptr(slot_src),
                                           _ptr(slot_dst), _ptr(cu_seqlens), n_seq, int(max_seqlen),
                                           float(scale), _ptr(out), _stream()), "ptv3_patch_attn_fwd")

    if _LAUNCH_TIMER is not None:
        _LAUNCH_TIMER.launch("patch_attn", (cu_seqlens, c), call)
    else:
        call()
    return out


def patch_attention_lse(qkv, num_heads, slot_src, slot_dst, cu_seqlens, max_seqlen, scale, dropout_p=0.0, seed=0):
    """patch_attention for training: (out, lse) with lse the (heads, n_pad) log-sum-exp rows the half-precision
    backward uses (None in fp32, where the backward recomputes them). dropout_p > 0: attention dropout, the kept
    probabilities chosen by a hash of (seed, head, query slot, key slot) that the backward recomputes."""
    _dev(qkv, slot_src, slot_dst, cu_seqlens)
    lib = _lib.load()
    qkv = qkv.contiguous()
    n, c3 = qkv.shape
    c = c3 // 3
    n_pad = slot_src.shape[0]
    out = torch.empty((n, c), dtype=qkv.dtype, device=qkv.device)
    lse = None
    if qkv.dtype != torch.float32:
        lse = torch.empty((int(num_heads), n_pad), dtype=torch.float32, device=qkv.device)
    _lib.check(lib.ptv3_patch_attn_fwd_lse(_ptr(qkv), _dtype_code(qkv), n, c, int(num_heads), _ptr(slot_src),
                                           _ptr(slot_dst), _ptr(cu_seqlens), cu_seqlens.shape[0] - 1, int(max_seqlen),
                                           n_pad, float(scale), float(dropout_p), int(seed) & 0xFFFFFFFF, _ptr(out),
                                           _ptr(lse), _stream()), "ptv3_patch_attn_fwd_lse")
    return out, lse


def patch_attention_bwd(qkv, out, dout, num_heads, slot_src, slot_dst, cu_seqlens, max_seqlen, scale, lse=None,
                        dropout_p=0.0, seed=0):
    """Gradient of patch_attention with respect to qkv, (N, 3C) laid out [dq | dk | dv]; lse from
    patch_attention_lse saves the backward kernel a sweep over the keys; dropout_p and seed as in the forward."""
    _dev(qkv, out, dout, slot_src, slot_dst, cu_seqlens)
    lib = _lib.load()
    qkv, out = qkv.contiguous(), out.contiguous()
    dout = dout.to(qkv.dtype).contiguous()
    n, c3 = qkv.shape
    c = c3 // 3
    n_pad = slot_src.shape[0]
    dqkv = torch.empty_like(qkv)
    code = _dtype_code(qkv)
    nbytes = lib.ptv3_patch_attn_bwd_workspace_bytes(code, n_pad, c, int(num_heads))
    ws = _ws(nbytes, qkv.device)
    _lib.check(lib.ptv3_patch_attn_bwd(_ptr(qkv), _ptr(out), _ptr(dout), code, n, c, int(num_heads), _ptr(slot_src),
                                       _ptr(slot_dst), _ptr(cu_seqlens), cu_seqlens.shape[0] - 1, int(max_seqlen),
                                       n_pad, float(scale), _ptr(lse), float(dropout_p), int(seed) & 0xFFFFFFFF,
                                       _ptr(dqkv), _ptr(ws), nbytes, _stream()), "ptv3_patch_attn_bwd")
    return dqkv


def patch_attention_rpe(qkv, num_heads, slot_src, slot_dst, cu_seqlens, max_seqlen, scale, grid_coord, rpe_table,
                        pos_bnd, dropout_p=0.0, seed=0):
    """patch_attention with the relative position bias of model.py:297-316 added to every score:
    fp32 qkv (N, 3C), grid_coord (N, 3) in point order, rpe_table (3 * (2 * pos_bnd + 1), H)."""
    _dev(qkv, slot_src, slot_dst, cu_seqlens, grid_coord, rpe_table)
    lib = _lib.load()
    if qkv.dtype != torch.float32:
        raise _lib.Ptv3Error("the relative position bias path computes in float32, as the reference's does")
    qkv = qkv.contiguous()
    n, c3 = qkv.shape
    c = c3 // 3
    g = grid_coord.to(torch.int32).contiguous()
    t = rpe_table.to(torch.float32).contiguous()
    if t.shape != (3 * (2 * pos_bnd + 1), num_heads) or g.shape != (n, 3):
        raise _lib.Ptv3Error("rpe_table must be (3 * (2 * pos_bnd + 1), heads) and grid_coord (N, 3)")
    out = torch.empty((n, c), dtype=torch.float32, device=qkv.device)
    _lib.check(lib.ptv3_patch_attn_rpe_fwd(_ptr(qkv), n, c, int(num_heads), _ptr(slot_src), _ptr(slot_dst),
                                           _ptr(cu_seqlens), cu_seqlens.shape[0] - 1, int(max_seqlen), float(scale),
                                           _ptr(g), _ptr(t), int(pos_bnd), float(dropout_p), int(seed) & 0xFFFFFFFF,
                                           _ptr(out), _stream()),
               "ptv3_patch_attn_rpe_fwd")
    return out


def patch_attention_rpe_bwd(qkv, out, dout, num_heads, slot_src, slot_dst, cu_seqlens, max_seqlen, scale, grid_coord,
                            rpe_table, pos_bnd, dropout_p=0.0, seed=0):
    """(dqkv, drpe_table) of patch_attention_rpe: fp32, the table's gradient (3 * (2 * pos_bnd + 1), H) in fp32."""
    _dev(qkv, out, dout, slot_src, slot_dst, cu_seqlens, grid_coord, rpe_table)
    lib = _lib.load()
    qkv, out = qkv.contiguous(), out.contiguous()
    dout = dout.to(qkv.dtype).contiguous()
    n, c3 = qkv.shape
    c = c3 // 3
    n_pad = slot_src.shape[0]
    g = grid_coord.to(torch.int32).contiguous()
    t = rpe_table.detach().to(torch.float32).contiguous()
    dqkv = torch.empty_like(qkv)
    dtable = torch.zeros_like(t)
    nbytes = lib.ptv3_patch_attn_bwd_workspace_bytes(0, n_pad, c, int(num_heads))
    ws = _ws(nbytes, qkv.device)
    _lib.check(lib.ptv3_patch_attn_rpe_bwd(_ptr(qkv), _ptr(out), _ptr(dout), 0, n, c, int(num_heads), _ptr(slot_src),
                                           _ptr(slot_dst), _ptr(cu_seqlens), cu_seqlens.shape[0] - 1, int(max_seqlen),
                                           n_pad, float(scale), None, float(dropout_p), int(seed) & 0xFFFFFFFF, _ptr(g),
                                           _ptr(t), int(pos_bnd), _ptr(dtable),
                                           _ptr(dqkv), _ptr(ws), nbytes, _stream()), "ptv3_patch_attn_rpe_bwd")
    return dqkv, dtable


def kmap_build(indices, ks, tap_major=False):
    """int32 neighbour map of (N,4) int32 [batch,x,y,z] voxels: (N, ks^3), or (ks^3, N) when
    tap_major (the layout the convolution kernels read coalesced)."""
    _dev(indices)
    lib = _lib.load()
    idx = indices.to(torch.int32).contiguous()
    n = idx.shape[0]
    shape = (ks ** 3, n) if tap_major else (n, ks ** 3)
    nbr = torch.empty(shape, dtype=torch.int32, device=idx.device)
    nbytes = lib.ptv3_kmap_workspace_bytes(n)
    ws = _ws(nbytes, idx.device)
    _lib.check(lib.ptv3_kmap_build(_ptr(idx), n, int(ks), int(bool(tap_major)), _ptr(nbr), _ptr(ws), nbytes,
                                   _stream()), "ptv3_kmap_build")
    return nbr


def subm_conv(feat, nbr, weight, bias=None, tap_major=False):
    """feat (N,Cin), nbr (N,V) int32 — or (V,N) when tap_major —, weight (Cout,V,Cin) or
    (Cout,k,k,k,Cin), bias (Cout,). Dense output-stationary form (every tap of every voxel)."""
    _dev(feat, nbr, weight, bias)
    lib = _lib.load()
    feat = feat.contiguous()
    nbr = nbr.contiguous()
    n, cin = feat.shape
    cout = weight.shape[0]
    taps = nbr.shape[0] if tap_major else nbr.shape[1]
    w = weight.reshape(cout, taps, cin).to(feat.dtype).contiguous()
    b = None if bias is None else bias.to(feat.dtype).contiguous()
    out = torch.empty((n, cout), dtype=feat.dtype, device=feat.device)
    _lib.check(lib.ptv3_subm_conv_fwd(_ptr(feat), _dtype_code(feat), n, cin, _ptr(nbr), taps,
                                      int(bool(tap_major)), _ptr(w), _ptr(b), cout, _ptr(out), _stream()),
               "ptv3_subm_conv_fwd")
    return out


def subm_conv_wgrad(feat, dout, nbr, with_bias=False):
    """Weight gradient (Cout, V, Cin) in fp32 of the submanifold convolution; nbr is the tap-major (V, N) map.
    with_bias: also the bias gradient (Cout,), summed in the same pass where the kernel allows (None otherwise)."""
    _dev(feat, dout, nbr)
    lib = _lib.load()
    feat = feat.contiguous()
    dout = dout.to(feat.dtype).contiguous()
    nbr = nbr.contiguous()
    n, cin = feat.shape
    cout = dout.shape[1]
    taps = nbr.shape[0]
    dw = torch.empty((cout, taps, cin), dtype=torch.float32, device=feat.device)
    fused = with_bias and feat.dtype != torch.float32 and cin % 8 == 0 and cout % 8 == 0
    db = torch.empty(cout, dtype=torch.float32, device=feat.device) if fused else None
    nbytes = lib.ptv3_subm_conv_wgrad_workspace_bytes(_dtype_code(feat), n, cin, cout, taps)
    ws = _ws(nbytes, feat.device) if nbytes else None
    _lib.check(lib.ptv3_subm_conv_wgrad(_ptr(feat), _ptr(dout), _dtype_code(feat), n, cin, cout, _ptr(nbr), taps,
                                        _ptr(dw), _ptr(db), _ptr(ws), nbytes, _stream()), "ptv3_subm_conv_wgrad")
    return (dw, db) if with_bias else dw


OUTER_WIDE_CHANNELS = 128   # from here on both sides, the weight-gradient kernels work on 128 x 128 blocks


def subm_conv_wgrad_pairs(feat, dout, plan, with_bias=False):
    """The same weight gradient (and bias gradient) from a ConvPlan's pair lists instead of the neighbour map
    (ptv3_subm_conv_wgrad_pairs): half precision, channels in 8s."""
    _dev(feat, dout)
    lib = _lib.load()
    feat = feat.contiguous()
    dout = dout.to(feat.dtype).contiguous()
    n, cin = feat.shape
    cout = dout.shape[1]
    dw = torch.empty((cout, plan.taps, cin), dtype=torch.float32, device=feat.device)
    db = torch.empty(cout, dtype=torch.float32, device=feat.device) if with_bias else None
    nbytes = lib.ptv3_subm_conv_wgrad_workspace_bytes(_dtype_code(feat), n, cin, cout, plan.taps)
    ws = _ws(nbytes, feat.device) if nbytes else None
    _lib.check(lib.ptv3_subm_conv_wgrad_pairs(_ptr(feat), _ptr(dout), _dtype_code(feat), n, cin, cout, _ptr(plan.tap_ptr),
                                              _ptr(plan.pair_in), _ptr(plan.pair_out()), plan.taps, _ptr(dw), _ptr(db),
                                              _ptr(ws), nbytes, _stream()), "ptv3_subm_conv_wgrad_pairs")
    return (dw, db) if with_bias else dw


class ConvPlan:
    """Active (input, output) pairs of a neighbour map, tap-major, plus each voxel's slots."""

    __slots__ = ("n", "taps", "_n_pairs", "tap_ptr", "row_ptr", "pair_in", "pair_slot", "_slot_pair", "_tiles",
                 "_pair_out")

    def pair_out(self):
        """The output voxel of every pair (the weight gradient's other index), made on first use."""
        if getattr(self, "_pair_out", None) is None:
            po = torch.empty(max(self.n_pairs, 1), dtype=torch.int32, device=self.pair_in.device)
            _lib.check(_lib.load().ptv3_conv_plan_pair_out(_ptr(self.row_ptr), _ptr(self.pair_slot), self.n, self.n_pairs,
                                                           _ptr(po), _stream()), "ptv3_conv_plan_pair_out")
            self._pair_out = po
        return self._pair_out

    @property
    def n_pairs(self):
        """Number of active pairs; a plan derived from another one learns it from a read-back at first use."""
        if isinstance(self._n_pairs, Readback):
            self._n_pairs = int(self._n_pairs.get()[0])
        return self._n_pairs

    @n_pairs.setter
    def n_pairs(self, value):
        self._n_pairs = value

    def density(self):
        return self.n_pairs / max(1, self.n * self.taps)

    def slot_pair(self):
        """Output-major pair words (tap << 24 | input row) for subm_conv_tiles, made on first use."""
        if getattr(self, "_slot_pair", None) is None:
            lib = _lib.load()
            sp = torch.empty(max(self.n_pairs, 1), dtype=torch.int32, device=self.pair_in.device)
            _lib.check(lib.ptv3_conv_plan_slots(_ptr(self.tap_ptr), self.taps, _ptr(self.pair_in), _ptr(self.pair_slot),
                                                self.n_pairs, _ptr(sp), _stream()), "ptv3_conv_plan_slots")
            self._slot_pair = sp
        return self._slot_pair

    def tiles(self, tile_voxels=128):
        """(tile_tap, tile_pair, vox_taps): every tile's pairs sorted by tap for subm_conv_tiles and subm_conv_sparse,
        made on first use, per tile size (128 outputs, or 96 for the 128-channel tile form)."""
        if getattr(self, "_tiles", None) is None:
            self._tiles = {}
        if tile_voxels not in self._tiles:
            lib = _lib.load()
            dev = self.pair_in.device
            tile_tap = torch.empty((lib.ptv3_conv_plan_tile_count_sized(self.n, tile_voxels), 32), dtype=torch.int32, device=dev)
            tile_pair = torch.empty(max(self.n_pairs, 1), dtype=torch.int32, device=dev)
            vox_taps = torch.empty(max(self.n, 1), dtype=torch.int32, device=dev)
            _lib.check(lib.ptv3_conv_plan_tiles_sized(_ptr(self.row_ptr), _ptr(self.slot_pair()), self.n, self.taps,
                                                      tile_voxels, _ptr(tile_tap), _ptr(tile_pair), _ptr(vox_taps),
                                                      _stream()), "ptv3_conv_plan_tiles_sized")
            self._tiles[tile_voxels] = (tile_tap, tile_pair, vox_taps)
        return self._tiles[tile_voxels]


def conv_plan(nbr, tap_major=False):
    """Pair lists for subm_conv_pairs from a (N, taps) — or tap-major (taps, N) — neighbour map.
    One host sync (the pair count)."""
    _dev(nbr)
    lib = _lib.load()
    nbr = nbr.contiguous()
    taps, n = nbr.shape if tap_major else nbr.shape[::-1]
    tm = int(bool(tap_major))
    dev = nbr.device
    plan = ConvPlan()
    plan.n, plan.taps = n, taps
    plan.tap_ptr = torch.empty(taps + 1, dtype=torch.int32, device=dev)
    count = torch.empty(1, dtype=torch.int64, device=dev)
    nbytes = lib.ptv3_conv_plan_workspace_bytes(n, taps)
    ws = _ws(nbytes, dev)
    _lib.check(lib.ptv3_conv_plan_count(_ptr(nbr), n, taps, tm, _ptr(plan.tap_ptr), _ptr(count), _ptr(ws),
                                        nbytes, _stream()), "ptv3_conv_plan_count")
    plan.n_pairs = int(count.item())
    plan.row_ptr = torch.empty(n + 1, dtype=torch.int32, device=dev)
    plan.pair_in = torch.empty(max(plan.n_pairs, 1), dtype=torch.int32, device=dev)
    plan.pair_slot = torch.empty(max(plan.n_pairs, 1), dtype=torch.int32, device=dev)
    _lib.check(lib.ptv3_conv_plan_fill(_ptr(nbr), n, taps, tm, _ptr(plan.tap_ptr), _ptr(plan.row_ptr),
                                       _ptr(plan.pair_in), _ptr(plan.pair_slot), _ptr(ws), nbytes, _stream()),
               "ptv3_conv_plan_fill")
    return plan


class PendingPlan:
    """conv_plan_direct between its two kernels: the pair count is on its way to the host."""

    __slots__ = ("plan", "idx", "ks", "ws", "nbytes", "count", "side_done")


# The first halves of the pair lists are queued on a second stream: chains of small, latency-bound
# kernels that depend on the coordinates only, they run beside the main stream's work (serialization,
# projections) instead of in front of it (0.08 ms per forward; the pooling clusters gained nothing there).
AHEAD_ON_SIDE_STREAM = True
_SIDE_STREAMS = {}


def side_stream(dev, index=0):
    """Side stream `index` of this device (default priority), made to wait for what the current stream holds."""
    side = _SIDE_STREAMS.get((dev, index))
    if side is None:
        side = _SIDE_STREAMS[(dev, index)] = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    return side


def _side_stream(dev):
    return side_stream(dev, 0)


class PrologueOverlap:
    """A stream and two private memory pools for index work that depends on a forward's inputs alone and may
    therefore run while the forward before it is still computing (PointTransformerV3.overlap_index_prologue).

    scope() runs its body on the prologue stream, which waits for nothing, with every allocation of the body routed
    to one of the two pools in turn; on leaving it the current stream is made to wait for the body's work.
    What the body allocates is used by the current stream afterwards without any per-tensor bookkeeping: a pool's
    memory is handed out again only two forwards later, after a host wait for an event that the current stream
    passed when the forward in between was entered -- behind the kernels of the forward that used the pool and behind
    whatever the caller queued on its results before calling again. The few tensors of a result that a caller may
    still read after that (PUBLIC_KEYS) are marked for the current stream by forward_queued()."""

    PUBLIC_KEYS = ("batch", "serialized_code", "serialized_order", "serialized_inverse", "pad", "unpad", "cu_seqlens_key")

    def __init__(self, device):
        self.device = device
        self.stream = torch.cuda.Stream(device=device)
        self.pools = [torch.cuda.MemPool(), torch.cuda.MemPool()]
        self.fence = [None, None]   # per pool: the current stream has passed every use of what it handed out
        self.turn = 0

    @contextlib.contextmanager
    def scope(self):
        global AHEAD_ON_SIDE_STREAM, IDLE_WORK_ALLOWED
        main = torch.cuda.current_stream(self.device)
        # the pool of the forward before this one: free again once the current stream has come this far
        entered = torch.cuda.Event()
        entered.record(main)
        self.fence[self.turn] = entered
        self.turn ^= 1
        if self.fence[self.turn] is not None:
            self.fence[self.turn].synchronize()   # recorded a forward ago: passed long since
        refresh_derived_copies()   # on the current stream, before it: the host is a forward's tail ahead of the GPU here
        ahead, AHEAD_ON_SIDE_STREAM = AHEAD_ON_SIDE_STREAM, False   # the shared side stream still holds the last forward's work
        idle, IDLE_WORK_ALLOWED = IDLE_WORK_ALLOWED, False
        try:
            with torch.cuda.stream(self.stream), torch.cuda.use_mem_pool(self.pools[self.turn], self.device):
                yield
                ready = torch.cuda.Event()
                ready.record(self.stream)
        finally:
            AHEAD_ON_SIDE_STREAM, IDLE_WORK_ALLOWED = ahead, idle
        main.wait_event(ready)

    def forward_queued(self, point):
        """The forward that entered scope() last has been queued and returns `point`: its index tensors that a caller
        may read on the current stream at any later time are marked for that stream (the allocator then holds their
        memory back until those reads are over); everything else of the index belongs to the forward."""
        main = torch.cuda.current_stream(self.device)
        for key in self.PUBLIC_KEYS:
            t = point.get(key)
            if isinstance(t, torch.Tensor) and t.is_cuda:
                t.record_stream(main)


def conv_plan_direct_start(indices, ks):
    """First half of conv_plan_direct: voxel hash and pair counts are queued and the total starts its
    way to the host; conv_plan_direct_finish completes the lists. Work queued in between overlaps
    the read-back instead of waiting behind it."""
    _dev(indices)
    lib = _lib.load()
    idx = indices.to(torch.int32).contiguous()
    n, taps = idx.shape[0], ks ** 3
    dev = idx.device
    plan = ConvPlan()
    plan.n, plan.taps = n, taps
    plan.tap_ptr = torch.empty(taps + 1, dtype=torch.int32, device=dev)
    count = torch.empty(1, dtype=torch.int64, device=dev)
    nbytes = lib.ptv3_kmap_plan_workspace_bytes(n, int(ks))
    ws = _ws(nbytes, dev)
    pend = PendingPlan()
    pend.plan, pend.idx, pend.ks, pend.ws, pend.nbytes = plan, idx, int(ks), ws, nbytes
    pend.side_done = None
    if AHEAD_ON_SIDE_STREAM and not Readback.blocking:
        side = _side_stream(dev)
        with torch.cuda.stream(side):
            _timed("kmap", (n, int(ks), "count"), lambda: _lib.check(
                lib.ptv3_kmap_plan_count(_ptr(idx), n, int(ks), _ptr(plan.tap_ptr), _ptr(count), _ptr(ws), nbytes,
                                         _stream()), "ptv3_kmap_plan_count"))
            pend.count = Readback(count)
            pend.side_done = torch.cuda.Event()
            pend.side_done.record(side)
        for t in (idx, plan.tap_ptr, count, ws):   # not to be reused before the second stream is through
            t.record_stream(side)
        return pend
    _timed("kmap", (n, int(ks), "count"), lambda: _lib.check(
        lib.ptv3_kmap_plan_count(_ptr(idx), n, int(ks), _ptr(plan.tap_ptr), _ptr(count), _ptr(ws), nbytes, _stream()),
        "ptv3_kmap_plan_count"))
    pend.count = Readback(count)
    return pend


def conv_plan_direct_finish(pend):
    lib = _lib.load()
    plan, idx, n = pend.plan, pend.idx, pend.plan.n
    dev = idx.device
    plan.n_pairs = int(pend.count.get()[0])
    if pend.side_done is not None:
        torch.cuda.current_stream(dev).wait_event(pend.side_done)
    plan.row_ptr = torch.empty(n + 1, dtype=torch.int32, device=dev)
    plan.pair_in = torch.empty(max(plan.n_pairs, 1), dtype=torch.int32, device=dev)
    plan.pair_slot = torch.empty(max(plan.n_pairs, 1), dtype=torch.int32, device=dev)
    _timed("kmap", (n, pend.ks, "fill"), lambda: _lib.check(
        lib.ptv3_kmap_plan_fill(_ptr(idx), n, pend.ks, _ptr(plan.tap_ptr), _ptr(plan.row_ptr), _ptr(plan.pair_in),
                                _ptr(plan.pair_slot), _ptr(pend.ws), pend.nbytes, _stream()), "ptv3_kmap_plan_fill"))
    return plan


def conv_plan_inner(plan5, pend5):
    """The 3x3x3 pair lists of the voxel set whose 5x5x5 lists plan5 holds, derived from them and from what
    the 5x5x5 count pass left in its workspace (pend5, the PendingPlan plan5 was finished from): no second
    voxel hash, no second neighbour search. Bit-identical to conv_plan_direct(indices, 3)."""
    lib = _lib.load()
    n, dev = plan5.n, plan5.tap_ptr.device
    assert plan5.taps == 125 and pend5.ks == 5
    plan = ConvPlan()
    plan.n, plan.taps = n, 27
    plan.tap_ptr = torch.empty(28, dtype=torch.int32, device=dev)
    found3 = torch.empty(n, dtype=torch.int32, device=dev)
    row_cnt = torch.empty(n, dtype=torch.int32, device=dev)
    row_ptr = torch.zeros(n + 1, dtype=torch.int32, device=dev)
    count = torch.empty(1, dtype=torch.int64, device=dev)
    def build():
        _lib.check(lib.ptv3_kmap_plan_inner_count(_ptr(plan5.tap_ptr), n, _ptr(pend5.ws), pend5.nbytes, _ptr(found3),
                                                  _ptr(row_cnt), _ptr(plan.tap_ptr), _ptr(count), _stream()),
                   "ptv3_kmap_plan_inner_count")
        plan.n_pairs = Readback(count)
        torch.cumsum(row_cnt, 0, dtype=torch.int32, out=row_ptr[1:])
        plan.row_ptr = row_ptr
        cap = max(plan5.n_pairs, 1)
        plan.pair_in = torch.empty(cap, dtype=torch.int32, device=dev)
        plan.pair_slot = torch.empty(cap, dtype=torch.int32, device=dev)
        _lib.check(lib.ptv3_kmap_plan_inner_fill(_ptr(plan5.tap_ptr), _ptr(plan5.row_ptr), _ptr(plan5.pair_in),
                                                 _ptr(plan5.pair_slot), n, plan5.n_pairs, _ptr(found3), _ptr(plan.tap_ptr),
                                                 _ptr(plan.row_ptr), _ptr(plan.pair_in), _ptr(plan.pair_slot), _stream()),
                   "ptv3_kmap_plan_inner_fill")

    _timed("kmap", (n, 3, "inner"), build)
    return plan


def conv_plan_direct(indices, ks):
    """The pair lists of conv_plan(kmap_build(indices, ks)) straight from the (N,4) int32
    [batch,x,y,z] voxel coordinates, without storing the neighbour map. One read-back (the pair count)."""
    return conv_plan_direct_finish(conv_plan_direct_start(indices, ks))


def subm_conv_pairs(feat, plan, weight, bias=None):
    """Submanifold convolution over the plan's active pairs only (fp16 / bf16)."""
    _dev(feat, weight, bias)
    lib = _lib.load()
    feat = feat.contiguous()
    n, cin = feat.shape
    cout = weight.shape[0]
    w = weight.reshape(cout, plan.taps, cin).to(feat.dtype).contiguous()
    b = None if bias is None else bias.to(feat.dtype).contiguous()
    y = torch.empty((max(plan.n_pairs, 1), cout), dtype=feat.dtype, device=feat.device)
    out = torch.empty((n, cout), dtype=feat.dtype, device=feat.device)

    def call():
        _lib.check(lib.ptv3_subm_conv_pairs_fwd(_ptr(feat), _dtype_code(feat), n, cin, plan.taps, plan.n_pairs,
                                                _ptr(plan.tap_ptr), _ptr(plan.row_ptr), _ptr(plan.pair_in),
                                                _ptr(plan.pair_slot), _ptr(w), _ptr(b), cout, _ptr(y), _ptr(out),
                                                _stream()), "ptv3_subm_conv_pairs_fwd")

    if _LAUNCH_TIMER is not None:
        _LAUNCH_TIMER.launch("subm_conv", (plan.n_pairs, n, cin, cout, plan.taps, "pair"), call)
    else:
        call()
    return out


CONV_TILE_CHANNELS = (64, 128)   # cin == cout widths of the tile form of the 3x3x3 convolution


def conv_pack_weight(weight, taps, dtype):
    """(cout, taps, cin) weight with cin == cout in MFMA fragment order for subm_conv_tiles."""
    _dev(weight)
    lib = _lib.load()
    c = weight.shape[0]
    w = weight.reshape(c, taps, c).to(dtype).contiguous()
    packed = torch.empty_like(w)
    _lib.check(lib.ptv3_subm_conv_pack_weight(_ptr(w), _dtype_code(w), c, taps, _ptr(packed), _stream()),
               "ptv3_subm_conv_pack_weight")
    return packed


TILE_CONV_RESIDENT = 512   # work-groups of the tile form the part holds at a time (two per CU)


def tile_voxels_for(n, channels):
    """Outputs per tile for the tile form: a launch runs in rounds of TILE_CONV_RESIDENT work-groups and costs whole
    rounds; a tile's cost is about a quarter fixed (its 27 weight matrices) and the rest in proportion to its
    outputs. 128 unless tiles of 96 (128 channels only) make the cheaper set of rounds: 146,195 voxels are 2.2
    rounds of 128-voxel tiles (three rounds paid) or 2.97 rounds of 96-voxel ones."""
    if channels != 128:
        return 128
    cost = {tv: -(-(-(-n // tv)) // TILE_CONV_RESIDENT) * (32 + tv) for tv in (128, 96)}
    return 96 if cost[96] < cost[128] else 128


def subm_conv_tiles(feat, plan, packed_weight, bias=None, tile_voxels=None):
    """3x3x3 submanifold convolution with cin == cout, sums kept on chip per tile of outputs (fp16 / bf16)."""
    _dev(feat, packed_weight, bias)
    lib = _lib.load()
    feat = feat.contiguous()
    n, c = feat.shape
    assert packed_weight.dtype == feat.dtype and packed_weight.numel() == plan.taps * c * c
    b = None if bias is None else bias.to(feat.dtype).contiguous()
    out = torch.empty((n, c), dtype=feat.dtype, device=feat.device)
    tv = tile_voxels_for(n, c) if tile_voxels is None else tile_voxels
    tile_tap, tile_pair, vox_taps = plan.tiles(tv)

    def call():
        _lib.check(lib.ptv3_subm_conv_tiles_fwd_sized(_ptr(feat), _dtype_code(feat), n, c, plan.taps, tv,
                                                      _ptr(packed_weight), _ptr(b), _ptr(tile_tap), _ptr(tile_pair),
                                                      _ptr(vox_taps), _ptr(out), _stream()),
                   "ptv3_subm_conv_tiles_fwd_sized")

    if _LAUNCH_TIMER is not None:
        _LAUNCH_TIMER.launch("subm_conv", (plan.n_pairs, n, c, c, plan.taps, "tile"), call)
    else:
        call()
    return out


_PACK_JOB = np.dtype([("weight", "<u8"), ("packed", "<u8"), ("channels", "<i4"), ("taps", "<i4"),
                      ("first_block", "<i8")])   # ptv3_pack_job
_PACK_TABLES = {}


def repack_conv_weights(modules, dtype, device):
    """Packed (fragment-order) copies, in dtype, of the weights of every 3x3x3 cin == cout convolution in `modules`
    whose copy is missing or older than its parameter (parameter_stamp): one launch for all of them. A module keeps
    its copies in module._packed[dtype] = ((stamp, device), tensor); float masters go through cast_cached first."""
    lib = _lib.load()
    jobs, blocks, done = [], 0, []
    for m in list(modules):
        w = m.weight
        if w.device != device or m.kernel_size != 3 or m.in_channels != m.out_channels or m.in_channels % 32:
            continue
        if not isinstance(getattr(m, "_packed", None), dict):
            m._packed = {}
        now = (parameter_stamp(w), w.device)
        held = m._packed.get(dtype)
        if held is not None and held[0] == now:
            continue
        src = cast_cached(w, dtype).detach()
        if not src.is_contiguous():
            src = src.contiguous()
        packed = held[1] if held is not None and held[1].device == device else torch.empty(
            (m.out_channels, 27, m.in_channels), dtype=dtype, device=device)
        jobs.append((src.data_ptr(), packed.data_ptr(), m.in_channels, 27, blocks))
        blocks += lib.ptv3_subm_conv_pack_weight_blocks(m.in_channels, 27)
        done.append((m, now, packed, src))
    if not jobs:
        return
    table = np.array(jobs, dtype=_PACK_JOB).tobytes()
    held = _PACK_TABLES.get((device, dtype))
    if held is None or held[0] != table:
        held = (table, torch.frombuffer(bytearray(table), dtype=torch.uint8).to(device))
        _PACK_TABLES[(device, dtype)] = held
    with torch.cuda.device(device):
        _lib.check(lib.ptv3_subm_conv_pack_weight_batch(held[1].data_ptr(), len(jobs), blocks, _stream()),
                   "ptv3_subm_conv_pack_weight_batch")
    for m, now, packed, _ in done:
        m._packed[dtype] = (now, packed)


CONV_SPARSE_CHANNELS = (32, 64)   # cin == cout widths of the sparse tile form


def subm_conv_sparse(feat, plan, packed_weight, bias=None):
    """3x3x3 submanifold convolution with cin == cout where voxels have few neighbours: the tiles and packed
    weight of subm_conv_tiles, work in proportion to the pairs (fp16 / bf16)."""
    _dev(feat, packed_weight, bias)
    lib = _lib.load()
    feat = feat.contiguous()
    n, c = feat.shape
    assert packed_weight.dtype == feat.dtype and packed_weight.numel() == plan.taps * c * c
    b = None if bias is None else bias.to(feat.dtype).contiguous()
    out = torch.empty((n, c), dtype=feat.dtype, device=feat.device)
    tile_tap, tile_pair, _ = plan.tiles()

    def call():
        _lib.check(lib.ptv3_subm_conv_sparse_fwd(_ptr(feat), _dtype_code(feat), n, c, plan.taps, _ptr(packed_weight),
                                                 _ptr(b), _ptr(tile_tap), _ptr(tile_pair), _ptr(out), _stream()),
                   "ptv3_subm_conv_sparse_fwd")

    if _LAUNCH_TIMER is not None:
        _LAUNCH_TIMER.launch("subm_conv", (plan.n_pairs, n, c, c, plan.taps, "sparse"), call)
    else:
        call()
    return out


class PendingClusters:
    __slots__ = ("cluster", "idx_ptr", "head", "count", "read", "with_offset")


def pool_clusters_start(code0, order0, shift, offset=None):
    """Queues the cluster kernels of pool_clusters and starts the read-back of the cluster count
    (and the pooled scene ends); pool_clusters_finish returns what pool_clusters does."""
    _dev(code0, order0, offset)
    lib = _lib.load()
    n = code0.shape[0]
    dev = code0.device
    order0 = order0.contiguous()
    pend = PendingClusters()
    pend.cluster = torch.empty(n, dtype=torch.int64, device=dev)
    pend.idx_ptr = torch.empty(n + 1, dtype=torch.int64, device=dev)
    pend.head = torch.empty(n, dtype=torch.int64, device=dev)
    nb = 0 if offset is None else offset.shape[0]
    pend.count = torch.empty(1 + nb, dtype=torch.int64, device=dev)   # cluster count, then the pooled scene ends
    pend.with_offset = offset is not None
    off = None if offset is None else offset.to(torch.int64).contiguous()
    nbytes = lib.ptv3_pool_clusters_workspace_bytes(n)
    ws = _ws(nbytes, dev)
    code0 = code0.contiguous()
    _lib.check(lib.ptv3_pool_clusters(_ptr(code0), _ptr(order0), n, int(shift), _ptr(off), nb,
                                      _ptr(pend.cluster), _ptr(pend.idx_ptr), _ptr(pend.head), _ptr(pend.count), _ptr(ws),
                                      nbytes, _stream()), "ptv3_pool_clusters")
    pend.read = Readback(pend.count)
    return pend


def pool_clusters_finish(pend):
    host = pend.read.get()
    m = int(host[0])
    if not pend.with_offset:
        return pend.cluster, pend.idx_ptr[: m + 1], pend.head[:m], m
    return pend.cluster, pend.idx_ptr[: m + 1], pend.head[:m], m, pend.count[1:], [int(v) for v in host[1:]]


def pool_clusters(code0, order0, shift, offset=None):
    """Clusters of code0 >> shift in sorted order. One read-back (the cluster count).

    Returns cluster (N,), idx_ptr (M+1,), head (M,), M; with `offset` (the parent's cumulative
    scene ends, on the device) also the pooled scene ends as a device tensor and as a Python
    list, read in the same device->host copy as the count. Scenes are runs of the sorted order
    (the scene id is the top of every code), so scene b ends with the cluster of its last point."""
    return pool_clusters_finish(pool_clusters_start(code0, order0, shift, offset))


def _row_perm(rows, k):
    """Host int32 array for the row_perm argument of the pooling kernels (None: identity)."""
    if rows is None:
        return None, None
    assert len(rows) == k
    arr = (ctypes.c_int32 * k)(*[int(r) for r in rows])
    return arr, ctypes.cast(arr, ctypes.c_void_p)


def pool_gather(code, shift, grid_coord, pool_depth, batch, head, rows=None):
    """Pooled code (k,M), grid_coord (M,3) int32, batch (M,) at the cluster heads, and the (M,4)
    int32 [batch, x, y, z] indices of the pooled sparse tensor. With rows (a host list), output
    row r of the code comes from input row rows[r]."""
    _dev(code, grid_coord, batch, head)
    lib = _lib.load()
    code = code.contiguous()
    k, n = code.shape
    m = head.shape[0]
    dev = code.device
    code_out = torch.empty((k, m), dtype=torch.int64, device=dev)
    gc = grid_coord.to(torch.int32).contiguous()
    gc_out = torch.empty((m, 3), dtype=torch.int32, device=dev)
    b = batch.to(torch.int64).contiguous()
    b_out = torch.empty(m, dtype=torch.int64, device=dev)
    idx_out = torch.empty((m, 4), dtype=torch.int32, device=dev)
    keep, perm = _row_perm(rows, k)
    _lib.check(lib.ptv3_pool_gather(_ptr(code), n, k, int(shift), _ptr(gc), int(pool_depth), _ptr(b),
                                    _ptr(head.contiguous()), m, perm, _ptr(code_out), _ptr(gc_out), _ptr(b_out),
                                    _ptr(idx_out), _stream()), "ptv3_pool_gather")
    return code_out, gc_out, b_out, idx_out


def pool_orders(order, cluster, m, rows=None):
    """Pooled serialization orders and inverses (k,M) from the parent's orders (k,N) and the
    cluster of every parent point — no sort (see ptv3_pool_orders). With rows (a host list),
    output row r comes from input row rows[r]."""
    _dev(order, cluster)
    lib = _lib.load()
    order = order.contiguous()
    k, n = order.shape
    dev = order.device
    order_out = torch.empty((k, m), dtype=torch.int64, device=dev)
    inverse_out = torch.empty((k, m), dtype=torch.int64, device=dev)
    nbytes = lib.ptv3_pool_orders_workspace_bytes(n, k)
    ws = _ws(nbytes, dev)
    keep, perm = _row_perm(rows, k)
    _lib.check(lib.ptv3_pool_orders(_ptr(order), _ptr(cluster.contiguous()), n, k, int(m), perm, _ptr(order_out),
                                    _ptr(inverse_out), _ptr(ws), nbytes, _stream()), "ptv3_pool_orders")
    return order_out, inverse_out


def segment_reduce(src, indices, idx_ptr, reduce="max"):
    """reduce(src[indices[idx_ptr[s]:idx_ptr[s+1]]]) per segment."""
    _dev(src, indices, idx_ptr)
    lib = _lib.load()
    src = src.contiguous()
    n, c = src.shape
    m = idx_ptr.shape[0] - 1
    out = torch.empty((m, c), dtype=src.dtype, device=src.device)
    _lib.check(lib.ptv3_segment_reduce(_ptr(src), _dtype_code(src), n, c, _ptr(indices.contiguous()),
                                       _ptr(idx_ptr.contiguous()), m, REDUCE_OPS[reduce], _ptr(out),
                                       _stream()), "ptv3_segment_reduce")
    return out


def segment_reduce_bwd(src, out, dout, indices, idx_ptr, reduce="max"):
    """Gradient of segment_reduce with respect to src (every row of src belongs to one segment)."""
    _dev(src, out, dout, indices, idx_ptr)
    lib = _lib.load()
    src, out = src.contiguous(), out.contiguous()
    dout = dout.to(src.dtype).contiguous()
    n, c = src.shape
    m = idx_ptr.shape[0] - 1
    dsrc = torch.empty_like(src)
    _lib.check(lib.ptv3_segment_reduce_bwd(_ptr(src), _ptr(out), _ptr(dout), _dtype_code(src), n, c,
                                           _ptr(indices.contiguous()), _ptr(idx_ptr.contiguous()), m,
                                           REDUCE_OPS[reduce], _ptr(dsrc), _stream()), "ptv3_segment_reduce_bwd")
    return dsrc


def unpool_add(parent, child, cluster):
    """parent + child[cluster]."""
    _dev(parent, child, cluster)
    lib = _lib.load()
    parent = parent.contiguous()
    child = child.to(parent.dtype).contiguous()
    n, c = parent.shape
    out = torch.empty_like(parent)
    _lib.check(lib.ptv3_unpool_add(_ptr(parent), _ptr(child), _dtype_code(parent), n, c,
                                   _ptr(cluster.contiguous()), child.shape[0], _ptr(out), _stream()),
               "ptv3_unpool_add")
    return out


def layer_norm(x, weight, bias, eps=1e-5, residual=None, mode=0, weight2=None, bias2=None, shift=None):
    """Row-wise LayerNorm fused with neighbouring residual adds.

    mode 0: LN(x).  mode 1: residual + LN(x).
    mode 2: (s + shift, LN(s)) with s = x + residual; shift (C,) is optional (the bias of a GEMM
    that will accumulate onto the first result).
    mode 3: (y, LN2(y)) with y = residual + LN(x) and LN2 using weight2/bias2."""
    _dev(x, weight, bias, residual, weight2, bias2, shift)
    lib = _lib.load()
    x = x.contiguous()
    n, c = x.shape
    dt = x.dtype
    w, b = weight.to(dt).contiguous(), bias.to(dt).contiguous()
    res = None if residual is None else residual.to(dt).contiguous()
    w2 = None if weight2 is None else weight2.to(dt).contiguous()
    b2 = None if bias2 is None else bias2.to(dt).contiguous()
    sh = None if shift is None else shift.to(dt).contiguous()
    out0 = torch.empty_like(x)
    out1 = torch.empty_like(x) if mode >= 2 else None
    _lib.check(lib.ptv3_layer_norm(_ptr(x), _ptr(res), _ptr(w), _ptr(b), _ptr(w2), _ptr(b2), _ptr(sh),
                                   _dtype_code(x), n, c, float(eps), int(mode), _ptr(out0), _ptr(out1), _stream()),
               "ptv3_layer_norm")
    return out0 if mode < 2 else (out0, out1)


LAYER_NORM_BWD_CHANNELS = (32, 64, 128, 256, 512)


def _code(t, fallback=0):
    return fallback if t is None else _DTYPE_CODE[t.dtype]


def add_layer_norm(skip, branch, row_scale, weight, bias, eps, sum_dtype=None, out_dtype=None, pre=None):
    """(sum, y) with sum = skip + branch * row_scale and y = LayerNorm(sum), every tensor read and written in its
    own dtype. skip and row_scale (N,) or (N, 1) may be None; sum is returned as None when skip is None (then
    y = LayerNorm(branch * row_scale)). sum_dtype defaults to the promoted dtype of skip and branch, out_dtype to it.
    pre = (weight, bias, eps) of a LayerNorm the branch goes through first, in the same pass."""
    _dev(skip, branch, row_scale, weight, bias)
    lib = _lib.load()
    branch = branch.contiguous()
    n, c = branch.shape
    skip = None if skip is None else skip.contiguous()
    row_scale = None if row_scale is None else row_scale.reshape(-1).contiguous()
    if sum_dtype is None:
        sum_dtype = branch.dtype if skip is None else torch.promote_types(skip.dtype, branch.dtype)
    out_dtype = out_dtype or sum_dtype
    total = None if skip is None else torch.empty((n, c), dtype=sum_dtype, device=branch.device)
    y = torch.empty((n, c), dtype=out_dtype, device=branch.device)
    w = weight.contiguous()
    b = bias.to(w.dtype).contiguous()
    pw = pb = None
    if pre is not None:
        pw, pb = pre[0].to(w.dtype).contiguous(), pre[1].to(w.dtype).contiguous()
    _lib.check(lib.ptv3_add_layer_norm_fwd(_ptr(skip), _code(skip), _ptr(branch), _code(branch), _ptr(row_scale),
                                           _code(row_scale), _ptr(w), _ptr(b), _code(w), n, c, float(eps), _ptr(total),
                                           _DTYPE_CODE[sum_dtype], _ptr(y), _DTYPE_CODE[out_dtype], _ptr(pw), _ptr(pb),
                                           float(pre[2]) if pre is not None else 0.0, _stream()),
               "ptv3_add_layer_norm_fwd")
    return total, y


def add_layer_norm_bwd(total, dy, dsum, row_scale, weight, eps, skip_dtype=None, branch_dtype=None, pre=None):
    """Backward of add_layer_norm: (dskip, dbranch, dweight, dbias); total is the sum the forward normalised, dsum
    the gradient reaching it past the LayerNorm (or None). dskip / dbranch are made in the given dtypes and are
    None where the dtype is None; dweight, dbias in fp32. pre = (x, weight, eps) of the LayerNorm the branch went
    through first (x its input): dbranch is then x's gradient, and that norm's (dweight, dbias) are returned too."""
    _dev(total, dy, dsum, row_scale, weight)
    lib = _lib.load()
    total, dy = total.contiguous(), dy.contiguous()
    dsum = None if dsum is None else dsum.contiguous()
    row_scale = None if row_scale is None else row_scale.reshape(-1).contiguous()
    n, c = total.shape
    dev = total.device
    dskip = None if skip_dtype is None else torch.empty((n, c), dtype=skip_dtype, device=dev)
    dbranch = None if branch_dtype is None else torch.empty((n, c), dtype=branch_dtype, device=dev)
    dwb = torch.zeros((4 if pre is not None else 2, c), dtype=torch.float32, device=dev)
    w = weight.contiguous()
    px = pw = None
    if pre is not None:
        px, pw = pre[0].contiguous(), pre[1].to(w.dtype).contiguous()
    _lib.check(lib.ptv3_add_layer_norm_bwd(_ptr(total), _code(total), _ptr(dy), _code(dy), _ptr(dsum), _code(dsum),
                                           _ptr(row_scale), _code(row_scale), _ptr(w), _code(w), n, c, float(eps),
                                           _ptr(dskip), _code(dskip), _ptr(dbranch), _code(dbranch), _ptr(dwb[0]),
                                           _ptr(dwb[1]), _ptr(px), _code(px), _ptr(pw),
                                           float(pre[2]) if pre is not None else 0.0,
                                           _ptr(dwb[2]) if pre is not None else None,
                                           _ptr(dwb[3]) if pre is not None else None, _stream()),
               "ptv3_add_layer_norm_bwd")
    if pre is not None:
        return dskip, dbranch, dwb[0], dwb[1], dwb[2], dwb[3]
    return dskip, dbranch, dwb[0], dwb[1]


def scaled_add(skip, branch, row_scale, out_dtype):
    """skip + branch * row_scale in out_dtype, each input read in its own dtype (ptv3_scaled_add); skip and
    row_scale (N,) or (N, 1) may be None."""
    _dev(skip, branch, row_scale)
    branch = branch.contiguous()
    n, c = branch.shape
    skip = None if skip is None else skip.contiguous()
    row_scale = None if row_scale is None else row_scale.reshape(-1).contiguous()
    out = torch.empty((n, c), dtype=out_dtype, device=branch.device)
    _lib.check(_lib.load().ptv3_scaled_add(_ptr(skip), _code(skip), _ptr(branch), _code(branch), _ptr(row_scale),
                                           _code(row_scale), n, c, _ptr(out), _DTYPE_CODE[out_dtype], _stream()),
               "ptv3_scaled_add")
    return out


LINEAR_LN_CHANNELS = (128, 256)   # square Linear + LayerNorm(s) + residual in one kernel
# where that measured faster than Linear kernel + LayerNorm kernel on MI355X: at 128 channels (weights in LDS;
# 146k rows: 35 us against 42-49) and at 256 (weights in registers, the LayerNorm sums exchanged between the four
# waves of a row through LDS; 38k rows: 25-27 us against 37-41)
LINEAR_LN_PAYS = (128, 256)


def linear_ln_ok(x, lin):
    return (x.is_cuda and x.dtype in (torch.float16, torch.bfloat16) and x.dim() == 2 and type(lin) is torch.nn.Linear
            and lin.in_features == lin.out_features and lin.in_features in LINEAR_LN_PAYS)


def linear_ln(x, lin, residual, ln, mode, ln2=None, shift=None):
    """layer_norm(lin(x), ..., residual=residual, mode=mode, ...) for a square nn.Linear in one kernel
    (modes 2 and 3 of layer_norm; same rounding points). Returns (out0, out1)."""
    _dev(x, lin.weight, residual, ln.weight)
    lib = _lib.load()
    x = x.contiguous()
    n, c = x.shape
    dt = x.dtype
    cast = lambda t: None if t is None else t.to(dt).contiguous()
    w, b, res = cast(lin.weight), cast(lin.bias), cast(residual)
    g1, b1 = cast(ln.weight), cast(ln.bias)
    g2, b2 = (cast(ln2.weight), cast(ln2.bias)) if ln2 is not None else (None, None)
    sh = cast(shift)
    out0, out1 = torch.empty_like(x), torch.empty_like(x)
    _lib.check(lib.ptv3_linear_ln_fwd(_ptr(x), _ptr(w), _ptr(b), _ptr(res), _ptr(g1), _ptr(b1), _ptr(g2), _ptr(b2), _ptr(sh),
                                      _dtype_code(x), n, c, int(mode), float(ln.eps), _ptr(out0), _ptr(out1), _stream()),
               "ptv3_linear_ln_fwd")
    return out0, out1


LINEAR_ROWS_IN = (32, 64, 128, 256, 512)   # input widths of the tall-and-skinny Linear kernel


def linear_rows_ok(x, weight):
    """True when linear_rows covers this layer: half precision, 32 ... 512 inputs, outputs in 32s."""
    return (x.is_cuda and x.dtype in (torch.float16, torch.bfloat16) and x.dim() == 2
            and weight.shape[1] in LINEAR_ROWS_IN and weight.shape[0] % 32 == 0)


def linear_rows_pays(x, weight, gelu=False):
    """Where the tall-and-skinny kernel measured at least as fast as a tiled GEMM (+ GELU launch) on
    MI355X: everything up to 256 inputs, all but the 3x-wide qkv at 512."""
    if not linear_rows_ok(x, weight):
        return False
    nout, k = weight.shape
    return k <= 256 or gelu or nout <= 2 * k


def linear(x, mod, gelu=False):
    """mod(x) for an nn.Linear (followed by exact GELU if gelu), on whichever path is faster."""
    if wants_grad(x, mod.weight, mod.bias):
        w, b = mod.weight, mod.bias
        xa = x.to(torch.get_autocast_dtype("cuda")) if (torch.is_autocast_enabled() and x.is_cuda) else x
        if (xa.is_cuda and xa.dim() == 2 and xa.dtype in (torch.float16, torch.bfloat16)
                and w.shape[0] % 8 == 0 and w.shape[1] % 8 == 0):
            from .autograd import Linear
            y = Linear.apply(xa, w, b)   # the weight gradient is a reduction over all rows: own kernel
            return torch.nn.functional.gelu(y) if gelu else y
        if not torch.is_autocast_enabled() and w.dtype != x.dtype:
            w, b = w.to(x.dtype), None if b is None else b.to(x.dtype)
        y = torch.nn.functional.linear(x, w, b)
        return torch.nn.functional.gelu(y) if gelu else y
    if linear_rows_pays(x, mod.weight, gelu):
        return linear_rows(x, mod.weight, mod.bias, gelu)
    if not gelu and linear_gemm_ok(x, mod.weight):
        return linear_gemm(x, mod.weight, mod.bias)
    return linear_any(x, mod.weight, mod.bias, gelu=gelu)


def linear_gelu(x, weight, bias=None):
    """(pre, gelu(pre)) with pre = x W^T + b from one pass over the rows (ptv3_linear_gelu_fwd): the training
    form of fc1 + act, which keeps the GELU's input for the backward."""
    _dev(x, weight, bias)
    x = x.contiguous()
    n, k = x.shape
    w = weight.to(x.dtype).contiguous()
    b = None if bias is None else bias.to(x.dtype).contiguous()
    pre = torch.empty((n, w.shape[0]), dtype=x.dtype, device=x.device)
    out = torch.empty_like(pre)
    _lib.check(_lib.load().ptv3_linear_gelu_fwd(_ptr(x), _ptr(w), _ptr(b), _dtype_code(x), n, k, w.shape[0], _ptr(pre),
                                                _ptr(out), _stream()), "ptv3_linear_gelu_fwd")
    return pre, out


def linear_gelu_bwd(dout, weight_t, pre):
    """(dout weight_t^T) * gelu'(pre): the gradient of fc2's output taken back to the GELU's input in one pass
    (ptv3_linear_gelu_bwd). weight_t (hidden, out) is fc2's weight transposed."""
    _dev(dout, weight_t, pre)
    dout, pre = dout.contiguous(), pre.contiguous()
    n, k = dout.shape
    w = weight_t.to(dout.dtype).contiguous()
    if pre.shape != (n, w.shape[0]) or pre.dtype != dout.dtype:
        raise _lib.Ptv3Error("linear_gelu_bwd: pre must be (rows, hidden) in dout's dtype")
    dpre = torch.empty_like(pre)
    _lib.check(_lib.load().ptv3_linear_gelu_bwd(_ptr(dout), _ptr(w), _ptr(pre), _dtype_code(dout), n, k, w.shape[0],
                                                _ptr(dpre), _stream()), "ptv3_linear_gelu_bwd")
    return dpre


def mlp(x, fc1, fc2):
    """fc2(gelu(fc1(x))) for two nn.Linear under autograd: the GELU rides on fc1's kernel going forward and on
    fc2's input gradient going back. None where the fused form does not apply (the caller takes the modules
    one by one)."""
    xa = x.to(torch.get_autocast_dtype("cuda")) if (torch.is_autocast_enabled() and x.is_cuda) else x
    if not (xa.is_cuda and xa.dim() == 2 and xa.dtype in (torch.float16, torch.bfloat16)
            and fc1.weight.dtype in (torch.float32, xa.dtype) and fc2.weight.dtype == fc1.weight.dtype
            and linear_rows_ok(xa, fc1.weight) and fc2.weight.shape[0] % 32 == 0
            and fc2.weight.shape[0] in (32, 64, 128, 256, 512)):
        return None
    from .autograd import Mlp
    return Mlp.apply(xa, fc1.weight, fc1.bias, fc2.weight, fc2.bias)


def linear_gemm(x, weight, bias=None, resid=None):
    """resid + x W^T + b through the tiled GEMM kernel (ptv3_linear_gemm_fwd): any number of inputs in 128s, outputs
    in 128s, fp16 / bf16. With resid the result is written over it (fc2 accumulating onto the stored sum)."""
    _dev(x, weight, bias, resid)
    x = x.contiguous()
    n, k = x.shape
    w = weight.to(x.dtype).contiguous()
    b = None if bias is None else bias.to(x.dtype).contiguous()
    if resid is not None and not (resid.is_contiguous() and resid.dtype == x.dtype and resid.shape == (n, w.shape[0])):
        raise _lib.Ptv3Error("linear_gemm: resid must be a contiguous (rows, outputs) tensor of x's dtype")
    out = resid if resid is not None else torch.empty((n, w.shape[0]), dtype=x.dtype, device=x.device)
    _lib.check(_lib.load().ptv3_linear_gemm_fwd(_ptr(x), _ptr(w), _ptr(b), _ptr(resid), _dtype_code(x), n, k, w.shape[0],
                                                _ptr(out), _stream()), "ptv3_linear_gemm_fwd")
    return out


def linear_any(x, weight, bias=None, gelu=False, resid=None):
    """resid + act(x W^T + b) for any shape and fp32 / fp16 / bf16 (ptv3_linear_any_fwd): the fp32 model and the
    half-precision widths the MFMA kernels do not take. x may have leading dimensions; with resid the result is
    written over it."""
    _dev(x, weight, bias, resid)
    if x.dtype not in _DTYPE_CODE:
        raise _lib.Ptv3Error(f"linear: unsupported dtype {x.dtype}")
    lead = x.shape[:-1]
    x2 = x.reshape(-1, x.shape[-1]).contiguous()
    n, k = x2.shape
    w = weight.to(x.dtype).contiguous()
    b = None if bias is None else bias.to(x.dtype).contiguous()
    if w.dim() != 2 or w.shape[1] != k:
        raise _lib.Ptv3Error(f"linear: weight {tuple(w.shape)} does not take {k} inputs")
    if resid is not None and not (resid.is_contiguous() and resid.dtype == x.dtype and resid.shape == (n, w.shape[0])):
        raise _lib.Ptv3Error("linear_any: resid must be a contiguous (rows, outputs) tensor of x's dtype")
    out = resid if resid is not None else torch.empty((n, w.shape[0]), dtype=x.dtype, device=x.device)
    _lib.check(_lib.load().ptv3_linear_any_fwd(_ptr(x2), _ptr(w), _ptr(b), _ptr(resid), _dtype_code(x2), n, k, w.shape[0],
                                               int(bool(gelu)), _ptr(out), _stream()), "ptv3_linear_any_fwd")
    return out if resid is not None else out.reshape(*lead, w.shape[0])


def linear_gemm_ok(x, weight):
    return (x.is_cuda and x.dim() == 2 and x.dtype in (torch.float16, torch.bfloat16) and weight.shape[1] % 128 == 0
            and weight.shape[0] % 128 == 0)


LINEAR_WIDE = True   # 256 inputs, outputs in 256s: the kernel with the weights resident in registers


def linear_rows(x, weight, bias=None, gelu=False):
    """act(x W^T + b) for many rows and few channels (see ptv3_linear_fwd); act = exact GELU if gelu."""
    _dev(x, weight, bias)
    lib = _lib.load()
    x = x.contiguous()
    n, k = x.shape
    w = weight.to(x.dtype).contiguous()
    b = None if bias is None else bias.to(x.dtype).contiguous()
    out = torch.empty((n, w.shape[0]), dtype=x.dtype, device=x.device)
    if LINEAR_WIDE and k == 256 and w.shape[0] % 256 == 0 and n >= 4096:
        _lib.check(lib.ptv3_linear_wide_fwd(_ptr(x), _ptr(w), _ptr(b), _dtype_code(x), n, k, w.shape[0], int(bool(gelu)),
                                            _ptr(out), _stream()), "ptv3_linear_wide_fwd")
        return out
    _lib.check(lib.ptv3_linear_fwd(_ptr(x), _ptr(w), _ptr(b), _dtype_code(x), n, k, w.shape[0], int(bool(gelu)),
                                   _ptr(out), _stream()), "ptv3_linear_fwd")
    return out


def linear_wgrad(x, dout, with_bias=False):
    """dout^T x in fp32, (Nout, K): the weight gradient of a Linear over many rows (fp16 / bf16); with_bias:
    also the column sums of dout (Nout,), the bias gradient, from the same pass."""
    _dev(x, dout)
    lib = _lib.load()
    x = x.contiguous()
    dout = dout.to(x.dtype).contiguous()
    n, k = x.shape
    nout = dout.shape[1]
    dw = torch.empty((nout, k), dtype=torch.float32, device=x.device)
    db = torch.empty(nout, dtype=torch.float32, device=x.device) if with_bias else None
    nbytes = lib.ptv3_linear_wgrad_workspace_bytes(n, k, nout)
    ws = _ws(nbytes, x.device) if nbytes else None
    _lib.check(lib.ptv3_linear_wgrad(_ptr(x), _ptr(dout), _dtype_code(x), n, k, nout, _ptr(dw), _ptr(db), _ptr(ws),
                                     nbytes, _stream()), "ptv3_linear_wgrad")
    return (dw, db) if with_bias else dw


def linear_bn_act(x, lin, bn, gelu):
    """gelu?(BatchNorm1d_inference(lin(x))) in one kernel for the layers linear_rows covers."""
    _dev(x, lin.weight, bn.running_mean)
    lib = _lib.load()
    x = x.contiguous()
    n, k = x.shape
    dt = x.dtype
    w = lin.weight.to(dt).contiguous()
    b = None if lin.bias is None else lin.bias.to(dt).contiguous()
    mean, var = bn.running_mean, bn.running_var
    stats_f32 = mean.dtype == torch.float32
    if not stats_f32 and mean.dtype != dt:
        mean, var, stats_f32 = mean.float(), var.float(), True
    g = None if bn.weight is None else bn.weight.to(dt).contiguous()
    be = None if bn.bias is None else bn.bias.to(dt).contiguous()
    out = torch.empty((n, w.shape[0]), dtype=dt, device=x.device)
    _lib.check(lib.ptv3_linear_bn_act_fwd(_ptr(x), _ptr(w), _ptr(b), _ptr(mean.contiguous()), _ptr(var.contiguous()),
                                          int(stats_f32), _ptr(g), _ptr(be), float(bn.eps), _dtype_code(x), n, k,
                                          w.shape[0], int(bool(gelu)), _ptr(out), _stream()), "ptv3_linear_bn_act_fwd")
    return out


MLP_FUSED_CHANNELS = (32, 64)             # widths of the fused block head / tail kernels
MLP_ONLY_FUSED_CHANNELS = (32, 64, 128, 256, 512)   # widths the fused MLP kernel supports
# widths at which the model uses it. At 32 ... 128 it beats fc1 + GELU and fc2 as separate launches by 1.8-2.4x; at
# 256 and 512 it is on a par with fc1 + GELU (linear_wide) and fc2 (tiled GEMM) as separate launches and keeps the
# 4C-wide hidden tensor out of HBM; (32, 64, 128) restores the separate layers there
MLP_ONLY_FUSED_PAYS = (32, 64, 128, 256, 512)


def mlp_fused(x, resid, w1, b1, w2, b2):
    """resid + fc2(GELU(fc1(x))) in one kernel (exact GELU). x, resid (N,C) fp16/bf16 with C in
    MLP_ONLY_FUSED_CHANNELS; w1 (4C,C), b1 (4C,), w2 (C,4C), b2 (C,)."""
    _dev(x, resid, w1, b1, w2, b2)
    lib = _lib.load()
    x = x.contiguous()
    resid = resid.to(x.dtype).contiguous()
    n, c = x.shape
    dt = x.dtype
    w1c, b1c, w2c, b2c = (t.to(dt).contiguous() for t in (w1, b1, w2, b2))
    out = torch.empty_like(x)
    _lib.check(lib.ptv3_mlp_fused(_ptr(x), _ptr(resid), _ptr(w1c), _ptr(b1c), _ptr(w2c), _ptr(b2c), _dtype_code(x),
                                  n, c, w1c.shape[0], _ptr(out), _stream()), "ptv3_mlp_fused")
    return out


MLP_PACKED_CHANNELS = (128, 256, 512)               # widths whose fused MLP streams its weights from a packed copy


def mlp_pack_weights(w1, w2, dtype, out=None):
    """fc1's (4C, C) and fc2's (C, 4C) weights in the order the wide fused MLP kernel streams them, as one
    tensor of 8 C^2 elements of dtype (ptv3_mlp_pack_weights); written into `out` when given."""
    _dev(w1, w2)
    lib = _lib.load()
    c = w2.shape[0]
    assert c in MLP_PACKED_CHANNELS and tuple(w1.shape) == (4 * c, c) and tuple(w2.shape) == (c, 4 * c)
    w1c, w2c = w1.detach().to(dtype).contiguous(), w2.detach().to(dtype).contiguous()
    if out is None:
        out = torch.empty(8 * c * c, dtype=dtype, device=w1.device)
    assert out.dtype == dtype and out.numel() == 8 * c * c and out.is_contiguous()
    _lib.check(lib.ptv3_mlp_pack_weights(_ptr(w1c), _ptr(w2c), _DTYPE_CODE[dtype], c, _ptr(out), _stream()),
               "ptv3_mlp_pack_weights")
    return out


def mlp_fused_packed(x, resid, packed, b1, b2):
    """mlp_fused with the weights as mlp_pack_weights leaves them (C in MLP_PACKED_CHANNELS): same results."""
    _dev(x, resid, packed, b1, b2)
    lib = _lib.load()
    x = x.contiguous()
    resid = resid.to(x.dtype).contiguous()
    n, c = x.shape
    dt = x.dtype
    assert packed.dtype == dt and packed.numel() == 8 * c * c
    b1c, b2c = b1.to(dt).contiguous(), b2.to(dt).contiguous()
    out = torch.empty_like(x)
    _lib.check(lib.ptv3_mlp_fused_packed(_ptr(x), _ptr(resid), _ptr(packed), _ptr(b1c), _ptr(b2c), _dtype_code(x),
                                         n, c, _ptr(out), _stream()), "ptv3_mlp_fused_packed")
    return out


_MLP_PACK_JOB = np.dtype([("w1", "<u8"), ("w2", "<u8"), ("packed", "<u8"), ("channels", "<i4"), ("reserved", "<i4"),
                          ("first_block", "<i8")])
_MLP_PACK_TABLES = {}
_MLP_PACK_USERS = weakref.WeakSet()   # the MLPs that have asked for packed weights: one stale copy has all redone


class HeadWeights:
    """The two Linear layers whose weights block_head_wide streams from one packed copy: the xCPE's C -> C and the
    attention's C -> 3C. Lives on the qkv module (so that it lasts as long as the layers) and holds the copy."""

    def __init__(self, cpe_linear, qkv_linear):
        self.parts = (cpe_linear, qkv_linear)

    @staticmethod
    def of(cpe_linear, qkv_linear):
        held = qkv_linear.__dict__.get("_head_weights")
        if held is None or held.parts[0] is not cpe_linear:
            held = qkv_linear.__dict__["_head_weights"] = HeadWeights(cpe_linear, qkv_linear)
        return held


def _pack_parts(m):
    """What a module's packed copy is made of: [(weight, rows / C or None for the MLP pair)], and C."""
    if isinstance(m, HeadWeights):
        c = m.parts[0].weight.shape[0]
        ok = tuple(m.parts[0].weight.shape) == (c, c) and tuple(m.parts[1].weight.shape) == (3 * c, c)
        return [(m.parts[0].weight, 1), (m.parts[1].weight, 3)], c, ok
    if hasattr(m, "fc1"):
        c = m.fc2.weight.shape[0]
        ok = tuple(m.fc1.weight.shape) == (4 * c, c) and tuple(m.fc2.weight.shape) == (c, 4 * c)
        return [(m.fc1.weight, None), (m.fc2.weight, None)], c, ok
    c = m.weight.shape[0]
    return [(m.weight, 1)], c, tuple(m.weight.shape) == (c, c)


def _pack_stamp(m, device):
    """What a module's packed copy was made from: the stamps of its weights."""
    mods = getattr(m, "_modules", None)
    if mods is not None and "fc1" in mods:   # an MLP, asked for at every use: without the lists of _pack_parts
        return (parameter_stamp(mods["fc1"]._parameters["weight"]), parameter_stamp(mods["fc2"]._parameters["weight"]), device)
    return tuple(parameter_stamp(w) for w, _ in _pack_parts(m)[0]) + (device,)


def repack_mlp_weights(modules, dtype, device):
    """Packed weight streams, in dtype, of every module in `modules` whose copy is missing or older than its
    parameters (parameter_stamp), one launch for all of them: MLPs (fc1: C -> 4C, fc2: 4C -> C), square Linear
    layers (C -> C, the attention's projection for block_tail_wide) and HeadWeights pairs (block_head_wide), C in
    MLP_PACKED_CHANNELS. A module keeps its copies in module._packed_stream[dtype] = ((stamps, device), tensor),
    redone in place."""
    lib = _lib.load()
    jobs, blocks, done = [], 0, []
    for m in list(modules):
        parts, c, ok = _pack_parts(m)
        if parts[0][0].device != device or c not in MLP_PACKED_CHANNELS or not ok:
            continue
        held = m.__dict__.setdefault("_packed_stream", {})
        now = _pack_stamp(m, device)
        entry = held.get(dtype)
        if entry is not None and entry[0] == now:
            continue
        srcs = [cast_cached(w, dtype).detach().contiguous() for w, _ in parts]
        mlp_pair = parts[0][1] is None
        total = 8 * c * c if mlp_pair else sum(k for _, k in parts) * c * c
        packed = entry[1] if entry is not None and entry[1].device == device else torch.empty(total, dtype=dtype, device=device)
        if mlp_pair:
            jobs.append((srcs[0].data_ptr(), srcs[1].data_ptr(), packed.data_ptr(), c, 0, blocks))
            blocks += lib.ptv3_mlp_pack_weights_blocks(c)
        else:
            at = 0
            for src, (_, k) in zip(srcs, parts):
                jobs.append((src.data_ptr(), 0, packed.data_ptr() + at * c * c * packed.element_size(), c, k, blocks))
                blocks += k * lib.ptv3_linear_pack_weights_blocks(c)
                at += k
        done.append((held, now, packed, srcs))
    if not jobs:
        return
    table = np.array(jobs, dtype=_MLP_PACK_JOB).tobytes()
    kept = _MLP_PACK_TABLES.get((device, dtype))
    if kept is None or kept[0] != table:
        kept = (table, torch.frombuffer(bytearray(table), dtype=torch.uint8).to(device))
        _MLP_PACK_TABLES[(device, dtype)] = kept
    with torch.cuda.device(device):
        _lib.check(lib.ptv3_mlp_pack_weights_batch(kept[1].data_ptr(), len(jobs), blocks, _stream()),
                   "ptv3_mlp_pack_weights_batch")
    for held, now, packed, _ in done:
        held[dtype] = (now, packed)


_IDLE_WORK.append(lambda: [repack_mlp_weights(_MLP_PACK_USERS, dtype, device) for device, dtype in list(_MLP_PACK_TABLES)])


def _packed_stream(m, dtype):
    """The module's packed copy in dtype, redone first (with every other stale one) when its parameters moved."""
    held = m.__dict__.get("_packed_stream")
    entry = held.get(dtype) if held else None
    # weights that moved to another device have other addresses: their stamp differs from the one held
    if entry is None or entry[0] != _pack_stamp(m, entry[0][-1]):
        _MLP_PACK_USERS.add(m)
        repack_mlp_weights(_MLP_PACK_USERS, dtype, _pack_parts(m)[0][0][0].device)
        entry = m._packed_stream[dtype]
    return entry[1]


BLOCK_TAIL_WIDE_CHANNELS = (128, 256)
# block_head_wide takes the same widths; where it measured faster than linear_ln + qkv Linear: 74 -> 59 us at
# 146k x 128, 46.5 -> 46 us at 37.7k x 256 (a pass there is too short for what it costs to start and to leave)
BLOCK_HEAD_WIDE_PAYS = (128,)


def block_tail_wide(attn, shortcut, proj, ln2, mlp):
    """sum = shortcut + proj(attn); returns sum + mlp.fc2(GELU(mlp.fc1(ln2(sum)))) from one kernel: the second half
    of a block (model.py:458-460, :595-602) at BLOCK_TAIL_WIDE_CHANNELS. attn, shortcut (N, C) fp16/bf16; proj a
    Linear C -> C, ln2 an affine LayerNorm, mlp with fc1: C -> 4C and fc2: 4C -> C (all with biases). The weights go
    through the modules' packed copies (repack_mlp_weights)."""
    _dev(attn, shortcut, proj.weight, mlp.fc1.weight, mlp.fc2.weight)
    lib = _lib.load()
    attn = attn.contiguous()
    dt = attn.dtype
    shortcut = shortcut.to(dt).contiguous()
    n, c = attn.shape
    assert c in (128, 256) and tuple(shortcut.shape) == (n, c)
    mlp_packed, proj_packed = _packed_stream(mlp, dt), _packed_stream(proj, dt)
    keep = [cast_cached(t, dt).detach().contiguous() for t in (proj.bias, ln2.weight, ln2.bias, mlp.fc1.bias, mlp.fc2.bias)]
    out = torch.empty_like(attn)
    _lib.check(lib.ptv3_block_tail_wide(_ptr(attn), _ptr(shortcut), _ptr(proj_packed), _ptr(keep[0]), _ptr(keep[1]),
                                        _ptr(keep[2]), float(ln2.eps), _ptr(mlp_packed), _ptr(keep[3]), _ptr(keep[4]),
                                        _dtype_code(attn), n, c, _ptr(out), _stream()), "ptv3_block_tail_wide")
    return out


def mlp_fused_module(x, resid, mlp):
    """resid + mlp(x) from the fused kernel for a module with fc1 and fc2. At MLP_PACKED_CHANNELS the weights go
    through a packed copy that the module keeps per dtype and that is redone, in place, when a parameter may have
    changed (parameter_stamp) -- together with every other module's that is stale, in one launch."""
    if x.shape[1] not in MLP_PACKED_CHANNELS:
        return mlp_fused(x, resid, mlp.fc1.weight, mlp.fc1.bias, mlp.fc2.weight, mlp.fc2.bias)
    return mlp_fused_packed(x, resid, _packed_stream(mlp, x.dtype), mlp.fc1.bias, mlp.fc2.bias)


def _opt(t, dt):
    return None if t is None else t.to(dt).contiguous()


def block_head_fused(conv, shortcut, cpe_linear, ln_cpe, ln1, qkv_linear):
    """feat = shortcut + ln_cpe(cpe_linear(conv)); qkv = qkv_linear(ln1(feat)) in one kernel.
    conv, shortcut (N,C) fp16/bf16 with C in MLP_FUSED_CHANNELS; the modules are a Linear C->C,
    two LayerNorms and a Linear C->3C. Returns (feat, qkv)."""
    _dev(conv, shortcut, cpe_linear.weight, qkv_linear.weight)
    lib = _lib.load()
    conv = conv.contiguous()
    dt = conv.dtype
    shortcut = shortcut.to(dt).contiguous()
    n, c = conv.shape
    keep = [_opt(t, dt) for t in (cpe_linear.weight, cpe_linear.bias, ln_cpe.weight, ln_cpe.bias, ln1.weight,
                                   ln1.bias, qkv_linear.weight, qkv_linear.bias)]
    feat = torch.empty_like(conv)
    qkv = torch.empty((n, 3 * c), dtype=dt, device=conv.device)
    _lib.check(lib.ptv3_block_head_fused(_ptr(conv), _ptr(shortcut), _ptr(keep[0]), _ptr(keep[1]), _ptr(keep[2]),
                                         _ptr(keep[3]), float(ln_cpe.eps), _ptr(keep[4]), _ptr(keep[5]),
                                         float(ln1.eps), _ptr(keep[6]), _ptr(keep[7]), _dtype_code(conv), n, c,
                                         _ptr(feat), _ptr(qkv), _stream()), "ptv3_block_head_fused")
    return feat, qkv


def block_tail_fused(attn, shortcut, proj, ln2, fc1, fc2):
    """feat = shortcut + proj(attn); returns feat + fc2(GELU(fc1(ln2(feat)))) from one kernel.
    attn, shortcut (N,C) fp16/bf16 with C in MLP_FUSED_CHANNELS and fc1: C->4C."""
    _dev(attn, shortcut, proj.weight, fc1.weight, fc2.weight)
    lib = _lib.load()
    attn = attn.contiguous()
    dt = attn.dtype
    shortcut = shortcut.to(dt).contiguous()
    n, c = attn.shape
    keep = [_opt(t, dt) for t in (proj.weight, proj.bias, ln2.weight, ln2.bias, fc1.weight, fc1.bias, fc2.weight,
                                   fc2.bias)]
    out = torch.empty_like(attn)
    _lib.check(lib.ptv3_block_tail_fused(_ptr(attn), _ptr(shortcut), _ptr(keep[0]), _ptr(keep[1]), _ptr(keep[2]),
                                         _ptr(keep[3]), float(ln2.eps), _ptr(keep[4]), _ptr(keep[5]), _ptr(keep[6]),
                                         _ptr(keep[7]), _dtype_code(attn), n, c, keep[4].shape[0], _ptr(out),
                                         _stream()), "ptv3_block_tail_fused")
    return out


def block_head_wide(conv, shortcut, cpe_linear, ln_cpe, ln1, qkv_linear):
    """feat = shortcut + ln_cpe(cpe_linear(conv)); qkv = qkv_linear(ln1(feat)) in one kernel at
    BLOCK_TAIL_WIDE_CHANNELS (model.py:541-545, :587-593, :450). conv, shortcut (N, C) fp16/bf16; the modules are a
    Linear C -> C, two affine LayerNorms and a Linear C -> 3C, all with biases. Returns (feat, qkv). The weights go
    through one packed copy of both matrices (HeadWeights, repack_mlp_weights)."""
    _dev(conv, shortcut, cpe_linear.weight, qkv_linear.weight)
    lib = _lib.load()
    conv = conv.contiguous()
    dt = conv.dtype
    shortcut = shortcut.to(dt).contiguous()
    n, c = conv.shape
    assert c in (128, 256) and tuple(shortcut.shape) == (n, c)
    packed = _packed_stream(HeadWeights.of(cpe_linear, qkv_linear), dt)
    keep = [cast_cached(t, dt).detach().contiguous() for t in (cpe_linear.bias, ln_cpe.weight, ln_cpe.bias, ln1.weight,
                                                                ln1.bias, qkv_linear.bias)]
    feat = torch.empty_like(conv)
    qkv = torch.empty((n, 3 * c), dtype=dt, device=conv.device)
    _lib.check(lib.ptv3_block_head_wide(_ptr(conv), _ptr(shortcut), _ptr(packed), _ptr(keep[0]), _ptr(keep[1]),
                                        _ptr(keep[2]), float(ln_cpe.eps), _ptr(keep[3]), _ptr(keep[4]), float(ln1.eps),
                                        _ptr(keep[5]), _dtype_code(conv), n, c, _ptr(feat), _ptr(qkv), _stream()),
               "ptv3_block_head_wide")
    return feat, qkv


BATCH_NORM_TRAIN_CHANNELS = (32, 64, 128, 256, 512)


def batch_norm_stats(x, eps, momentum=0.0, running_mean=None, running_var=None):
    """(3, C) fp32: mean, rsqrt(var + eps) and biased variance of the rows of x; float32 running averages, when
    given, are updated in place as a BatchNorm1d in training mode does."""
    _dev(x, running_mean, running_var)
    lib = _lib.load()
    x = x.contiguous()
    n, c = x.shape
    stats = torch.empty((3, c), dtype=torch.float32, device=x.device)
    ws = torch.empty(2 * c, dtype=torch.float32, device=x.device)
    _lib.check(lib.ptv3_batch_norm_stats(_ptr(x), _dtype_code(x), n, c, float(eps), float(momentum), _ptr(running_mean),
                                         _ptr(running_var), _ptr(stats), _ptr(ws), _stream()), "ptv3_batch_norm_stats")
    return stats


def batch_norm_bwd(x, dout, stats, weight, bias, gelu, batch_stats):
    """(dx, dweight, dbias) of [GELU of] BatchNorm1d over the rows of x; stats[0] = mean, stats[1] = rstd; the
    parameter gradients in fp32."""
    _dev(x, dout, stats, weight, bias)
    lib = _lib.load()
    x, dout = x.contiguous(), dout.contiguous()
    n, c = x.shape
    dx = torch.empty_like(x)
    dwb = torch.empty((2, c), dtype=torch.float32, device=x.device)
    w = None if weight is None else weight.contiguous()
    b = None if bias is None else bias.to(w.dtype if w is not None else bias.dtype).contiguous()
    _lib.check(lib.ptv3_batch_norm_bwd(_ptr(x), _dtype_code(x), _ptr(dout), _dtype_code(dout), _ptr(stats), _ptr(w), _ptr(b),
                                       _code(w if w is not None else b), n, c, int(bool(gelu)), int(bool(batch_stats)),
                                       _ptr(dx), _dtype_code(dx), _ptr(dwb), _stream()), "ptv3_batch_norm_bwd")
    return dx, dwb[0], dwb[1]


def bn_act(x, running_mean, running_var, weight, bias, eps, gelu):
    """Inference-mode BatchNorm1d, optionally followed by exact GELU, in one pass. The running
    statistics may be float32 or of x's dtype."""
    _dev(x, running_mean, running_var, weight, bias)
    lib = _lib.load()
    x = x.contiguous()
    n, c = x.shape
    dt = x.dtype
    stats_f32 = running_mean.dtype == torch.float32
    if not stats_f32 and running_mean.dtype != dt:
        running_mean, running_var, stats_f32 = running_mean.float(), running_var.float(), True
    w = None if weight is None else weight.to(dt).contiguous()
    b = None if bias is None else bias.to(dt).contiguous()
    out = torch.empty_like(x)
    _lib.check(lib.ptv3_bn_act(_ptr(x), _ptr(running_mean.contiguous()), _ptr(running_var.contiguous()),
                               int(stats_f32), _ptr(w), _ptr(b), _dtype_code(x), n, c, float(eps), int(bool(gelu)),
                               _ptr(out), _stream()), "ptv3_bn_act")
    return out
