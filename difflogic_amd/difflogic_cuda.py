"""Drop-in for the reference's extension module ``difflogic_cuda``
(difflogic/cuda/difflogic.cpp:45-84): the same six functions on torch tensors, implemented by
the gfx950 kernels of libdifflogic_hip.so.

Differences from the reference that callers can observe:
* work is enqueued on torch's current stream for the tensors' device and the call returns
  without a device-wide synchronisation (the reference blocks after every kernel);
* HIP errors raise RuntimeError instead of terminating the process
  (difflogic/cuda/difflogic_kernel.cu:22-28 calls exit());
* ``backward_x`` gives a neuron with a[n] == b[n] the derivative d/da + d/db, as autograd does
  for the python implementation (the reference's kernel counts d/da twice,
  difflogic_kernel.cu:215-218).
"""
import ctypes

import torch

from . import _lib

_FLOAT_CODES = {torch.float16: _lib.DL_F16, torch.float32: _lib.DL_F32, torch.float64: _lib.DL_F64}
_WORD_BITS = {torch.int8: 8, torch.uint8: 8, torch.int16: 16, torch.int32: 32, torch.int64: 64}
_BITS_TO_DTYPE = {8: torch.int8, 16: torch.int16, 32: torch.int32, 64: torch.int64}


def _check_input(t, name):
    # difflogic_kernel.cu:13-17 (CHECK_CUDA, CHECK_CONTIGUOUS)
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _check_index(t, name, numel=None):
    _check_input(t, name)
    if t.dtype != torch.int64 or t.dim() != 1:
        raise RuntimeError(f"expected {name} to be a 1-D int64 tensor, got {t.dtype} with {t.dim()} dims")
    if numel is not None and t.numel() != numel:
        raise RuntimeError(f"{name} has {t.numel()} elements, expected {numel}")


def _float_code(t, name):
    code = _FLOAT_CODES.get(t.dtype)
    if code is None:
        raise RuntimeError(f'"{name}" not implemented for \'{t.dtype}\'')
    return code


_MIXED_CODES = {torch.float16: _lib.DL_F16_W32, torch.float64: _lib.DL_F64_W32}


def _layer_code(x, w, name):
    """dtype code of a layer call: activations ``x`` and gate weights / logits / probabilities ``w`` of one float
    dtype (the reference's functions), or fp32 ``w`` next to half / double ``x`` (a layer with fp32 weights on
    half / double inputs: experiments/main.py:19-23,286)."""
    if w.dtype == x.dtype:
        return _float_code(x, name)
    if w.dtype == torch.float32 and x.dtype in _MIXED_CODES:
        return _MIXED_CODES[x.dtype]
    raise RuntimeError(f"{name}: expected weights of the activations' dtype ({x.dtype}) or float32, got {w.dtype}")


def _same_device(*tensors):
    dev = tensors[0].device
    for t in tensors[1:]:
        if t.device != dev:
            raise RuntimeError(f"all tensors must be on the same device, got {dev} and {t.device}")
    return dev


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(dev):
    """torch's current stream on ``dev`` as the void* the C ABI takes."""
    if _raw_stream is not None and dev.index is not None:
        return _raw_stream(dev.index)                            # no Stream object on the hot path
    return torch.cuda.current_stream(dev).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def _on(dev):
    """Device guard for a launch: nothing to do when ``dev`` is already current."""
    if dev.index is None or torch.cuda.current_device() == dev.index:
        return _NO_GUARD
    return torch.cuda.device(dev)


def _raise(status, what):
    msg = f"{what}: {_lib.status_string(status)}"
    if status in (_lib.DL_ERR_BIT_COUNT, _lib.DL_ERR_NOT_DIVISIBLE):
        raise ValueError(msg)
    raise RuntimeError(msg)


def _p(t):
    """The tensor's device address as the bindings take it (argtypes say void *; a plain int converts without an
    object of its own, which counts on the paths that are bound by the host)."""
    return t.data_ptr()


def forward(x, a, b, w, schedule=None):
    """x [in,B], a/b [out] int64, w [out,16] -> y [out,B]   (difflogic.cpp:46-51).
    ``schedule`` (an EvalSchedule of (a, b); not in the reference) selects the chained kernel:
    same result, one gathered input row per neuron instead of two."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (w, "w")):
        _check_input(t, n)
    if x.dim() != 2 or w.dim() != 2 or w.shape[1] != 16:
        raise RuntimeError(f"expected x [in,B] and w [out,16], got {tuple(x.shape)} {x.dtype}, "
                           f"{tuple(w.shape)} {w.dtype}")
    code = _layer_code(x, w, "logic_layer_cuda_forward")
    out_dim = w.shape[0]
    _check_index(a, "a", out_dim)
    _check_index(b, "b", out_dim)
    dev = _same_device(x, a, b, w)
    in_dim, batch = x.shape
    y = torch.empty((out_dim, batch), dtype=x.dtype, device=dev)
    lib = _lib.load()
    with _on(dev):
        st = _lib.DL_ERR_TOO_LARGE
        if schedule is not None and out_dim > 0 and batch > 0:
            _check_schedule(schedule, in_dim, out_dim, dev)
            st = lib.dl_logic_forward_chained(_p(x), _p(schedule.verts), _p(schedule.neuron), _p(schedule.flip),
                                              schedule.steps, _p(w), _p(y), None, in_dim, out_dim, batch, code,
                                              _stream(dev))
        if st == _lib.DL_ERR_TOO_LARGE:
            st = lib.dl_logic_forward(_p(x), _p(a), _p(b), _p(w), _p(y), in_dim, out_dim, batch, code, _stream(dev))
    if st:
        _raise(st, "logic_layer_cuda_forward")
    return y


def backward_w(x, a, b, grad_y, schedule=None):
    """-> grad_w [out,16]   (difflogic.cpp:52-56).  ``schedule`` selects the chained kernel
    (bit-identical result in fp32 / fp64)."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (grad_y, "grad_y")):
        _check_input(t, n)
    code = _float_code(x, "logic_layer_cuda_backward_w")
    if x.dim() != 2 or grad_y.dim() != 2 or grad_y.shape[1] != x.shape[1] or grad_y.dtype != x.dtype:
        raise RuntimeError(f"expected x [in,B] and grad_y [out,B] of one dtype, got {tuple(x.shape)} {x.dtype}, "
                           f"{tuple(grad_y.shape)} {grad_y.dtype}")
    out_dim = grad_y.shape[0]
    _check_index(a, "a", out_dim)
    _check_index(b, "b", out_dim)
    dev = _same_device(x, a, b, grad_y)
    in_dim, batch = x.shape
    grad_w = torch.empty((out_dim, 16), dtype=x.dtype, device=dev)
    lib = _lib.load()
    with _on(dev):
        st = _lib.DL_ERR_TOO_LARGE
        if schedule is not None and out_dim > 0 and batch > 0:
            _check_schedule(schedule, in_dim, out_dim, dev)
            st = lib.dl_logic_backward_w_chained(_p(x), _p(schedule.verts), _p(schedule.neuron), _p(schedule.flip),
                                                 schedule.steps, _p(grad_y), None, _p(grad_w), in_dim, out_dim, batch,
                                                 code, _stream(dev))
        if st == _lib.DL_ERR_TOO_LARGE:
            st = lib.dl_logic_backward_w(_p(x), _p(a), _p(b), _p(grad_y), _p(grad_w), in_dim, out_dim, batch, code,
                                         _stream(dev))
    if st:
        _raise(st, "logic_layer_cuda_backward_w")
    return grad_w


def backward_x(x, a, b, w, grad_y, given_x_indices_of_y_start, given_x_indices_of_y, scale=1.0):
    """-> grad_x [in,B]   (difflogic.cpp:57-62).  ``scale`` multiplies the result (1.0 = the
    reference's function); LogicLayer passes its grad_factor here."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (w, "w"), (grad_y, "grad_y"),
                 (given_x_indices_of_y_start, "given_x_indices_of_y_start"),
                 (given_x_indices_of_y, "given_x_indices_of_y")):
        _check_input(t, n)
    if (x.dim() != 2 or grad_y.dim() != 2 or grad_y.shape[1] != x.shape[1] or grad_y.dtype != x.dtype
            or w.dim() != 2 or w.shape != (grad_y.shape[0], 16)):
        raise RuntimeError(f"expected x [in,B], w [out,16], grad_y [out,B] of one dtype, got {tuple(x.shape)}, "
                           f"{tuple(w.shape)}, {tuple(grad_y.shape)}")
    code = _layer_code(x, w, "logic_layer_cuda_backward_x")
    in_dim, batch = x.shape
    out_dim = grad_y.shape[0]
    _check_index(a, "a", out_dim)
    _check_index(b, "b", out_dim)
    _check_index(given_x_indices_of_y_start, "given_x_indices_of_y_start", in_dim + 1)
    _check_index(given_x_indices_of_y, "given_x_indices_of_y", 2 * out_dim)
    dev = _same_device(x, a, b, w, grad_y, given_x_indices_of_y_start, given_x_indices_of_y)
    grad_x = torch.empty_like(x)
    with _on(dev):
        st = _lib.load().dl_logic_backward_x(_p(x), _p(a), _p(b), _p(w), _p(grad_y), _p(given_x_indices_of_y_start),
                                             _p(given_x_indices_of_y), _p(grad_x), in_dim, out_dim, batch,
                                             float(scale), code, _stream(dev))
    if st:
        _raise(st, "logic_layer_cuda_backward_x")
    return grad_x


def forward_logits(x, a, b, logits, schedule=None):
    """``forward(x, a, b, softmax(logits, -1))`` with the softmax computed inside the kernel.
    Returns (y [out,B], probs [out,16]); ``probs`` feeds backward_x / backward_logits.  Not part of
    the reference's extension (difflogic/difflogic.py:123-126 runs the softmax in torch).
    ``logits`` have x's dtype, or are float32 next to a half / double x (``probs`` are float32 then,
    and so is what backward_logits / backward_chained return for them).
    ``schedule`` (an EvalSchedule of (a, b)) selects the chained kernel: same result, one
    gathered input row per neuron instead of two."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (logits, "logits")):
        _check_input(t, n)
    if x.dim() != 2 or logits.dim() != 2 or logits.shape[1] != 16 or x.shape[1] == 0:
        raise RuntimeError(f"expected x [in,B>0] and logits [out,16], got {tuple(x.shape)} {x.dtype}, "
                           f"{tuple(logits.shape)} {logits.dtype}")
    code = _layer_code(x, logits, "logic_layer_cuda_forward")
    out_dim = logits.shape[0]
    _check_index(a, "a", out_dim)
    _check_index(b, "b", out_dim)
    dev = _same_device(x, a, b, logits)
    in_dim, batch = x.shape
    y = torch.empty((out_dim, batch), dtype=x.dtype, device=dev)
    probs = torch.empty((out_dim, 16), dtype=logits.dtype, device=dev)
    lib = _lib.load()
    with _on(dev):
        st = _lib.DL_ERR_TOO_LARGE
        if schedule is not None and out_dim > 0:
            _check_schedule(schedule, in_dim, out_dim, dev)
            st = lib.dl_logic_forward_chained(_p(x), _p(schedule.verts), _p(schedule.neuron), _p(schedule.flip),
                                              schedule.steps, _p(logits), _p(y), _p(probs), in_dim, out_dim, batch, code,
                                              _stream(dev))
        if st == _lib.DL_ERR_TOO_LARGE:
            st = lib.dl_logic_forward_logits(_p(x), _p(a), _p(b), _p(logits), _p(y), _p(probs), in_dim, out_dim, batch,
                                             code, _stream(dev))
    if st:
        _raise(st, "logic_layer_cuda_forward_logits")
    return y, probs


def _check_schedule(schedule, in_dim, out_dim, dev):
    if schedule.in_dim != in_dim or schedule.out_dim != out_dim or schedule.verts.device != dev:
        raise RuntimeError(f"schedule is for a {schedule.in_dim}->{schedule.out_dim} layer on {schedule.verts.device}, "
                           f"the call is for {in_dim}->{out_dim} on {dev}")


def backward_logits(x, a, b, grad_y, probs, schedule=None):
    """Gradient with respect to the gate logits: backward_w chained with the softmax backward,
    ``p * (g - (p * g).sum(-1, keepdim=True))`` with ``g = backward_w(x, a, b, grad_y)``.
    ``schedule`` selects the chained kernel (bit-identical result)."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (grad_y, "grad_y"), (probs, "probs")):
        _check_input(t, n)
    if (x.dim() != 2 or grad_y.dim() != 2 or grad_y.shape[1] != x.shape[1] or grad_y.dtype != x.dtype
            or probs.shape != (grad_y.shape[0], 16)):
        raise RuntimeError(f"expected x [in,B], grad_y [out,B], probs [out,16] of one dtype, got {tuple(x.shape)}, "
                           f"{tuple(grad_y.shape)}, {tuple(probs.shape)}")
    code = _layer_code(x, probs, "logic_layer_cuda_backward_w")
    out_dim = grad_y.shape[0]
    _check_index(a, "a", out_dim)
    _check_index(b, "b", out_dim)
    dev = _same_device(x, a, b, grad_y, probs)
    in_dim, batch = x.shape
    grad_logits = torch.empty((out_dim, 16), dtype=probs.dtype, device=dev)
    lib = _lib.load()
    with _on(dev):
        st = _lib.DL_ERR_TOO_LARGE
        if schedule is not None and out_dim > 0 and batch > 0:
            _check_schedule(schedule, in_dim, out_dim, dev)
            st = lib.dl_logic_backward_w_chained(_p(x), _p(schedule.verts), _p(schedule.neuron), _p(schedule.flip),
                                                 schedule.steps, _p(grad_y), _p(probs), _p(grad_logits), in_dim, out_dim,
                                                 batch, code, _stream(dev))
        if st == _lib.DL_ERR_TOO_LARGE:
            st = lib.dl_logic_backward_logits(_p(x), _p(a), _p(b), _p(grad_y), _p(probs), _p(grad_logits), in_dim,
                                              out_dim, batch, code, _stream(dev))
    if st:
        _raise(st, "logic_layer_cuda_backward_logits")
    return grad_logits


def backward_chained(x, w, grad_y, schedule, scale=1.0, softmax_backward=False):
    """backward_w (or backward_logits when ``softmax_backward``; ``w`` are then the probabilities
    that forward_logits returned) and backward_x in one pass along ``schedule``.  Returns
    (grad_w [out,16], grad_x [in,B]), or None where the fused pass does not apply (the caller
    then uses the separate functions).  Not part of the reference's extension."""
    for t, n in ((x, "x"), (w, "w"), (grad_y, "grad_y")):
        _check_input(t, n)
    if (x.dim() != 2 or grad_y.dim() != 2 or grad_y.shape[1] != x.shape[1] or grad_y.dtype != x.dtype
            or w.shape != (grad_y.shape[0], 16)):
        raise RuntimeError(f"expected x [in,B], w [out,16], grad_y [out,B] of one dtype, got {tuple(x.shape)}, "
                           f"{tuple(w.shape)}, {tuple(grad_y.shape)}")
    code = _layer_code(x, w, "logic_layer_cuda_backward")
    dev = _same_device(x, w, grad_y)
    in_dim, batch = x.shape
    out_dim = grad_y.shape[0]
    if in_dim == 0 or out_dim == 0 or batch == 0:
        return None
    _check_schedule(schedule, in_dim, out_dim, dev)
    dst, fix_vertex, fix_start, n_fix, rows = schedule.backward_plan()
    if rows > in_dim * BACKWARD_CHAIN_MAX_OVERFLOW:
        return None
    grad_w = torch.empty((out_dim, 16), dtype=w.dtype, device=dev)
    grad_x = torch.empty_like(x)
    lib = _lib.load()
    ws_bytes = lib.dl_logic_backward_chained_workspace_bytes(rows, out_dim, batch, code)
    if ws_bytes < 0:
        _raise(-ws_bytes, "logic_layer_cuda_backward_chained")
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    with _on(dev):
        st = lib.dl_logic_backward_chained(
            _p(x), _p(schedule.verts), _p(schedule.neuron), _p(schedule.flip), _p(dst), schedule.steps, _p(w),
            _p(grad_y), 1 if softmax_backward else 0, _p(fix_vertex) if n_fix else None,
            _p(fix_start) if n_fix else None, n_fix, rows, _p(grad_w), _p(grad_x),
            _p(workspace) if ws_bytes else None, in_dim, out_dim, batch, float(scale), code, _stream(dev))
    if st == _lib.DL_ERR_TOO_LARGE:
        return None
    if st:
        _raise(st, "logic_layer_cuda_backward_chained")
    return grad_w, grad_x


def forward_logits_lower(x_lower, a_lower, b_lower, logits_lower, logits, schedule):
    """``forward_logits(forward_logits(x_lower, ...)[0], a, b, logits, schedule)`` in one kernel that
    recomputes the rows of the intermediate activation instead of writing and reading them
    (``schedule``: the EvalSchedule of the upper layer's (a, b)).  Returns (y [out,B],
    probs_lower [in,16], probs [out,16]) with the values the two calls give, or None where the
    kernel does not apply (rows longer than 2 KB or not whole 16-byte vectors).  Not part of the
    reference's extension."""
    for t, n in ((x_lower, "x_lower"), (a_lower, "a_lower"), (b_lower, "b_lower"), (logits_lower, "logits_lower"),
                 (logits, "logits")):
        _check_input(t, n)
    code = _float_code(x_lower, "logic_layer_cuda_forward")
    if (x_lower.dim() != 2 or logits_lower.dim() != 2 or logits_lower.shape[1] != 16 or logits.dim() != 2
            or logits.shape[1] != 16 or logits_lower.dtype != x_lower.dtype or logits.dtype != x_lower.dtype
            or x_lower.shape[1] == 0):
        raise RuntimeError(f"expected x_lower [in0,B>0] and logits [*,16] of one dtype, got {tuple(x_lower.shape)} "
                           f"{x_lower.dtype}, {tuple(logits_lower.shape)}, {tuple(logits.shape)}")
    in_dim, out_dim = logits_lower.shape[0], logits.shape[0]
    _check_index(a_lower, "a_lower", in_dim)
    _check_index(b_lower, "b_lower", in_dim)
    dev = _same_device(x_lower, a_lower, b_lower, logits_lower, logits)
    in0, batch = x_lower.shape
    if in0 == 0 or in_dim == 0 or out_dim == 0:
        return None
    _check_schedule(schedule, in_dim, out_dim, dev)
    y = torch.empty((out_dim, batch), dtype=x_lower.dtype, device=dev)
    probs = torch.empty((out_dim, 16), dtype=x_lower.dtype, device=dev)
    # rows of lower neurons that feed nothing are never visited: zero probabilities give them a zero gradient
    probs_lower = torch.zeros((in_dim, 16), dtype=x_lower.dtype, device=dev)
    with _on(dev):
        st = _lib.load().dl_logic_forward_chained_lower(
            _p(x_lower), _p(a_lower), _p(b_lower), _p(logits_lower), _p(probs_lower), _p(schedule.verts),
            _p(schedule.neuron), _p(schedule.flip), schedule.steps, _p(logits), _p(y), _p(probs), in0, in_dim, out_dim,
            batch, code, _stream(dev))
    if st == _lib.DL_ERR_TOO_LARGE:
        return None
    if st:
        _raise(st, "logic_layer_cuda_forward_chained_lower")
    return y, probs_lower, probs


def backward_chained_lower(x, w, grad_y, schedule, x_lower, a_lower, b_lower, w_lower, scale=1.0,
                           softmax_backward=False, softmax_backward_lower=True):
    """backward_chained for a layer whose input ``x`` is the output of a layer that needs no
    input gradient (a model's first layer), with that lower layer's backward_w in the same pass:
    the grad_x rows are consumed where they are finished instead of being written and read
    back.  ``w_lower`` [in,16]: the lower layer's probabilities; with ``softmax_backward_lower``
    the second result is the gradient of its logits, else of its probabilities.  ``x`` may be
    None (fp32 / fp64): its rows are then recomputed from the lower layer (forward_logits_lower
    never stored them).  Returns (grad_w [out,16], grad_w_lower [in,16]), or None where the fused
    pass does not apply.  Not part of the reference's extension."""
    for t, n in ((w, "w"), (grad_y, "grad_y"), (x_lower, "x_lower"), (a_lower, "a_lower"), (b_lower, "b_lower"),
                 (w_lower, "w_lower")):
        _check_input(t, n)
    code = _float_code(grad_y, "logic_layer_cuda_backward")
    dtype = grad_y.dtype
    out_dim, batch = grad_y.shape if grad_y.dim() == 2 else (0, 0)
    in_dim = w_lower.shape[0]
    if x is not None:
        _check_input(x, "x")
        if x.dim() != 2 or tuple(x.shape) != (in_dim, batch) or x.dtype != dtype:
            raise RuntimeError(f"expected x [{in_dim},{batch}] {dtype}, got {tuple(x.shape)} {x.dtype}")
    if grad_y.dim() != 2 or w.shape != (out_dim, 16) or w.dtype != dtype:
        raise RuntimeError(f"expected w [out,16], grad_y [out,B] of one dtype, got {tuple(w.shape)}, {tuple(grad_y.shape)}")
    if x_lower.dim() != 2 or x_lower.shape[1] != batch or x_lower.dtype != dtype:
        raise RuntimeError(f"expected x_lower [in_lower,{batch}] {dtype}, got {tuple(x_lower.shape)} {x_lower.dtype}")
    if w_lower.shape != (in_dim, 16) or w_lower.dtype != dtype:
        raise RuntimeError(f"expected w_lower [{in_dim},16] {dtype}, got {tuple(w_lower.shape)} {w_lower.dtype}")
    _check_index(a_lower, "a_lower", in_dim)
    _check_index(b_lower, "b_lower", in_dim)
    dev = _same_device(w, grad_y, x_lower, a_lower, b_lower, w_lower)
    if in_dim == 0 or out_dim == 0 or batch == 0 or x_lower.shape[0] == 0:
        return None
    if x is None and dtype == torch.float16:
        return None
    _check_schedule(schedule, in_dim, out_dim, dev)
    dst, fix_vertex, fix_start, n_fix, rows = schedule.backward_plan()
    if rows > in_dim * BACKWARD_CHAIN_MAX_OVERFLOW:
        return None
    grad_w = torch.empty((out_dim, 16), dtype=dtype, device=dev)
    grad_w_lower = torch.empty((in_dim, 16), dtype=dtype, device=dev)
    fix_rows = torch.empty((n_fix, batch), dtype=dtype, device=dev) if n_fix else None
    lib = _lib.load()
    ws_bytes = lib.dl_logic_backward_chained_workspace_bytes(rows, out_dim, batch, code)
    if ws_bytes < 0:
        _raise(-ws_bytes, "logic_layer_cuda_backward_chained")
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    with _on(dev):
        st = lib.dl_logic_backward_chained_lower(
            _p(x) if x is not None else None, _p(schedule.verts), _p(schedule.neuron), _p(schedule.flip), _p(dst),
            schedule.steps, _p(w), _p(grad_y), 1 if softmax_backward else 0, _p(fix_vertex) if n_fix else None,
            _p(fix_start) if n_fix else None, n_fix, rows, _p(grad_w), _p(fix_rows) if n_fix else None,
            _p(workspace) if ws_bytes else None, _p(x_lower), _p(a_lower), _p(b_lower), _p(w_lower),
            1 if softmax_backward_lower else 0, _p(grad_w_lower), in_dim, out_dim, batch, float(scale), code, _stream(dev))
    if st == _lib.DL_ERR_TOO_LARGE:
        return None
    if st:
        _raise(st, "logic_layer_cuda_backward_chained_lower")
    return grad_w, grad_w_lower


# backward_chained gives way to the separate kernels when the partial rows it would park in the
# overflow buffer exceed this fraction of the input rows (wirings with many high-degree inputs).
BACKWARD_CHAIN_MAX_OVERFLOW = 0.25


def eval(x, a, b, w):  # noqa: A001  (the reference's name)
    """x [in,W] int words, w [out] uint8 gate ids -> y [out,W]   (difflogic.cpp:63-68)."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (w, "w")):
        _check_input(t, n)
    bits = _WORD_BITS.get(x.dtype)
    if bits is None:
        raise RuntimeError(f'"logic_layer_cuda_eval_kernel" not implemented for \'{x.dtype}\'')
    if x.dim() != 2 or w.dim() != 1 or w.dtype != torch.uint8:
        raise RuntimeError(f"expected x [in,W] and w [out] uint8, got {tuple(x.shape)}, {tuple(w.shape)} {w.dtype}")
    out_dim = w.shape[0]
    _check_index(a, "a", out_dim)
    _check_index(b, "b", out_dim)
    dev = _same_device(x, a, b, w)
    in_dim, words = x.shape
    y = torch.empty((out_dim, words), dtype=x.dtype, device=dev)
    with _on(dev):
        st = _lib.load().dl_logic_eval(_p(x), _p(a), _p(b), _p(w), _p(y), in_dim, out_dim, words, bits, _stream(dev))
    if st:
        _raise(st, "logic_layer_cuda_eval")
    return y


def gate_ids(weights):
    """uint8 [out] argmax gate per neuron of float weights / logits [out, 16]:
    ``weights.argmax(-1).to(torch.uint8)`` (difflogic/difflogic.py:146) in one kernel.  Not part
    of the reference's extension."""
    _check_input(weights, "weights")
    code = _float_code(weights, "gate_ids")
    if weights.dim() != 2 or weights.shape[1] != 16:
        raise RuntimeError(f"expected weights [out,16], got {tuple(weights.shape)}")
    ids = torch.empty(weights.shape[0], dtype=torch.uint8, device=weights.device)
    with _on(weights.device):
        st = _lib.load().dl_gate_ids(_p(weights), _p(ids), weights.shape[0], code, _stream(weights.device))
    if st:
        _raise(st, "gate_ids")
    return ids


def gate_ids_folded(weights, a, b, state=None):
    """gate_ids and one step of fold_gate_constants in one kernel: (ids, state_out) for a layer with wiring
    ``a``, ``b`` whose input rows are constant where ``state`` says so (uint8 [in]: 0 varies, 1 all zeros, 2 all
    ones; None: all vary).  ``ids`` uint8 [out] are the argmax gates with those constants folded in, ``state_out``
    uint8 [out] the constants among the layer's outputs.  Not part of the reference's extension."""
    _check_input(weights, "weights")
    code = _float_code(weights, "gate_ids")
    if weights.dim() != 2 or weights.shape[1] != 16:
        raise RuntimeError(f"expected weights [out,16], got {tuple(weights.shape)}")
    out_dim = weights.shape[0]
    _check_index(a, "a", out_dim)
    _check_index(b, "b", out_dim)
    dev = _same_device(weights, a, b) if state is None else _same_device(weights, a, b, state)
    if state is not None:
        _check_input(state, "state")
        if state.dtype != torch.uint8 or state.dim() != 1:
            raise RuntimeError(f"expected state [in] uint8, got {tuple(state.shape)} {state.dtype}")
    both = torch.empty((2, out_dim), dtype=torch.uint8, device=dev)
    with _on(dev):
        st = _lib.load().dl_gate_ids_folded(_p(weights), code, _p(a), _p(b), _p(state) if state is not None else None,
                                            _p(both[0]), _p(both[1]), out_dim, _stream(dev))
    if st:
        _raise(st, "gate_ids_folded")
    return both[0], both[1]


def fold_gate_constants(layers):
    """``layers`` = [(a, b, w), ...] applied one after the other to rows that vary -> the same list
    with gate ids in which constants are folded: a neuron that reads a constant neuron (gate id 0 or
    15, or constant through its own inputs) gets the one-input gate it amounts to.  Same function,
    bit for bit; the packed kernels then fetch nothing for the ignored inputs.  Not part of the
    reference's extension."""
    out, state = [], None
    lib = _lib.load()
    for a, b, w in layers:
        _check_input(w, "w")
        if w.dim() != 1 or w.dtype != torch.uint8:
            raise RuntimeError(f"expected w [out] uint8, got {tuple(w.shape)} {w.dtype}")
        _check_index(a, "a", w.shape[0])
        _check_index(b, "b", w.shape[0])
        dev = _same_device(a, b, w)
        folded = torch.empty_like(w)
        consts = torch.empty_like(w)
        with _on(dev):
            st = lib.dl_fold_gate_constants(_p(a), _p(b), _p(w), _p(state) if state is not None else None, _p(folded),
                                            _p(consts), w.shape[0], _stream(dev))
        if st:
            _raise(st, "fold_gate_constants")
        out.append((a, b, folded))
        state = consts
    return out


def tensor_packbits_cuda(t, bit_count):
    """bool [F,B] -> (int{bit_count} [F, ceil(B/bit_count)], pad_len)   (difflogic.cpp:69-74)."""
    _check_input(t, "t")
    if bit_count not in _BITS_TO_DTYPE:
        raise ValueError("`bit_count` has to be in { 8, 16, 32, 64 }")
    if t.dtype != torch.bool or t.dim() != 2:
        raise RuntimeError(f"expected t to be a 2-D bool tensor, got {t.dtype} with {t.dim()} dims")
    features, batch = t.shape
    words = -(-batch // bit_count)
    out = torch.empty((features, words), dtype=_BITS_TO_DTYPE[bit_count], device=t.device)
    pad = ctypes.c_int64(0)
    with _on(t.device):
        st = _lib.load().dl_tensor_packbits(_p(t), _p(out), features, batch, bit_count, ctypes.byref(pad),
                                            _stream(t.device))
    if st:
        _raise(st, "tensor_packbits_cuda")
    return out, int(pad.value)


def tensor_packbits_batch_major(x, bit_count):
    """bool [B,F] (sample-major, as the user holds it) -> (int{bit_count} [F, ceil(B/bit_count)],
    pad_len): the transpose and tensor_packbits_cuda of difflogic/packbitstensor.py:15-16 in
    one kernel.  Not part of the reference's extension; PackBitsTensor uses it."""
    _check_input(x, "x")
    if bit_count not in _BITS_TO_DTYPE:
        raise ValueError("`bit_count` has to be in { 8, 16, 32, 64 }")
    if x.dtype != torch.bool or x.dim() != 2:
        raise RuntimeError(f"expected x to be a 2-D bool tensor, got {x.dtype} with {x.dim()} dims")
    batch, features = x.shape
    words = -(-batch // bit_count)
    out = torch.empty((features, words), dtype=_BITS_TO_DTYPE[bit_count], device=x.device)
    pad = ctypes.c_int64(0)
    with _on(x.device):
        st = _lib.load().dl_tensor_packbits_batch_major(_p(x), _p(out), batch, features, bit_count, ctypes.byref(pad),
                                                        _stream(x.device))
    if st:
        _raise(st, "tensor_packbits_batch_major")
    return out, int(pad.value)


def tensor_packbits_batch_major_rows(x, row_bytes):
    """bool [B,F] (sample-major) -> int64 [F, row_bytes / 8]: the packing of
    difflogic/packbitstensor.py:15-16 into rows of ``row_bytes`` bytes (a multiple of 8, at least
    B bits); sample s is bit s % 64 of word s / 64, bits past the batch are zero.  The bytes are
    those of int{8,16,32} words as well.  Not part of the reference's extension; PackBitsTensor
    uses it."""
    _check_input(x, "x")
    if x.dtype != torch.bool or x.dim() != 2:
        raise RuntimeError(f"expected x to be a 2-D bool tensor, got {x.dtype} with {x.dim()} dims")
    batch, features = x.shape
    if row_bytes % 8 or row_bytes * 8 < batch:
        raise RuntimeError(f"row_bytes ({row_bytes}) has to be a multiple of 8 that holds {batch} bits")
    out = torch.empty((features, row_bytes // 8), dtype=torch.int64, device=x.device)
    with _on(x.device):
        st = _lib.load().dl_tensor_packbits_batch_major_rows(_p(x), _p(out), batch, features, row_bytes, _stream(x.device))
    if st:
        _raise(st, "tensor_packbits_batch_major_rows")
    return out


def groupbitsum(b, pad_len, k):
    """int words [out,W] -> int32 [W*bits - pad_len, k]   (difflogic.cpp:75-83)."""
    _check_input(b, "b")
    bits = _WORD_BITS.get(b.dtype)
    if bits is None or b.dim() != 2:
        raise RuntimeError(f'"groupbitsum_kernel" not implemented for \'{b.dtype}\' with {b.dim()} dims')
    if k <= 0 or b.shape[0] % k != 0:
        raise ValueError(f"in_dim ({b.shape[0]}) has to be divisible by k ({k}) but it is not")
    in_dim, words = b.shape
    batch = words * bits - int(pad_len)
    if pad_len < 0 or batch < 0:
        raise RuntimeError(f"pad_len ({pad_len}) has to be in [0, {words * bits}]")
    out = torch.empty((batch, k), dtype=torch.int32, device=b.device)
    with _on(b.device):
        st = _lib.load().dl_groupbitsum(_p(b), _p(out), in_dim, words, bits, int(pad_len), int(k), _stream(b.device))
    if st:
        _raise(st, "groupbitsum")
    return out


MAX_FUSE_DEPTH = 4          # layers dl_logic_eval_fused can fold into one kernel
MAX_FUSE_DEPTH_COUNT = 2    # layers dl_logic_eval_fused_groupbitsum can fold


def _fused_args(x, layers):
    """Validates a group of consecutive layers [(a, b, w), ...] applied to x and builds the host
    arrays of device pointers the C ABI takes."""
    _check_input(x, "x")
    bits = _WORD_BITS.get(x.dtype)
    if bits is None:
        raise RuntimeError(f'"logic_layer_cuda_eval_kernel" not implemented for \'{x.dtype}\'')
    if x.dim() != 2 or not layers:
        raise RuntimeError(f"expected x [in,W] and at least one layer, got {tuple(x.shape)}, {len(layers)} layers")
    dims = [x.shape[0]]
    tensors = [x]
    for a, b, w in layers:
        _check_input(w, "w")
        if w.dim() != 1 or w.dtype != torch.uint8:
            raise RuntimeError(f"expected w [out] uint8, got {tuple(w.shape)} {w.dtype}")
        _check_index(a, "a", w.shape[0])
        _check_index(b, "b", w.shape[0])
        dims.append(w.shape[0])
        tensors += [a, b, w]
    dev = _same_device(*tensors)
    depth = len(layers)
    ptrs = lambda i: (ctypes.c_void_p * depth)(*[l[i].data_ptr() for l in layers])  # noqa: E731
    return dev, bits, depth, ptrs(0), ptrs(1), ptrs(2), (ctypes.c_int64 * (depth + 1))(*dims), dims


def _fused_workspace(depth, out_dim, dev):
    n = _lib.load().dl_logic_eval_fused_workspace_bytes(depth, out_dim)
    return torch.empty(max(1, -(-n // 8)), dtype=torch.int64, device=dev)


def eval_fused(x, layers):
    """``eval`` applied once per layer of ``layers`` = [(a, b, w), ...] (at most MAX_FUSE_DEPTH),
    in one kernel that never writes the intermediate activations.  Not part of the reference's
    extension.  Falls back to one ``eval`` per layer where the fused kernel does not apply."""
    dev, bits, depth, pa, pb, pw, pdims, dims = _fused_args(x, layers)
    if depth > MAX_FUSE_DEPTH:
        raise RuntimeError(f"at most {MAX_FUSE_DEPTH} layers can be fused, got {depth}")
    words = x.shape[1]
    if depth == 1 or 0 in dims or words == 0:
        st = _lib.DL_ERR_TOO_LARGE
    else:
        y = torch.empty((dims[-1], words), dtype=x.dtype, device=dev)
        ws = _fused_workspace(depth, dims[-1], dev)
        with _on(dev):
            st = _lib.load().dl_logic_eval_fused(_p(x), depth, pa, pb, pw, pdims, _p(y), words, bits, _p(ws),
                                                 _stream(dev))
    if st == _lib.DL_ERR_TOO_LARGE:
        for a, b, w in layers:
            x = eval(x, a, b, w)
        return x
    if st:
        _raise(st, "logic_layer_cuda_eval_fused")
    return y


class EvalSchedule:
    """Device-resident evaluation schedule of one layer's wiring (see eval_chained): the order in
    which dl_logic_eval_chained walks the layer's neurons so that consecutive ones share an
    input.  Built on the host from (a, b); depends on nothing else."""

    def __init__(self, a, b, in_dim):
        import numpy as np
        lib = _lib.load()
        a_h = np.ascontiguousarray(a.detach().cpu().numpy(), dtype=np.int64)
        b_h = np.ascontiguousarray(b.detach().cpu().numpy(), dtype=np.int64)
        out_dim = a_h.shape[0]
        chunk = lib.dl_eval_schedule_chunk()
        cap = lib.dl_eval_schedule_capacity(out_dim, chunk)
        verts = np.empty(cap + 1, dtype=np.int32)
        neuron = np.empty(cap, dtype=np.int32)
        flip = np.empty(cap, dtype=np.uint8)
        steps = lib.dl_eval_schedule_build(a_h.ctypes.data, b_h.ctypes.data, int(in_dim), out_dim, chunk,
                                           verts.ctypes.data, neuron.ctypes.data, flip.ctypes.data)
        if steps < 0:
            _raise(-steps, "eval_schedule_build")
        self.in_dim, self.out_dim, self.steps, self.chunk = int(in_dim), out_dim, int(steps), chunk
        self.verts = torch.from_numpy(verts[:steps + 1].copy()).to(a.device)
        self.neuron = torch.from_numpy(neuron[:steps].copy()).to(a.device)
        self.flip = torch.from_numpy(flip[:steps].copy()).to(a.device)
        self._host = (verts[:steps + 1].copy(), neuron[:steps].copy())
        self._backward = None
        self._count_plans = {}

    def count_plan(self, k):
        """(slot, runs, padded_steps, blocks) plan for eval_chained_groupbitsum with ``k`` classes (slot,
        runs on the device), built on first use per k; None where the chained count does not
        apply (too many classes)."""
        if k not in self._count_plans:
            import numpy as np
            lib = _lib.load()
            _, neuron = self._host
            padded = lib.dl_count_chain_padded_steps(self.steps)
            slot = np.empty(max(1, padded), dtype=np.uint8)
            runs = np.empty(max(1, padded // lib.dl_count_chain_block() * k), dtype=np.uint16)
            blocks = ctypes.c_int(0)
            got = lib.dl_count_chain_plan_build(neuron.ctypes.data, self.steps, self.out_dim, int(k), slot.ctypes.data,
                                                runs.ctypes.data, ctypes.byref(blocks))
            if got == -_lib.DL_ERR_TOO_LARGE:
                self._count_plans[k] = None
            elif got < 0:
                _raise(-got, "count_chain_plan_build")
            else:
                dev = self.verts.device
                # uint16 has no torch dtype on every build: the table travels as int16 with the same bits
                self._count_plans[k] = (torch.from_numpy(slot).to(dev), torch.from_numpy(runs.view(np.int16)).to(dev),
                                        int(got), int(blocks.value))
        return self._count_plans[k]

    def backward_plan(self):
        """(dst, fix_vertex, fix_start, n_fix, overflow_rows) for backward_chained, built on first
        use: where each schedule position's grad_x row goes and which inputs are summed from
        several partial rows afterwards."""
        if self._backward is None:
            import ctypes
            import numpy as np
            lib = _lib.load()
            verts, neuron = self._host
            dst = np.empty(self.steps + 1, dtype=np.int32)
            fix_vertex = np.empty(self.in_dim, dtype=np.int32)
            fix_start = np.empty(self.in_dim + 1, dtype=np.int32)
            n_fix = ctypes.c_int64(0)
            rows = lib.dl_backward_schedule_build(verts.ctypes.data, neuron.ctypes.data, self.steps, self.in_dim,
                                                  dst.ctypes.data, fix_vertex.ctypes.data, fix_start.ctypes.data,
                                                  ctypes.byref(n_fix))
            if rows < 0:
                _raise(-rows, "backward_schedule_build")
            n = int(n_fix.value)
            dev = self.verts.device
            self._backward = (torch.from_numpy(dst).to(dev), torch.from_numpy(fix_vertex[:n].copy()).to(dev),
                              torch.from_numpy(fix_start[:n + 1].copy()).to(dev), n, int(rows))
        return self._backward


class _WiringCache:
    """Results derived from wiring tensors (schedules, count orders), kept only while those
    tensors are alive: an entry holds weak references to its tensors and is dropped when one of
    them is collected, so a freed tensor's address can never be mistaken for a new tensor at the
    same address, and nothing is pinned beyond the wiring's own lifetime.  The key also carries
    the tensors' version counters, so in-place edits of the wiring rebuild the entry (writes
    through ``.data`` are invisible to the counter: replace the tensors, or call
    ``invalidate_wiring`` / ``LogicLayer.invalidate_wiring`` after such a write).  Thread-safe."""

    def __init__(self):
        import threading
        self._lock = threading.Lock()
        self._entries = {}

    def get(self, tensors, extra, build):
        import weakref
        key = tuple((t.data_ptr(), t._version, t.shape[0]) for t in tensors) + tuple(extra)
        with self._lock:
            hit = self._entries.get(key)
            if hit is not None and all(r() is t for r, t in zip(hit[0], tensors)):
                return hit[1]
        value = build()

        def drop(_ref, key=key, cache=weakref.ref(self)):
            me = cache()
            if me is not None:
                with me._lock:
                    me._entries.pop(key, None)

        with self._lock:
            # stale versions of the same tensors go: one entry per set of live tensors
            n = len(tensors)
            same = lambda k: (len(k) == len(key) and k[n:] == key[n:]                           # noqa: E731
                              and all(u[0] == v[0] for u, v in zip(k[:n], key[:n])))
            for old in [k for k in self._entries if same(k)]:
                del self._entries[old]
            self._entries[key] = (tuple(weakref.ref(t, drop) for t in tensors), value)
        return value

    def __len__(self):
        return len(self._entries)

    def drop(self, tensors):
        """Forgets every entry built from one of ``tensors`` (matched by storage address)."""
        ptrs = {t.data_ptr() for t in tensors}
        with self._lock:
            for key in [k for k, (refs, _) in self._entries.items() if any(k[i][0] in ptrs for i in range(len(refs)))]:
                del self._entries[key]


_SCHEDULES = _WiringCache()


def schedule_for(a, b, in_dim):
    """The cached EvalSchedule of the wiring (a, b): lives as long as the tensors do, rebuilt when
    they are replaced or modified in place."""
    return _SCHEDULES.get((a, b), (int(in_dim),), lambda: EvalSchedule(a, b, in_dim))


def invalidate_wiring(*tensors):
    """Forgets everything derived from the index tensors ``tensors`` (evaluation schedules, count plans and
    orders), so that the next call rebuilds it from their current contents.  Needed after writing into index
    tensors through ``.data`` (or any other way that leaves their version counter alone): in-place
    operations that autograd sees and replaced tensors are noticed without it."""
    _SCHEDULES.drop(tensors)
    _COUNT_ORDERS.drop(tensors)


def live_inputs(layers, live_out=None):
    """For consecutive layers [(a, b, w), ...] (``w`` uint8 gate ids) whose last one's output rows
    are needed where ``live_out`` [out] is non-zero (None: all of them): a list with, per layer,
    the uint8 vector of its INPUT rows that some needed neuron looks at (an input its gate ignores
    does not count).  ``result[i]`` is what ``eval_chained(..., out_live=)`` takes for the group that
    produces the input of ``layers[i]``.  Not part of the reference's extension."""
    lib = _lib.load()
    res = [None] * len(layers)
    # one cleared buffer for all layers' vectors (each starts on a 16-byte boundary): one fill instead of one per layer
    starts, total = [0] * len(layers), 0
    for i in range(1, len(layers)):
        starts[i], total = total, total + -(-int(layers[i - 1][2].shape[0]) // 16) * 16
    pool = torch.zeros(max(1, total), dtype=torch.uint8, device=layers[0][2].device) if layers else None
    for i in range(len(layers) - 1, -1, -1):
        a, b, w = layers[i]
        _check_input(w, "w")
        _check_index(a, "a", w.shape[0])
        _check_index(b, "b", w.shape[0])
        dev = _same_device(a, b, w, pool)
        in_dim = int(layers[i - 1][2].shape[0]) if i > 0 else None
        if in_dim is None:
            break                                     # the first layer's input rows are the caller's data
        live_in = pool[starts[i]:starts[i] + in_dim]
        with _on(dev):
            st = lib.dl_mark_live_inputs(_p(a), _p(b), _p(w), _p(live_out) if live_out is not None else None, _p(live_in),
                                         w.shape[0], _stream(dev))
        if st:
            _raise(st, "mark_live_inputs")
        res[i] = live_out = live_in
    return res


def eval_chained(x, layers, schedule=None, out_live=None):
    """Same result as ``eval_fused(x, layers)``; the group's top layer is walked along
    ``schedule`` (default: the cached schedule of its wiring), which halves the rows gathered per
    neuron.  ``out_live`` (uint8 [out], see live_inputs): output rows marked 0 will not be read and
    may be left unwritten.  Not part of the reference's extension.  Falls back to eval_fused where
    it does not apply."""
    dev, bits, depth, pa, pb, pw, pdims, dims = _fused_args(x, layers)
    if depth > MAX_FUSE_DEPTH:
        raise RuntimeError(f"at most {MAX_FUSE_DEPTH} layers can be fused, got {depth}")
    words = x.shape[1]
    if 0 in dims or words == 0:
        return eval_fused(x, layers)
    if schedule is None:
        schedule = schedule_for(layers[-1][0], layers[-1][1], dims[-2])
    if schedule.in_dim != dims[-2] or schedule.out_dim != dims[-1]:
        raise RuntimeError(f"schedule is for a {schedule.in_dim}->{schedule.out_dim} layer, the group ends in "
                           f"{dims[-2]}->{dims[-1]}")
    if out_live is not None and (out_live.dtype != torch.uint8 or out_live.shape != (dims[-1],) or out_live.device != dev
                                 or not out_live.is_contiguous()):
        raise RuntimeError(f"expected out_live to be a contiguous uint8 [{dims[-1]}] tensor on {dev}")
    y = torch.empty((dims[-1], words), dtype=x.dtype, device=dev)
    nbytes = _lib.load().dl_logic_eval_chained_workspace_bytes(depth, dims[-2], schedule.steps)
    ws = torch.empty(max(1, -(-nbytes // 8)), dtype=torch.int64, device=dev)      # torch aligns allocations to 512 bytes
    with _on(dev):
        st = _lib.load().dl_logic_eval_chained(_p(x), depth, pa, pb, pw, pdims, _p(schedule.verts), _p(schedule.neuron),
                                               _p(schedule.flip), schedule.steps,
                                               _p(out_live) if out_live is not None else None, _p(y), words, bits,
                                               _p(ws) if ws is not None else None, _stream(dev))
    if st == _lib.DL_ERR_TOO_LARGE:
        return eval_fused(x, layers)
    if st:
        _raise(st, "logic_layer_cuda_eval_chained")
    return y


_COUNT_ORDERS = _WiringCache()


def count_order_for(layers, in_dim, k):
    """Cached neuron order for eval_fused_groupbitsum over ``layers`` (the net's last one or two
    layers, [(a, b, w), ...]): neurons of a class that read the same input rows are walked by
    the same workgroup.  Built on the host from the wiring alone; lives as long as the index
    tensors do and is rebuilt when they are replaced or modified in place."""
    idx = [t for a, b, _ in layers for t in (a, b)]

    def build():
        import numpy as np
        lib = _lib.load()
        host = [np.ascontiguousarray(t.detach().cpu().numpy(), dtype=np.int64) for t in idx]
        out_dim = host[-1].shape[0]
        order = np.empty(out_dim, dtype=np.int32)
        if len(layers) == 2:
            low_a, low_b, top_a, top_b = (h.ctypes.data for h in host)
            mid = host[0].shape[0]
        else:
            (top_a, top_b), low_a, low_b, mid = (h.ctypes.data for h in host), None, None, 0
        st = lib.dl_count_order_build(top_a, top_b, low_a, low_b, int(in_dim), mid, out_dim, int(k),
                                      lib.dl_count_group(), order.ctypes.data)
        if st:
            _raise(st, "count_order_build")
        return torch.from_numpy(order).to(idx[0].device)

    return _COUNT_ORDERS.get(tuple(idx), (int(in_dim), int(k)), build)


def eval_chained_groupbitsum(x, layers, pad_len, k, schedule=None):
    """Same result as ``eval_fused_groupbitsum(x, layers, pad_len, k)`` for the net's last one or
    two layers; the top layer is walked along ``schedule`` (default: the cached schedule of its
    wiring), which halves the rows gathered per neuron.  Returns None where it does not apply
    (the caller then uses eval_fused_groupbitsum).  Not part of the reference's extension."""
    dev, bits, depth, pa, pb, pw, pdims, dims = _fused_args(x, layers)
    if depth > MAX_FUSE_DEPTH_COUNT:
        raise RuntimeError(f"at most {MAX_FUSE_DEPTH_COUNT} layers can be fused with the count, got {depth}")
    out_dim, words = dims[-1], x.shape[1]
    if k <= 0 or out_dim % k != 0:
        raise ValueError(f"in_dim ({out_dim}) has to be divisible by k ({k}) but it is not")
    batch = words * bits - int(pad_len)
    if pad_len < 0 or batch < 0:
        raise RuntimeError(f"pad_len ({pad_len}) has to be in [0, {words * bits}]")
    if 0 in dims or batch == 0 or (words * bits) % 64:
        return None
    if schedule is None:
        schedule = schedule_for(layers[-1][0], layers[-1][1], dims[-2])
    if schedule.in_dim != dims[-2] or schedule.out_dim != dims[-1] or schedule.verts.device != dev:
        raise RuntimeError(f"schedule is for a {schedule.in_dim}->{schedule.out_dim} layer on {schedule.verts.device}, "
                           f"the group ends in {dims[-2]}->{dims[-1]} on {dev}")
    plan = schedule.count_plan(int(k))
    if plan is None:
        return None
    slot, runs, padded, blocks = plan
    lib = _lib.load()
    out = torch.empty((batch, k), dtype=torch.int32, device=dev)
    nbytes = lib.dl_logic_eval_chained_groupbitsum_workspace_bytes(padded, blocks, words, bits, int(k))
    ws = torch.empty(max(2, -(-nbytes // 8)), dtype=torch.int64, device=dev)
    with _on(dev):
        st = lib.dl_logic_eval_chained_groupbitsum(_p(x), depth, pa, pb, pw, pdims, _p(schedule.verts),
                                                   _p(schedule.neuron), _p(schedule.flip), schedule.steps, _p(slot),
                                                   _p(runs), padded, blocks, _p(out), words, bits, int(pad_len), int(k),
                                                   _p(ws), _stream(dev))
    if st == _lib.DL_ERR_TOO_LARGE:
        return None
    if st:
        _raise(st, "logic_layer_cuda_eval_chained_groupbitsum")
    return out


def eval_fused_groupbitsum(x, layers, pad_len, k, order=None):
    """groupbitsum(eval(... eval(x, layer 0) ..., last layer), pad_len, k) for the net's last
    one or two layers without materialising their output.  Not part of the reference's
    extension.  Falls back to the separate kernels where the fused one does not apply.
    ``order`` (see count_order_for) changes the cache traffic, not the result."""
    dev, bits, depth, pa, pb, pw, pdims, dims = _fused_args(x, layers)
    if depth > MAX_FUSE_DEPTH_COUNT:
        raise RuntimeError(f"at most {MAX_FUSE_DEPTH_COUNT} layers can be fused with the count, got {depth}")
    out_dim, words = dims[-1], x.shape[1]
    if k <= 0 or out_dim % k != 0:
        raise ValueError(f"in_dim ({out_dim}) has to be divisible by k ({k}) but it is not")
    batch = words * bits - int(pad_len)
    if pad_len < 0 or batch < 0:
        raise RuntimeError(f"pad_len ({pad_len}) has to be in [0, {words * bits}]")
    if order is not None and (order.dtype != torch.int32 or order.shape != (out_dim,) or order.device != dev
                              or not order.is_contiguous()):
        raise RuntimeError(f"expected order to be a contiguous int32 [{out_dim}] tensor on {dev}")
    if 0 in dims:
        st = _lib.DL_ERR_TOO_LARGE
    else:
        out = torch.empty((batch, k), dtype=torch.int32, device=dev)
        nbytes = _lib.load().dl_logic_eval_fused_groupbitsum_workspace_bytes(depth, out_dim, words, bits, int(k))
        ws = torch.empty(max(2, -(-nbytes // 8)), dtype=torch.int64, device=dev)
        with _on(dev):
            st = _lib.load().dl_logic_eval_fused_groupbitsum(_p(x), depth, pa, pb, pw, pdims, _p(out), words, bits,
                                                             int(pad_len), int(k),
                                                             _p(order) if order is not None else None, _p(ws),
                                                             _stream(dev))
    if st == _lib.DL_ERR_TOO_LARGE:
        return groupbitsum(eval_fused(x, layers), pad_len, k)
    if st:
        _raise(st, "logic_layer_cuda_eval_fused_groupbitsum")
    return out


MAX_NET_DEPTH = 16          # layers dl_logic_net_lds_groupbitsum can carry through LDS


def net_lds_max_width():
    """Widest layer (and input) the LDS-resident whole-net kernel takes."""
    return int(_lib.load().dl_logic_net_lds_max_width())


def _net_lds_thinned(x, bool_input, batch, layers, dims, k, words, bits, pad_len, out, dev, folded=False):
    lib = _lib.load()
    depth = len(layers)
    ptrs = lambda i: (ctypes.c_void_p * depth)(*[l[i].data_ptr() for l in layers])  # noqa: E731
    pdims = (ctypes.c_int64 * (depth + 1))(*dims)
    ws = torch.empty(max(1, lib.dl_logic_net_lds_workspace_bytes(depth, pdims) // 4), dtype=torch.int32, device=dev)
    with _on(dev):
        return lib.dl_logic_net_lds_groupbitsum_thinned(_p(x), 1 if bool_input else 0, batch, depth, ptrs(0), ptrs(1), ptrs(2),
                                                        1 if folded else 0, pdims, _p(out), words, bits, int(pad_len), int(k),
                                                        _p(ws), _stream(dev))


def eval_net_lds(x, layers, pad_len, k, scheduled=True, thin=False, folded=False):
    """groupbitsum(eval(... eval(x, layer 0) ..., last layer), pad_len, k) for a whole narrow net
    (every layer and the input at most net_lds_max_width() wide, at most MAX_NET_DEPTH layers) in
    one kernel that keeps the activations in LDS.  ``scheduled``: hidden layers are walked along
    their (cached) evaluation schedules where that fits, which nearly halves their LDS reads; the
    result is the same.  ``thin``: instead, the net is thinned for this call (constants folded, neurons that
    no gate looks at neither evaluated nor stored; pays where many gates ignore an input; ``folded``: the gate ids
    have the constants folded in already, so the kernels that would do it are left out).  Returns None where
    the kernel does not apply (the caller then uses the streaming kernels).  Not part of the reference's
    extension."""
    dev, bits, depth, pa, pb, pw, pdims, dims = _fused_args(x, layers)
    out_dim, words = dims[-1], x.shape[1]
    if k <= 0 or out_dim % k != 0:
        raise ValueError(f"in_dim ({out_dim}) has to be divisible by k ({k}) but it is not")
    batch = words * bits - int(pad_len)
    if pad_len < 0 or batch < 0:
        raise RuntimeError(f"pad_len ({pad_len}) has to be in [0, {words * bits}]")
    if depth > MAX_NET_DEPTH or 0 in dims or max(dims) > net_lds_max_width():
        return None
    lib = _lib.load()
    out = torch.empty((batch, k), dtype=torch.int32, device=dev)
    if thin:
        st = _net_lds_thinned(x, False, batch, layers, dims, k, words, bits, pad_len, out, dev, folded)
        if st == _lib.DL_ERR_TOO_LARGE:
            return None
        if st:
            _raise(st, "logic_net_lds_groupbitsum_thinned")
        return out
    ws = torch.empty(max(1, lib.dl_logic_net_lds_workspace_bytes(depth, pdims) // 4), dtype=torch.int32, device=dev)
    scheds = [schedule_for(a, b, dims[i]) for i, (a, b, _) in enumerate(layers[:-1])] if scheduled else []
    with _on(dev):
        if scheds:
            n = len(scheds)
            pv = (ctypes.c_void_p * n)(*[sc.verts.data_ptr() for sc in scheds])
            pn = (ctypes.c_void_p * n)(*[sc.neuron.data_ptr() for sc in scheds])
            pf = (ctypes.c_void_p * n)(*[sc.flip.data_ptr() for sc in scheds])
            ps = (ctypes.c_int64 * n)(*[sc.steps for sc in scheds])
            st = lib.dl_logic_net_lds_groupbitsum_scheduled(_p(x), depth, pa, pb, pw, pdims, pv, pn, pf, ps, _p(out), words,
                                                            bits, int(pad_len), int(k), _p(ws), _stream(dev))
        else:
            st = lib.dl_logic_net_lds_groupbitsum(_p(x), depth, pa, pb, pw, pdims, _p(out), words, bits, int(pad_len),
                                                  int(k), _p(ws), _stream(dev))
    if st == _lib.DL_ERR_TOO_LARGE:
        return None
    if st:
        _raise(st, "logic_net_lds_groupbitsum")
    return out


def eval_net_lds_bool(x, layers, k, scheduled=True, thin=False, folded=False):
    """eval_net_lds on the bool input itself: ``x`` [B, in] bool (sample-major, as PackBitsTensor
    receives it) -> int32 [B, k], the result of packing x with 64-bit words, evaluating every layer
    and groupbitsum, in one kernel that packs the input on its way into LDS (no pack kernel, no
    packed input in memory).  Returns None where the kernel does not apply (in not a multiple of
    16, input and widest hidden layer together beyond net_lds_max_width(), unaligned x).  Not part
    of the reference's extension."""
    _check_input(x, "x")
    if x.dtype != torch.bool or x.dim() != 2 or not layers:
        raise RuntimeError(f"expected x [B,in] bool and at least one layer, got {x.dtype} {tuple(x.shape)}")
    batch, in_dim = x.shape
    dims, tensors = [in_dim], [x]
    for a, b, w in layers:
        _check_input(w, "w")
        if w.dim() != 1 or w.dtype != torch.uint8:
            raise RuntimeError(f"expected w [out] uint8, got {tuple(w.shape)} {w.dtype}")
        _check_index(a, "a", w.shape[0])
        _check_index(b, "b", w.shape[0])
        dims.append(w.shape[0])
        tensors += [a, b, w]
    dev = _same_device(*tensors)
    depth, out_dim = len(layers), dims[-1]
    if k <= 0 or out_dim % k != 0:
        raise ValueError(f"in_dim ({out_dim}) has to be divisible by k ({k}) but it is not")
    if depth > MAX_NET_DEPTH or 0 in dims or max(dims) > net_lds_max_width() or in_dim % 16 != 0:
        return None
    ptrs = lambda i: (ctypes.c_void_p * depth)(*[l[i].data_ptr() for l in layers])  # noqa: E731
    pdims = (ctypes.c_int64 * (depth + 1))(*dims)
    lib = _lib.load()
    out = torch.empty((batch, k), dtype=torch.int32, device=dev)
    if batch == 0:
        return out
    if thin:
        st = _net_lds_thinned(x, True, batch, layers, dims, k, 0, 64, 0, out, dev, folded)
        if st == _lib.DL_ERR_TOO_LARGE:
            return None
        if st:
            _raise(st, "logic_net_lds_groupbitsum_thinned")
        return out
    ws = torch.empty(max(1, lib.dl_logic_net_lds_workspace_bytes(depth, pdims) // 4), dtype=torch.int32, device=dev)
    scheds = [schedule_for(a, b, dims[i]) for i, (a, b, _) in enumerate(layers[:-1])] if scheduled else []
    n = len(scheds)
    pv = (ctypes.c_void_p * n)(*[sc.verts.data_ptr() for sc in scheds]) if n else None
    pn = (ctypes.c_void_p * n)(*[sc.neuron.data_ptr() for sc in scheds]) if n else None
    pf = (ctypes.c_void_p * n)(*[sc.flip.data_ptr() for sc in scheds]) if n else None
    ps = (ctypes.c_int64 * n)(*[sc.steps for sc in scheds]) if n else None
    with _on(dev):
        st = lib.dl_logic_net_lds_groupbitsum_bool(_p(x), batch, depth, ptrs(0), ptrs(1), ptrs(2), pdims, pv, pn, pf, ps,
                                                   _p(out), int(k), _p(ws), _stream(dev))
    if st == _lib.DL_ERR_TOO_LARGE:
        return None
    if st:
        _raise(st, "logic_net_lds_groupbitsum_bool")
    return out


def eval_fused_groupbitsum_noalloc(x, layers, pad_len, k, out, order=None):
    """eval_fused_groupbitsum into the caller's ``out`` (int32 [batch, k], contiguous) through the
    entry point that allocates no device memory: its workspace is a static device array of
    ``_lib.DL_STATIC_SCRATCH_BYTES`` inside the library (one copy per GPU, shared by all calls on
    that GPU, so calls must not overlap in time on one GPU).  Raises RuntimeError when the call
    needs more scratch than that or when rows are not whole 64-bit words; there is no fallback.
    Not part of the reference's extension."""
    dev, bits, depth, pa, pb, pw, pdims, dims = _fused_args(x, layers)
    if depth > MAX_FUSE_DEPTH_COUNT:
        raise RuntimeError(f"at most {MAX_FUSE_DEPTH_COUNT} layers can be fused with the count, got {depth}")
    out_dim, words = dims[-1], x.shape[1]
    if k <= 0 or out_dim % k != 0:
        raise ValueError(f"in_dim ({out_dim}) has to be divisible by k ({k}) but it is not")
    batch = words * bits - int(pad_len)
    if pad_len < 0 or batch < 0:
        raise RuntimeError(f"pad_len ({pad_len}) has to be in [0, {words * bits}]")
    _check_input(out, "out")
    if out.dtype != torch.int32 or tuple(out.shape) != (batch, k) or out.device != dev:
        raise RuntimeError(f"expected out to be int32 [{batch}, {k}] on {dev}, got {out.dtype} {tuple(out.shape)}")
    if order is not None and (order.dtype != torch.int32 or order.shape != (out_dim,) or order.device != dev
                              or not order.is_contiguous()):
        raise RuntimeError(f"expected order to be a contiguous int32 [{out_dim}] tensor on {dev}")
    with _on(dev):
        st = _lib.load().dl_logic_eval_fused_groupbitsum_noalloc(_p(x), depth, pa, pb, pw, pdims, _p(out), words, bits,
                                                                 int(pad_len), int(k),
                                                                 _p(order) if order is not None else None,
                                                                 _stream(dev))
    if st:
        _raise(st, "logic_layer_cuda_eval_fused_groupbitsum_noalloc")
    return out


def forward_group_sum(x, a, b, logits, k, tau):
    """``group_sum_forward(forward_logits(x, a, b, logits)[0], k, tau)`` without the layer's output
    ever being written: returns (sums [B, k], probs [out, 16]).  Not part of the reference's
    extension."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (logits, "logits")):
        _check_input(t, n)
    code = _float_code(x, "logic_layer_cuda_forward")
    if x.dim() != 2 or logits.dim() != 2 or logits.shape[1] != 16 or logits.dtype != x.dtype or 0 in x.shape:
        raise RuntimeError(f"expected x [in>0,B>0] and logits [out,16] of one dtype, got {tuple(x.shape)} {x.dtype}, "
                           f"{tuple(logits.shape)} {logits.dtype}")
    out_dim = logits.shape[0]
    if k <= 0 or out_dim == 0 or out_dim % k != 0:
        raise ValueError(f"in_dim ({out_dim}) has to be divisible by k ({k}) but it is not")
    _check_index(a, "a", out_dim)
    _check_index(b, "b", out_dim)
    dev = _same_device(x, a, b, logits)
    in_dim, batch = x.shape
    lib = _lib.load()
    y = torch.empty((batch, k), dtype=x.dtype, device=dev)
    probs = torch.empty((out_dim, 16), dtype=x.dtype, device=dev)
    ws = torch.empty(max(1, lib.dl_group_sum_workspace_bytes(out_dim, batch, k, code)), dtype=torch.uint8, device=dev)
    with _on(dev):
        st = lib.dl_logic_forward_group_sum(_p(x), _p(a), _p(b), _p(logits), _p(probs), _p(y), _p(ws), in_dim, out_dim,
                                            batch, int(k), float(tau), code, _stream(dev))
    if st:
        _raise(st, "logic_layer_cuda_forward_group_sum")
    return y, probs


def backward_group_sum(x, a, b, probs, grad_cls, start, idx, schedule, scale, want_x, want_w):
    """Gradients of forward_group_sum: ``grad_cls`` [k, B] is the gradient of the sums, transposed
    and already divided by tau; every neuron of class c sees row c as its grad_y (the broadcast
    matrix is never built).  Returns (grad_logits or None, grad_x or None)."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (probs, "probs"), (grad_cls, "grad_cls")):
        _check_input(t, n)
    code = _float_code(x, "logic_layer_cuda_backward")
    in_dim, batch = x.shape
    out_dim = probs.shape[0]
    k = grad_cls.shape[0]
    if grad_cls.shape != (k, batch) or grad_cls.dtype != x.dtype or probs.shape != (out_dim, 16) or out_dim % k:
        raise RuntimeError(f"expected grad_cls [k,B] and probs [out,16] of x's dtype, got {tuple(grad_cls.shape)}, "
                           f"{tuple(probs.shape)}")
    dev = _same_device(x, a, b, probs, grad_cls)
    lib = _lib.load()
    if want_x and want_w and schedule is not None:
        _check_schedule(schedule, in_dim, out_dim, dev)
        dst, fix_vertex, fix_start, n_fix, rows = schedule.backward_plan()
        if rows <= in_dim * BACKWARD_CHAIN_MAX_OVERFLOW:
            grad_w = torch.empty((out_dim, 16), dtype=x.dtype, device=dev)
            grad_x = torch.empty_like(x)
            ws_bytes = lib.dl_logic_backward_chained_workspace_bytes(rows, out_dim, batch, code)
            if ws_bytes < 0:
                _raise(-ws_bytes, "logic_layer_cuda_backward_chained")
            workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
            with _on(dev):
                st = lib.dl_logic_backward_chained_grouped(
                    _p(x), _p(schedule.verts), _p(schedule.neuron), _p(schedule.flip), _p(dst), schedule.steps, _p(probs),
                    _p(grad_cls), 1, _p(fix_vertex) if n_fix else None, _p(fix_start) if n_fix else None, n_fix, rows,
                    _p(grad_w), _p(grad_x), _p(workspace) if ws_bytes else None, in_dim, out_dim, batch, k, float(scale),
                    code, _stream(dev))
            if st == _lib.DL_OK:
                return grad_w, grad_x
            if st != _lib.DL_ERR_TOO_LARGE:
                _raise(st, "logic_layer_cuda_backward_chained_grouped")
    grad_w = grad_x = None
    with _on(dev):
        if want_x:
            _check_index(start, "given_x_indices_of_y_start", in_dim + 1)
            _check_index(idx, "given_x_indices_of_y", 2 * out_dim)
            grad_x = torch.empty_like(x)
            st = lib.dl_logic_backward_x_grouped(_p(x), _p(a), _p(b), _p(probs), _p(grad_cls), _p(start), _p(idx),
                                                 _p(grad_x), in_dim, out_dim, batch, k, float(scale), code, _stream(dev))
            if st:
                _raise(st, "logic_layer_cuda_backward_x_grouped")
        if want_w:
            grad_w = torch.empty((out_dim, 16), dtype=x.dtype, device=dev)
            st = lib.dl_logic_backward_logits_grouped(_p(x), _p(a), _p(b), _p(grad_cls), _p(probs), _p(grad_w), in_dim,
                                                      out_dim, batch, k, code, _stream(dev))
            if st:
                _raise(st, "logic_layer_cuda_backward_logits_grouped")
    return grad_w, grad_x


def group_sum_forward(x, k, tau):
    """Feature-major GroupSum: x [out,B] -> [B,k] = per-class sums over neurons / tau
    (difflogic/difflogic.py:195-196 on the layout the layer kernels produce)."""
    _check_input(x, "x")
    code = _float_code(x, "group_sum_forward")
    if x.dim() != 2:
        raise RuntimeError(f"expected x [out,B], got {tuple(x.shape)}")
    out_dim, batch = x.shape
    if k <= 0 or out_dim % k != 0:
        raise ValueError(f"in_dim ({out_dim}) has to be divisible by k ({k}) but it is not")
    lib = _lib.load()
    y = torch.empty((batch, k), dtype=x.dtype, device=x.device)
    ws = torch.empty(max(1, lib.dl_group_sum_workspace_bytes(out_dim, batch, k, code)), dtype=torch.uint8,
                     device=x.device)
    with _on(x.device):
        st = lib.dl_group_sum_forward(_p(x), _p(y), _p(ws), out_dim, batch, int(k), float(tau), code, _stream(x.device))
    if st:
        _raise(st, "group_sum_forward")
    return y


def group_sum_backward(grad_y, out_dim, tau):
    """grad_y [B,k] -> grad_x [out,B]: every neuron of class c receives grad_y[:, c] / tau."""
    _check_input(grad_y, "grad_y")
    code = _float_code(grad_y, "group_sum_backward")
    batch, k = grad_y.shape
    if k <= 0 or out_dim % k != 0:
        raise ValueError(f"in_dim ({out_dim}) has to be divisible by k ({k}) but it is not")
    grad_x = torch.empty((out_dim, batch), dtype=grad_y.dtype, device=grad_y.device)
    with _on(grad_y.device):
        st = _lib.load().dl_group_sum_backward(_p(grad_y), _p(grad_x), out_dim, batch, int(k), float(tau), code,
                                               _stream(grad_y.device))
    if st:
        _raise(st, "group_sum_backward")
    return grad_x
