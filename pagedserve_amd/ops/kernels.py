"""Python faces of the HIP kernels: shape checks on the host, then one C call.

Every function takes torch tensors that live on the GPU, checks what the kernel and
its grid assume (devices, dtypes, contiguity, extents) and launches on torch's
current stream.  There is no other implementation behind these functions.
"""

import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p

import torch

from .library import load_library

F32 = 0
BF16 = 1
MAX_STREAMS = 8   # copies of the residual stream that ps_hyper_step takes (csrc/streams.hip)

EPILOGUES = {"none": 0, "gelu_tanh": 1, "gelu_erf": 2, "residual": 3, "relu2": 4}

_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}

_SIGNATURES = {
    "ps_embed": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                 c_int, c_int, c_int, c_float, c_void_p, c_float, c_int, c_void_p],
    "ps_norm": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_int,
                c_int, c_void_p],
    "ps_gemm_nt": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                   c_int, c_int, c_int, c_void_p],
    "ps_kv_write": [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                    c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ps_attention_rowwise": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                             c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                             c_int, c_float, c_int, c_void_p, c_void_p, c_int64, c_float, c_int,
                             c_void_p],
    "ps_hyper_step": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p,
                      c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "ps_streams_expand": [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "ps_streams_collapse": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "ps_attention_prepare": [c_void_p, c_int64, c_int, c_int, c_int, c_void_p, c_int64, c_void_p,
                             c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_int, c_void_p,
                             c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                             c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                             c_void_p],
    "ps_differential_combine": [c_void_p, c_int64, c_void_p, c_float, c_float, c_void_p, c_int64,
                                c_void_p, c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ps_differential_merge": [c_void_p, c_int64, c_void_p, c_int, c_void_p, c_float, c_float, c_void_p,
                              c_int64, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ps_head_gate": [c_void_p, c_int64, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p],
    "ps_gla_decay": [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_float, c_void_p, c_int,
                     c_int, c_int, c_void_p],
    "ps_gla_scan": [c_void_p, c_int64, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                    c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_int,
                    c_void_p],
    "ps_scan_pieces": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p],
    "ps_decay_join": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                      c_void_p],
    "ps_row_norm_gate": [c_void_p, c_void_p, c_float, c_void_p, c_int64, c_void_p, c_int64, c_int,
                         c_int, c_int, c_void_p],
    "ps_conv_silu": [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                     c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ps_attention_prepare_heads": [c_void_p, c_int64, c_int, c_int, c_int, c_void_p, c_int64, c_void_p,
                                   c_void_p, c_void_p, c_int, c_int, c_float, c_int, c_float, c_void_p,
                                   c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                   c_int, c_int, c_int, c_void_p],
    "ps_latent_prepare": [c_void_p, c_int64, c_void_p, c_int64, c_int, c_int, c_void_p, c_int64, c_void_p, c_void_p,
                          c_float, c_void_p, c_int, c_int, c_float, c_void_p, c_void_p, c_void_p, c_int,
                          c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ps_block_linear": [c_void_p, c_int, c_int64, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int,
                        c_int64, c_int, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p],
    "ps_lru_scan": [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_float, c_void_p,
                    c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ps_step_size": [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                     c_void_p],
    "ps_selective_scan": [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p, c_int64,
                          c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                          c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                          c_int, c_int, c_int, c_void_p],
    "ps_stream_step": [c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_float, c_void_p,
                       c_void_p, c_int, c_int, c_int, c_void_p],
    "ps_silu_columns": [c_void_p, c_int64, c_int, c_int, c_int, c_void_p],
    "ps_silu_gate": [c_void_p, c_int64, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p],
    "ps_pair_norm_mix": [c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_float, c_void_p, c_int,
                         c_int, c_void_p],
    "ps_moe_route": [c_void_p, c_int64, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float,
                     c_int, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p],
    "ps_moe_experts_grouped": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                               c_int, c_void_p],
    "ps_moe_experts": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                       c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p],
    "ps_gla_output": [c_void_p, c_void_p, c_float, c_void_p, c_int64, c_void_p, c_int64, c_int,
                      c_int, c_int, c_int, c_void_p],
    "ps_softcap": [c_void_p, c_int64, c_int, c_int, c_float, c_void_p],
    "ps_attention_decode": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                            c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                            c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_void_p, c_void_p,
                            c_int64, c_float, c_int, c_void_p],
    "ps_attention_decode_shared": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                                   c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                   c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_int64,
                                   c_float, c_void_p],
    "ps_attention_decode_partial": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                                    c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                    c_int, c_int, c_float, c_int, c_int, c_int, c_void_p, c_float, c_int,
                                    c_void_p],
    "ps_attention_merge_linear": [c_void_p, c_int64, c_void_p, c_int, c_int, c_int, c_int, c_void_p,
                                  c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p],
    "ps_attention_tiled_f32": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                               c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                               c_int, c_int, c_int, c_float, c_int, c_void_p, c_void_p, c_int64, c_float,
                               c_void_p],
    "ps_attention_prefill": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                             c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                             c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_void_p, c_void_p, c_int64,
                             c_float, c_int, c_void_p],
    "ps_attention_mixed": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int,
                           c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                           c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_void_p,
                           c_int64, c_float, c_int, c_void_p],
    "ps_sample": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
}

_BOUND = {}


def _fn(name):
    fn = _BOUND.get(name)
    if fn is None:
        fn = getattr(load_library(), name)
        fn.argtypes = _SIGNATURES[name]
        fn.restype = c_int
        _BOUND[name] = fn
    return fn


class KernelError(RuntimeError):
    pass


def _call(name, *args):
    status = _fn(name)(*args)
    if status != 0:
        message = load_library().ps_last_error().decode("utf-8", "replace")
        raise KernelError(f"{name} failed ({status}): {message}")


_STREAM_HANDLE = None


def _stream():
    if _STREAM_HANDLE is not None:
        return _STREAM_HANDLE
    return torch.cuda.current_stream().cuda_stream


class on_stream:
    """While active, every kernel of this module is launched on ``stream`` (which must be
    torch's current stream, so that torch's own work keeps its order with them) without asking
    torch for it at each launch: that question costs as much as the rest of a launch."""

    def __init__(self, stream: "torch.cuda.Stream"):
        self.handle = stream.cuda_stream

    def __enter__(self):
        global _STREAM_HANDLE
        self.previous = _STREAM_HANDLE
        _STREAM_HANDLE = self.handle
        return self

    def __exit__(self, *exc):
        global _STREAM_HANDLE
        _STREAM_HANDLE = self.previous
        return False


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"dtype {dtype} is not supported by the kernels "
                          "(float32 and bfloat16 are)") from None


def _check(tensor, name, dtype=None, ndim=None):
    if not isinstance(tensor, torch.Tensor):
        raise KernelError(f"{name} must be a tensor")
    if not tensor.is_cuda:
        raise KernelError(f"{name} must live on the GPU; the engine has no CPU path")
    if dtype is not None and tensor.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {tensor.dtype}")
    if ndim is not None and tensor.ndim != ndim:
        raise KernelError(f"{name} must have {ndim} dimensions, got shape {tuple(tensor.shape)}")
    return tensor


def _rows(tensor, name):
    """2-D tensor with unit stride in its last dimension; returns the row stride."""
    if tensor.ndim != 2 or (tensor.shape[1] > 1 and tensor.stride(1) != 1):
        raise KernelError(f"{name} must be 2-D with contiguous rows, got shape "
                          f"{tuple(tensor.shape)} strides {tuple(tensor.stride())}")
    return tensor.stride(0) if tensor.shape[0] > 1 else max(tensor.stride(0), tensor.shape[1])


def _ptr(tensor):
    return 0 if tensor is None else tensor.data_ptr()


def embed(table, pos_table, ids, positions, out, token_src=None, carried=None, scale=1.0, norm=None):
    """out[t] = scale * table[id(t)] + pos_table[positions[t]] as float (pos_table may be None).
    id(t) is ``ids[t]``, or ``carried[token_src[t]]`` where ``token_src[t] >= 0``: a token
    that an earlier step chose on the device.  ``norm = (gamma, eps)``: every row is then
    RMS-normed in the same launch, ``out / sqrt(mean(out^2) + eps) * gamma``."""
    _check(table, "table", ndim=2)
    _check(ids, "ids", torch.int32, 1)
    _check(out, "out", torch.float32, 2)
    tokens = ids.numel()
    width = table.shape[1]
    if not (table.is_contiguous() and out.is_contiguous() and ids.is_contiguous()):
        raise KernelError("embed: tensors must be contiguous")
    if out.shape[0] < tokens or out.shape[1] != width:
        raise KernelError(f"embed: out {tuple(out.shape)} does not fit {tokens} rows of {width}")
    max_positions = 0
    if pos_table is not None:
        _check(pos_table, "pos_table", table.dtype, 2)
        _check(positions, "positions", torch.int32, 1)
        if pos_table.shape[1] != width or not pos_table.is_contiguous():
            raise KernelError("embed: position table must be contiguous and as wide as the table")
        if positions.numel() != tokens or not positions.is_contiguous():
            raise KernelError("embed: one position per token is needed")
        max_positions = pos_table.shape[0]
    if token_src is not None:
        _check(token_src, "token_src", torch.int32, 1)
        _check(carried, "carried", torch.int32, 1)
        if token_src.numel() != tokens or not token_src.is_contiguous() or not carried.is_contiguous():
            raise KernelError("embed: one source index per token is needed")
    gamma, eps = None, 1.0
    if norm is not None:
        gamma, eps = norm
        _float_vector(gamma, "norm gamma", width)
    _call("ps_embed", table.data_ptr(), _ptr(pos_table), ids.data_ptr(), _ptr(token_src),
          _ptr(carried if token_src is not None else None),
          _ptr(positions if pos_table is not None else None), out.data_ptr(), tokens, width,
          table.shape[0], max_positions, float(scale), _ptr(gamma), float(eps),
          dtype_code(table.dtype), _stream())
    return out


def norm(x, gamma, beta, eps, out, rows=None, rms=False):
    """out[r] = norm(x[rows[r]]) * gamma + beta; statistics in float."""
    _check(x, "x", torch.float32, 2)
    _check(gamma, "gamma", torch.float32, 1)
    _check(out, "out", ndim=2)
    width = x.shape[1]
    if not (x.is_contiguous() and out.is_contiguous() and gamma.is_contiguous()):
        raise KernelError("norm: tensors must be contiguous")
    if gamma.numel() != width or out.shape[1] != width:
        raise KernelError("norm: widths of x, gamma and out differ")
    if beta is not None:
        _check(beta, "beta", torch.float32, 1)
        if beta.numel() != width or not beta.is_contiguous():
            raise KernelError("norm: beta does not match the width")
    if rows is not None:
        _check(rows, "rows", torch.int32, 1)
        n_rows = rows.numel()
    else:
        n_rows = x.shape[0]
    if out.shape[0] < n_rows:
        raise KernelError("norm: out has too few rows")
    _call("ps_norm", x.data_ptr(), _ptr(rows), gamma.data_ptr(), _ptr(beta), out.data_ptr(),
          n_rows, width, float(eps), 1 if rms else 0, dtype_code(out.dtype), _stream())
    return out


def gemm_nt(a, w, bias, out, epilogue="none"):
    """out[m, n] = epilogue(sum_k a[m, k] w[n, k] + bias[n]).

    ``epilogue='residual'`` adds the product into the float tensor ``out``."""
    _check(a, "a", ndim=2)
    _check(w, "w", a.dtype, 2)
    _check(out, "out", ndim=2)
    lda = _rows(a, "a")
    ldc = _rows(out, "out")
    m, k = a.shape
    n = w.shape[0]
    if w.shape[1] != k or not w.is_contiguous():
        raise KernelError(f"gemm_nt: w {tuple(w.shape)} must be contiguous [n, {k}]")
    if out.shape[0] != m or out.shape[1] != n:
        raise KernelError(f"gemm_nt: out {tuple(out.shape)} must be [{m}, {n}]")
    if bias is not None:
        _check(bias, "bias", torch.float32, 1)
        if bias.numel() != n or not bias.is_contiguous():
            raise KernelError("gemm_nt: bias does not match n")
    if epilogue not in EPILOGUES:
        raise KernelError(f"gemm_nt: unknown epilogue {epilogue!r}")
    _call("ps_gemm_nt", a.data_ptr(), w.data_ptr(), _ptr(bias), out.data_ptr(), m, n, k, lda, ldc,
          dtype_code(a.dtype), dtype_code(out.dtype), EPILOGUES[epilogue], _stream())
    return out


class _LinearArgs(ctypes.Structure):
    _fields_ = [
        ("a", c_void_p), ("w", c_void_p), ("bias", c_void_p), ("c", c_void_p),
        ("m", c_int), ("n", c_int), ("k", c_int), ("lda", c_int), ("ldc", c_int),
        ("dtype", c_int), ("c_dtype", c_int), ("epilogue", c_int),
        ("norm_h", c_void_p), ("norm_rows", c_void_p), ("gamma", c_void_p), ("beta", c_void_p),
        ("norm_out", c_void_p), ("eps", c_float), ("rms", c_int), ("ldh", c_int),
        ("k_pool", c_void_p), ("v_pool", c_void_p), ("tok_item", c_void_p), ("tok_pos", c_void_p),
        ("tables", c_void_p),
        ("table_width", c_int), ("q_cols", c_int), ("kv_cols", c_int), ("head_dim", c_int),
        ("kv_heads", c_int), ("page_size", c_int), ("num_pages", c_int),
        ("w_packed", c_void_p),
        ("a_packed", c_int), ("c_packed_request", c_int), ("c_rows", c_int),
        ("norm_out_rows", c_int), ("c_layout", ctypes.POINTER(c_int)),
        ("top_tokens", c_void_p), ("top_keys", c_void_p), ("top_ticket", c_void_p),
        ("top_done", ctypes.POINTER(c_int)),
        ("scatter_only", c_int),
    ]


class PendingNorm:
    """A norm that has not run yet: the float rows, the parameters, and scratch for the
    normed rows.  ``linear`` fuses it into the product when the kernel can; ``materialize``
    runs it on its own."""

    def __init__(self, h, gamma, beta, eps, rms, scratch, rows=None):
        self.h = h
        self.gamma = gamma
        self.beta = beta
        self.eps = float(eps)
        self.rms = bool(rms)
        self.scratch = scratch
        self.rows = rows

    @property
    def count(self):
        return self.rows.numel() if self.rows is not None else self.h.shape[0]

    def materialize(self):
        count = self.count
        return norm(self.h, self.gamma, self.beta, self.eps, self.scratch[:count], rows=self.rows,
                    rms=self.rms)[:count]


def pack_decode_weight(w):
    """A second copy of the bfloat16 matrix ``w [n, k]`` (k a multiple of 64, else None) for
    the products of few rows: rows padded to a multiple of 16, every 16 x 64 tile laid out in
    the order in which a wave's lanes hold the MFMA operand (``csrc/pagedserve_hip.h`` gives the
    formula), so that a wave's load is 1 KB of consecutive memory.  Made once when weights are
    bound; it doubles the memory of the matrices it is made for."""
    if w.dtype != torch.bfloat16 or w.ndim != 2 or w.shape[1] % 64 != 0 or not w.is_cuda:
        return None
    n, k = w.shape
    padded_rows = -(-n // 16) * 16
    source = w if padded_rows == n else torch.cat([w, w.new_zeros((padded_rows - n, k))])
    # [tile, row in tile, step, lane group, half, 8] -> [tile, step, half, lane group, row, 8]
    return source.view(padded_rows // 16, 16, k // 64, 4, 2, 8).permute(0, 2, 4, 3, 1, 5).contiguous()


def _row_capacity(tensor, columns: int) -> int:
    """Rows of ``columns`` values that fit from the tensor's first element to the end of its
    storage (a workspace slice ``buffer[:tokens]`` has room for the whole buffer)."""
    if tensor.ndim != 2 or tensor.shape[1] != columns or not tensor.is_contiguous():
        return 0
    elements = tensor.untyped_storage().nbytes() // tensor.element_size() - tensor.storage_offset()
    return int(elements // columns)


TOP_SLOTS = 16   # keys per row of a TopChoice (csrc/linear.h: PS_TOP_SLOTS)


class TopChoice:
    """What a product needs to choose each row's token in its own epilogue: 16 keys per row
    and 17 tickets, zero between launches (the kernel leaves them so).  One per stream: launches
    that share it must not overlap."""

    def __init__(self, rows: int, device):
        self.rows = int(rows)
        # 256 bytes from key to key and from ticket to ticket (csrc/linear.h: PS_TOP_STRIDE)
        self.keys = torch.zeros(self.rows * TOP_SLOTS * 32, dtype=torch.int64, device=device)
        self.ticket = torch.zeros((1 + TOP_SLOTS) * 64, dtype=torch.int32, device=device)


_MEMO_LIMIT = 512
# What a memoized call keeps is the bytes of its argument block, nothing that the garbage
# collector has to walk (a stream of requests leaves tens of thousands of blocks behind; as
# ctypes structures with two result integers each they made a full collection take 90 ms, in
# the middle of a step).  The two result integers that a block points at are these, shared by
# all memoized calls: a call's results are read before the next call is made.
_MEMO_LAYOUT = c_int(0)
_MEMO_DONE = c_int(0)


def _memo_key(x, out, scatter, a_packed, choose):
    """What may differ between two calls of one call site, in two parts: the row count and
    the addresses of the step's buffers and index arrays, which the same call site of another
    layer meets too, and the addresses that tell the site's own operands apart where it may be
    called with several (its norm's parameters; the cache pools, of which a block that runs
    twice in a step has two pairs).  Weights, bias and flags are the site's own and in neither."""
    if isinstance(x, PendingNorm):
        step = (x.count, x.h.data_ptr(), _ptr(x.rows), x.scratch.data_ptr(), out.data_ptr())
        site = (x.gamma.data_ptr(),)
    else:
        step = (x.shape[0], x.data_ptr(), x.stride(0), out.data_ptr(), a_packed)
        site = ()
    if scatter is not None:
        step += (scatter[2].data_ptr(), scatter[3].data_ptr(), scatter[4].data_ptr())
        site += (scatter[0].data_ptr(), scatter[1].data_ptr())
    if choose is not None:
        step += (choose[1].data_ptr(),)
    return step, site


def _field_ranges(names):
    return tuple((getattr(_LinearArgs, name).offset,
                  getattr(_LinearArgs, name).offset + getattr(_LinearArgs, name).size) for name in names)


# The fields of an argument block by who decides them.  The site's own: its weights and bias,
# equal on every call, and the norm parameters and pools that the call was made with (the second
# part of ``_memo_key``).  The step's: equal for the same call site of every layer within a step
# (the layers share the workspace and the index arrays).  All others are sizes, codes and flags.
_SITE_FIELDS = ("w", "bias", "gamma", "beta", "k_pool", "v_pool", "w_packed")
_STEP_FIELDS = ("a", "c", "m", "lda", "ldc", "norm_h", "norm_rows", "norm_out", "tok_item", "tok_pos",
                "tables", "table_width", "a_packed", "c_rows", "norm_out_rows", "c_layout",
                "top_tokens", "top_keys", "top_ticket", "top_done")
_SITE_RANGES = _field_ranges(_SITE_FIELDS)
_SIZE_RANGES = _field_ranges(name for name, _ in _LinearArgs._fields_
                             if name not in _SITE_FIELDS and name not in _STEP_FIELDS)
_NULL = bytes(ctypes.sizeof(c_void_p))


def _sibling_block(sibling: bytes, own: bytes):
    """The argument block of this site for a step whose block for the same call site of another
    layer is ``sibling`` (checked in this step, same buffers and index arrays), from ``own``, a
    checked block of this site for other rows: the step's fields of the one with the site's
    fields of the other.  None where the two sites do not agree in every size, code and flag,
    or in which of their own operands they have at all."""
    for begin, end in _SIZE_RANGES:
        if sibling[begin:end] != own[begin:end]:
            return None
    block = bytearray(sibling)
    for begin, end in _SITE_RANGES:
        if (sibling[begin:end] == _NULL) != (own[begin:end] == _NULL):
            return None
        block[begin:end] = own[begin:end]
    return bytes(block)


def linear(x, w, bias, out, epilogue="none", scatter=None, packed=None, a_packed=False,
           packed_out=False, choose=None, scatter_only=False, memo=None, shared=None):
    """out = epilogue(x w^T + bias) where ``x`` is a tensor or a ``PendingNorm``.

    ``scatter = (k_pool, v_pool, tok_item, tok_pos, tables, q_cols, kv_cols)`` also stores the
    key and value columns of a ``[q | k | v]`` output into their cache pages.  ``packed`` is
    ``pack_decode_weight(w)`` or None; the kernels for few rows read it instead of ``w``.
    ``scatter_only=True`` says that nobody reads the key and value columns of ``out``: a kernel
    may then leave them unwritten (unspecified afterwards), which the one for many rows does.

    Between two products of 17 to 64 rows the activations may travel in the order in which the
    second one's lanes hold them (``csrc/linear.h: packed_offset``).  ``packed_out=True`` allows
    that for ``out`` (whose storage must have room for the rows rounded up to 16) and makes the
    call return ``(out, written_packed)``; the buffer then goes to the next call with
    ``a_packed=written_packed`` and means nothing to anyone else.

    ``choose = (TopChoice, tokens)`` asks for ``tokens[r]`` = the column of the largest value of
    row ``r`` of a float ``out`` (the lowest on ties), as ``sample`` gives it without a
    temperature; the call then returns ``(out, chosen)``, and where ``chosen`` is False the
    kernel that ran could not do it and ``tokens`` is untouched.

    ``memo``: a dict that belongs to ONE call site, whose ``w``, ``bias``, ``packed``, epilogue
    and flags are the same on every call (a part's product).  The checked argument block of a
    call is kept in it under the row count and the addresses of the other operands, and a call
    that finds its block goes straight to the library: checking and filling the block costs
    the host more than the launch, and a step that is not replayed from a graph issues four
    such calls a layer.  Whoever binds other weights clears the dict; and because a block also
    holds the room behind the addresses (rows that a buffer has space for), a site keeps one
    dict per set of buffers (``parts.base.site_memo``).

    ``shared``: a dict that lives for ONE step and is handed to the calls of all layers.  A
    step with a row count that a site has not seen finds nothing in the site's memo; but the
    same call site of the layer before has just had its block checked for the very same
    buffers and index arrays, and left it here.  This site's block is then that one with the
    site's own operands (weights, bias, norm parameters, pools) taken from a block that this
    site was checked with for the same norm parameters and pools, provided the two agree in
    every size, code and flag: one check per step instead of one per layer."""
    if memo is not None:
        step_key, site_key = _memo_key(x, out, scatter, a_packed, choose)
        key = step_key + site_key
        kept = memo.get(key)
        if kept is None and shared is not None:
            # (a checked block of this site with these very norm parameters and pools)
            sibling, own = shared.get(step_key), memo.get(("site",) + site_key)
            if sibling is not None and own is not None:
                kept = _sibling_block(sibling, own)
                if kept is not None:
                    if len(memo) >= _MEMO_LIMIT:
                        memo.clear()
                        memo[("site",) + site_key] = own
                    memo[key] = kept
        if kept is not None:
            # (the library reads the block and writes through the pointers in it only)
            status = _BOUND["ps_linear_bytes"](kept, _stream())
            if status != 0:
                raise KernelError(f"ps_linear failed ({status}): "
                                  f"{load_library().ps_last_error().decode('utf-8', 'replace')}")
            if packed_out:
                return out, bool(_MEMO_LAYOUT.value)
            if choose is not None:
                return out, bool(_MEMO_DONE.value)
            return out
    _check(w, "w", ndim=2)
    _check(out, "out", ndim=2)
    n, k = w.shape
    if not w.is_contiguous():
        raise KernelError("linear: w must be contiguous")
    args = _LinearArgs()
    if isinstance(x, PendingNorm):
        _check(x.h, "norm input", torch.float32, 2)
        _check(x.gamma, "gamma", torch.float32, 1)
        if x.h.shape[1] != k or x.gamma.numel() != k or not x.h.is_contiguous():
            raise KernelError("linear: norm input rows must be contiguous and k wide")
        if x.beta is not None:
            _check(x.beta, "beta", torch.float32, 1)
        m = x.count
        _check(x.scratch, "norm scratch", w.dtype, 2)
        if x.scratch.shape[0] < m or x.scratch.shape[1] != k or not x.scratch.is_contiguous():
            raise KernelError("linear: norm scratch must be contiguous [>= m, k]")
        if x.rows is not None:
            _check(x.rows, "rows", torch.int32, 1)
        args.norm_h = x.h.data_ptr()
        args.norm_rows = _ptr(x.rows)
        args.gamma = x.gamma.data_ptr()
        args.beta = _ptr(x.beta)
        args.norm_out = x.scratch.data_ptr()
        args.eps = x.eps
        args.rms = 1 if x.rms else 0
        args.ldh = k
        args.lda = k
        args.norm_out_rows = _row_capacity(x.scratch, k)
        if a_packed:
            raise KernelError("linear: a pending norm has no packed rows")
    else:
        _check(x, "x", w.dtype, 2)
        if x.shape[1] != k:
            raise KernelError(f"linear: x {tuple(x.shape)} does not match w {tuple(w.shape)}")
        m = x.shape[0]
        args.a = x.data_ptr()
        args.lda = _rows(x, "x")
        if a_packed:
            if _row_capacity(x, k) < -(-m // 16) * 16:
                raise KernelError("linear: packed input rows need a dense buffer with room for "
                                  "the row count rounded up to 16")
            args.a_packed = 1
    if out.shape[0] != m or out.shape[1] != n:
        raise KernelError(f"linear: out {tuple(out.shape)} must be [{m}, {n}]")
    if bias is not None:
        _check(bias, "bias", torch.float32, 1)
        if bias.numel() != n or not bias.is_contiguous():
            raise KernelError("linear: bias does not match n")
    if epilogue not in EPILOGUES:
        raise KernelError(f"linear: unknown epilogue {epilogue!r}")
    args.w = w.data_ptr()
    if packed is not None:
        if (packed.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or not packed.is_cuda
                or not packed.is_contiguous() or k % 64 != 0
                or packed.numel() != -(-n // 16) * 16 * k):
            raise KernelError(f"linear: the packed copy does not belong to w {tuple(w.shape)}")
        args.w_packed = packed.data_ptr()
    args.bias = _ptr(bias)
    args.c = out.data_ptr()
    args.m, args.n, args.k = m, n, k
    args.ldc = _rows(out, "out")
    args.dtype = dtype_code(w.dtype)
    args.c_dtype = dtype_code(out.dtype)
    args.epilogue = EPILOGUES[epilogue]
    if scatter is not None:
        k_pool, v_pool, tok_item, tok_pos, tables, q_cols, kv_cols = scatter
        pages, kv_heads, page_size, head_dim = _check_pools(k_pool, v_pool, w.dtype)
        _check_step_index(tok_item, tok_pos, tables, m)
        args.k_pool = k_pool.data_ptr()
        args.v_pool = v_pool.data_ptr()
        args.tok_item = tok_item.data_ptr()
        args.tok_pos = tok_pos.data_ptr()
        args.tables = tables.data_ptr()
        args.table_width = tables.shape[1]
        args.q_cols, args.kv_cols = int(q_cols), int(kv_cols)
        args.head_dim, args.kv_heads = head_dim, kv_heads
        args.page_size, args.num_pages = page_size, pages
        args.scatter_only = 1 if scatter_only else 0
    layout = _MEMO_LAYOUT if memo is not None else c_int(0)
    if packed_out:
        args.c_packed_request = 1
        args.c_rows = _row_capacity(out, n)
        args.c_layout = ctypes.pointer(layout)
    done = _MEMO_DONE if memo is not None else c_int(0)
    if choose is not None:
        top, tokens = choose
        _check(tokens, "tokens", torch.int32, 1)
        if out.dtype != torch.float32 or epilogue != "none" or scatter is not None or packed_out:
            raise KernelError("linear: tokens are chosen from a plain float output")
        if tokens.numel() < m or not tokens.is_contiguous():
            raise KernelError(f"linear: {m} rows need as many tokens")
        if top.rows >= m:            # (more rows than there are keys for: the caller samples)
            args.top_tokens = tokens.data_ptr()
            args.top_keys = top.keys.data_ptr()
            args.top_ticket = top.ticket.data_ptr()
            args.top_done = ctypes.pointer(done)
    lib = load_library()
    fn = _BOUND.get("ps_linear")
    if fn is None:
        lib.ps_linear_args_size.restype = c_int
        if lib.ps_linear_args_size() != ctypes.sizeof(_LinearArgs):
            raise KernelError("ps_linear: the argument block of this module "
                              f"({ctypes.sizeof(_LinearArgs)} bytes) is not the library's "
                              f"({lib.ps_linear_args_size()} bytes); rebuild the library")
        fn = lib.ps_linear
        fn.argtypes = [ctypes.POINTER(_LinearArgs), c_void_p]
        fn.restype = c_int
        _BOUND["ps_linear"] = fn
        # the same entry point taking the block as a bytes object (a second function object:
        # argument types belong to the object, not to the symbol)
        from_bytes = lib["ps_linear"]
        from_bytes.argtypes = [ctypes.c_char_p, c_void_p]
        from_bytes.restype = c_int
        _BOUND["ps_linear_bytes"] = from_bytes
    status = fn(ctypes.byref(args), _stream())
    if status != 0:
        raise KernelError(f"ps_linear failed ({status}): {lib.ps_last_error().decode('utf-8', 'replace')}")
    if memo is not None:
        if len(memo) >= _MEMO_LIMIT:
            memo.clear()
        memo[key] = memo[("site",) + site_key] = bytes(args)
        if shared is not None:
            shared[step_key] = memo[key]
    if packed_out:
        return out, bool(layout.value)
    if choose is not None:
        return out, bool(done.value)
    return out


def _check_pools(k_pool, v_pool, dtype):
    _check(k_pool, "k_pool", dtype, 4)
    _check(v_pool, "v_pool", dtype, 4)
    if k_pool.shape != v_pool.shape or not (k_pool.is_contiguous() and v_pool.is_contiguous()):
        raise KernelError("key and value pools must be contiguous and of one shape")
    return k_pool.shape  # pages, kv_heads, page_size, head_dim


def _check_step_index(tok_item, tok_pos, tables, tokens, direct_items=False):
    """``direct_items``: the caller's kernel takes ``tok_item=None`` for "token t is item t"."""
    _check(tok_pos, "tok_pos", torch.int32, 1)
    _check(tables, "tables", torch.int32, 2)
    if tok_item is None:
        if not direct_items:
            raise KernelError("this kernel needs the item index of every token")
        if tables.shape[0] < tokens:
            raise KernelError("without item indices the block table needs a row per token")
    else:
        _check(tok_item, "tok_item", torch.int32, 1)
        if tok_item.numel() < tokens or not tok_item.is_contiguous():
            raise KernelError("one item index per token is needed, contiguous")
    if tok_pos.numel() < tokens:
        raise KernelError("one position per token is needed")
    if not (tok_pos.is_contiguous() and tables.is_contiguous()):
        raise KernelError("step index tensors must be contiguous")


def kv_write(k, v, k_pool, v_pool, tok_item, tok_pos, tables):
    """Store rows of k and v ([tokens, kv_heads*head_dim]) at their positions' pages."""
    _check(k, "k", ndim=2)
    _check(v, "v", k.dtype, 2)
    pages, kv_heads, page_size, head_dim = _check_pools(k_pool, v_pool, k.dtype)
    stride = _rows(k, "k")
    if _rows(v, "v") != stride or v.shape != k.shape:
        raise KernelError("kv_write: k and v must share shape and row stride")
    if k.shape[1] != kv_heads * head_dim:
        raise KernelError(f"kv_write: rows of {k.shape[1]} do not match {kv_heads} x {head_dim}")
    tokens = k.shape[0]
    _check_step_index(tok_item, tok_pos, tables, tokens)
    _call("ps_kv_write", k.data_ptr(), v.data_ptr(), stride, k_pool.data_ptr(), v_pool.data_ptr(),
          tok_item.data_ptr(), tok_pos.data_ptr(), tables.data_ptr(), tables.shape[1], tokens,
          kv_heads, head_dim, page_size, pages, dtype_code(k.dtype), _stream())


def _attention_args(q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, tok_list,
                    direct_items=False):
    _check(q, "q", ndim=2)
    _check(out, "out", q.dtype, 2)
    pages, kv_heads, page_size, head_dim = _check_pools(k_pool, v_pool, q.dtype)
    q_stride = _rows(q, "q")
    out_stride = _rows(out, "out")
    tokens = q.shape[0]
    if q.shape[1] != heads * head_dim or out.shape[1] != heads * head_dim or out.shape[0] != tokens:
        raise KernelError("attention: q/out rows must hold heads x head_dim values")
    _check_step_index(tok_item, tok_pos, tables, tokens, direct_items)
    count = tokens
    if tok_list is not None:
        _check(tok_list, "tok_list", torch.int32, 1)
        if not tok_list.is_contiguous():
            raise KernelError("attention: tok_list must be contiguous")
        count = tok_list.numel()
    return pages, kv_heads, page_size, head_dim, q_stride, out_stride, count


def _check_sink(sink, heads):
    """One float per head that enters the softmax's denominator as ``exp(sink[head])``, or None."""
    if sink is None:
        return 0
    _check(sink, "sink", torch.float32, 1)
    if sink.numel() != heads or not sink.is_contiguous():
        raise KernelError(f"attention: the sink needs one float per head ({heads})")
    return sink.data_ptr()


def _check_gate(gate, tokens, heads):
    """(address, row stride) of the gates: a float per token and head whose sigmoid multiplies
    the head's output (columns of a wider float tensor), or (0, 0) for None."""
    if gate is None:
        return 0, 0
    _check(gate, "gate", torch.float32, 2)
    if gate.shape[0] < tokens or gate.shape[1] != heads:
        raise KernelError(f"attention: gates must be float [>= {tokens}, {heads}], got {tuple(gate.shape)}")
    return gate.data_ptr(), _rows(gate, "gate")


def _check_cap(softcap):
    """A cap ``c > 0`` on the scaled scores (``c tanh(s / c)`` enters the softmax), or 0 for none."""
    softcap = float(softcap or 0.0)
    if not softcap >= 0.0 or softcap == float("inf"):
        raise KernelError(f"attention: a score cap must be positive and finite (0: none), got {softcap}")
    return softcap


def attention_rowwise(q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, scale, window=0,
                      tok_list=None, sink=None, gate=None, softcap=0.0):
    """out[t, h] = softmax(q[t, h] . K * scale) V over the cached keys of t's request, for the
    tokens in ``tok_list`` (all when it is None).  ``sink``: one float per head whose
    exponential joins the denominator (a score that has no key and no value)."""
    pages, kv_heads, page_size, head_dim, q_stride, out_stride, count = _attention_args(
        q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, tok_list)
    sink = _check_sink(sink, heads)
    _call("ps_attention_rowwise", q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
          out.data_ptr(), out_stride, _ptr(tok_list), tok_item.data_ptr(), tok_pos.data_ptr(),
          tables.data_ptr(), tables.shape[1], count, heads, kv_heads, head_dim, page_size, pages,
          float(scale), int(window), sink, *_check_gate(gate, q.shape[0], heads), _check_cap(softcap),
          dtype_code(q.dtype), _stream())
    return out


def decode_keys_per_block(head_dim: int, waves: int = 4) -> int:
    """Keys that one block of the split-KV kernel visits per iteration."""
    lanes = -(-head_dim // 8)
    lanes_per_key = 2 if lanes <= 2 else 4 if lanes <= 4 else 8 if lanes <= 8 else 16 if lanes <= 16 else 32
    return (64 // lanes_per_key) * (8 if waves == 16 else 4) * waves


def attention_decode(q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, scale, splits,
                     partial=None, window=0, tok_list=None, waves=4, sink=None, gate=None, softcap=0.0):
    """The same result as ``attention_rowwise`` by the split-KV kernel; ``partial`` is float
    scratch of ``count * heads * splits * (head_dim + 2)`` values when ``splits > 1``.
    ``tok_item=None`` says that token t is item t (row t of ``tables``), as in a step of single
    tokens: the kernel then fetches its block table one trip to memory earlier."""
    pages, kv_heads, page_size, head_dim, q_stride, out_stride, count = _attention_args(
        q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, tok_list, direct_items=True)
    floats = 0
    if splits > 1:
        _check(partial, "partial", torch.float32)
        if not partial.is_contiguous():
            raise KernelError("attention_decode: scratch must be contiguous")
        floats = partial.numel()
    _call("ps_attention_decode", q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
          out.data_ptr(), out_stride, _ptr(partial if splits > 1 else None), floats,
          _ptr(tok_list), _ptr(tok_item), tok_pos.data_ptr(), tables.data_ptr(),
          tables.shape[1], count, heads, kv_heads, head_dim, page_size, pages, float(scale),
          int(window), int(splits), int(waves), _check_sink(sink, heads),
          *_check_gate(gate, q.shape[0], heads), _check_cap(softcap), dtype_code(q.dtype), _stream())
    return out


SHARED_DECODE_KEYS = 64       # keys per tile of the kernel below
SHARED_DECODE_HEADS = 16      # heads of a group that one block serves


def shared_decode_supported(dtype, heads, kv_heads, head_dim, sink=None) -> bool:
    """Whether ``attention_decode_shared`` takes a layer and pays: bfloat16, no sink, and at least
    six query heads to a key/value head (with fewer, a block's tile of 16 heads is mostly empty
    and the kernel per head is as fast)."""
    return (dtype == torch.bfloat16 and sink is None and head_dim % 8 == 0 and 0 < head_dim <= 256
            and heads % kv_heads == 0 and heads // kv_heads >= 6)


def attention_decode_shared(q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, scale, splits, partial,
                            window=0, tok_list=None, gate=None, softcap=0.0):
    """``attention_decode`` by blocks that load a tile of keys once for all heads of a group (up
    to 16) and work on the matrix cores; ``v_pool`` may be ``k_pool``.  ``partial``: float scratch of
    ``count * heads * splits * (head_dim + 2)`` values, also with one range."""
    pages, kv_heads, page_size, head_dim, q_stride, out_stride, count = _attention_args(
        q, k_pool, v_pool, q if out is None else out, tok_item, tok_pos, tables, heads, tok_list,
        direct_items=True)
    if q.dtype != torch.bfloat16:
        raise KernelError("attention_decode_shared: bfloat16 only")
    if out is None and gate is not None:
        raise KernelError("attention_decode_shared: a gate needs output rows")
    _check(partial, "partial", torch.float32)
    if not partial.is_contiguous():
        raise KernelError("attention_decode_shared: scratch must be contiguous")
    _call("ps_attention_decode_shared", q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
          _ptr(out), out_stride, partial.data_ptr(), partial.numel(), _ptr(tok_list), _ptr(tok_item),
          tok_pos.data_ptr(), tables.data_ptr(), tables.shape[1], count, heads, kv_heads, head_dim,
          page_size, pages, float(scale), int(window), int(splits), *_check_gate(gate, q.shape[0], heads),
          _check_cap(softcap), _stream())
    return out


def decode_supported(head_dim) -> bool:
    """Whether the split-KV kernel takes this head size (a lane fetches eight consecutive head
    dimensions of a key in one piece); the row-wise kernel takes every size up to 256."""
    return head_dim % 8 == 0 and 0 < head_dim <= 256


def merge_linear_supported(dtype, tokens, head_dim, packed) -> bool:
    """Whether ``attention_decode_partial`` + ``attention_merge_linear`` take a step: bfloat16,
    up to 16 single-token items, a head size that is a multiple of 64, and the packed copy of the
    output projection's matrix."""
    return (dtype == torch.bfloat16 and packed is not None and 1 <= tokens <= 16
            and head_dim % 64 == 0 and head_dim <= 256)


def attention_decode_partial(q, k_pool, v_pool, partial, tok_item, tok_pos, tables, heads, scale, splits,
                             window=0, tok_list=None, waves=4, sink=None, softcap=0.0):
    """The per-range records of decode attention only (``partial``: float scratch of
    ``count * heads * splits * (head_dim + 2)`` values); ``attention_merge_linear`` merges them.
    ``tok_item=None``: token t is item t, as for ``attention_decode``."""
    _check(q, "q", ndim=2)
    pages, kv_heads, page_size, head_dim = _check_pools(k_pool, v_pool, q.dtype)
    q_stride = _rows(q, "q")
    tokens = q.shape[0]
    if q.shape[1] != heads * head_dim:
        raise KernelError("attention: q rows must hold heads x head_dim values")
    _check_step_index(tok_item, tok_pos, tables, tokens, direct_items=True)
    count = tokens
    if tok_list is not None:
        _check(tok_list, "tok_list", torch.int32, 1)
        if not tok_list.is_contiguous():
            raise KernelError("attention: tok_list must be contiguous")
        count = tok_list.numel()
    _check(partial, "partial", torch.float32)
    if not partial.is_contiguous():
        raise KernelError("attention_decode_partial: scratch must be contiguous")
    _call("ps_attention_decode_partial", q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
          partial.data_ptr(), partial.numel(), _ptr(tok_list), _ptr(tok_item), tok_pos.data_ptr(),
          tables.data_ptr(), tables.shape[1], count, heads, kv_heads, head_dim, page_size, pages,
          float(scale), int(window), int(splits), int(waves), _check_sink(sink, heads),
          _check_cap(softcap), dtype_code(q.dtype), _stream())
    return count


def attention_merge_linear(partial, count, heads, head_dim, splits, w, packed, bias, residual, tok_list=None,
                           heads_per_block=0):
    """residual[t] += (merged attention output of row r) w^T + bias for the ``count`` rows whose
    records ``attention_decode_partial`` left in ``partial``; ``packed`` is ``pack_decode_weight(w)``.
    ``heads_per_block``: 0 (the library chooses), 1, 2 or 4 heads whose results a block sums
    before it adds them to the rows."""
    _check(partial, "partial", torch.float32)
    _check(residual, "residual", torch.float32, 2)
    _check(w, "w", torch.bfloat16, 2)
    n, k = w.shape
    if k != heads * head_dim or residual.shape[1] != n:
        raise KernelError(f"attention_merge_linear: w {tuple(w.shape)} does not fit {heads} heads of "
                          f"{head_dim} and rows of {residual.shape[1]}")
    if packed is None or packed.dtype != torch.bfloat16 or not packed.is_contiguous() \
            or packed.numel() != -(-n // 16) * 16 * k:
        raise KernelError("attention_merge_linear: the packed copy does not belong to w")
    if bias is not None:
        _check(bias, "bias", torch.float32, 1)
        if bias.numel() != n:
            raise KernelError("attention_merge_linear: bias does not match n")
    if tok_list is None and residual.shape[0] < count:
        raise KernelError("attention_merge_linear: fewer residual rows than records")
    _call("ps_attention_merge_linear", partial.data_ptr(), partial.numel(), _ptr(tok_list), int(count),
          int(heads), int(head_dim), int(splits), packed.data_ptr(), _ptr(bias), residual.data_ptr(),
          _rows(residual, "residual"), n, int(heads_per_block), _stream())
    return residual


PREFILL_TILE = 64          # queries per block of the tiled prefill kernel
PREFILL_SMALL_TILE = 32    # and of its variant for steps with few tiles (head sizes up to 128)
PREFILL_LARGE_TILE = 128   # and of its variant for long prompts (head sizes up to 64)
PREFILL_LARGE_TILE_HEAD_DIM = 64
PREFILL_TABLE_MAX = 2048   # block-table entries of an item that it keeps in LDS
_PREFILL_CHECKED = False


def prefill_limits():
    """(queries per tile, widest block table) as the loaded library was built."""
    lib = load_library()
    lib.ps_attention_prefill_query_tile.restype = c_int
    lib.ps_attention_prefill_table_max.restype = c_int
    return lib.ps_attention_prefill_query_tile(), lib.ps_attention_prefill_table_max()


def prefill_small_tile():
    """Queries per tile of the variant for few tiles, as the loaded library was built."""
    lib = load_library()
    lib.ps_attention_prefill_small_tile.restype = c_int
    return lib.ps_attention_prefill_small_tile()


def prefill_large_tile():
    """(queries per tile, largest head size) of the variant for long prompts, as the loaded
    library was built."""
    lib = load_library()
    lib.ps_attention_prefill_large_tile.restype = c_int
    lib.ps_attention_prefill_large_tile_head_dim.restype = c_int
    return lib.ps_attention_prefill_large_tile(), lib.ps_attention_prefill_large_tile_head_dim()


def _check_prefill_constants():
    global _PREFILL_CHECKED
    if not _PREFILL_CHECKED:
        built = prefill_limits() + (prefill_small_tile(),) + prefill_large_tile()
        if built != (PREFILL_TILE, PREFILL_TABLE_MAX, PREFILL_SMALL_TILE, PREFILL_LARGE_TILE,
                     PREFILL_LARGE_TILE_HEAD_DIM):
            raise KernelError(f"attention_prefill: this module lists queries in tiles of {PREFILL_TILE}, "
                              f"{PREFILL_SMALL_TILE} or {PREFILL_LARGE_TILE} (head sizes up to "
                              f"{PREFILL_LARGE_TILE_HEAD_DIM}) and tables of up to {PREFILL_TABLE_MAX}, "
                              f"the library was built for {built}; rebuild the library")
        _PREFILL_CHECKED = True


def prefill_supported(dtype, head_dim, table_width=0) -> bool:
    """Whether the tiled matrix-core kernel takes this storage type, head size and width of
    the block tables (it keeps a tile's table entries in LDS)."""
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= 256
            and table_width <= PREFILL_TABLE_MAX)


def prefill_small_tile_pays(heads, head_dim, tiles) -> bool:
    """Whether ``tiles`` tiles of 64 queries of ``heads`` heads leave so many compute units
    without a block (half of them or more) that tiles of 32 queries are the better cut: a
    prompt portion of some hundred tokens beside decoded ones."""
    return head_dim <= 128 and 2 * heads * tiles <= compute_units()


def prefill_large_tile_pays(heads, head_dim, large_tiles, max_kv_len=0) -> bool:
    """Whether ``large_tiles`` tiles of 128 queries of ``heads`` heads are the better cut: from
    three blocks per compute unit on (two are resident at a time; with fewer the block that
    sees the most keys decides, and it is twice as long) and where a request holds 2,048 keys
    or more (``max_kv_len``: no query sees more; 0 = unknown).  Measured against the tiles of
    64, four of whose blocks share a compute unit: 2 x 4,096 tokens of 12 heads, 768 blocks, 86
    against 97 us; 2 x 4,096 of 25 heads 178 against 202; 2 x 3,072 of 25 heads 107 against 117;
    4 x 2,048 of 12 heads 57 against 59; but 4 x 1,024 of 25 heads, 800 blocks, 35 against 33; 16 x
    512 of 12 heads 24 against 22; 2 x 3,072 of 12 heads, 576 blocks, 65 against 56."""
    return (head_dim <= PREFILL_LARGE_TILE_HEAD_DIM and heads * large_tiles >= 3 * compute_units()
            and (max_kv_len <= 0 or max_kv_len >= 2048))


def attention_prefill(q, k_pool, v_pool, out, tile_item, tile_q0, cu_tokens, kv_lens, tables,
                      heads, scale, window=0, max_kv_len=0, query_tile=PREFILL_TILE, memo=None,
                      shared=None, sink=None, gate=None, softcap=0.0):
    """Attention of items with several tokens, ``query_tile`` (64, 32 or 128) queries per block,
    on the matrix cores.  Blocks start in the order of the tile list, which is cut for that size:
    the tiles that see the most keys belong first.
    ``max_kv_len`` (no query sees more keys; 0 = unknown) only steers the launch shape.
    ``memo``, ``shared``: as in ``attention_mixed``."""
    key = step_key = None
    if memo is not None:
        step_key = ("prefill", q.data_ptr(), q.shape[0], out.data_ptr(),
                    tile_item.data_ptr(), tile_item.numel(), tile_q0.data_ptr(), cu_tokens.data_ptr(),
                    cu_tokens.numel(), kv_lens.data_ptr(), tables.data_ptr(), tables.shape[1], heads, scale,
                    window, max_kv_len, query_tile, _ptr(sink), _ptr(gate), softcap)
        key = step_key + (k_pool.data_ptr(), v_pool.data_ptr())
        kept = memo.get(key) or _sibling_call(memo, shared, key, step_key, k_pool, v_pool)
        if kept is not None:
            _call("ps_attention_prefill", *kept, _stream())
            return out
    _check_prefill_constants()
    _check(q, "q", torch.bfloat16, 2)
    _check(out, "out", torch.bfloat16, 2)
    pages, kv_heads, page_size, head_dim = _check_pools(k_pool, v_pool, q.dtype)
    q_stride = _rows(q, "q")
    out_stride = _rows(out, "out")
    if q.shape[1] != heads * head_dim or out.shape != q.shape:
        raise KernelError("attention_prefill: q/out rows must hold heads x head_dim values")
    for name, tensor in (("tile_item", tile_item), ("tile_q0", tile_q0), ("cu_tokens", cu_tokens),
                         ("kv_lens", kv_lens)):
        _check(tensor, name, torch.int32, 1)
        if not tensor.is_contiguous():
            raise KernelError(f"attention_prefill: {name} must be contiguous")
    _check(tables, "tables", torch.int32, 2)
    tiles = tile_item.numel()
    items = kv_lens.numel()
    if tile_q0.numel() != tiles or cu_tokens.numel() != items + 1 or tables.shape[0] != items \
            or not tables.is_contiguous():
        raise KernelError("attention_prefill: inconsistent tile or item arrays")
    _kept_call("ps_attention_prefill", memo, key,
               (q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
                out.data_ptr(), out_stride, tile_item.data_ptr(), tile_q0.data_ptr(), tiles,
                cu_tokens.data_ptr(), kv_lens.data_ptr(), tables.data_ptr(), tables.shape[1], heads,
                kv_heads, head_dim, page_size, pages, float(scale), int(window), int(max_kv_len),
                int(query_tile), _check_sink(sink, heads), *_check_gate(gate, q.shape[0], heads),
                _check_cap(softcap), dtype_code(q.dtype)),
               shared, step_key, (kv_heads, head_dim, page_size, pages, q.dtype))
    return out


def tiled_f32_supported(dtype, head_dim) -> bool:
    """Whether ``attention_tiled_f32`` takes the shape: float storage, head sizes that are
    multiples of 4 up to 128."""
    return dtype == torch.float32 and head_dim % 4 == 0 and 4 <= head_dim <= 128


_TILED_F32_CHECKED = False


def attention_tiled_f32(q, k_pool, v_pool, out, tile_item, tile_q0, cu_tokens, kv_lens, tables, heads,
                        scale, window=0, sink=None, gate=None, softcap=0.0):
    """Attention of items with several tokens in true 32-bit, ``PREFILL_TILE`` queries per
    block: keys and values pass through LDS once per tile of queries instead of once per query
    (``attention_rowwise``), scores and sums are plain float arithmetic.  The tile list is the
    one of ``attention_prefill`` at that size."""
    global _TILED_F32_CHECKED
    if not _TILED_F32_CHECKED:
        lib = load_library()
        lib.ps_attention_tiled_f32_tile.restype = c_int
        if lib.ps_attention_tiled_f32_tile() != PREFILL_TILE:
            raise KernelError(f"the library's 32-bit tiled attention takes tiles of "
                              f"{lib.ps_attention_tiled_f32_tile()} queries, this module lists tiles "
                              f"of {PREFILL_TILE}; rebuild the library")
        _TILED_F32_CHECKED = True
    _check(q, "q", torch.float32, 2)
    _check(out, "out", torch.float32, 2)
    pages, kv_heads, page_size, head_dim = _check_pools(k_pool, v_pool, q.dtype)
    q_stride = _rows(q, "q")
    out_stride = _rows(out, "out")
    if q.shape[1] != heads * head_dim or out.shape != q.shape:
        raise KernelError("attention_tiled_f32: q/out rows must hold heads x head_dim values")
    for name, tensor in (("tile_item", tile_item), ("tile_q0", tile_q0), ("cu_tokens", cu_tokens),
                         ("kv_lens", kv_lens)):
        _check(tensor, name, torch.int32, 1)
        if not tensor.is_contiguous():
            raise KernelError(f"attention_tiled_f32: {name} must be contiguous")
    _check(tables, "tables", torch.int32, 2)
    tiles = tile_item.numel()
    items = kv_lens.numel()
    if tile_q0.numel() != tiles or cu_tokens.numel() != items + 1 or tables.shape[0] != items \
            or not tables.is_contiguous():
        raise KernelError("attention_tiled_f32: inconsistent tile or item arrays")
    _call("ps_attention_tiled_f32", q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
          out.data_ptr(), out_stride, tile_item.data_ptr(), tile_q0.data_ptr(), tiles,
          cu_tokens.data_ptr(), kv_lens.data_ptr(), tables.data_ptr(), tables.shape[1], heads,
          kv_heads, head_dim, page_size, pages, float(scale), int(window), _check_sink(sink, heads),
          *_check_gate(gate, q.shape[0], heads), _check_cap(softcap), _stream())
    return out


def mixed_supported(dtype, head_dim, table_width=0) -> bool:
    """Whether one launch can take a step's one-token items and its items of several tokens
    together (``attention_mixed``): bfloat16, head sizes of 16 to 64 in steps of 16."""
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 64
            and table_width <= PREFILL_TABLE_MAX)


def _kept_call(name, memo, key, args, shared=None, step_key=None, pool_shape=None):
    """Calls ``name`` with ``args`` and keeps them under ``key``: the next call of this site
    with the same addresses and counts skips the checks that led to them (a step that is not
    replayed from a graph is issued by the host at the GPU's own pace, and the checks of an
    attention call take as long as three launches).  ``shared`` (a dict that lives for one
    step) gets them too, under the part of the key that the same call of the other layers
    shares, with the pools' shape and type."""
    _call(name, *args, _stream())
    if memo is not None:
        if len(memo) >= 256:
            memo.clear()
        memo[key] = args
        memo["site", args[2], args[3]] = pool_shape
        if shared is not None:
            shared[step_key] = (args, pool_shape)


def _sibling_call(memo, shared, key, step_key, k_pool, v_pool):
    """The arguments of an attention call whose checks the same call of another layer has
    passed in this step (same queries' buffer, same index arrays), for this site's pools:
    theirs with the two pool addresses replaced, if these are the pools that this site has been
    checked with and of the other site's shape and type.  None otherwise."""
    if shared is None:
        return None
    pools = (k_pool.data_ptr(), v_pool.data_ptr())
    sibling, own = shared.get(step_key), memo.get(("site",) + pools)
    if sibling is None or own is None:
        return None
    args, pool_shape = sibling
    if own != pool_shape:
        return None
    args = args[:2] + pools + args[4:]
    if len(memo) >= 256:
        memo.clear()
        memo[("site",) + pools] = own
    memo[key] = args
    return args


def attention_mixed(q, k_pool, v_pool, out, tok_list, tok_item, positions, tile_item, tile_q0,
                    cu_tokens, kv_lens, tables, heads, scale, window=0, memo=None, shared=None,
                    sink=None, gate=None, softcap=0.0):
    """The attention of a step that mixes decoded tokens with prompt portions, in one launch:
    the tokens listed in ``tok_list`` (the step's one-token items) as ``attention_decode`` with
    one range of keys computes them, the tiles of 64 queries listed in ``tile_item`` /
    ``tile_q0`` as ``attention_prefill`` does; blocks of both kinds share the compute units.
    ``memo`` (a dict of the call site, for the buffers of one workspace): what a checked call
    handed to the library, by the operands' addresses and counts.  ``shared`` (a dict that
    lives for one step, handed to the calls of all layers): what the same call of the layer
    before was checked with in this step; only the pools differ, and a site whose pools have
    been checked before takes the rest from there."""
    key = step_key = None
    if memo is not None:
        step_key = ("mixed", q.data_ptr(), q.shape[0], out.data_ptr(),
                    tok_list.data_ptr(), tok_list.numel(), tok_item.data_ptr(), positions.data_ptr(),
                    tile_item.data_ptr(), tile_item.numel(), tile_q0.data_ptr(), cu_tokens.data_ptr(),
                    cu_tokens.numel(), kv_lens.data_ptr(), tables.data_ptr(), tables.shape[1], heads, scale, window,
                    _ptr(sink), _ptr(gate), softcap)
        key = step_key + (k_pool.data_ptr(), v_pool.data_ptr())
        kept = memo.get(key) or _sibling_call(memo, shared, key, step_key, k_pool, v_pool)
        if kept is not None:
            _call("ps_attention_mixed", *kept, _stream())
            return out
    _check_prefill_constants()
    _check(q, "q", torch.bfloat16, 2)
    _check(out, "out", torch.bfloat16, 2)
    pages, kv_heads, page_size, head_dim = _check_pools(k_pool, v_pool, q.dtype)
    q_stride = _rows(q, "q")
    out_stride = _rows(out, "out")
    if q.shape[1] != heads * head_dim or out.shape != q.shape:
        raise KernelError("attention_mixed: q/out rows must hold heads x head_dim values")
    for name, tensor in (("tok_list", tok_list), ("tok_item", tok_item), ("positions", positions),
                         ("tile_item", tile_item), ("tile_q0", tile_q0), ("cu_tokens", cu_tokens),
                         ("kv_lens", kv_lens)):
        _check(tensor, name, torch.int32, 1)
        if not tensor.is_contiguous():
            raise KernelError(f"attention_mixed: {name} must be contiguous")
    _check(tables, "tables", torch.int32, 2)
    tiles = tile_item.numel()
    items = kv_lens.numel()
    tokens = q.shape[0]
    if tile_q0.numel() != tiles or cu_tokens.numel() != items + 1 or tables.shape[0] != items \
            or not tables.is_contiguous() or tok_item.numel() != tokens or positions.numel() != tokens \
            or tok_list.numel() > tokens:
        raise KernelError("attention_mixed: inconsistent token, tile or item arrays")
    _kept_call("ps_attention_mixed", memo, key,
               (q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
                out.data_ptr(), out_stride, tok_list.data_ptr(), tok_list.numel(), tok_item.data_ptr(),
                positions.data_ptr(), tile_item.data_ptr(), tile_q0.data_ptr(), tiles,
                cu_tokens.data_ptr(), kv_lens.data_ptr(), tables.data_ptr(), tables.shape[1], heads,
                kv_heads, head_dim, page_size, pages, float(scale), int(window),
                _check_sink(sink, heads), *_check_gate(gate, q.shape[0], heads), _check_cap(softcap),
                dtype_code(q.dtype)),
               shared, step_key, (kv_heads, head_dim, page_size, pages, q.dtype))
    return out


def _float_rows(tensor, name, rows, columns):
    _check(tensor, name, torch.float32, 2)
    if tensor.shape[0] < rows or tensor.shape[1] != columns or not tensor.is_contiguous():
        raise KernelError(f"{name} must be contiguous float [>= {rows}, {columns}], got {tuple(tensor.shape)}")
    return tensor.data_ptr()


def _float_vector(tensor, name, count):
    _check(tensor, name, torch.float32)
    if tensor.numel() != count or not tensor.is_contiguous():
        raise KernelError(f"{name} must hold {count} floats, got shape {tuple(tensor.shape)}")
    return tensor.data_ptr()


def hyper_step(x, tokens, width, streams, write=None, read=None, zero=None):
    """One pass over the copies of the residual stream ``x`` (float ``[>= tokens, streams * width]``).

    ``write = (y, mix, out)``: every copy becomes a mixture of the old copies plus a share of
    the sublayer's result, ``x'_t = sum_s mix[s, t] x_s + out[t] y`` (``y``: float ``[tokens, width]``).
    ``read = (in, gamma, eps, normed)``: ``u = sum_s in[s] x'_s`` and its RMS norm times ``gamma``
    is written to ``normed`` (engine dtype).  ``zero``: a float ``[tokens, width]`` buffer that is
    cleared (it may be ``y``: the next sublayer's products add into it)."""
    _float_rows(x, "x", tokens, streams * width)
    y = mix = out_w = in_w = gamma = normed = None
    eps, out_code = 1.0, F32
    if write is not None:
        y, mix, out_w = write
        _float_rows(y, "y", tokens, width)
        _float_vector(mix, "mix", streams * streams)
        _float_vector(out_w, "out weights", streams)
    if read is not None:
        in_w, gamma, eps, normed = read
        _float_vector(in_w, "in weights", streams)
        _float_vector(gamma, "gamma", width)
        _check(normed, "normed", ndim=2)
        if normed.shape[0] < tokens or normed.shape[1] != width or not normed.is_contiguous():
            raise KernelError("hyper_step: normed must be contiguous [>= tokens, width]")
        out_code = dtype_code(normed.dtype)
    if zero is not None:
        _float_rows(zero, "zero", tokens, width)
    _call("ps_hyper_step", x.data_ptr(), _ptr(y), _ptr(mix), _ptr(out_w), _ptr(in_w), _ptr(gamma),
          float(eps), _ptr(normed), _ptr(zero), tokens, width, streams, out_code, _stream())


def streams_expand(e, x, tokens, width, streams):
    """``x[t, s] = e[t]`` for every copy ``s``."""
    _float_rows(e, "e", tokens, width)
    _float_rows(x, "x", tokens, streams * width)
    _call("ps_streams_expand", e.data_ptr(), x.data_ptr(), tokens, width, streams, _stream())


def streams_collapse(x, rows, out, width, streams):
    """``out[r] = sum_s x[rows[r], s]`` (all rows in order when ``rows`` is None)."""
    _check(x, "x", torch.float32, 2)
    if x.shape[1] != streams * width or not x.is_contiguous():
        raise KernelError("streams_collapse: x must be contiguous [tokens, streams * width]")
    if rows is not None:
        _check(rows, "rows", torch.int32, 1)
        count = rows.numel()
    else:
        count = x.shape[0]
    _float_rows(out, "out", count, width)
    _call("ps_streams_collapse", x.data_ptr(), _ptr(rows), out.data_ptr(), count, width, streams, _stream())
    return out[:count]


def attention_prepare(proj, columns, q_out, k_pool, v_pool, tok_item, tok_pos, tables, heads,
                      key_dim, value_dim, q_gamma=None, k_gamma=None, eps=1e-6, freqs=None,
                      rot_dims=0, v_first=None, v_lambda=None, v_mode=0, value_heads=0, store=True,
                      query_maps=1):
    """Norm, rotation, value mixing and cache write of an attention layer's projection
    (``csrc/pagedserve_hip.h: ps_attention_prepare``).  ``proj``: float ``[tokens, ld]`` with
    the query, key and value columns at ``columns = (q, k, v)``; the pools' head size is the
    width that every head is stored with.  ``value_heads`` (0: as many as key heads): the
    projection holds that many value heads and key/value head j caches value head ``j %
    value_heads``.  ``store=False``: only the queries are prepared, nothing is cached (a layer
    that reads another layer's keys and values; its projection has no key or value columns).
    ``query_maps > 1``: a key head holds that many runs of ``key_dim / query_maps`` dimensions side
    by side, a query head has one run's dimensions, and query head j is written at the places of
    run ``j % query_maps`` of its row, zeros elsewhere: it scores against its own run only."""
    _check(proj, "proj", torch.float32, 2)
    ld = _rows(proj, "proj")
    tokens = proj.shape[0]
    pages, kv_heads, page_size, cache_dim = _check_pools(k_pool, v_pool, q_out.dtype)
    _check(q_out, "q_out", ndim=2)
    q_stride = _rows(q_out, "q_out")
    if q_out.shape[0] < tokens or q_out.shape[1] != heads * cache_dim:
        raise KernelError("attention_prepare: q_out must hold heads x cached head size per row")
    q_col, k_col, v_col = columns
    value_heads = int(value_heads) or kv_heads
    if value_heads < 1 or kv_heads % value_heads or (v_mode and value_heads != kv_heads):
        raise KernelError(f"attention_prepare: {value_heads} value heads under {kv_heads} key heads")
    query_maps = int(query_maps)
    if query_maps < 1 or key_dim % query_maps or (query_maps > 1 and (rot_dims or q_gamma is not None)):
        raise KernelError(f"attention_prepare: {query_maps} runs in keys of {key_dim} (no rotation or norm with runs)")
    q_dim = key_dim // query_maps
    needed = q_col + heads * q_dim
    if store:
        needed = max(needed, k_col + kv_heads * key_dim, v_col + value_heads * value_dim)
    if needed > proj.shape[1]:
        raise KernelError("attention_prepare: the projection's rows are too short for its columns")
    _check_step_index(tok_item, tok_pos, tables, tokens)
    if q_gamma is not None:
        _float_vector(q_gamma, "q_gamma", heads * key_dim)
    if k_gamma is not None:
        _float_vector(k_gamma, "k_gamma", kv_heads * key_dim)
    if rot_dims:
        _float_vector(freqs, "freqs", rot_dims // 2)
    if v_mode:
        _check(v_first, "v_first", q_out.dtype, 2)
        if v_first.shape[0] < tokens or v_first.shape[1] != kv_heads * value_dim or not v_first.is_contiguous():
            raise KernelError("attention_prepare: v_first must be contiguous [>= tokens, kv_heads * value_dim]")
    if v_mode == 2:
        _float_vector(v_lambda, "v_lambda", 1)
    _call("ps_attention_prepare", proj.data_ptr(), ld, q_col, k_col, v_col, q_out.data_ptr(), q_stride,
          k_pool.data_ptr(), v_pool.data_ptr(), _ptr(q_gamma), _ptr(k_gamma), float(eps), _ptr(freqs),
          int(rot_dims), _ptr(v_first), _ptr(v_lambda), int(v_mode), tok_item.data_ptr(),
          tok_pos.data_ptr(), tables.data_ptr(), tables.shape[1], tokens, heads, kv_heads, key_dim,
          value_dim, cache_dim, page_size, pages, value_heads, 1 if store else 0, q_dim, query_maps,
          dtype_code(q_out.dtype), _stream())


def differential_combine(context, lam, factor, eps, gate, out, heads, value_dim, cache_dim, map_major=True):
    """Behind the attention kernels of a differential layer (``csrc/differential.hip``):
    ``context [tokens, 2 * heads * cache_dim]`` holds map m of head h at head ``m * heads + h``
    (``map_major``) or ``2 * h + m``; ``out[t, h] = rms_norm(map0 - lam * map1) * factor * sigmoid(gate[t, h])`` over
    the head's ``value_dim`` values, ``lam`` a float tensor of one number, ``gate`` float columns
    ``[tokens, heads * value_dim]`` of a wider tensor or None."""
    _check(context, "context", ndim=2)
    _check(out, "out", context.dtype, 2)
    tokens = context.shape[0]
    if context.shape[1] != 2 * heads * cache_dim or context.stride(1) != 1:
        raise KernelError(f"differential_combine: context must be [tokens, 2 x {heads} x {cache_dim}]")
    if out.shape[0] < tokens or out.shape[1] != heads * value_dim or out.stride(1) != 1:
        raise KernelError(f"differential_combine: out must be [>= {tokens}, {heads} x {value_dim}]")
    if not 0 < value_dim <= min(cache_dim, 256):
        raise KernelError(f"differential_combine: {value_dim} values in heads cached {cache_dim} wide (up to 256)")
    _float_vector(lam, "lam", 1)
    gate_ld = 0
    if gate is not None:
        _check(gate, "gate", torch.float32, 2)
        if gate.shape[0] < tokens or gate.shape[1] != heads * value_dim or gate.stride(1) != 1:
            raise KernelError("differential_combine: gate must be float [>= tokens, heads * value_dim]")
        gate_ld = gate.stride(0)
    _call("ps_differential_combine", context.data_ptr(), _rows(context, "context"), lam.data_ptr(),
          float(factor), float(eps), _ptr(gate), gate_ld, out.data_ptr(), _rows(out, "out"), tokens,
          heads, value_dim, cache_dim, 1 if map_major else 0, dtype_code(context.dtype), _stream())


def differential_merge(partial, count, splits, lam, factor, eps, gate, out, heads, value_dim, cache_dim,
                       map_major=True, tok_list=None):
    """``differential_combine`` for decoded tokens, from the records that ``attention_decode_partial``
    or ``attention_decode_shared(out=None)`` left in ``partial`` for ``count`` tokens, ``2 * heads``
    heads and ``splits`` key ranges: the ranges of both maps are merged in float, then the
    difference, the norm, the factor and the gate; ``out [>= tokens, heads * value_dim]`` gets the
    rows ``tok_list`` (None: the first ``count``)."""
    _check(partial, "partial", torch.float32)
    _check(out, "out", ndim=2)
    if not partial.is_contiguous() or partial.numel() < count * 2 * heads * splits * (cache_dim + 2):
        raise KernelError("differential_merge: too few records")
    if out.shape[1] != heads * value_dim or out.stride(1) != 1 or (tok_list is None and out.shape[0] < count):
        raise KernelError(f"differential_merge: out must be [>= {count}, {heads} x {value_dim}]")
    if not 0 < value_dim <= min(cache_dim, 256) or not 1 <= splits <= 64:
        raise KernelError(f"differential_merge: {value_dim} values in heads cached {cache_dim} wide, {splits} ranges")
    _float_vector(lam, "lam", 1)
    gate_ld = 0
    if gate is not None:
        _check(gate, "gate", torch.float32, 2)
        if gate.shape[0] < out.shape[0] or gate.shape[1] != heads * value_dim or gate.stride(1) != 1:
            raise KernelError("differential_merge: gate must be float [>= tokens, heads * value_dim]")
        gate_ld = gate.stride(0)
    if tok_list is not None:
        _check(tok_list, "tok_list", torch.int32, 1)
        if tok_list.numel() != count or not tok_list.is_contiguous():
            raise KernelError("differential_merge: tok_list must name the tokens of the records")
    _call("ps_differential_merge", partial.data_ptr(), partial.numel(), _ptr(tok_list), int(count),
          lam.data_ptr(), float(factor), float(eps), _ptr(gate), gate_ld, out.data_ptr(), _rows(out, "out"),
          heads, cache_dim, value_dim, int(splits), 1 if map_major else 0, dtype_code(out.dtype), _stream())


def attention_prepare_heads(proj, columns, q_out, k_pool, v_pool, tok_item, tok_pos, tables, heads,
                            key_dim, value_dim, freqs=None, rot_dims=0, halves=True, magnitude=1.0,
                            head_norm=False, eps=1e-6):
    """``attention_prepare`` for layers that treat every head on its own: rotation of the first
    ``rot_dims`` dimensions of each head (``halves``: dimension i with i + rot_dims / 2, else 2i
    with 2i + 1; cosine and sine times ``magnitude``), then ``head_norm``: each head divided by its
    root mean square over ``key_dim`` (no weight).  ``columns = (q_col, k_col, v_col)``; the value
    columns are stored as projected and may be the key columns."""
    _check(proj, "proj", torch.float32, 2)
    _check(q_out, "q_out", ndim=2)
    pages, kv_heads, page_size, cache_dim = _check_pools(k_pool, v_pool, q_out.dtype)
    tokens = proj.shape[0]
    q_col, k_col, v_col = (int(c) for c in columns)
    ld = _rows(proj, "proj")
    if max(q_col + heads * key_dim, k_col + kv_heads * key_dim, v_col + kv_heads * value_dim) > proj.shape[1]:
        raise KernelError("attention_prepare_heads: the projection's rows are too short for its columns")
    if q_out.shape[0] < tokens or q_out.shape[1] != heads * cache_dim:
        raise KernelError(f"attention_prepare_heads: q_out must be [>= {tokens}, {heads} x {cache_dim}]")
    if cache_dim < max(key_dim, value_dim) or cache_dim > 256:
        raise KernelError(f"attention_prepare_heads: cached heads of {cache_dim} must hold keys of "
                          f"{key_dim} and values of {value_dim}, up to 256")
    _check_step_index(tok_item, tok_pos, tables, tokens)
    if rot_dims:
        _float_vector(freqs, "freqs", rot_dims // 2)
    _call("ps_attention_prepare_heads", proj.data_ptr(), ld, q_col, k_col, v_col, q_out.data_ptr(),
          _rows(q_out, "q_out"), k_pool.data_ptr(), v_pool.data_ptr(), _ptr(freqs), int(rot_dims),
          1 if halves else 0, float(magnitude), 1 if head_norm else 0, float(eps), tok_item.data_ptr(),
          tok_pos.data_ptr(), tables.data_ptr(), tables.shape[1], tokens, heads, kv_heads, key_dim,
          value_dim, cache_dim, page_size, pages, dtype_code(q_out.dtype), _stream())


def latent_prepare(proj, q_col, kv_col, q_out, k_pool, gamma, eps, tok_item, tok_pos, tables, heads,
                   dim, rank, freqs=None, rot_dims=0, halves=True, magnitude=1.0, queries=None):
    """Latent attention between projection and attention: the token's cached row becomes
    ``[rms_norm(latent) * gamma | rotated key part | zeros]`` and every head's query row gets its
    rotated part at ``rank .. rank + rot_dims - 1`` and zeros behind (the first ``rank`` places
    are left to the caller).  ``proj``: per head ``[dim | rot_dims]`` from ``q_col`` on, ``[rank |
    rot_dims]`` from ``kv_col`` on.  ``queries``: float rows of their own that hold the heads'
    queries from ``q_col`` on (queries that came through a latent), else they lie in ``proj``.
    ``k_pool [pages, 1, page, cache_dim]``."""
    _check(proj, "proj", torch.float32, 2)
    _check(q_out, "q_out", ndim=2)
    _check(k_pool, "k_pool", q_out.dtype, 4)
    pages, kv_heads, page_size, cache_dim = k_pool.shape
    tokens = proj.shape[0]
    if kv_heads != 1 or not k_pool.is_contiguous() or cache_dim < rank + rot_dims:
        raise KernelError(f"latent_prepare: the pool {tuple(k_pool.shape)} must hold one row of at "
                          f"least {rank + rot_dims} per token")
    if queries is None:
        queries = proj
    else:
        _check(queries, "queries", torch.float32, 2)
        if queries.shape[0] < tokens:
            raise KernelError("latent_prepare: too few rows of queries")
    if q_col + heads * (dim + rot_dims) > queries.shape[1] or kv_col + rank + rot_dims > proj.shape[1]:
        raise KernelError("latent_prepare: the projection's rows are too short for its columns")
    if q_out.shape[0] < tokens or q_out.shape[1] != heads * cache_dim:
        raise KernelError(f"latent_prepare: q_out must be [>= {tokens}, {heads} x {cache_dim}]")
    _float_vector(gamma, "gamma", rank)
    _check_step_index(tok_item, tok_pos, tables, tokens)
    if rot_dims:
        _float_vector(freqs, "freqs", rot_dims // 2)
    _call("ps_latent_prepare", proj.data_ptr(), _rows(proj, "proj"), queries.data_ptr(),
          _rows(queries, "queries"), int(q_col), int(kv_col),
          q_out.data_ptr(), _rows(q_out, "q_out"), k_pool.data_ptr(), gamma.data_ptr(), float(eps),
          _ptr(freqs), int(rot_dims), 1 if halves else 0, float(magnitude), tok_item.data_ptr(),
          tok_pos.data_ptr(), tables.data_ptr(), tables.shape[1], tokens, heads, int(dim), int(rank),
          cache_dim, page_size, pages, dtype_code(q_out.dtype), _stream())


def head_gate(context, gate, heads, head_dim):
    """``context[t, h, :] *= sigmoid(gate[t, h])``; ``gate``: float columns of a wider tensor."""
    _check(context, "context", ndim=2)
    _check(gate, "gate", torch.float32, 2)
    tokens = context.shape[0]
    if context.shape[1] != heads * head_dim or gate.shape[0] < tokens or gate.shape[1] != heads:
        raise KernelError("head_gate: context [tokens, heads * head_dim] and gate [tokens, heads] needed")
    _call("ps_head_gate", context.data_ptr(), _rows(context, "context"), gate.data_ptr(),
          _rows(gate, "gate"), tokens, heads, head_dim, dtype_code(context.dtype), _stream())


def gla_decay(proj, low_col, w, bias, tau, alpha):
    """``alpha[t, c] = sigmoid(bias[c] + sum_r proj[t, low_col + r] w[c, r]) ** (1 / tau)`` in float."""
    _check(proj, "proj", torch.float32, 2)
    _check(w, "w", ndim=2)
    tokens = proj.shape[0]
    channels, rank = w.shape
    if not w.is_contiguous() or low_col + rank > proj.shape[1]:
        raise KernelError("gla_decay: w must be contiguous and its rank fit the projection's rows")
    if bias is not None:
        _float_vector(bias, "bias", channels)
    _float_rows(alpha, "alpha", tokens, channels)
    _call("ps_gla_decay", proj.data_ptr(), _rows(proj, "proj"), low_col, rank, w.data_ptr(), _ptr(bias),
          float(tau), alpha.data_ptr(), tokens, channels, dtype_code(w.dtype), _stream())


def gla_scan(proj, columns, alpha, state, out, cu_tokens, slots, heads, key_dim, value_dim, q_scale,
             longest=0, head_decay=None, silu_inputs=False):
    """The recurrence of gated linear attention over the step's items, token after token
    (``csrc/pagedserve_hip.h: ps_gla_scan``); ``state``: float ``[slots, heads, key_dim, value_dim]``.
    ``longest``: no item brings more tokens than that (0: unknown); it steers the launch shape only.
    ``head_decay``: float ``[heads]``, one decay per head for all its key channels and all tokens
    (``alpha`` is then ``None``).  ``silu_inputs``: queries, keys and values pass silu first."""
    _check(proj, "proj", torch.float32, 2)
    tokens = proj.shape[0]
    q_col, k_col, v_col = columns
    if max(q_col + heads * key_dim, k_col + heads * key_dim, v_col + heads * value_dim) > proj.shape[1]:
        raise KernelError("gla_scan: the projection's rows are too short for its columns")
    if head_decay is not None:
        _float_vector(head_decay, "head_decay", heads)
        if alpha is not None:
            raise KernelError("gla_scan: decays per head and per channel are both given")
    else:
        _float_rows(alpha, "alpha", tokens, heads * key_dim)
    _float_rows(out, "out", tokens, heads * value_dim)
    _check(state, "state", torch.float32, 4)
    if tuple(state.shape[1:]) != (heads, key_dim, value_dim) or not state.is_contiguous():
        raise KernelError(f"gla_scan: state {tuple(state.shape)} must be [slots, {heads}, {key_dim}, {value_dim}]")
    _check(cu_tokens, "cu_tokens", torch.int32, 1)
    _check(slots, "slots", torch.int32, 1)
    items = slots.numel()
    if cu_tokens.numel() != items + 1 or not (cu_tokens.is_contiguous() and slots.is_contiguous()):
        raise KernelError("gla_scan: cu_tokens must hold one entry more than slots")
    _call("ps_gla_scan", proj.data_ptr(), _rows(proj, "proj"), q_col, k_col, v_col, _ptr(alpha),
          state.data_ptr(), out.data_ptr(), cu_tokens.data_ptr(), slots.data_ptr(), items,
          state.shape[0], heads, key_dim, value_dim, float(q_scale), int(longest), _ptr(head_decay),
          int(bool(silu_inputs)), _stream())


def scan_pieces(cu_tokens, items, piece, max_pieces, piece_cu, item_first):
    """Cut the step's items into pieces of ``piece`` tokens: ``piece_cu`` (int32, ``max_pieces + 1``:
    the pieces' token ranges, empty behind the last piece) and ``item_first`` (int32, ``items + 1``).
    ``max_pieces`` must be at least ``tokens // piece + items``."""
    _check(cu_tokens, "cu_tokens", torch.int32, 1)
    _check(piece_cu, "piece_cu", torch.int32, 1)
    _check(item_first, "item_first", torch.int32, 1)
    if cu_tokens.numel() != items + 1 or piece_cu.numel() < max_pieces + 1 or item_first.numel() < items + 1:
        raise KernelError("scan_pieces: an index array is too small")
    _call("ps_scan_pieces", cu_tokens.data_ptr(), items, int(piece), int(max_pieces), piece_cu.data_ptr(),
          item_first.data_ptr(), _stream())


def decay_join(piece_states, state, piece_cu, item_first, slots, head_decay):
    """``piece_states`` (float ``[pieces, heads, ...]``): what every piece leaves from a zero state;
    they get the state at every piece's start, ``state[slot]`` the item's last (``csrc/gla.hip``)."""
    _check(piece_states, "piece_states", torch.float32)
    _check(state, "state", torch.float32)
    heads = state.shape[1]
    per_head = state[0, 0].numel()
    if (piece_states.ndim != state.ndim or tuple(piece_states.shape[1:]) != tuple(state.shape[1:])
            or not (piece_states.is_contiguous() and state.is_contiguous())):
        raise KernelError("decay_join: the pieces' states must have the slots' shape")
    _float_vector(head_decay, "head_decay", heads)
    items = slots.numel()
    if item_first.numel() < items + 1 or piece_cu.numel() < piece_states.shape[0] + 1:
        raise KernelError("decay_join: an index array is too small")
    _call("ps_decay_join", piece_states.data_ptr(), state.data_ptr(), piece_cu.data_ptr(),
          item_first.data_ptr(), slots.data_ptr(), head_decay.data_ptr(), items, heads, per_head, _stream())


def row_norm_gate(o, weight, eps, gate, out):
    """``out[t] = rms_norm(o[t]) * weight * sigmoid(gate[t])``: the norm over the whole row."""
    _check(gate, "gate", torch.float32, 2)
    tokens, columns = gate.shape
    _float_rows(o, "o", tokens, columns)
    _float_vector(weight, "weight", columns)
    _check(out, "out", ndim=2)
    if out.shape[0] < tokens or out.shape[1] != columns:
        raise KernelError("row_norm_gate: out must hold the gate's rows and columns")
    _call("ps_row_norm_gate", o.data_ptr(), weight.data_ptr(), float(eps), gate.data_ptr(),
          _rows(gate, "gate"), out.data_ptr(), _rows(out, "out"), tokens, columns,
          dtype_code(out.dtype), _stream())


def _step_items(cu_tokens, slots, what):
    _check(cu_tokens, "cu_tokens", torch.int32, 1)
    _check(slots, "slots", torch.int32, 1)
    items = slots.numel()
    if cu_tokens.numel() != items + 1 or not (cu_tokens.is_contiguous() and slots.is_contiguous()):
        raise KernelError(f"{what}: cu_tokens must hold one entry more than slots")
    return items


def _scan_state(state, channels, states, taps, what):
    _check(state, "state", torch.float32, 3)
    if tuple(state.shape[1:]) != (channels, states + taps - 1) or not state.is_contiguous():
        raise KernelError(f"{what}: state {tuple(state.shape)} must be [slots, {channels}, "
                          f"{states + taps - 1}]")


def conv_silu(proj, u_col, weight, bias, state, states, x, tok_item, cu_tokens, slots, activation=True):
    """``x[t, c] = silu(bias[c] + sum_j weight[c, j] u[t - taps + 1 + j, c])`` with the raw inputs
    ``u = proj[:, u_col:u_col + channels]`` of the step and, before the step's first token of an
    item, the inputs that the item's slot kept (``state[slot, c, states:]``, oldest first).
    ``activation=False``: the plain convolution, without the silu; ``x`` may be float."""
    _check(proj, "proj", torch.float32, 2)
    _check(weight, "weight", torch.float32, 2)
    tokens = proj.shape[0]
    channels, taps = weight.shape
    if not weight.is_contiguous() or u_col + channels > proj.shape[1]:
        raise KernelError("conv_silu: the projection's rows are too short for its channels")
    if bias is not None:
        _float_vector(bias, "bias", channels)
    _scan_state(state, channels, states, taps, "conv_silu")
    _check(x, "x", ndim=2)
    if x.shape[0] < tokens or x.shape[1] != channels or not x.is_contiguous():
        raise KernelError("conv_silu: x must be contiguous [>= tokens, channels]")
    _check(tok_item, "tok_item", torch.int32, 1)
    if tok_item.numel() < tokens:
        raise KernelError("conv_silu: tok_item is shorter than the step")
    _step_items(cu_tokens, slots, "conv_silu")
    _call("ps_conv_silu", proj.data_ptr(), _rows(proj, "proj"), u_col, weight.data_ptr(), _ptr(bias),
          state.data_ptr(), states, x.data_ptr(), tok_item.data_ptr(), cu_tokens.data_ptr(),
          slots.data_ptr(), tokens, channels, taps, 1 if activation else 0, dtype_code(x.dtype),
          _stream())


def lru_scan(proj, y_col, x_col, u, gates, block, lam, decay_scale, state, out, cu_tokens, slots, taps):
    """The gated linear recurrence with one state per channel, per item and token after token:
    ``a = exp(-decay_scale * sigmoid(gr[t, c]) * softplus(lam[c]))``, ``S = a S + sqrt(1 - a^2)
    sigmoid(gi[t, c]) u[t, c]``, ``out[t, c] = S * gelu_tanh(proj[t, y_col + c])``; a row of
    ``gates`` holds, for every run of ``block`` channels, their ``gr`` and then their ``gi``.
    ``state [slots, channels, taps]``: S, then the channel's last ``taps - 1`` raw inputs of the
    convolution (``proj[:, x_col + c]``), which this launch also keeps up to date."""
    _check(proj, "proj", torch.float32, 2)
    tokens = proj.shape[0]
    channels = lam.numel()
    _float_rows(u, "u", tokens, channels)
    _float_rows(gates, "gates", tokens, 2 * channels)
    _float_vector(lam, "lam", channels)
    _scan_state(state, channels, 1, taps, "lru_scan")
    _check(out, "out", ndim=2)
    if out.shape[0] < tokens or out.shape[1] != channels or not out.is_contiguous():
        raise KernelError("lru_scan: out must be contiguous [>= tokens, channels]")
    if max(y_col, x_col) + channels > proj.shape[1] or min(y_col, x_col) < 0:
        raise KernelError("lru_scan: the projection's rows are too short for its channels")
    items = _step_items(cu_tokens, slots, "lru_scan")
    _call("ps_lru_scan", proj.data_ptr(), _rows(proj, "proj"), int(y_col), int(x_col), u.data_ptr(),
          gates.data_ptr(), int(block), lam.data_ptr(), float(decay_scale), state.data_ptr(), out.data_ptr(),
          cu_tokens.data_ptr(), slots.data_ptr(), items, tokens, channels, int(taps),
          dtype_code(out.dtype), _stream())


def block_linear(x, x_step, w, bias, out, out_step, gate=None, k=None):
    """A product with a block-diagonal matrix.  ``w [blocks, n, kw]`` (stored ``[out, in]``);
    block ``b`` reads the ``k`` (default ``kw``) columns of ``x`` from ``b * x_step`` on and
    writes the ``n`` columns of ``out`` from ``b * out_step`` on, plus ``bias[b * n + j]``, times
    ``sigmoid(gate[t, b * n + j])`` where ``gate`` (float) is given.  ``x`` and ``out`` may be float
    or of the matrices' type (a float matrix takes and gives float rows)."""
    _check(x, "x", ndim=2)
    _check(w, "w", ndim=3)
    _check(out, "out", ndim=2)
    blocks, n, kw = w.shape
    k = kw if k is None else int(k)
    if k != kw or not w.is_contiguous():
        raise KernelError(f"block_linear: w {tuple(w.shape)} must be contiguous [blocks, n, {k}]")
    tokens = x.shape[0]
    if out.shape[0] < tokens:
        raise KernelError("block_linear: out has too few rows")
    x_ld, out_ld = _rows(x, "x"), _rows(out, "out")
    if x.shape[1] < (blocks - 1) * x_step + k or out.shape[1] < (blocks - 1) * out_step + n:
        raise KernelError(f"block_linear: rows of {x.shape[1]} / {out.shape[1]} do not hold {blocks} "
                          f"blocks of {k} inputs ({x_step} apart) / {n} outputs ({out_step} apart)")
    if bias is not None:
        _float_vector(bias, "bias", blocks * n)
    gate_ptr, gate_ld = 0, 0
    if gate is not None:
        _check(gate, "gate", torch.float32, 2)
        if gate.shape[0] < tokens or gate.shape[1] != blocks * n:
            raise KernelError(f"block_linear: gates must be float [>= {tokens}, {blocks * n}]")
        gate_ptr, gate_ld = gate.data_ptr(), _rows(gate, "gate")
    _call("ps_block_linear", x.data_ptr(), dtype_code(x.dtype), x_ld, int(x_step), w.data_ptr(),
          dtype_code(w.dtype), _ptr(bias), out.data_ptr(), dtype_code(out.dtype), out_ld, int(out_step),
          gate_ptr, gate_ld, blocks, n, k, tokens, _stream())
    return out


def step_size(low, w, bias, dt):
    """``dt[t, c] = softplus(bias[c] + sum_r low[t, r] w[c, r])`` in float; ``low``: float columns of
    a wider buffer."""
    _check(low, "low", torch.float32, 2)
    _check(w, "w", ndim=2)
    tokens = low.shape[0]
    channels, rank = w.shape
    if not w.is_contiguous() or low.shape[1] != rank or low.stride(1) != 1:
        raise KernelError("step_size: low must hold the weight's rank in columns")
    if bias is not None:
        _float_vector(bias, "bias", channels)
    _float_rows(dt, "dt", tokens, channels)
    _call("ps_step_size", low.data_ptr(), low.stride(0), rank, w.data_ptr(), _ptr(bias), dt.data_ptr(),
          tokens, channels, dtype_code(w.dtype), _stream())


SCAN_PIECE = 32     # tokens of a piece of the selective scan's launch in pieces
SCAN_FUSED_RANK = 256   # largest rank of the step-size projection that the scan works out itself


def selective_scan_records(tokens, items, channels, states):
    """Floats of the two scratch buffers (records, sums) that ``selective_scan`` needs to cut a
    step of so many tokens and items into pieces."""
    entries = tokens // SCAN_PIECE + 2 * items
    return entries * channels * states, entries * channels


def selective_scan(x, dt, bc, b_col, c_col, proj, u_col, z_col, a_log, skip, state, y, cu_tokens,
                   slots, taps, scratch=None, step_weights=None):
    """The selective recurrence over the step's items (``csrc/pagedserve_hip.h: ps_selective_scan``);
    ``state``: float ``[slots, channels, states + taps - 1]``.  ``scratch = (records, sums)``: float
    buffers of at least ``selective_scan_records(...)`` elements; with them the items are cut into
    pieces that run side by side (three launches: for steps with long portions).
    ``dt=None`` with ``step_weights = (low_col, w, bias)``: the step sizes are worked out inside the
    launch from the columns ``low_col...`` of ``bc`` (``w``: ``[channels, rank]`` of x's dtype, rank <= 256)."""
    _check(x, "x", ndim=2)
    tokens, channels = x.shape
    _check(a_log, "a_log", torch.float32, 2)
    states = a_log.shape[1]
    if a_log.shape[0] != channels or not a_log.is_contiguous() or not x.is_contiguous():
        raise KernelError("selective_scan: a_log must be contiguous [channels, states]")
    low_col, step_w, step_bias, rank = 0, None, None, 0
    if dt is not None:
        _float_rows(dt, "dt", tokens, channels)
    else:
        if step_weights is None:
            raise KernelError("selective_scan: neither step sizes nor the weights to work them out")
        low_col, step_w, step_bias = step_weights
        _check(step_w, "step weights", x.dtype, 2)
        rank = step_w.shape[1]
        if (step_w.shape[0] != channels or not step_w.is_contiguous() or rank > SCAN_FUSED_RANK
                or low_col < 0 or low_col + rank > bc.shape[1]):
            raise KernelError("selective_scan: step weights must be contiguous [channels, rank <= 256]")
        if step_bias is not None:
            _float_vector(step_bias, "step bias", channels)
    _float_vector(skip, "skip", channels)
    _check(bc, "bc", torch.float32, 2)
    _check(proj, "proj", torch.float32, 2)
    if bc.shape[0] < tokens or max(b_col, c_col) + states > bc.shape[1] or bc.stride(1) != 1:
        raise KernelError("selective_scan: bc is too small for the step's B and C")
    if proj.shape[0] < tokens or max(u_col, z_col) + channels > proj.shape[1] or proj.stride(1) != 1:
        raise KernelError("selective_scan: proj is too small for the step's inputs and gates")
    _scan_state(state, channels, states, taps, "selective_scan")
    _check(y, "y", x.dtype, 2)
    if y.shape[0] < tokens or y.shape[1] != channels or not y.is_contiguous():
        raise KernelError("selective_scan: y must be contiguous [>= tokens, channels]")
    items = _step_items(cu_tokens, slots, "selective_scan")
    records = sums = None
    if scratch is not None:
        records, sums = scratch
        need = selective_scan_records(tokens, items, channels, states)
        _check(records, "records", torch.float32, 1)
        _check(sums, "sums", torch.float32, 1)
        if records.numel() < need[0] or sums.numel() < need[1]:
            raise KernelError("selective_scan: the scratch for the pieces is too small")
    _call("ps_selective_scan", x.data_ptr(), _ptr(dt), bc.data_ptr(), bc.stride(0), b_col, c_col,
          proj.data_ptr(), proj.stride(0), u_col, z_col, a_log.data_ptr(), skip.data_ptr(),
          state.data_ptr(), y.data_ptr(), cu_tokens.data_ptr(), slots.data_ptr(), items, channels,
          states, taps, tokens, _ptr(records), _ptr(sums), _ptr(step_w), _ptr(step_bias), low_col, rank,
          dtype_code(x.dtype), _stream())


def stream_step(h, tokens, width, add=None, bias=None, norm=None, zero=None):
    """One pass over the float stream ``h`` (``[>= tokens, width]``), every piece optional:
    ``add = (y, factor)``: ``h += factor * y``, or ``add = (y, factor, column_scale)`` with a float
    per column: ``h += factor * column_scale * y``; ``bias``: a float row added to every token;
    ``norm = (gamma, eps, normed)``: the RMS norm of the new ``h`` times ``gamma`` goes to ``normed``
    (engine dtype); ``zero``: a float ``[tokens, width]`` buffer that is cleared (it may be ``y``)."""
    _float_rows(h, "h", tokens, width)
    y, factor, gamma, eps, normed, code, column_scale = None, 0.0, None, 1.0, None, F32, None
    if add is not None:
        y, factor = add[0], add[1]
        _float_rows(y, "y", tokens, width)
        if len(add) > 2 and add[2] is not None:
            column_scale = add[2]
            _float_vector(column_scale, "column_scale", width)
    if bias is not None:
        _float_vector(bias, "bias", width)
    if norm is not None:
        gamma, eps, normed = norm
        _float_vector(gamma, "gamma", width)
        _check(normed, "normed", ndim=2)
        if normed.shape[0] < tokens or normed.shape[1] != width or not normed.is_contiguous():
            raise KernelError("stream_step: normed must be contiguous [>= tokens, width]")
        code = dtype_code(normed.dtype)
    if zero is not None:
        _float_rows(zero, "zero", tokens, width)
    _call("ps_stream_step", h.data_ptr(), _ptr(y), float(factor), _ptr(column_scale), _ptr(bias), _ptr(gamma), float(eps),
          _ptr(normed), _ptr(zero), tokens, width, code, _stream())


GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def silu_gate(gu, out, activation="silu"):
    """``out[t, c] = act(gu[t, c]) * gu[t, inner + c]`` for float ``gu`` of ``2 * inner`` columns;
    ``act``: ``silu`` or ``gelu_tanh``."""
    if activation not in GATE_ACTIVATIONS:
        raise KernelError(f"silu_gate: activation {activation!r}; known: {', '.join(GATE_ACTIVATIONS)}")
    _check(gu, "gu", torch.float32, 2)
    _check(out, "out", ndim=2)
    tokens, inner = gu.shape[0], gu.shape[1] // 2
    if gu.shape[1] != 2 * inner or out.shape[0] < tokens or out.shape[1] != inner:
        raise KernelError("silu_gate: gu must hold twice out's columns")
    _call("ps_silu_gate", gu.data_ptr(), _rows(gu, "gu"), out.data_ptr(), _rows(out, "out"), tokens,
          inner, GATE_ACTIVATIONS[activation], dtype_code(out.dtype), _stream())


def silu_columns(rows, first, count):
    """``rows[:, first:first + count] = silu(...)`` in place (float rows)."""
    _check(rows, "rows", torch.float32, 2)
    if first < 0 or count <= 0 or first + count > rows.shape[1]:
        raise KernelError("silu_columns: the columns lie outside the rows")
    _call("ps_silu_columns", rows.data_ptr(), _rows(rows, "rows"), first, count, rows.shape[0], _stream())


def pair_norm_mix(a, b, weight_a, weight_b, eps, share, y, tokens, width):
    """``y += share * (rms_norm(a) * weight_a + rms_norm(b) * weight_b)``; ``a`` and ``b`` (float
    ``[tokens, width]``) are cleared."""
    _float_rows(a, "a", tokens, width)
    _float_rows(b, "b", tokens, width)
    _float_rows(y, "y", tokens, width)
    _float_vector(weight_a, "weight_a", width)
    _float_vector(weight_b, "weight_b", width)
    _call("ps_pair_norm_mix", a.data_ptr(), b.data_ptr(), weight_a.data_ptr(), weight_b.data_ptr(),
          float(eps), float(share), y.data_ptr(), tokens, width, _stream())


def moe_route(x, router, groups, keep, top, scale, ids, weights, sigmoid=False, correction=None,
              group_top=1, normalise=False, fixed=0):
    """The experts that every row of ``x`` chooses (``ids``, int32 ``[tokens, top]``) and their
    weights (float): softmax (or ``sigmoid``) over all experts of the 32-bit logits, group-limited
    choice, the scores times ``scale`` (``csrc/moe.hip``).  ``correction``: a float per expert
    that is added to the scores for the choice only; ``group_top``: a group's score is the sum of
    that many of its largest choice scores; ``normalise``: the chosen scores are divided by
    their sum before ``scale``.  ``fixed``: that many more columns of ``ids`` and ``weights`` are
    filled with the numbers ``experts, experts + 1, ..`` and the weight one (experts that every token
    uses, for ``moe_experts(extra=...)``)."""
    if correction is not None:
        _float_vector(correction, "correction", router.shape[0])
    if not 1 <= int(group_top) <= 8:
        raise KernelError(f"moe_route: group_top {group_top} must lie in 1..8")
    _check(x, "x", ndim=2)
    _check(router, "router", torch.float32, 2)
    tokens, width = x.shape
    experts = router.shape[0]
    if router.shape[1] != width or not router.is_contiguous() or x.stride(1) != 1:
        raise KernelError("moe_route: router must be contiguous [experts, width]")
    _check(ids, "ids", torch.int32, 2)
    _check(weights, "weights", torch.float32, 2)
    for tensor in (ids, weights):
        if tensor.shape[0] < tokens or tensor.shape[1] != top + fixed or not tensor.is_contiguous():
            raise KernelError("moe_route: ids and weights must be contiguous [>= tokens, top + fixed]")
    _call("ps_moe_route", x.data_ptr(), x.stride(0), router.data_ptr(), tokens, width, experts,
          int(groups), int(keep), int(top), float(scale), 1 if sigmoid else 0, _ptr(correction),
          int(group_top), 1 if normalise else 0, int(fixed), ids.data_ptr(), weights.data_ptr(),
          dtype_code(x.dtype), _stream())


MOE_TILE = 128            # pairs per tile of the sorted path (csrc/moe.hip)
MOE_GROUPED_FROM = 128    # (token, choice) pairs from which the sorted path on the matrix cores is taken


def moe_grouped_supported(dtype, width, inner) -> bool:
    return dtype == torch.bfloat16 and width % 8 == 0 and inner % 8 == 0


def moe_grouped_tiles(pairs, experts) -> int:
    """Tiles of ``MOE_TILE`` sorted pairs that ``pairs`` pairs of ``experts`` experts can need at most."""
    return -(-pairs // MOE_TILE) + experts


def moe_experts_grouped(x, w1, w2, ids, weights, hidden, out, order, tile_expert, y, gated=True):
    """``moe_experts`` for many rows in bfloat16: the pairs sorted by expert, the products on the
    matrix cores.  ``out``: float ``[>= tokens * top, width]``, ``order``: int32 ``[>= tiles * MOE_TILE]``,
    ``tile_expert``: int32 ``[>= tiles]`` scratch with ``tiles = moe_grouped_tiles(tokens * top, experts)``."""
    _check(x, "x", torch.bfloat16, 2)
    tokens, width = x.shape
    _check(w1, "w1", x.dtype, 3)
    _check(w2, "w2", x.dtype, 3)
    experts, inner = w2.shape[0], w2.shape[2]
    if (tuple(w1.shape) != (experts, (2 if gated else 1) * inner, width) or tuple(w2.shape) != (experts, width, inner)
            or not (w1.is_contiguous() and w2.is_contiguous()) or x.stride(1) != 1):
        raise KernelError("moe_experts_grouped: w1 [experts, (2) * inner, width] and w2 [experts, width, inner] needed")
    _check(ids, "ids", torch.int32, 2)
    _check(weights, "weights", torch.float32, 2)
    top = ids.shape[1]
    if not (ids.is_contiguous() and weights.is_contiguous()) or weights.shape[1] != top:
        raise KernelError("moe_experts_grouped: ids and weights must be contiguous [tokens, top]")
    tiles = moe_grouped_tiles(tokens * top, experts)
    _check(hidden, "hidden", x.dtype, 2)
    if hidden.shape[0] < tokens * top or hidden.shape[1] != inner or not hidden.is_contiguous():
        raise KernelError("moe_experts_grouped: hidden must be contiguous [>= tokens * top, inner]")
    _float_rows(out, "out", tokens * top, width)
    _check(order, "order", torch.int32, 1)
    _check(tile_expert, "tile_expert", torch.int32, 1)
    if order.numel() < tiles * MOE_TILE or tile_expert.numel() < tiles:
        raise KernelError("moe_experts_grouped: the scratch for the sorted pairs is too small")
    _float_rows(y, "y", tokens, width)
    _call("ps_moe_experts_grouped", x.data_ptr(), x.stride(0), w1.data_ptr(), w2.data_ptr(), ids.data_ptr(),
          weights.data_ptr(), hidden.data_ptr(), out.data_ptr(), order.data_ptr(), tile_expert.data_ptr(),
          y.data_ptr(), tokens, width, inner, experts, top, 1 if gated else 0, _stream())


def moe_experts(x, w1, w2, ids, weights, hidden, y, gated=True, extra=None):
    """``y[t] += sum_j weights[t, j] W2[e] (silu(W1[e][:inner] x_t) * (W1[e][inner:] x_t))`` with
    ``e = ids[t, j]``; ``w1``: ``[experts, 2 * inner, width]``, ``w2``: ``[experts, width, inner]``.
    ``gated=False``: the plain form ``W2[e] relu(W1[e] x_t)^2`` with ``w1 [experts, inner, width]``.
    ``extra = (w1x, w2x)``: experts numbered from ``experts`` on, in tensors of their own of the same
    form (``moe_route(fixed=...)`` names them for every token)."""
    _check(x, "x", ndim=2)
    tokens, width = x.shape
    _check(w1, "w1", x.dtype, 3)
    _check(w2, "w2", x.dtype, 3)
    experts, inner = w2.shape[0], w2.shape[2]
    if (tuple(w1.shape) != (experts, (2 if gated else 1) * inner, width) or tuple(w2.shape) != (experts, width, inner)
            or not (w1.is_contiguous() and w2.is_contiguous()) or x.stride(1) != 1):
        raise KernelError("moe_experts: w1 [experts, (2) * inner, width] and w2 [experts, width, inner] needed")
    top = ids.shape[1]
    _check(ids, "ids", torch.int32, 2)
    _check(weights, "weights", torch.float32, 2)
    _check(hidden, "hidden", x.dtype, 2)
    if hidden.shape[0] < tokens * top or hidden.shape[1] != inner or not hidden.is_contiguous():
        raise KernelError("moe_experts: hidden must be contiguous [>= tokens * top, inner]")
    if not (ids.is_contiguous() and weights.is_contiguous()) or weights.shape[1] != top:
        raise KernelError("moe_experts: ids and weights must be contiguous [tokens, top]")
    w1x = w2x = None
    if extra is not None:
        w1x, w2x = extra
        _check(w1x, "extra w1", x.dtype, 3)
        _check(w2x, "extra w2", x.dtype, 3)
        if (tuple(w1x.shape[1:]) != tuple(w1.shape[1:]) or tuple(w2x.shape[1:]) != tuple(w2.shape[1:])
                or w1x.shape[0] != w2x.shape[0] or not (w1x.is_contiguous() and w2x.is_contiguous())):
            raise KernelError("moe_experts: the extra experts must have the form of the others")
    _float_rows(y, "y", tokens, width)
    _call("ps_moe_experts", x.data_ptr(), x.stride(0), w1.data_ptr(), w2.data_ptr(), ids.data_ptr(),
          weights.data_ptr(), hidden.data_ptr(), y.data_ptr(), tokens, width, inner, top,
          1 if gated else 0, experts, _ptr(w1x), _ptr(w2x), dtype_code(x.dtype), _stream())


def gla_output(o, weight, eps, gate, out, heads, value_dim):
    """``out[t, h] = rms_norm(o[t, h]) * weight * silu(gate[t, h])`` over each head's values."""
    _check(gate, "gate", torch.float32, 2)
    tokens = gate.shape[0]
    _float_rows(o, "o", tokens, heads * value_dim)
    _float_vector(weight, "weight", value_dim)
    _check(out, "out", ndim=2)
    if gate.shape[1] != heads * value_dim or out.shape[0] < tokens or out.shape[1] != heads * value_dim:
        raise KernelError("gla_output: gate and out must hold heads x value_dim columns")
    _call("ps_gla_output", o.data_ptr(), weight.data_ptr(), float(eps), gate.data_ptr(), _rows(gate, "gate"),
          out.data_ptr(), _rows(out, "out"), tokens, heads, value_dim, dtype_code(out.dtype), _stream())


def softcap(logits, cap):
    """``logits <- cap * tanh(logits / cap)`` in place (float rows of a possibly wider buffer)."""
    _check(logits, "logits", torch.float32, 2)
    if logits.shape[0]:
        _call("ps_softcap", logits.data_ptr(), _rows(logits, "logits"), logits.shape[0], logits.shape[1],
              float(cap), _stream())
    return logits


def sample(logits, inv_temperature, uniform, out):
    """out[r] = argmax(logits[r]) where inv_temperature[r] == 0, else the inverse-CDF draw of
    softmax(logits[r] * inv_temperature[r]) at uniform[r]."""
    _check(logits, "logits", torch.float32, 2)
    _check(out, "out", torch.int32, 1)
    ld = _rows(logits, "logits")
    rows, vocab = logits.shape
    if out.numel() < rows:
        raise KernelError("sample: out has too few entries")
    if inv_temperature is not None:
        _check(inv_temperature, "inv_temperature", torch.float32, 1)
        _check(uniform, "uniform", torch.float32, 1)
        if inv_temperature.numel() < rows or uniform.numel() < rows:
            raise KernelError("sample: one temperature and one uniform number per row are needed")
    _call("ps_sample", logits.data_ptr(), ld, _ptr(inv_temperature), _ptr(uniform),
          out.data_ptr(), rows, vocab, _stream())
    return out


class StepGraph:
    """An executable HIP graph of the launches issued between ``begin`` and ``end`` on the
    current (non-default) stream."""

    def __init__(self):
        self.handle = None
        self.nodes = 0
        self.replays = 0

    @staticmethod
    def begin():
        lib = load_library()
        lib.ps_graph_begin.argtypes = [c_void_p]
        lib.ps_graph_begin.restype = c_int
        if lib.ps_graph_begin(_stream()) != 0:
            raise KernelError(lib.ps_last_error().decode())

    def end(self):
        lib = load_library()
        lib.ps_graph_end.argtypes = [c_void_p, ctypes.POINTER(c_void_p), ctypes.POINTER(c_int)]
        lib.ps_graph_end.restype = c_int
        handle = c_void_p()
        nodes = c_int(0)
        if lib.ps_graph_end(_stream(), ctypes.byref(handle), ctypes.byref(nodes)) != 0:
            raise KernelError(lib.ps_last_error().decode())
        self.handle = handle
        self.nodes = nodes.value

    @staticmethod
    def abort():
        lib = load_library()
        lib.ps_graph_abort.argtypes = [c_void_p]
        lib.ps_graph_abort(_stream())

    def launch(self):
        fn = _BOUND.get("ps_graph_launch")
        if fn is None:
            fn = load_library().ps_graph_launch
            fn.argtypes = [c_void_p, c_void_p]
            fn.restype = c_int
            _BOUND["ps_graph_launch"] = fn
        if fn(self.handle, _stream()) != 0:
            raise KernelError(load_library().ps_last_error().decode())
        self.replays += 1

    def destroy(self):
        if self.handle is not None:
            lib = load_library()
            lib.ps_graph_destroy.argtypes = [c_void_p]
            lib.ps_graph_destroy(self.handle)
            self.handle = None


_COMPUTE_UNITS = None


def compute_units() -> int:
    """Compute units of the current device (asked once)."""
    global _COMPUTE_UNITS
    if _COMPUTE_UNITS is None:
        _COMPUTE_UNITS = max(1, device_info()["compute_units"])
    return _COMPUTE_UNITS


def device_info():
    units = ctypes.c_int(0)
    lds = ctypes.c_int(0)
    arch = ctypes.create_string_buffer(64)
    fn = load_library().ps_device_info
    fn.restype = c_int
    status = fn(ctypes.byref(units), ctypes.byref(lds), arch, 64)
    if status != 0:
        raise KernelError(load_library().ps_last_error().decode())
    return {"compute_units": units.value, "lds_bytes": lds.value, "arch": arch.value.decode()}
