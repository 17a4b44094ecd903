"""The kernels as Python functions over torch tensors on the GPU.

Every function checks on the host that shapes, types and layouts are what its kernel and grid
assume, then launches on torch's current stream.  There is no other implementation behind
these names: without the built library, or with tensors that are not on the GPU, they raise.
"""
from __future__ import annotations

import contextlib
import ctypes
import threading

import torch

from .build import load_library

PAGE_TOKENS = 64          # tokens in a cache page; the kernels are compiled with the same number
MAX_HEAD_DIM = 256
_F32, _BF16, _I32 = torch.float32, torch.bfloat16, torch.int32


class KernelError(RuntimeError):
    pass


_scope = threading.local()


def _stream():
    held = getattr(_scope, "stream", None)
    return held if held is not None else ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


@contextlib.contextmanager
def stream_scope():
    """Within the scope every kernel of this thread is launched on the stream that is current when the scope
    is entered, asked for once (a model's forward pass launches some 300 kernels and never changes the
    stream; asking torch each time costs more than the launch).  Scopes nest; code that switches streams
    inside one opens a new one."""
    before = getattr(_scope, "stream", None)
    _scope.stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    try:
        yield
    finally:
        _scope.stream = before


def _ptr(t):
    return ctypes.c_void_p(0) if t is None else ctypes.c_void_p(t.data_ptr())


def _need(t, name, dtypes, shape=None):
    # the checks in the order of their cost; the messages are built only when one fails
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name}: expected a tensor, got {type(t).__name__}")
    dt = t.dtype
    if dt is not dtypes and (dtypes.__class__ is torch.dtype or dt not in dtypes):
        want = dtypes if isinstance(dtypes, (tuple, list)) else (dtypes,)
        raise KernelError(f"{name}: dtype {dt}, expected {' or '.join(str(d) for d in want)}")
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor lies on {t.device}; the kernels of synaptix_amd run on the GPU only")
    if not t.is_contiguous():
        raise KernelError(f"{name}: tensor is not contiguous")
    if shape is not None:
        got = t.shape
        ok = len(shape) == len(got)
        if ok:
            for s, g in zip(shape, got):
                if s is not None and s != g:
                    ok = False
                    break
        if not ok:
            raise KernelError(f"{name}: shape {list(got)}, expected {[('*' if s is None else s) for s in shape]}")


def _call(lib, fn, *args):
    if _timing is not None:
        return _timed_call(lib, fn, args)
    rc = getattr(lib, fn)(*args)
    if rc != 0:
        raise KernelError(lib.syn_last_error().decode(errors="replace"))


# ----------------------------------------------------------------------------- per-op times
# The reference can time every op of a forward pass by synchronising the device around it
# (crates/synaptix-models/llm/common/src/model.rs:22-99: prof(name, f), a table of (ms, calls) by name,
# sorted by time, switched on for prefill or decode; off during graph capture).  Here the ops are the
# kernel entry points; op_timing() switches the same thing on for the code inside it.

_timing = None      # None, or {entry point: [milliseconds, calls]}


def _timed_call(lib, fn, args):
    import time
    if torch.cuda.is_current_stream_capturing():
        raise KernelError("op_timing: per-op times need eager steps (synchronising is not allowed while a graph is captured)")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    rc = getattr(lib, fn)(*args)
    torch.cuda.synchronize()
    slot = _timing.setdefault(fn, [0.0, 0])
    slot[0] += (time.perf_counter() - t0) * 1e3
    slot[1] += 1
    if rc != 0:
        raise KernelError(lib.syn_last_error().decode(errors="replace"))


def timing_active() -> bool:
    return _timing is not None


class OpTimes(dict):
    """{entry point: [milliseconds, calls]} with the reference's report: sorted by time, with shares."""

    def report(self) -> str:
        total = sum(v[0] for v in self.values()) or 1.0
        lines = [f"{'op':34s} {'ms':>10s} {'calls':>7s} {'share':>7s}"]
        for name, (ms, calls) in sorted(self.items(), key=lambda kv: -kv[1][0]):
            lines.append(f"{name:34s} {ms:10.3f} {calls:7d} {100 * ms / total:6.1f}%")
        lines.append(f"{'total':34s} {total:10.3f}")
        return "\n".join(lines)


@contextlib.contextmanager
def op_timing():
    """Within the scope every kernel entry point is timed with the device synchronised before and after it
    (so the times include each launch's latency and nothing overlaps); yields the table that fills up.
    Steps inside the scope must be eager: captured steps are refused."""
    global _timing
    before, _timing = _timing, OpTimes()
    try:
        yield _timing
    finally:
        _timing = before


def _is_f32(t):
    return 1 if t.dtype == _F32 else 0


# The activations of a gated feed-forward that the kernels apply (codes of gate_activation in csrc/common.h).
# "swiglu_limit" comes with its bound, as the pair ("swiglu_limit", limit):
#   g <- min(g, limit), u <- clamp(u, -limit, limit);  g sigmoid(1.702 g) (u + 1)
ACTIVATIONS = {"silu": 0, "swish": 0, "gelu_tanh": 1, "swiglu_limit": 2}


def activation_code(name) -> int:
    if isinstance(name, (tuple, list)) and len(name) == 2:
        name = name[0]
    if name not in ACTIVATIONS:
        raise KernelError(f"activation {name!r}: the kernels apply {sorted(set(ACTIVATIONS))}")
    return ACTIVATIONS[name]


def _activation_args(activation):
    """(code, limit) as the entry points take them; an activation with a bound is the pair (name, bound)."""
    code = activation_code(activation)
    limit = 0.0
    if code == ACTIVATIONS["swiglu_limit"]:
        if not isinstance(activation, (tuple, list)) or not float(activation[1]) > 0.0:
            raise KernelError("activation 'swiglu_limit' comes with its bound: ('swiglu_limit', limit), limit > 0")
        limit = float(activation[1])
    return code, ctypes.c_float(limit)


# ----------------------------------------------------------------------------- rows

def embed(table, ids, resid, scale=1.0):
    """resid[n, :] = scale * table[ids[n], :] as float.  table [V, H] bf16|f32 (or bf16 in fragment order, pack_weight: four
    dimensions), ids [N] int32, resid [N, H] f32."""
    if isinstance(table, torch.Tensor) and table.dim() == 4:
        _need(table, "embed.table", _BF16, (None, None, 64, 8))
        H, kind = table.shape[1] * 32, 2
    else:
        _need(table, "embed.table", (_BF16, _F32), (None, None))
        H, kind = table.shape[1], _is_f32(table)
    _need(ids, "embed.ids", _I32, (None,))
    _need(resid, "embed.resid", _F32, (ids.shape[0], H))
    _call(load_library("core"), "syn_embed", _ptr(table), kind, _ptr(ids), _ptr(resid), ids.shape[0], H,
          ctypes.c_float(scale), _stream())


def add_rmsnorm(resid, delta, gain, eps, out, rows=None, gain_offset=0.0):
    """rows is None:  resid += delta (when given), out = RMSNorm(resid) * (gain_offset + gain), for every row.
    rows [n] int32: out[i] = RMSNorm(resid[rows[i]] + delta[rows[i]]) * gain; resid is not written.
    delta may be [S, N, H]: partial sums that are added up on the way."""
    _need(resid, "add_rmsnorm.resid", _F32, (None, None))
    N, H = resid.shape
    n_parts = 1
    if delta is not None:
        if delta.dim() == 3:
            n_parts = delta.shape[0]
            _need(delta, "add_rmsnorm.delta", _F32, (n_parts, N, H))
        else:
            _need(delta, "add_rmsnorm.delta", _F32, (N, H))
    _need(gain, "add_rmsnorm.gain", (_BF16, _F32), (H,))
    n_out = N
    if rows is not None:
        _need(rows, "add_rmsnorm.rows", _I32, (None,))
        n_out = rows.shape[0]
    _need(out, "add_rmsnorm.out", (_BF16, _F32), (n_out, H))
    _call(load_library("core"), "syn_add_rmsnorm", _ptr(resid), _ptr(delta), n_parts, N, _ptr(rows), n_out, _ptr(gain),
          _is_f32(gain), ctypes.c_float(gain_offset), ctypes.c_float(eps), _ptr(out), _is_f32(out), H, _stream())


def rmsnorm_rows(x, gain, eps, out, gain_offset=0.0):
    """out = RMSNorm(x) * (gain_offset + gain) over the last axis; x [..., D] bf16|f32, out like x."""
    _need(x, "rmsnorm_rows.x", (_BF16, _F32))
    D = x.shape[-1]
    _need(gain, "rmsnorm_rows.gain", (_BF16, _F32), (D,))
    _need(out, "rmsnorm_rows.out", x.dtype, tuple(x.shape))
    _call(load_library("core"), "syn_rmsnorm_rows", _ptr(x), _is_f32(x), _ptr(gain), _is_f32(gain),
          ctypes.c_float(gain_offset), ctypes.c_float(eps), _ptr(out), x.numel() // D, D, _stream())


def swiglu(gate_up, out, activation="silu"):
    """out[n, i] = act(gate_up[n, i]) * gate_up[n, I + i]."""
    _need(gate_up, "swiglu.gate_up", (_BF16, _F32), (None, None))
    N, I2 = gate_up.shape
    if I2 % 2:
        raise KernelError(f"swiglu: fused width {I2} is odd")
    _need(out, "swiglu.out", gate_up.dtype, (N, I2 // 2))
    _call(load_library("core"), "syn_swiglu", _ptr(gate_up), _ptr(out), _is_f32(gate_up), N, I2 // 2,
          *_activation_args(activation), _stream())


# ----------------------------------------------------------------------------- matrix product

def _packed_shape(w, name, K):
    """(N, K) of a weight in fragment order (pack_weight), checked against the rows' width."""
    _need(w, name, _BF16, (None, K // 32 if K % 32 == 0 else -1, 64, 8))
    return w.shape[0] * 16


def gemm(x, w, out, force_simt=False):
    """out[M, N] = x[M, K] . w[N, K]^T with 32-bit accumulation.
    float x float -> float (plain FMA); bf16 x bf16 -> bf16 or float (MFMA).
    A float out of shape [S, M, N] (bf16 operands) receives S partial sums over slices of K
    instead; their sum over S is the product.
    w may be the weight in fragment order (pack_weight: four dimensions): the tiles for 9 rows and more read it
    where K is a multiple of 128; for other K the product runs in blocks of 16 rows through gemm_packed."""
    _need(x, "gemm.x", (_BF16, _F32), (None, None))
    M, K = x.shape
    packed = isinstance(w, torch.Tensor) and w.dim() == 4
    if packed:
        if x.dtype != _BF16 or force_simt:
            raise KernelError("gemm: a weight in fragment order takes bf16 rows and the MFMA kernels")
        N = _packed_shape(w, "gemm.w", K)
        if K % 128:
            if out.dim() == 3 and out.shape[0] != 1:
                raise KernelError(f"gemm: no slices of K = {K} over a weight in fragment order")
            rows = out[0] if out.dim() == 3 else out
            for m0 in range(0, M, PACKED_BLOCK_ROWS):
                gemm_packed(x[m0:m0 + PACKED_BLOCK_ROWS], w, rows[m0:m0 + PACKED_BLOCK_ROWS])
            return
    else:
        _need(w, "gemm.w", x.dtype, (None, K))
        N = w.shape[0]
    slices = 1
    if out.dim() == 3:
        slices = out.shape[0]
        if x.dtype != _BF16 or force_simt or (M > 64 and K % 64):
            raise KernelError("gemm: partial sums over slices of K need bf16 operands (and beyond 64 rows a K "
                              "that is a multiple of 64)")
        _need(out, "gemm.out", _F32, (slices, M, N))
        code = 2
    elif x.dtype == _F32:
        _need(out, "gemm.out", _F32, (M, N))
        code = 0
    else:
        _need(out, "gemm.out", (_BF16, _F32), (M, N))
        code = 2 if out.dtype == _F32 else 1
    _call(load_library("core"), "syn_gemm", _ptr(x), _ptr(w), _ptr(out), code, M, N, K, 1 if force_simt else 0,
          slices, 1 if packed else 0, _stream())


PAIR = 16   # rows of the gate and of the up projection alternate in turns of this many


def pair_rows(gate, up):
    """The weight of gemm_swiglu: rows of `gate` and of `up` [I, K] in turns of 16 -> [2 I, K]."""
    I, K = gate.shape
    if up.shape != gate.shape or I % PAIR:
        raise KernelError(f"pair_rows: shapes {tuple(gate.shape)}, {tuple(up.shape)} (rows in turns of {PAIR})")
    return torch.stack([gate.view(I // PAIR, PAIR, K), up.view(I // PAIR, PAIR, K)], 1).reshape(2 * I, K).contiguous()


def gemm_swiglu(x, w_paired, out, activation="silu"):
    """out[M, I] = act(x . Wg^T) * (x . Wu^T) in bf16 with w_paired = pair_rows(Wg, Wu): the
    activation on the 32-bit sums inside the product, so that the two products are never stored.
    w_paired may be in fragment order (pack_weight of the paired rows), as for gemm."""
    _need(x, "gemm_swiglu.x", _BF16, (None, None))
    M, K = x.shape
    packed = isinstance(w_paired, torch.Tensor) and w_paired.dim() == 4
    if packed:
        N = _packed_shape(w_paired, "gemm_swiglu.w", K)
    else:
        _need(w_paired, "gemm_swiglu.w", _BF16, (None, K))
        N = w_paired.shape[0]
    if N % (2 * PAIR) or K % 8:
        raise KernelError(f"gemm_swiglu: {N} paired rows, K = {K} (multiples of {2 * PAIR} and of 8)")
    _need(out, "gemm_swiglu.out", _BF16, (M, N // 2))
    if packed and K % 128:
        for m0 in range(0, M, PACKED_BLOCK_ROWS):
            gemm_packed(x[m0:m0 + PACKED_BLOCK_ROWS], w_paired, out[m0:m0 + PACKED_BLOCK_ROWS], paired=True,
                        activation=activation)
        return
    _call(load_library("core"), "syn_gemm_swiglu", _ptr(x), _ptr(w_paired), _ptr(out), M, N, K,
          *_activation_args(activation), 1 if packed else 0, _stream())


PACKED_BLOCK_ROWS = 16   # the most rows that a product of gemm_packed takes
PACKED_MAX_ROWS = 8   # up to this many rows of x the products over packed weights are the faster ones
PACKED_MAX_ROWS_GATED = 16   # the gated product, whose waves take two groups of rows of W for every fragment of x
PACKED_WIDE_N = 32768   # from this many rows of W on (an output head) the products over packed weights stay the faster
                        # ones up to 16 rows of x (151,936 x 4,096 at 16 rows: 222 us on tiles, as at 8 rows in fragments)


def packed_max_rows(n_out: int) -> int:
    """Up to how many rows of x a plain product with a packed weight of n_out rows takes the kernels for few rows."""
    return PACKED_BLOCK_ROWS if n_out >= PACKED_WIDE_N else PACKED_MAX_ROWS


def pack_weight(w):
    """A copy of the bf16 weight w [N, K] in the order of the MFMA fragments that the products for few
    rows take: [N / 16, K / 32, 64, 8] with lane = 16 * (k % 32 // 8) + n % 16 (every load of a wave is then
    1 KB of consecutive bytes).  None if the shape or the type does not allow it (N a multiple of 16, K of 32)."""
    if w.dtype != _BF16 or w.dim() != 2 or w.shape[0] % 16 or w.shape[1] % 32:
        return None
    N, K = w.shape
    return w.view(N // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).reshape(N // 16, K // 32, 64, 8).contiguous()


def unpack_weight(wp):
    """The inverse of pack_weight: [N, K]."""
    nt, nks = wp.shape[:2]
    return wp.view(nt, nks, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(nt * 16, nks * 32).contiguous()


def gemm_packed(x, wp, out, paired=False, activation="silu", row_scale=None, resid_norm=None):
    """out[M, N] (bf16 or float) = x[M, K] . W^T for M <= 16 with wp = pack_weight(W); paired: W holds gate and
    up rows in turns of 16 (pair_rows) and out [M, N / 2] bf16 = act(gate) * up.  A float out of shape
    [S, M, N] receives S partial sums over slices of K instead.

    The two halves of an RMSNorm that lies between two such products (csrc/gemm.hip: RowNorm):
    resid_norm = (resid [M, N] float, gain [N], gain_offset, xs [M, N] bf16, ss [M, N / 16] float) with out None:
    the sums are added into resid, xs = (gain_offset + gain) * resid, ss = sums of resid^2 over groups of 16 columns;
    row_scale = (ss [M, G] float, dim, eps): the sums of row m are multiplied by rsqrt(sum(ss[m]) / dim + eps), which
    makes this the product over the normed rows when x is the xs that came with ss."""
    _need(x, "gemm_packed.x", _BF16, (None, None))
    M, K = x.shape
    if K % 32:
        raise KernelError(f"gemm_packed: K = {K} is no multiple of 32")
    _need(wp, "gemm_packed.wp", _BF16, (None, K // 32, 64, 8))
    N = wp.shape[0] * 16
    if M > 16 or (paired and N % 32):
        raise KernelError(f"gemm_packed: M = {M} (at most 16), N = {N}")
    slices = 1
    ss = resid = xs = ss_out = gain = None
    groups = dim = 0
    eps = gain_offset = 0.0
    if row_scale is not None:
        ss, dim, eps = row_scale
        _need(ss, "gemm_packed.row_scale", _F32, (M, None))
        groups = ss.shape[1]
        if groups < 1 or dim < 1:
            raise KernelError(f"gemm_packed: a row statistic of {groups} groups over {dim} columns")
    if resid_norm is not None:
        resid, gain, gain_offset, xs, ss_out = resid_norm
        if paired or out is not None:
            raise KernelError("gemm_packed: the product before a norm is not gated and has no output beside resid, xs and ss")
        _need(resid, "gemm_packed.resid", _F32, (M, N))
        _need(gain, "gemm_packed.gain", (_BF16, _F32), (N,))
        _need(xs, "gemm_packed.xs", _BF16, (M, N))
        _need(ss_out, "gemm_packed.ss", _F32, (M, N // 16))
        out_code = 2
    elif paired:
        _need(out, "gemm_packed.out", _BF16, (M, N // 2))
        out_code = 1
    elif out.dim() == 3:          # float partial sums over slices of K, which the reader adds
        slices = out.shape[0]
        _need(out, "gemm_packed.out", _F32, (slices, M, N))
        out_code = 2
    else:
        _need(out, "gemm_packed.out", (_BF16, _F32), (M, N))
        out_code = 2 if out.dtype == _F32 else 1
    if row_scale is None and resid_norm is None:
        _call(load_library("core"), "syn_gemm_packed", _ptr(x), _ptr(wp), _ptr(out), out_code,
              M, N, K, 1 if paired else 0, *_activation_args(activation), slices, _stream())
        return
    _call(load_library("core"), "syn_gemm_packed_norm", _ptr(x), _ptr(wp), _ptr(out), out_code, M, N, K,
          1 if paired else 0, *_activation_args(activation), slices, _ptr(ss), int(groups), int(dim), ctypes.c_float(eps),
          _ptr(resid), _ptr(xs), _ptr(ss_out), _ptr(gain), _is_f32(gain) if gain is not None else 0,
          ctypes.c_float(gain_offset), _stream())


_compute_units = None


def compute_units() -> int:
    """Compute units of the GPU that the rules below fill: asked of the device once (256 on an MI355X, which is also
    what the rules assume where no GPU is present, as in tests of the rules themselves).  The C side asks the
    device the same question (csrc/gemm.hip: compute_units)."""
    global _compute_units
    if _compute_units is None:
        _compute_units = (torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
                          if torch.cuda.is_available() else 256)
    return _compute_units


def packed_slices(N, K):
    """Into how many slices of K gemm_packed is cut when its reader can add partial sums.  It has a workgroup
    for every 16 rows of W, each with a fixed share of the weight stream; when their number is no
    multiple of the compute units the last round runs half empty (N = 5120: 320 workgroups, two rounds for
    the work of 1.25; N = 2560: 160 compute units of 256).  The smallest cut that fills its rounds to 90 %
    is taken, if one exists among up to 8 slices of at least 1,024."""
    groups, units = -(-N // 16), compute_units()

    def fill(s):
        work = groups * s / units
        return work / -(-groups * s // units)

    best = 1
    for s in (1, 2, 3, 4, 5, 6, 8):
        if s > 1 and K // s < 1024:
            break
        if fill(s) >= 0.9:
            return s
        if fill(s) > fill(best) + 0.05:
            best = s
    return best


def gemm_slices(M, N, K, dtype):
    """Into how many slices of K a product is cut when its reader can add partial sums.  A product
    with few rows of W has too few workgroups (one for every 64 rows) to pull the weights at speed.
    The cut aims at one round of workgroups over the 256 compute units; up to 32 rows of x, where the
    tiles keep three k-tiles in flight, four slices are enough (and leave the reader fewer partial
    sums to add); measured at the shapes of an 8B model (N = 4096 and 6144, K = 4096 and 12288) for
    1, 8, 32 and 64 rows."""
    if dtype != _BF16 or K % 8 != 0 or N > 16384 or K < 2048:
        return 1
    units = compute_units()
    if M > 64:
        # prompts: 256 x 256 tiles are the most efficient, but a narrow product has too few of them for
        # the 256 compute units (128 at 2,048 rows and N = 4096); two or four slices of K fill the chip,
        # at the price of partial sums of M x N floats each
        if K % 128:
            return 1
        if M <= 512:
            # short prompts: still bound by reading W; tiles of 128 rows of W (and of 128 rows of x up to 256 rows,
            # of 256 beyond), cut until they fill the compute units
            tiles = (-(-M // 128) if M <= 256 else -(-M // 256)) * -(-N // 128)
            most, slices = min(8, units // tiles, K // 512), 1
            while slices * 2 <= most:
                slices *= 2
            if slices > 1:
                return slices
        tiles = -(-M // 256) * -(-N // 256)
        return 4 if tiles * 4 <= units and K >= 8192 else (2 if tiles * 2 <= units else 1)
    if M <= 32:
        # 64 rows of W a workgroup, up to three workgroups a compute unit
        most = min(4, 3 * units // -(-N // 64), K // 512)
    else:
        # 128 rows of W a workgroup, one workgroup a compute unit
        most = min(8, units // -(-N // 128), K // 512)
    slices = 1
    while slices * 2 <= most:
        slices *= 2
    return slices


# ----------------------------------------------------------------------------- attention

def v_pages_to_kernel_order(v):
    """V pages [..., kv_heads, hd, 64] as plain (dim, token) rows -> the same shape holding each page
    in the order the bf16 kernels keep it (fragment after fragment of the decode kernel's MFMA: half of
    the tokens, 16 dims, lane group of 8 tokens, dim, token).  Float pages are plain and stay as they are."""
    if v.dtype != _BF16:
        return v
    lead, hd = v.shape[:-2], v.shape[-2]
    x = v.reshape(*lead, hd // 16, 16, 2, 4, 8)            # [dt, r, h, g, e]
    n = len(lead)
    x = x.permute(*range(n), n + 2, n + 0, n + 3, n + 1, n + 4)   # [h, dt, g, r, e]
    return x.reshape(*lead, hd, 64).contiguous()


def v_pages_from_kernel_order(v):
    """The inverse of v_pages_to_kernel_order."""
    if v.dtype != _BF16:
        return v
    lead, hd = v.shape[:-2], v.shape[-2]
    x = v.reshape(*lead, 2, hd // 16, 4, 16, 8)            # [h, dt, g, r, e]
    n = len(lead)
    x = x.permute(*range(n), n + 1, n + 3, n + 0, n + 2, n + 4)   # [dt, r, h, g, e]
    return x.reshape(*lead, hd, 64).contiguous()


def _check_pages(k_pages, v_pages, dtype, nkv, hd, name):
    _need(k_pages, name + ".k_pages", dtype, (None, nkv, PAGE_TOKENS, hd))
    _need(v_pages, name + ".v_pages", dtype, (k_pages.shape[0], nkv, hd, PAGE_TOKENS))


def qk_norm_rope_kv_write(qkv, q_out, k_pages, v_pages, page_table, tok_seq, tok_pos, q_gain, k_gain, eps,
                          cos, sin, n_heads, n_kv_heads, head_dim, write_kv=True, gain_offset=0.0):
    """qkv [N, width] in the activation type, or float partial sums [S, N, width] that are added first.
    Split a fused [q | k | v] projection row into heads; RMSNorm q and k heads (if gains are
    given; the gain is gain_offset + its tensor), rotate them at tok_pos (if tables are given; their width is rotary_dim / 2), write q to
    q_out [N, nh*hd], k and v into the cache pages of sequence tok_seq[n] at position tok_pos[n]
    (not with write_kv False: a layer that reads a cache which another layer writes)."""
    nh, nkv, hd = n_heads, n_kv_heads, head_dim
    n_parts = 0
    if qkv.dim() == 3:          # float partial sums [S, N, width] of a product cut along K
        n_parts = qkv.shape[0]
        _need(qkv, "qk_norm_rope_kv_write.qkv", _F32, (n_parts, None, (nh + 2 * nkv) * hd))
        N = qkv.shape[1]
        _need(q_out, "qk_norm_rope_kv_write.q_out", (_BF16, _F32), (N, nh * hd))
    else:
        _need(qkv, "qk_norm_rope_kv_write.qkv", (_BF16, _F32), (None, (nh + 2 * nkv) * hd))
        N = qkv.shape[0]
        _need(q_out, "qk_norm_rope_kv_write.q_out", qkv.dtype, (N, nh * hd))
    _check_pages(k_pages, v_pages, q_out.dtype, nkv, hd, "qk_norm_rope_kv_write")
    _need(page_table, "qk_norm_rope_kv_write.page_table", _I32, (None, None))
    _need(tok_seq, "qk_norm_rope_kv_write.tok_seq", _I32, (N,))
    _need(tok_pos, "qk_norm_rope_kv_write.tok_pos", _I32, (N,))
    if hd > MAX_HEAD_DIM:
        raise KernelError(f"qk_norm_rope_kv_write: head size {hd} exceeds {MAX_HEAD_DIM}")
    gain_f32 = 0
    if (q_gain is None) != (k_gain is None):
        raise KernelError("qk_norm_rope_kv_write: q and k gains come together")
    if q_gain is not None:
        _need(q_gain, "qk_norm_rope_kv_write.q_gain", (_BF16, _F32), (hd,))
        _need(k_gain, "qk_norm_rope_kv_write.k_gain", q_gain.dtype, (hd,))
        gain_f32 = _is_f32(q_gain)
    rot = 0
    if cos is not None:
        _need(cos, "qk_norm_rope_kv_write.cos", _F32, (None, None))
        _need(sin, "qk_norm_rope_kv_write.sin", _F32, tuple(cos.shape))
        rot = 2 * cos.shape[1]
        if rot > hd:
            raise KernelError(f"qk_norm_rope_kv_write: rotary size {rot} exceeds head size {hd}")
    _call(load_library("core"), "syn_qk_norm_rope_kv_write", _ptr(qkv), n_parts, _ptr(q_out), _ptr(k_pages), _ptr(v_pages),
          _is_f32(q_out), _ptr(page_table), page_table.shape[1], _ptr(tok_seq), _ptr(tok_pos), _ptr(q_gain), _ptr(k_gain),
          gain_f32, ctypes.c_float(gain_offset), ctypes.c_float(eps), _ptr(cos), _ptr(sin), rot, N, nh, nkv, hd,
          1 if write_kv else 0, _stream())


def _score_terms(name, slopes, softcap, n_heads):
    """The optional terms on the scores as the entry points take them: (pointer to slopes [n_heads] float or null,
    soft cap as a C float; 0 = none).  score = cap * tanh(score / cap), then - slope[head] * (query position - key
    position); see csrc/common.h: ScoreTerms."""
    if slopes is not None:
        _need(slopes, name + ".slopes", _F32, (n_heads,))
    softcap = float(softcap or 0.0)
    if softcap < 0.0:
        raise KernelError(f"{name}: a soft cap of {softcap}")
    return _ptr(slopes), ctypes.c_float(softcap)


def attention_f32(q, k_pages, v_pages, page_table, tok_seq, tok_pos, out, scale, window, n_heads, n_kv_heads,
                  head_dim, slopes=None, softcap=0.0):
    """True 32-bit attention of every token (prefill and decode alike).  slopes, softcap: see _score_terms."""
    nh, nkv, hd = n_heads, n_kv_heads, head_dim
    _need(q, "attention_f32.q", _F32, (None, nh * hd))
    N = q.shape[0]
    _check_pages(k_pages, v_pages, _F32, nkv, hd, "attention_f32")
    _need(page_table, "attention_f32.page_table", _I32, (None, None))
    _need(tok_seq, "attention_f32.tok_seq", _I32, (N,))
    _need(tok_pos, "attention_f32.tok_pos", _I32, (N,))
    _need(out, "attention_f32.out", _F32, (N, nh * hd))
    _call(load_library("core"), "syn_attention_f32", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(page_table),
          page_table.shape[1], _ptr(tok_seq), _ptr(tok_pos), _ptr(out), ctypes.c_float(scale), int(window or 0),
          N, nh, nkv, hd, *_score_terms("attention_f32", slopes, softcap, nh), _stream())


def _attn_lib(hd):
    if hd % 16 != 0 or not (16 <= hd <= MAX_HEAD_DIM):
        raise KernelError(f"bf16 attention: head size {hd} is not one of 16, 32, ..., {MAX_HEAD_DIM}")
    return load_library(f"attn_hd{hd}")


def attention_prefill_bf16(q, k_pages, v_pages, page_table, seq_start, seq_past, out, scale, window, n_heads,
                           n_kv_heads, head_dim, variant=0, slopes=None, softcap=0.0, skip_below=0):
    """Causal attention of the new tokens of each sequence over its cache (which already holds them).
    seq_start [B+1]: offsets of the sequences' new tokens in q; seq_past [B]: tokens cached before.
    variant: 0 = the kernel's own choice, 1 = waves of 16 query rows (every head size), 2 = waves of 32
    query rows (head sizes 64 and 128); for comparisons.  slopes, softcap: see _score_terms (they take the kernel
    with waves of 16 rows).  skip_below: sequences with fewer new tokens than this are left out and their rows of
    `out` stay as they are (2: single tokens, which the caller hands to attention_decode_bf16)."""
    nh, nkv, hd = n_heads, n_kv_heads, head_dim
    _need(q, "attention_prefill.q", _BF16, (None, nh * hd))
    N = q.shape[0]
    _check_pages(k_pages, v_pages, _BF16, nkv, hd, "attention_prefill")
    _need(page_table, "attention_prefill.page_table", _I32, (None, None))
    _need(seq_start, "attention_prefill.seq_start", _I32, (None,))
    B = seq_start.shape[0] - 1
    _need(seq_past, "attention_prefill.seq_past", _I32, (B,))
    if page_table.shape[0] < B:
        raise KernelError(f"attention_prefill: page table has {page_table.shape[0]} rows for {B} sequences")
    _need(out, "attention_prefill.out", _BF16, (N, nh * hd))
    _call(_attn_lib(hd), "syn_attention_prefill_bf16", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(page_table),
          page_table.shape[1], _ptr(seq_start), _ptr(seq_past), B, N, _ptr(out), ctypes.c_float(scale),
          int(window or 0), nh, nkv, hd, int(variant), *_score_terms("attention_prefill", slopes, softcap, nh),
          int(skip_below), _stream())


def decode_splits(n_seqs, n_kv_heads, max_pages):
    """How many ways the key blocks of a sequence are split in decode.  A workgroup has up to 8
    waves that take a block each at a time; a wave that takes several blocks one after another
    pays a trip to memory for each, so the keys are split until about 2,048 waves run, but not so
    far that a split holds fewer than four blocks.  Contexts from 6K tokens on are split further,
    up to 1,024 workgroups, while a split keeps eight blocks.  One split needs no merge.
    Measured inside a graph at 1 to 32 sequences of 512 to 32K tokens (32 heads, 8 kv heads of 128):
    8 sequences of 2,100 tokens: 4 splits 19 us, 1 split 29 us, 8 splits 23 us; one sequence: 8
    splits 10.7 us, 4 splits 12.8 us; 8 sequences of 8K tokens: 16 splits 54 us, 4 splits 60 us."""
    groups = max(1, n_seqs * n_kv_heads)
    want = -(-2048 // (groups * 8))
    splits = max(1, min(want, 1 if max_pages <= 8 else max_pages // 4, 64))
    if max_pages >= 96 and groups < 256:             # (with a workgroup for every compute unit more splits only cost merging:
        more = min(64, 1024 // groups)               # 32 sequences of 8K tokens unsplit 160 us, in 4 splits 166 us)
        if more > splits and max_pages // more >= 8:
            splits = more
    return int(splits)


def _decode_work(name, counters, items, B, n_splits, n_heads, n_kv_heads):
    """The optional arguments of the decode kernels.  counters: int32, at least B * kv heads * ceil(group / 16),
    zero (the kernel leaves them zero): with them the splits are merged inside the one launch where its grid is
    small enough for that to pay.  items: int32 [4 * B * n_splits + 2 * B], the work list that hands longer
    sequences more splits (runtime.decode_items lays it out)."""
    n_items = 0
    if items is not None:
        _need(items, f"{name}.items", _I32, (4 * B * n_splits + 2 * B,))
        n_items = B * n_splits
    if counters is not None:
        chunks = -(-(n_heads // n_kv_heads) // 16)
        _need(counters, f"{name}.counters", _I32)
        if counters.numel() < B * n_kv_heads * chunks:
            raise KernelError(f"{name}: {counters.numel()} counters for {B} sequences x {n_kv_heads * chunks}")
    return _ptr(counters), _ptr(items), n_items


def attention_decode_bf16(q, k_pages, v_pages, page_table, seq_len, out, workspace, n_splits, scale, window,
                          n_heads, n_kv_heads, head_dim, slopes=None, softcap=0.0, counters=None, items=None):
    """One query for each sequence (its last token, already in the cache); seq_len [B] counts it.
    workspace: float [B * nh * n_splits * (hd + 2)].  slopes, softcap: see _score_terms; counters,
    items: see _decode_work."""
    nh, nkv, hd = n_heads, n_kv_heads, head_dim
    _need(q, "attention_decode.q", _BF16, (None, nh * hd))
    B = q.shape[0]
    _check_pages(k_pages, v_pages, _BF16, nkv, hd, "attention_decode")
    _need(page_table, "attention_decode.page_table", _I32, (None, None))
    if page_table.shape[0] < B:
        raise KernelError(f"attention_decode: page table has {page_table.shape[0]} rows for {B} sequences")
    _need(seq_len, "attention_decode.seq_len", _I32, (B,))
    _need(out, "attention_decode.out", _BF16, (B, nh * hd))
    _need(workspace, "attention_decode.workspace", _F32)
    if workspace.numel() < B * nh * n_splits * (hd + 2):
        raise KernelError(f"attention_decode: workspace of {workspace.numel()} floats is too small")
    if slopes is None and not softcap and counters is None and items is None:
        _call(_attn_lib(hd), "syn_attention_decode_bf16", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(page_table),
              page_table.shape[1], _ptr(seq_len), B, _ptr(out), _ptr(workspace), int(n_splits), ctypes.c_float(scale),
              int(window or 0), nh, nkv, hd, _stream())
        return
    _call(_attn_lib(hd), "syn_attention_decode_terms_bf16", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(page_table),
          page_table.shape[1], _ptr(seq_len), B, _ptr(out), _ptr(workspace), int(n_splits), ctypes.c_float(scale),
          int(window or 0), nh, nkv, hd, *_score_terms("attention_decode", slopes, softcap, nh),
          *_decode_work("attention_decode", counters, items, B, n_splits, nh, nkv), _stream())


def attention_decode_fused_bf16(qkv, k_pages, v_pages, page_table, seq_len, out, workspace, n_splits, scale, window,
                                n_heads, n_kv_heads, head_dim, q_gain, k_gain, eps, cos, sin, write_kv=True,
                                gain_offset=0.0, slopes=None, softcap=0.0, counters=None, items=None):
    """attention_decode_bf16 for one new token a sequence whose q, k and v come straight from the
    fused projection: qkv [B, (nh + 2 nkv) * hd] in bf16, or float partial sums [S, B, ...] that are
    added first.  The q/k RMSNorm (if gains are given), the rotation at position seq_len - 1 (if
    tables are given) and, with write_kv, the write of the new k and v into the cache pages happen
    inside the attention kernel; seq_len [B] counts the new token.  counters, items: see _decode_work."""
    nh, nkv, hd = n_heads, n_kv_heads, head_dim
    width = (nh + 2 * nkv) * hd
    n_parts = 0
    if qkv.dim() == 3:
        n_parts = qkv.shape[0]
        _need(qkv, "attention_decode_fused.qkv", _F32, (n_parts, None, width))
        B = qkv.shape[1]
    else:
        _need(qkv, "attention_decode_fused.qkv", _BF16, (None, width))
        B = qkv.shape[0]
    _check_pages(k_pages, v_pages, _BF16, nkv, hd, "attention_decode_fused")
    _need(page_table, "attention_decode_fused.page_table", _I32, (None, None))
    if page_table.shape[0] < B:
        raise KernelError(f"attention_decode_fused: page table has {page_table.shape[0]} rows for {B} sequences")
    _need(seq_len, "attention_decode_fused.seq_len", _I32, (B,))
    _need(out, "attention_decode_fused.out", _BF16, (B, nh * hd))
    _need(workspace, "attention_decode_fused.workspace", _F32)
    if workspace.numel() < B * nh * n_splits * (hd + 2):
        raise KernelError(f"attention_decode_fused: workspace of {workspace.numel()} floats is too small")
    gain_f32 = 0
    if (q_gain is None) != (k_gain is None):
        raise KernelError("attention_decode_fused: q and k gains come together")
    if q_gain is not None:
        _need(q_gain, "attention_decode_fused.q_gain", (_BF16, _F32), (hd,))
        _need(k_gain, "attention_decode_fused.k_gain", q_gain.dtype, (hd,))
        gain_f32 = _is_f32(q_gain)
    rot = 0
    if cos is not None:
        _need(cos, "attention_decode_fused.cos", _F32, (None, None))
        _need(sin, "attention_decode_fused.sin", _F32, tuple(cos.shape))
        rot = 2 * cos.shape[1]
        if rot > hd:
            raise KernelError(f"attention_decode_fused: rotary size {rot} exceeds head size {hd}")
    _call(_attn_lib(hd), "syn_attention_decode_fused_bf16", _ptr(qkv), n_parts, _ptr(k_pages), _ptr(v_pages),
          _ptr(page_table), page_table.shape[1], _ptr(seq_len), B, _ptr(out), _ptr(workspace), int(n_splits),
          ctypes.c_float(scale), int(window or 0), nh, nkv, hd, _ptr(q_gain), _ptr(k_gain), gain_f32,
          ctypes.c_float(gain_offset), ctypes.c_float(eps), _ptr(cos), _ptr(sin), rot, 1 if write_kv else 0,
          *_score_terms("attention_decode_fused", slopes, softcap, nh),
          *_decode_work("attention_decode_fused", counters, items, B, n_splits, nh, nkv), _stream())


# ----------------------------------------------------------------------------- residual streams, dynamic tanh

ROWNORM_NONE, ROWNORM_DYT = 0, 1
STREAMS_MAX = 16


def _streams(X, name):
    """X as [N, S, W]: a plain residual [N, W] counts as one stream."""
    _need(X, name, _F32)
    if X.dim() == 2:
        return X.shape[0], 1, X.shape[1]
    if X.dim() != 3 or not (1 <= X.shape[1] <= STREAMS_MAX):
        raise KernelError(f"{name}: shape {list(X.shape)}, expected [N, W] or [N, S, W] with up to {STREAMS_MAX} streams")
    return tuple(X.shape)


def streams_read_norm(X, in_w, out, dyt=None, rows=None, delta=None):
    """out[i] = norm(sum_s in_w[s] X[row, s] (+ delta[row])), row = rows[i] or i.  X [N, S, W] float (or [N, W]);
    in_w float [S] or None (every weight 1: the sum of the streams); dyt = (alpha [1], gain [W], shift [W]) float:
    tanh(alpha u) gain + shift, None: u itself; delta [N, W] or partial sums [P, N, W] float, with one stream only
    (without rows it is added into X as well); out [n, W] bf16 or float."""
    N, S, W = _streams(X, "streams_read_norm.X")
    if in_w is not None:
        _need(in_w, "streams_read_norm.in_w", _F32, (S,))
    n_out = N
    if rows is not None:
        _need(rows, "streams_read_norm.rows", _I32, (None,))
        n_out = rows.shape[0]
    n_parts = 0
    if delta is not None:
        if S != 1:
            raise KernelError("streams_read_norm: a delta comes with one stream")
        n_parts = delta.shape[0] if delta.dim() == 3 else 1
        _need(delta, "streams_read_norm.delta", _F32, (n_parts, N, W) if delta.dim() == 3 else (N, W))
    alpha = gain = shift = None
    if dyt is not None:
        alpha, gain, shift = dyt
        _need(alpha, "streams_read_norm.alpha", _F32)
        _need(gain, "streams_read_norm.gain", _F32, (W,))
        _need(shift, "streams_read_norm.shift", _F32, (W,))
        if alpha.numel() != 1:
            raise KernelError("streams_read_norm: alpha is one number")
    _need(out, "streams_read_norm.out", (_BF16, _F32), (n_out, W))
    _call(load_library("core"), "syn_streams_read_norm", _ptr(X), _ptr(delta), n_parts, N, _ptr(rows), n_out, _ptr(in_w),
          S, W, ROWNORM_NONE if dyt is None else ROWNORM_DYT, _ptr(alpha), _ptr(gain), _ptr(shift), _ptr(out),
          _is_f32(out), _stream())


def streams_update(X, mix, out_w, terms, read=None):
    """X[n, t] = sum_s mix[s, t] X[n, s] + out_w[t] y[n] in place, all streams from the old ones;
    y = sum over `terms` of scale * (sum of the term's partial sums + bias).  terms: one or two (tensor [N, W] or
    [P, N, W] float, scale, bias [W] float or None).
    read = (in_w [S] float, dyt or None, out [N, W] bf16 or float): what the next sublayer reads leaves in the same
    pass, out[n] = norm(sum_t in_w[t] X'[n, t]) with dyt as in streams_read_norm."""
    N, S, W = _streams(X, "streams_update.X")
    _need(mix, "streams_update.mix", _F32, (S, S))
    _need(out_w, "streams_update.out_w", _F32, (S,))
    if not (1 <= len(terms) <= 2):
        raise KernelError(f"streams_update: {len(terms)} terms (one or two)")
    args = []
    for y, scale, bias in list(terms) + [(None, 0.0, None)] * (2 - len(terms)):
        parts = 0
        if y is not None:
            parts = y.shape[0] if y.dim() == 3 else 1
            _need(y, "streams_update.y", _F32, (parts, N, W) if y.dim() == 3 else (N, W))
            if bias is not None:
                _need(bias, "streams_update.bias", _F32, (W,))
        args += [_ptr(y), parts, ctypes.c_float(scale), _ptr(bias)]
    nxt = [_ptr(None), ROWNORM_NONE, _ptr(None), _ptr(None), _ptr(None), _ptr(None), 0]
    if read is not None:
        in_w, dyt, out = read
        _need(in_w, "streams_update.read.in_w", _F32, (S,))
        _need(out, "streams_update.read.out", (_BF16, _F32), (N, W))
        alpha = gain = shift = None
        if dyt is not None:
            alpha, gain, shift = dyt
            _need(alpha, "streams_update.read.alpha", _F32)
            _need(gain, "streams_update.read.gain", _F32, (W,))
            _need(shift, "streams_update.read.shift", _F32, (W,))
        nxt = [_ptr(in_w), ROWNORM_NONE if dyt is None else ROWNORM_DYT, _ptr(alpha), _ptr(gain), _ptr(shift), _ptr(out),
               _is_f32(out)]
    _call(load_library("core"), "syn_streams_update", _ptr(X), N, S, W, _ptr(mix), _ptr(out_w), *args, *nxt, _stream())


def streams_start(x, X):
    """X[n, s] = x[n] for every stream: x [N, W] float, X [N, S, W] float."""
    _need(x, "streams_start.x", _F32, (None, None))
    N, W = x.shape
    _need(X, "streams_start.X", _F32, (N, None, W))
    _call(load_library("core"), "syn_streams_start", _ptr(x), _ptr(X), N, X.shape[1], W, _stream())


# ----------------------------------------------------------------------------- attention with terms, a kept window, a sink

WINDOW_ATTENTION_MAX_DIM = 640


def _check_window_pages(k_pages, v_pages, dtype, nkv, dim, vdim, name, v_share=1):
    if v_share < 1 or nkv % v_share:
        raise KernelError(f"{name}: {nkv} kv heads in shares of {v_share} value heads")
    _need(k_pages, name + ".k_pages", dtype, (None, nkv, PAGE_TOKENS, dim))
    _need(v_pages, name + ".v_pages", dtype, (k_pages.shape[0], nkv // v_share, vdim, PAGE_TOKENS))


def window_intake(proj, bias, q_out, k_pages, v_pages, page_table, tok_seq, tok_pos, q_gain, k_gain, eps,
                  n_heads, n_kv_heads, dim, vdim, write_kv=True, rotation=None, v_share=1, pairs=False):
    """proj [N, width] float: the fused projection [q | k | v | ...]; bias float [>= q, k, v columns] or None.  q and k
    heads get their bias and (with gains, float [dim]) an RMSNorm over the head; q goes to q_out [N, nh * dim], k and v
    (with its bias) into the pages of sequence tok_seq[n] at position tok_pos[n].
    rotation = (cos, sin) float [positions, rot / 2]: the first `rot` values of every q and k head are then turned by
    the angles of the token's position, value i paired with value i + rot / 2 (the caller sees to it that the tables
    reach the step's last position); with `pairs` value 2 i is paired with value 2 i + 1.  v_share: there are
    nkv / v_share value heads (and rows of v in proj).  write_kv False: the pages are another layer's and are left
    alone; proj and bias then need to hold the queries only."""
    nh, nkv = n_heads, n_kv_heads
    _need(proj, "window_intake.proj", _F32, (None, None))
    N, width = proj.shape
    if v_share < 1 or nkv % v_share:
        raise KernelError(f"window_intake: {nkv} kv heads in shares of {v_share} value heads")
    nv = nkv // v_share
    used = (nh + nkv) * dim + nv * vdim if write_kv else nh * dim
    if width < used:
        raise KernelError(f"window_intake: rows of {width} values do not hold {'q, k and v' if write_kv else 'q'} ({used})")
    if bias is not None:
        _need(bias, "window_intake.bias", _F32, (None,))
        if bias.shape[0] < used:
            raise KernelError(f"window_intake: a bias of {bias.shape[0]} values for {used} columns")
    _need(q_out, "window_intake.q_out", (_BF16, _F32), (N, nh * dim))
    _check_window_pages(k_pages, v_pages, q_out.dtype, nkv, dim, vdim, "window_intake", v_share)
    _need(page_table, "window_intake.page_table", _I32, (None, None))
    cos = sin = None
    rot = 0
    if rotation is not None and rotation[0] is not None:
        cos, sin = rotation
        _need(cos, "window_intake.cos", _F32, (None, None))
        _need(sin, "window_intake.sin", _F32, tuple(cos.shape))
        rot = 2 * cos.shape[1]
        if rot > dim:
            raise KernelError(f"window_intake: a rotation of {rot} values of heads of {dim}")
    _need(tok_seq, "window_intake.tok_seq", _I32, (N,))
    _need(tok_pos, "window_intake.tok_pos", _I32, (N,))
    if (q_gain is None) != (k_gain is None):
        raise KernelError("window_intake: q and k gains come together")
    if q_gain is not None:
        _need(q_gain, "window_intake.q_gain", _F32, (dim,))
        _need(k_gain, "window_intake.k_gain", _F32, (dim,))
    _call(load_library("core"), "syn_window_intake", _ptr(proj), width, _ptr(bias), _ptr(q_out), _ptr(k_pages),
          _ptr(v_pages), _is_f32(q_out), _ptr(page_table), page_table.shape[1], _ptr(tok_seq), _ptr(tok_pos),
          _ptr(q_gain), _ptr(k_gain), ctypes.c_float(eps), _ptr(cos), _ptr(sin), rot, 1 if pairs else 0, N, nh, nkv, nv,
          dim, vdim, 1 if write_kv else 0, _stream())


def window_attention(q, k_pages, v_pages, page_table, tok_seq, tok_pos, out, scale, n_heads, n_kv_heads, dim, vdim,
                     window=0, keep_first=0, sink_one=False, slopes=None, log_bias=None, softcap=0.0, gate=None,
                     gate_bias=None, v_share=1, sinks=None, chunk=0, gate_per_head=False):
    """v_share: that many neighbouring kv heads read the values of one value head (v_pages holds nkv / v_share heads).
    Attention of every token (prompts and single tokens alike) whose query is q [N, nh * dim] over the pages
    (which already hold the tokens): score = scale q.k [soft cap] - slopes[h] (i - j) - r1[h] ln(1 + r2[h] (i - j))
    with log_bias = (r1, r2) float [nh]; key j is seen by i iff j <= i and (no window or i - j < window or
    j < keep_first) and (no chunk or j // chunk == i // chunk or j < keep_first); sink_one: one more in the softmax's
    denominator; sinks float [nh]: exp(sinks[h]) more (a learned score of a key without a value); gate: a float view
    [N, >= nh * vdim] (with gate_per_head [N, >= nh]: one number a head) with row stride gate.stride(0) whose sigmoid
    multiplies the result; out [N, nh * vdim] in q's type."""
    nh, nkv = n_heads, n_kv_heads
    _need(q, "window_attention.q", (_BF16, _F32), (None, nh * dim))
    N = q.shape[0]
    _check_window_pages(k_pages, v_pages, q.dtype, nkv, dim, vdim, "window_attention", v_share)
    _need(page_table, "window_attention.page_table", _I32, (None, None))
    _need(tok_seq, "window_attention.tok_seq", _I32, (N,))
    _need(tok_pos, "window_attention.tok_pos", _I32, (N,))
    _need(out, "window_attention.out", q.dtype, (N, nh * vdim))
    if max(dim, vdim) > WINDOW_ATTENTION_MAX_DIM:
        raise KernelError(f"window_attention: head sizes {dim}, {vdim} exceed {WINDOW_ATTENTION_MAX_DIM}")
    r1 = r2 = None
    if log_bias is not None:
        r1, r2 = log_bias
        _need(r1, "window_attention.r1", _F32, (nh,))
        _need(r2, "window_attention.r2", _F32, (nh,))
    if slopes is not None:
        _need(slopes, "window_attention.slopes", _F32, (nh,))
    gate_stride = 0
    n_gate = nh if gate_per_head else nh * vdim
    if gate is not None:
        gate_stride = _float_rows_view(gate, "window_attention.gate", N, n_gate)
        if gate_bias is not None:
            _need(gate_bias, "window_attention.gate_bias", _F32, (n_gate,))
    _sink_and_chunk("window_attention", sinks, sink_one, chunk, nh)
    _call(load_library("core"), "syn_window_attention", _ptr(q), _ptr(k_pages), _ptr(v_pages), _is_f32(q),
          _ptr(page_table), page_table.shape[1], _ptr(tok_seq), _ptr(tok_pos), _ptr(gate), gate_stride,
          _ptr(gate_bias if gate is not None else None), _ptr(out), ctypes.c_float(scale), N, nh, nkv, dim, vdim,
          _ptr(slopes), _ptr(r1), _ptr(r2), ctypes.c_float(float(softcap or 0.0)), int(window or 0), int(keep_first or 0),
          1 if sink_one else 0, int(v_share), _ptr(sinks), int(chunk or 0), 1 if gate_per_head else 0, _stream())


def _sink_and_chunk(name, sinks, sink_one, chunk, n_heads):
    if sinks is not None:
        _need(sinks, name + ".sinks", _F32, (n_heads,))
        if sink_one:
            raise KernelError(f"{name}: a learned sink and a sink of one together")
    if chunk is not None and chunk < 0:
        raise KernelError(f"{name}: chunks of {chunk} positions")


WINDOW_PREFILL_MAX_DIM = 128


def window_prefill_takes(dim, vdim) -> bool:
    """Whether the bf16 prompt kernel on the matrix cores takes these head sizes (multiples of 16 up to 128)."""
    return dim % 16 == 0 and vdim % 16 == 0 and 16 <= dim <= WINDOW_PREFILL_MAX_DIM and 16 <= vdim <= WINDOW_PREFILL_MAX_DIM


def window_attention_prefill_bf16(q, k_pages, v_pages, page_table, seq_start, seq_past, out, scale, n_heads, n_kv_heads,
                                  dim, vdim, window=0, keep_first=0, sink_one=False, slopes=None, log_bias=None,
                                  softcap=0.0, gate=None, gate_bias=None, v_share=1, sinks=None, chunk=0,
                                  gate_per_head=False):
    """window_attention for the new tokens of each sequence of a step in bf16, on the matrix cores: seq_start [B + 1]
    offsets of the sequences' new tokens in q, seq_past [B] tokens cached before (the pages already hold the new
    ones).  Scores and weights are 32-bit; a weight meets V as two bf16 numbers (16 bits of mantissa)."""
    nh, nkv = n_heads, n_kv_heads
    if not window_prefill_takes(dim, vdim):
        raise KernelError(f"window_attention_prefill: head sizes {dim} and {vdim} (multiples of 16 up to {WINDOW_PREFILL_MAX_DIM})")
    _need(q, "window_attention_prefill.q", _BF16, (None, nh * dim))
    N = q.shape[0]
    _check_window_pages(k_pages, v_pages, _BF16, nkv, dim, vdim, "window_attention_prefill", v_share)
    _need(page_table, "window_attention_prefill.page_table", _I32, (None, None))
    _need(seq_start, "window_attention_prefill.seq_start", _I32, (None,))
    B = seq_start.shape[0] - 1
    _need(seq_past, "window_attention_prefill.seq_past", _I32, (B,))
    if page_table.shape[0] < B:
        raise KernelError(f"window_attention_prefill: page table has {page_table.shape[0]} rows for {B} sequences")
    _need(out, "window_attention_prefill.out", _BF16, (N, nh * vdim))
    r1 = r2 = None
    if log_bias is not None:
        r1, r2 = log_bias
        _need(r1, "window_attention_prefill.r1", _F32, (nh,))
        _need(r2, "window_attention_prefill.r2", _F32, (nh,))
    if slopes is not None:
        _need(slopes, "window_attention_prefill.slopes", _F32, (nh,))
    gate_stride = 0
    n_gate = nh if gate_per_head else nh * vdim
    if gate is not None:
        gate_stride = _float_rows_view(gate, "window_attention_prefill.gate", N, n_gate)
        if gate_bias is not None:
            _need(gate_bias, "window_attention_prefill.gate_bias", _F32, (n_gate,))
    _sink_and_chunk("window_attention_prefill", sinks, sink_one, chunk, nh)
    _call(load_library("core"), "syn_window_attention_prefill_bf16", _ptr(q), _ptr(k_pages), _ptr(v_pages),
          _ptr(page_table), page_table.shape[1], _ptr(seq_start), _ptr(seq_past), B, N, _ptr(gate), gate_stride,
          _ptr(gate_bias if gate is not None else None), _ptr(out), ctypes.c_float(scale), nh, nkv, dim, vdim,
          _ptr(slopes), _ptr(r1), _ptr(r2), ctypes.c_float(float(softcap or 0.0)), int(window or 0), int(keep_first or 0),
          1 if sink_one else 0, int(v_share), _ptr(sinks), int(chunk or 0), 1 if gate_per_head else 0, _stream())


def _float_rows_view(t, name, n_rows, n_cols):
    """A float tensor [n_rows, >= n_cols] whose rows may be pieces of longer rows (columns of a fused projection):
    returns the row stride in elements."""
    if not isinstance(t, torch.Tensor) or t.dtype != _F32 or not t.is_cuda or t.dim() != 2:
        raise KernelError(f"{name}: expected a float matrix on the GPU")
    if t.shape[0] != n_rows or t.shape[1] < n_cols or t.stride(1) != 1 or t.stride(0) < t.shape[1]:
        raise KernelError(f"{name}: shape {list(t.shape)} with strides {list(t.stride())}, expected [{n_rows}, >= {n_cols}] rows")
    return t.stride(0)


# ----------------------------------------------------------------------------- matrix memory

MATRIX_MEMORY_MAX_DIM = 256


def matrix_memory_state_size(dim, vdim) -> int:
    """Floats of a (slot, head)'s state: S [dim, vdim] by rows, n [dim], m."""
    return dim * vdim + dim + 1


def matrix_memory_scan(proj, i_bias, f_bias, gate_cap, q_scale, state, seq_start, seq_slot, out, n_heads, dim, vdim,
                       chunked=False, scratch=None):
    """The cell of csrc/matrix_memory.hip over the new tokens of every sequence of the step, in order, from and into
    state [rows, H, dim * vdim + dim + 1] float (row = seq_slot[b]; a negative slot takes the last row).
    proj [N, width] float: [q | k | v | gate | i | f] of the fused projection; out [N, H * vdim] float.
    chunked: 32 tokens at a time (prompts) instead of token by token (single tokens); the same sums in another order.
    scratch: with chunked, a function (name, floats) -> float tensor for the chunks' partial states (StepContext.scratch;
    default: a new tensor)."""
    H = n_heads
    _need(proj, "matrix_memory_scan.proj", _F32, (None, None))
    N, width = proj.shape
    if width < 2 * H * dim + 2 * H * vdim + 2 * H:
        raise KernelError(f"matrix_memory_scan: rows of {width} values are too short")
    if dim > MATRIX_MEMORY_MAX_DIM:
        raise KernelError(f"matrix_memory_scan: keys of {dim} values (at most {MATRIX_MEMORY_MAX_DIM})")
    for name, t in (("i_bias", i_bias), ("f_bias", f_bias)):
        if t is not None:
            _need(t, f"matrix_memory_scan.{name}", _F32, (H,))
    _need(state, "matrix_memory_scan.state", _F32, (None, H, matrix_memory_state_size(dim, vdim)))
    _need(seq_start, "matrix_memory_scan.seq_start", _I32, (None,))
    B = seq_start.shape[0] - 1
    _need(seq_slot, "matrix_memory_scan.seq_slot", _I32, (B,))
    _need(out, "matrix_memory_scan.out", _F32, (N, H * vdim))
    lib = load_library("core")
    work = None
    if chunked:
        lib.syn_matrix_memory_chunk_scratch.restype = ctypes.c_long
        need = lib.syn_matrix_memory_chunk_scratch(N, B, H, dim, vdim)
        work = scratch("matrix_memory_chunks", need) if scratch is not None else torch.empty(need, dtype=_F32, device=proj.device)
        _need(work, "matrix_memory_scan.scratch", _F32)
        if work.numel() < need:
            raise KernelError(f"matrix_memory_scan: scratch of {work.numel()} floats, {need} are needed")
    _call(lib, "syn_matrix_memory_scan", _ptr(proj), width, _ptr(i_bias), _ptr(f_bias),
          ctypes.c_float(float(gate_cap or 0.0)), ctypes.c_float(q_scale), _ptr(state), state.shape[0], _ptr(seq_start),
          _ptr(seq_slot), B, _ptr(out), H, dim, vdim, 1 if chunked else 0, N, _ptr(work), _stream())


def head_norm_gate(o, gain, eps, gate, out, n_heads, vdim, silu_first=False):
    """out[n, h] = o[n, h] / rms(o[n, h]) * gain[h] * sigmoid(gate[n, h]): o [N, H * vdim] float, gain float [H * vdim]
    or None, gate a float view [N, >= H * vdim] (see _float_rows_view) or None, out [N, H * vdim] bf16 or float.
    silu_first: the gate comes before the norm, x = o * silu(gate), out = x / rms(x) * gain."""
    _need(o, "head_norm_gate.o", _F32, (None, n_heads * vdim))
    N = o.shape[0]
    if gain is not None:
        _need(gain, "head_norm_gate.gain", _F32, (n_heads * vdim,))
    stride = _float_rows_view(gate, "head_norm_gate.gate", N, n_heads * vdim) if gate is not None else 0
    _need(out, "head_norm_gate.out", (_BF16, _F32), (N, n_heads * vdim))
    _call(load_library("core"), "syn_head_norm_gate", _ptr(o), _ptr(gain), ctypes.c_float(eps), _ptr(gate), stride,
          _ptr(out), _is_f32(out), N, n_heads, vdim, 1 if silu_first else 0, _stream())


# ----------------------------------------------------------------------------- short convolutions and scans over a state

SHORT_CONV_MAX_TAPS = 16
SCAN_MAX_ROWS = 256       # rows of a head's state: the state space's N, the delta rule's key size


def _step_seqs(name, seq_start, seq_slot):
    _need(seq_start, name + ".seq_start", _I32, (None,))
    B = seq_start.shape[0] - 1
    _need(seq_slot, name + ".seq_slot", _I32, (B,))
    return B


def short_conv(u, weight, bias, state, tok_seq, tok_pos, seq_start, seq_past, seq_slot, out, silu=False):
    """A causal convolution over each sequence's own tokens, one filter a channel:
    out[t, c] = act(bias[c] + sum_j weight[c, j] u[t - taps + 1 + j, c]), zeros before a sequence's first token.
    u: a float view [N, C] whose rows may be pieces of longer rows (columns of a fused projection); weight float
    [C, taps]; bias float [C] or None; state float [rows, taps - 1, C]: the last taps - 1 inputs of the sequence in row
    seq_slot[b] (a negative slot: the last row), read for the tokens before this step and written for the next one;
    out float [N, C].  Every sequence of the step brings at least one token (with as many tokens as sequences, one each:
    output and state then take one launch)."""
    _need(weight, "short_conv.weight", _F32, (None, None))
    C, taps = weight.shape
    N = tok_seq.shape[0]
    stride = _float_rows_view(u, "short_conv.u", N, C)
    if not 1 <= taps <= SHORT_CONV_MAX_TAPS:
        raise KernelError(f"short_conv: {taps} taps (1 to {SHORT_CONV_MAX_TAPS})")
    if bias is not None:
        _need(bias, "short_conv.bias", _F32, (C,))
    _need(state, "short_conv.state", _F32, (None, max(taps - 1, 0), C))
    _need(tok_seq, "short_conv.tok_seq", _I32, (N,))
    _need(tok_pos, "short_conv.tok_pos", _I32, (N,))
    B = _step_seqs("short_conv", seq_start, seq_slot)
    _need(seq_past, "short_conv.seq_past", _I32, (B,))
    _need(out, "short_conv.out", _F32, (N, C))
    _call(load_library("core"), "syn_short_conv", _ptr(u), stride, _ptr(weight), _ptr(bias), 1 if silu else 0, _ptr(state),
          state.shape[0], _ptr(tok_seq), _ptr(tok_pos), _ptr(seq_start), _ptr(seq_past), _ptr(seq_slot), _ptr(out), N, B, C,
          taps, _stream())


def state_space_scan(xbc, dt, dt_bias, a_log, d_skip, state, seq_start, seq_slot, out, n_heads, vdim, n_state, n_groups,
                     single_tokens=False):
    """The state space with a scalar decay a head over the new tokens of every sequence of the step, in order:
        step = softplus(dt + dt_bias[h]);  S <- exp(-exp(a_log[h]) step) S + step B x^T;  y = S^T C + d_skip[h] x
    xbc float [N, H * vdim + 2 G * n_state]: x, B and C (head h reads group h // (H / G)); dt a float view [N, >= H];
    state float [rows, H, n_state, vdim] (row seq_slot[b]; a negative slot: the last row); out float [N, H * vdim].
    single_tokens: every sequence brings one token (the kernel is then laid out for moving the state, not for a chain of
    tokens; the results are the same)."""
    H, G = n_heads, n_groups
    if G <= 0 or H % G:
        raise KernelError(f"state_space_scan: {H} heads do not divide into {G} groups")
    if n_state > SCAN_MAX_ROWS:
        raise KernelError(f"state_space_scan: a state of {n_state} rows (at most {SCAN_MAX_ROWS})")
    _need(xbc, "state_space_scan.xbc", _F32, (None, H * vdim + 2 * G * n_state))
    N = xbc.shape[0]
    stride = _float_rows_view(dt, "state_space_scan.dt", N, H)
    for name, t in (("dt_bias", dt_bias), ("a_log", a_log), ("d_skip", d_skip)):
        _need(t, f"state_space_scan.{name}", _F32, (H,))
    _need(state, "state_space_scan.state", _F32, (None, H, n_state, vdim))
    B = _step_seqs("state_space_scan", seq_start, seq_slot)
    _need(out, "state_space_scan.out", _F32, (N, H * vdim))
    _call(load_library("core"), "syn_state_space_scan", _ptr(xbc), _ptr(dt), stride, _ptr(dt_bias), _ptr(a_log),
          _ptr(d_skip), _ptr(state), state.shape[0], _ptr(seq_start), _ptr(seq_slot), B, 1 if single_tokens else max(N, 2),
          _ptr(out), H, vdim, n_state, G, _stream())


def channel_delta_scan(qkv, beta, a, a_bias, a_log, q_scale, unit_eps, state, seq_start, seq_slot, out, n_heads,
                       n_key_heads, dim, vdim, single_tokens=False):
    """The delta rule with a decay for every key channel over the new tokens of every sequence of the step, in order.
    With q and k made unit vectors (x / sqrt(sum x^2 + unit_eps); q also times q_scale), b = sigmoid(beta) and
    g = exp(-exp(a_log[h]) softplus(a + a_bias)) for each (head, key channel):
        S <- diag(g) S;  u = b (v - S^T k);  S <- S + k u^T;  o = S^T q
    qkv float [N, 2 K * dim + H * vdim]: q and k of the K key heads (head h reads key head h // (H / K)), v; beta a
    float view [N, >= H]; a a float view [N, >= H * dim]; a_bias float [H * dim]; a_log float [H]; state float
    [rows, H, dim, vdim] (row seq_slot[b]; a negative slot: the last row); out float [N, H * vdim].
    single_tokens: as for state_space_scan."""
    H, K = n_heads, n_key_heads
    if K <= 0 or H % K:
        raise KernelError(f"channel_delta_scan: {H} heads do not divide into {K} key heads")
    if dim > SCAN_MAX_ROWS:
        raise KernelError(f"channel_delta_scan: keys of {dim} values (at most {SCAN_MAX_ROWS})")
    _need(qkv, "channel_delta_scan.qkv", _F32, (None, 2 * K * dim + H * vdim))
    N = qkv.shape[0]
    stride = _float_rows_view(beta, "channel_delta_scan.beta", N, H)
    a_stride = _float_rows_view(a, "channel_delta_scan.a", N, H * dim)
    _need(a_bias, "channel_delta_scan.a_bias", _F32, (H * dim,))
    _need(a_log, "channel_delta_scan.a_log", _F32, (H,))
    _need(state, "channel_delta_scan.state", _F32, (None, H, dim, vdim))
    B = _step_seqs("channel_delta_scan", seq_start, seq_slot)
    _need(out, "channel_delta_scan.out", _F32, (N, H * vdim))
    _call(load_library("core"), "syn_channel_delta_scan", _ptr(qkv), _ptr(beta), stride, _ptr(a), a_stride, _ptr(a_bias),
          _ptr(a_log),
          ctypes.c_float(q_scale), ctypes.c_float(unit_eps), _ptr(state), state.shape[0], _ptr(seq_start), _ptr(seq_slot), B,
          1 if single_tokens else max(N, 2), _ptr(out), H, K, dim, vdim, _stream())


def diff_heads(a, out, lam, eps, post, n_kv_heads, heads_per_kv, vdim):
    """Two softmax maps over the same values joined: a [N, G * 2 * R * vdim] holds, for each of the G kv heads, the R
    heads' results of the first map and then of the second; out [N, G * R * vdim] = rms_norm(a1 - lam a2) * post for
    each head (the norm over the head's vdim values, eps inside the root, no gain)."""
    G, R = n_kv_heads, heads_per_kv
    _need(a, "diff_heads.a", (_BF16, _F32), (None, G * 2 * R * vdim))
    N = a.shape[0]
    _need(out, "diff_heads.out", a.dtype, (N, G * R * vdim))
    _call(load_library("core"), "syn_diff_heads", _ptr(a), _ptr(out), _is_f32(a), ctypes.c_float(lam), ctypes.c_float(eps),
          ctypes.c_float(post), N, G, R, vdim, _stream())


# ----------------------------------------------------------------------------- sampling

def sample_rows(logits, temperature, uniform, out):
    """out[r] = argmax (last of equal maxima) where temperature[r] <= 0 or temperature is None,
    else a draw from softmax(logits[r] / temperature[r]) by inverse CDF with uniform[r]."""
    _need(logits, "sample_rows.logits", _F32, (None, None))
    R, V = logits.shape
    if temperature is not None:
        _need(temperature, "sample_rows.temperature", _F32, (R,))
        _need(uniform, "sample_rows.uniform", _F32, (R,))
    _need(out, "sample_rows.out", _I32, (R,))
    _call(load_library("core"), "syn_sample_rows", _ptr(logits), _ptr(temperature),
          _ptr(uniform if temperature is not None else None), _ptr(out), R, V, _stream())


def filter_rows(logits, out, temperature, top_k, top_p, min_p, repetition, presence, frequency,
                ids=None, id_start=None, counts=None):
    """The processors in front of the sampler, one workgroup a row of logits [R, V] (float): repetition penalty,
    presence / frequency penalty, temperature, top-k, top-p, min-p, in this order; what is dropped becomes -inf
    in `out` (which may be `logits`).  Every option is an array with one entry a row: temperature (<= 0 or 1:
    the row is not divided), top_k (int32; 0: off), top_p (>= 1: off), min_p (0: off), repetition (1: off),
    presence, frequency (0: off).  ids (int32, flat) and id_start (int32 [R + 1]) give each row the tokens that
    the penalties look at; counts (int32 [R * V], zero) is their scratch memory, left zero."""
    _need(logits, "filter_rows.logits", _F32, (None, None))
    R, V = logits.shape
    _need(out, "filter_rows.out", _F32, (R, V))
    for name, t, dt in (("temperature", temperature, _F32), ("top_k", top_k, _I32), ("top_p", top_p, _F32),
                        ("min_p", min_p, _F32), ("repetition", repetition, _F32), ("presence", presence, _F32),
                        ("frequency", frequency, _F32)):
        _need(t, f"filter_rows.{name}", dt, (R,))
    if (ids is None) != (id_start is None):
        raise KernelError("filter_rows: ids and id_start come together")
    if ids is not None:
        _need(ids, "filter_rows.ids", _I32, (None,))
        _need(id_start, "filter_rows.id_start", _I32, (R + 1,))
        _need(counts, "filter_rows.counts", _I32)
        if counts.numel() < R * V:
            raise KernelError(f"filter_rows: {counts.numel()} counters for {R} rows of {V}")
    _call(load_library("core"), "syn_filter_rows", _ptr(logits), _ptr(out), R, V, _ptr(temperature), _ptr(top_k),
          _ptr(top_p), _ptr(min_p), _ptr(repetition), _ptr(presence), _ptr(frequency), _ptr(ids), _ptr(id_start),
          _ptr(counts), _stream())


# ----------------------------------------------------------------------------- what the machine gives

def measure_ceilings(device="cuda:0", read_bytes=1 << 30, repeats=5):
    """(memory read rate in GB/s, bf16 MFMA rate in TFLOP/s) of kernels that do nothing else: the
    best of `repeats` passes over a buffer of read_bytes, and of a launch that keeps every matrix
    unit busy from registers.  Measurements, to stand beside the vendor's peaks."""
    lib = load_library("core")
    buf = torch.empty(read_bytes // 4, dtype=torch.int32, device=device).zero_()
    sink = torch.zeros(4, dtype=torch.int32, device=device)
    fsink = torch.zeros(4, dtype=torch.float32, device=device)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def best(launch):
        launch()
        torch.cuda.synchronize()
        times = []
        for _ in range(repeats):
            start.record()
            launch()
            end.record()
            end.synchronize()
            times.append(start.elapsed_time(end) * 1e-3)
        return min(times)

    t_read = best(lambda: _call(lib, "syn_probe_read", _ptr(buf), ctypes.c_size_t(buf.numel() * 4), _ptr(sink), _stream()))
    groups, iters = 256 * 8, 4096
    t_mfma = best(lambda: _call(lib, "syn_probe_mfma", groups, iters, _ptr(fsink), _stream()))
    flops = groups * 4 * iters * 4 * 2 * 32 * 32 * 16
    return buf.numel() * 4 / t_read / 1e9, flops / t_mfma / 1e12


# ----------------------------------------------------------------------------- scaled residual terms

def add_scaled_rmsnorm(resid, terms, gain, eps, out, rows=None):
    """resid += sum_t scale_t * delta_t for up to two terms (delta float [N, H] or partial sums [S, N, H], scale float
    [H] or None), then out = RMSNorm(resid) * gain when `out` is given.  rows [n] int32: only those rows are summed and
    normed, resid is not written.  A term may be a triple (delta, scale, row_gate): row_gate a float view [N, 1] (a
    column of longer rows) whose sigmoid multiplies the term's rows."""
    _need(resid, "add_scaled_rmsnorm.resid", _F32, (None, None))
    N, H = resid.shape
    if not 1 <= len(terms) <= 2:
        raise KernelError(f"add_scaled_rmsnorm: {len(terms)} terms (one or two)")
    args, gates = [], []
    for i, term in enumerate(terms):
        d, s = term[0], term[1]
        g = term[2] if len(term) > 2 else None
        parts = d.shape[0] if d.dim() == 3 else 1
        _need(d, f"add_scaled_rmsnorm.delta{i}", _F32, (parts, N, H) if d.dim() == 3 else (N, H))
        if s is not None:
            _need(s, f"add_scaled_rmsnorm.scale{i}", _F32, (H,))
        args += [_ptr(d), parts, _ptr(s)]
        gates += [_ptr(g), 0 if g is None else _float_rows_view(g, f"add_scaled_rmsnorm.row_gate{i}", N, 1)]
    if len(terms) == 1:
        args += [_ptr(None), 1, _ptr(None)]
        gates += [_ptr(None), 0]
    n_out = N
    if rows is not None:
        _need(rows, "add_scaled_rmsnorm.rows", _I32, (None,))
        n_out = rows.shape[0]
    if out is not None:
        _need(gain, "add_scaled_rmsnorm.gain", (_BF16, _F32), (H,))
        _need(out, "add_scaled_rmsnorm.out", (_BF16, _F32), (n_out, H))
    elif rows is not None:
        raise KernelError("add_scaled_rmsnorm: gathered rows without an output")
    _call(load_library("core"), "syn_add_scaled_rmsnorm", _ptr(resid), N, _ptr(rows), n_out, *args, *gates, _ptr(gain),
          0 if gain is None else _is_f32(gain), ctypes.c_float(eps), _ptr(out), 0 if out is None else _is_f32(out), H,
          _stream())


# ----------------------------------------------------------------------------- products by group (experts, heads)

def _grouped(name, a, lda, a_group, w, w_group, ldw, out, ldo, o_group, M, N, K, groups, seg=None, a_rows=None,
             o_rows=None, row_weight=None, gate=None, gate_ld=0, gate_group=0, gate_col=0, act=0, rows_bound=0,
             force_simt=False, w_packed=False, pair=None):
    L = ctypes.c_long
    _call(load_library("core"), "syn_grouped_product", _ptr(a), L(lda), L(a_group), _ptr(w), L(w_group), L(ldw), _ptr(out),
          L(ldo), L(o_group), _is_f32(a), _is_f32(out), _ptr(seg), _ptr(a_rows), _ptr(o_rows), _ptr(row_weight), _ptr(gate),
          L(gate_ld), L(gate_group), int(gate_col), int(act), int(M), int(N), int(K), int(groups), int(rows_bound),
          int(force_simt), int(bool(w_packed)), *((0, ctypes.c_float(0.0)) if pair is None else (pair[0] + 1, pair[1])),
          _stream())


def heads_product(x, w, out, out_offset=0, gate=None, gate_per_value=True, force_simt=False):
    """A linear map for each head:  out[n, h, out_offset + j] = sum_k x[n, h, k] * w[h, j, k]  [* sigmoid(gate)].
    x [N, heads, K] and w [heads, J, K] in the engine's type, out [N, heads, >= out_offset + J] in that type.
    gate: float rows (columns of a fused projection, any row stride) that hold heads * J values (one for each output,
    gate_per_value) or `heads` values (one a head).  force_simt (tests): 0 the kernel that the sizes call for, 1 plain
    FMA, 2 and 3 the matrix cores with operands straight from memory, 16 and 64 outputs a wave."""
    _need(x, "heads_product.x", (_BF16, _F32), (None, None, None))
    N, Hn, K = x.shape
    _need(w, "heads_product.w", x.dtype, (Hn, None, K))
    J = w.shape[1]
    _need(out, "heads_product.out", x.dtype, (N, Hn, None))
    Jo = out.shape[2]
    if out_offset < 0 or out_offset + J > Jo:
        raise KernelError(f"heads_product: {J} outputs at {out_offset} do not fit rows of {Jo}")
    kw = {}
    if gate is not None:
        need = Hn * J if gate_per_value else Hn
        kw = dict(gate=gate, gate_ld=_float_rows_view(gate, "heads_product.gate", N, need),
                  gate_group=J if gate_per_value else 1, gate_col=1 if gate_per_value else 0)
    if out_offset:
        out = out.view(-1)[out_offset:]
    _grouped("heads_product", x, Hn * K, K, w, J * K, K, out, Hn * Jo, Jo, N, J, K, Hn, force_simt=force_simt, **kw)


ROUTE_MAX_EXPERTS, ROUTE_MAX_TOP = 1024, 64


def route_topk(logits, bias, ids, weights):
    """The choice of a mixture's router: logits [N, E] float (the 32-bit sums of the router's product) + bias [E];
    ids [N, top] int32 the experts with the largest logits (largest first, the lower index of equal ones), weights
    [N, top] float the softmax over those logits alone."""
    _need(logits, "route_topk.logits", _F32, (None, None))
    N, E = logits.shape
    if bias is not None:
        _need(bias, "route_topk.bias", _F32, (E,))
    _need(ids, "route_topk.ids", _I32, (N, None))
    top = ids.shape[1]
    _need(weights, "route_topk.weights", _F32, (N, top))
    if not (0 < top <= min(E, ROUTE_MAX_TOP)) or E > ROUTE_MAX_EXPERTS:
        raise KernelError(f"route_topk: the {top} largest of {E} experts (at most {ROUTE_MAX_TOP} of {ROUTE_MAX_EXPERTS})")
    _call(load_library("core"), "syn_route_topk", _ptr(logits), _ptr(bias), _ptr(ids), _ptr(weights), N, E, top, _stream())


def route_sort(ids, weights, n_experts):
    """The router's choices sorted by expert.  Returns (seg_start [E + 1], tok_of, pair_of, part_of int32 [N * top],
    weight_of float [N * top]): the places seg_start[e] .. seg_start[e + 1] belong to expert e; a place holds the token,
    the pair n * top + t, the pair's row t * N + n in partial sums [top, N], and the pair's weight."""
    _need(ids, "route_sort.ids", _I32, (None, None))
    N, top = ids.shape
    _need(weights, "route_sort.weights", _F32, (N, top))
    if not 0 < n_experts <= ROUTE_MAX_EXPERTS:
        raise KernelError(f"route_sort: {n_experts} experts (at most {ROUTE_MAX_EXPERTS})")
    lists = torch.empty((3, N * top), dtype=_I32, device=ids.device)
    seg = torch.empty(n_experts + 1, dtype=_I32, device=ids.device)
    weight_of = torch.empty(N * top, dtype=_F32, device=ids.device)
    _call(load_library("core"), "syn_route_sort", _ptr(ids), _ptr(weights), _ptr(seg), _ptr(lists[0]), _ptr(lists[1]),
          _ptr(lists[2]), _ptr(weight_of), N, top, n_experts, _stream())
    return seg, lists[0], lists[1], lists[2], weight_of


def route_scores(logits, correction, ids, weights, n_groups=1, keep_groups=1, renorm=False, scale=1.0):
    """A router that scores every expert: s = softmax(logits [N, E] float) over all E; the choice is made on
    s + correction [E] among the members of the keep_groups best of n_groups equal groups of neighbours (a group's
    score: its largest choice score); ids [N, top] int32 the chosen (largest first, the lower index of equal ones),
    weights [N, top] float their s, divided by their sum with renorm, times `scale`.  logits may be the first columns of
    longer rows (a view with a row stride)."""
    if isinstance(logits, torch.Tensor) and logits.dim() == 2:
        ld = _float_rows_view(logits, "route_scores.logits", logits.shape[0], logits.shape[1])
    else:
        raise KernelError("route_scores.logits: expected a float matrix on the GPU")
    N, E = logits.shape
    if correction is not None:
        _need(correction, "route_scores.correction", _F32, (E,))
    _need(ids, "route_scores.ids", _I32, (N, None))
    top = ids.shape[1]
    _need(weights, "route_scores.weights", _F32, (N, top))
    if E > ROUTE_MAX_EXPERTS or n_groups <= 0 or E % n_groups or not 0 < keep_groups <= n_groups:
        raise KernelError(f"route_scores: {E} experts (at most {ROUTE_MAX_EXPERTS}) in {n_groups} groups, {keep_groups} kept")
    if not 0 < top <= min(keep_groups * (E // n_groups), ROUTE_MAX_TOP):
        raise KernelError(f"route_scores: the {top} largest of {keep_groups} groups of {E // n_groups} (at most {ROUTE_MAX_TOP})")
    _call(load_library("core"), "syn_route_scores", _ptr(logits), _ptr(correction), _ptr(ids), _ptr(weights), N, E, ld, top,
          int(n_groups), int(keep_groups), 1 if renorm else 0, ctypes.c_float(float(scale)), _stream())


def route_identity(x, out, seg, first, last, a_rows, o_rows, weight_of):
    """Experts first .. last - 1 of a sorted choice (route_sort) are the identity: out[o_rows[r]] = weight_of[r] *
    x[a_rows[r]] for the places r of their segments.  x [*, H] in the engine's type, out [*, H] float."""
    _need(x, "route_identity.x", (_BF16, _F32), (None, None))
    H = x.shape[1]
    _need(out, "route_identity.out", _F32, (None, H))
    _need(seg, "route_identity.seg", _I32, (None,))
    if not 0 <= first <= last < seg.shape[0]:
        raise KernelError(f"route_identity: experts {first} .. {last} of {seg.shape[0] - 1}")
    _need(a_rows, "route_identity.a_rows", _I32, (None,))
    P = a_rows.shape[0]
    _need(o_rows, "route_identity.o_rows", _I32, (P,))
    _need(weight_of, "route_identity.weight_of", _F32, (P,))
    _call(load_library("core"), "syn_route_identity", _ptr(x), _is_f32(x), _ptr(out), _ptr(seg), int(first), int(last),
          _ptr(a_rows), _ptr(o_rows), _ptr(weight_of), P, H, _stream())


def pack_expert_weights(w):
    """Matrices [E, J, K] in the order of the MFMA fragments, each as pack_weight lays it out: [E, J / 16, K / 32, 64, 8]
    (a wave's load of a k-step is then 1 KB of consecutive bytes); None if the type or the sizes do not allow it."""
    if w.dtype != _BF16 or w.dim() != 3 or w.shape[1] % 16 or w.shape[2] % 32:
        return None
    E, J, K = w.shape
    return w.view(E, J // 16, 16, K // 32, 4, 8).permute(0, 1, 3, 4, 2, 5).reshape(E, J // 16, K // 32, 64, 8).contiguous()


def pair_expert_rows(gate, up):
    """Gate and up matrices [E, J, K] as one [E, 2 J, K] whose rows alternate (2 j: gate row j, 2 j + 1: up row j): what
    experts_product(gated=...) multiplies with."""
    E, J, K = gate.shape
    return torch.stack([gate, up], 2).reshape(E, 2 * J, K).contiguous()


def experts_product(x, w, out, seg, a_rows, o_rows, row_weight=None, gelu=False, force_simt=False, gated=None):
    """out[o_rows[r]] = epilogue(x[a_rows[r]] . w[e]^T) for the places r of each expert e's segment.  x [*, K] in the
    engine's type, w [E, J, K] in that type (or bf16 in fragment order, pack_expert_weights: five dimensions), out
    [*, J] in that type or float; the index lists come from route_sort and
    must stay inside x and out (the caller sees to that: they are on the device).  Epilogue: the exact GELU, then the
    row's weight, each if asked for.  gated: an activation of the gated products (ACTIVATIONS; one with a bound as the
    pair (name, bound)): w then holds gate and up rows in turns (pair_expert_rows), and out [*, J / 2] receives the
    activation of each pair of sums.  force_simt: as in heads_product."""
    _need(x, "experts_product.x", (_BF16, _F32), (None, None))
    K = x.shape[1]
    packed = isinstance(w, torch.Tensor) and w.dim() == 5
    if packed:
        _need(x, "experts_product.x", _BF16, (None, None))
        _need(w, "experts_product.w", _BF16, (None, None, K // 32 if K % 32 == 0 else -1, 64, 8))
        E, J = w.shape[0], w.shape[1] * 16
    else:
        _need(w, "experts_product.w", x.dtype, (None, None, K))
        E, J = w.shape[0], w.shape[1]
    pair = None
    if gated is not None:
        if gelu or J % 2:
            raise KernelError(f"experts_product: a gated activation over {J} rows in pairs, and no other activation")
        pair = _activation_args(gated)
    _need(out, "experts_product.out", (x.dtype, _F32), (None, J // 2 if pair else J))
    _need(seg, "experts_product.seg", _I32, (E + 1,))
    _need(a_rows, "experts_product.a_rows", _I32, (None,))
    P = a_rows.shape[0]
    _need(o_rows, "experts_product.o_rows", _I32, (P,))
    if row_weight is not None:
        _need(row_weight, "experts_product.row_weight", _F32, (P,))
    _grouped("experts_product", x, K, 0, w, J * K, K, out, J // 2 if pair else J, 0, P, J, K, E, seg=seg, a_rows=a_rows,
             o_rows=o_rows, row_weight=row_weight, act=1 if gelu else 0, rows_bound=P, force_simt=force_simt,
             w_packed=packed, pair=pair)


# ----------------------------------------------------------------------------- latent attention: intake

def latent_v_pages_to_kernel_order(v):
    """Value pages [..., rank, 64] of latent attention from plain rows into the order of the bf16 kernel's fragments
    (csrc/latent_attention.hip, la_v_offset); for tests and tools, on any device."""
    rank = v.shape[-2]
    if rank % 16 or v.shape[-1] != PAGE_TOKENS:
        raise KernelError(f"latent_v_pages_to_kernel_order: pages of {rank} x {v.shape[-1]}")
    d = torch.arange(rank, device=v.device)[:, None]
    slot = torch.arange(PAGE_TOKENS, device=v.device)[None, :]
    half, s = slot >> 5, slot & 31
    e = (s & 3) + 4 * (s >> 4)
    offset = (((((d >> 4) * 2 + half) * 64 + ((s & 15) >> 2) * 16 + (d & 15)) << 3) + e).reshape(-1)
    out = torch.empty_like(v).reshape(*v.shape[:-2], rank * PAGE_TOKENS)
    out[..., offset] = v.reshape(*v.shape[:-2], rank * PAGE_TOKENS)
    return out.reshape(v.shape)


def latent_intake(proj, gain, eps, cos, sin, q_nope, q_full, k_pages, v_pages, page_table, tok_seq, tok_pos,
                  n_heads, dim, rot_dim, rank, max_position, write_kv=True, v_fragments=False):
    """From the fused projection proj [N, >= heads * (dim + rot_dim) + rank + rot_dim] float: q_nope [N, heads * dim];
    the rotated query parts into q_full [N, heads * (rank + rot_dim)] behind each head's first `rank` places; the
    token's cache row [RMSNorm(latent) * gain | rotated key part] into k_pages [pages, 1, 64, rank + rot_dim] and the
    normed latent as its value into v_pages [pages, 1, rank, 64].  cos, sin [capacity, pairs]: pairs (2i, 2i + 1) of
    the rotated parts are turned, what lies behind 2 * pairs passes.  v_fragments: the value pages are kept in the order
    of the bf16 attention kernel's fragments (what latent_attention reads when it runs in tiles)."""
    _need(proj, "latent_intake.proj", _F32, (None, None))
    N, width = proj.shape
    R = rank + rot_dim
    if width < n_heads * (dim + rot_dim) + R:
        raise KernelError(f"latent_intake: rows of {width} values do not hold {n_heads} queries and the latent")
    _need(gain, "latent_intake.gain", (_BF16, _F32), (rank,))
    n_pairs, capacity = 0, 0
    if cos is not None:
        _need(cos, "latent_intake.cos", _F32, (None, None))
        capacity, n_pairs = cos.shape
        _need(sin, "latent_intake.sin", _F32, (capacity, n_pairs))
        if 2 * n_pairs > rot_dim or max_position >= capacity:
            raise KernelError(f"latent_intake: {n_pairs} pairs in {rot_dim} values, position {max_position} of {capacity}")
    _need(q_nope, "latent_intake.q_nope", (_BF16, _F32), (N, n_heads * dim))
    _need(q_full, "latent_intake.q_full", q_nope.dtype, (N, n_heads * R))
    _need(k_pages, "latent_intake.k_pages", q_nope.dtype, (None, 1, PAGE_TOKENS, R))
    _need(v_pages, "latent_intake.v_pages", q_nope.dtype, (k_pages.shape[0], 1, rank, PAGE_TOKENS))
    _need(page_table, "latent_intake.page_table", _I32, (None, None))
    _need(tok_seq, "latent_intake.tok_seq", _I32, (N,))
    _need(tok_pos, "latent_intake.tok_pos", _I32, (N,))
    _call(load_library("core"), "syn_latent_intake", _ptr(proj), width, _ptr(gain), _is_f32(gain), ctypes.c_float(eps),
          _ptr(cos), _ptr(sin), n_pairs, capacity, int(max_position), _ptr(q_nope), _ptr(q_full), _ptr(k_pages),
          _ptr(v_pages), _is_f32(q_nope), _ptr(page_table), page_table.shape[1], _ptr(tok_seq), _ptr(tok_pos), N, n_heads,
          dim, rot_dim, rank, int(bool(write_kv)), int(bool(v_fragments)), _stream())


# ----------------------------------------------------------------------------- latent attention

LATENT_ATTENTION_MAX_ROW = WINDOW_ATTENTION_MAX_DIM      # plain FMA: 32-bit, and sizes that the tiles do not take
LATENT_TILED_MAX_RANK, LATENT_TILED_MAX_ROW = 512, 640


def latent_attention_tiled(rank, rot_dim) -> bool:
    """Whether the bf16 kernel on the matrix cores takes these sizes."""
    return (rank % 16 == 0 and (rank + rot_dim) % 16 == 0 and 0 < rank <= LATENT_TILED_MAX_RANK
            and rank + rot_dim <= LATENT_TILED_MAX_ROW)


def latent_attention_takes(rank, rot_dim, dtype=_F32) -> bool:
    if dtype == _BF16 and latent_attention_tiled(rank, rot_dim):
        return True
    return 0 < rank and rank + rot_dim <= LATENT_ATTENTION_MAX_ROW


def _latent_tiles(n_tokens, n_heads, n_seqs, max_pages):
    """(a bound on the workgroups, the splits of a tile's pages, whether a workgroup's waves share a tile of 16 (token,
    head) rows): many tiles run whole, a wave each and four of a sequence a workgroup."""
    tiles = (n_tokens * n_heads + 15) // 16 + n_seqs
    if tiles >= 256:
        # (a workgroup for every four tiles of a sequence: the bound counts those)
        return (n_tokens * n_heads + 63) // 64 + n_seqs, 1, False
    # few tiles: the four waves of a workgroup work on a tile together, and its pages are cut into splits until some
    # 1,024 workgroups have work
    return tiles, max(1, min(int(max_pages), 1024 // tiles, 1024)), True


def latent_attention_workspace(n_tokens, n_heads, n_seqs, rank, max_pages) -> int:
    """Floats of workspace that latent_attention needs for a step of these sizes (0: none)."""
    tiles, splits, _ = _latent_tiles(n_tokens, n_heads, n_seqs, max_pages)
    return tiles * splits * 16 * (rank + 2) if splits > 1 else 0


def latent_attention(q_full, k_pages, v_pages, page_table, tok_seq, tok_pos, out, scale, n_heads, rank, rot_dim, window=0,
                     seqs=None, workspace=None, force_simt=False):
    """Attention of `n_heads` queries a token over one shared key row a cached token: q_full [N, heads * (rank +
    rot_dim)], key rows k_pages [pages, 1, 64, rank + rot_dim] whose first `rank` values are the row's value (v_pages
    [pages, 1, rank, 64] holds them once more, along the keys); out [N, heads * rank] = sum_j softmax_j(scale q . k_j)
    k_j[:rank] over the keys at or before the query's position (window > 0: the last `window` of them).  Scores,
    weights and sums are 32-bit.  seqs = (seq_start [B + 1], seq_past [B]): the step's sequences, whose new tokens lie
    one after another at positions seq_past[b] ..; with them bf16 runs in tiles on the matrix cores where the sizes
    allow (latent_attention_tiled), with `workspace` floats (latent_attention_workspace) for tiles cut into splits; the
    value pages are then in the order of that kernel's fragments (latent_intake(v_fragments=True),
    latent_v_pages_to_kernel_order)."""
    R = rank + rot_dim
    if q_full.dtype == _BF16 and seqs is not None and latent_attention_tiled(rank, rot_dim) and not force_simt:
        seq_start, seq_past = seqs
        _need(q_full, "latent_attention.q", _BF16, (None, n_heads * R))
        N = q_full.shape[0]
        _need(k_pages, "latent_attention.k_pages", _BF16, (None, 1, PAGE_TOKENS, R))
        _need(v_pages, "latent_attention.v_pages", _BF16, (k_pages.shape[0], 1, rank, PAGE_TOKENS))
        _need(page_table, "latent_attention.page_table", _I32, (None, None))
        _need(seq_past, "latent_attention.seq_past", _I32, (None,))
        B = seq_past.shape[0]
        _need(seq_start, "latent_attention.seq_start", _I32, (B + 1,))
        if page_table.shape[0] < B:
            raise KernelError(f"latent_attention: page table has {page_table.shape[0]} rows for {B} sequences")
        _need(out, "latent_attention.out", _BF16, (N, n_heads * rank))
        tiles, splits, share = _latent_tiles(N, n_heads, B, page_table.shape[1])
        floats = 0
        if splits > 1:
            need = tiles * splits * 16 * (rank + 2)
            if workspace is None:
                workspace = torch.empty(need, dtype=_F32, device=q_full.device)
            _need(workspace, "latent_attention.workspace", _F32, (None,))
            floats = workspace.shape[0]
            if floats < need:
                raise KernelError(f"latent_attention: a workspace of {floats} floats, {need} needed")
        _call(load_library("core"), "syn_latent_attention_bf16", _ptr(q_full), _ptr(k_pages), _ptr(v_pages), _ptr(page_table),
              page_table.shape[1], _ptr(seq_start), _ptr(seq_past), B, _ptr(out), _ptr(workspace if splits > 1 else None),
              ctypes.c_long(floats), ctypes.c_float(scale), tiles, n_heads, rank, rot_dim, int(window or 0), splits, int(share), _stream())
        return
    window_attention(q_full, k_pages, v_pages, page_table, tok_seq, tok_pos, out, scale, n_heads, 1, R, rank, window=window)
