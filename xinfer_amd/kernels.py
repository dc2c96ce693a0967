"""Python bindings of the gfx950 kernel library (csrc/kernels/*.hip) through ctypes.

Every function checks on the host that operand shapes, types, devices and layouts match
what the kernel and its grid assume, and raises `KernelError` otherwise: a kernel is
never launched on operands it was not written for.  Kernels run on torch's current HIP
stream.  There is no other implementation behind these functions: if the library
cannot be built or loaded, importing fails loudly.
"""
from __future__ import annotations

import ctypes
import functools
from typing import Optional

import torch

from .csrc.build import load_kernels


class KernelError(RuntimeError):
    pass


F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}

_lib = None


def lib():
    global _lib
    if _lib is None:
        l = load_kernels()
        l.xi_last_error.restype = ctypes.c_char_p
        _lib = l
    return _lib


def _code(t: torch.Tensor, what: str) -> int:
    try:
        return _CODE[t.dtype]
    except KeyError:
        raise KernelError(f"{what}: dtype {t.dtype} is not supported (float32 or bfloat16)") from None


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("kernel operands must live on the GPU (there is no CPU path)")
        if not t.is_contiguous():
            raise KernelError(f"kernel operand of shape {tuple(t.shape)} is not contiguous")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise KernelError("kernel operands live on different devices")


def _p(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> ctypes.c_void_p:
    """The current HIP stream of the current device (asked for at every launch: the runner
    records graphs on a side stream)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ok(rc: int) -> None:
    if rc != 0:
        raise KernelError(lib().xi_last_error().decode())


def _want(t: torch.Tensor, dtype: torch.dtype, what: str) -> None:
    if t.dtype != dtype:
        raise KernelError(f"{what} must be {dtype}, got {t.dtype}")


# ---------------------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """out[t] = float32(table[ids[t]]) * scale.  ids: int32 [T], values in [0, rows) (caller checks)."""
    _dev(table, ids, out)
    _want(ids, torch.int32, "embed: ids")
    if table.dim() != 2 or ids.dim() != 1:
        raise KernelError("embed: table must be [V, H] and ids [T]")
    T, H = ids.shape[0], table.shape[1]
    if out is None:
        out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    elif out.shape != (T, H) or out.dtype != torch.float32:
        raise KernelError("embed: out must be float32 [T, H]")
    _ok(lib().xi_embed(_p(table), _code(table, "embed"), _p(ids), _p(out), T, H, ctypes.c_float(scale), _stream()))
    return out


def counter_normal_(out: torch.Tensor, key: int, scale: float = 1.0, shift: float = 0.0, first: int = 0) -> torch.Tensor:
    """out.flat[i] = normal(key, first + i) * scale + shift, rounded once to out's type (float32 or
    bfloat16): seeded normal values that depend on (key, index) alone, bit for bit those of
    `weights.counter_normal.counter_normal` on the CPU."""
    _dev(out)
    if not (0 <= key < 1 << 64) or first < 0:
        raise KernelError("counter_normal: the key is a 64-bit number and the first index is not negative")
    _ok(lib().xi_counter_normal(_p(out), ctypes.c_uint64(out.numel()), ctypes.c_uint64(first), ctypes.c_uint64(key),
                                ctypes.c_float(scale), ctypes.c_float(shift), _code(out, "counter_normal"), _stream()))
    return out


def stream_read(t: torch.Tensor, workgroups: int = 2048, chunk_bytes: int = 1 << 18) -> None:
    """Reads all of a tensor's memory and keeps nothing: the plain read-only stream that the
    weight-streaming kernels are measured against.  A workgroup reads whole chunks of
    `chunk_bytes` (a multiple of 8 KB)."""
    _dev(t)
    _ok(lib().xi_stream_read(_p(t), ctypes.c_int64(t.numel() * t.element_size()), int(workgroups),
                             ctypes.c_int64(chunk_bytes), _stream()))


def lane_xor_probe(values: torch.Tensor) -> torch.Tensor:
    """values [64] float32 -> [8, 64]: row i < 6 holds values[l ^ (1 << i)] as the kernels' exchange
    between lanes gives it, row 6 the wave's sum and row 7 its maximum in every lane (for tests)."""
    _dev(values)
    _want(values, torch.float32, "lane_xor_probe: values")
    if values.shape != (64,):
        raise KernelError("lane_xor_probe: 64 values, one a lane")
    out = torch.empty((8, 64), dtype=torch.float32, device=values.device)
    _ok(lib().xi_lane_xor_probe(_p(values), _p(out), _stream()))
    return out


def softcap_(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """logits = cap * tanh(logits / cap), in place, float32."""
    _dev(logits)
    _want(logits, torch.float32, "softcap: logits")
    if not cap > 0:
        raise KernelError(f"softcap: the cap must be positive, got {cap}")
    _ok(lib().xi_softcap(_p(logits), ctypes.c_int64(logits.numel()), ctypes.c_float(cap), _stream()))
    return logits


def add_rmsnorm(resid: torch.Tensor, y: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None, y_scale: float = 1.0) -> torch.Tensor:
    """s = resid (+ y_scale * y); out = rms(s) * weight in `out_dtype`.  Without `rows` every row is
    normed and the sum is written back into resid; with `rows` (int32 indices) only those
    rows are produced and resid is left alone.  y may be a stack [P, T, H] of float32 partial
    sums, which are added in order."""
    _dev(resid, y, weight, rows, out)
    _want(resid, torch.float32, "add_rmsnorm: residual stream")
    _want(weight, torch.float32, "add_rmsnorm: weight")
    if resid.dim() != 2 or weight.shape != (resid.shape[1],):
        raise KernelError(f"add_rmsnorm: resid {tuple(resid.shape)} and weight {tuple(weight.shape)} do not match")
    parts = 1
    if y is not None and y.dim() == 3:
        if y.dtype != torch.float32 or tuple(y.shape[1:]) != tuple(resid.shape):
            raise KernelError(f"add_rmsnorm: partial sums {tuple(y.shape)} {y.dtype} must be float32 [P, T, H]")
        parts = int(y.shape[0])
    elif y is not None and y.shape != resid.shape:
        raise KernelError(f"add_rmsnorm: y {tuple(y.shape)} differs from resid {tuple(resid.shape)}")
    H = resid.shape[1]
    if rows is not None:
        _want(rows, torch.int32, "add_rmsnorm: rows")
        n = rows.shape[0]
    else:
        n = resid.shape[0]
    if out is None:
        out = torch.empty((n, H), dtype=out_dtype, device=resid.device)
    elif out.shape != (n, H) or out.dtype != out_dtype:
        raise KernelError("add_rmsnorm: out has the wrong shape or dtype")
    _ok(lib().xi_add_rmsnorm(_p(resid), _p(y), _code(y, "add_rmsnorm") if y is not None else F32, parts,
                             int(resid.shape[0]), _p(weight), ctypes.c_float(eps), _p(out),
                             _code(out, "add_rmsnorm"), _p(rows), n, H, ctypes.c_float(y_scale), _stream()))
    return out


def silu_mul(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = silu(gate_up[:, :I]) * gate_up[:, I:]"""
    _dev(gate_up, out)
    if gate_up.dim() != 2 or gate_up.shape[1] % 2:
        raise KernelError("silu_mul: input must be [T, 2I]")
    T, I = gate_up.shape[0], gate_up.shape[1] // 2
    if out is None:
        out = torch.empty((T, I), dtype=gate_up.dtype, device=gate_up.device)
    elif out.shape != (T, I) or out.dtype != gate_up.dtype:
        raise KernelError("silu_mul: out has the wrong shape or dtype")
    _ok(lib().xi_silu_mul(_p(gate_up), _p(out), _code(gate_up, "silu_mul"), T, I, _stream()))
    return out


ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}
UNGATED_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "relu2": 2}     # relu2: the square of relu


def act_(x: torch.Tensor, act: str) -> torch.Tensor:
    """x <- act(x) in place, an activation without a gate (see UNGATED_ACTIVATIONS)."""
    _dev(x)
    if act not in UNGATED_ACTIVATIONS:
        raise KernelError(f"act: unknown activation {act!r}")
    _ok(lib().xi_act(_p(x), _code(x, "act"), UNGATED_ACTIVATIONS[act], ctypes.c_int64(x.numel()), _stream()))
    return x


def scaled_sum(acc: Optional[torch.Tensor], y: torch.Tensor, factor: float) -> torch.Tensor:
    """acc + factor * y in float32 (acc None: factor * y in a new tensor; else in place).  y: rows [T, H] in
    either precision, or a stack [P, T, H] of float32 partial sums, which are added in order first."""
    _dev(acc, y)
    parts = 1
    if y.dim() == 3:
        _want(y, torch.float32, "scaled_sum: partial sums")
        parts = int(y.shape[0])
    elif y.dim() != 2:
        raise KernelError("scaled_sum: rows [T, H] or partial sums [P, T, H]")
    shape = tuple(y.shape[-2:])
    first = acc is None
    if first:
        acc = torch.empty(shape, dtype=torch.float32, device=y.device)
    elif acc.dtype != torch.float32 or tuple(acc.shape) != shape:
        raise KernelError(f"scaled_sum: the sum {tuple(acc.shape)} {acc.dtype} must be float32 {shape}")
    _ok(lib().xi_scaled_sum(_p(acc), int(first), _p(y), _code(y, "scaled_sum"), parts, ctypes.c_int64(acc.numel()),
                            ctypes.c_float(factor), _stream()))
    return acc


def scale_(x: torch.Tensor, factor: float) -> torch.Tensor:
    """x <- x * factor in place (float32)."""
    _dev(x)
    _want(x, torch.float32, "scale")
    _ok(lib().xi_scale(_p(x), ctypes.c_int64(x.numel()), ctypes.c_float(factor), _stream()))
    return x


def gated_add_(out: torch.Tensor, y: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """out[t] += sigmoid(gate[t]) * y[t]: out float32 [T, H], y [T, H], gate float32 [T] or a column [T, X][:, 0]
    (one number a token)."""
    _dev(out, y)
    _want(out, torch.float32, "gated_add: out")
    _want(gate, torch.float32, "gated_add: gate")
    if out.dim() != 2 or y.shape != out.shape or gate.dim() != 1 or gate.shape[0] != out.shape[0] or not gate.is_cuda:
        raise KernelError(f"gated_add: out {tuple(out.shape)}, y {tuple(y.shape)} and gate {tuple(gate.shape)} do not match")
    _ok(lib().xi_gated_add(_p(out), _p(y), _code(y, "gated_add"), _p(gate), int(gate.stride(0)) if gate.shape[0] > 1 else 1,
                           int(out.shape[0]), int(out.shape[1]), _stream()))
    return out


def _columns(t: torch.Tensor, width: int, what: str):
    """A [T, width] view of a packed projection: its pointer stays, the row stride is handed to the kernel."""
    if t.dim() != 2 or t.shape[1] != width or t.stride(1) != 1 or not t.is_cuda:
        raise KernelError(f"{what}: {tuple(t.shape)} with strides {t.stride()} is not [T, {width}] rows")
    return int(t.stride(0)) if t.shape[0] > 1 else width


SCAN_CHUNK = 64           # tokens of a chunk of a long portion (see `linear_scan`); 0: every portion is walked in one piece
SCAN_CHUNKS_MOST = 512    # chunks of a step at most (their states are kept side by side): longer steps get longer chunks


def scan_chunk_plan(q_lens, chunk: Optional[int] = None):
    """How a step's portions are walked by `linear_scan`: (whole, long, chunks) with `whole` the batch rows walked in
    one piece (single tokens and portions of less than two chunks) and, for the others, `long` = [(row, first chunk,
    number of chunks)] and `chunks` = [(first token within the portion, tokens)] in the order of their numbers."""
    chunk = SCAN_CHUNK if chunk is None else int(chunk)
    total = sum(int(n) for n in q_lens)
    if chunk > 0 and total > chunk * SCAN_CHUNKS_MOST:
        chunk = -(-total // SCAN_CHUNKS_MOST // 16) * 16
    whole, long, chunks = [], [], []
    for b, n in enumerate(q_lens):
        n = int(n)
        if chunk <= 0 or n < 2 * chunk:
            whole.append(b)
            continue
        count = -(-n // chunk)
        long.append((b, len(chunks), count))
        chunks += [(c * chunk, min(chunk, n - c * chunk)) for c in range(count)]
    return whole, long, chunks


def _scan_launch(q, k, v, qs, ks, vs, z, z_bias, tau, head_decay, step, ss, step_bias, decay_log, gates, v_cols, group_heads,
                 state_in, in_stride, in_idx, state_out, out_stride, out_idx,
                 first, last, out, decay_out, items, H, dk, dv, q_scale, k_scale):
    _ok(lib().xi_linear_scan(_p(q), ctypes.c_longlong(qs), _p(k), ctypes.c_longlong(ks), _p(v), ctypes.c_longlong(vs),
                             _code(q, "linear_scan"), _p(z), _p(z_bias), ctypes.c_float(tau), _p(head_decay),
                             _p(step), ctypes.c_longlong(ss), _p(step_bias), _p(decay_log), _p(gates), int(v_cols),
                             int(group_heads), _p(state_in),
                             ctypes.c_longlong(in_stride), _p(in_idx), _p(state_out), ctypes.c_longlong(out_stride),
                             _p(out_idx), ctypes.c_void_p(first), ctypes.c_void_p(last), _p(out), _p(decay_out), int(items),
                             H, dk, dv, ctypes.c_float(q_scale), ctypes.c_float(k_scale), _stream()))


def linear_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, state: torch.Tensor, state_slots: torch.Tensor,
                cu_q: torch.Tensor, heads: int, key_dim: int, value_dim: int, z: Optional[torch.Tensor] = None,
                tau: float = 1.0, head_decay: Optional[torch.Tensor] = None, q_scale: float = 1.0,
                k_scale: float = 1.0, z_bias: Optional[torch.Tensor] = None, q_lens=None, plan_cache=None,
                step: Optional[torch.Tensor] = None, step_bias: Optional[torch.Tensor] = None,
                decay_log: Optional[torch.Tensor] = None, groups: Optional[int] = None,
                gates: Optional[torch.Tensor] = None, value_cols: Optional[int] = None) -> torch.Tensor:
    """Linear attention with a decaying float32 state per request and head, S <- diag(a) S + k v^T, o = S^T q,
    token by token from the state each request's slot holds (left there afterwards).  q, k [T, H dk] and
    v [T, H dv] may be column ranges of a packed projection.  The decay: `z` float32 [T, H dk], `z_bias`
    float32 [H dk] (or None) and `tau` (a = sigmoid(z + bias)^(1 / tau) per token and key channel) or `head_decay` float32 [H] (a constant per head),
    or `step` [T, H] (columns of a projection, in q's type), `step_bias` and `decay_log` float32 [H]: the step size d =
    softplus(step + step_bias), a = exp(-exp(decay_log) d) per token and head, and the token's value row times d.
    Or `gates` float32 [T, H, 2], made beforehand: a = gates[t, h, 0] and the token's value row times gates[t, h, 1].
    `value_cols` = value_dim - 1: v is [T, H (value_dim - 1)] and the state's last column reads the value 1 (it then
    holds the decayed sum of the weighted keys alone, and the results' last column that sum times q).
    `groups` G: q and k are [T, G dk] and head h reads the columns of group h // (H / G).
    state float32 [slots, H, dk, dv] (slots may be strided); state_slots int64 [B]; cu_q int32 [B + 1].
    Returns o float32 [T, H, dv].
    `q_lens` (the host's copy of the portions' lengths; None: nothing of the step is read on the host, as a step
    of single tokens wants it): portions of two chunks and more (`SCAN_CHUNK`) are cut into chunks that are walked
    side by side in three launches (each chunk's own share from a zero state; the states the chunks start from,
    one after the other; the chunks' results), the others in one piece.  `plan_cache`: a dict of the step in which
    the index arrays of this cutting are kept for the next layer."""
    H, dk, dv = int(heads), int(key_dim), int(value_dim)
    T = q.shape[0]
    G = H if groups is None else int(groups)
    if G <= 0 or H % G:
        raise KernelError(f"linear_scan: {H} heads in {G} groups")
    vc = dv if value_cols is None else int(value_cols)
    if vc not in (dv, dv - 1) or vc <= 0:
        raise KernelError(f"linear_scan: {vc} value columns for a state of {dv}")
    qs, ks, vs = _columns(q, G * dk, "linear_scan: q"), _columns(k, G * dk, "linear_scan: k"), _columns(v, H * vc, "linear_scan: v")
    if k.shape[0] != T or v.shape[0] != T or q.dtype != k.dtype or q.dtype != v.dtype or not (q.device == k.device == v.device):
        raise KernelError("linear_scan: q, k and v must be rows of the same tokens, type and device")
    _dev(z, head_decay, state_slots, cu_q, z_bias, step_bias, decay_log, gates)
    ss = 0
    if gates is not None:
        if z is not None or head_decay is not None or step is not None:
            raise KernelError("linear_scan: ready-made gates come alone")
        _want(gates, torch.float32, "linear_scan: gates")
        if tuple(gates.shape) != (T, H, 2) or not gates.is_contiguous():
            raise KernelError(f"linear_scan: gates {tuple(gates.shape)} must be [{T}, {H}, 2]")
    if step is not None:
        if z is not None or head_decay is not None or step_bias is None or decay_log is None:
            raise KernelError("linear_scan: a step size comes with its bias and its rate, and alone")
        ss = _columns(step, H, "linear_scan: step")
        if step.shape[0] != T or step.dtype != q.dtype or step.device != q.device:
            raise KernelError("linear_scan: the step sizes must be rows of the same tokens, type and device")
        for t_, what in ((step_bias, "step_bias"), (decay_log, "decay_log")):
            _want(t_, torch.float32, f"linear_scan: {what}")
            if t_.shape != (H,):
                raise KernelError(f"linear_scan: {what} {tuple(t_.shape)} must be [{H}]")
    if z_bias is not None and (z is None or z_bias.dtype != torch.float32 or z_bias.shape != (H * dk,)):
        raise KernelError(f"linear_scan: the bias of the decay's logits must be float32 [{H * dk}], beside z")
    if step is None and gates is None and (z is None) == (head_decay is None):
        raise KernelError("linear_scan: a decay per token (z) or per head (head_decay), one of them")
    if step is not None or gates is not None:
        pass
    elif z is not None:
        _want(z, torch.float32, "linear_scan: z")
        if z.shape != (T, H * dk) or not tau > 0:
            raise KernelError(f"linear_scan: z {tuple(z.shape)} must be [{T}, {H * dk}] and tau positive")
    else:
        _want(head_decay, torch.float32, "linear_scan: head_decay")
        if head_decay.shape != (H,):
            raise KernelError(f"linear_scan: head_decay {tuple(head_decay.shape)} must be [{H}]")
    _want(state, torch.float32, "linear_scan: state")
    _want(state_slots, torch.int64, "linear_scan: state_slots")
    _want(cu_q, torch.int32, "linear_scan: cu_q")
    if (state.dim() != 4 or tuple(state.shape[1:]) != (H, dk, dv) or not state.is_cuda or state.device != q.device
            or state[0].stride() != (dk * dv, dv, 1)):
        raise KernelError(f"linear_scan: state {tuple(state.shape)} must be [slots, {H}, {dk}, {dv}] with whole slots")
    B = state_slots.shape[0]
    if cu_q.shape != (B + 1,) or dk > 256:
        raise KernelError("linear_scan: cu_q must be [B + 1]; key heads of up to 256 channels")
    if q_lens is not None and (len(q_lens) != B or sum(int(n) for n in q_lens) != T):
        raise KernelError("linear_scan: the portions' lengths do not add up to the step's tokens")
    out = torch.empty((T, H, dv), dtype=torch.float32, device=q.device)
    slot_stride = int(state.stride(0)) if state.shape[0] > 1 else H * dk * dv
    common = (q, k, v, qs, ks, vs, z, z_bias, tau, head_decay, step, ss, step_bias, decay_log, gates, vc, H // G)
    whole, long, chunks = scan_chunk_plan(q_lens) if q_lens is not None else (None, [], [])
    if not long:            # every request in one piece, straight from the step's own arrays
        _scan_launch(*common, state, slot_stride, state_slots, state, slot_stride, state_slots, cu_q.data_ptr(),
                     cu_q.data_ptr() + 4, out, None, B, H, dk, dv, q_scale, k_scale)
        return out
    key = ("linear_scan_plan", SCAN_CHUNK)
    plan = plan_cache.get(key) if plan_cache is not None else None
    if plan is None:             # the same for every layer of the step: made once
        starts = [0]
        for n in q_lens:
            starts.append(starts[-1] + int(n))
        C, L, W = len(chunks), len(long), len(whole)
        first, last, hands_on = [0] * C, [0] * C, [False] * C
        for b, c0, count in long:
            for c in range(count):
                first[c0 + c] = starts[b] + chunks[c0 + c][0]
                last[c0 + c] = first[c0 + c] + chunks[c0 + c][1]
                hands_on[c0 + c] = c + 1 < count          # a portion's last chunk hands no share on
        i32 = torch.tensor(first + last
                           + [f if h else 0 for f, h in zip(first, hands_on)] + [l if h else 0 for l, h in zip(last, hands_on)]
                           + [c0 for _, c0, _ in long] + [n for _, _, n in long]
                           + [starts[b] for b in whole] + [starts[b + 1] for b in whole], dtype=torch.int32).to(q.device)
        i64 = torch.tensor([c if h else -1 for c, h in enumerate(hands_on)] + list(range(C)) + [-1] * C
                           + [b for b, _, _ in long] + [c0 + n - 1 for _, c0, n in long] + whole, dtype=torch.int64).to(q.device)
        long_slots = state_slots.index_select(0, i64[3 * C:3 * C + L])
        keep = i64[2 * C:3 * C]         # where launch 3 leaves a chunk's last state: a portion's last chunk in the slot
        keep.index_copy_(0, i64[3 * C + L:3 * C + 2 * L], long_slots)
        slots_w = state_slots.index_select(0, i64[3 * C + 2 * L:]) if W else None
        plan = dict(C=C, L=L, W=W, first=i32[:C], last=i32[C:2 * C], first1=i32[2 * C:3 * C], last1=i32[3 * C:4 * C],
                    c0=i32[4 * C:4 * C + L], n=i32[4 * C + L:4 * C + 2 * L], wfirst=i32[4 * C + 2 * L:4 * C + 2 * L + W],
                    wlast=i32[4 * C + 2 * L + W:], share_to=i64[:C], every=i64[C:2 * C], keep=keep, long_slots=long_slots,
                    slots_w=slots_w)
        if plan_cache is not None:
            plan_cache[key] = plan
    P = plan
    C, per = P["C"], H * dk * dv
    shares = torch.empty((C, H, dk, dv), dtype=torch.float32, device=q.device)
    begins = torch.empty((C, H, dk, dv), dtype=torch.float32, device=q.device)
    decays = torch.empty((C, H, dk), dtype=torch.float32, device=q.device)
    _scan_launch(*common, None, 0, None, shares, per, P["share_to"], P["first1"].data_ptr(), P["last1"].data_ptr(), None, decays,
                 C, H, dk, dv, q_scale, k_scale)
    _ok(lib().xi_chunk_carry(_p(state), ctypes.c_longlong(slot_stride), _p(P["long_slots"]), _p(P["c0"]), _p(P["n"]), _p(shares),
                             _p(decays), _p(begins), P["L"], H, dk, dv, _stream()))
    _scan_launch(*common, begins, per, P["every"], state, slot_stride, P["keep"], P["first"].data_ptr(), P["last"].data_ptr(), out,
                 None, C, H, dk, dv, q_scale, k_scale)
    if P["W"]:
        _scan_launch(*common, state, slot_stride, P["slots_w"], state, slot_stride, P["slots_w"], P["wfirst"].data_ptr(),
                     P["wlast"].data_ptr(), out, None, P["W"], H, dk, dv, q_scale, k_scale)
    return out


def head_norm_gate(o: torch.Tensor, weight: Optional[torch.Tensor], eps: float, gate: torch.Tensor,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """o float32 [T, H, dv]: each head divided by its root mean square over dv (eps inside the root), times
    `weight` float32 [dv] (shared by the heads; None: no weight), times silu(gate) (gate [T, H dv], may be a
    column range of a packed projection, in `out_dtype`).  Returns [T, H dv] in `out_dtype`."""
    _dev(o, weight)
    _want(o, torch.float32, "head_norm_gate: o")
    if o.dim() != 3:
        raise KernelError("head_norm_gate: o must be [T, H, dv]")
    T, H, dv = o.shape
    gs = _columns(gate, H * dv, "head_norm_gate: gate")
    if gate.shape[0] != T or gate.dtype != out_dtype or gate.device != o.device:
        raise KernelError("head_norm_gate: the gate must be rows of the same tokens in the output's type")
    if weight is not None:
        _want(weight, torch.float32, "head_norm_gate: weight")
        if weight.shape != (dv,):
            raise KernelError(f"head_norm_gate: weight {tuple(weight.shape)} must be [{dv}]")
    out = torch.empty((T, H * dv), dtype=out_dtype, device=o.device)
    _ok(lib().xi_head_norm_gate(_p(o), _p(weight), ctypes.c_float(eps), _p(gate), ctypes.c_longlong(gs), _p(out),
                                _code(out, "head_norm_gate"), T, H, dv, _stream()))
    return out


def act_mul(gate_up: torch.Tensor, act: str = "silu", row_scale: Optional[torch.Tensor] = None,
            row_of: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = act(gate_up[:, :I]) * gate_up[:, I:] for an activation of `ACTIVATIONS` (float32 inside).  `row_scale`
    (float32; row t's factor is row_scale[row_of[t]], or row_scale[t] without `row_of` int32 [T]) multiplies gate and
    up first: a factor on the input of the two products."""
    _dev(gate_up, row_scale, row_of)
    if row_scale is not None:
        _want(row_scale, torch.float32, "act_mul: row_scale")
        if row_of is not None:
            _want(row_of, torch.int32, "act_mul: row_of")
        if not row_scale.is_contiguous() or (row_of if row_of is not None else row_scale).numel() < gate_up.shape[0]:
            raise KernelError("act_mul: a factor a row is needed")
    if act not in ACTIVATIONS:
        raise KernelError(f"act_mul: unknown activation {act!r} ({', '.join(ACTIVATIONS)})")
    if gate_up.dim() != 2 or gate_up.shape[1] % 2:
        raise KernelError("act_mul: input must be [T, 2I]")
    T, I = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((T, I), dtype=gate_up.dtype, device=gate_up.device)
    _ok(lib().xi_act_mul(_p(gate_up), _p(out), _code(gate_up, "act_mul"), ACTIVATIONS[act], T, I, _p(row_scale),
                         _p(row_of if row_scale is not None else None), _stream()))
    return out


def embed_sinusoid(table: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor, freq: torch.Tensor,
                   scale: float = 1.0, rows_dtype: Optional[torch.dtype] = None):
    """out[t, c] = float32(table[ids[t], c]) * scale + (sin if c even else cos)(positions[t] * freq[c // 2]).
    Returns (out float32 [T, H], rows): rows is out rounded to `rows_dtype`, None if not asked for."""
    _dev(table, ids, positions, freq)
    _want(ids, torch.int32, "embed_sinusoid: ids")
    _want(positions, torch.int32, "embed_sinusoid: positions")
    _want(freq, torch.float32, "embed_sinusoid: freq")
    if table.dim() != 2 or ids.dim() != 1 or positions.shape != ids.shape:
        raise KernelError("embed_sinusoid: table must be [V, H], ids and positions [T]")
    T, H = ids.shape[0], table.shape[1]
    if freq.shape != ((H + 1) // 2,):
        raise KernelError(f"embed_sinusoid: {tuple(freq.shape)} frequencies for a width of {H}")
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    rows = None if rows_dtype is None else torch.empty((T, H), dtype=rows_dtype, device=table.device)
    _ok(lib().xi_embed_sinusoid(_p(table), _code(table, "embed_sinusoid"), _p(ids), _p(positions), _p(freq), _p(out),
                                _p(rows), _code(rows, "embed_sinusoid") if rows is not None else F32, T, H,
                                ctypes.c_float(scale), _stream()))
    return out, rows


def rmsnorm_add(resid: torch.Tensor, y: torch.Tensor, weight: Optional[torch.Tensor], eps: float,
                rows_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """resid += rms(y) * weight in place (float32), y [T, H] or a stack [P, T, H] of partial sums added in
    order; without `weight` resid += y.  Returns resid rounded to `rows_dtype` ([T, H]) if asked for."""
    _dev(resid, y, weight)
    _want(resid, torch.float32, "rmsnorm_add: residual stream")
    if resid.dim() != 2:
        raise KernelError("rmsnorm_add: the residual stream must be [T, H]")
    T, H = resid.shape
    parts = 1
    if y.dim() == 3:
        parts = int(y.shape[0])
        if tuple(y.shape[1:]) != (T, H) or parts < 1:
            raise KernelError(f"rmsnorm_add: partial sums {tuple(y.shape)} must be [P, {T}, {H}]")
    elif tuple(y.shape) != (T, H):
        raise KernelError(f"rmsnorm_add: y {tuple(y.shape)} differs from resid {(T, H)}")
    if weight is not None:
        _want(weight, torch.float32, "rmsnorm_add: weight")
        if weight.shape != (H,):
            raise KernelError(f"rmsnorm_add: weight {tuple(weight.shape)} is not [{H}]")
    rows = None if rows_dtype is None else torch.empty((T, H), dtype=rows_dtype, device=resid.device)
    _ok(lib().xi_rmsnorm_add(_p(resid), _p(y), _code(y, "rmsnorm_add"), parts, _p(weight), ctypes.c_float(eps), _p(rows),
                             _code(rows, "rmsnorm_add") if rows is not None else F32, T, H, _stream()))
    return rows


def qkv_rows(qkv: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
             slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, num_heads: int, num_kv_heads: int,
             head_dim: int, value_dim: int, v_grouped: bool = False, v_other: Optional[torch.Tensor] = None,
             mix: float = 0.0, cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None, rotary_dim: int = 0,
             positions: Optional[torch.Tensor] = None) -> torch.Tensor:
    """A packed projection [T, nq d + nkv d + nkv dv] made ready for attention without rotation: RMSNorm
    over the whole q part and the whole k part (weights float32 [nq d] and [nkv d]; none: no norm), v
    blended with `v_other` ([T, nkv dv], rows may be a strided view: another layer's values of the same
    tokens) as (1 - mix) v + mix v_other, k and v into the paged cache at `slots`.  Returns q [T, nq, d].
    With `rotary_dim` r > 0 (and no norm) the pairs (c, c + r / 2) of every q and k head turn by the token's
    angles first: `cos` / `sin` float32 [positions, r / 2], `positions` int32 [T]."""
    _dev(qkv, q_weight, k_weight, slots, k_cache, v_cache, cos, sin, positions)
    rot = int(rotary_dim)
    if rot:
        if q_weight is not None or rot % 2 or not (0 < rot <= int(head_dim)):
            raise KernelError(f"qkv_rows: {rot} rotated dims of a head of {head_dim} (even, and no norm over the projection)")
        if cos is None or sin is None or positions is None or cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != rot // 2:
            raise KernelError(f"qkv_rows: the rotation's tables must be [positions, {rot // 2}]")
        _want(cos, torch.float32, "qkv_rows: cos")
        _want(sin, torch.float32, "qkv_rows: sin")
        _want(positions, torch.int32, "qkv_rows: positions")
        if positions.shape != (qkv.shape[0],):
            raise KernelError("qkv_rows: positions must be [T]")
    nq, nkv, d, dv = int(num_heads), int(num_kv_heads), int(head_dim), int(value_dim)
    if qkv.dim() != 2 or qkv.shape[1] != nq * d + nkv * d + nkv * dv:
        raise KernelError(f"qkv_rows: qkv {tuple(qkv.shape)} is not [T, {nq * d + nkv * d + nkv * dv}]")
    T = qkv.shape[0]
    _want(slots, torch.int64, "qkv_rows: slots")
    if slots.shape != (T,):
        raise KernelError("qkv_rows: slots must be [T]")
    for w, n in ((q_weight, nq * d), (k_weight, nkv * d)):
        if w is not None:
            _want(w, torch.float32, "qkv_rows: norm weight")
            if w.shape != (n,):
                raise KernelError(f"qkv_rows: norm weight {tuple(w.shape)} is not [{n}]")
    _check_cache(k_cache, v_cache, nkv, d, qkv.dtype, v_grouped, "qkv_rows", dv=dv)
    stride = 0
    if v_other is not None:
        if (not v_other.is_cuda or v_other.device != qkv.device or v_other.dtype != qkv.dtype or v_other.dim() != 2
                or tuple(v_other.shape) != (T, nkv * dv) or v_other.stride(1) != 1):
            raise KernelError(f"qkv_rows: the other values {tuple(v_other.shape)} {v_other.dtype} must be [{T}, {nkv * dv}] "
                              "rows of the projection's type")
        stride = int(v_other.stride(0))
    q_out = torch.empty((T, nq, d), dtype=qkv.dtype, device=qkv.device)
    _ok(lib().xi_qkv_rows(_p(qkv), _code(qkv, "qkv_rows"), _p(q_weight), _p(k_weight), ctypes.c_float(eps), _p(v_other),
                          ctypes.c_longlong(stride), ctypes.c_float(mix), _p(slots), _p(q_out), _p(k_cache), _p(v_cache),
                          int(k_cache.shape[2]), T, nq, nkv, d, dv, int(bool(v_grouped)), _p(cos if rot else None),
                          _p(sin if rot else None), rot, _p(positions if rot else None), _stream()))
    return q_out


def moe_route(x: torch.Tensor, router: torch.Tensor, bias: Optional[torch.Tensor], top: int, all_scores: bool = False,
              extra_rows: int = 0, sigmoid: bool = False):
    """Router of a mixture of experts: z = router @ x + bias in float32 (router float32 [E, H]), the `top`
    largest (ties: the lower index), weights = softmax over the chosen logits, or with `all_scores` the
    softmax over all experts, the chosen scores divided by their sum + 1e-20.  Returns
    (idx int32 [T, top], weights float32 [T, top]), the chosen in descending order of their logits.
    `extra_rows` X > 0: the router's last X rows are no experts but further float32 products of the same
    rows (a shared branch's gate); their results come back as a third value, float32 [T, X]."""
    _dev(x, router, bias)
    X = int(extra_rows)
    if X < 0 or X >= router.shape[0]:
        raise KernelError(f"moe_route: {X} further rows of a router of {router.shape[0]}")
    _want(router, torch.float32, "moe_route: router weight")
    if x.dim() != 2 or router.dim() != 2 or router.shape[1] != x.shape[1]:
        raise KernelError(f"moe_route: x {tuple(x.shape)} and the router {tuple(router.shape)} do not match")
    T, H = x.shape
    E = router.shape[0] - X
    if bias is not None:
        _want(bias, torch.float32, "moe_route: bias")
        if bias.shape != (E,):
            raise KernelError(f"moe_route: bias {tuple(bias.shape)} is not [{E}]")
    if not (0 < top <= min(E, 64)) or E > 1024:
        raise KernelError(f"moe_route: {top} of {E} experts (at most 64 of 1024)")
    idx = torch.empty((T, top), dtype=torch.int32, device=x.device)
    wt = torch.empty((T, top), dtype=torch.float32, device=x.device)
    extra = torch.empty((T, X), dtype=torch.float32, device=x.device) if X else None
    _ok(lib().xi_moe_route(_p(x), _code(x, "moe_route"), _p(router), _p(bias), _p(idx), _p(wt), T, H, E, int(top),
                           2 if sigmoid else int(bool(all_scores)), _p(extra), X, _stream()))
    return (idx, wt, extra) if X else (idx, wt)


MOE_GROUPED = True        # False: every step takes the experts one (token, expert) pair at a time


def moe_grouped_takes(T: int, top: int, E: int, H: int, F: int, dtype: torch.dtype, force: bool = False) -> bool:
    """Whether a step's experts go through the grouped matrix-core products: bfloat16, sizes in eights,
    and more pairs than experts (with fewer, most pairs have an expert of their own and a pair at a time
    reads no more weights, in two launches instead of four); `force`: only whether the sizes are taken."""
    if dtype != torch.bfloat16 or H % 8 or F % 8 or E > 1024 or T < 1:
        return False
    return force or (MOE_GROUPED and T * top > E)


MOE_LIBRARY_ROWS = 64     # rows an expert on average from which a step of portions takes the vendor library's products


def moe_experts_library(x: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, idx: torch.Tensor, wt: torch.Tensor,
                        act: str = "silu", gated: bool = True, weigh_input: bool = False) -> torch.Tensor:
    """`moe_experts` for steps of many tokens in bfloat16: the pairs sorted by expert on the device, the rows
    gathered in that order, and one plain product of the vendor library an expert and projection (as the
    dense feed-forward's products of many rows go to the library); the hand-written kernels do the sort,
    the activation and the combine.  Reads the experts' row counts on the host: for steps that bring
    portions, which are never recorded into a graph.  `weigh_input`: see `moe_experts` (gated experts)."""
    _dev(x, gate_up, down, idx, wt)
    T, H = x.shape
    E, F2, _ = gate_up.shape
    F, top = (F2 // 2 if gated else F2), int(idx.shape[1])
    if x.dtype != torch.bfloat16 or gate_up.dtype != torch.bfloat16 or down.dtype != torch.bfloat16:
        raise KernelError("moe_experts_library: operands must be bfloat16")
    if act not in (ACTIVATIONS if gated else UNGATED_ACTIVATIONS):
        raise KernelError(f"moe_experts_library: unknown activation {act!r}")
    if gate_up.shape != (E, (2 if gated else 1) * F, H) or down.shape != (E, H, F) or idx.shape != (T, top) or wt.shape != (T, top):
        raise KernelError("moe_experts_library: x [T, H], gate_up [E, 2F, H] (up alone: [E, F, H]), down [E, H, F], idx and weights [T, top]")
    _want(idx, torch.int32, "moe_experts_library: idx")
    _want(wt, torch.float32, "moe_experts_library: weights")
    P = T * top
    most = int(lib().xi_moe_tiles_most(P, E, 128))
    ints = torch.empty((2 * P + 3 * most + 1,), dtype=torch.int32, device=x.device)
    order, slot_of = ints[:P], ints[P:2 * P]
    _ok(lib().xi_moe_sort(_p(idx), P, E, 128, _p(order), _p(slot_of), _p(ints[2 * P:2 * P + most]),
                          _p(ints[2 * P + most:2 * P + 2 * most]), _p(ints[2 * P + 2 * most:2 * P + 3 * most]),
                          _p(ints[2 * P + 3 * most:]), _stream()))
    if weigh_input and not gated:
        raise KernelError("moe_experts_library: a weight on the input is built for gated experts")
    wt_in = wt.reshape(-1).contiguous() if weigh_input else None
    if weigh_input:
        wt = torch.ones_like(wt)
    counts = torch.bincount(idx.reshape(-1), minlength=E).tolist()          # the one read on the host
    rows = x.index_select(0, torch.div(order, top, rounding_mode="floor"))
    y = torch.empty((P, H), dtype=torch.float32, device=x.device)
    at = 0
    for e, n in enumerate(counts[:E]):
        if n:
            mid = torch.nn.functional.linear(rows[at:at + n], gate_up[e])
            if weigh_input:
                mid = act_mul(mid, act, row_scale=wt_in, row_of=order[at:at + n])
            else:
                mid = act_mul(mid, act) if gated else act_(mid, act)
            torch.mm(mid, down[e].t(), out_dtype=torch.float32, out=y[at:at + n])
            at += n
    out = torch.empty((T, H), dtype=torch.float32, device=x.device)
    _ok(lib().xi_moe_combine(_p(y), _p(slot_of), _p(wt), _p(out), T, H, top, _stream()))
    return out


def moe_experts(x: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, idx: torch.Tensor, wt: torch.Tensor,
                act: str = "silu", grouped: Optional[bool] = None, tile_rows: Optional[int] = None,
                gated: bool = True, weigh_input: bool = False) -> torch.Tensor:
    """sum over a token's chosen experts e (in the order of `idx`) of wt * down[e] @ (act(gate[e] @ x) * (up[e] @ x)):
    gate_up [E, 2F, H] (gate rows first), down [E, H, F], idx int32 / wt float32 [T, top].  Float32 [T, H].
    `gated` False: experts without a gate, wt * down[e] @ act(up[e] @ x), `gate_up` the up rows alone [E, F, H].
    One (token, expert) pair at a time, every sum in an order fixed by the sizes: the form of the
    float32 path and of steps with few tokens.  `grouped` (None: chosen by `moe_grouped_takes`): the pairs
    sorted by expert on the device and each expert's rows multiplied in tiles on the matrix cores.
    `weigh_input`: the weight multiplies the expert's input instead of its output, sum of expert_e(wt * x): it goes
    onto the float32 sums of the gate and up products, before the activation."""
    _dev(x, gate_up, down, idx, wt)
    acts = ACTIVATIONS if gated else UNGATED_ACTIVATIONS
    if act not in acts:
        raise KernelError(f"moe_experts: unknown activation {act!r}")
    if gate_up.dim() != 3 or down.dim() != 3 or x.dim() != 2:
        raise KernelError("moe_experts: x [T, H], gate_up [E, 2F, H], down [E, H, F]")
    T, H = x.shape
    E, F2, _ = gate_up.shape
    F = F2 // 2 if gated else F2
    if gate_up.shape != (E, (2 if gated else 1) * F, H) or down.shape != (E, H, F) or x.dtype != gate_up.dtype or x.dtype != down.dtype:
        raise KernelError(f"moe_experts: x {tuple(x.shape)} {x.dtype}, gate_up {tuple(gate_up.shape)} {gate_up.dtype} and "
                          f"down {tuple(down.shape)} {down.dtype} do not match")
    _want(idx, torch.int32, "moe_experts: idx")
    _want(wt, torch.float32, "moe_experts: weights")
    if idx.dim() != 2 or idx.shape[0] != T or wt.shape != idx.shape:
        raise KernelError("moe_experts: idx and weights must be [T, top]")
    top = int(idx.shape[1])
    out = torch.empty((T, H), dtype=torch.float32, device=x.device)
    wt_in = None
    if weigh_input:
        wt_in, wt = wt.contiguous(), torch.ones_like(wt)
    if grouped is None:
        grouped = moe_grouped_takes(T, top, E, H, F, x.dtype)
    if grouped:
        if not moe_grouped_takes(T, top, E, H, F, x.dtype, force=True):
            raise KernelError(f"moe_experts: the grouped form takes bfloat16 and sizes in eights, not {x.dtype} H={H} F={F}")
        P = T * top
        if tile_rows is None:                        # rows of a tile: as many as most experts fill
            tile_rows = 128 if P >= 96 * E else 64 if P >= 48 * E else 32
        bm = int(tile_rows)
        if bm not in (32, 64, 128):
            raise KernelError("moe_experts: tiles of 32, 64 or 128 rows")
        most = int(lib().xi_moe_tiles_most(P, E, bm))
        ints = torch.empty((2 * P + 3 * most + 1,), dtype=torch.int32, device=x.device)
        order, slot_of = ints[:P], ints[P:2 * P]
        t_e, t_r0, t_n, n_tiles = (ints[2 * P:2 * P + most], ints[2 * P + most:2 * P + 2 * most],
                                   ints[2 * P + 2 * most:2 * P + 3 * most], ints[2 * P + 3 * most:])
        _ok(lib().xi_moe_sort(_p(idx), P, E, bm, _p(order), _p(slot_of), _p(t_e), _p(t_r0), _p(t_n), _p(n_tiles), _stream()))
        mid = torch.empty((P, F), dtype=torch.bfloat16, device=x.device)
        _ok(lib().xi_moe_group(_p(x), _p(order), top, _p(gate_up), _p(t_e), _p(t_r0), _p(t_n), _p(n_tiles), most, _p(mid),
                               F, H, bm, 1 if gated else 2, acts[act], _p(wt_in), _stream()))
        y = torch.empty((P, H), dtype=torch.float32, device=x.device)
        _ok(lib().xi_moe_group(_p(mid), _p(order), top, _p(down), _p(t_e), _p(t_r0), _p(t_n), _p(n_tiles), most, _p(y),
                               H, F, bm, 0, 0, None, _stream()))
        _ok(lib().xi_moe_combine(_p(y), _p(slot_of), _p(wt), _p(out), T, H, top, _stream()))
        return out
    mid = torch.empty((T * top, F), dtype=x.dtype, device=x.device)
    code = _code(x, "moe_experts")
    _ok(lib().xi_moe_gate_up(_p(x), _p(gate_up), _p(idx), _p(mid), code, acts[act], int(bool(gated)), T, H, F, E, top, _p(wt_in),
                             _stream()))
    _ok(lib().xi_moe_down(_p(mid), _p(down), _p(idx), _p(wt), _p(out), code, T, H, F, E, top, _stream()))
    return out


def qk_norm_rope_kv(qkv: torch.Tensor, q_weight: Optional[torch.Tensor],
                    k_weight: Optional[torch.Tensor], eps: float, cos: torch.Tensor,
                    sin: torch.Tensor, rotary_dim: int, interleaved: bool,
                    positions: torch.Tensor, slots: torch.Tensor, k_cache: torch.Tensor,
                    v_cache: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                    q_out: Optional[torch.Tensor] = None, v_grouped: bool = False,
                    vector_min_tokens: int = 128, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Per-head RMSNorm of q and k (if weights are given), rotation by position, q to q_out
    [T, nq, d], k and v into the paged cache [pages, nkv, page_size, d] at `slots`; with
    `v_grouped` the V pool is [pages, nkv, page_size / 8, d, 8] (eight keys side by side for every
    dim: what the matrix-core attention reads).  From `vector_min_tokens` tokens
    on, bfloat16 with the grouped pool runs the vectorized kernel.  `bias` (float32, one
    value per element of a packed row) is added to the rows first, in float32.  `qkv` may be a
    stack [slices, T, width] of float32 partial sums (`linear_mid`), added here in slice order;
    q and the cache then have the cache's dtype and the form of one wave per head runs."""
    _dev(qkv, q_weight, k_weight, cos, sin, positions, slots, k_cache, v_cache, q_out, bias)
    nq, nkv, d = num_heads, num_kv_heads, head_dim
    slices, dtype = 0, qkv.dtype
    if qkv.dim() == 3:            # float32 partial sums [slices, T, width] of a product cut along K
        _want(qkv, torch.float32, "qk_norm_rope_kv: partial sums")
        slices, dtype = int(qkv.shape[0]), k_cache.dtype
        if not (0 < slices <= 64) or not qkv.is_contiguous():
            raise KernelError(f"qk_norm_rope_kv: partial sums {tuple(qkv.shape)} must be contiguous [1..64, T, width]")
    T = qkv.shape[-2]
    if qkv.dim() not in (2, 3) or qkv.shape[-1] != (nq + 2 * nkv) * d:
        raise KernelError(f"qk_norm_rope_kv: qkv {tuple(qkv.shape)} is not [T, {(nq + 2 * nkv) * d}]")
    _want(positions, torch.int32, "qk_norm_rope_kv: positions")
    _want(slots, torch.int64, "qk_norm_rope_kv: slots")
    _want(cos, torch.float32, "qk_norm_rope_kv: cos")
    _want(sin, torch.float32, "qk_norm_rope_kv: sin")
    if positions.shape != (T,) or slots.shape != (T,):
        raise KernelError("qk_norm_rope_kv: positions and slots must be [T]")
    if cos.dim() != 2 or cos.shape[1] != rotary_dim // 2 or sin.shape != cos.shape:
        raise KernelError(f"qk_norm_rope_kv: cos/sin {tuple(cos.shape)} are not [positions, {rotary_dim // 2}]")
    for w in (q_weight, k_weight):
        if w is not None:
            _want(w, torch.float32, "qk_norm_rope_kv: norm weight")
            if w.shape != (d,):
                raise KernelError("qk_norm_rope_kv: norm weight must be [head_dim]")
    if bias is not None:
        _want(bias, torch.float32, "qk_norm_rope_kv: bias")
        if bias.shape != (qkv.shape[-1],):
            raise KernelError(f"qk_norm_rope_kv: bias {tuple(bias.shape)} is not [{qkv.shape[-1]}]")
    _check_cache(k_cache, v_cache, nkv, d, dtype, v_grouped, "qk_norm_rope_kv")
    if q_out is None:
        q_out = torch.empty((T, nq, d), dtype=dtype, device=qkv.device)
    elif q_out.shape != (T, nq, d) or q_out.dtype != dtype:
        raise KernelError("qk_norm_rope_kv: q_out has the wrong shape or dtype")
    _ok(lib().xi_qk_norm_rope_kv(
        _p(qkv), _code(q_out, "qk_norm_rope_kv"), slices, _p(bias), _p(q_weight), _p(k_weight), ctypes.c_float(eps),
        _p(cos), _p(sin), int(rotary_dim), int(bool(interleaved)), _p(positions), _p(slots),
        _p(q_out), _p(k_cache), _p(v_cache), int(k_cache.shape[2]), T, nq, nkv, d,
        int(bool(v_grouped)), int(vector_min_tokens), _stream()))
    return q_out


def _check_cache(k_cache, v_cache, nkv, d, dtype, v_grouped, what, dv=None, key_heads=None):
    """K pool [pages, nkv, page, d]; V pool [pages, nkv, page, dv], or [pages, nkv, page / 8, dv, 8] if in
    groups of eight keys (dv: the value head size, d unless given; `key_heads`: the K pool's heads where they are
    not the V pool's)."""
    dv = d if dv is None else int(dv)
    nkk = nkv if key_heads is None else int(key_heads)
    if k_cache.dim() != 4 or k_cache.shape[1] != nkk or k_cache.shape[3] != d or k_cache.dtype != dtype:
        raise KernelError(f"{what}: K pool {tuple(k_cache.shape)} {k_cache.dtype} does not match "
                          f"[pages, {nkk}, page_size, {d}] {dtype}")
    pages, _, page, _ = k_cache.shape
    if v_grouped and page % 8:
        raise KernelError(f"{what}: V in groups of eight keys needs pages of a multiple of 8 tokens, not {page}")
    want = (pages, nkv, page // 8, dv, 8) if v_grouped else (pages, nkv, page, dv)
    if tuple(v_cache.shape) != want or v_cache.dtype != dtype:
        raise KernelError(f"{what}: V pool {tuple(v_cache.shape)} {v_cache.dtype} does not match {want} {dtype}")


def attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_tables: torch.Tensor, tok_seq: torch.Tensor, positions: torch.Tensor,
                      scale: float, window: int = 0, out: Optional[torch.Tensor] = None,
                      v_grouped: bool = False, softcap: float = 0.0,
                      slopes: Optional[torch.Tensor] = None, sinks: Optional[torch.Tensor] = None,
                      value_dim: Optional[int] = None) -> torch.Tensor:
    """Causal paged GQA attention for any mix of tokens.  q [T, nq, d]; caches
    [pages, nkv, page_size, d] (the V pool's last size, the value head size, may differ);
    block_tables int32 [B, max_pages]; tok_seq / positions
    int32 [T] name each token's row of block_tables and its absolute position.
    window = 0 keeps all keys, w > 0 the last w (the query's own key included).
    `softcap` c > 0: scores become c * tanh(score / c); `slopes` float32 [nq]: head h's scores lose
    slopes[h] * (distance from the query to the key); `sinks` float32 [nq]: head h's softmax has exp(sinks[h]) in
    its denominator beside the keys' weights.  `v_cache` None: a key's first `value_dim` dims are its value (one
    pool for both: attention over a latent)."""
    _dev(q, k_cache, v_cache, block_tables, tok_seq, positions, out, slopes, sinks)
    if q.dim() != 3:
        raise KernelError("attention: q must be [T, nq, d]")
    T, nq, d = q.shape
    if k_cache.dim() != 4:
        raise KernelError("attention: the K pool must be [pages, nkv, page_size, d]")
    nkk, page = int(k_cache.shape[1]), k_cache.shape[2]
    nkv = nkk if v_cache is None else int(v_cache.shape[1])       # the K pool may hold fewer heads than the V pool
    if nkk <= 0 or nkv <= 0 or nq % nkk or nq % nkv:
        raise KernelError(f"attention: {nq} query heads on {nkk} key heads and {nkv} value heads")
    if v_cache is None:
        dv = int(value_dim or 0)
        if not (0 < dv <= d) or v_grouped or k_cache.shape[3] != d or k_cache.dtype != q.dtype:
            raise KernelError(f"attention: values inside the keys need 0 < value_dim <= {d} and a pool [pages, nkv, page, {d}]")
    else:
        dv = int(v_cache.shape[3])
        _check_cache(k_cache, v_cache, nkv, d, q.dtype, v_grouped, "attention", dv=dv, key_heads=nkk)
    if sinks is not None:
        _want(sinks, torch.float32, "attention: sinks")
        if sinks.shape != (nq,):
            raise KernelError(f"attention: sinks {tuple(sinks.shape)} must be one a query head, [{nq}]")
    for t, name in ((block_tables, "block_tables"), (tok_seq, "tok_seq"), (positions, "positions")):
        _want(t, torch.int32, f"attention: {name}")
    if block_tables.dim() != 2 or tok_seq.shape != (T,) or positions.shape != (T,):
        raise KernelError("attention: block_tables must be [B, max_pages], tok_seq and positions [T]")
    if slopes is not None:
        _want(slopes, torch.float32, "attention: slopes")
        if slopes.shape != (nq,):
            raise KernelError(f"attention: slopes {tuple(slopes.shape)} must be one a query head, [{nq}]")
    if not softcap >= 0:
        raise KernelError(f"attention: the soft cap must be positive (0: none), got {softcap}")
    if out is None:
        out = torch.empty((T, nq * dv), dtype=q.dtype, device=q.device)
    elif out.shape != (T, nq * dv) or out.dtype != q.dtype:
        raise KernelError("attention: out has the wrong shape or dtype")
    _ok(lib().xi_attention_generic(
        _p(q), _p(k_cache), _p(v_cache), _code(q, "attention"), _p(block_tables),
        int(block_tables.shape[1]), _p(tok_seq), _p(positions), _p(out), ctypes.c_float(scale),
        int(window), int(page), T, nq, nkv, d, dv, int(bool(v_grouped)), ctypes.c_float(softcap), _p(slopes), _p(sinks),
        int(v_cache is None), nkk, _stream()))
    return out


def gemm_tn(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
            out: Optional[torch.Tensor] = None, accumulate: bool = False) -> torch.Tensor:
    """y = x @ w.T with x [M, K], w [N, K]; float32 accumulation in ascending k.
    `accumulate` adds the product to `out` instead of overwriting it."""
    _dev(x, w, out)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"gemm: x {tuple(x.shape)} and w {tuple(w.shape)} do not match")
    if x.dtype != w.dtype:
        raise KernelError(f"gemm: x is {x.dtype} but w is {w.dtype}")
    M, K = x.shape
    N = w.shape[0]
    if out is None:
        if accumulate:
            raise KernelError("gemm: accumulate needs an output to add to")
        out = torch.empty((M, N), dtype=out_dtype or x.dtype, device=x.device)
    elif out.shape != (M, N) or (out_dtype is not None and out.dtype != out_dtype):
        raise KernelError("gemm: out has the wrong shape or dtype")
    _ok(lib().xi_gemm_tn(_p(x), _p(w), _p(out), M, N, K, _code(x, "gemm"), _code(out, "gemm"),
                         int(bool(accumulate)), _stream()))
    return out


DECODE_WORKGROUPS = 512             # workgroups of the split-K decode kernel a launch of mixed lengths aims at: two a compute unit
DECODE_KEYS_LEAST = 128             # keys of a workgroup: from one 32-key step a wave
DECODE_KEYS_MOST = 512              # to four, in batches of mixed lengths
DECODE_WORKGROUP_KEYS = 32          # what a workgroup costs beyond its keys (start, page numbers, merge, partial results), in keys
DECODE_SPLITS_MOST = 1024           # splits of a sequence that the search below tries
DECODE_WHOLE_KEYS = 2048            # mixed lengths, one and a half pairs a compute unit and more: a workgroup's keys at most


def decode_keys_per_workgroup(pairs: int, span: int, similar: bool = False) -> int:
    return _decode_keys_per_workgroup(int(pairs), int(span), bool(similar))


@functools.lru_cache(maxsize=4096)
def _decode_keys_per_workgroup(pairs: int, span: int, similar: bool) -> int:
    """Keys per workgroup of the split-K decode kernel for `pairs` (sequence, kv head) pairs of
    up to `span` keys (a multiple of 128; more than `span`: a workgroup takes a whole sequence and
    there is no second kernel).

    `similar` (the sequences are about equally long): the number of splits s that makes the least
    of rounds(s) * (keys of a split + DECODE_WORKGROUP_KEYS), rounds(s) = ceil(pairs * s /
    compute units): the compute units take the workgroups in turn, so the launch lasts as long
    as the unit with the most of them, and a workgroup costs about 32 keys' time beyond its keys.
    One round of large chunks wins where it exists (8 sequences of 4,096 keys on 8 kv heads: 4
    splits, 31.7 us against 32.2 at 8 and 33.8 at 16; 16 sequences of 8,500 keys, 64 query heads:
    2 splits, 104 us against 121 at 17; one sequence of 4,096: 32 splits of 128 keys, 11.2 us
    against 13.0 at 16), whole sequences from 256 pairs on.

    Otherwise (mixed lengths): 128, 256 or 512 keys, whichever makes about DECODE_WORKGROUPS
    workgroups: larger chunks lose there (64 sequences of 256 to 2,304 keys: 75 us at 512, 81 at
    1,024), since the short sequences' workgroups end early and the long ones' run on.  From one
    and a half pairs a compute unit on there are enough workgroups to even that out (the scheduler
    puts the long sequences first), and a workgroup's start and end cost more than the chunks'
    balance gains: whole sequences up to DECODE_WHOLE_KEYS keys, chunks of that many beyond (192
    sequences of 100 to 768 keys, longest first: 64 us against 72 in chunks of 512, and 80 in chunks
    of 512 in random order; 64 of 256 to 2,304: 64 against 68; 48 of 100 to 768: 20.5 against 21.9);
    from one pair a compute unit on chunks of 1,024 (32 sequences of 500 to 4,000: 60 us against 65
    at 512 and 63 whole)."""
    if similar:
        chunks = max(1, -(-int(span) // 128))
        plans = []
        for s in range(1, min(chunks, DECODE_SPLITS_MOST) + 1):
            kpw = -(-chunks // s) * 128
            splits = -(-chunks * 128 // kpw)
            cost = -(-pairs * splits // COMPUTE_UNITS) * (kpw + DECODE_WORKGROUP_KEYS)
            plans.append((cost, kpw, splits))
        # a workgroup alone on its compute unit does not draw the unit's share of the memory
        # bandwidth: with workgroups for fewer than seven eighths of the units more, smaller ones are
        # ahead (one sequence of 8,704 keys: 16.8 us in 544 workgroups of 128 keys, 18.9 in 184 of
        # 384; three of them: 27.4 us in 240 workgroups of 896 keys, 30.5 in 408 of 512)
        filling = [p for p in plans if pairs * p[2] >= COMPUTE_UNITS * 7 // 8]
        best = min(filling or [max(plans, key=lambda p: p[2])], key=lambda p: (p[0], -p[1]))
        if best[2] == 1:
            return (span + 128) // 128 * 128          # more than span: one split
        return best[1]
    if 2 * pairs >= 3 * COMPUTE_UNITS:
        return (span + 128) // 128 * 128 if span <= DECODE_WHOLE_KEYS else DECODE_WHOLE_KEYS
    if pairs >= COMPUTE_UNITS and span > 1024:
        return 1024
    kpw = DECODE_KEYS_LEAST
    while kpw < DECODE_KEYS_MOST and pairs * span >= 2 * kpw * DECODE_WORKGROUPS:
        kpw *= 2
    return kpw


def mfma_attention_supported(nq: int, nkv: int, d: int, page: int) -> bool:
    return bool(lib().xi_attention_mfma_supported(nq, nkv, d, page))


def decode_attention_takes(nq: int, nkv: int, d: int) -> bool:
    """Whether the split-K decode kernel takes these head counts and this head size: up to 16 query
    heads per kv head (the columns of one tile), and the waves' partial results of a group must
    fit the LDS through which they are merged."""
    g = nq // nkv
    return g <= 16 and (4 * g * d + 8 * g) * 4 <= 64 * 1024


def attention_prefill_bf16(q, k_cache, vt_cache, block_tables, tiles, cu_q, ctx_lens, scale, window=0, out=None,
                           small=False):
    """MFMA attention for any mix of portions.  tiles int32 [n, 2] = (sequence, first query
    token of a block of `prefill_block(d, nq // nkv, small)` tokens within the sequence's
    portion); `small` selects the workgroup shape (see `prefill_tiles`): 0 eight waves, 1 four
    waves and half the block, 2 (head sizes 32, 64, 128, 256) eight waves in two groups that split
    a tile's keys, the block of shape 1."""
    _dev(q, k_cache, vt_cache, block_tables, tiles, cu_q, ctx_lens, out)
    T, nq, d = q.shape
    nkv, page = k_cache.shape[1], k_cache.shape[2]
    _want(q, torch.bfloat16, "attention_prefill: q")
    _check_cache(k_cache, vt_cache, nkv, d, torch.bfloat16, True, "attention_prefill")
    for t, name in ((block_tables, "block_tables"), (tiles, "tiles"), (cu_q, "cu_q"), (ctx_lens, "ctx_lens")):
        _want(t, torch.int32, f"attention_prefill: {name}")
    B = ctx_lens.shape[0]
    if block_tables.shape[0] != B or cu_q.shape != (B + 1,) or tiles.dim() != 2 or tiles.shape[1] != 2:
        raise KernelError("attention_prefill: block_tables [B, pages], cu_q [B+1], ctx_lens [B], tiles [n, 2] expected")
    if out is None:
        out = torch.empty((T, nq * d), dtype=q.dtype, device=q.device)
    # head sizes 32, 64, 128, 256: the kernel whose tiles reach LDS through a ring of direct loads
    ring = PREFILL_RING and prefill_ring_supported(d)
    if int(small) == 2 and not ring:
        raise KernelError(f"attention_prefill: the shape of two groups of waves needs a head size of 32, 64, 128 or 256, got {d}")
    entry = lib().xi_attention_prefill_ring_bf16 if ring else lib().xi_attention_prefill_bf16
    _ok(entry(
        _p(q), _p(k_cache), _p(vt_cache), _p(block_tables), int(block_tables.shape[1]), _p(tiles),
        int(tiles.shape[0]), _p(cu_q), _p(ctx_lens), _p(out), ctypes.c_float(scale), int(window), int(page),
        nq, nkv, d, int(small), _stream()))
    return out


PREFILL_RING = True       # False: every head size goes to the kernel that copies tiles through registers


def prefill_ring_supported(d: int) -> bool:
    return bool(lib().xi_attention_prefill_ring_supported(int(d)))


def prefill_block(d: int, group: int = 1, small: bool = False) -> int:
    """Query positions per workgroup of the prefill kernel for a head size, a number of
    query heads per kv head and a workgroup shape."""
    return int(lib().xi_attention_prefill_block(int(d), int(group), int(small)))


COMPUTE_UNITS = 256
MIXED_DECODE_FROM = 4          # single-token sequences at the head of a mixed batch from which they may go to the decode
MIXED_DECODE_WORK = 40_000     # kernel: where sequences x longest context x reads of a kv head's keys reach this,
MIXED_DECODE_CONTEXT = 4096    # or the longest context this (measured on MI355X beside a portion of 2,000 tokens:
                               # 40 query heads on 8 kv heads, 64 sequences at 1,500 keys: 450 -> 155 us a layer)


def prefill_tiles(q_lens, ctx_lens, d: int, nq: int, nkv: int, small=None, first_seq: int = 0, block_of=None):
    """The query blocks of a batch of portions for the prefill kernel: (rows, shape).
    rows = [(sequence, first query of the block)] in launch order.  A block's work grows
    with the keys it sees, and the compute units take workgroups in launch order, so the
    blocks are sorted by work and laid out in a zigzag over rounds of one workgroup per
    compute unit.  The shape (chosen here unless given) is 0, eight waves and the full block,
    where that makes two workgroups a compute unit or more; with fewer blocks 1, four waves and
    half the block: twice the workgroups, two of them resident on a compute unit, and the
    zigzag gives a unit that got a long block in the first round a short one in the second; and
    with so few blocks that even those leave compute units with one workgroup (a prompt of 2,048
    tokens on 8 kv heads) 2, where the head size allows: eight waves in two groups that split a
    tile's keys, so that the longest block, which ends up alone on its unit, walks its keys with
    twice the waves (2,048 tokens, 32 query heads: 60 -> 56 us; 1,024: 31 -> 28).  Shape 0 has one
    workgroup per unit at a time: longest first."""
    g = nq // nkv
    heads = nkv * (g // (4 if g % 4 == 0 else 2 if g % 2 == 0 else 1))     # workgroups per query block
    two_groups = block_of is None          # (`block_of(small)`: another kernel's block sizes, shapes 0 and 1 only)
    if block_of is None:
        block_of = lambda shape: prefill_block(d, g, shape)
    big = block_of(0)
    if small is None:
        blocks = sum(-(-n // big) for n in q_lens[first_seq:])
        small = 0 if blocks * heads >= 2 * COMPUTE_UNITS else 1
        if small and two_groups and PREFILL_RING and prefill_ring_supported(d):
            half = block_of(1)
            if sum(-(-n // half) for n in q_lens[first_seq:]) * heads <= 2 * COMPUTE_UNITS:
                small = 2
    small = int(small)
    qb = block_of(small)
    rows = [(b, q0) for b, n in enumerate(q_lens) if b >= first_seq for q0 in range(0, n, qb)]
    rows.sort(key=lambda t: -(ctx_lens[t[0]] - q_lens[t[0]] + t[1]))
    per_round = max(1, COMPUTE_UNITS // heads)
    out = []
    for i in range(0, len(rows), per_round):
        chunk = rows[i:i + per_round]
        out += chunk if (small != 1 or (i // per_round) % 2 == 0) else chunk[::-1]
    return out, small


BIASED_MFMA = True        # False: scores with options go to the generic kernel in bfloat16 too
HEAD_ROWS_FROM = 4        # query heads on one kv head from which a step of single tokens makes them the rows of a block


def attention_biased_supported(nq: int, nkv: int, d: int, dv: int, page: int) -> bool:
    return bool(lib().xi_attention_biased_supported(int(nq), int(nkv), int(d), int(dv), int(page)))


def attention_biased_block(d: int, dv: int, group: int = 1, small: int = 0) -> int:
    """Query positions per workgroup of `attention_biased_bf16` for the two head sizes, a number of
    query heads per kv head and a workgroup shape (0: eight waves, 1: four)."""
    return int(lib().xi_attention_biased_block(int(d), int(dv), int(group), int(small)))


BIASED_SPLIT_WORKGROUPS = 512     # workgroups a launch of single tokens aims at (two a compute unit)
BIASED_SPLIT_KEYS_LEAST = 128     # keys of a slice at least


def biased_split_keys(workgroups: int, span: int) -> int:
    """Keys a slice (a multiple of 64; 0: no slices) for a step of single tokens that would make `workgroups`
    workgroups, each walking up to `span` keys: slices until the launch has about BIASED_SPLIT_WORKGROUPS."""
    want = BIASED_SPLIT_WORKGROUPS // max(1, int(workgroups))
    most = int(span) // BIASED_SPLIT_KEYS_LEAST
    splits = min(want, most)
    if splits < 2:
        return 0
    return -(-int(span) // splits // 64) * 64


def attention_biased_bf16(q, k_cache, vt_cache, block_tables, tiles, cu_q, ctx_lens, scale, window=0, softcap=0.0,
                          slopes=None, out=None, small=0, split_keys=0, span=0, sinks=None, rows_heads=0):
    """Matrix-core attention for any mix of portions with the score's options (`softcap`, `slopes`: see
    `attention_generic`; `sinks` as there) and a value head size of its own: q [T, nq, d], K pool [pages, nkv, page, d], V pool
    [pages, nkv, page / 8, dv, 8]; tiles int32 [n, 2] = (sequence, first query token of a block of
    `attention_biased_block(d, dv, nq // nkv, small)` tokens within the sequence's portion).  Returns [T, nq * dv].
    `split_keys` > 0 (steps in which every sequence brings one token, a tile a token): each workgroup walks one slice
    of that many keys of the up to `span` a token sees, and a second kernel puts the slices together.
    `rows_heads` H > 0 (one kv head, single tokens): q is [tokens * H, 1, d], a sequence's H rows are the query heads
    of its one new token, all at its last position, `cu_q` counts rows, `sinks` is [H] and blocks may hold many rows.
    The V pool may then have G > 1 heads beside the one key head: rows h H / G .. (h + 1) H / G - 1 read value head h, and
    no block of `tiles` may cross such a border."""
    _dev(q, k_cache, vt_cache, block_tables, tiles, cu_q, ctx_lens, out, slopes, sinks)
    T, nq, d = q.shape
    nkk, nkv, page, dv = int(k_cache.shape[1]), int(vt_cache.shape[1]), k_cache.shape[2], int(vt_cache.shape[3])
    if nkk <= 0 or nkv % nkk:
        raise KernelError(f"attention_biased: {nkv} kv heads on {nkk} key heads")
    rows_kv = 1
    if rows_heads and nkk == 1 and nkv > 1:         # heads as rows over one key head and several value heads
        if int(rows_heads) % nkv:
            raise KernelError(f"attention_biased: {rows_heads} heads as rows on {nkv} value heads")
        rows_kv, nkv = nkv, 1
    _want(q, torch.bfloat16, "attention_biased: q")
    if sinks is not None:
        _want(sinks, torch.float32, "attention_biased: sinks")
        if sinks.shape != (int(rows_heads) or nq,):
            raise KernelError(f"attention_biased: sinks {tuple(sinks.shape)} must be one a query head, [{int(rows_heads) or nq}]")
    if rows_heads and (nq != 1 or nkv != 1 or slopes is not None or T % int(rows_heads)):
        raise KernelError("attention_biased: rows that are a token's heads come with one head, no slopes and whole tokens")
    _check_cache(k_cache, vt_cache, nkv * rows_kv, d, torch.bfloat16, True, "attention_biased", dv=dv, key_heads=nkk)
    for t, name in ((block_tables, "block_tables"), (tiles, "tiles"), (cu_q, "cu_q"), (ctx_lens, "ctx_lens")):
        _want(t, torch.int32, f"attention_biased: {name}")
    B = ctx_lens.shape[0]
    if block_tables.dim() != 2 or block_tables.shape[0] != B or cu_q.shape != (B + 1,) or tiles.dim() != 2 or tiles.shape[1] != 2:
        raise KernelError("attention_biased: block_tables [B, pages], cu_q [B+1], ctx_lens [B], tiles [n, 2] expected")
    if not attention_biased_supported(nq, nkv, d, dv, page):
        raise KernelError(f"attention_biased: sizes nq={nq} nkv={nkv} d={d} dv={dv} page={page} are not taken")
    if slopes is not None:
        _want(slopes, torch.float32, "attention_biased: slopes")
        if slopes.shape != (nq,):
            raise KernelError(f"attention_biased: slopes {tuple(slopes.shape)} must be one a query head, [{nq}]")
    if int(small) not in (0, 1) or not softcap >= 0:
        raise KernelError("attention_biased: the shape is 0 or 1, the soft cap positive or 0")
    if out is None:
        out = torch.empty((T, nq * dv), dtype=q.dtype, device=q.device)
    elif out.shape != (T, nq * dv) or out.dtype != q.dtype:
        raise KernelError("attention_biased: out has the wrong shape or dtype")
    part_o = part_ml = None
    max_splits = 0
    if split_keys:
        if split_keys % 64 or split_keys < 0 or span <= 0 or (not rows_heads and (tiles.shape[0] != T or B != T)) or (
                rows_heads and B * int(rows_heads) != T):
            raise KernelError("attention_biased: slices are multiples of 64 keys, for steps of single tokens with a tile each")
        max_splits = (int(span) + 63) // int(split_keys) + 1
        part_o = torch.empty((T, nq, max_splits, dv), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T, nq, max_splits, 2), dtype=torch.float32, device=q.device)
    _ok(lib().xi_attention_biased_bf16(
        _p(q), _p(k_cache), _p(vt_cache), _p(block_tables), int(block_tables.shape[1]), _p(tiles), int(tiles.shape[0]),
        _p(cu_q), _p(ctx_lens), _p(out), ctypes.c_float(scale), ctypes.c_float(softcap), _p(slopes), _p(sinks), int(window),
        int(page), nq, nkv, d, dv, int(small), _p(part_o), _p(part_ml), int(split_keys), int(max_splits), int(T), int(rows_heads),
        nkk, rows_kv, _stream()))
    return out


def attention_decode_bf16(q, k_cache, vt_cache, block_tables, ctx_lens, max_ctx_len, scale, window=0, out=None,
                          keys_per_workgroup=None, similar=False):
    """Split-K MFMA attention for a batch in which every sequence has one token (q [B, nq, d]).
    `keys_per_workgroup` (a multiple of 128) is chosen from the batch if not given (`similar`:
    see `decode_keys_per_workgroup`)."""
    _dev(q, k_cache, vt_cache, block_tables, ctx_lens, out)
    B, nq, d = q.shape
    nkv, page = k_cache.shape[1], k_cache.shape[2]
    _want(q, torch.bfloat16, "attention_decode: q")
    _check_cache(k_cache, vt_cache, nkv, d, torch.bfloat16, True, "attention_decode")
    _want(block_tables, torch.int32, "attention_decode: block_tables")
    _want(ctx_lens, torch.int32, "attention_decode: ctx_lens")
    if block_tables.shape[0] != B or ctx_lens.shape != (B,):
        raise KernelError("attention_decode: one block table row and one context length per sequence")
    span = min(int(max_ctx_len), int(window) + 31) if window > 0 else int(max_ctx_len)
    kpw = int(keys_per_workgroup or decode_keys_per_workgroup(B * nkv, span, similar))
    max_splits = span // kpw + 1
    part_o = torch.empty((B, nq, max_splits, d), dtype=torch.float32, device=q.device)
    part_ml = torch.empty((B, nq, max_splits, 2), dtype=torch.float32, device=q.device)
    if out is None:
        out = torch.empty((B, nq * d), dtype=q.dtype, device=q.device)
    _ok(lib().xi_attention_decode_bf16(
        _p(q), _p(k_cache), _p(vt_cache), _p(block_tables), int(block_tables.shape[1]), _p(ctx_lens), _p(out),
        _p(part_o), _p(part_ml), max_splits, kpw, ctypes.c_float(scale), int(window), int(page), B, nq, nkv, d,
        _stream()))
    return out


def attention_decode_packed_bf16(qkv, q_weight, k_weight, eps, cos, sin, rotary_dim, interleaved, positions, slots,
                                 k_cache, vt_cache, block_tables, ctx_lens, max_ctx_len, num_heads, scale, window=0,
                                 bias=None, out=None, keys_per_workgroup=None, similar=False):
    """What `qk_norm_rope_kv` and `attention_decode_bf16` do one after the other for a batch in which
    every sequence has one token, in one launch less: `qkv` is the packed projection
    [B, (nq + 2 nkv) d] in bfloat16, or a stack [slices, B, width] of float32 partial sums; the new
    keys and values go into the cache at `slots` on the way (the same bits as the other kernel's)."""
    _dev(qkv, q_weight, k_weight, cos, sin, positions, slots, k_cache, vt_cache, block_tables, ctx_lens, out, bias)
    nq, nkv, page, d = int(num_heads), k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    slices = 0
    if qkv.dim() == 3:
        _want(qkv, torch.float32, "attention_decode_packed: partial sums")
        slices = int(qkv.shape[0])
        if not (0 < slices <= 64):
            raise KernelError(f"attention_decode_packed: {slices} slices of partial sums, at most 64")
    else:
        _want(qkv, torch.bfloat16, "attention_decode_packed: qkv")
    if qkv.dim() not in (2, 3) or qkv.shape[-1] != (nq + 2 * nkv) * d:
        raise KernelError(f"attention_decode_packed: qkv {tuple(qkv.shape)} is not [B, {(nq + 2 * nkv) * d}]")
    B = int(qkv.shape[-2])
    _check_cache(k_cache, vt_cache, nkv, d, torch.bfloat16, True, "attention_decode_packed")
    _want(block_tables, torch.int32, "attention_decode_packed: block_tables")
    _want(ctx_lens, torch.int32, "attention_decode_packed: ctx_lens")
    _want(positions, torch.int32, "attention_decode_packed: positions")
    _want(slots, torch.int64, "attention_decode_packed: slots")
    _want(cos, torch.float32, "attention_decode_packed: cos")
    _want(sin, torch.float32, "attention_decode_packed: sin")
    if block_tables.shape[0] != B or ctx_lens.shape != (B,) or positions.shape != (B,) or slots.shape != (B,):
        raise KernelError("attention_decode_packed: one block table row, context length, position and slot per sequence")
    if cos.dim() != 2 or cos.shape[1] != rotary_dim // 2 or sin.shape != cos.shape:
        raise KernelError(f"attention_decode_packed: cos/sin {tuple(cos.shape)} are not [positions, {rotary_dim // 2}]")
    for w in (q_weight, k_weight):
        if w is not None:
            _want(w, torch.float32, "attention_decode_packed: norm weight")
            if w.shape != (d,):
                raise KernelError("attention_decode_packed: norm weight must be [head_dim]")
    if bias is not None:
        _want(bias, torch.float32, "attention_decode_packed: bias")
        if bias.shape != (qkv.shape[-1],):
            raise KernelError(f"attention_decode_packed: bias {tuple(bias.shape)} is not [{qkv.shape[-1]}]")
    span = min(int(max_ctx_len), int(window) + 31) if window > 0 else int(max_ctx_len)
    kpw = int(keys_per_workgroup or decode_keys_per_workgroup(B * nkv, span, similar))
    max_splits = span // kpw + 1
    part_o = torch.empty((B, nq, max_splits, d), dtype=torch.float32, device=qkv.device)
    part_ml = torch.empty((B, nq, max_splits, 2), dtype=torch.float32, device=qkv.device)
    if out is None:
        out = torch.empty((B, nq * d), dtype=torch.bfloat16, device=qkv.device)
    elif out.shape != (B, nq * d) or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise KernelError("attention_decode_packed: out has the wrong shape or dtype")
    _ok(lib().xi_attention_decode_packed_bf16(
        _p(qkv), slices, _p(bias), _p(q_weight), _p(k_weight), ctypes.c_float(eps), _p(cos), _p(sin), int(rotary_dim),
        int(bool(interleaved)), _p(positions), _p(slots), _p(k_cache), _p(vt_cache), _p(block_tables),
        int(block_tables.shape[1]), _p(ctx_lens), _p(out), _p(part_o), _p(part_ml), max_splits, kpw,
        ctypes.c_float(scale), int(window), int(page), B, nq, nkv, d, _stream()))
    return out


def attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, ctx, group: int,
              scale: float, window: int = 0, v_grouped: bool = False, softcap: float = 0.0,
              slopes: Optional[torch.Tensor] = None, sinks: Optional[torch.Tensor] = None,
              value_dim: Optional[int] = None) -> torch.Tensor:
    """Attention of one step's tokens over the paged cache of `group`; chooses the kernel
    from the precision and the shape of the batch: float32, or sizes the matrix-core
    kernels do not take, go to the generic kernel; bfloat16 batches of single tokens to
    the split-K decode kernel; everything else to the prefill kernel.  Scores with a soft cap
    or a distance bias, a softmax with sinks, and values of another head size than the keys, have
    matrix-core kernels of their own (`attention_biased_bf16`).  `v_cache` None: a key's first
    `value_dim` dims are its value, which only the generic kernel reads that way."""
    T, nq, d = q.shape
    nkk, page = int(k_cache.shape[1]), k_cache.shape[2]
    nkv = nkk if v_cache is None else int(v_cache.shape[1])      # the K pool may hold fewer heads (see `attention_generic`)
    bt = ctx.block_tables[group]
    if v_cache is None:
        return attention_generic(q, k_cache, None, bt, ctx.tok_seq, ctx.positions, scale, window, softcap=softcap,
                                 slopes=slopes, sinks=sinks, value_dim=value_dim)
    if softcap > 0 or slopes is not None or sinks is not None or v_cache.shape[3] != d or nkk != nkv:
        dv = int(v_cache.shape[3])
        if q.dtype == torch.bfloat16 and v_grouped and BIASED_MFMA and attention_biased_supported(nq, nkv, d, dv, page):
            if (ctx.max_q_len == 1 and nkk == 1 and nkv > 1 and nq // nkv >= HEAD_ROWS_FROM and slopes is None and sinks is None
                    and q.is_contiguous()):
                # single tokens whose heads all read the one key head and, group by group, a value head of their own:
                # a group's heads are the rows of its blocks, so a tile of keys is read once a group and not once
                # for every few heads
                per = nq // nkv
                key = ("attention_biased_group_rows", d, dv, nq, nkv)
                cached = ctx.scratch.get(key)
                if cached is None:
                    small = 1 if attention_biased_block(d, dv, 1, 1) >= per else 0
                    rows = attention_biased_block(d, dv, 1, small)
                    nb = -(-per // rows)                    # blocks a group; made on the device: the step may be recorded
                    blocks = nkv * nb
                    firsts = (torch.arange(nkv, dtype=torch.int32, device=q.device).repeat_interleave(nb) * per
                              + torch.arange(nb, dtype=torch.int32, device=q.device).repeat(nkv) * rows)
                    seqs = torch.arange(ctx.num_seqs, dtype=torch.int32, device=q.device).repeat_interleave(blocks)
                    first = firsts.repeat(ctx.num_seqs)
                    cached = (torch.stack([seqs, first], dim=1).contiguous(), small, ctx.cu_q * nq, blocks)
                    ctx.scratch[key] = cached
                tiles, small, cu_rows, blocks = cached
                span = min(int(ctx.max_ctx_len), int(window) + 63) if window > 0 else int(ctx.max_ctx_len)
                split = biased_split_keys(ctx.num_seqs * blocks, span)
                out = attention_biased_bf16(q.view(T * nq, 1, d), k_cache, v_cache, bt, tiles, cu_rows, ctx.ctx_lens, scale, window,
                                            softcap=softcap, small=small, split_keys=split, span=span, rows_heads=nq)
                return out.view(T, nq * dv)
            if ctx.max_q_len == 1 and nkv == 1 and nq >= HEAD_ROWS_FROM and slopes is None and q.is_contiguous():
                # single tokens whose heads all read the one kv head: the heads are the rows of a block, so a tile
                # of keys is read once for all of them (nothing of the step is read on the host)
                key = ("attention_biased_head_rows", d, dv, nq)
                cached = ctx.scratch.get(key)
                if cached is None:
                    small = 1 if attention_biased_block(d, dv, 1, 1) >= nq else 0
                    rows = attention_biased_block(d, dv, 1, small)
                    blocks = -(-nq // rows)
                    seqs = torch.arange(ctx.num_seqs, dtype=torch.int32, device=q.device).repeat_interleave(blocks)
                    first = (torch.arange(blocks, dtype=torch.int32, device=q.device) * rows).repeat(ctx.num_seqs)
                    cached = (torch.stack([seqs, first], dim=1).contiguous(), small, ctx.cu_q * nq, blocks)
                    ctx.scratch[key] = cached
                tiles, small, cu_rows, blocks = cached
                span = min(int(ctx.max_ctx_len), int(window) + 63) if window > 0 else int(ctx.max_ctx_len)
                split = biased_split_keys(ctx.num_seqs * blocks, span)
                out = attention_biased_bf16(q.view(T * nq, 1, d), k_cache, v_cache, bt, tiles, cu_rows, ctx.ctx_lens, scale, window,
                                            softcap=softcap, small=small, split_keys=split, span=span, sinks=sinks, rows_heads=nq)
                return out.view(T, nq * dv)
            key = ("attention_biased_tiles", d, dv, nq, nkv)
            cached = ctx.scratch.get(key)
            if cached is None:
                if ctx.max_q_len == 1:       # a step of single tokens: a block a sequence, nothing of the step read here
                    one = torch.arange(ctx.num_seqs, dtype=torch.int32, device=q.device)
                    cached = (torch.stack([one, torch.zeros_like(one)], dim=1).contiguous(), 1)
                else:
                    q_lens = [ctx.cu_q_host[b + 1] - ctx.cu_q_host[b] for b in range(ctx.num_seqs)]
                    rows, small = prefill_tiles(q_lens, ctx.ctx_lens_host, d, nq, nkv,
                                                block_of=lambda shape: attention_biased_block(d, dv, nq // nkv, shape))
                    cached = (torch.tensor(rows, dtype=torch.int32, device=q.device).reshape(-1, 2), small)
                ctx.scratch[key] = cached
            tiles, small = cached
            split, span = 0, 0
            if ctx.max_q_len == 1:           # single tokens: slices of the keys where the sequences alone leave the chip idle
                g = nq // nkv
                span = min(int(ctx.max_ctx_len), int(window) + 63) if window > 0 else int(ctx.max_ctx_len)
                split = biased_split_keys(ctx.num_seqs * nkv * (g // (4 if g % 4 == 0 else 2 if g % 2 == 0 else 1)), span)
            return attention_biased_bf16(q, k_cache, v_cache, bt, tiles, ctx.cu_q, ctx.ctx_lens, scale, window,
                                         softcap=softcap, slopes=slopes, small=small, split_keys=split, span=span, sinks=sinks)
        return attention_generic(q, k_cache, v_cache, bt, ctx.tok_seq, ctx.positions, scale, window,
                                 v_grouped=v_grouped, softcap=softcap, slopes=slopes, sinks=sinks)
    if q.dtype == torch.bfloat16 and v_grouped and mfma_attention_supported(nq, nkv, d, page):
        g = nq // nkv
        if ctx.max_q_len == 1 and decode_attention_takes(nq, nkv, d):
            return attention_decode_bf16(q, k_cache, v_cache, bt, ctx.ctx_lens, ctx.max_ctx_len, scale, window,
                                         similar=getattr(ctx, "similar_lengths", False))
        key = ("attention_tiles", d, nq, nkv)
        cached = ctx.scratch.get(key)
        if cached is None:
            q_lens = [ctx.cu_q_host[b + 1] - ctx.cu_q_host[b] for b in range(ctx.num_seqs)]
            # The sequences at the head of the batch that bring one token (the scheduler puts the
            # decoding requests first) go to the decode kernel, which reads a kv head's keys once
            # for all its query heads and splits a context over workgroups; the prefill kernel
            # would give each of them a 16-row tile with one row in use.
            # The two kernels run one after the other, so it pays only where the prefill kernel
            # would have much to do for those sequences: keys times the times it reads them (once
            # per group of query heads it takes together), or a long context for one workgroup to walk.
            lead = 0
            while lead < len(q_lens) and q_lens[lead] == 1:
                lead += 1
            lead_ctx = max(ctx.ctx_lens_host[:lead]) if lead else 0
            reads = g // (4 if g % 4 == 0 else 2 if g % 2 == 0 else 1)
            if (lead < MIXED_DECODE_FROM or not decode_attention_takes(nq, nkv, d)
                    or not (lead * lead_ctx * reads >= MIXED_DECODE_WORK or lead_ctx >= MIXED_DECODE_CONTEXT)):
                lead = 0
            rows, small = prefill_tiles(q_lens, ctx.ctx_lens_host, d, nq, nkv, first_seq=lead)
            cached = (torch.tensor(rows, dtype=torch.int32, device=q.device).reshape(-1, 2), small, lead,
                      lead_ctx if lead else 0)
            ctx.scratch[key] = cached
        tiles, small, lead, lead_ctx = cached
        out = None
        if lead:
            out = torch.empty((T, nq * d), dtype=q.dtype, device=q.device)
            attention_decode_bf16(q[:lead], k_cache, v_cache, bt[:lead], ctx.ctx_lens[:lead], lead_ctx, scale, window,
                                  out=out[:lead])
        return attention_prefill_bf16(q, k_cache, v_cache, bt, tiles, ctx.cu_q, ctx.ctx_lens, scale, window,
                                      out=out, small=small)
    return attention_generic(q, k_cache, v_cache, bt, ctx.tok_seq, ctx.positions, scale, window,
                             v_grouped=v_grouped)


SKINNY_MAX_ROWS = 64      # most rows the streaming kernel takes
SKINNY_ROWS = 8           # up to this many rows it is faster than the vendor library (measured)
SKINNY_SPLIT_ROWS = 64    # the same where the consumer takes partial sums over slices of K,
SKINNY_SPLIT_FROM = 17    # which pays from this many rows on (fewer rows: the unsplit product)
SKINNY_GATED_ROWS = 32    # the same for the fused gate/up/silu form, which also saves a kernel


def linear_skinny(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
                  gated: bool = False, out: Optional[torch.Tensor] = None, allow_split: bool = False,
                  row_tiles: int = 0, waves: int = 0) -> torch.Tensor:
    """bfloat16 x [M, K] @ w [N, K]^T for M <= 64 rows with the streaming matrix-core kernel.
    `gated`: w is [2N, K] = [gate; up] and the result is silu(x @ gate^T) * (x @ up^T), [M, N].
    `allow_split`: for narrow outputs the kernel may cut K into slices across workgroups and
    return float32 partial sums [slices, M, N] for the consumer to add in order (the fused
    add + RMSNorm does).  `row_tiles`, `waves`: 0 = chosen from the sizes."""
    _dev(x, w, out)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("linear_skinny: operands must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"linear_skinny: x {tuple(x.shape)} and w {tuple(w.shape)} do not match")
    M, K = x.shape
    N = w.shape[0]
    if gated:
        if N % 2:
            raise KernelError("linear_skinny: a gated weight must be [2N, K]")
        N //= 2
    if M > SKINNY_MAX_ROWS or K % 8:
        raise KernelError(f"linear_skinny: M={M} must be <= {SKINNY_MAX_ROWS} and K={K} a multiple of 8")
    assert SKINNY_MAX_ROWS == int(lib().xi_linear_skinny_max_rows())
    slices = int(lib().xi_linear_skinny_slices(N, K, int(bool(gated)), int(bool(allow_split))))
    if slices > 1:
        out_dtype, shape = torch.float32, (slices, M, N)
    else:
        out_dtype, shape = out_dtype or torch.bfloat16, (M, N)
    if out is None:
        out = torch.empty(shape, dtype=out_dtype, device=x.device)
    elif tuple(out.shape) != shape or out.dtype != out_dtype:
        raise KernelError("linear_skinny: out has the wrong shape or dtype")
    _ok(lib().xi_linear_skinny(_p(x), _p(w), _p(out), M, N, K, _code(out, "linear_skinny"), int(bool(gated)),
                               int(bool(allow_split)), int(row_tiles), int(waves), _stream()))
    return out


def linear_skinny_plan(M: int, N: int, K: int, gated: bool = False, allow_split: bool = False):
    """What `linear_skinny` chooses for these sizes: (slices of K, row tiles per workgroup, output
    features per workgroup, workgroups).  Only the slices change a sum's order."""
    L = lib()
    ks = int(L.xi_linear_skinny_slices(N, K, int(bool(gated)), int(bool(allow_split))))
    rt = int(L.xi_linear_skinny_row_tiles(M, N, K, int(bool(gated)), int(bool(allow_split))))
    rows = int(L.xi_linear_skinny_rows(M, N, K, int(bool(gated)), int(bool(allow_split))))
    return ks, rt, rows, -(-N // rows) * ks


MID_ROTATE = 1            # workgroup tile t of the tiled products starts t * this many k tiles into its slice and
MID_GATED_ROTATE = 1      # wraps around (0: all start at the slice's first tile, which measured 5% slower in a
                          # decode step: every workgroup then asks for the same offset of its rows at the same time)
MID_ROWS = 256            # most rows of the tiled product for narrow outputs (`linear_mid`)
MID_WIDE_FROM = 4         # rows from which it is ahead of the streaming kernel on an output so wide that it needs no
                          # slices (the head: 215 against 242 us at 8 rows, 238 against 349 at 64, vocabulary 151936)
MID_FROM = 17             # from this many rows on it is used, where the caller takes partial sums,
MID_WIDEST = 12288        # for outputs up to this wide (N = 10240, K = 5120: 21 / 23 / 30 us at 17 / 64 / 128 rows against
                          # 24 / 31 / 39 in the library), and above 128 rows (two passes over w) for weights from
MID_BLOCK = 128           # (rows of one pass)
MID_TWO_BLOCKS = 32 << 20  # this many bytes on (below, the library is ahead: 8 MB at 256 rows, 16 against 9 us)


def linear_mid_slices(N: int, K: int) -> int:
    """The slices of K in which `linear_mid` answers for an output of N features; 0 if it does
    not take the sizes."""
    return int(lib().xi_linear_mid_slices(int(N), int(K)))


def linear_mid(x: torch.Tensor, w: torch.Tensor, depth: int = 0) -> torch.Tensor:
    """bfloat16 x [M, K] @ w [N, K]^T for up to MID_ROWS rows as float32 partial sums
    [slices, M, N], to be added in order (the fused add + RMSNorm does): the tiled kernel for
    decode batches too large for `linear_skinny` and outputs too narrow for the library.
    `depth`: tiles of loads a thread keeps in flight, 0 = the default; the result does not depend on it."""
    _dev(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("linear_mid: operands must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"linear_mid: x {tuple(x.shape)} and w {tuple(w.shape)} do not match")
    M, K = x.shape
    N = w.shape[0]
    slices = linear_mid_slices(N, K)
    if not (0 < M <= MID_ROWS) or slices < 1:
        raise KernelError(f"linear_mid: M={M} must be 1..{MID_ROWS} and K={K} a multiple of 64")
    y = torch.empty((slices, M, N), dtype=torch.float32, device=x.device)
    _ok(lib().xi_linear_mid(_p(x), _p(w), _p(y), M, N, K, int(depth), int(MID_ROTATE), _stream()))
    return y


TILE_SPLIT_ROWS = 1024        # most rows of a product that the many-row tiled kernel takes with K cut into slices
TILE_SPLIT_K = 512            # least K of a slice
TILE_SPLIT_BYTES = 8 << 20    # a weight up to this size is left to the library (level there, measured at Qwen3-0.6B sizes)
TILE_SHAPES = ((128, 256), (256, 128), (256, 256))     # rows of x by rows of w a workgroup, by `shape` of `linear_tile`
TILE_FILL_RATE = 58e9         # bytes a second that one compute unit's loads bring into its LDS
TILE_STREAM_RATE = 5e12       # bytes a second that the chip streams from memory


def tile_split_plan(M: int, N: int, K: int):
    """(slices, tile shape) of x [M, K] @ w [N, K]^T in the many-row tiled kernel (`linear_tile`) for a
    narrow output at 129 to 1,024 rows, slices 1 = it is not used.  A narrow output gives too few
    tiles for the chip's 256 compute units (256 rows by 4,096 features: 32 tiles of 256 x 128), so K
    is cut into slices, each a workgroup's own, with float32 partial sums [slices, M, N] for the
    caller to add in order.  Slices (2 to 16, whole tiles of 64 k, a slice at least 512 long) and tile shape are
    those with the least cost in a model of two terms that fits what was measured on MI355X within a
    tenth: a workgroup brings (rows of x + rows of w of its tile) x its slice of K into LDS at 58 GB/s
    (that, not the matrix cores, bounds these shapes: x is fetched again by every workgroup, so
    tiles with as many rows of w as of x are ahead where x is a whole tile's rows), rounds of 256
    workgroups one after the other, never faster than the weight streams from memory; and the
    partial sums are written and read again, 8 bytes an element and slice.  256 rows of N = 5120,
    K = 17408: 4 slices of 256 x 128 tiles 71 us, 8 slices of 256 x 256 tiles 55.  Beyond 256 rows
    only for K >= 2 N (the down projection): the reader of the partial sums reads `slices` float32
    values for every bfloat16 one, which a smaller gain does not pay for.  Up to 128 rows the tiled
    kernel of few rows (`linear_mid`) is level or ahead."""
    if not (MID_BLOCK < M <= TILE_SPLIT_ROWS) or (M > MID_ROWS and K < 2 * N) or N % 4 or K % 64 \
            or N * K * 2 <= TILE_SPLIT_BYTES:
        return 1, 0
    best = None
    k_tiles = K // 64
    for shape in ((1, 0, 2) if M <= 256 else (0, 1, 2)):      # (among equals: every row of w in one workgroup)
        bm, bn = TILE_SHAPES[shape]
        tiles = -(-M // bm) * -(-N // bn)
        for slices in range(2, 17):
            longest = -(-k_tiles // slices) * 64               # the slices differ by a tile at most
            if longest < TILE_SPLIT_K:
                break
            rounds = -(-tiles * slices // COMPUTE_UNITS)
            fill = rounds * (bm + bn) * longest * 2 / TILE_FILL_RATE
            cost = max(fill, N * K * 2 / TILE_STREAM_RATE) + slices * M * N * 8 / TILE_STREAM_RATE
            if best is None or cost < best[0] - 1e-9:
                best = (cost, slices, shape)
    return (best[1], best[2]) if best is not None else (1, 0)


def linear_tile_takes(M: int, N: int, K: int, slices: int = 1) -> bool:
    """Whether the many-row tiled product takes a shape: K in whole tiles of 64, a tile a slice at least, N in fours."""
    return bool(lib().xi_linear_tile_takes(int(M), int(N), int(K), int(slices)))


def linear_tile(x: torch.Tensor, w: torch.Tensor, slices: int = 1, partial: bool = False,
                shape: Optional[int] = None) -> torch.Tensor:
    """bfloat16 x [M, K] @ w [N, K]^T on the matrix cores for many rows: bfloat16 [M, N], or with
    `partial` (needed for more than one slice) float32 partial sums [slices, M, N] over slices of K
    (whole tiles of 64, equal but for one tile).  `shape` 0: workgroup tiles of 128 rows by 256 features, 1: 256 by 128; None: the
    one that makes fewer tiles (128 by 256 at equal numbers); 2: 256 by 256."""
    _dev(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("linear_tile: operands must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"linear_tile: x {tuple(x.shape)} and w {tuple(w.shape)} do not match")
    M, K = x.shape
    N = w.shape[0]
    partial = bool(partial) or slices > 1
    if not linear_tile_takes(M, N, K, slices):
        raise KernelError(f"linear_tile: M={M} N={N} K={K} in {slices} slices is not taken")
    if shape is None:
        shape = 1 if -(-M // 256) * -(-N // 128) < -(-M // 128) * -(-N // 256) else 0
    if partial:
        y = torch.empty((slices, M, N), dtype=torch.float32, device=x.device)
    else:
        y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    _ok(lib().xi_linear_tile(_p(x), _p(w), _p(y), M, N, K, int(slices), int(partial), int(shape), _stream()))
    return y


MID_GATED_ROWS = 128      # most rows of the gated form of the tiled product
MID_GATED_FEATURES = 0    # features a workgroup of it owns; 0: chosen from N (the fewest workgroups that are a multiple of 256)
MID_GATED_UP_TO = 64      # it is used up to this many rows (more: its reads of x from L2 outweigh the library's
                          # weakness); measured on MI355X at the gate/up sizes of Qwen3-8B, 14B and 32B, it is
MID_GATED_FROM = 2        # ahead of the streaming kernel from this many rows on, and from the first row where
MID_GATED_BIG = 300 << 20  # the weight has this many bytes (the streaming kernel falls behind on large weights)


def gated_uses_mid(M: int, w: torch.Tensor) -> bool:
    """Whether the gated product of M rows with w [2N, K] goes to `linear_mid_gated`."""
    if w.dtype != torch.bfloat16 or w.shape[1] % 64 or w.shape[1] < 64 or w.shape[0] % 2:
        return False
    return (MID_GATED_FROM <= M <= MID_GATED_UP_TO) or (0 < M < MID_GATED_FROM and w.numel() * 2 >= MID_GATED_BIG)


def linear_mid_gated(x: torch.Tensor, w: torch.Tensor, ss: Optional[torch.Tensor] = None, eps: float = 0.0,
                     features: Optional[int] = None, act: str = "silu") -> torch.Tensor:
    """act(x @ gate^T) * (x @ up^T), act silu unless given (`ACTIVATIONS`), in bfloat16 for w = [gate; up] [2N, K] and up to MID_GATED_ROWS
    rows with the tiled kernel: one pass over w whatever the number of rows.  `ss` [M, parts]
    float32 (up to FOLD_ROWS rows): x is the first half of a folded RMSNorm (`linear_fold_out`)
    and the rows of the products are multiplied by rsqrt(sum(ss[row]) / K + eps) first.
    `features`: the features a workgroup owns (up to 64, up to 128 for up to 64 rows), for
    measurements and tests; chosen from the sizes if not given."""
    _dev(x, w, ss)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("linear_mid_gated: operands must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or w.shape[0] % 2:
        raise KernelError(f"linear_mid_gated: x {tuple(x.shape)} and w {tuple(w.shape)} ([2N, K]) do not match")
    M, K = x.shape
    N = w.shape[0] // 2
    if not (0 < M <= MID_GATED_ROWS) or K % 64 or K < 64:
        raise KernelError(f"linear_mid_gated: M={M} must be 1..{MID_GATED_ROWS} and K={K} a multiple of 64")
    parts = 0
    if ss is not None:
        _want(ss, torch.float32, "linear_mid_gated: ss")
        if M > FOLD_ROWS or ss.dim() != 2 or ss.shape[0] != M or not (0 < ss.shape[1] <= FOLD_PARTS):
            raise KernelError(f"linear_mid_gated: a folded norm takes up to {FOLD_ROWS} rows and ss [M, up to "
                              f"{FOLD_PARTS} parts], got M={M}, ss {tuple(ss.shape)}")
        parts = int(ss.shape[1])
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    _ok(lib().xi_linear_mid_gated(_p(x), _p(w), _p(y), M, N, K, _p(ss), parts, ctypes.c_float(eps), int(MID_GATED_ROTATE),
                                  int(features if features is not None else MID_GATED_FEATURES), ACTIVATIONS[act], _stream()))
    return y


FOLD_ROWS = 16            # most rows of the products that carry a folded norm between them
FOLD_PARTS = 512          # most parts of a row's sum of squares the product after the norm adds up


def linear_fold_parts(M: int, N: int, K: int) -> int:
    """The parts in which `linear_fold_out` hands on each row's sum of squares for these sizes."""
    return int(lib().xi_linear_skinny_fold_parts(int(M), int(N), int(K)))


def linear_fold_out(x: torch.Tensor, w: torch.Tensor, resid: torch.Tensor, norm_weight: torch.Tensor):
    """The product before an RMSNorm, for up to FOLD_ROWS rows: resid [M, N] float32 += x [M, K] @
    w [N, K]^T in place; returns (xg, ss): xg [M, N] bfloat16 = round(resid * norm_weight), ss
    [M, parts] float32 the sums of squares of the rows of resid in parts.  `linear_fold_in` is the
    product after the norm; between them no norm kernel runs."""
    _dev(x, w, resid, norm_weight)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("linear_fold_out: operands must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"linear_fold_out: x {tuple(x.shape)} and w {tuple(w.shape)} do not match")
    M, K = x.shape
    N = w.shape[0]
    if not (0 < M <= FOLD_ROWS) or K % 8:
        raise KernelError(f"linear_fold_out: M={M} must be 1..{FOLD_ROWS} and K={K} a multiple of 8")
    _want(resid, torch.float32, "linear_fold_out: resid")
    _want(norm_weight, torch.float32, "linear_fold_out: norm weight")
    if tuple(resid.shape) != (M, N) or tuple(norm_weight.shape) != (N,) or not resid.is_contiguous():
        raise KernelError(f"linear_fold_out: resid {tuple(resid.shape)} / norm weight {tuple(norm_weight.shape)} "
                          f"do not match [M={M}, N={N}]")
    parts = linear_fold_parts(M, N, K)
    xg = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    ss = torch.empty((M, parts), dtype=torch.float32, device=x.device)
    _ok(lib().xi_linear_skinny_fold_out(_p(x), _p(w), M, N, K, _p(resid), _p(norm_weight), _p(xg), _p(ss), _stream()))
    return xg, ss


def linear_fold_in(xg: torch.Tensor, ss: torch.Tensor, eps: float, w: torch.Tensor,
                   out_dtype: Optional[torch.dtype] = None, gated: bool = False) -> torch.Tensor:
    """The product after an RMSNorm whose first half `linear_fold_out` did: (xg @ w^T) with each
    row multiplied by rsqrt(sum(ss[row]) / K + eps), one rounding; `gated` as in `linear_skinny`."""
    _dev(xg, ss, w)
    if xg.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("linear_fold_in: operands must be bfloat16")
    if xg.dim() != 2 or w.dim() != 2 or xg.shape[1] != w.shape[1]:
        raise KernelError(f"linear_fold_in: x {tuple(xg.shape)} and w {tuple(w.shape)} do not match")
    M, K = xg.shape
    N = w.shape[0]
    if gated:
        if N % 2:
            raise KernelError("linear_fold_in: a gated weight must be [2N, K]")
        N //= 2
    _want(ss, torch.float32, "linear_fold_in: ss")
    if not (0 < M <= FOLD_ROWS) or K % 8 or ss.dim() != 2 or ss.shape[0] != M or not (0 < ss.shape[1] <= FOLD_PARTS) \
            or not ss.is_contiguous():
        raise KernelError(f"linear_fold_in: M={M} (1..{FOLD_ROWS}), K={K} (multiple of 8), ss {tuple(ss.shape)} "
                          f"([M, up to {FOLD_PARTS} parts])")
    out_dtype = out_dtype or torch.bfloat16
    if gated and out_dtype != torch.bfloat16:
        raise KernelError("linear_fold_in: the gated form writes bfloat16")
    y = torch.empty((M, N), dtype=out_dtype, device=xg.device)
    _ok(lib().xi_linear_skinny_fold_in(_p(xg), _p(w), _p(y), M, N, K, _code(y, "linear_fold_in"), int(bool(gated)),
                                       _p(ss), int(ss.shape[1]), ctypes.c_float(eps), _stream()))
    return y


THIN_ROTATE = 0           # workgroup b of the thin product starts b * this many k tiles into K (see MID_ROTATE;
                          # here it measured no gain: 0)


def thin_ahead(M: int, w: torch.Tensor) -> bool:
    """Whether a product of M <= FOLD_ROWS rows with whole sums goes to the thin kernel: wherever it
    takes the sizes (K a multiple of 256).  Measured in decode steps at Qwen3-8B, 14B and 32B sizes
    against the streaming kernel: level at one row, 1 to 3% of a step ahead from two rows on."""
    if w.dtype != torch.bfloat16 or not (0 < M <= FOLD_ROWS):
        return False
    return 0 < linear_thin_parts(w.shape[0], w.shape[1]) <= FOLD_PARTS


def linear_thin_parts(N: int, K: int) -> int:
    """Workgroups of the thin product for an output of N features (the parts in which
    `linear_thin_fold_out` hands on a row's sum of squares); 0 if it does not take the sizes."""
    return int(lib().xi_linear_thin_parts(int(N), int(K)))


def _thin_operands(what: str, x: torch.Tensor, w: torch.Tensor):
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"{what}: operands must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"{what}: x {tuple(x.shape)} and w {tuple(w.shape)} do not match")
    M, K = x.shape
    N = w.shape[0]
    if not (0 < M <= FOLD_ROWS) or linear_thin_parts(N, K) < 1:
        raise KernelError(f"{what}: M={M} must be 1..{FOLD_ROWS} and K={K} a multiple of 256")
    return M, N, K


def linear_thin(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """bfloat16 x [M, K] @ w [N, K]^T for up to FOLD_ROWS rows, whole sums (no slices of K) with few
    output features per workgroup, loaded as whole lines through LDS: the shape of the products
    around a folded norm."""
    _dev(x, w)
    M, N, K = _thin_operands("linear_thin", x, w)
    y = torch.empty((M, N), dtype=out_dtype or torch.bfloat16, device=x.device)
    _ok(lib().xi_linear_thin(_p(x), _p(w), _p(y), M, N, K, _code(y, "linear_thin"), int(THIN_ROTATE), _stream()))
    return y


def linear_thin_fold_out(x: torch.Tensor, w: torch.Tensor, resid: torch.Tensor, norm_weight: torch.Tensor):
    """`linear_fold_out` with the thin kernel: resid [M, N] float32 += x @ w^T in place; returns
    (xg, ss) with ss [M, linear_thin_parts(N, K)]."""
    _dev(x, w, resid, norm_weight)
    M, N, K = _thin_operands("linear_thin_fold_out", x, w)
    _want(resid, torch.float32, "linear_thin_fold_out: resid")
    _want(norm_weight, torch.float32, "linear_thin_fold_out: norm weight")
    if tuple(resid.shape) != (M, N) or tuple(norm_weight.shape) != (N,):
        raise KernelError(f"linear_thin_fold_out: resid {tuple(resid.shape)} / norm weight {tuple(norm_weight.shape)} "
                          f"do not match [M={M}, N={N}]")
    xg = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    ss = torch.empty((M, linear_thin_parts(N, K)), dtype=torch.float32, device=x.device)
    _ok(lib().xi_linear_thin_fold_out(_p(x), _p(w), M, N, K, _p(resid), _p(norm_weight), _p(xg), _p(ss),
                                      int(THIN_ROTATE), _stream()))
    return xg, ss


def linear_thin_fold_in(xg: torch.Tensor, ss: torch.Tensor, eps: float, w: torch.Tensor,
                        out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """`linear_fold_in` (plain form) with the thin kernel."""
    _dev(xg, ss, w)
    M, N, K = _thin_operands("linear_thin_fold_in", xg, w)
    _want(ss, torch.float32, "linear_thin_fold_in: ss")
    if ss.dim() != 2 or ss.shape[0] != M or not (0 < ss.shape[1] <= FOLD_PARTS):
        raise KernelError(f"linear_thin_fold_in: ss {tuple(ss.shape)} is not [M={M}, up to {FOLD_PARTS} parts]")
    y = torch.empty((M, N), dtype=out_dtype or torch.bfloat16, device=xg.device)
    _ok(lib().xi_linear_thin_fold_in(_p(xg), _p(w), _p(y), M, N, K, _code(y, "linear_thin_fold_in"), _p(ss),
                                     int(ss.shape[1]), ctypes.c_float(eps), int(THIN_ROTATE), _stream()))
    return y


def linear_bf16(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
                skinny_rows: int = SKINNY_ROWS, allow_split: bool = False) -> torch.Tensor:
    """bfloat16 x @ w.T with float32 accumulation, rounded once to `out_dtype` (bfloat16 or
    float32).  Up to `skinny_rows` rows (decode): the hand-written streaming kernel, which with
    `allow_split` may answer with float32 partial sums [slices, M, N] for a narrow output.  More
    rows: the vendor library (hipBLASLt through torch), which the reference's engine also
    uses for its matrix products."""
    _dev(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("linear_bf16: operands must be bfloat16")
    out_dtype = out_dtype or torch.bfloat16
    if out_dtype == torch.float32 and MID_WIDE_FROM <= x.shape[0] <= MID_GATED_ROWS \
            and linear_mid_slices(w.shape[0], w.shape[1]) == 1:
        return linear_mid(x, w)[0]           # a wide output in float32 (the head): one slice is the result
    if allow_split and MID_BLOCK < x.shape[0] <= TILE_SPLIT_ROWS:
        slices, shape = tile_split_plan(x.shape[0], w.shape[0], w.shape[1])
        if slices > 1:
            return linear_tile(x, w, slices, partial=True, shape=shape)
    if allow_split and MID_FROM <= x.shape[0] <= MID_ROWS and linear_mid_slices(w.shape[0], w.shape[1]) > 0 \
            and w.shape[0] <= MID_WIDEST and (x.shape[0] <= MID_BLOCK or w.numel() * 2 >= MID_TWO_BLOCKS):
        return linear_mid(x, w)
    if (allow_split and x.shape[1] % 8 == 0 and x.shape[0] >= SKINNY_SPLIT_FROM
            and int(lib().xi_linear_skinny_slices(w.shape[0], w.shape[1], 0, 1)) > 1):
        skinny_rows = max(skinny_rows, SKINNY_SPLIT_ROWS)
    else:
        allow_split = False
    if not allow_split and thin_ahead(x.shape[0], w):
        return linear_thin(x, w, out_dtype)
    if 0 < x.shape[0] <= min(skinny_rows, SKINNY_MAX_ROWS) and x.shape[1] % 8 == 0:
        return linear_skinny(x, w, out_dtype, allow_split=allow_split)
    if out_dtype == torch.float32:
        return torch.mm(x, w.t(), out_dtype=torch.float32)
    return torch.nn.functional.linear(x, w)


# ---- an embedding that looks at the token before; what a run of layers adds when it starts ----------------
def embed_pair(table: torch.Tensor, pairs: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor, tok_seq: torch.Tensor,
               cu_q: torch.Tensor, state_slots: torch.Tensor, last: torch.Tensor, scale: float, buckets: int,
               mul_prev: int, mul_cur: int) -> torch.Tensor:
    """out[t] = float32(table[ids[t]]) * scale + float32(pairs[row(t)]), row(t) = (prev * mul_prev + ids[t] * mul_cur)
    mod buckets with prev the token before t in its sequence, and row `buckets` at position 0.  The token before a
    portion's first token is `last[state_slots[b]]` (int32 [slots]: what `keep_last_token` left there)."""
    _dev(table, pairs, ids, positions, tok_seq, cu_q, state_slots, last)
    for t, name in ((ids, "ids"), (positions, "positions"), (tok_seq, "tok_seq"), (cu_q, "cu_q"), (last, "last")):
        _want(t, torch.int32, f"embed_pair: {name}")
    _want(state_slots, torch.int64, "embed_pair: state_slots")
    if table.dim() != 2 or pairs.dim() != 2 or pairs.shape[1] != table.shape[1] or pairs.dtype != table.dtype:
        raise KernelError("embed_pair: table [V, H] and pairs [buckets + 1, H] of one type")
    T, H, B = ids.shape[0], table.shape[1], state_slots.shape[0]
    if int(buckets) <= 0 or pairs.shape[0] != int(buckets) + 1 or int(mul_prev) < 0 or int(mul_cur) < 0:
        raise KernelError(f"embed_pair: {pairs.shape[0]} rows of pairs for {buckets} buckets and one more")
    if positions.shape != (T,) or tok_seq.shape != (T,) or cu_q.shape != (B + 1,) or last.dim() != 1:
        raise KernelError("embed_pair: positions and tok_seq [T], cu_q [B + 1], last [slots]")
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _ok(lib().xi_embed_pair(_p(table), _p(pairs), _code(table, "embed_pair"), _p(ids), _p(positions), _p(tok_seq), _p(cu_q),
                            _p(state_slots), _p(last), _p(out), T, H, ctypes.c_float(scale), ctypes.c_longlong(int(buckets)),
                            ctypes.c_longlong(int(mul_prev)), ctypes.c_longlong(int(mul_cur)), _stream()))
    return out


def keep_last_token(ids: torch.Tensor, cu_q: torch.Tensor, state_slots: torch.Tensor, last: torch.Tensor) -> None:
    """last[state_slots[b]] = the last token of sequence b's portion in this step."""
    _dev(ids, cu_q, state_slots, last)
    for t, name in ((ids, "ids"), (cu_q, "cu_q"), (last, "last")):
        _want(t, torch.int32, f"keep_last_token: {name}")
    _want(state_slots, torch.int64, "keep_last_token: state_slots")
    B = state_slots.shape[0]
    if cu_q.shape != (B + 1,) or last.dim() != 1 or ids.dim() != 1:
        raise KernelError("keep_last_token: ids [T], cu_q [B + 1], last [slots]")
    _ok(lib().xi_keep_last_token(_p(ids), _p(cu_q), _p(state_slots), _p(last), B, _stream()))


def stream_start(resid: torch.Tensor, pending: Optional[torch.Tensor], factor: float, first: Optional[torch.Tensor],
                 vec: Optional[torch.Tensor]) -> torch.Tensor:
    """resid += factor * pending (+ first) (+ vec), in place, float32: `pending` rows [T, H] in either precision or a
    stack [P, T, H] of float32 partial sums (or None), `first` float32 [T, H] or None, `vec` float32 [H] or None."""
    _dev(resid, pending, first, vec)
    _want(resid, torch.float32, "stream_start: the stream")
    if resid.dim() != 2:
        raise KernelError("stream_start: the stream must be [T, H]")
    T, H = resid.shape
    parts, code = 1, F32
    if pending is not None:
        if pending.dim() == 3:
            _want(pending, torch.float32, "stream_start: partial sums")
            parts = int(pending.shape[0])
        if tuple(pending.shape[-2:]) != (T, H) or pending.dim() not in (2, 3):
            raise KernelError(f"stream_start: the branch {tuple(pending.shape)} does not fit the stream {(T, H)}")
        code = _code(pending, "stream_start")
    if first is not None and (first.dtype != torch.float32 or tuple(first.shape) != (T, H)):
        raise KernelError("stream_start: the embedding's output must be float32 [T, H]")
    if vec is not None and (vec.dtype != torch.float32 or tuple(vec.shape) != (H,)):
        raise KernelError("stream_start: the vector must be float32 [H]")
    _ok(lib().xi_stream_start(_p(resid), _p(pending), code, parts, ctypes.c_float(factor), _p(first), _p(vec), T, H, _stream()))
    return resid


# ---- a projection's heads made ready one by one: rotation, then a unit norm ---------------------------------
def head_rows(qkv: torch.Tensor, slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, num_heads: int,
              num_kv_heads: int, head_dim: int, value_dim: int, v_grouped: bool = False, cos: Optional[torch.Tensor] = None,
              sin: Optional[torch.Tensor] = None, rotary_dim: int = 0, interleaved: bool = False,
              positions: Optional[torch.Tensor] = None, unit_norm: bool = False, eps: float = 0.0) -> torch.Tensor:
    """A packed projection [T, nq d + nkv d + nkv dv]: the first `rotary_dim` dims of every q and k head turn by the
    token's position (pairs (2i, 2i + 1) if `interleaved`, else (i, i + r / 2); `cos` / `sin` float32 [positions, r / 2]),
    then, with `unit_norm`, each head is divided by its root mean square over d (eps inside the root); k and v go into
    the paged cache at `slots`.  Returns q [T, nq, d]."""
    _dev(qkv, slots, k_cache, v_cache, cos, sin, positions)
    nq, nkv, d, dv, rot = int(num_heads), int(num_kv_heads), int(head_dim), int(value_dim), int(rotary_dim)
    if qkv.dim() != 2 or qkv.shape[1] != nq * d + nkv * d + nkv * dv:
        raise KernelError(f"head_rows: qkv {tuple(qkv.shape)} is not [T, {nq * d + nkv * d + nkv * dv}]")
    T = qkv.shape[0]
    _want(slots, torch.int64, "head_rows: slots")
    if slots.shape != (T,) or d > 1024:
        raise KernelError("head_rows: slots must be [T]; heads of up to 1024 dims")
    if rot:
        if rot % 2 or not (0 < rot <= d) or cos is None or sin is None or positions is None:
            raise KernelError(f"head_rows: {rot} rotated dims of a head of {d} need tables and positions")
        _want(cos, torch.float32, "head_rows: cos")
        _want(sin, torch.float32, "head_rows: sin")
        _want(positions, torch.int32, "head_rows: positions")
        if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != rot // 2 or positions.shape != (T,):
            raise KernelError(f"head_rows: the rotation's tables must be [positions, {rot // 2}], positions [T]")
    _check_cache(k_cache, v_cache, nkv, d, qkv.dtype, v_grouped, "head_rows", dv=dv)
    q_out = torch.empty((T, nq, d), dtype=qkv.dtype, device=qkv.device)
    _ok(lib().xi_head_rows(_p(qkv), _code(qkv, "head_rows"), _p(slots), _p(q_out), _p(k_cache), _p(v_cache),
                           int(k_cache.shape[2]), T, nq, nkv, d, dv, int(bool(v_grouped)), _p(cos if rot else None),
                           _p(sin if rot else None), rot, int(bool(interleaved)), _p(positions if rot else None),
                           int(bool(unit_norm)), ctypes.c_float(eps), _stream()))
    return q_out


# ---- attention over a latent ---------------------------------------------------------------------------------
def latent_rows(proj: torch.Tensor, q_offset: int, down_offset: int, norm_weight: torch.Tensor, eps: float,
                slots: torch.Tensor, pool: torch.Tensor, q_full: torch.Tensor, heads: int, dim: int, rot_dim: int,
                rank: int, cos: torch.Tensor, sin: torch.Tensor, interleaved: bool, positions: torch.Tensor,
                values: Optional[torch.Tensor] = None, q_rows: Optional[torch.Tensor] = None) -> None:
    """From the packed projection `proj` [T, W] (the heads' q parts [H, dim + rot_dim] from column `q_offset`, the down
    projection [rank + rot_dim] from `down_offset`): the latent = RMSNorm(down[:rank]) * norm_weight and the turned
    down[rank:] into `pool` [pages, 1, page, rank + rot_dim] at `slots`; every head's turned q part into
    q_full[:, h, rank:] (q_full [T, H, rank + rot_dim]).  `values` [pages, 1, page / 8, rank, 8]: the latent once
    more, in groups of eight tokens, as the matrix-core attention kernels read values.  `q_rows` [T, >= q_offset +
    H (dim + rot_dim)]: the heads' q parts are rows of this tensor instead of `proj`'s."""
    _dev(proj, norm_weight, slots, pool, q_full, cos, sin, positions, values, q_rows)
    H, d, r, rank = int(heads), int(dim), int(rot_dim), int(rank)
    if proj.dim() != 2 or q_full.dtype != proj.dtype or pool.dtype != proj.dtype:
        raise KernelError("latent_rows: the projection, the pool and q of one type")
    T, W = proj.shape
    if q_rows is not None and (q_rows.dim() != 2 or q_rows.shape[0] != T or q_rows.dtype != proj.dtype or q_rows.stride(1) != 1):
        raise KernelError("latent_rows: the q parts must be rows of the same tokens and type")
    QW = W if q_rows is None else int(q_rows.shape[1])
    if q_offset < 0 or down_offset < 0 or q_offset + H * (d + r) > QW or down_offset + rank + r > W:
        raise KernelError(f"latent_rows: rows of {W} do not hold the q parts and the down projection")
    if tuple(q_full.shape) != (T, H, rank + r) or pool.dim() != 4 or pool.shape[1] != 1 or pool.shape[3] != rank + r:
        raise KernelError(f"latent_rows: q {tuple(q_full.shape)} must be [{T}, {H}, {rank + r}], the pool [pages, 1, page, {rank + r}]")
    _want(norm_weight, torch.float32, "latent_rows: the norm's weight")
    _want(slots, torch.int64, "latent_rows: slots")
    _want(positions, torch.int32, "latent_rows: positions")
    _want(cos, torch.float32, "latent_rows: cos")
    _want(sin, torch.float32, "latent_rows: sin")
    if (norm_weight.shape != (rank,) or slots.shape != (T,) or positions.shape != (T,) or r % 2 or cos.shape != sin.shape
            or cos.dim() != 2 or cos.shape[1] != r // 2):
        raise KernelError(f"latent_rows: weight [{rank}], slots and positions [T], tables [positions, {r // 2}]")
    if values is not None and (values.dtype != proj.dtype or pool.shape[2] % 8
                               or tuple(values.shape) != (pool.shape[0], 1, pool.shape[2] // 8, rank, 8)):
        raise KernelError(f"latent_rows: the values' pool {tuple(values.shape)} must be [{pool.shape[0]}, 1, page / 8, {rank}, 8]")
    _ok(lib().xi_latent_rows(_p(proj), ctypes.c_longlong(W), int(q_offset), int(down_offset), _code(proj, "latent_rows"),
                             _p(norm_weight), ctypes.c_float(eps), _p(slots), _p(pool), _p(values), int(pool.shape[2]), _p(q_full), T, H,
                             d, r, rank, _p(cos), _p(sin), int(bool(interleaved)), _p(positions), _p(q_rows),
                             ctypes.c_longlong(0 if q_rows is None else (int(q_rows.stride(0)) if T > 1 else QW)), _stream()))


def head_linear(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t, h, n] = sum_k x[t, h, k] * w[h, n, k] for every head, float32 sums; with `gate`
    [T, H, N], out *= sigmoid(gate); a gate [T, H] is one number a head.  bfloat16 operands whose K is contiguous in whole 16-byte chunks run on the
    matrix cores; others, and float32, on the vector units in ascending k.  All operands may be strided views ([T, H, .] of packed rows; w [H, N, K] with
    either N or K contiguous) of one type; `out` [T, H, N] is written in place."""
    for t in (x, w, out, gate):
        if t is not None and (not t.is_cuda or t.dtype != x.dtype or t.device != x.device):
            raise KernelError("head_linear: operands of one type on one GPU")
    if x.dim() != 3 or w.dim() != 3 or out.dim() != 3:
        raise KernelError("head_linear: x [T, H, K], w [H, N, K], out [T, H, N]")
    T, H, K = x.shape
    N = w.shape[1]
    each = gate is None or gate.dim() == 3
    if (tuple(w.shape) != (H, N, K) or tuple(out.shape) != (T, H, N)
            or (gate is not None and tuple(gate.shape) != ((T, H, N) if each else (T, H)))):
        raise KernelError(f"head_linear: x {tuple(x.shape)}, w {tuple(w.shape)} and out {tuple(out.shape)} do not match")
    if x.stride(2) != 1 or out.stride(2) != 1 or (gate is not None and each and gate.stride(2) != 1) or 1 not in (w.stride(1), w.stride(2)):
        raise KernelError("head_linear: the last axis of x, out and the gate, and N or K of w, must be contiguous")
    ll = ctypes.c_longlong
    g = gate if gate is not None else out
    _ok(lib().xi_head_linear(_p(x), ll(x.stride(0)), ll(x.stride(1)), _p(w), ll(w.stride(0)), ll(w.stride(1)), ll(w.stride(2)),
                             _p(out), ll(out.stride(0)), ll(out.stride(1)), _p(gate), ll(g.stride(0)), ll(g.stride(1)),
                             int(each), _code(x, "head_linear"), T, H, N, K, _stream()))
    return out


# ---- around the state of a selective state-space mixer ---------------------------------------------------------
def causal_conv(u: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, tails: torch.Tensor, state_slots: torch.Tensor,
                tok_seq: torch.Tensor, cu_q: torch.Tensor) -> torch.Tensor:
    """out[t, c] = silu(bias[c] + sum_j weight[c, j] u[t - (taps - 1) + j, c]) within each sequence; inputs from before
    the step's portion come from the request's tail (`tails` float32 [slots, taps - 1, C], oldest first; slots may be
    strided), which is left as it is (`conv_tail` moves it on).  u [T, C] may be columns of a packed projection;
    weight float32 [C, taps], bias float32 [C].  Returns [T, C] in u's type."""
    _dev(weight, bias, state_slots, tok_seq, cu_q)
    T, C = u.shape
    us = _columns(u, C, "causal_conv: u")
    _want(weight, torch.float32, "causal_conv: weight")
    _want(bias, torch.float32, "causal_conv: bias")
    _want(tails, torch.float32, "causal_conv: tails")
    _want(state_slots, torch.int64, "causal_conv: state_slots")
    _want(tok_seq, torch.int32, "causal_conv: tok_seq")
    _want(cu_q, torch.int32, "causal_conv: cu_q")
    taps = int(weight.shape[1]) if weight.dim() == 2 else 0
    B = state_slots.shape[0]
    if weight.dim() != 2 or weight.shape[0] != C or taps < 1 or bias.shape != (C,) or tok_seq.shape != (T,) or cu_q.shape != (B + 1,):
        raise KernelError(f"causal_conv: weight [{C}, taps], bias [{C}], tok_seq [T], cu_q [B + 1]")
    if (tails.dim() != 3 or tuple(tails.shape[1:]) != (taps - 1, C) or not tails.is_cuda or tails.device != u.device
            or (taps > 1 and tails[0].stride() != (C, 1))):
        raise KernelError(f"causal_conv: tails {tuple(tails.shape)} must be [slots, {taps - 1}, {C}] with whole slots")
    out = torch.empty((T, C), dtype=u.dtype, device=u.device)
    stride = int(tails.stride(0)) if tails.shape[0] > 1 else (taps - 1) * C
    _ok(lib().xi_causal_conv(_p(u), ctypes.c_longlong(us), _code(u, "causal_conv"), _p(weight), _p(bias), _p(tails),
                             ctypes.c_longlong(stride), _p(state_slots), _p(tok_seq), _p(cu_q), _p(out), T, C, taps, _stream()))
    return out


def conv_tail(u: torch.Tensor, tails: torch.Tensor, state_slots: torch.Tensor, cu_q: torch.Tensor) -> None:
    """Moves every request's tail on by its portion of this step: afterwards it holds the last taps - 1 inputs."""
    _dev(state_slots, cu_q)
    T, C = u.shape
    us = _columns(u, C, "conv_tail: u")
    _want(tails, torch.float32, "conv_tail: tails")
    _want(state_slots, torch.int64, "conv_tail: state_slots")
    _want(cu_q, torch.int32, "conv_tail: cu_q")
    B = state_slots.shape[0]
    if tails.dim() != 3 or tails.shape[2] != C or cu_q.shape != (B + 1,) or not tails.is_cuda or tails.device != u.device:
        raise KernelError(f"conv_tail: tails {tuple(tails.shape)} must be [slots, taps - 1, {C}], cu_q [B + 1]")
    taps = int(tails.shape[1]) + 1
    if taps > 1 and tails[0].stride() != (C, 1):
        raise KernelError("conv_tail: whole slots")
    stride = int(tails.stride(0)) if tails.shape[0] > 1 else (taps - 1) * C
    _ok(lib().xi_conv_tail(_p(u), ctypes.c_longlong(us), _code(u, "conv_tail"), _p(tails), ctypes.c_longlong(stride),
                           _p(state_slots), _p(cu_q), B, C, taps, _stream()))


def gated_group_norm(y: torch.Tensor, x: torch.Tensor, skip: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, eps: float,
                     groups: int, out_dtype: torch.dtype) -> torch.Tensor:
    """v = (y + skip[h] x) * silu(z), then each of `groups` equal parts of a row divided by its root mean square (eps
    inside the root), times `weight`.  y float32 [T, H, dv]; x, z [T, H dv] in `out_dtype` (may be columns of packed
    rows); skip float32 [H]; weight float32 [H dv].  Returns [T, H dv] in `out_dtype`."""
    _dev(y, skip, weight)
    _want(y, torch.float32, "gated_group_norm: y")
    if y.dim() != 3:
        raise KernelError("gated_group_norm: y must be [T, H, dv]")
    T, H, dv = y.shape
    W = H * dv
    xs, zs = _columns(x, W, "gated_group_norm: x"), _columns(z, W, "gated_group_norm: z")
    if x.shape[0] != T or z.shape[0] != T or x.dtype != out_dtype or z.dtype != out_dtype or x.device != y.device or z.device != y.device:
        raise KernelError("gated_group_norm: x and z must be rows of the same tokens in the output's type")
    _want(skip, torch.float32, "gated_group_norm: skip")
    _want(weight, torch.float32, "gated_group_norm: weight")
    if skip.shape != (H,) or weight.shape != (W,) or int(groups) <= 0 or W % int(groups):
        raise KernelError(f"gated_group_norm: skip [{H}], weight [{W}], and groups that divide {W}")
    out = torch.empty((T, W), dtype=out_dtype, device=y.device)
    _ok(lib().xi_gated_group_norm(_p(y), _p(x), ctypes.c_longlong(xs), _p(skip), _p(z), ctypes.c_longlong(zs), _p(weight),
                                  ctypes.c_float(eps), _p(out), _code(out, "gated_group_norm"), T, W, dv, int(groups), _stream()))
    return out


# ---- around the state of a matrix memory ----------------------------------------------------------------------------
def mlstm_gates(z: torch.Tensor, bias: torch.Tensor, cap: float, m_state: torch.Tensor, state_slots: torch.Tensor,
                cu_q: torch.Tensor, heads: int):
    """The gates of a matrix memory for a step's tokens.  z float32 [T, 2 H] (rows may be a column range): the input
    gate's logits, then the forget gate's; bias float32 [2 H]; log_in = cap tanh((z_i + b_i) / cap), log_keep =
    logsigmoid(cap tanh((z_f + b_f) / cap)); the running maximum m' = max(log_keep + m, log_in) is walked token by token
    from m_state float32 [slots, H] (left there afterwards).  Returns gates float32 [T, H, 2] = (exp(log_keep + m - m'),
    exp(log_in - m')) and floor float32 [T, H] = exp(-m')."""
    _dev(bias, state_slots, cu_q)
    H = int(heads)
    _want(z, torch.float32, "mlstm_gates: z")
    _want(bias, torch.float32, "mlstm_gates: bias")
    _want(m_state, torch.float32, "mlstm_gates: m_state")
    _want(state_slots, torch.int64, "mlstm_gates: state_slots")
    _want(cu_q, torch.int32, "mlstm_gates: cu_q")
    zs = _columns(z, 2 * H, "mlstm_gates: z")
    T, B = z.shape[0], state_slots.shape[0]
    if bias.shape != (2 * H,) or cu_q.shape != (B + 1,) or m_state.dim() != 2 or m_state.shape[1] != H or m_state.stride(1) != 1:
        raise KernelError(f"mlstm_gates: bias [{2 * H}], cu_q [B + 1], m_state [slots, {H}] expected")
    gates = torch.empty((T, H, 2), dtype=torch.float32, device=z.device)
    floor = torch.empty((T, H), dtype=torch.float32, device=z.device)
    stride = int(m_state.stride(0)) if m_state.shape[0] > 1 else H
    _ok(lib().xi_mlstm_gates(_p(z), ctypes.c_longlong(zs), _p(bias), ctypes.c_float(cap), _p(m_state), ctypes.c_longlong(stride),
                             _p(state_slots), _p(cu_q), _p(gates), _p(floor), int(B), H, _stream()))
    return gates, floor


def mlstm_finish(o: torch.Tensor, floor: torch.Tensor, weight: torch.Tensor, eps: float, gate: torch.Tensor,
                 out_dtype: torch.dtype) -> torch.Tensor:
    """o float32 [T, H, dv + 1] (a matrix memory's results; the last column is n . q): y = o[:dv] / (max(|o[dv]|, floor) +
    1e-6), each head of y divided by its root mean square over dv (eps inside the root), times `weight` float32 [H dv],
    times sigmoid(gate) (gate [T, H dv], may be a column range of a packed projection, in `out_dtype`).  Returns
    [T, H dv] in `out_dtype`."""
    _dev(o, floor, weight)
    _want(o, torch.float32, "mlstm_finish: o")
    _want(floor, torch.float32, "mlstm_finish: floor")
    _want(weight, torch.float32, "mlstm_finish: weight")
    if o.dim() != 3 or o.shape[2] < 2 or not o.is_contiguous():
        raise KernelError("mlstm_finish: o must be [T, H, dv + 1]")
    T, H, dv = o.shape[0], o.shape[1], o.shape[2] - 1
    gs = _columns(gate, H * dv, "mlstm_finish: gate")
    if (gate.shape[0] != T or gate.dtype != out_dtype or gate.device != o.device or tuple(floor.shape) != (T, H)
            or not floor.is_contiguous() or weight.shape != (H * dv,)):
        raise KernelError(f"mlstm_finish: gate rows of the same tokens in the output's type, floor [T, H], weight [{H * dv}]")
    out = torch.empty((T, H * dv), dtype=out_dtype, device=o.device)
    _ok(lib().xi_mlstm_finish(_p(o), _p(floor), _p(weight), ctypes.c_float(eps), _p(gate), ctypes.c_longlong(gs), _p(out),
                              _code(out, "mlstm_finish"), T, H, dv, _stream()))
    return out


# ---- rows of an attention with a short convolution and mixed heads -----------------------------------------------------
def conv_qkv_rows(qkv: torch.Tensor, conv_weight: Optional[torch.Tensor], tails: Optional[torch.Tensor],
                  state_slots: torch.Tensor, tok_seq: torch.Tensor, cu_q: torch.Tensor, q_weight: Optional[torch.Tensor],
                  k_weight: Optional[torch.Tensor], eps: float, slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, v_grouped: bool = False,
                  value_unit_norm: bool = False, talk: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The first nq d + nkv d + nkv dv columns of a packed projection made ready for attention: a causal convolution per
    channel over the last `taps` tokens (`conv_weight` float32 [C, taps]; None: none; one tap: a factor a channel; inputs
    from before the step come from `tails` float32 [slots, taps - 1, C] at `state_slots`, which `conv_tail` moves on afterwards), RMSNorm over the
    whole q part and the whole k part (weights float32; None: none), every value head divided by its root mean square
    (`value_unit_norm`), k and v into the paged cache at `slots`.  With `talk` float32 [nq, nq] (head h's score is
    sum_g talk[h, g] (q_g . k)) the sum is taken on the query's side: the result is q' [T, nq, nkv d] and the K pool
    [pages, 1, page, nkv d] holds a token's whole k row as one head; without, q [T, nq, d] and a K pool [pages, nkv, page, d]."""
    _dev(conv_weight, state_slots, tok_seq, cu_q, q_weight, k_weight, slots, k_cache, v_cache, talk)
    nq, nkv, d, dv = int(num_heads), int(num_kv_heads), int(head_dim), int(value_dim)
    C = nq * d + nkv * d + nkv * dv
    if qkv.dim() != 2 or qkv.shape[1] < C or qkv.stride(1) != 1:
        raise KernelError(f"conv_qkv_rows: rows {tuple(qkv.shape)} do not hold {C} channels")
    T = qkv.shape[0]
    stride = int(qkv.stride(0)) if T > 1 else int(qkv.shape[1])
    taps = 1
    tail_stride = 0
    if conv_weight is not None:
        _want(conv_weight, torch.float32, "conv_qkv_rows: the convolution's weight")
        if conv_weight.dim() != 2 or conv_weight.shape[0] != C or not conv_weight.is_contiguous():
            raise KernelError(f"conv_qkv_rows: the convolution's weight {tuple(conv_weight.shape)} must be [{C}, taps]")
        taps = int(conv_weight.shape[1])
    if taps > 1:
        if tails is None:
            raise KernelError("conv_qkv_rows: a convolution needs the requests' tails")
        _want(tails, torch.float32, "conv_qkv_rows: tails")
        _want(state_slots, torch.int64, "conv_qkv_rows: state_slots")
        _want(tok_seq, torch.int32, "conv_qkv_rows: tok_seq")
        _want(cu_q, torch.int32, "conv_qkv_rows: cu_q")
        if tails.dim() != 3 or tuple(tails.shape[1:]) != (taps - 1, C) or tails[0].stride() != (C, 1) or tok_seq.shape != (T,):
            raise KernelError(f"conv_qkv_rows: tails {tuple(tails.shape)} must be [slots, {taps - 1}, {C}] with whole slots")
        tail_stride = int(tails.stride(0)) if tails.shape[0] > 1 else (taps - 1) * C
    for w, n in ((q_weight, nq * d), (k_weight, nkv * d)):
        if w is not None:
            _want(w, torch.float32, "conv_qkv_rows: norm weight")
            if w.shape != (n,):
                raise KernelError(f"conv_qkv_rows: norm weight {tuple(w.shape)} is not [{n}]")
    if (q_weight is None) != (k_weight is None):
        raise KernelError("conv_qkv_rows: q and k norm weights come together")
    _want(slots, torch.int64, "conv_qkv_rows: slots")
    if slots.shape != (T,):
        raise KernelError("conv_qkv_rows: slots must be [T]")
    if talk is not None:
        _want(talk, torch.float32, "conv_qkv_rows: talk")
        if tuple(talk.shape) != (nq, nq) or not talk.is_contiguous():
            raise KernelError(f"conv_qkv_rows: talk {tuple(talk.shape)} must be [{nq}, {nq}]")
        _check_cache(k_cache, v_cache, nkv, nkv * d, qkv.dtype, v_grouped, "conv_qkv_rows", dv=dv, key_heads=1)
        q_out = torch.empty((T, nq, nkv * d), dtype=qkv.dtype, device=qkv.device)
    else:
        _check_cache(k_cache, v_cache, nkv, d, qkv.dtype, v_grouped, "conv_qkv_rows", dv=dv)
        q_out = torch.empty((T, nq, d), dtype=qkv.dtype, device=qkv.device)
    _ok(lib().xi_conv_qkv_rows(_p(qkv), ctypes.c_longlong(stride), _code(qkv, "conv_qkv_rows"), _p(conv_weight), taps,
                               _p(tails if taps > 1 else None), ctypes.c_longlong(tail_stride),
                               _p(state_slots if taps > 1 else None), _p(tok_seq if taps > 1 else None),
                               _p(cu_q if taps > 1 else None), _p(q_weight), _p(k_weight), ctypes.c_float(eps),
                               int(bool(value_unit_norm)), _p(talk), _p(slots), _p(q_out), _p(k_cache), _p(v_cache),
                               int(k_cache.shape[2]), T, nq, nkv, d, dv, int(bool(v_grouped)), _stream()))
    return q_out


def head_gate_(x: torch.Tensor, gate: torch.Tensor, heads: int) -> torch.Tensor:
    """x [T, H dv] *= sigmoid(gate[t, h]) head by head, in place; gate [T, H] may be a column range of a packed
    projection, in x's type."""
    _dev(x)
    H = int(heads)
    if x.dim() != 2 or x.shape[1] % H or not x.is_contiguous():
        raise KernelError(f"head_gate: x {tuple(x.shape)} is not [T, {H} dv]")
    gs = _columns(gate, H, "head_gate: gate")
    if gate.shape[0] != x.shape[0] or gate.dtype != x.dtype or gate.device != x.device:
        raise KernelError("head_gate: the gate must be rows of the same tokens in x's type")
    _ok(lib().xi_head_gate(_p(x), _p(gate), ctypes.c_longlong(gs), _code(x, "head_gate"), int(x.shape[0]), H, int(x.shape[1]) // H,
                           _stream()))
    return x


def rows_rmsnorm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """x [T, n] (rows may be a column range of a packed projection, float32 or bfloat16) -> x * rsqrt(mean(x^2) + eps) *
    weight (float32 [n]; None: no weight) in `out_dtype`; float32 inside."""
    _dev(weight)
    if x.dim() != 2 or x.stride(1) != 1 or not x.is_cuda:
        raise KernelError(f"rows_rmsnorm: {tuple(x.shape)} with strides {x.stride()} is not rows")
    T, n = x.shape
    if weight is not None:
        _want(weight, torch.float32, "rows_rmsnorm: weight")
        if weight.shape != (n,):
            raise KernelError(f"rows_rmsnorm: weight {tuple(weight.shape)} is not [{n}]")
    out = torch.empty((T, n), dtype=out_dtype, device=x.device)
    stride = int(x.stride(0)) if T > 1 else n
    _ok(lib().xi_rows_rmsnorm(_p(x), ctypes.c_longlong(stride), _code(x, "rows_rmsnorm"), _p(weight), ctypes.c_float(eps), _p(out),
                              _code(out, "rows_rmsnorm"), int(T), int(n), _stream()))
    return out
