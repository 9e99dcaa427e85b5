"""Typed Python wrappers around the HIP kernels.

Each wrapper checks on the host what the kernel assumes about its operands
(device, dtype, strides, sizes) and launches on torch's current HIP stream, so
the calls can be captured into a HIP graph like any other stream work.
"""
from __future__ import annotations

import ctypes

import numpy as np
import torch

from . import lib

F32, BF16 = 0, 1


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return F32
    if dt == torch.bfloat16:
        return BF16
    raise TypeError(f"kernels take float32 or bfloat16 storage, not {dt}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current HIP stream of the current device (also under graph capture, which switches it)."""
    if _raw_stream is not None:  # the handle alone: a tenth of the cost of building a Stream object per launch
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _need_gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise lib.KernelError("kernel operands must live on the GPU; there is no CPU path")


def _ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


def _rows(t: torch.Tensor) -> int:
    """Row stride of a 2-D tensor whose rows are contiguous."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"expected a 2-D tensor with contiguous rows, got shape {tuple(t.shape)} stride {t.stride()}")
    return t.stride(0)


def _is_param_f32(w: torch.Tensor, act_dtype: torch.dtype) -> int:
    if w.dtype == torch.float32:
        return 1
    if w.dtype != act_dtype:
        raise TypeError(f"a parameter vector must be float32 or the activation dtype {act_dtype}, not {w.dtype}")
    return 0


def embedding(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, src: torch.Tensor | None = None,
              last: torch.Tensor | None = None, scale: float = 1.0) -> torch.Tensor:
    """out[t] = table[ids[t]] * scale; ids int32 [T], table [V, W], out [T, W] (out may be float32 beside a bfloat16 table). src, last (int32, both or neither): where
    src[t] >= 0 the id is last[src[t]], a token the step before sampled, which only the device knows so far."""
    _need_gpu(ids, table, out, src, last)
    assert ids.dtype == torch.int32 and ids.is_contiguous()
    assert (src is None) == (last is None)
    if src is not None:
        assert src.dtype == last.dtype == torch.int32 and src.numel() >= ids.numel()
    assert table.is_contiguous() and out.is_contiguous()
    T = ids.numel()
    V, W = table.shape
    assert out.shape[0] >= T and out.shape[1] == W
    if scale != 1.0 or table.dtype != out.dtype:     # a stream wider than the table, or a multiplied embedding
        lib.call("dinfer_embedding_to", dtype_code(table.dtype), dtype_code(out.dtype), ids.data_ptr(), table.data_ptr(),
                 out.data_ptr(), T, V, W, float(scale), _ptr(src), _ptr(last), _stream())
        return out
    lib.call("dinfer_embedding", dtype_code(table.dtype), ids.data_ptr(), table.data_ptr(), out.data_ptr(), T, V, W,
             _ptr(src), _ptr(last), _stream())
    return out


GATED_ACTS = {"silu": 0, "gelu_tanh": 2}   # activations the gated kernels know -> their code in the C interface
MAX_HEAD_DIM = 512         # the largest head the norm / rotation / plain attention kernels hold in registers


def gated_act(gate_up: torch.Tensor, out: torch.Tensor, tokens: int, act: str = "silu") -> torch.Tensor:
    """out[t, i] = act(gate_up[t, i]) * gate_up[t, I + i]."""
    _need_gpu(gate_up, out)
    if act not in GATED_ACTS:
        raise lib.KernelError(f"gated activation {act!r} has no kernel (known: {sorted(GATED_ACTS)})")
    inter = out.shape[1]
    assert gate_up.shape[1] == 2 * inter and gate_up.dtype == out.dtype and out.is_contiguous()
    assert gate_up.shape[0] >= tokens and out.shape[0] >= tokens
    lib.call("dinfer_gated_act", dtype_code(out.dtype), GATED_ACTS[act], gate_up.data_ptr(), out.data_ptr(), tokens, inter,
             _rows(gate_up), _stream())
    return out


def add_inplace(dst: torch.Tensor, src: torch.Tensor, n: int | None = None) -> None:
    """dst[:n] += src[:n] (flat), summed in float and rounded once."""
    _need_gpu(dst, src)
    assert dst.dtype == src.dtype and dst.is_contiguous() and src.is_contiguous()
    n = dst.numel() if n is None else n
    assert n <= dst.numel() and n <= src.numel()
    lib.call("dinfer_add_inplace", dtype_code(dst.dtype), dst.data_ptr(), src.data_ptr(), n, _stream())


def scale_softcap(x: torch.Tensor, rows: int, scale: float = 1.0, cap: float | None = None) -> None:
    """In place on the first `rows` rows of x: x *= scale, then x = cap * tanh(x / cap) where a cap is given."""
    _need_gpu(x)
    assert x.shape[0] >= rows
    lib.call("dinfer_scale_softcap", dtype_code(x.dtype), x.data_ptr(), _rows(x), rows, x.shape[1], float(scale),
             float(cap) if cap else 0.0, _stream())


def widen(src: torch.Tensor, dst: torch.Tensor, n: int | None = None) -> None:
    _need_gpu(src, dst)
    assert dst.dtype == torch.float32 and dst.is_contiguous() and src.is_contiguous()
    n = src.numel() if n is None else n
    lib.call("dinfer_widen", dtype_code(src.dtype), src.data_ptr(), dst.data_ptr(), n, _stream())


def fill_zero(t: torch.Tensor) -> None:
    """Zero-fills a tensor with a kernel (safe inside a captured graph)."""
    _need_gpu(t)
    nbytes = t.numel() * t.element_size()
    assert t.is_contiguous() and nbytes % 4 == 0 and t.data_ptr() % 4 == 0
    lib.call("dinfer_fill_u32", t.data_ptr(), 0, nbytes // 4, _stream())


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, eps: float, n_rows: int, *,
            residual: torch.Tensor | None = None, rows: torch.Tensor | None = None,
            weight_offset: float = 0.0) -> torch.Tensor:
    """out[r] = rmsnorm(x[src(r)]) * (weight + weight_offset).

    residual: updated in place to round(x + residual) first, and that sum is normed.
    rows: int32 indices of the n_rows source rows (gather); default identity.
    """
    _need_gpu(x, weight, out, residual, rows)
    width = out.shape[1]
    assert x.shape[1] == width and weight.numel() == width and weight.is_contiguous() and out.is_contiguous()
    assert x.dtype == out.dtype and out.shape[0] >= n_rows
    if rows is None:
        assert x.shape[0] >= n_rows
    else:
        assert rows.dtype == torch.int32 and rows.is_contiguous() and rows.numel() >= n_rows
    if residual is not None:
        assert residual.dtype == x.dtype and residual.shape == x.shape
    lib.call("dinfer_rmsnorm", dtype_code(x.dtype), x.data_ptr(), _ptr(residual), _ptr(rows), weight.data_ptr(),
             _is_param_f32(weight, x.dtype), out.data_ptr(), n_rows, width, _rows(x),
             _rows(residual) if residual is not None else 0, float(eps), float(weight_offset), _stream())
    return out


# activations of one argument -> their code in the C interface ("gelu": with the error function)
ACTS = {"silu": 0, "relu2": 1, "gelu_tanh": 2, "gelu": 3, "sigmoid": 4, "tanh": 5}


def act(x: torch.Tensor, out: torch.Tensor, tokens: int, kind: str) -> torch.Tensor:
    """out[t, i] = act(x[t, i]); out may be x."""
    _need_gpu(x, out)
    if kind not in ACTS:
        raise lib.KernelError(f"activation {kind!r} has no kernel (known: {sorted(ACTS)})")
    n = out.shape[1]
    assert x.shape[1] == n and x.dtype == out.dtype and x.shape[0] >= tokens and out.shape[0] >= tokens
    lib.call("dinfer_act", dtype_code(x.dtype), ACTS[kind], x.data_ptr(), _rows(x), out.data_ptr(), _rows(out), tokens, n,
             _stream())
    return out


def gate(x: torch.Tensor, g: torch.Tensor, tokens: int, kind: str, group: int = 1) -> torch.Tensor:
    """x[t, i] *= act(g[t, i // group]) in place; x and g are views (blocks of wider buffers), g of a `group`-th of
    x's columns: one gate for every `group` consecutive columns (a head), or one each."""
    _need_gpu(x, g)
    if kind not in ACTS:
        raise lib.KernelError(f"activation {kind!r} has no kernel (known: {sorted(ACTS)})")
    n = x.shape[1]
    assert group >= 1 and g.shape[1] * group == n and x.dtype == g.dtype and x.shape[0] >= tokens and g.shape[0] >= tokens
    lib.call("dinfer_gate", dtype_code(x.dtype), ACTS[kind], x.data_ptr(), _rows(x), g.data_ptr(), _rows(g), tokens, n,
             group, _stream())
    return x


def token_shift(x: torch.Tensor, out: torch.Tensor, state: torch.Tensor, mix: torch.Tensor, *, cu_seqlens: torch.Tensor,
                seq_lens: torch.Tensor, state_slots: torch.Tensor, num_reqs: int, max_rows: int) -> torch.Tensor:
    """out[t] = x[t] + (x of the token before - x[t]) * mix, per request: inside a portion the row above, for its first
    row the request's kept row state[slot] (zeros where the request starts), which then takes the portion's last row.
    state [slots, width] in x's dtype, mix float32 [width]; max_rows: the longest portion of the step."""
    _need_gpu(x, out, state, mix, cu_seqlens, seq_lens, state_slots)
    width = mix.numel()
    assert mix.dtype == torch.float32 and mix.is_contiguous()
    assert x.dtype == out.dtype == state.dtype and state.is_contiguous() and state.shape[1] == width
    assert x.shape[1] >= width and out.shape[1] >= width and x.data_ptr() != out.data_ptr()
    assert cu_seqlens.dtype == seq_lens.dtype == state_slots.dtype == torch.int32
    lib.call("dinfer_token_shift", dtype_code(x.dtype), x.data_ptr(), _rows(x), out.data_ptr(), _rows(out),
             state.data_ptr(), mix.data_ptr(), cu_seqlens.data_ptr(), seq_lens.data_ptr(), state_slots.data_ptr(),
             num_reqs, max_rows, width, _stream())
    return out


def layernorm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor, eps: float,
              n_rows: int, *, residual: torch.Tensor | None = None, rows: torch.Tensor | None = None) -> torch.Tensor:
    """out[r] = (x[src r] - mean) / sqrt(var + eps) * weight + bias, in float. residual: updated in place to
    round(x + residual) in its own type first (it may be float32 beside a bfloat16 x), and that sum is normed.
    rows: int32 indices of the n_rows source rows; default identity."""
    _need_gpu(x, weight, bias, out, residual, rows)
    width = out.shape[1]
    assert x.shape[1] == width and weight.numel() == width and weight.is_contiguous() and out.is_contiguous()
    assert bias is None or (bias.numel() == width and bias.is_contiguous() and bias.dtype == weight.dtype)
    assert out.shape[0] >= n_rows
    if rows is None:
        assert x.shape[0] >= n_rows
    else:
        assert rows.dtype == torch.int32 and rows.is_contiguous() and rows.numel() >= n_rows
    if residual is not None:
        assert residual.shape == x.shape
    lib.call("dinfer_layernorm", x.data_ptr(), dtype_code(x.dtype), _ptr(residual),
             dtype_code(residual.dtype) if residual is not None else 0, _ptr(rows), weight.data_ptr(), _ptr(bias),
             dtype_code(weight.dtype), out.data_ptr(), dtype_code(out.dtype), n_rows, width, _rows(x),
             _rows(residual) if residual is not None else 0, float(eps), _stream())
    return out


def rmsnorm_stream(stream: torch.Tensor, n_rows: int, *, branch: torch.Tensor | None = None,
                   branch_weight: torch.Tensor | None = None, branch_eps: float = 0.0, branch_offset: float = 0.0,
                   mult: float = 1.0, out: torch.Tensor | None = None, weight: torch.Tensor | None = None,
                   eps: float = 0.0, offset: float = 0.0, rows: torch.Tensor | None = None) -> torch.Tensor | None:
    """With a branch: stream += mult * rmsnorm(branch) * (branch_weight + branch_offset), in place. With an out:
    out[r] = rmsnorm(stream[src r]) * (weight + offset). rows: int32 source rows (both steps act on those rows only).
    Stream, branch and out may each be float32 or bfloat16; the two weights share a type."""
    _need_gpu(stream, branch, branch_weight, out, weight, rows)
    width = stream.shape[1]
    params = [t for t in (branch_weight, weight) if t is not None]
    assert params and all(t.dtype == params[0].dtype and t.numel() == width and t.is_contiguous() for t in params)
    if branch is not None:
        assert branch_weight is not None and branch.shape[1] == width
    if out is not None:
        assert weight is not None and out.is_contiguous() and out.shape[1] == width and out.shape[0] >= n_rows
    if rows is not None:
        assert rows.dtype == torch.int32 and rows.is_contiguous() and rows.numel() >= n_rows
    else:
        assert stream.shape[0] >= n_rows and (branch is None or branch.shape[0] >= n_rows)
    lib.call("dinfer_rmsnorm_stream", _ptr(branch), dtype_code(branch.dtype) if branch is not None else 0,
             _rows(branch) if branch is not None else 0, _ptr(branch_weight), float(branch_eps), float(branch_offset),
             float(mult), stream.data_ptr(), dtype_code(stream.dtype), _rows(stream), _ptr(rows), _ptr(weight),
             dtype_code(params[0].dtype), _ptr(out), dtype_code(out.dtype) if out is not None else 0, float(eps),
             float(offset), n_rows, width, _stream())
    return out


def axpby(a: torch.Tensor, alpha: float, b: torch.Tensor, beta: float, out: torch.Tensor, rows: int) -> torch.Tensor:
    """out[:rows] = alpha * a[:rows] + beta * b[:rows]; out may be a or b."""
    _need_gpu(a, b, out)
    cols = out.shape[1]
    assert a.shape[1] == cols and b.shape[1] == cols and a.dtype == b.dtype == out.dtype
    assert min(a.shape[0], b.shape[0], out.shape[0]) >= rows
    done = 0
    while done < rows:      # (the launch takes up to 65,535 rows)
        n = min(rows - done, 65535)
        lib.call("dinfer_axpby", dtype_code(a.dtype), a[done:].data_ptr(), _rows(a), float(alpha), b[done:].data_ptr(),
                 _rows(b), float(beta), out[done:].data_ptr(), _rows(out), n, cols, _stream())
        done += n
    return out


def add_rows(x: torch.Tensor, rows: int, a: torch.Tensor | None = None, vec: torch.Tensor | None = None) -> None:
    """x[:rows] += a[:rows] + vec (each optional), float arithmetic, one rounding."""
    _need_gpu(x, a, vec)
    width = x.shape[1]
    assert x.shape[0] >= rows and (a is None or (a.shape[1] == width and a.shape[0] >= rows))
    assert vec is None or (vec.numel() == width and vec.is_contiguous())
    done = 0
    while done < rows:
        n = min(rows - done, 65535)
        lib.call("dinfer_add_rows", x[done:].data_ptr(), dtype_code(x.dtype), _rows(x),
                 a[done:].data_ptr() if a is not None else None, dtype_code(a.dtype) if a is not None else 0,
                 _rows(a) if a is not None else 0, _ptr(vec), dtype_code(vec.dtype) if vec is not None else 0, n, width,
                 _stream())
        done += n


# ---- gated delta rule ----------------------------------------------------------------------------
DELTA_MAX_DIM = 256      # the largest key size of the recurrence kernel (a thread holds 32 rows of a column)
DELTA_MAX_HEAD = 512     # the largest key or value size of the kernels around it
DELTA_MAX_TAPS = 16


def delta_work_columns(qk_heads: int, heads: int, dim: int, vdim: int) -> int:
    """Columns of the float rows between the delta rule's kernels: q | k | v | step sizes | decays."""
    return 2 * qk_heads * dim + heads * vdim + 2 * heads


def delta_prep(proj: torch.Tensor, tokens: int, *, qkv_off: int, b_off: int, a_off: int, taps: torch.Tensor,
               a_log: torch.Tensor, dt_bias: torch.Tensor, conv_state: torch.Tensor | None, state_slots: torch.Tensor,
               cu_seqlens: torch.Tensor, seq_lens: torch.Tensor, work: torch.Tensor, num_reqs: int, qk_heads: int,
               heads: int, dim: int, vdim: int, eps: float, q_scale: float, taps_t: torch.Tensor | None = None) -> None:
    """Short convolution (over the step's rows and the request's stored inputs), silu, unit q and k, step sizes and
    decays: proj [T, *] -> work [T, delta_work_columns] float32. taps_t: the taps transposed [K, channels]; with them
    the kernel that takes 8 channels a lane serves the sizes it fits."""
    _need_gpu(proj, taps, a_log, dt_bias, conv_state, state_slots, cu_seqlens, seq_lens, work)
    C = 2 * qk_heads * dim + heads * vdim
    K = taps.shape[1]
    assert taps.dtype == torch.float32 and tuple(taps.shape) == (C, K) and taps.is_contiguous()
    assert a_log.dtype == dt_bias.dtype == torch.float32 and a_log.numel() == heads == dt_bias.numel()
    assert work.dtype == torch.float32 and work.shape[0] >= tokens and work.shape[1] >= C + 2 * heads
    assert proj.shape[0] >= tokens and max(qkv_off + C, b_off + heads, a_off + heads) <= proj.shape[1]
    if K > 1:
        assert conv_state is not None and conv_state.dtype == proj.dtype and conv_state.is_contiguous()
        assert tuple(conv_state.shape[1:]) == (C, K - 1)
    if taps_t is not None:
        assert taps_t.dtype == torch.float32 and tuple(taps_t.shape) == (K, C) and taps_t.is_contiguous()
    lib.call("dinfer_delta_prep", dtype_code(proj.dtype), proj.data_ptr(), _rows(proj), qkv_off, b_off, a_off,
             taps.data_ptr(), _ptr(taps_t), a_log.data_ptr(), dt_bias.data_ptr(), _ptr(conv_state) if K > 1 else None,
             state_slots.data_ptr(), cu_seqlens.data_ptr(), seq_lens.data_ptr(), work.data_ptr(), _rows(work), num_reqs,
             tokens, qk_heads, heads, dim, vdim, K, float(eps), float(q_scale), _stream())


def delta_conv_update(proj: torch.Tensor, *, qkv_off: int, conv_state: torch.Tensor, state_slots: torch.Tensor,
                      cu_seqlens: torch.Tensor, seq_lens: torch.Tensor, num_reqs: int) -> None:
    """The step's last taps - 1 inputs a channel become the request's stored inputs (run after delta_prep)."""
    _need_gpu(proj, conv_state, state_slots, cu_seqlens, seq_lens)
    _, C, K1 = conv_state.shape
    if K1 == 0:
        return
    assert conv_state.dtype == proj.dtype and conv_state.is_contiguous() and qkv_off + C <= proj.shape[1]
    lib.call("dinfer_delta_conv_update", dtype_code(proj.dtype), proj.data_ptr(), _rows(proj), qkv_off,
             conv_state.data_ptr(), state_slots.data_ptr(), cu_seqlens.data_ptr(), seq_lens.data_ptr(), num_reqs, C,
             K1 + 1, _stream())


def delta_recurrence(work: torch.Tensor, state: torch.Tensor, out: torch.Tensor, *, state_slots: torch.Tensor,
                     cu_seqlens: torch.Tensor, seq_lens: torch.Tensor, num_reqs: int, qk_heads: int, heads: int,
                     dim: int, vdim: int) -> torch.Tensor:
    """The recurrence over each request's rows of the step. state [slots, heads, vdim, dim] float32 (a head's matrix
    transposed), updated in place; out [T, heads * vdim] float32."""
    _need_gpu(work, state, out, state_slots, cu_seqlens, seq_lens)
    assert work.dtype == state.dtype == out.dtype == torch.float32 and state.is_contiguous()
    assert tuple(state.shape[1:]) == (heads, vdim, dim) and out.shape[1] >= heads * vdim
    assert work.shape[1] >= delta_work_columns(qk_heads, heads, dim, vdim)
    lib.call("dinfer_delta_recurrence", work.data_ptr(), _rows(work), state.data_ptr(), state_slots.data_ptr(),
             cu_seqlens.data_ptr(), seq_lens.data_ptr(), out.data_ptr(), _rows(out), num_reqs, qk_heads, heads, dim, vdim,
             _stream())
    return out


def delta_out(o: torch.Tensor, proj: torch.Tensor, g_off: int, weight: torch.Tensor, out: torch.Tensor, tokens: int, *,
              heads: int, vdim: int, eps: float, col_off: int = 0, out_scale: float = 1.0, gate: str = "silu") -> torch.Tensor:
    """out[t, col_off + h vdim + d] = o / rms_d(o) * weight[d] * silu(proj[t, g_off + h vdim + d]) * out_scale.
    weight of heads * vdim entries: a head's own gains at h vdim. gate: "silu" or "sigmoid"."""
    _need_gpu(o, proj, weight, out)
    per_head = weight.numel() == heads * vdim and heads > 1
    assert gate in ("silu", "sigmoid")
    assert o.dtype == torch.float32 and weight.dtype == torch.float32 and (per_head or weight.numel() == vdim)
    assert proj.dtype == out.dtype and min(o.shape[0], proj.shape[0], out.shape[0]) >= tokens
    assert g_off + heads * vdim <= proj.shape[1] and col_off + heads * vdim <= out.shape[1]
    lib.call("dinfer_delta_out", dtype_code(out.dtype), o.data_ptr(), _rows(o), proj.data_ptr(), _rows(proj), g_off,
             weight.data_ptr(), out.data_ptr(), _rows(out), col_off, tokens, heads, vdim, float(eps), float(out_scale),
             int(per_head), 1 if gate == "sigmoid" else 0, _stream())
    return out


# ---- delta rule with a decay and a removal rate a key channel ----------------------------------------
CHANNEL_DELTA_MAX_LOW = 512     # the largest inner size of the decay's low-rank projection


def channel_delta_work_columns(heads: int, dim: int) -> int:
    """Columns of the float rows between the two kernels: r * w | u | k | w | a * u | v | c1 | c2."""
    return 6 * heads * dim + 2 * heads


def channel_delta_prep(proj: torch.Tensor, tokens: int, *, r_off: int, k_off: int, v_off: int, a_off: int, low_off: int,
                       a_bias: torch.Tensor, w2: torch.Tensor, w0: torch.Tensor, work: torch.Tensor, heads: int, dim: int,
                       eps: float, rate: float, z: torch.Tensor | None = None) -> None:
    """From the step's projections: the unit key u = k / sqrt(sum k^2 + eps), the removal rate a = sigmoid(. + a_bias),
    the decay w = exp(-rate * sigmoid(w2 tanh(low) + w0)), and what the recurrence reads of them, in float32.
    z: float32 [T, heads * dim], w2 tanh(low) where the caller has made it by a matrix product of its own."""
    _need_gpu(proj, a_bias, w2, w0, work, z)
    if z is not None:
        assert z.dtype == torch.float32 and z.shape[0] >= tokens and z.shape[1] >= heads * dim
    hd = heads * dim
    low = w2.shape[1]
    assert a_bias.dtype == w2.dtype == w0.dtype == torch.float32 and w2.is_contiguous()
    assert a_bias.numel() == hd == w0.numel() and w2.shape[0] == hd
    assert work.dtype == torch.float32 and work.shape[0] >= tokens and work.shape[1] >= channel_delta_work_columns(heads, dim)
    assert proj.shape[0] >= tokens and max(r_off, k_off, v_off, a_off) + hd <= proj.shape[1] and low_off + low <= proj.shape[1]
    lib.call("dinfer_channel_delta_prep", dtype_code(proj.dtype), proj.data_ptr(), _rows(proj), r_off, k_off, v_off, a_off,
             low_off, a_bias.data_ptr(), w2.data_ptr(), w0.data_ptr(), low, work.data_ptr(), _rows(work), tokens, heads,
             dim, float(eps), float(rate), _ptr(z), _rows(z) if z is not None else 0, _stream())


def channel_delta_recurrence(work: torch.Tensor, state: torch.Tensor, out: torch.Tensor, *, state_slots: torch.Tensor,
                             cu_seqlens: torch.Tensor, seq_lens: torch.Tensor, num_reqs: int, heads: int,
                             dim: int) -> torch.Tensor:
    """S <- diag(w) S - (a u)(u^T S) + k v^T, o = S^T r over each request's rows of the step. state [slots, heads, dim,
    dim] float32 (a head's matrix transposed), updated in place; out [T, heads * dim] float32."""
    _need_gpu(work, state, out, state_slots, cu_seqlens, seq_lens)
    assert work.dtype == state.dtype == out.dtype == torch.float32 and state.is_contiguous()
    assert tuple(state.shape[1:]) == (heads, dim, dim) and out.shape[1] >= heads * dim
    assert work.shape[1] >= channel_delta_work_columns(heads, dim)
    lib.call("dinfer_channel_delta_recurrence", work.data_ptr(), _rows(work), state.data_ptr(), state_slots.data_ptr(),
             cu_seqlens.data_ptr(), seq_lens.data_ptr(), out.data_ptr(), _rows(out), num_reqs, heads, dim, _stream())
    return out


# ---- recurrences with a scalar decay ---------------------------------------------------------------
DECAY_MAX_DIM = 256      # the largest key size of the recurrence kernel


def rot_widen(proj: torch.Tensor, tokens: int, *, q_off: int, k_off: int, v_off: int, positions: torch.Tensor,
              cos_sin: torch.Tensor | None, rotary_dim: int, k_scale: float, work: torch.Tensor, heads: int, dim: int,
              vdim: int) -> torch.Tensor:
    """work[t] = rotated q (heads dim) | rotated k * k_scale | v (heads vdim), float32; the first rotary_dim entries
    of a head turn in pairs (i, i + rotary_dim / 2) by the table row [cos | sin] of the token's position."""
    _need_gpu(proj, positions, cos_sin, work)
    assert work.dtype == torch.float32 and work.shape[0] >= tokens and work.shape[1] >= heads * (2 * dim + vdim)
    assert proj.shape[0] >= tokens and max(q_off + heads * dim, k_off + heads * dim, v_off + heads * vdim) <= proj.shape[1]
    assert positions.dtype == torch.int32 and positions.numel() >= tokens
    if cos_sin is not None:
        assert cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.shape[1] == rotary_dim
    lib.call("dinfer_rot_widen", dtype_code(proj.dtype), proj.data_ptr(), _rows(proj), q_off, k_off, v_off,
             positions.data_ptr(), _ptr(cos_sin), rotary_dim if cos_sin is not None else 0, float(k_scale), work.data_ptr(),
             _rows(work), tokens, heads, dim, vdim, _stream())
    return work


def conv_silu(proj: torch.Tensor, tokens: int, *, x_off: int, dt_off: int, taps: torch.Tensor, bias: torch.Tensor | None,
              a_log: torch.Tensor, dt_bias: torch.Tensor, conv_state: torch.Tensor | None, state_slots: torch.Tensor,
              cu_seqlens: torch.Tensor, seq_lens: torch.Tensor, work: torch.Tensor, num_reqs: int) -> torch.Tensor:
    """Short causal convolution with bias over the step's rows and the request's stored inputs, then silu, for the
    C = taps.shape[0] channels from column x_off; step sizes dt = softplus(proj[dt_off + h] + dt_bias[h]) and decays
    exp(-exp(a_log[h]) dt). work [T, >= C + 2 H] float32: channels | dt | decay."""
    _need_gpu(proj, taps, bias, a_log, dt_bias, conv_state, state_slots, cu_seqlens, seq_lens, work)
    C, K = taps.shape
    H = a_log.numel()
    assert taps.dtype == torch.float32 and taps.is_contiguous() and a_log.dtype == dt_bias.dtype == torch.float32
    assert dt_bias.numel() == H and (bias is None or (bias.dtype == torch.float32 and bias.numel() == C))
    assert work.dtype == torch.float32 and work.shape[0] >= tokens and work.shape[1] >= C + 2 * H
    assert proj.shape[0] >= tokens and max(x_off + C, dt_off + H) <= proj.shape[1]
    if K > 1:
        assert conv_state is not None and conv_state.dtype == proj.dtype and conv_state.is_contiguous()
        assert tuple(conv_state.shape[1:]) == (C, K - 1)
    lib.call("dinfer_conv_silu", dtype_code(proj.dtype), proj.data_ptr(), _rows(proj), x_off, dt_off, taps.data_ptr(),
             _ptr(bias), a_log.data_ptr(), dt_bias.data_ptr(), _ptr(conv_state) if K > 1 else None, state_slots.data_ptr(),
             cu_seqlens.data_ptr(), seq_lens.data_ptr(), work.data_ptr(), _rows(work), num_reqs, tokens, C, H, K, _stream())
    return work


def decay_recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, gain: torch.Tensor | None,
                     state: torch.Tensor, out: torch.Tensor, *, state_slots: torch.Tensor, cu_seqlens: torch.Tensor,
                     seq_lens: torch.Tensor, num_reqs: int, groups: int, heads: int, dim: int, vdim: int) -> torch.Tensor:
    """Per request and head, token by token: S <- decay S + gain k v^T, out = S^T q. q, k: float32 views [T, groups dim]
    (head h reads group h // (heads / groups)); v [T, heads vdim]; decay [T, heads], or [heads] for one decay a head;
    gain [T, heads] or None. state [slots, heads, vdim, dim] float32, updated in place; out [T, >= heads vdim] float32."""
    _need_gpu(q, k, v, decay, gain, state, out, state_slots, cu_seqlens, seq_lens)
    tensors = [q, k, v, decay, state, out] + ([gain] if gain is not None else [])
    assert all(t.dtype == torch.float32 for t in tensors) and state.is_contiguous()
    assert tuple(state.shape[1:]) == (heads, vdim, dim) and out.shape[1] >= heads * vdim
    assert q.shape[1] >= groups * dim and k.shape[1] >= groups * dim and v.shape[1] >= heads * vdim
    if decay.dim() == 1:
        assert decay.numel() == heads and decay.is_contiguous()
        ldd = 0
    else:
        assert decay.shape[1] >= heads
        ldd = _rows(decay)
    assert gain is None or gain.shape[1] >= heads
    lib.call("dinfer_decay_recurrence", q.data_ptr(), _rows(q), k.data_ptr(), _rows(k), v.data_ptr(), _rows(v),
             decay.data_ptr(), ldd, _ptr(gain), _rows(gain) if gain is not None else 0, state.data_ptr(),
             state_slots.data_ptr(), cu_seqlens.data_ptr(), seq_lens.data_ptr(), out.data_ptr(), _rows(out), num_reqs,
             groups, heads, dim, vdim, _stream())
    return out


def gated_group_norm(y: torch.Tensor, z: torch.Tensor, z_off: int, out: torch.Tensor, tokens: int, *, groups: int,
                     group: int, eps: float, weight: torch.Tensor | None = None, x: torch.Tensor | None = None,
                     skip: torch.Tensor | None = None, vdim: int = 0, col_off: int = 0, out_scale: float = 1.0,
                     gate_first: bool = True) -> torch.Tensor:
    """u = (y + skip[c // vdim] x) * silu(z[:, z_off + c]); out[:, col_off + c] = u / rms over c's group of `group`
    columns (eps inside the root) * weight[c] * out_scale. gate_first False: the gate multiplies after the norm
    instead. y, x float32; z and out in the activations' type."""
    _need_gpu(y, z, out, weight, x, skip)
    n = groups * group
    assert y.dtype == torch.float32 and y.shape[1] >= n and z.dtype == out.dtype
    assert min(y.shape[0], z.shape[0], out.shape[0]) >= tokens and z_off + n <= z.shape[1] and col_off + n <= out.shape[1]
    assert weight is None or (weight.dtype == torch.float32 and weight.numel() == n and weight.is_contiguous())
    if skip is not None:
        assert x is not None and x.dtype == torch.float32 and x.shape[1] >= n and x.shape[0] >= tokens
        assert skip.dtype == torch.float32 and vdim > 0 and skip.numel() * vdim == n
    lib.call("dinfer_gated_group_norm", dtype_code(out.dtype), y.data_ptr(), _rows(y), _ptr(x) if skip is not None else None,
             _rows(x) if skip is not None else 0, _ptr(skip), int(vdim), z.data_ptr(), _rows(z), z_off, _ptr(weight),
             out.data_ptr(), _rows(out), col_off, tokens, groups, group, float(eps), float(out_scale), 1 if gate_first else 0, _stream())
    return out


# ---- several residual streams ----------------------------------------------------------------------
STREAMS_MAX = 8          # streams a token the kernel holds in registers
STREAMS_MAX_WIDTH = 12288


def streams_expand(src: torch.Tensor, x: torch.Tensor, tokens: int, n: int) -> torch.Tensor:
    """x[t, s W + c] = src[t, c] for every stream s < n; x float32 [T, n W]."""
    _need_gpu(src, x)
    W = src.shape[1]
    assert x.dtype == torch.float32 and x.shape[1] == n * W and min(src.shape[0], x.shape[0]) >= tokens
    lib.call("dinfer_streams_expand", dtype_code(src.dtype), src.data_ptr(), _rows(src), x.data_ptr(), _rows(x), tokens, n,
             W, _stream())
    return x


def streams_step(x: torch.Tensor, n_rows: int, n: int, *, dtype: torch.dtype, branch: torch.Tensor | None = None,
                 mix: torch.Tensor | None = None, out_weights: torch.Tensor | None = None,
                 read: torch.Tensor | None = None, gain: torch.Tensor | None = None, bias: torch.Tensor | None = None,
                 eps: float = 0.0, out: torch.Tensor | None = None, u_out: torch.Tensor | None = None,
                 rows: torch.Tensor | None = None):
    """One pass over the rows of x (float32 [T, n W], n streams side by side): with a branch y [T, W],
    x_t <- sum_s mix[s, t] x_s + out_weights[t] y for all streams at once; with `read`, u = sum_s read[s] x_s, which goes
    to u_out (float32) as it is, or, with gain (and bias), through a layer norm to out (in `dtype`, the type of branch
    and out). rows: int32 source rows; then the streams themselves stay as they are."""
    _need_gpu(x, branch, mix, out_weights, read, gain, bias, out, u_out, rows)
    W = x.shape[1] // n
    assert x.dtype == torch.float32 and x.shape[1] == n * W
    small = [t for t in (mix, out_weights, read, gain, bias) if t is not None]
    assert all(t.dtype == torch.float32 and t.is_contiguous() for t in small)
    if branch is not None:
        assert branch.dtype == dtype and branch.shape[1] == W and mix.numel() == n * n and out_weights.numel() == n
        assert rows is not None or branch.shape[0] >= n_rows
    if read is not None:
        assert read.numel() == n
        if gain is not None:
            assert gain.numel() == W and (bias is None or bias.numel() == W)
            assert out is not None and out.dtype == dtype and out.shape[1] == W and out.shape[0] >= n_rows
        else:
            assert u_out is not None and u_out.dtype == torch.float32 and u_out.shape[1] == W and u_out.shape[0] >= n_rows
    if rows is not None:
        assert rows.dtype == torch.int32 and rows.is_contiguous() and rows.numel() >= n_rows
    else:
        assert x.shape[0] >= n_rows
    lib.call("dinfer_streams_step", dtype_code(dtype), x.data_ptr(), _rows(x), n, W, _ptr(rows), _ptr(branch),
             _rows(branch) if branch is not None else 0, _ptr(mix), _ptr(out_weights), _ptr(read), _ptr(gain), _ptr(bias),
             float(eps), _ptr(out), _rows(out) if out is not None else 0, _ptr(u_out),
             _rows(u_out) if u_out is not None else 0, n_rows, _stream())
    return out if gain is not None else u_out


# ---- latent attention ----------------------------------------------------------------------------
# Cache pages [blocks, page, R + dr]: one row a token, the normed latent and then the rotated shared key part.
LATENT_MAX_RANK = 1024   # the largest latent the attention kernels hold in registers
LATENT_MAX_KEY = 1280    # the largest latent + rotated part


def latent_cache_shape(blocks: int, page_size: int, rank: int, rot_dim: int) -> tuple:
    return (blocks, page_size, rank + rot_dim)


def latent_post(proj: torch.Tensor, tokens: int, *, heads: int, dim: int, rot_dim: int, rank: int, q_off: int,
                c_off: int | None, gain: torch.Tensor | None, eps: float, positions: torch.Tensor,
                cos_sin: torch.Tensor | None, rotary_dim: int, qa: torch.Tensor, cache: torch.Tensor | None,
                slot_mapping: torch.Tensor | None, cache_t: torch.Tensor | None = None, style: int = 1,
                q_src: torch.Tensor | None = None) -> None:
    """From the step's projections: every head's rotated query part goes, rotated, into qa (head h at h*(rank+rot_dim),
    behind the rank entries the caller fills), and, where the layer has a down projection of its own (c_off), the
    token's latent (RMS-normed with `gain`) and rotated shared key part go to its cache slot (the latent also into
    cache_t [blocks, rank, page], the pages transposed, where that is given). style: 1 turns pairs (2i, 2i+1), 0 pairs
    (i, i + rotary_dim/2). q_src: the queries come from this buffer (at its column q_off) instead of from proj."""
    _need_gpu(proj, gain, positions, cos_sin, qa, cache, slot_mapping, cache_t, q_src)
    assert proj.shape[0] >= tokens and qa.shape[0] >= tokens and qa.dtype == proj.dtype
    qs = proj if q_src is None else q_src
    assert qs.dtype == proj.dtype and qs.shape[0] >= tokens
    assert q_off + heads * (dim + rot_dim) <= qs.shape[1] and qa.shape[1] >= heads * (rank + rot_dim)
    assert positions.dtype == torch.int32 and positions.numel() >= tokens
    if cos_sin is not None:
        assert cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.shape[1] == rotary_dim
    write = c_off is not None and slot_mapping is not None
    if write:
        assert c_off + rank + rot_dim <= proj.shape[1] and gain is not None and gain.numel() == rank
        assert slot_mapping.dtype == torch.int64 and slot_mapping.numel() >= tokens
        assert cache is not None and cache.dtype == proj.dtype and cache.is_contiguous()
        assert cache.shape[-1] == rank + rot_dim and cache.dim() == 3
        if cache_t is not None:
            assert cache_t.dtype == cache.dtype and cache_t.is_contiguous()
            assert tuple(cache_t.shape) == (cache.shape[0], rank, cache.shape[1])
    lib.call("dinfer_latent_post", dtype_code(proj.dtype), proj.data_ptr(), tokens, _rows(proj), q_off,
             c_off if write else -1, heads, dim, rot_dim, rank, _ptr(gain) if write else 0,
             _is_param_f32(gain, proj.dtype) if write else 0, float(eps), positions.data_ptr(), _ptr(cos_sin),
             rotary_dim if cos_sin is not None else 0, qa.data_ptr(), _rows(qa), _ptr(cache) if write else 0,
             _ptr(cache_t) if write else 0, cache.shape[1] if write else 0, _ptr(slot_mapping) if write else 0,
             int(style), _ptr(q_src), _rows(q_src) if q_src is not None else 0, _stream())


def _check_latent(qa, out, cache, block_table, cu_seqlens, seq_lens, num_reqs, tokens, heads, rank, rot_dim, page_size):
    assert qa.dtype == out.dtype == cache.dtype and cache.is_contiguous()
    assert tuple(cache.shape[1:]) == (page_size, rank + rot_dim)
    assert block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous()
    assert block_table.shape[0] >= num_reqs
    assert cu_seqlens.dtype == torch.int32 and cu_seqlens.numel() >= num_reqs + 1
    assert seq_lens.dtype == torch.int32 and seq_lens.numel() >= num_reqs
    assert qa.shape[1] >= heads * (rank + rot_dim) and out.shape[1] >= heads * rank
    assert qa.shape[0] >= tokens and out.shape[0] >= tokens


def latent_attn_ref(qa: torch.Tensor, out: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor,
                    cu_seqlens: torch.Tensor, seq_lens: torch.Tensor, num_reqs: int, tokens: int, *, scale: float,
                    window: int, heads: int, rank: int, rot_dim: int, page_size: int) -> torch.Tensor:
    """Plain attention over the latent pages (any sizes, float arithmetic): out[t, h*rank : (h+1)*rank] = the
    softmax-weighted sum of the latents, scores scale * <qa[t, h], cache row>."""
    _need_gpu(qa, out, cache, block_table, cu_seqlens, seq_lens)
    _check_latent(qa, out, cache, block_table, cu_seqlens, seq_lens, num_reqs, tokens, heads, rank, rot_dim, page_size)
    lib.call("dinfer_latent_attn_ref", dtype_code(qa.dtype), qa.data_ptr(), _rows(qa), out.data_ptr(), _rows(out),
             cache.data_ptr(), block_table.data_ptr(), block_table.shape[1], cu_seqlens.data_ptr(), seq_lens.data_ptr(),
             num_reqs, tokens, float(scale), int(window), heads, rank, rot_dim, page_size, _stream())
    return out


def latent_mfma_supports(rank: int, rot_dim: int, page_size: int) -> bool:
    return bool(lib.get("dinfer_latent_mfma_supports")(rank, rot_dim, page_size))


def latent_attn_mfma(qa: torch.Tensor, out: torch.Tensor, cache: torch.Tensor, cache_t: torch.Tensor,
                     block_table: torch.Tensor, cu_seqlens: torch.Tensor, seq_lens: torch.Tensor, num_reqs: int,
                     tokens: int, splits: int, part: torch.Tensor | None, *, scale: float, window: int, heads: int,
                     rank: int, rot_dim: int, page_size: int) -> torch.Tensor:
    """latent_attn_ref on the matrix cores (bfloat16): cache_t [blocks, rank, page] holds the latents once more, the
    pages transposed. splits > 1 (steps in which every request brings one row): each request's keys are cut into that
    many parts on the device and merged; part: float32 scratch of tokens * heads * splits * (rank + 4)."""
    _need_gpu(qa, out, cache, cache_t, block_table, cu_seqlens, seq_lens, part)
    _check_latent(qa, out, cache, block_table, cu_seqlens, seq_lens, num_reqs, tokens, heads, rank, rot_dim, page_size)
    assert qa.dtype == torch.bfloat16 and cache_t.dtype == torch.bfloat16 and cache_t.is_contiguous()
    assert tuple(cache_t.shape) == (cache.shape[0], rank, page_size)
    if splits > 1:
        assert part is not None and part.dtype == torch.float32 and part.is_contiguous() and tokens == num_reqs
    lib.call("dinfer_latent_attn_mfma", qa.data_ptr(), _rows(qa), out.data_ptr(), _rows(out), _ptr(part),
             part.numel() if part is not None else 0, cache.data_ptr(), cache_t.data_ptr(), block_table.data_ptr(),
             block_table.shape[1], cu_seqlens.data_ptr(), seq_lens.data_ptr(), num_reqs, tokens, float(scale),
             int(window), heads, rank, rot_dim, page_size, int(splits), _stream())
    return out


# ---- many small products in one launch ---------------------------------------------------------------
def heads_nt(a: torch.Tensor, a_off: int, a_stride: int, w: torch.Tensor, out: torch.Tensor, c_off: int, c_stride: int,
             m: int, *, gate: torch.Tensor | None = None, gate_off: int = 0) -> torch.Tensor:
    """For every head z: out[:m, c_off + z*c_stride : ... + N] = a[:m, a_off + z*a_stride : ... + K] @ w[z].T with
    w [heads, N, K]; gate: the rows of head z are multiplied by sigmoid(gate[:, gate_off + z])."""
    _need_gpu(a, w, out, gate)
    heads, n, k = w.shape
    assert w.is_contiguous() and a.dtype == w.dtype == out.dtype
    assert a.shape[0] >= m and out.shape[0] >= m
    assert a_off + (heads - 1) * a_stride + k <= a.shape[1] and c_off + (heads - 1) * c_stride + n <= out.shape[1]
    es = a.element_size()
    if gate is not None:
        assert gate.dtype == a.dtype and gate.shape[0] >= m and gate_off + heads <= gate.shape[1]
    lib.call("dinfer_heads_nt", dtype_code(a.dtype), a.data_ptr() + a_off * es, _rows(a), a_stride, w.data_ptr(), k, n * k,
             out.data_ptr() + c_off * es, _rows(out), c_stride, m, n, k, heads,
             gate.data_ptr() + gate_off * es if gate is not None else 0, _rows(gate) if gate is not None else 0, _stream())
    return out


MOE_MAX_EXPERTS = 1024   # the routing and sorting kernels keep one number an expert in LDS
MOE_MAX_TOP = 64         # a lane of the routing wave keeps one choice


EXPERT_ACTS = {"silu": 2, "gelu": 3}    # activations the plain (not gated) expert products apply -> their code


def moe_tile_rows(dtype: torch.dtype, entries: int, experts: int, k_in: int, k_mid: int) -> int:
    """Rows of a row tile for the two products of a routed layer over `entries` (token, choice) pairs: what the kernel
    that will run them takes (16 where an expert gets few rows, 128 for many, 64 on the vector ALUs)."""
    return int(lib.get("dinfer_moe_tile_rows")(dtype_code(dtype), entries, experts, k_in, k_mid))


def moe_max_tiles(entries: int, experts: int, tile_rows: int) -> int:
    """Length of the work list for `entries` (token, choice) pairs: every expert may end with a tile that is not full."""
    return -(-entries // tile_rows) + experts


def moe_route(x: torch.Tensor, router: torch.Tensor, shared_gate_w: torch.Tensor | None, idx: torch.Tensor,
              share: torch.Tensor, shared_gate: torch.Tensor | None, tokens: int, top: int, z: torch.Tensor,
              all_scores: bool = False, correction: torch.Tensor | None = None) -> None:
    """Per token: logits x @ router.T in float (router float32 [experts, width]), idx[t] the `top` largest (lowest index
    among equals), share[t] the softmax over them; shared_gate[t] = sigmoid(x . shared_gate_w) where that is given.
    z: float32 scratch of tokens * (experts + 1) for the logits. all_scores: the scores are the softmax over all
    experts, the choice goes by score + correction (float32 [experts], or none) and share[t] holds the chosen scores
    as they are."""
    _need_gpu(x, router, shared_gate_w, idx, share, shared_gate, z, correction)
    if correction is not None:
        assert all_scores and correction.dtype == torch.float32 and correction.numel() == router.shape[0]
    experts, width = router.shape
    assert router.dtype == torch.float32 and router.is_contiguous() and x.shape[1] == width and x.shape[0] >= tokens
    assert idx.dtype == torch.int32 and share.dtype == torch.float32 and idx.is_contiguous() and share.is_contiguous()
    assert idx.numel() >= tokens * top and share.numel() >= tokens * top
    assert z.dtype == torch.float32 and z.is_contiguous() and z.numel() >= tokens * (experts + 1)
    if shared_gate_w is not None:
        assert shared_gate_w.dtype == torch.float32 and shared_gate_w.numel() == width and shared_gate_w.is_contiguous()
        assert shared_gate is None or (shared_gate.dtype == torch.float32 and shared_gate.numel() >= tokens)
    lib.call("dinfer_moe_route", dtype_code(x.dtype), x.data_ptr(), _rows(x), tokens, router.data_ptr(),
             _ptr(shared_gate_w), experts, top, width, z.data_ptr(), idx.data_ptr(), share.data_ptr(),
             _ptr(shared_gate) if shared_gate_w is not None else 0, int(all_scores), _ptr(correction), _stream())


def moe_scatter(idx: torch.Tensor, entries: int, experts: int, offsets: torch.Tensor, perm: torch.Tensor,
                tiles: torch.Tensor, tile_rows: int, real_experts: int | None = None) -> None:
    """Sorts the entries (token * top + choice) by expert: offsets [experts + 1], perm [entries] (sorted place -> entry),
    tiles [n, 2] the work list of experts_nt ((expert, first sorted place) per row tile, -1 beyond the last).
    real_experts: the experts from there on have no weights and get no tiles."""
    _need_gpu(idx, offsets, perm, tiles)
    assert idx.dtype == offsets.dtype == perm.dtype == tiles.dtype == torch.int32
    assert idx.numel() >= entries and perm.numel() >= entries and offsets.numel() >= experts + 1
    assert tiles.is_contiguous() and tiles.dim() == 2 and tiles.shape[1] == 2
    n = moe_max_tiles(entries, experts, tile_rows)
    assert tiles.shape[0] >= n
    lib.call("dinfer_moe_scatter", idx.data_ptr(), entries, experts, tile_rows, offsets.data_ptr(), perm.data_ptr(),
             tiles.data_ptr(), n, int(real_experts or experts), _stream())


def experts_nt(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, entries: int, tiles: torch.Tensor,
               offsets: torch.Tensor, perm: torch.Tensor, *, gated: bool, a_div: int, c_to_perm: bool,
               tile_rows: int, act: str | None = None) -> torch.Tensor:
    """The products of all experts in one launch. w [experts, rows, K]; gated: rows = 2 N, gate rows first, and
    out = silu(a Wg^T) * (a Wu^T). a_div > 0: the row of sorted place i is a[perm[i] // a_div] (the step's tokens),
    0: a[i]. c_to_perm: the result of sorted place i goes to out[perm[i]], else to out[i]. tile_rows: what moe_scatter
    made the work list with. act (not gated): "silu" or "gelu" (error function) on every result."""
    _need_gpu(a, w, out, tiles, offsets, perm)
    if act is not None and (gated or act not in EXPERT_ACTS):
        raise lib.KernelError(f"experts: activation {act!r} has no kernel here (known: {sorted(EXPERT_ACTS)}, not gated)")
    experts, rows, k = w.shape
    n = rows // 2 if gated else rows
    assert w.is_contiguous() and a.dtype == w.dtype == out.dtype and a.shape[1] == k and out.shape[1] == n
    assert out.shape[0] >= entries and (a_div > 0 or a.shape[0] >= entries)
    lib.call("dinfer_experts_nt", dtype_code(a.dtype), 1 if gated else EXPERT_ACTS[act] if act else 0, a.data_ptr(), _rows(a), w.data_ptr(), k,
             rows * k, out.data_ptr(), _rows(out), n, k, tiles.data_ptr(), moe_max_tiles(entries, experts, tile_rows),
             int(tile_rows), offsets.data_ptr(), perm.data_ptr(), int(a_div), 1 if c_to_perm else 0, _stream())
    return out


def moe_combine(y: torch.Tensor, share: torch.Tensor, top: int, shared: torch.Tensor | None,
                shared_gate: torch.Tensor | None, out: torch.Tensor, tokens: int, idx: torch.Tensor | None = None,
                real_experts: int = 0, x: torch.Tensor | None = None) -> torch.Tensor:
    """out[t] = sum_c share[t, c] * y[t * top + c] (+ shared_gate[t] * shared[t], or + shared[t] without a gate).
    idx, real_experts, x: a choice idx[t, c] >= real_experts stands for an expert whose output is its input: x[t] takes
    the place of y[t * top + c]."""
    _need_gpu(y, share, shared, shared_gate, out, idx, x)
    if idx is not None:
        assert idx.dtype == torch.int32 and idx.numel() >= tokens * top and x is not None
        assert x.dtype == out.dtype and x.shape[1] >= out.shape[1] and x.shape[0] >= tokens
    width = out.shape[1]
    assert y.shape[1] == width and y.dtype == out.dtype and y.shape[0] >= tokens * top and out.shape[0] >= tokens
    assert share.dtype == torch.float32 and share.numel() >= tokens * top
    if shared is not None:
        assert shared.dtype == out.dtype and shared.shape[1] == width and shared.shape[0] >= tokens
        assert shared_gate is None or (shared_gate.dtype == torch.float32 and shared_gate.numel() >= tokens)
    lib.call("dinfer_moe_combine", dtype_code(y.dtype), y.data_ptr(), _rows(y), share.data_ptr(), top, _ptr(shared),
             _rows(shared) if shared is not None else 0, _ptr(shared_gate), out.data_ptr(), _rows(out), tokens, width,
             _ptr(idx), int(real_experts), _ptr(x) if idx is not None else 0, _rows(x) if idx is not None else 0, _stream())
    return out


# ---- cache page layouts ------------------------------------------------------------------------
# K pages [blocks, kv_heads, D / 8, page, 8]: the 8-element pieces of consecutive keys are contiguous,
# so the rows of an MFMA operand (consecutive keys, one piece) are read as contiguous memory.
# V pages [blocks, kv_heads, D, page]: transposed, a row holds one dimension of a page's keys.
def k_cache_shape(blocks: int, kv_heads: int, page_size: int, head_dim: int) -> tuple:
    """A head size that is no multiple of 8 leaves its last piece filled in part (the plain kernels take that; the
    matrix-core kernels take whole pieces only)."""
    return (blocks, kv_heads, -(-head_dim // 8), page_size, 8)


def v_cache_shape(blocks: int, kv_heads: int, page_size: int, head_dim: int) -> tuple:
    return (blocks, kv_heads, head_dim, page_size)


def k_cache_pack(rows: torch.Tensor) -> torch.Tensor:
    """[blocks, kv_heads, page, D] (one row per key) -> the layout of K pages."""
    nb, hkv, page, d = rows.shape
    if d % 8:       # the last piece is filled in part
        rows = torch.cat([rows, rows.new_zeros(nb, hkv, page, 8 - d % 8)], dim=-1)
    return rows.view(nb, hkv, page, -1, 8).permute(0, 1, 3, 2, 4).contiguous()


def k_cache_rows(pages: torch.Tensor) -> torch.Tensor:
    """The layout of K pages -> [blocks, kv_heads, page, D] (one row per key)."""
    nb, hkv, pieces, page, _ = pages.shape
    return pages.permute(0, 1, 3, 2, 4).reshape(nb, hkv, page, pieces * 8)


def _check_pages(k_cache, v_cache, kv_heads, head_dim, page_size, v_dim=None) -> None:
    nb = k_cache.shape[0]
    assert tuple(k_cache.shape) == k_cache_shape(nb, kv_heads, page_size, head_dim) and k_cache.is_contiguous()
    if v_cache is not None:
        vd = head_dim if v_dim is None else v_dim
        assert tuple(v_cache.shape) == v_cache_shape(nb, kv_heads, page_size, vd) and v_cache.is_contiguous()


def qkv_post(qkv: torch.Tensor, tokens: int, *, heads: int, kv_heads: int, head_dim: int, q_off: int, k_off: int,
             v_off: int, q_gain: torch.Tensor | None, k_gain: torch.Tensor | None, eps: float, gain_offset: float,
             positions: torch.Tensor, cos_sin: torch.Tensor | None, rotary_dim: int, rope_style: int,
             k_cache: torch.Tensor | None, v_cache: torch.Tensor | None, slot_mapping: torch.Tensor | None,
             page_size: int, token_runs: bool = True, v_dim: int | None = None, bias: torch.Tensor | None = None,
             q_temp: tuple | None = None, q_head_scale: torch.Tensor | None = None) -> None:
    """Per-head q/k norm, rotation, q written back in place, k and v written to the cache pages.
    bias: float32 [q heads | k heads | v heads], added to the product's output first. q_temp (coef, every): q is
    multiplied by 1 + coef ln(floor((p + 1) / every) + 1) at position p, together with the norm. q_head_scale: float32
    [heads], q of head h is multiplied by its entry with the norm (a temperature on the head's scores).
    v_dim: the size of a value head where it is not head_dim. v_cache None beside a k_cache: the values are not stored
    (a layer whose values are its keys reads them from the key pages).

    k_cache and v_cache in the page layouts above; slot_mapping int64 [T] (None: nothing is written
    to the cache and k is written back in place, as q is). token_runs: the tokens come in runs of consecutive positions (prompt portions, not
    single decoded tokens); it only chooses the faster of two ways of writing V.
    """
    _need_gpu(qkv, q_gain, k_gain, positions, cos_sin, k_cache, v_cache, slot_mapping, q_head_scale)
    ld = _rows(qkv)
    assert qkv.shape[0] >= tokens
    vd = head_dim if v_dim is None else v_dim
    assert max(q_off + heads * head_dim, k_off + kv_heads * head_dim, v_off + kv_heads * vd) <= qkv.shape[1]
    assert positions.dtype == torch.int32 and positions.numel() >= tokens
    wf32 = 0
    if q_gain is not None:
        assert q_gain.numel() == head_dim and k_gain is not None and k_gain.numel() == head_dim
        wf32 = _is_param_f32(q_gain, qkv.dtype)
        assert _is_param_f32(k_gain, qkv.dtype) == wf32
    if cos_sin is not None:
        assert cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.shape[1] == rotary_dim
    if bias is not None:
        assert bias.dtype == torch.float32 and bias.is_contiguous()
        assert bias.numel() == (heads + kv_heads) * head_dim + kv_heads * vd
    if q_temp is not None:
        assert q_gain is not None and int(q_temp[1]) > 0
    if q_head_scale is not None:
        assert q_gain is not None and q_head_scale.dtype == torch.float32 and q_head_scale.numel() == heads
    if slot_mapping is not None:
        assert slot_mapping.dtype == torch.int64 and slot_mapping.numel() >= tokens
        assert k_cache is not None
        _check_pages(k_cache, v_cache, kv_heads, head_dim, page_size, vd)
        assert k_cache.dtype == qkv.dtype and (v_cache is None or v_cache.dtype == qkv.dtype)
    lib.call("dinfer_qkv_post", dtype_code(qkv.dtype), qkv.data_ptr(), tokens, ld, q_off, k_off, v_off,
             _ptr(q_gain), _ptr(k_gain), wf32, float(eps), float(gain_offset), positions.data_ptr(), _ptr(cos_sin),
             rotary_dim, rope_style, _ptr(k_cache), _ptr(v_cache), _ptr(slot_mapping), heads, kv_heads, head_dim,
             page_size, int(token_runs), vd, _ptr(bias), float(q_temp[0]) if q_temp else 0.0,
             int(q_temp[1]) if q_temp else 0, _ptr(q_head_scale), _stream())


def attn_paged_ext(q: torch.Tensor, out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor | None,
                   block_table: torch.Tensor, cu_seqlens: torch.Tensor, seq_lens: torch.Tensor, num_reqs: int,
                   tokens: int, *, scale: float, window: int, heads: int, kv_heads: int, head_dim: int, page_size: int,
                   v_dim: int | None = None, keep_first: int = 0, sinks: torch.Tensor | None = None,
                   slope_exp: float = 0.0, out_scale: float = 1.0) -> torch.Tensor:
    """The plain kernel with its options: keys j < keep_first stay visible behind the window; sinks (float32 [heads])
    join the softmax's denominator; slope_exp E takes 2^(-E (h + 1) / heads) * distance off the scores; values of size
    v_dim, or read from the key pages (v_cache None); the output times out_scale. Any storage type."""
    _need_gpu(q, out, k_cache, v_cache, block_table, cu_seqlens, seq_lens, sinks)
    vd = head_dim if v_dim is None else v_dim
    _check_pages(k_cache, v_cache, kv_heads, head_dim, page_size, vd)
    assert q.dtype == out.dtype == k_cache.dtype and q.shape[0] >= tokens and out.shape[0] >= tokens
    assert q.shape[1] >= heads * head_dim and out.shape[1] >= heads * vd
    assert block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.shape[0] >= num_reqs
    assert cu_seqlens.dtype == torch.int32 and seq_lens.dtype == torch.int32
    if sinks is not None:
        assert sinks.dtype == torch.float32 and sinks.numel() == heads and sinks.is_contiguous()
    lib.call("dinfer_attn_paged_ext", dtype_code(q.dtype), q.data_ptr(), _rows(q), out.data_ptr(), _rows(out),
             k_cache.data_ptr(), _ptr(v_cache), block_table.data_ptr(), block_table.shape[1], cu_seqlens.data_ptr(),
             seq_lens.data_ptr(), num_reqs, tokens, float(scale), int(window), int(keep_first), _ptr(sinks),
             float(slope_exp), heads, kv_heads, head_dim, vd, page_size, float(out_scale), _stream())
    return out


def attn_paged_ref(q: torch.Tensor, out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                   block_table: torch.Tensor, cu_seqlens: torch.Tensor, seq_lens: torch.Tensor, num_reqs: int,
                   tokens: int, *, scale: float, window: int, heads: int, kv_heads: int, head_dim: int,
                   page_size: int) -> torch.Tensor:
    """Plain paged attention (any head size); q is a view whose row t holds the heads at columns h*D."""
    _need_gpu(q, out, k_cache, v_cache, block_table, cu_seqlens, seq_lens)
    assert q.dtype == out.dtype == k_cache.dtype == v_cache.dtype
    assert block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous()
    assert block_table.shape[0] >= num_reqs
    assert cu_seqlens.dtype == torch.int32 and cu_seqlens.numel() >= num_reqs + 1
    assert seq_lens.dtype == torch.int32 and seq_lens.numel() >= num_reqs
    _check_pages(k_cache, v_cache, kv_heads, head_dim, page_size)
    assert q.shape[1] >= heads * head_dim and out.shape[1] >= heads * head_dim
    assert q.shape[0] >= tokens and out.shape[0] >= tokens
    lib.call("dinfer_attn_paged_ref", dtype_code(q.dtype), q.data_ptr(), _rows(q), out.data_ptr(), _rows(out),
             k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), block_table.shape[1],
             cu_seqlens.data_ptr(), seq_lens.data_ptr(), num_reqs, tokens, float(scale), int(window), heads,
             kv_heads, head_dim, page_size, _stream())
    return out


def attn_paged_diff(q: torch.Tensor, out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    block_table: torch.Tensor, cu_seqlens: torch.Tensor, seq_lens: torch.Tensor, num_reqs: int,
                    tokens: int, *, scale: float, window: int, heads: int, kv_heads: int, head_dim: int, v_dim: int,
                    page_size: int, lam: float, eps: float, post: float) -> torch.Tensor:
    """Differential attention, plain kernel: a query head holds two queries of head_dim entries side by side, a key
    head two keys (pages of heads of 2 head_dim); both softmax attentions run over the same values and
    out = unit_rms(a1 - lam a2, eps) * post, head h at column h v_dim."""
    _need_gpu(q, out, k_cache, v_cache, block_table, cu_seqlens, seq_lens)
    assert q.dtype == out.dtype == k_cache.dtype == v_cache.dtype
    assert block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous()
    assert block_table.shape[0] >= num_reqs
    assert cu_seqlens.dtype == torch.int32 and cu_seqlens.numel() >= num_reqs + 1
    assert seq_lens.dtype == torch.int32 and seq_lens.numel() >= num_reqs
    _check_pages(k_cache, v_cache, kv_heads, 2 * head_dim, page_size, v_dim)
    assert q.shape[1] >= heads * 2 * head_dim and out.shape[1] >= heads * v_dim
    assert q.shape[0] >= tokens and out.shape[0] >= tokens
    lib.call("dinfer_attn_paged_diff", dtype_code(q.dtype), q.data_ptr(), _rows(q), out.data_ptr(), _rows(out),
             k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), block_table.shape[1],
             cu_seqlens.data_ptr(), seq_lens.data_ptr(), num_reqs, tokens, float(scale), int(window), heads, kv_heads,
             head_dim, v_dim, page_size, float(lam), float(eps), float(post), _stream())
    return out


def diff_combine(pairs: torch.Tensor, out: torch.Tensor, tokens: int, *, heads: int, v_dim: int, lam: float, eps: float,
                 post: float) -> torch.Tensor:
    """The end of differential heads whose two maps were computed as heads of their own: pairs [T, 2 heads v_dim]
    (a head's first map, then its second) -> out[t, h] = unit_rms(a1 - lam a2, eps) * post."""
    _need_gpu(pairs, out)
    assert pairs.dtype == out.dtype and pairs.shape[1] >= 2 * heads * v_dim and out.shape[1] >= heads * v_dim
    assert pairs.shape[0] >= tokens and out.shape[0] >= tokens
    lib.call("dinfer_diff_combine", dtype_code(out.dtype), pairs.data_ptr(), _rows(pairs), out.data_ptr(), _rows(out), tokens,
             heads, v_dim, float(lam), float(eps), float(post), _stream())
    return out


def attn_mfma_supports(head_dim: int, page_size: int, heads: int, kv_heads: int) -> bool:
    return bool(lib.get("dinfer_attn_mfma_supports")(head_dim, page_size, heads, kv_heads))


def _check_paged(q, out, k_cache, v_cache, block_table, seq_lens, num_reqs, heads, kv_heads, head_dim, page_size):
    assert q.dtype == out.dtype == k_cache.dtype == v_cache.dtype == torch.bfloat16
    assert block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous()
    assert block_table.shape[0] >= num_reqs and seq_lens.dtype == torch.int32 and seq_lens.numel() >= num_reqs
    _check_pages(k_cache, v_cache, kv_heads, head_dim, page_size)
    assert q.shape[1] >= heads * head_dim and out.shape[1] >= heads * head_dim


def attn_flash(q, out, k_cache, v_cache, block_table, cu_seqlens, seq_lens, num_reqs: int, tokens: int,
               max_q_len: int, *, scale: float, window: int, heads: int, kv_heads: int, head_dim: int,
               page_size: int, skip_single: bool = False):
    """MFMA flash attention over the pages: rows with or without history, causal, optional window."""
    _need_gpu(q, out, k_cache, v_cache, block_table, cu_seqlens, seq_lens)
    _check_paged(q, out, k_cache, v_cache, block_table, seq_lens, num_reqs, heads, kv_heads, head_dim, page_size)
    assert cu_seqlens.dtype == torch.int32 and cu_seqlens.numel() >= num_reqs + 1
    assert q.shape[0] >= tokens and out.shape[0] >= tokens
    lib.call("dinfer_attn_flash", q.data_ptr(), _rows(q), out.data_ptr(), _rows(out), k_cache.data_ptr(),
             v_cache.data_ptr(), block_table.data_ptr(), block_table.shape[1], cu_seqlens.data_ptr(),
             seq_lens.data_ptr(), num_reqs, max_q_len, float(scale), int(window), heads, kv_heads, head_dim,
             page_size, 1 if skip_single else 0, _stream())
    return out


def attn_flash_ext(q, out, k_cache, v_cache, block_table, cu_seqlens, seq_lens, num_reqs: int, max_q_len: int, *,
                   scale: float, window: int, heads: int, kv_heads: int, head_dim: int, page_size: int,
                   keep_first: int = 0, sinks: torch.Tensor | None = None, slope_exp: float = 0.0,
                   out_scale: float = 1.0) -> torch.Tensor:
    """The matrix-core flash kernel with the options of attn_paged_ext (bfloat16, values of the keys' size, in value
    pages), for prompt portions and single rows alike."""
    _need_gpu(q, out, k_cache, v_cache, block_table, cu_seqlens, seq_lens, sinks)
    _check_paged(q, out, k_cache, v_cache, block_table, seq_lens, num_reqs, heads, kv_heads, head_dim, page_size)
    if sinks is not None:
        assert sinks.dtype == torch.float32 and sinks.numel() == heads and sinks.is_contiguous()
    lib.call("dinfer_attn_flash_ext", q.data_ptr(), _rows(q), out.data_ptr(), _rows(out), k_cache.data_ptr(),
             v_cache.data_ptr(), block_table.data_ptr(), block_table.shape[1], cu_seqlens.data_ptr(), seq_lens.data_ptr(),
             num_reqs, max_q_len, float(scale), int(window), int(keep_first), _ptr(sinks), float(slope_exp),
             float(out_scale), heads, kv_heads, head_dim, page_size, _stream())
    return out


def attn_decode(q, out, part, k_cache, v_cache, block_table, cu_seqlens, seq_lens, num_reqs: int, splits: int, *,
                scale: float, window: int, heads: int, kv_heads: int, head_dim: int, page_size: int):
    """Split-K attention for requests that bring one row. cu_seqlens None: row b is request b;
    given: only the requests with one row are served (mixed batches). Each request's keys are cut
    into `splits` equal parts on the device, so the launch shape does not depend on the lengths."""
    _need_gpu(q, out, part, k_cache, v_cache, block_table, cu_seqlens, seq_lens)
    _check_paged(q, out, k_cache, v_cache, block_table, seq_lens, num_reqs, heads, kv_heads, head_dim, page_size)
    assert part.dtype == torch.float32 and part.is_contiguous()
    lib.call("dinfer_attn_decode", q.data_ptr(), _rows(q), out.data_ptr(), _rows(out), part.data_ptr(),
             part.numel(), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), block_table.shape[1],
             _ptr(cu_seqlens), seq_lens.data_ptr(), num_reqs, splits, float(scale), int(window), heads, kv_heads,
             head_dim, page_size, _stream())
    return out


def attn_decode_post_supports(head_dim: int) -> bool:
    return bool(lib.get("dinfer_attn_decode_post_supports")(head_dim))


def attn_decode_post(qkv, out, part, k_cache, v_cache, block_table, seq_lens, num_reqs: int, splits: int, *,
                     scale: float, window: int, heads: int, kv_heads: int, head_dim: int, page_size: int, q_off: int,
                     k_off: int, v_off: int, q_gain, k_gain, eps: float, gain_offset: float, positions, cos_sin,
                     slot_mapping):
    """attn_decode for a step in which every request brings one row, straight from the q|k|v product: the per-head
    norms, the rotation (pairs (i, i + head_dim/2), the whole head) and the write of the new key and value into their
    pages happen inside the attention kernel. qkv stays as the product left it. slot_mapping None: nothing is written."""
    _need_gpu(qkv, out, part, k_cache, v_cache, block_table, seq_lens, q_gain, k_gain, positions, cos_sin, slot_mapping)
    _check_paged(qkv, out, k_cache, v_cache, block_table, seq_lens, num_reqs, heads, kv_heads, head_dim, page_size)
    assert part.dtype == torch.float32 and part.is_contiguous() and qkv.shape[0] >= num_reqs
    assert max(q_off + heads * head_dim, k_off + kv_heads * head_dim, v_off + kv_heads * head_dim) <= qkv.shape[1]
    assert q_off % 8 == 0 and k_off % 8 == 0 and v_off % 8 == 0
    assert positions.dtype == torch.int32 and positions.numel() >= num_reqs
    if q_gain is not None:   # (gains kept in 32-bit go through qkv_post)
        assert k_gain is not None and q_gain.numel() == k_gain.numel() == head_dim
        assert q_gain.dtype == k_gain.dtype == torch.bfloat16
    if cos_sin is not None:
        assert cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.shape[1] == head_dim
    if slot_mapping is not None:
        assert slot_mapping.dtype == torch.int64 and slot_mapping.numel() >= num_reqs
    base, es = qkv.data_ptr(), qkv.element_size()
    lib.call("dinfer_attn_decode_post", base + q_off * es, base + k_off * es, base + v_off * es, _rows(qkv),
             out.data_ptr(), _rows(out), part.data_ptr(), part.numel(), k_cache.data_ptr(), v_cache.data_ptr(),
             block_table.data_ptr(), block_table.shape[1], seq_lens.data_ptr(), num_reqs, splits, float(scale),
             int(window), heads, kv_heads, head_dim, page_size, _ptr(q_gain), _ptr(k_gain), float(eps),
             float(gain_offset), positions.data_ptr(), _ptr(cos_sin), _ptr(slot_mapping), _stream())
    return out


def gemm_ref(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int) -> torch.Tensor:
    """out[:m] = a[:m] @ w.T on the vector ALUs with float accumulation (true 32-bit for float operands)."""
    _need_gpu(a, w, out)
    n, k = w.shape
    assert a.shape[1] == k and out.shape[1] == n and a.dtype == w.dtype
    assert a.shape[0] >= m and out.shape[0] >= m
    out_f32 = 1 if out.dtype == torch.float32 else 0
    if not out_f32:
        assert out.dtype == a.dtype
    lib.call("dinfer_gemm_ref", dtype_code(a.dtype), out_f32, a.data_ptr(), _rows(a), w.data_ptr(), _rows(w),
             out.data_ptr(), _rows(out), m, n, k, _stream())
    return out


def gemm_small_m(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, *, row_tiles: int = 0,
                 waves: int = 0) -> torch.Tensor:
    """out[:m] = a[:m] @ w.T for m <= 64, bf16 operands, weight streamed once (MFMA, split-K in the workgroup)."""
    _need_gpu(a, w, out)
    n, k = w.shape
    assert a.dtype == w.dtype == torch.bfloat16 and a.shape[1] == k and out.shape[1] == n
    assert a.shape[0] >= m and out.shape[0] >= m and out.dtype in (torch.bfloat16, torch.float32)
    lib.call("dinfer_gemm_small_m", 1 if out.dtype == torch.float32 else 0, a.data_ptr(), _rows(a), w.data_ptr(),
             _rows(w), out.data_ptr(), _rows(out), m, n, k, row_tiles, waves, _stream())
    return out


def gemm_small_m_gated(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, *, waves: int = 0) -> torch.Tensor:
    """out[:m] = silu(a @ wg.T) * (a @ wu.T) for w = [wg; wu] stacked [2N, K], m <= 32, bf16: both
    projections of a gated feed-forward and the activation in one weight-streaming kernel."""
    _need_gpu(a, w, out)
    k = w.shape[1]
    n = w.shape[0] // 2
    assert w.shape[0] == 2 * n and a.dtype == w.dtype == out.dtype == torch.bfloat16
    assert a.shape[1] == k and out.shape[1] == n and a.shape[0] >= m and out.shape[0] >= m
    lib.call("dinfer_gemm_small_m_gated", a.data_ptr(), _rows(a), w.data_ptr(), _rows(w), out.data_ptr(), _rows(out),
             m, n, k, waves, _stream())
    return out


def gemm_small_m_sink(a: torch.Tensor, w: torch.Tensor, stream_: torch.Tensor, xg: torch.Tensor, gain: torch.Tensor,
                      stats: torch.Tensor, m: int, *, gain_offset: float = 0.0) -> int:
    """stream_[:m] += a[:m] @ w.T in place (the residual stream: summed in float, rounded once), and what the RMSNorm
    that reads it next needs: xg[:m] = stream_ * (gain + gain_offset), stats[r, j] = sum of squares of stream_[r] over
    columns g j .. g j + g - 1, g being 16 or 8 as the kernel for these sizes has it. Returns how many of them a token
    has (ceil(n / g)). m <= 32, bf16."""
    _need_gpu(a, w, stream_, xg, gain, stats)
    n, k = w.shape
    assert a.dtype == w.dtype == stream_.dtype == xg.dtype == torch.bfloat16 and stats.dtype == torch.float32
    assert a.shape[1] == k and stream_.shape[1] == n and xg.shape[1] == n and gain.numel() == n and gain.is_contiguous()
    cols = -(-n // lib.get("dinfer_gemm_small_m_sink_stats_columns")(m, n, k))
    assert min(a.shape[0], stream_.shape[0], xg.shape[0], stats.shape[0]) >= m and stats.shape[1] >= cols
    lib.call("dinfer_gemm_small_m_sink", a.data_ptr(), _rows(a), w.data_ptr(), _rows(w), stream_.data_ptr(), _rows(stream_),
             xg.data_ptr(), _rows(xg), gain.data_ptr(), _is_param_f32(gain, torch.bfloat16), float(gain_offset),
             stats.data_ptr(), _rows(stats), m, n, k, _stream())
    return cols


def gemm_small_m_scaled(xg: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, stats: torch.Tensor, cols: int,
                        eps: float, width: int, *, gated: bool = False) -> torch.Tensor:
    """out[:m] = (xg[:m] @ w.T) * rsqrt(sum(stats[r, :cols]) / width + eps) per row r: with xg and stats from
    gemm_small_m_sink, the product of the RMS-normed stream with w. gated: w = [wg; wu] stacked and
    out = silu(scaled gate) * scaled up. m <= 32, bf16."""
    _need_gpu(xg, w, out, stats)
    k = w.shape[1]
    n = w.shape[0] // 2 if gated else w.shape[0]
    assert xg.dtype == w.dtype == out.dtype == torch.bfloat16 and stats.dtype == torch.float32
    assert xg.shape[1] == k and out.shape[1] == n and min(xg.shape[0], out.shape[0], stats.shape[0]) >= m
    assert 0 < cols <= stats.shape[1]
    lib.call("dinfer_gemm_small_m_scaled", xg.data_ptr(), _rows(xg), w.data_ptr(), _rows(w), out.data_ptr(), _rows(out),
             m, n, k, 1 if gated else 0, stats.data_ptr(), _rows(stats), cols, float(eps), width, _stream())
    return out


def gemm_mid_m_workspace(m: int, n: int, k: int, *, gated: bool = False, ks: int = 0, rt: int = 0) -> int:
    """Bytes of float workspace gemm_mid_m needs for these sizes (0: the product is stored directly)."""
    need = ctypes.c_int64(0)
    lib.call("dinfer_gemm_mid_m_workspace", m, n, k, 1 if gated else 0, ks, rt, ctypes.addressof(need))
    return need.value


def gemm_mid_m(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, workspace: torch.Tensor | None = None, *,
               gated: bool = False, ks: int = 0, rt: int = 0) -> torch.Tensor:
    """out[:m] = a[:m] @ w.T for m <= 64 (made for 17 to 64), bf16 operands; gated: w = [wg; wu] stacked
    [2N, K] and out = silu(a @ wg.T) * (a @ wu.T). A narrow weight is cut into slices of k whose float
    partial sums go through `workspace` and are added in slice order by a second kernel."""
    _need_gpu(a, w, out, workspace)
    k = w.shape[1]
    n = w.shape[0] // 2 if gated else w.shape[0]
    assert a.dtype == w.dtype == torch.bfloat16 and a.shape[1] == k and out.shape[1] == n
    assert a.shape[0] >= m and out.shape[0] >= m and out.dtype in (torch.bfloat16, torch.float32)
    assert workspace is None or workspace.is_contiguous()
    lib.call("dinfer_gemm_mid_m", 1 if out.dtype == torch.float32 else 0, a.data_ptr(), _rows(a), w.data_ptr(), _rows(w),
             out.data_ptr(), _rows(out), m, n, k, 1 if gated else 0, ks, rt, _ptr(workspace),
             workspace.numel() * workspace.element_size() if workspace is not None else 0, _stream())
    return out


GEMM_MID_SINK_MAX_N = 8192   # columns a workgroup of gemm_mid_m_sink's second kernel holds in registers


def gemm_mid_m_sink(a: torch.Tensor, w: torch.Tensor, stream_: torch.Tensor, out: torch.Tensor, gain: torch.Tensor,
                    gain_offset: float, eps: float, m: int, workspace: torch.Tensor, *, ks: int = 0, rt: int = 0) -> None:
    """stream_[:m] += a[:m] @ w.T in place (the float sum of the slices and the stream, rounded once) and out[:m] = the
    RMSNorm of the new rows (gain + gain_offset, eps): gemm_mid_m's product with a second kernel that is also the add
    and the norm. bf16, m <= 64, N <= GEMM_MID_SINK_MAX_N."""
    _need_gpu(a, w, stream_, out, gain, workspace)
    n, k = w.shape
    assert a.dtype == w.dtype == stream_.dtype == out.dtype == torch.bfloat16 and a.shape[1] == k
    assert stream_.shape[1] == n and out.shape[1] == n and gain.numel() == n and gain.is_contiguous()
    assert a.shape[0] >= m and stream_.shape[0] >= m and out.shape[0] >= m and workspace.is_contiguous()
    assert gain.dtype in (torch.bfloat16, torch.float32)
    lib.call("dinfer_gemm_mid_m_sink", a.data_ptr(), _rows(a), w.data_ptr(), _rows(w), stream_.data_ptr(), _rows(stream_),
             out.data_ptr(), _rows(out), gain.data_ptr(), 1 if gain.dtype == torch.float32 else 0, float(gain_offset),
             float(eps), m, n, k, ks, rt, workspace.data_ptr(), workspace.numel() * workspace.element_size(), _stream())


def gemm_wide_supports(m: int, n: int, k: int) -> bool:
    """Whether gemm_wide takes a product of m rows with a weight of n rows (gated: n of each half) and k columns."""
    return bool(lib.get("dinfer_gemm_wide_supports")(m, n, k))


def gemm_wide(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, *, gated: bool = False,
              stats: torch.Tensor | None = None, cols: int = 0, eps: float = 0.0, width: int = 0) -> torch.Tensor:
    """out[:m] = a[:m] @ w.T for m <= 64 and a weight of many rows (96 of them a workgroup), bf16 operands, out bf16 or
    float32; gated: w = [wg; wu] stacked [2N, K] and out = silu(a @ wg.T) * (a @ wu.T). stats [m, >= cols] float32:
    row r of the result is multiplied by rsqrt(sum(stats[r, :cols]) / width + eps) first (a norm carried by the
    product before this one). K a multiple of 512, N of 16."""
    _need_gpu(a, w, out, stats)
    k = w.shape[1]
    n = w.shape[0] // 2 if gated else w.shape[0]
    assert a.dtype == w.dtype == torch.bfloat16 and a.shape[1] == k and out.shape[1] == n
    assert a.shape[0] >= m and out.shape[0] >= m and out.dtype in (torch.bfloat16, torch.float32)
    if stats is not None:
        assert stats.dtype == torch.float32 and stats.shape[0] >= m and stats.shape[1] >= cols > 0 and width > 0
    lib.call("dinfer_gemm_wide", 1 if out.dtype == torch.float32 else 0, a.data_ptr(), _rows(a), w.data_ptr(), _rows(w),
             out.data_ptr(), _rows(out), m, n, k, 1 if gated else 0, _ptr(stats), _rows(stats) if stats is not None else 0,
             int(cols), float(eps), int(width), _stream())
    return out


def argmax_scratch(rows: int, vocab: int, device) -> torch.Tensor:
    """The scratch with which argmax spreads each of up to `rows` rows over many workgroups."""
    n = ctypes.c_int64(0)
    lib.call("dinfer_argmax_scratch_bytes", rows, vocab, ctypes.addressof(n))
    return torch.empty(n.value, dtype=torch.uint8, device=device)


def argmax(logits: torch.Tensor, out: torch.Tensor, rows: int, scratch: torch.Tensor | None = None) -> torch.Tensor:
    """out[r] = the index of the largest of logits[r] (the lowest such index). scratch (argmax_scratch): a long row
    is spread over many workgroups instead of taken by one."""
    _need_gpu(logits, out, scratch)
    assert logits.dtype == torch.float32 and out.dtype == torch.int32 and out.numel() >= rows
    assert scratch is None or (scratch.dtype == torch.uint8 and scratch.is_contiguous())
    lib.call("dinfer_argmax", logits.data_ptr(), _rows(logits), out.data_ptr(), rows, logits.shape[1], _ptr(scratch),
             0 if scratch is None else scratch.numel(), _stream())
    return out


def sample(logits: torch.Tensor, work: torch.Tensor | None, out: torch.Tensor, rows: int, *,
           temperature: torch.Tensor | None, top_k: torch.Tensor | None = None, top_p: torch.Tensor | None = None,
           min_p: torch.Tensor | None = None, seeds: torch.Tensor | None = None,
           offsets: torch.Tensor | None = None) -> torch.Tensor:
    """One token per row. temperature None: all rows greedy. seeds/offsets are int64 holding the uint64 bits."""
    _need_gpu(logits, work, out, temperature, top_k, top_p, min_p, seeds, offsets)
    vocab = logits.shape[1]
    assert logits.dtype == torch.float32 and out.dtype == torch.int32 and out.numel() >= rows
    if temperature is not None:
        assert temperature.dtype == torch.float32 and temperature.numel() >= rows
        assert work is not None and work.dtype == torch.float32 and work.is_contiguous()
        assert work.numel() >= rows * vocab
        assert seeds is not None and offsets is not None
        assert seeds.dtype == torch.int64 and offsets.dtype == torch.int64
        assert seeds.numel() >= rows and offsets.numel() >= rows
    for t, dt in ((top_k, torch.int32), (top_p, torch.float32), (min_p, torch.float32)):
        assert t is None or (t.dtype == dt and t.numel() >= rows)
    lib.call("dinfer_sample", logits.data_ptr(), _rows(logits), _ptr(work), _ptr(temperature), _ptr(top_k),
             _ptr(top_p), _ptr(min_p), _ptr(seeds), _ptr(offsets), out.data_ptr(), rows, vocab, _stream())
    return out


# One row of dinfer_sample_rows: what to do with a row of logits.
SAMPLE_ROW = np.dtype([("temperature", "<f4"), ("top_k", "<i4"), ("top_p", "<f4"), ("min_p", "<f4"),
                       ("seed", "<u8"), ("offset", "<u8")])


def sample_scratch_bytes(rows: int, vocab: int) -> int:
    n = ctypes.c_int64(0)
    lib.call("dinfer_sample_scratch_bytes", rows, vocab, ctypes.addressof(n))
    return n.value


def sample_rows(logits: torch.Tensor, work: torch.Tensor, scratch: torch.Tensor, packed: torch.Tensor,
                out: torch.Tensor, rows: int, any_filter: bool = True, force_generic: bool = False) -> torch.Tensor:
    """One token per row by the rule of `sample`, a row spread over many workgroups. packed: uint8 device
    tensor holding `rows` records of SAMPLE_ROW; work [rows, vocab] float32 and scratch (uint8,
    sample_scratch_bytes) are the kernels' own memory between their launches. any_filter=False promises
    that no row has top-k or top-p."""
    _need_gpu(logits, work, scratch, packed, out)
    vocab = logits.shape[1]
    assert logits.dtype == torch.float32 and out.dtype == torch.int32 and out.numel() >= rows
    assert work.dtype == torch.float32 and work.is_contiguous() and work.numel() >= rows * vocab
    assert packed.dtype == torch.uint8 and packed.is_contiguous() and packed.numel() >= rows * SAMPLE_ROW.itemsize
    assert scratch.dtype == torch.uint8 and scratch.is_contiguous()
    lib.call("dinfer_sample_rows", logits.data_ptr(), _rows(logits), work.data_ptr(), scratch.data_ptr(),
             scratch.numel(), packed.data_ptr(), out.data_ptr(), rows, vocab, int(any_filter), int(force_generic), _stream())
    return out


# One row of penalties_dense: which history slot a row of logits takes its penalties from (< 0: none).
PENALTY_ROW = np.dtype([("slot", "<i4"), ("repetition", "<f4"), ("frequency", "<f4"), ("presence", "<f4")])


def history_add(history: torch.Tensor, entries: torch.Tensor) -> None:
    """history [slots, vocab] int32; entries [n, 3] int32 = (slot, token, kind): kind 0 marks a token of the
    prompt, kind 1 counts one more occurrence among the outputs."""
    _need_gpu(history, entries)
    assert history.dtype == torch.int32 and history.is_contiguous() and history.dim() == 2
    assert entries.dtype == torch.int32 and entries.is_contiguous() and entries.dim() == 2 and entries.shape[1] == 3
    lib.call("dinfer_history_add", history.data_ptr(), history.shape[0], history.shape[1], entries.data_ptr(),
             entries.shape[0], _stream())


def penalties_dense(logits: torch.Tensor, rows: int, history: torch.Tensor, packed: torch.Tensor) -> None:
    """In place on logits: row r takes repetition / frequency / presence penalties from history[slot_r]
    (packed: uint8 device tensor of `rows` PENALTY_ROW records; slot < 0 leaves the row alone)."""
    _need_gpu(logits, history, packed)
    assert logits.dtype == torch.float32 and history.dtype == torch.int32 and history.is_contiguous()
    assert history.shape[1] == logits.shape[1]
    assert packed.dtype == torch.uint8 and packed.is_contiguous() and packed.numel() >= rows * PENALTY_ROW.itemsize
    lib.call("dinfer_penalties_dense", logits.data_ptr(), _rows(logits), history.data_ptr(), history.shape[0],
             packed.data_ptr(), rows, logits.shape[1], _stream())


MAX_TOP_LOGPROBS = 32


def logit_bias(logits: torch.Tensor, rows: int, entries: torch.Tensor, values: torch.Tensor) -> None:
    """In place: logits[row, token] += value for entries [n, 2] int32 = (row, token) and values [n] float32.
    A (row, token) pair occurs once."""
    _need_gpu(logits, entries, values)
    assert logits.dtype == torch.float32 and entries.dtype == torch.int32 and values.dtype == torch.float32
    assert entries.is_contiguous() and entries.dim() == 2 and entries.shape[1] == 2
    assert values.is_contiguous() and values.numel() == entries.shape[0] and logits.shape[0] >= rows
    lib.call("dinfer_logit_bias", logits.data_ptr(), _rows(logits), entries.data_ptr(), values.data_ptr(),
             entries.shape[0], rows, logits.shape[1], _stream())


def logprobs(logits: torch.Tensor, chosen: torch.Tensor, top: torch.Tensor, out_ids: torch.Tensor,
             out_lp: torch.Tensor, rank: torch.Tensor, rows: int) -> None:
    """Per row r with top[r] >= 0, from the log-softmax of logits[r]: out_ids[r, 0], out_lp[r, 0] = chosen[r] and its
    log-probability; columns 1..top[r] the most probable tokens, falling (equal values: lower index first);
    rank[r] = how many tokens have a larger logit than the chosen one. out_ids / out_lp are [>= rows, stride] with
    stride <= MAX_TOP_LOGPROBS + 1; top[r] is cut to stride - 1."""
    _need_gpu(logits, chosen, top, out_ids, out_lp, rank)
    assert logits.dtype == torch.float32 and out_lp.dtype == torch.float32
    assert chosen.dtype == top.dtype == out_ids.dtype == rank.dtype == torch.int32
    assert out_ids.is_contiguous() and out_lp.is_contiguous() and out_ids.shape == out_lp.shape and out_ids.dim() == 2
    assert min(logits.shape[0], chosen.numel(), top.numel(), rank.numel(), out_ids.shape[0]) >= rows
    lib.call("dinfer_logprobs", logits.data_ptr(), _rows(logits), chosen.data_ptr(), top.data_ptr(),
             out_ids.shape[1], out_ids.data_ptr(), out_lp.data_ptr(), rank.data_ptr(), rows, logits.shape[1],
             _stream())


# ---- measured ceilings ---------------------------------------------------------------------------
def measured_hbm_read(device, nbytes: int = 4 << 30, repeats: int = 3) -> float:
    """Bytes per second a kernel that only reads reaches on `nbytes` of device memory (far beyond the caches):
    the best of `repeats` runs."""
    buf = torch.empty(nbytes // 4, dtype=torch.float32, device=device)
    buf.zero_()
    blocks = 256
    out = torch.empty(blocks * 8, dtype=torch.float32, device=device)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for _ in range(repeats + 1):      # the first run loads the kernel
        start.record()
        lib.call("dinfer_stream_read", buf.data_ptr(), buf.numel() * 4, blocks, out.data_ptr(), _stream())
        end.record()
        end.synchronize()
        best = min(best, start.elapsed_time(end) * 1e-3)
    del buf
    return nbytes / best


def measured_mfma_bf16(device, repeats: int = 3) -> float:
    """Flops per second of chains of independent bf16 MFMAs on registers, every SIMD busy: the best of `repeats` runs."""
    blocks, iters = 256 * 8, 2048
    out = torch.empty(blocks * 256, dtype=torch.float32, device=device)
    flops = ctypes.c_int64(0)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for _ in range(repeats + 1):
        start.record()
        lib.call("dinfer_mfma_loop", iters, blocks, out.data_ptr(), ctypes.addressof(flops), _stream())
        end.record()
        end.synchronize()
        best = min(best, start.elapsed_time(end) * 1e-3)
    return flops.value / best
