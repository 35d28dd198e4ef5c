"""Host side of the kernels for mixers with state of fixed size (csrc/recurrent.hip): the short
causal convolution with its activation and unit vectors, the gated delta rule, and the gated norm a
head that follows it. Operand checks, then the launch."""
import torch

from ..errors import BackendError
from . import lib
from .ops import _check, _stream, dtype_code

MAX_TAPS = 16
MAX_KEY_DIM = 256


def conv_silu(proj, taps, conv_state, meta, out, n_unit, unit_dim, n_scaled, scale, unit_eps, n_plain, plain_dim):
    """out[t, c] = silu(sum_j taps[c, j] * input[t - (K - 1) + j, c]) over the first C columns of proj
    (f32 [T, ld]); inputs from before the step come from conv_state (f32 [slots, K - 1, C]), which is
    then moved on. The first n_unit sections of unit_dim channels become unit vectors (the first
    n_scaled of them times `scale`), the n_plain sections of plain_dim that follow stay as they are."""
    T, ld = proj.shape
    C, K = taps.shape
    _check(proj, "proj", torch.float32, (T, ld))
    _check(taps, "taps", torch.float32, (C, K))
    _check(conv_state, "conv_state", torch.float32, (None, max(K - 1, 1), C))
    _check(out, "out", torch.float32, (T, C))
    _check(meta.seq_of, "seq_of", torch.int32, (T,))
    _check(meta.seq_starts, "seq_starts", torch.int32, (meta.num_seqs + 1,))
    _check(meta.slots, "slots", torch.int32, (meta.num_seqs,))
    if n_unit * unit_dim + n_plain * plain_dim != C or ld < C or not 1 <= K <= MAX_TAPS:
        raise BackendError(f"conv: sections {n_unit} x {unit_dim} + {n_plain} x {plain_dim} do not fit {C} channels "
                           f"of {K} taps")
    lib.call("recurrent", "hb_conv_silu", proj.data_ptr(), ld, taps.data_ptr(), conv_state.data_ptr(),
             meta.seq_of.data_ptr(), meta.seq_starts.data_ptr(), meta.slots.data_ptr(), out.data_ptr(), T,
             meta.num_seqs, C, K, n_unit, unit_dim, n_scaled, float(scale), float(unit_eps), n_plain, plain_dim,
             _stream())


def gated_delta(qkv, proj, b_off, a_off, a_log, dt_bias, state, meta, out, kv_heads, heads, D, V):
    """The delta rule over every sequence of the step; qkv f32 [T, 2 kv_heads D + heads V] (queries,
    keys, values), proj f32 [T, ld] with column b_off + h (beta's pre-activation) and a_off + h (the
    decay's), state f32 [slots, heads, D, V] advanced in place, out f32 [T, heads V]."""
    T, C = qkv.shape
    _check(qkv, "qkv", torch.float32, (T, 2 * kv_heads * D + heads * V))
    _check(proj, "proj", torch.float32, (T, None))
    ld = proj.shape[1]
    if not (0 <= b_off and b_off + heads <= ld and 0 <= a_off and a_off + heads <= ld):
        raise BackendError("delta rule: the gate columns lie outside the projection's rows")
    _check(a_log, "A_log", torch.float32, (heads,))
    _check(dt_bias, "dt_bias", torch.float32, (heads,))
    _check(state, "state", torch.float32, (None, heads, D, V))
    _check(out, "out", torch.float32, (T, heads * V))
    _check(meta.seq_starts, "seq_starts", torch.int32, (meta.num_seqs + 1,))
    _check(meta.slots, "slots", torch.int32, (meta.num_seqs,))
    if heads % kv_heads or not 0 < D <= MAX_KEY_DIM:
        raise BackendError(f"delta rule: {heads} heads on {kv_heads} key heads of {D}")
    lib.call("recurrent", "hb_gated_delta", qkv.data_ptr(), C, proj.data_ptr(), ld, b_off, a_off, a_log.data_ptr(),
             dt_bias.data_ptr(), state.data_ptr(), meta.seq_starts.data_ptr(), meta.slots.data_ptr(),
             out.data_ptr(), meta.num_seqs, kv_heads, heads, D, V, _stream())


def gated_head_norm(o, proj, g_off, weight, out, heads, V, eps):
    """out[t, h, :] = o[t, h, :] / rms * weight * silu(proj[t, g_off + h V ...]); out in any dtype."""
    T = o.shape[0]
    _check(o, "o", torch.float32, (T, heads * V))
    _check(proj, "proj", torch.float32, (T, None))
    if g_off < 0 or g_off + heads * V > proj.shape[1]:
        raise BackendError("gated norm: the gate columns lie outside the projection's rows")
    _check(weight, "weight", torch.float32, (V,))
    _check(out, "out", None, (T, heads * V))
    lib.call("recurrent", "hb_gated_head_norm", o.data_ptr(), proj.data_ptr(), proj.shape[1], g_off, weight.data_ptr(),
             out.data_ptr(), dtype_code(out), T, heads, V, float(eps), _stream())
