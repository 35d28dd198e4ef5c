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


def gated_delta(qkv, proj, b_off, a_off, a_log, dt_bias, state, meta, out, kv_heads, heads, D, V, decay=None):
    """The delta rule over every sequence of the step; qkv f32 [T, 2 kv_heads D + heads V] (queries,
    keys, values), proj f32 [T, ld] with column b_off + h (beta's pre-activation) and a_off + h (the
    decay's), state f32 [slots, heads, D, V] advanced in place, out f32 [T, heads V].
    decay f32 [T, heads D]: a factor a key channel, as `channel_decay` leaves it; a_off, a_log and
    dt_bias are then not read (they may be None)."""
    T, C = qkv.shape
    if decay is not None:
        _check(decay, "decay", torch.float32, (T, heads * D))
        a_off = 0
    else:
        _check(a_log, "A_log", torch.float32, (heads,))
        _check(dt_bias, "dt_bias", torch.float32, (heads,))
    _check(qkv, "qkv", torch.float32, (T, 2 * kv_heads * D + heads * V))
    _check(proj, "proj", torch.float32, (T, None))
    ld = proj.shape[1]
    if not (0 <= b_off and b_off + heads <= ld and 0 <= a_off and a_off + heads <= ld):
        raise BackendError("delta rule: the gate columns lie outside the projection's rows")
    _check(state, "state", torch.float32, (None, heads, D, V))
    _check(out, "out", torch.float32, (T, heads * V))
    _check(meta.seq_starts, "seq_starts", torch.int32, (meta.num_seqs + 1,))
    _check(meta.slots, "slots", torch.int32, (meta.num_seqs,))
    if heads % kv_heads or not 0 < D <= MAX_KEY_DIM:
        raise BackendError(f"delta rule: {heads} heads on {kv_heads} key heads of {D}")
    lib.call("recurrent", "hb_gated_delta", qkv.data_ptr(), C, proj.data_ptr(), ld, b_off, a_off,
             None if decay is not None else a_log.data_ptr(), None if decay is not None else dt_bias.data_ptr(),
             None if decay is None else decay.data_ptr(), state.data_ptr(), meta.seq_starts.data_ptr(),
             meta.slots.data_ptr(),
             out.data_ptr(), meta.num_seqs, kv_heads, heads, D, V, _stream())


def gated_head_norm(o, proj, g_off, weight, out, heads, V, eps, gate="silu"):
    """out[t, h, :] = o[t, h, :] / rms * weight * gate(proj[t, g_off + h V ...]), gate "silu" or
    "sigmoid"; out in any dtype."""
    if gate not in ("silu", "sigmoid"):
        raise BackendError(f"gated norm: unknown gate {gate!r}")
    T = o.shape[0]
    _check(o, "o", torch.float32, (T, heads * V))
    _check(proj, "proj", torch.float32, (T, None))
    if g_off < 0 or g_off + heads * V > proj.shape[1]:
        raise BackendError("gated norm: the gate columns lie outside the projection's rows")
    _check(weight, "weight", torch.float32, (V,))
    _check(out, "out", None, (T, heads * V))
    lib.call("recurrent", "hb_gated_head_norm", o.data_ptr(), proj.data_ptr(), proj.shape[1], g_off, weight.data_ptr(),
             out.data_ptr(), dtype_code(out), T, heads, V, float(eps), 1 if gate == "sigmoid" else 0, _stream())


def channel_decay(z, z_off, a_log, dt_bias, out, heads, D):
    """out[t, h, d] = exp(-exp(a_log[h]) * softplus(z[t, z_off + h D + d] + dt_bias[h, d])): the delta rule's
    decay a key channel from its pre-activation. z f32 [T, ld]; out f32 [T, heads D], which may be z
    itself (z_off 0, ld = heads D)."""
    T, ld = z.shape
    _check(z, "z", torch.float32, (T, ld))
    _check(out, "out", torch.float32, (T, heads * D))
    _check(a_log, "A_log", torch.float32, (heads,))
    _check(dt_bias, "dt_bias", torch.float32, (heads * D,))
    if z_off < 0 or z_off + heads * D > ld or (out.data_ptr() == z.data_ptr() and (z_off or ld != heads * D)):
        raise BackendError("channel decay: the pre-activations lie outside their rows")
    lib.call("recurrent", "hb_channel_decay", z.data_ptr() + 4 * z_off, ld, a_log.data_ptr(), dt_bias.data_ptr(),
             out.data_ptr(), T, heads, D, _stream())
