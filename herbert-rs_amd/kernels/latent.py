"""Host side of the attention over latent rows (csrc/attention_latent.hip): what a token writes
(its cache row [latent | rotated part] and its rotated query parts) and the attention itself."""
import torch

from ..errors import BackendError
from . import lib
from .ops import _check, _ptr, _stream, dtype_code

MAX_RANK = 1024
MAX_ROT = 128


def _check_pages(meta, cache, T, width):
    _check(meta.positions, "positions", torch.int32, (T,))
    _check(meta.seq_of, "seq_of", torch.int32, (T,))
    _check(meta.slots, "slots", torch.int32, (None,))
    _check(cache.page_table, "page_table", torch.int32, (None, None))
    _check(cache.k, "latent pages", None, (None, 1, cache.page_size, width))


def latent_write(proj, q_off, down_off, norm_w, q_full, inv_freq, meta, cache, H, qd, rank, rot, rot_dims, eps,
                 write_cache=True, q_plain=None):
    """proj f32 [T, ld]: columns [down_off, + rank + rot) -> the tokens' cache rows (the latent RMS-normed
    with norm_w, the rest rotated); columns [q_off, + H (qd + rot)) are the queries, whose rotated parts
    go into q_full f32 [T, H (rank + rot)] and, if q_plain (bf16 [T, H qd]) is given, whose unrotated
    parts are copied there."""
    T, ld = proj.shape
    _check(proj, "proj", torch.float32, (T, ld))
    if min(q_off, down_off) < 0 or q_off + H * (qd + rot) > ld or down_off + rank + rot > ld:
        raise BackendError("latent write: the columns lie outside the projection's rows")
    _check(norm_w, "norm_w", torch.float32, (rank,))
    _check(q_full, "q_full", torch.float32, (T, H * (rank + rot)))
    if rot_dims:
        _check(inv_freq, "inv_freq", torch.float32, (rot_dims // 2,))
    if rot_dims % 2 or not 0 <= rot_dims <= rot:
        raise BackendError(f"latent write: {rot_dims} rotated entries of {rot}")
    _check_pages(meta, cache, T, rank + rot)
    if q_plain is not None:
        _check(q_plain, "q_plain", torch.bfloat16, (T, H * qd))
    base = proj.data_ptr()
    lib.call("attention_latent", "hb_latent_write", base + 4 * down_off, ld, norm_w.data_ptr(), base + 4 * q_off, ld,
             q_full.data_ptr(), _ptr(q_plain), _ptr(inv_freq), meta.positions.data_ptr(), meta.seq_of.data_ptr(),
             meta.slots.data_ptr(), cache.page_table.data_ptr(), cache.page_table.shape[1], cache.page_size,
             cache.k.data_ptr(), dtype_code(cache.k), T, H, qd, rank, rot, rot_dims, float(eps),
             1 if write_cache else 0, _stream())


def latent_attention_plain(q_full, meta, cache, out, gate, gate_off, H, rank, rot, scale):
    """out[t, h, :rank] = softmax over the slot's rows j <= position of (q_full[t, h] . row_j * scale)
    times the rows' first `rank` entries, times sigmoid(gate[t, gate_off + h]) if gate (f32 [T, ld]) is given."""
    T = q_full.shape[0]
    _check(q_full, "q_full", torch.float32, (T, H * (rank + rot)))
    _check(out, "out", cache.k.dtype, (T, H * rank))
    _check_pages(meta, cache, T, rank + rot)
    if rank > MAX_RANK or rot > MAX_ROT:
        raise BackendError(f"latent attention: a latent of {rank} + {rot}, the kernel takes up to {MAX_RANK} + {MAX_ROT}")
    gate_ptr, gate_ld = None, 0
    if gate is not None:
        _check(gate, "gate", torch.float32, (T, None))
        gate_ld = gate.shape[1]
        if gate_off < 0 or gate_off + H > gate_ld:
            raise BackendError("latent attention: the gate's columns lie outside its rows")
        gate_ptr = gate.data_ptr() + 4 * gate_off
    lib.call("attention_latent", "hb_latent_attention_plain", q_full.data_ptr(), cache.k.data_ptr(), out.data_ptr(),
             dtype_code(cache.k), gate_ptr, gate_ld, meta.positions.data_ptr(), meta.seq_of.data_ptr(),
             meta.slots.data_ptr(), cache.page_table.data_ptr(), cache.page_table.shape[1], cache.page_size, T, H,
             rank, rot, float(scale), _stream())
