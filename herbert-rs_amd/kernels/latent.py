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


CHUNK = 32
TARGET_WAVES = 1024        # a decode step's keys are cut into ranges until about this many waves run


def mfma_takes(cache, rank, rot):
    """True if the matrix-core kernel takes this latent: bfloat16 rows, the latent and the rotated part in
    steps of 32, up to 512 + 128."""
    return (cache.k.dtype == torch.bfloat16 and rank % 32 == 0 and 0 < rank <= 512 and rot % 32 == 0 and rot <= 128
            and cache.page_size % CHUNK == 0)


def latent_attention_mfma(q_full, meta, cache, out, gate, gate_off, H, rank, rot, scale, buffer):
    """latent_attention_plain on the matrix cores (see mfma_takes). A step of one token a sequence cuts its
    keys into ranges, whose partial results lie in scratch from `buffer(name, shape, dtype)`."""
    T = q_full.shape[0]
    _check(q_full, "q_full", torch.float32, (T, H * (rank + rot)))
    _check(out, "out", torch.bfloat16, (T, H * rank))
    _check_pages(meta, cache, T, rank + rot)
    if not mfma_takes(cache, rank, rot):
        raise BackendError(f"latent attention: the matrix-core kernel does not take a latent of {rank} + {rot}")
    gate_ptr, gate_ld = None, 0
    if gate is not None:
        _check(gate, "gate", torch.float32, (T, None))
        gate_ld = gate.shape[1]
        if gate_off < 0 or gate_off + H > gate_ld:
            raise BackendError("latent attention: the gate's columns lie outside its rows")
        gate_ptr = gate.data_ptr() + 4 * gate_off
    splits, per = 1, 1 << 30
    if meta.max_new == 1:
        # the grid must not depend on the contexts themselves (a recorded step is replayed at others of its bucket)
        chunks = -(-max(meta.context_bucket, meta.max_context) // CHUNK)
        blocks = T * ((H + 15) // 16)
        splits = max(1, min(TARGET_WAVES // blocks, chunks, 64))
        per = -(-chunks // splits)
    part_acc = part_ml = None
    if splits > 1:
        part_acc = buffer("latent_partial", (T * H * splits, rank), torch.float32)
        part_ml = buffer("latent_partial_ml", (T * H * splits, 2), torch.float32)
    lib.call("attention_latent", "hb_latent_attention_mfma", q_full.data_ptr(), cache.k.data_ptr(), out.data_ptr(),
             _ptr(part_acc), _ptr(part_ml), gate_ptr, gate_ld, meta.positions.data_ptr(), meta.seq_of.data_ptr(),
             meta.slots.data_ptr(), cache.page_table.data_ptr(), cache.page_table.shape[1], cache.page_size, T, H,
             rank, rot, float(scale), splits, per, _stream())
