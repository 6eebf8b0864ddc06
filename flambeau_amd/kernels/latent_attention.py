"""The kernel set of attention over cached latent rows: folding the key expansion into the queries,
attention itself, and the value expansion with the heads' gates.

``PlainLatentAttention`` is the 32-bit path (and bfloat16 with the tuned kernels switched off, or at
sizes the matrix-core kernels do not take): everything between the query projection and the output
projection in float.  ``TunedLatentAttention`` runs each of the three on the matrix cores where its
sizes allow (``fl_*_takes``), each on its own: the folded queries are then bfloat16, the weighted sums
stay float."""
from __future__ import annotations

import torch

from . import ops
from .library import call, load
from .sets import register_kernel_set


class LatentWeights:
    """The expansions of one mixer as the kernels read them."""

    def __init__(self, uk, uv, n_heads):
        self.uk, self.uv, self.n_heads = uk, uv, n_heads           # [H * D, R] and [H * Dv, R], as loaded
        self.uk_by_head = None                                      # [H, R, D]: the key expansion transposed head by head


class PlainLatentAttention:
    def __init__(self, rt):
        self.rt = rt

    def prepare(self, uk, uv, n_heads) -> LatentWeights:
        return LatentWeights(uk, uv, n_heads)

    def attend(self, q, w: LatentWeights, cache, step, table, scale, window, gate, gate_col0, out):
        """``q`` float32 ``[n, H * D]`` -> ``out [n, H * Dv]`` (compute dtype): fold, attend, expand and gate."""
        rt, n, H, R = self.rt, q.shape[0], w.n_heads, cache.width
        qa = rt.buffer("la_qa", n, H * R, torch.float32)
        ops.heads_matmul(q, w.uk, qa, H, transposed=False)
        z = rt.buffer("la_z", n, H * R, torch.float32)
        ops.latent_attention(qa, z, cache, step.positions, step.tok_seq, table, H, scale, window)
        return ops.heads_matmul(z, w.uv, out, H, transposed=True, gate=gate, gate_col0=gate_col0)

    def signature(self, batch, n_heads: int):
        """What the kernels decide from the contexts' lengths (part of a recorded step's key)."""
        return ()

    def metadata(self, batch, mixers) -> dict:
        """Integer arrays the kernels want uploaded with the step (work lists); none here."""
        return {}


SPLIT_TARGET_WAVES = 1024     # four per compute unit
SPLIT_MIN_KEYS = 64           # a part of the keys is at least one chunk of 64


def key_splits(batch, n_heads: int) -> int:
    """Into how many parts the matrix-core kernel deals the keys of every token: a step of few rows
    behind long contexts (decoding) has too few (token, 16 heads) units to fill the chip."""
    units = batch.n_tokens * -(-n_heads // 16)
    most = max(1, batch.max_ctx_len // SPLIT_MIN_KEYS)
    parts = max(1, min(SPLIT_TARGET_WAVES // max(units, 1), most, 64))
    return 1 << (parts.bit_length() - 1)          # a power of two: few different launches while contexts grow


def shared_tiles(batch, groups: int):
    """The blocks of the kernel that shares its keys among four waves: ``[n, 4]`` = (first token, tokens, first
    group of 16 heads, groups) with tokens x groups <= 4 and all tokens of one request.  The list's length
    follows from the rows per request alone."""
    import numpy as np
    out = []
    if groups >= 4:
        for q0, ql in zip(batch.q_starts, batch.q_lens):
            for t in range(q0, q0 + ql):
                out += [(t, 1, g0, min(4, groups - g0)) for g0 in range(0, groups, 4)]
    else:
        per = 4 // groups
        for q0, ql in zip(batch.q_starts, batch.q_lens):
            out += [(t, min(per, q0 + ql - t), 0, groups) for t in range(q0, q0 + ql, per)]
    return np.asarray(out, dtype=np.int32).reshape(-1, 4)


class TunedLatentAttention(PlainLatentAttention):
    def signature(self, batch, n_heads):
        return key_splits(batch, n_heads)

    def metadata(self, batch, mixers):
        """One list of blocks per number of head groups among the model's mixers."""
        return {f"latent_tiles_{g}": shared_tiles(batch, g) for g in sorted({-(-m.n_heads // 16) for m in mixers})}

    def prepare(self, uk, uv, n_heads):
        w = LatentWeights(uk, uv, n_heads)
        D, R = uk.shape[0] // n_heads, uk.shape[1]
        if uk.dtype == torch.bfloat16 and load().fl_heads_matmul_mfma_takes(D, R):
            w.uk_by_head = uk.view(n_heads, D, R).transpose(1, 2).contiguous()
        return w

    def attend(self, q, w, cache, step, table, scale, window, gate, gate_col0, out):
        rt, n, H, R = self.rt, q.shape[0], w.n_heads, cache.width
        D, Dv = q.shape[1] // H, out.shape[1] // H
        lib = load()
        on_cores = cache.pool.dtype == torch.bfloat16 and bool(lib.fl_latent_attention_mfma_takes(R, cache.page_size))
        qa = rt.buffer("la_qa16" if on_cores else "la_qa", n, H * R, torch.bfloat16 if on_cores else torch.float32)
        if w.uk_by_head is not None:
            heads_matmul_mfma(q, w.uk_by_head, qa, H)
        else:
            ops.heads_matmul(q, w.uk, qa, H, transposed=False)
        z = rt.buffer("la_z", n, H * R, torch.float32)
        tiles = step.extra.get(f"latent_tiles_{-(-H // 16)}") if on_cores else None
        if on_cores and tiles is not None and key_splits(step.host, H) == 1:
            # a step of many rows (prompt portions): blocks of four waves share every chunk of keys through LDS
            latent_attention_shared(qa, z, cache, step.positions, step.tok_seq, table, H, scale, window, tiles)
        elif on_cores:
            n_split = key_splits(step.host, H)
            part_o = part_ml = None
            if n_split > 1:
                rows = n * -(-H // 16) * n_split * 16
                part_o = rt.buffer("la_part_o", rows, R, torch.float32, max_rows=16 * (SPLIT_TARGET_WAVES + 64))
                part_ml = rt.buffer("la_part_ml", rows, 2, torch.float32, max_rows=16 * (SPLIT_TARGET_WAVES + 64))
            latent_attention_mfma(qa, z, cache, step.positions, step.tok_seq, table, H, scale, window, n_split, part_o, part_ml,
                                  dealt=True)
        else:
            ops.latent_attention(qa, z, cache, step.positions, step.tok_seq, table, H, scale, window)
        if w.uv.dtype == torch.bfloat16 and lib.fl_heads_matmul_mfma_takes(R, Dv):
            return heads_matmul_mfma(z, w.uv.view(H, Dv, R), out, H, gate=gate, gate_col0=gate_col0)
        return ops.heads_matmul(z, w.uv, out, H, transposed=True, gate=gate, gate_col0=gate_col0)


def heads_matmul_mfma(x, w, out, n_heads, gate=None, gate_col0=0):
    """``out[t, h] = x[t, h] @ w[h].T`` on the matrix cores; ``w`` bfloat16 ``[H, J, K]``."""
    n, H = x.shape[0], int(n_heads)
    _, J, K = w.shape
    call("fl_heads_matmul_mfma", ops._check(x, "heads_matmul.x", None, (n, H * K)), ops.dtype_code(x.dtype), H * K,
         ops._check(w, "heads_matmul.w", torch.bfloat16, (H, J, K)), ops._check(out, "heads_matmul.out", None, (n, H * J)),
         ops.dtype_code(out.dtype), n, H, K, J,
         ops._check(gate, "heads_matmul.gate", torch.float32, (n, None)) if gate is not None else None,
         gate.shape[1] if gate is not None else 0, int(gate_col0), ops.stream_handle())
    return out


def latent_attention_mfma(qa, z, cache, positions, tok_seq, block_table, n_heads, scale, window=0, n_split=1,
                          part_o=None, part_ml=None, dealt=False):
    """``dealt``: the form with a block of four waves per (token, 16 heads, part of the keys), for steps of few rows
    (else one wave each).  ``n_split`` > 1: every token's keys are dealt out to that many waves; ``part_o`` (float32, at least
    ``n * ceil(H / 16) * n_split * 16`` rows of R) and ``part_ml`` (as many rows of 2) hold their sums."""
    n, R = qa.shape[0], cache.width
    if n_split > 1:
        rows = n * -(-n_heads // 16) * n_split * 16
        ops._check(part_o, "latent_attention.part_o", torch.float32, (None, R))
        ops._check(part_ml, "latent_attention.part_ml", torch.float32, (None, 2))
        if part_o.shape[0] < rows or part_ml.shape[0] < rows:
            raise ops.KernelError(f"latent_attention: {n_split} parts need {rows} rows of workspace")
    call("fl_latent_attention_dealt" if dealt else "fl_latent_attention_mfma", ops._check(qa, "latent_attention.qa", torch.bfloat16, (n, n_heads * R)),
         ops._check(z, "latent_attention.z", torch.float32, (n, n_heads * R)),
         ops._check(cache.pool, "latent_attention.pool", torch.bfloat16),
         ops._check(positions, "latent_attention.positions", torch.int32, (n,)),
         ops._check(tok_seq, "latent_attention.tok_seq", torch.int32, (n,)),
         ops._check(block_table, "latent_attention.block_table", torch.int32, (None, None)), block_table.shape[1],
         n, int(n_heads), R, cache.page_size, cache.n_pages, float(scale), int(window), int(n_split),
         part_o.data_ptr() if n_split > 1 else None, part_ml.data_ptr() if n_split > 1 else None, ops.stream_handle())
    return z


def latent_attention_shared(qa, z, cache, positions, tok_seq, block_table, n_heads, scale, window, tiles):
    """The matrix-core kernel whose blocks share their keys; ``tiles``: ``shared_tiles`` on the device."""
    n, R = qa.shape[0], cache.width
    call("fl_latent_attention_shared", ops._check(qa, "latent_attention.qa", torch.bfloat16, (n, n_heads * R)),
         ops._check(z, "latent_attention.z", torch.float32, (n, n_heads * R)),
         ops._check(cache.pool, "latent_attention.pool", torch.bfloat16),
         ops._check(positions, "latent_attention.positions", torch.int32, (n,)),
         ops._check(tok_seq, "latent_attention.tok_seq", torch.int32, (n,)),
         ops._check(block_table, "latent_attention.block_table", torch.int32, (None, None)), block_table.shape[1],
         int(n_heads), R, cache.page_size, cache.n_pages, float(scale), int(window),
         ops._check(tiles, "latent_attention.tiles", torch.int32, (None, 4)), tiles.shape[0], ops.stream_handle())
    return z


register_kernel_set("latent_attention", PlainLatentAttention, TunedLatentAttention)
