"""Dispatch of the sequence-mixer ops of hybrid decoders: GPU -> the HIP
kernels of mixers.hip (loud failure if the library is missing), CPU ->
torch_ref. All ops take a SeqBatch: T new tokens of B sequences laid end to
end, each continuing its sequence from its own past length, so a prompt
portion and a decoded token are one case.

Activations and weights are bfloat16 or float32 (`dt`); norms, scores,
softmax weights, decays, gates, recurrent state and the residual are float32
in both.
"""

from __future__ import annotations

import ctypes
import dataclasses
from typing import List, Optional, Tuple

import torch

from opsagent_amd.ops import torch_ref


@dataclasses.dataclass
class SeqBatch:
    """Geometry of one flat multi-sequence step. Host lists mirror the
    device tensors (launch geometry and the CPU path read the lists)."""

    cu: List[int]                 # [B+1] token offsets
    past: List[int]               # [B] tokens already in cache/state
    slots: List[int]              # [B] state-slot rows
    cu_t: torch.Tensor            # int32 [B+1]
    past_t: torch.Tensor          # int32 [B]
    slots_t: torch.Tensor         # int32 [B]
    seq_of_t: torch.Tensor        # int32 [T]
    slot_mapping: torch.Tensor    # int32 [T] flat kv-cache slot per token
    block_table: torch.Tensor     # int32 [B, max_blocks]
    # upper bounds used for launch geometry; a captured graph keeps them
    max_chunk: int = 0
    max_total: int = 0

    @property
    def num_seqs(self) -> int:
        return len(self.cu) - 1

    @property
    def num_tokens(self) -> int:
        return self.cu[-1]

    @staticmethod
    def build(chunks: List[Tuple[int, int, int, List[int]]], block_size: int,
              device, max_blocks: Optional[int] = None) -> "SeqBatch":
        """chunks: per sequence (past_len, count, state_slot, block ids)."""
        cu, past, slots, seq_of, slot_map, bt = [0], [], [], [], [], []
        nb = max((len(c[3]) for c in chunks), default=1)
        max_blocks = max(max_blocks or 0, nb, 1)
        for b, (p, n, slot, blocks) in enumerate(chunks):
            cu.append(cu[-1] + n)
            past.append(p)
            slots.append(slot if slot is not None else 0)
            seq_of.extend([b] * n)
            for pos in range(p, p + n):
                slot_map.append(blocks[pos // block_size] * block_size + pos % block_size)
            bt.extend(blocks)
            bt.extend([0] * (max_blocks - len(blocks)))
        # one host->device copy; the tensors are views of it
        B, T = len(chunks), cu[-1]
        flat = torch.tensor(cu + past + slots + seq_of + slot_map + bt,
                            dtype=torch.int32).to(device)
        o1, o2, o3, o4, o5 = B + 1, 2 * B + 1, 3 * B + 1, 3 * B + 1 + T, 3 * B + 1 + 2 * T
        return SeqBatch(
            cu=cu, past=past, slots=slots, cu_t=flat[:o1], past_t=flat[o1:o2],
            slots_t=flat[o2:o3], seq_of_t=flat[o3:o4], slot_mapping=flat[o4:o5],
            block_table=flat[o5:].view(B, max_blocks),
            max_chunk=max((c[1] for c in chunks), default=0),
            max_total=max((c[0] + c[1] for c in chunks), default=0),
        )


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return 0
    if t.dtype == torch.float32:
        return 1
    raise TypeError(f"unsupported activation type {t.dtype}")


def _lib():
    from opsagent_amd.ops import hip_lib

    return hip_lib.get_mixers_lib(), hip_lib


def _rows(t: torch.Tensor) -> int:
    """Row stride of a 2-D view whose rows are contiguous."""
    assert t.dim() == 2 and (t.shape[1] == 1 or t.stride(1) == 1), "rows must be contiguous"
    return t.stride(0)


def embed_rows(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """table[ids] as a float32 residual stream [T, C]."""
    if not table.is_cuda:
        return table[ids].float()
    lib, hip = _lib()
    T, C = ids.shape[0], table.shape[1]
    out = torch.empty(T, C, dtype=torch.float32, device=table.device)
    assert ids.dtype == torch.int64 and table.is_contiguous()
    hip.check(lib.oa_embed_rows(hip.current_stream_ptr(), table.data_ptr(), ids.data_ptr(),
                                out.data_ptr(), T, C, _dt(table)), "oa_embed_rows")
    return out


def causal_conv_seq(x: torch.Tensor, w: torch.Tensor, state: torch.Tensor, sb: SeqBatch,
                    add_input: bool, act_silu: bool) -> torch.Tensor:
    """(x +) causal per-channel convolution over time (-> silu), continued
    from and carried into state [slots, taps-1, C] float32. x [T, C] may be a
    column slice of a wider buffer; out has w's type."""
    T, C = x.shape
    taps = w.shape[1]
    assert w.shape[0] == C and state.shape[1:] == (taps - 1, C)
    if not x.is_cuda:
        return torch_ref.causal_conv_seq(x, w, state, sb.cu, sb.past, sb.slots,
                                         add_input, act_silu, w.dtype)
    lib, hip = _lib()
    out = torch.empty(T, C, dtype=w.dtype, device=x.device)
    assert w.is_contiguous() and state.is_contiguous() and state.dtype == torch.float32
    rc = lib.oa_causal_conv_seq(
        hip.current_stream_ptr(), x.data_ptr(), _rows(x), _dt(x), w.data_ptr(),
        state.data_ptr(), out.data_ptr(), C, sb.seq_of_t.data_ptr(), sb.cu_t.data_ptr(),
        sb.past_t.data_ptr(), sb.slots_t.data_ptr(), T, sb.num_seqs, C, taps,
        int(add_input), int(act_silu), _dt(w), sb.max_chunk)
    hip.check(rc, "oa_causal_conv_seq")
    return out


def group_rms_norm(y: torch.Tensor, w: torch.Tensor, groups: int, eps: float,
                   residual: Optional[torch.Tensor] = None,
                   want_copy: bool = True) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """RMS norm over `groups` consecutive parts, times w. With `residual`
    (float32 [T, C], updated in place): residual += norm. Returns (residual,
    copy) where copy is the result in w's type (None unless want_copy)."""
    T, C = y.shape
    if not y.is_cuda:
        if residual is not None:
            r = torch_ref.group_rms_norm(y, w, groups, eps, residual, w.dtype)
            return r, (r.to(w.dtype) if want_copy else None)
        return None, torch_ref.group_rms_norm(y, w, groups, eps, None, w.dtype)
    lib, hip = _lib()
    copy = torch.empty(T, C, dtype=w.dtype, device=y.device) if (want_copy or residual is None) else None
    if residual is not None:
        assert residual.dtype == torch.float32 and residual.is_contiguous()
    rc = lib.oa_group_rmsnorm(
        hip.current_stream_ptr(), y.data_ptr(), _rows(y), _dt(y), w.data_ptr(),
        residual.data_ptr() if residual is not None else None,
        copy.data_ptr() if copy is not None else None, T, C, groups, eps, _dt(w))
    hip.check(rc, "oa_group_rmsnorm")
    return residual, copy


def attn_qkv_prepare(qkv: torch.Tensor, bias: Optional[torch.Tensor], q_norm_w: torch.Tensor, k_norm_w: torch.Tensor,
                     H: int, G: int, D: int, Dv: int, eps: float, k_cache: torch.Tensor,
                     v_cache: torch.Tensor, sb: SeqBatch) -> torch.Tensor:
    """qkv [T, >= H*D + G*D + G*Dv] (q | k | v columns first; bias over these
    columns is added first, if given). Norms q and k over their whole
    projections, v per head; writes k, v to the paged cache; returns q
    [T, H, D]."""
    T = qkv.shape[0]
    if not qkv.is_cuda:
        return torch_ref.attn_qkv_prepare(qkv, bias, q_norm_w, k_norm_w, H, G, D, Dv, eps,
                                          k_cache, v_cache, sb.slot_mapping)
    lib, hip = _lib()
    assert k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype
    assert k_cache.shape[2:] == (G, D) and v_cache.shape[2:] == (G, Dv)
    q = torch.empty(T, H, D, dtype=qkv.dtype, device=qkv.device)
    rc = lib.oa_attn_prepare(
        hip.current_stream_ptr(), qkv.data_ptr(), _rows(qkv),
        bias.data_ptr() if bias is not None else None, q_norm_w.data_ptr(),
        k_norm_w.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
        sb.slot_mapping.data_ptr(), sb.cu_t.data_ptr(), sb.num_seqs, T, H, G, D, Dv, eps,
        _dt(qkv))
    hip.check(rc, "oa_attn_prepare")
    return q


_GEOM = {}


def attn_geometry(H: int, G: int, D: int, Dv: int, dt: int, max_chunk: int) -> Tuple[int, int]:
    """(query tokens per tile, keys per staged tile) of the attention kernel
    for steps whose longest portion is max_chunk tokens."""
    key = (H, G, D, Dv, dt, max_chunk >= 32)
    if key not in _GEOM:
        lib, hip = _lib()
        vals = [ctypes.c_int() for _ in range(4)]
        rc = lib.oa_attn_bias_geometry(H, G, D, Dv, dt, max_chunk,
                                       *[ctypes.byref(v) for v in vals])
        hip.check(rc, "oa_attn_bias_geometry")
        _GEOM[key] = (vals[0].value, vals[1].value)
    return _GEOM[key]


def attention_biased_paged(q: torch.Tensor, gate_logits: torch.Tensor, k_cache: torch.Tensor,
                           v_cache: torch.Tensor, sb: SeqBatch, scale: float,
                           slopes: torch.Tensor) -> torch.Tensor:
    """Causal softmax attention over each sequence's cached keys with score
    q.k*scale - slope_h*(i-j); head outputs times sigmoid(gate_logits[t, h]).
    q [T,H,D]; gate_logits [T,H] (may be a column slice). Returns [T, H*Dv]."""
    T, H, D = q.shape
    nb, bs, G, Dv = v_cache.shape
    if not q.is_cuda:
        return torch_ref.attention_biased_paged(q, gate_logits, k_cache, v_cache, sb.cu,
                                                sb.past, sb.block_table, scale, slopes)
    lib, hip = _lib()
    dt = _dt(q)
    TQ, KT = attn_geometry(H, G, D, Dv, dt, sb.max_chunk)
    ntiles = sum((sb.cu[b + 1] - sb.cu[b] + TQ - 1) // TQ for b in range(sb.num_seqs))
    # few tiles and long contexts: split the keys over blocks to fill the chip
    nkt = max(1, (sb.max_total + KT - 1) // KT)
    nsplit = 1
    if ntiles * G < 256 and nkt >= 8:
        nsplit = int(min(nkt // 4, max(1, 512 // max(1, ntiles * G)), 64))
    out = torch.empty(T, H * Dv, dtype=q.dtype, device=q.device)
    part_o = part_ml = None
    if nsplit > 1:
        part_o = torch.empty(T * H * nsplit, Dv, dtype=torch.float32, device=q.device)
        part_ml = torch.empty(T * H * nsplit, 2, dtype=torch.float32, device=q.device)
    assert slopes.dtype == torch.float32 and q.is_contiguous()
    rc = lib.oa_attn_bias_paged(
        hip.current_stream_ptr(), q.data_ptr(), gate_logits.data_ptr(), _rows(gate_logits),
        k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(),
        part_o.data_ptr() if part_o is not None else None,
        part_ml.data_ptr() if part_ml is not None else None,
        sb.cu_t.data_ptr(), sb.past_t.data_ptr(), sb.block_table.data_ptr(),
        sb.block_table.shape[1], bs, slopes.data_ptr(), T, sb.num_seqs, ntiles, H, G, D, Dv,
        float(scale), nsplit, dt, sb.max_chunk)
    hip.check(rc, "oa_attn_bias_paged")
    return out


def channel_delta_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                       b_logits: torch.Tensor, a: torch.Tensor, dt_bias: torch.Tensor,
                       a_log: torch.Tensor, norm_w: torch.Tensor, gate_logits: torch.Tensor,
                       state: torch.Tensor, sb: SeqBatch, H: int, G: int, D: int, Dv: int,
                       eps: float) -> torch.Tensor:
    """Gated delta rule with one decay per head and key channel, through to
    the gated read-out norm. q,k [T, G*D], v [T, H*Dv] (after convolution and
    silu), b_logits [T,H], a [T,H*D], gate_logits [T,H*Dv] — all may be
    column slices. state [slots,H,Dv,D] float32 (S transposed: a value
    column's key rows contiguous) is continued and updated.
    Returns rms_norm_per_head(S^T q) * norm_w * sigmoid(gate) as [T, H*Dv]
    in norm_w's type."""
    T = q.shape[0]
    if not q.is_cuda:
        o = torch_ref.channel_delta_rule(
            q.reshape(T, G, D), k.reshape(T, G, D), v.reshape(T, H, Dv), b_logits, a,
            dt_bias, a_log, state, sb.cu, sb.past, sb.slots)
        return torch_ref.gated_head_rms_norm(o, norm_w, gate_logits, eps, norm_w.dtype)
    lib, hip = _lib()
    out = torch.empty(T, H * Dv, dtype=norm_w.dtype, device=q.device)
    assert state.dtype == torch.float32 and state.is_contiguous()
    assert state.shape[1:] == (H, Dv, D)
    # one block per (sequence, head) runs the recurrence of ALL value columns
    # on one CU; long portions of few sequences split the columns over blocks
    # instead (the head norm then runs as its own launch on a float32 buffer)
    csplit, o_raw = 1, None
    pairs = sb.num_seqs * H
    if sb.max_chunk >= 64 and pairs < 192:
        for c in (8, 4, 2):
            if Dv % (4 * c) == 0 and Dv // c >= 16 and pairs * c <= 512:
                csplit = c
                break
    if D > 128 and Dv // csplit > 64:
        # 256-row columns: more than 64 columns per block would hold two or
        # four columns per lane pass and spill registers; split instead
        for c in (2, 4):
            if c >= csplit and Dv % (4 * c) == 0 and Dv // c <= 64:
                csplit = c
                break
    if csplit > 1:
        o_raw = torch.empty(T, H * Dv, dtype=torch.float32, device=q.device)
    rc = lib.oa_delta_rule_fused(
        hip.current_stream_ptr(), q.data_ptr(), _rows(q), k.data_ptr(), _rows(k),
        v.data_ptr(), _rows(v), b_logits.data_ptr(), _rows(b_logits), a.data_ptr(), _rows(a),
        dt_bias.data_ptr(), a_log.data_ptr(), norm_w.data_ptr(), gate_logits.data_ptr(),
        _rows(gate_logits), state.data_ptr(), out.data_ptr(),
        o_raw.data_ptr() if o_raw is not None else None, sb.cu_t.data_ptr(),
        sb.past_t.data_ptr(), sb.slots_t.data_ptr(), T, sb.num_seqs, H, G, D, Dv, eps, _dt(q),
        csplit)
    hip.check(rc, "oa_delta_rule_fused")
    return out


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(logits / cap) in float32."""
    if not logits.is_cuda:
        return torch_ref.softcap(logits, cap)
    lib, hip = _lib()
    x = logits.contiguous()
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    hip.check(lib.oa_softcap(hip.current_stream_ptr(), x.data_ptr(), out.data_ptr(),
                             x.numel(), float(cap), _dt(x)), "oa_softcap")
    return out


def silu_mul_rows(gu: torch.Tensor, inter: int) -> torch.Tensor:
    """silu(gu[:, :I]) * gu[:, I:] for a contiguous [M, 2I] buffer of any
    supported float type."""
    if not gu.is_cuda:
        g, u = gu.split([inter, inter], dim=-1)
        return torch_ref.silu_mul(g, u)
    lib, hip = _lib()
    assert gu.is_contiguous() and gu.shape[-1] == 2 * inter
    M = gu.numel() // (2 * inter)
    out = torch.empty(*gu.shape[:-1], inter, dtype=gu.dtype, device=gu.device)
    hip.check(lib.oa_silu_mul_rows(hip.current_stream_ptr(), gu.data_ptr(), out.data_ptr(),
                                   M, inter, _dt(gu)), "oa_silu_mul_rows")
    return out
