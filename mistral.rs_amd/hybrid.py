"""Layer-list ("hybrid") decoders served in their checkpoint dtype: every layer is `x += mixer(norm(x))` then optionally `x += feed_forward(norm(x))` (or both sublayers
reading two norms of the same x: `parallel_sublayers`), the mixer being one of the registered kinds (`MIXERS`: state-space-duality recurrence, paged softmax attention with a
sliding window / position chunks / kept first tokens / a learned sink, paged sigmoid attention with a distance bias and mixed head scores, sink attention with convolved
projections, retention, latent attention, the gated delta rule, a matrix memory with exponential gates, two mixers side by side), the feed-forward one of `FEED_FORWARDS`
(sigmoid-routed experts with a gated shared expert, softmax-routed clamped-GLU experts, routed squared-ReLU experts weighted over the chosen logits, dense xIELU and SiLU-GLU
layers).  The norms are RMS norms (plain or one-plus weights) before every sublayer, or layer norms with bias before AND after every sublayer (`HybridSpec.norm`,
`post_norms`).  The Gekilix, Sobunex, Setopel and Gifopel architectures (config.json `"architecture"`) are such lists.

The step function is `HybridDecoder.forward_batch(batch)`: ONE ragged batch -- prompt portions of any length next to single decoded tokens -- through the HIP kernels of
csrc/hyb_kernels.hip and csrc/hyb_gemm.hip (C ABI, this process's current stream; PyTorch owns buffers and the stream, nothing else).  What the sequences carry between
steps lives outside the step: K / V pages addressed through the block tables of `KVCacheManager`, convolution taps and recurrent states in the slots of `StateSlotPool`
(kv_cache_manager.py).  The scheduler's engine (scheduler.PagedEngine) and the trace runner (bin/trace_run) both drive this function.

Precision: the residual stream, norms, positions and angles, attention scores / softmax / weighted sums, router scores, decays, step sizes and recurrent states are f32 in
every mode.  `dtype="bfloat16"`: weights, GEMM operands and K / V pages in bf16, f32 accumulation; `dtype="float32"`: everything f32 (the bf16 checkpoint widened exactly).
There is no CPU path: the kernels raise if libmrs_hybrid.so is missing.
"""
from __future__ import annotations

import ctypes as C
import json
import math
import os
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence

import numpy as np
import torch

from . import _lib

_vp, _i, _l, _f = C.c_void_p, C.c_int32, C.c_int64, C.c_float
DTYPES = {"bfloat16": (1, torch.bfloat16), "float32": (2, torch.float32)}

_SIGS = {
    "mrs_hyb_embed": [_vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "mrs_hyb_rmsnorm": [_vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _f, _i, _i, _vp, _i, _i, _vp],
    "mrs_hyb_conv": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "mrs_hyb_conv_qkv_cache": [_vp, _i] + [_vp] * 12 + [_i] * 8 + [_f, _i, _i, _vp],
    "mrs_hyb_decay_scan": [_vp, _i] + [_vp] * 12 + [_i] * 7 + [_vp],
    "mrs_hyb_paged_attn_opts": [_vp] * 7 + [_i] * 9 + [_f, _i, _vp, _vp, _vp, _i, _i, _f, _i, _vp, _i, _vp, _i, _i, _vp],
    "mrs_hyb_rotary_half": [_vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _f, _i, _vp],
    "mrs_hyb_latent_norm_cache": [_vp, _i, _i, _i, _vp, _vp, _vp, _vp, _f, _i, _i, _vp],
    "mrs_hyb_hyper_step": [_vp] * 8 + [_i, _i, _i, _f, _i, _i, _vp],
    "mrs_hyb_gemm_batched": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _l, _l, _l, _i, _vp],
    "mrs_hyb_conv_silu": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "mrs_hyb_ssd_scan": [_vp] * 16 + [_i] * 10 + [_vp],
    "mrs_hyb_qk_norm_rope_cache": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _f, _i, _vp],
    "mrs_hyb_paged_window_attn": [_vp] * 7 + [_i] * 9 + [_f, _i, _vp, _vp, _vp, _i, _i, _vp],
    "mrs_hyb_route_sigmoid_topk": [_vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp],
    "mrs_hyb_moe_dispatch": [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp],
    "mrs_hyb_moe_gather": [_vp, _vp, _vp, _i, _vp, _i, _i, _i, _vp],
    "mrs_hyb_glu_silu": [_vp, _vp, _i, _i, _i, _vp],
    "mrs_hyb_moe_combine": [_vp, _vp, _vp, _i, _vp, _vp, _i, _i, _vp],
    "mrs_hyb_gather_rows": [_vp, _vp, _vp, _i, _i, _vp],
    "mrs_hyb_route_softmax_topk": [_vp, _vp, _i, _i, _i, _i, _f, _vp, _vp, _vp],
    "mrs_hyb_moe_combine_weighted": [_vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _vp],
    "mrs_hyb_glu_clamped": [_vp, _vp, _i, _i, _f, _f, _i, _vp],
    "mrs_hyb_bias_xielu": [_vp, _i, _vp, _vp, _i, _i, _f, _f, _i, _vp],
    "mrs_hyb_layernorm": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _f, _i, _vp],
    "mrs_hyb_layernorm_pair": [_vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _f, _i, _vp],
    "mrs_hyb_qkv_bias_temp_cache": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i, _i, _vp],
    "mrs_hyb_paged_talk_sigmoid_attn": [_vp] * 9 + [_i, _vp] + [_i] * 8 + [_f, _i, _vp, _vp, _vp, _i, _i, _vp, _i, _vp],
    "mrs_hyb_gated_scan": [_vp, _i] + [_vp] * 11 + [_i] * 8 + [_f, _vp],
    "mrs_hyb_qk_headnorm_rope_cache": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _f, _i, _vp],
    "mrs_hyb_paged_attn_chunked": [_vp] * 7 + [_i] * 8 + [_f, _i, _vp, _vp, _vp, _i, _i, _f, _i, _vp, _vp, _i, _i, _vp, _i, _vp],
    "mrs_hyb_route_topk_softmax": [_vp, _vp, _vp, _i, _i, _i, _i, _f, _vp, _vp, _vp],
    "mrs_hyb_rmsnorm_pair": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _f, _i, _i, _vp],
    "mrs_hyb_delta_prep": [_vp, _i, _vp, _i, _i, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "mrs_hyb_delta_step_prep": [_vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _i] + [_vp] * 7 + [_i] * 6 + [_vp],
    "mrs_hyb_delta_scan": [_vp, _i] + [_vp] * 12 + [_i] * 9 + [_vp],
    "mrs_hyb_exp_gates": [_vp, _i, _i, _i, _vp, _vp, _f] + [_vp] * 8 + [_i, _i, _i, _vp],
    "mrs_hyb_head_norm_gate": [_vp, _i, _vp, _vp, _i, _vp, _i, _i, _vp, _i, _i, _i, _f, _i, _vp],
    "mrs_hyb_norm_pair_add": [_vp, _i, _vp, _vp, _vp, _vp, _i, _i, _f, _f, _i, _vp],
    "mrs_hyb_round_cols": [_vp, _i, _vp, _i, _i, _i, _vp],
    "mrs_hyb_relu_sq": [_vp, _vp, _i, _i, _i, _vp],
    "mrs_hyb_gemm": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _i, _l, _i, _vp],
    "mrs_hyb_gemv": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _l, _i, _vp, _vp, _i, _vp],
    "mrs_hyb_gemv_act": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _l, _i, _vp, _vp, _i, _vp, _f, _f, _vp],
}
_RECUR = {"mrs_hyb_rmsnorm_pair", "mrs_hyb_delta_prep", "mrs_hyb_delta_step_prep", "mrs_hyb_delta_scan", "mrs_hyb_exp_gates", "mrs_hyb_head_norm_gate", "mrs_hyb_norm_pair_add", "mrs_hyb_round_cols",
          "mrs_hyb_relu_sq"}   # launchers of csrc/hyb_recur.hip (their own error text)
_fns: dict = {}
_step_stream: Optional[int] = None   # the stream handle of the step in progress (looked up once per forward_batch, not once per launch)


def _call(name: str, *args) -> None:
    """One kernel launcher of libmrs_hybrid.so on the current stream (appended as the last argument).  Tensors pass as device pointers."""
    fn = _fns.get(name)
    if fn is None:
        fn = _fns[name] = _lib.sym("hybrid", name, _SIGS[name], C.c_int)
    conv = [a.data_ptr() if isinstance(a, torch.Tensor) else a for a in args]
    if fn(*conv, _step_stream if _step_stream is not None else torch.cuda.current_stream().cuda_stream) != 0:
        err = _lib.sym("hybrid", "mrs_hyb_recur_last_error" if name in _RECUR else "mrs_hyb_gemm_last_error" if "gem" in name else ("mrs_hyb_talk_last_error" if "talk" in name else "mrs_hyb_last_error"), [], C.c_char_p)()
        raise ValueError((err or b"").decode() or name)


# ------------------------------------------------------------------------------------------------------------------ what a step sees
@dataclass
class RaggedBatch:
    """A step's tokens as one flat row range: entry s owns rows [seq_start[s], seq_start[s + 1]) at positions seq_pos0[s] + i."""
    rows: int
    entries: int
    max_blocks: int
    tokens: torch.Tensor        # i32 [rows]
    tok_seq: torch.Tensor       # i32 [rows]  entry of the row
    tok_pos: torch.Tensor       # i32 [rows]  position in its sequence
    seq_start: torch.Tensor     # i32 [entries + 1]
    seq_pos0: torch.Tensor      # i32 [entries]  position of the entry's first row (0: the sequence starts here, its state slot counts as zero)
    seq_slot: torch.Tensor      # i32 [entries]  state slot
    block_tables: torch.Tensor  # i32 [entries, max_blocks]
    slot_mapping: torch.Tensor  # i64 [rows]  K / V page slot = block * block_size + offset
    want: torch.Tensor          # i32 [n]  rows whose logits are wanted
    # every entry's rows cut into segments of at most SEGMENT rows (linear recurrences run the segments of a long portion in parallel)
    segments: int = 0
    seg_entry: Optional[torch.Tensor] = None   # i32 [segments]
    seg_row0: Optional[torch.Tensor] = None    # i32 [segments]  first row
    seg_len: Optional[torch.Tensor] = None     # i32 [segments]
    ent_seg0: Optional[torch.Tensor] = None    # i32 [entries + 1]  first segment of every entry, then the total
    seg_rows: int = 0                          # rows of the longest segment (1: every entry brings one decoded token)
    host_blocks: Optional[List[Sequence[int]]] = None   # every entry's block ids covering its last position (host copy; `build` keeps it)
    host_lens: Optional[List[int]] = None               # rows of every entry (host copy; `build` keeps it)
    _context: Optional[tuple] = None
    _entries: Optional[tuple] = None
    _long: Optional[dict] = None

    def segment_table(self, rows: int):
        """The batch's entries cut into segments of at most `rows` rows (another cut than SEGMENT, for a scan whose pass between the segments is dear):
        (seg_entry, seg_row0, seg_len, ent_seg0, segments)."""
        if rows == RaggedBatch.SEGMENT or self.host_lens is None:
            return self.seg_entry, self.seg_row0, self.seg_len, self.ent_seg0, self.segments
        if self._long is None:
            self._long = {}
        if rows not in self._long:
            nseg = sum(max(1, -(-n // rows)) for n in self.host_lens)
            t = np.zeros(3 * nseg + self.entries + 1, dtype=np.int32)
            sge, sgr, sgl, es0 = t[:nseg], t[nseg:2 * nseg], t[2 * nseg:3 * nseg], t[3 * nseg:]
            z = r = 0
            for s, n in enumerate(self.host_lens):
                es0[s] = z
                for a0 in range(0, max(n, 1), rows):
                    sge[z], sgr[z], sgl[z] = s, r + a0, min(rows, n - a0)
                    z += 1
                r += n
            es0[self.entries] = z
            d = torch.from_numpy(t).to(self.tokens.device)
            self._long[rows] = (d[:nseg], d[nseg:2 * nseg], d[2 * nseg:3 * nseg], d[3 * nseg:], nseg)
        return self._long[rows]

    def entry_table(self):
        """A segment table with ONE segment per entry, however long: (seg_entry, seg_row0, seg_len, ent_seg0) for a scan that runs every entry as one chain."""
        if self.segments == self.entries:
            return self.seg_entry, self.seg_row0, self.seg_len, self.ent_seg0
        if self._entries is None:
            iota = torch.arange(self.entries + 1, dtype=torch.int32, device=self.tokens.device)
            self._entries = (iota[:-1], self.seq_start[:-1], (self.seq_start[1:] - self.seq_start[:-1]).contiguous(), iota)
        return self._entries

    def context_blocks(self):
        """The blocks that hold the batch's whole contexts, renumbered densely: (tables i32 [entries, max_blocks] of dense ids, source i32 [n] = the pool block behind
        dense block d, n).  A mixer that expands its cached rows for a prompt step (keys and values from latent rows) gathers the source blocks into a scratch and reads the
        scratch through these tables."""
        if self._context is None:
            if self.host_blocks is None:
                raise ValueError("RaggedBatch: this batch was not built from entries")
            tables = np.zeros((self.entries, self.max_blocks), dtype=np.int32)
            src: List[int] = []
            for s, blocks in enumerate(self.host_blocks):
                tables[s, :len(blocks)] = np.arange(len(src), len(src) + len(blocks), dtype=np.int32)
                src.extend(int(x) for x in blocks)
            dev = self.tokens.device
            self._context = (torch.from_numpy(tables).to(dev), torch.tensor(src, dtype=torch.int32, device=dev), len(src))
        return self._context

    SEGMENT = int(os.environ.get("MRS_HYB_SEGMENT", "64"))   # rows per segment

    @staticmethod
    def build(entries: Sequence[dict], block_size: int, device) -> "RaggedBatch":
        """entries: dicts with `tokens`, `pos0`, `slot` (state slot or 0), `blocks` (the sequence's block ids, covering pos0 + len(tokens)), `want` (local indices)."""
        S = len(entries)
        lens = [len(e["tokens"]) for e in entries]
        T = sum(lens)
        mb = max(1, max((len(e["blocks"]) for e in entries), default=1))
        L = RaggedBatch.SEGMENT
        nseg = sum(max(1, -(-n // L)) for n in lens)
        sizes = (T, T, T, S + 1, S, S, S * mb, nseg, nseg, nseg, S + 1)
        ints = np.zeros(sum(sizes), dtype=np.int32)
        o = 0
        views = []
        for n in sizes:
            views.append(ints[o:o + n])
            o += n
        tok, tseq, tpos, sst, sp0, ssl, bt, sge, sgr, sgl, es0 = views
        z = 0
        host_blocks = []
        bt = bt.reshape(S, mb)
        slots = np.zeros(T, dtype=np.int64)
        want: List[int] = []
        r = 0
        for s, e in enumerate(entries):
            n, p0 = lens[s], int(e["pos0"])
            blocks = np.asarray(e["blocks"], dtype=np.int64)
            if n and (p0 + n - 1) // block_size >= len(blocks):
                raise ValueError("RaggedBatch: the entry's blocks do not cover its last position")
            host_blocks.append(blocks[:(p0 + n - 1) // block_size + 1] if n else blocks[:0])
            tok[r:r + n] = e["tokens"]
            tseq[r:r + n] = s
            pos = np.arange(p0, p0 + n, dtype=np.int64)
            tpos[r:r + n] = pos
            sst[s] = r
            sp0[s] = p0
            ssl[s] = int(e.get("slot") or 0)
            bt[s, :len(blocks)] = blocks
            if n:
                slots[r:r + n] = blocks[pos // block_size] * block_size + pos % block_size
            want.extend(r + int(j) for j in e.get("want", ()))
            es0[s] = z
            for a0 in range(0, max(n, 1), L):
                sge[z], sgr[z], sgl[z] = s, r + a0, min(L, n - a0)
                z += 1
            r += n
        sst[S] = T
        es0[S] = z
        dev_ints = torch.from_numpy(ints).to(device)
        o = 0
        dv = []
        for n in sizes:
            dv.append(dev_ints[o:o + n])
            o += n
        return RaggedBatch(T, S, mb, dv[0], dv[1], dv[2], dv[3], dv[4], dv[5], dv[6].view(S, mb), torch.from_numpy(slots).to(device),
                           torch.tensor(want, dtype=torch.int32, device=device), nseg, dv[7], dv[8], dv[9], dv[10], max(1, min(L, max(lens, default=1))), host_blocks, lens)


# ------------------------------------------------------------------------------------------------------------------ layer descriptions
@dataclass
class RotarySpec:
    """Rotary on the first `dims` dimensions of a head: a pair turns by position * f_i, f_i = base^(-2i / dims), optionally rescaled by wavelength (`scaling`: factor, low,
    high, original -- wavelengths under original / high keep f, over original / low use f / factor, linear blend between).  `layout`: "interleaved" pairs (2i, 2i + 1) or
    "half" pairs (i, i + dims / 2)."""
    dims: int
    base: float
    scaling: Optional[dict] = None
    layout: str = "interleaved"

    def frequencies(self) -> np.ndarray:
        i = np.arange(self.dims // 2, dtype=np.float64)
        f = np.float64(self.base) ** (-2.0 * i / self.dims)
        if self.scaling:
            fac, lo, hi, orig = (float(self.scaling[k]) for k in ("factor", "low", "high", "original"))
            wl = 2.0 * math.pi / f
            s = (orig / wl - lo) / (hi - lo)
            mid = (1.0 - s) * f / fac + s * f
            f = np.where(wl < orig / hi, f, np.where(wl > orig / lo, f / fac, mid))
        return f.astype(np.float32)


@dataclass
class AttentionSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0            # 0: every earlier token
    keep_first: int = 0        # tokens at the start of the sequence that stay visible behind the window
    rotary: Optional[RotarySpec] = None
    qk_norm: bool = True       # plain-weight RMS norm over the whole query / key projection, before rotation
    chunk: int = 0             # > 0: position i sees j <= i only when floor(i / chunk) == floor(j / chunk) (chunks counted from position 0; excludes `window`)
    head_norm: bool = False    # the query / key norm runs per head with weights [dim] shared by the heads
    sink: bool = False         # the softmax's denominator has one more term e^{sink_h}, a learned number per head (tensor `sink`)
    head_gate: bool = False    # head h's output is multiplied by sigmoid(Wg h)_h, one logit per head (tensor `g` [heads, width])


@dataclass
class DeltaRuleSpec:
    """Gated delta rule (DeltaRuleMixer): S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  `decay`: "head" = one decay per head from the projection `a`,
    "channel" = one per head and key channel from the two-step projection `a1`, `a2`.  `gate`: "silu" = SiLU of the full projection `g`, "sigmoid_lowrank" = sigmoid of the
    two-step projection `g1`, `g2` (the inner sizes of both two-step projections come from the tensors)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay: str = "head"
    gate: str = "silu"


@dataclass
class MlstmSpec:
    """Matrix memory with exponential input / forget gates and a running stabiliser (MlstmMixer)."""
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass
class ParallelSpec:
    """Two mixers side by side on the same input; the result is half the sum of their outputs, each normed over the model width (ParallelMixer)."""
    left_kind: str
    left: object
    right_kind: str
    right: object


@dataclass
class TalkAttentionSpec:
    """Sigmoid attention with a distance bias, mixed head scores, a query temperature and a per-head output gate (TalkSigmoidAttention)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0            # 0: every earlier token
    temp_coef: float = 0.0     # query factor 1 + temp_coef ln(floor((pos + 1) / temp_every) + 1); temp_every 0: none
    temp_every: int = 0
    kv_from: Optional[int] = None   # index of the layer whose K / V pages this layer reads (it has no key / value projections then)


@dataclass
class SinkAttentionSpec:
    """Causal softmax attention with a zero-score sink, capped scores, convolved projections, a query temperature and an elementwise output gate (GatedSinkAttention)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: int = 0              # taps of the causal convolution over q / k / v (0: none)
    softcap: float = 0.0       # 0: scores are not capped
    temp_coef: float = 0.0     # query factor 1 + temp_coef ln(floor((pos + 1) / temp_every) + 1); temp_every 0: none
    temp_every: int = 0
    kv_from: Optional[int] = None   # index of the layer whose K / V pages this layer reads (it has no key / value projections then)
    sink: bool = True


@dataclass
class RetentionSpec:
    """Decayed linear attention: per head S <- decay S + k v^T, o = S^T q (RetentionMixer)."""
    heads: int
    dim: int
    vdim: int
    decay: List[float]
    rotary: Optional[RotarySpec] = None


@dataclass
class LatentAttentionSpec:
    """Softmax attention whose keys and values are expanded from one cached low-rank row per token (LatentAttention)."""
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    scale: float


@dataclass
class Mamba2Spec:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


@dataclass
class MoeSpec:
    experts: int
    top: int
    ff: int
    shared_ff: int = 0         # 0: no shared expert
    kind = "moe"               # key into FEED_FORWARDS


@dataclass
class ClampedMoeSpec:
    """Softmax-routed experts with a clamped GLU (ClampedSoftmaxMoe)."""
    experts: int
    top: int
    ff: int
    limit: float
    route_scale: float = 1.0
    shared_ff: int = 0         # 0: no shared expert
    shared_limit: float = 0.0
    kind = "moe_softmax_clamped"


@dataclass
class TopkSoftmaxMoeSpec:
    """Routed squared-ReLU experts without gates; the weights are a softmax over the chosen logits (TopkSoftmaxReluSqMoe)."""
    experts: int
    top: int
    ff: int
    shared_ff: int = 0
    kind = "moe_topk_softmax_relu2"


@dataclass
class DenseSpec:
    """down(xIELU(up h + b) ) + b (XieluFeedForward)."""
    ff: int
    kind = "dense_xielu"


@dataclass
class GluSpec:
    """down(silu(gate h) * (up h)) (GluFeedForward)."""
    ff: int
    kind = "dense_glu_silu"


@dataclass
class LayerSpec:
    kind: str
    mixer: object
    ff: Optional[object]       # MoeSpec | ClampedMoeSpec | DenseSpec | None
    prefix: str                # tensor-name prefix of the layer
    weights_of: Optional[int] = None   # index of the layer whose tensors (mixer, feed-forward, norms) this layer uses; its pages and state slots are its own


@dataclass
class HybridSpec:
    vocab: int
    width: int
    eps: float
    layers: List[LayerSpec]
    embed: str = "embed"
    final_norm: str = "final.norm"
    head: str = "head"
    norm: str = "rms_one_plus"   # "rms_one_plus": x / rms * (1 + w);  "rms": x / rms * w;  "layer": (x - mean) / sqrt(var + eps) * w + b, the bias being the tensor `<name>.b`
    parallel_sublayers: bool = False   # x += mixer(norm1(x)) + feed_forward(norm2(x)), both norms of the same x (else one sublayer after the other)
    post_norms: bool = False     # every sublayer's output is normed (`norm1b` / `norm2b`) before it joins the residual stream
    embed_norm: Optional[str] = None   # tensor of a norm (of the model's kind) applied to the embedding rows
    residual_mult: float = 1.0   # every sublayer's output is multiplied by this before it joins the residual stream(s)
    streams: int = 0             # > 0: that many residual streams with per-sublayer read / write / mixing weights (`hc1.*` / `hc2.*`: in [S], out [S], mix [S, S] from -> to)


def gekilix_spec(cfg: dict) -> HybridSpec:
    """config.json of a Gekilix checkpoint -> the layer list.  Every size and every model-dependent constant comes from the file."""
    layers = []
    for i, L in enumerate(cfg["layers"]):
        m = L["mixer"]
        if L["type"] == "mamba2":
            mixer = Mamba2Spec(int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["conv"]), int(m.get("norm_groups", 1)))
        elif L["type"] == "attention":
            rot = m.get("rot")
            mask = m.get("mask") or {}
            mixer = AttentionSpec(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]), int(mask.get("size", 0) or 0),
                                  int(mask.get("keep_first", 0) or 0),
                                  RotarySpec(int(rot["dims"]), float(rot["base"]), rot.get("scaling")) if rot and int(rot.get("dims", 0)) > 0 else None)
        else:
            raise ValueError(f"Gekilix: unknown layer type {L['type']!r}")
        f = L.get("mlp")
        ff = None
        if f:
            if f.get("kind", "moe") != "moe":
                raise ValueError(f"Gekilix: unknown feed-forward kind {f.get('kind')!r}")
            sh = f.get("shared")
            ff = MoeSpec(int(f["router"]["experts"]), int(f["router"]["top"]), int(f["expert"]["ff"]), int(sh["ff"]) if sh else 0)
        layers.append(LayerSpec(L["type"], mixer, ff, f"l{i}."))
    return HybridSpec(int(cfg["vocab"]), int(cfg["width"]), float(cfg["norm"]["eps"]), layers)


def sobunex_spec(cfg: dict) -> HybridSpec:
    """config.json of a Sobunex checkpoint -> the layer list: layer norms (weight and bias) before and after every sublayer, sigmoid attention mixers (some reading an
    earlier layer's K / V pages), dense xIELU or softmax-routed clamped-GLU feed-forwards.  Every size and every model-dependent constant comes from the file."""
    layers = []
    for i, L in enumerate(cfg["layers"]):
        m = L["mixer"]
        if L["type"] != "attention":
            raise ValueError(f"Sobunex: unknown layer type {L['type']!r}")
        mask, qt = m.get("mask") or {}, m.get("q_temp") or {}
        src = m.get("kv_from")
        if src is not None and not 0 <= int(src) < i:
            raise ValueError(f"Sobunex: layer {i} reads the keys of layer {src}, which does not run before it")
        mixer = TalkAttentionSpec(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]), int(mask.get("size", 0) or 0),
                                  float(qt.get("coef", 0.0) or 0.0), int(qt.get("every", 0) or 0) if qt.get("coef") else 0, None if src is None else int(src))
        f = L.get("mlp")
        ff = None
        if f:
            if f.get("kind") == "dense":
                ff = DenseSpec(int(f["ff"]))
            elif f.get("kind") == "moe":
                r, sh = f["router"], f.get("shared")
                ff = ClampedMoeSpec(int(r["experts"]), int(r["top"]), int(f["expert"]["ff"]), float(f["expert"]["limit"]), float(r.get("scale", 1.0)),
                                    int(sh["ff"]) if sh else 0, float(sh["limit"]) if sh else 0.0)
            else:
                raise ValueError(f"Sobunex: unknown feed-forward kind {f.get('kind')!r}")
        layers.append(LayerSpec("talk_attention", mixer, ff, f"l{i}."))
    for i, ls in enumerate(layers):
        j = ls.mixer.kv_from
        if j is not None:
            o = layers[j].mixer
            if o.kv_from is not None or (o.kv_heads, o.dim, o.vdim) != (ls.mixer.kv_heads, ls.mixer.dim, ls.mixer.vdim):
                raise ValueError(f"Sobunex: layer {i} cannot read the keys and values of layer {j} (no projections of its own there, or other head sizes)")
    return HybridSpec(int(cfg["vocab"]), int(cfg["width"]), float(cfg["norm"]["eps"]), layers, norm="layer", post_norms=True)


def setopel_spec(cfg: dict) -> HybridSpec:
    """config.json of a Setopel checkpoint -> the layer list: a normed embedding, one-plus RMS norms in front of every sublayer, sublayer outputs scaled by `residual_mult`,
    optionally several residual streams; mixers `attention` (sink softmax, convolved q / k / v, some reading an earlier layer's pages), `retention` and `latent_attention`;
    SiLU-GLU feed-forwards.  Every size and every model-dependent constant comes from the file; a key that is absent switches its mechanism off."""
    layers = []
    for i, L in enumerate(cfg["layers"]):
        m, kind = L["mixer"], L["type"]
        if kind == "attention":
            qt = m.get("q_temp") or {}
            src = m.get("kv_from")
            if src is not None and not 0 <= int(src) < i:
                raise ValueError(f"Setopel: layer {i} reads the keys of layer {src}, which does not run before it")
            mixer = SinkAttentionSpec(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"]), float(m["scale"]), int(m.get("conv", 0) or 0),
                                      float(m.get("softcap", 0.0) or 0.0), float(qt.get("coef", 0.0) or 0.0), int(qt.get("every", 0) or 0) if qt.get("coef") else 0,
                                      None if src is None else int(src))
            kind = "sink_attention"
        elif kind == "retention":
            rot = m.get("rot")
            decay = [float(d) for d in m["decay"]]
            if len(decay) != int(m["heads"]):
                raise ValueError(f"Setopel: layer {i} lists {len(decay)} decays for {m['heads']} heads")
            mixer = RetentionSpec(int(m["heads"]), int(m["dim"]), int(m["vdim"]), decay,
                                  RotarySpec(int(rot["dims"]), float(rot["base"]), None, "half") if rot and int(rot.get("dims", 0)) > 0 else None)
        elif kind == "latent_attention":
            mixer = LatentAttentionSpec(int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"]), float(m["scale"]))
        else:
            raise ValueError(f"Setopel: unknown layer type {L['type']!r}")
        f = L.get("mlp")
        ff = None
        if f:
            if f.get("kind") != "dense":
                raise ValueError(f"Setopel: unknown feed-forward kind {f.get('kind')!r}")
            ff = GluSpec(int(f["ff"]))
        layers.append(LayerSpec(kind, mixer, ff, f"l{i}."))
    for i, ls in enumerate(layers):
        j = getattr(ls.mixer, "kv_from", None)
        if j is not None:
            o = layers[j].mixer
            if not isinstance(o, SinkAttentionSpec) or o.kv_from is not None or (o.kv_heads, o.dim, o.vdim) != (ls.mixer.kv_heads, ls.mixer.dim, ls.mixer.vdim):
                raise ValueError(f"Setopel: layer {i} cannot read the keys and values of layer {j} (no projections of its own there, or other head sizes)")
    return HybridSpec(int(cfg["vocab"]), int(cfg["width"]), float(cfg["norm"]["eps"]), layers, embed_norm="embed.norm", residual_mult=float(cfg.get("residual_mult", 1.0)),
                      streams=int(cfg.get("streams", 0) or 0))


def gifopel_spec(cfg: dict) -> HybridSpec:
    """config.json of a Gifopel checkpoint -> the layer list: plain-weight RMS norms, layers whose mixer and feed-forward read two norms of the same residual row, mixers
    `channel_delta` (delta rule with decays per key channel), `mlstm`, `parallel` (chunked sink attention next to a delta rule with decays per head), dense SiLU-GLU or routed
    squared-ReLU feed-forwards, layers that use another layer's tensors, a head tied to the embedding.  Every size and every model-dependent constant comes from the file."""
    def delta(m, decay, gate):
        return DeltaRuleSpec(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"]), int(m["conv"]), decay, gate)

    def attention(m):
        rot, mask = m.get("rot"), m.get("mask") or {}
        return AttentionSpec(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"]), float(m["scale"]), 0, 0,
                             RotarySpec(int(rot["dims"]), float(rot["base"])) if rot and int(rot.get("dims", 0)) > 0 else None, True,
                             chunk=int(mask.get("size", 0) or 0), head_norm=True, sink=True, head_gate=True)
    layers = []
    for i, L in enumerate(cfg["layers"]):
        m, kind = L["mixer"], L["type"]
        if kind == "channel_delta":
            kind, mixer = "delta_rule", delta(m, "channel", "sigmoid_lowrank")
        elif kind == "mlstm":
            mixer = MlstmSpec(int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"]))
        elif kind == "parallel":
            mixer = ParallelSpec("attention", attention(m["left"]), "delta_rule", delta(m["right"], "head", "silu"))
        else:
            raise ValueError(f"Gifopel: unknown layer type {L['type']!r}")
        f = L.get("mlp")
        ff = None
        if f:
            if f.get("kind") == "dense":
                ff = GluSpec(int(f["ff"]))
            elif f.get("kind") == "moe":
                ff = TopkSoftmaxMoeSpec(int(f["router"]["experts"]), int(f["router"]["top"]), int(f["expert"]["ff"]))
            else:
                raise ValueError(f"Gifopel: unknown feed-forward kind {f.get('kind')!r}")
        src = L.get("weights_of")
        layers.append(LayerSpec(kind, mixer, ff, f"l{i if src is None else int(src)}.", None if src is None else int(src)))
    for i, ls in enumerate(layers):
        j = ls.weights_of
        if j is not None:
            if not 0 <= j < len(layers) or j == i or layers[j].weights_of is not None:
                raise ValueError(f"Gifopel: layer {i} uses the tensors of layer {j}, which has none of its own")
            if (layers[j].kind, layers[j].mixer, layers[j].ff) != (ls.kind, ls.mixer, ls.ff):
                raise ValueError(f"Gifopel: layer {i} uses the tensors of layer {j} but is described differently")
    return HybridSpec(int(cfg["vocab"]), int(cfg["width"]), float(cfg["norm"]["eps"]), layers, head="embed", norm="rms", parallel_sublayers=True)


# ------------------------------------------------------------------------------------------------------------------ mixers and feed-forwards
class _Module:
    out_bias = None            # f32 bias of the module's last product, left to the caller (a norm that follows adds it while it reads the product)
    wants_f32_input = False    # feed-forwards: the normed rows are needed in f32 too (routers)

    def __init__(self, model: "HybridDecoder"):
        self.m = model

    def w(self, get, name, gemm: bool):
        """A checkpoint tensor on the device: GEMM operands in the serving dtype, everything else f32."""
        t = get(name)
        return t.to(self.m.device, self.m.torch_dtype if gemm else torch.float32).contiguous()

    def carried(self):
        return ()

    def share_from(self, other: "_Module") -> None:
        """Use `other`'s loaded tensors (a layer that borrows another layer's weights); what this module carries per sequence -- pages, taps, states -- stays its own."""
        mine = {k for k, v in self.__dict__.items() if isinstance(v, torch.Tensor) and any(v is t for t in self.carried())}
        for k, v in other.__dict__.items():
            if k not in mine and k != "m":
                setattr(self, k, v)


class Mamba2Mixer(_Module):
    """in-projection -> [z | x | B | C | dt]; causal convolution + SiLU over x, B, C; dt = softplus(dt + bias); per head S <- exp(-exp(A_log) dt) S + dt B x^T,
    y = S^T C + D x; y * silu(z); RMS norm in `norm_groups` parts; out-projection.  Carries the last conv - 1 inputs and S (f32) per sequence slot."""

    def __init__(self, model, spec: Mamba2Spec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix
        if spec.inner % spec.norm_groups or spec.heads % spec.groups:
            raise ValueError("mamba2: heads % groups and (heads * vdim) % norm_groups must be 0")
        slots, dev = model.state_slots, model.device
        self.conv_state = torch.zeros(slots, spec.conv_channels, max(spec.conv - 1, 1), dtype=torch.float32, device=dev)
        self.ssm_state = torch.zeros(slots, spec.heads, spec.state, spec.vdim, dtype=torch.float32, device=dev)

    def load(self, get):
        s, p = self.s, self.p
        self.w_in, self.w_o = self.w(get, p + "in", True), self.w(get, p + "o", True)
        self.conv_w, self.conv_b = self.w(get, p + "conv", False), self.w(get, p + "conv.b", False)
        self.dt_bias, self.A_log, self.D, self.norm = (self.w(get, p + n, False) for n in ("dt_bias", "A_log", "D", "norm"))
        n_in = 2 * s.inner + 2 * s.groups * s.state + s.heads
        if tuple(self.w_in.shape) != (n_in, self.m.spec.width) or tuple(self.conv_w.shape) != (s.conv_channels, s.conv):
            raise ValueError(f"{p}: tensor shapes do not match the mixer's sizes")

    def carried(self):
        return (self.conv_state, self.ssm_state)

    def forward(self, h, x, b: RaggedBatch, accumulate: bool = True):
        s, m = self.s, self.m
        T = b.rows
        u = m.linear(h, self.w_in)                                         # f32 [T, z | x B C | dt]
        xbc = torch.empty(T, s.conv_channels, dtype=torch.float32, device=m.device)
        _call("mrs_hyb_conv_silu", u[:, s.inner:], u.stride(0), self.conv_w, self.conv_b, self.conv_state, b.tok_seq, b.seq_start, b.seq_pos0, b.seq_slot, xbc,
              T, b.entries, s.conv_channels, s.conv)
        y = torch.empty(T, s.inner, dtype=torch.float32, device=m.device)
        steps = torch.empty(T, s.heads, 2, dtype=torch.float32, device=m.device)
        carry = decay = None
        if b.segments > b.entries:   # some portion is longer than a segment: scratch for the segments' local end states
            carry = torch.empty(b.segments, s.heads, s.state, s.vdim, dtype=torch.float32, device=m.device)
            decay = torch.empty(b.segments, s.heads, dtype=torch.float32, device=m.device)
        _call("mrs_hyb_ssd_scan", xbc, u, self.dt_bias, self.A_log, self.D, self.ssm_state, y, b.seq_pos0, b.seq_slot, b.seg_entry, b.seg_row0, b.seg_len, b.ent_seg0,
              steps, carry, decay, T, b.entries, b.segments, s.conv_channels, u.stride(0), s.inner + s.conv_channels, s.heads, s.vdim, s.state, s.groups)
        yn = m.norm(y, self.norm, one_plus=False, parts=s.norm_groups, gate=u)   # y * silu(z) (z = the first `inner` columns of u), then the grouped norm
        m.linear(yn, self.w_o, out=x, accumulate=accumulate)

    def state_bytes_per_slot(self) -> int:
        return 4 * (self.conv_state[0].numel() + self.ssm_state[0].numel())


class WindowAttention(_Module):
    """q, k, v projections (one product); plain-weight RMS norm over the WHOLE query and key projections; interleaved rotary on the first dims of every head; K / V into
    pages; softmax over the keys j <= i with i - j < window or j < keep_first (true positions throughout); out-projection.  Grouped heads: query head h reads key / value
    head h // (heads / kv_heads); key and value head sizes are independent."""

    def __init__(self, model, spec: AttentionSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix
        dev, bs, nb = model.device, model.block_size, model.num_blocks
        self.k_cache = torch.zeros(nb, spec.kv_heads, bs, spec.dim, dtype=model.torch_dtype, device=dev)
        self.v_cache = torch.zeros(nb, spec.kv_heads, bs, spec.vdim, dtype=model.torch_dtype, device=dev)
        self.freq = torch.from_numpy(spec.rotary.frequencies()).to(dev) if spec.rotary else torch.zeros(1, dtype=torch.float32, device=dev)

    def load(self, get):
        s, p = self.s, self.p
        q, k, v = (get(p + n) for n in ("q", "k", "v"))
        if q.shape[0] != s.heads * s.dim or k.shape[0] != s.kv_heads * s.dim or v.shape[0] != s.kv_heads * s.vdim:
            raise ValueError(f"{p}: projection shapes do not match the mixer's sizes")
        parts = [q, k, v]
        if s.head_gate:
            parts.append(get(p + "g"))
            if tuple(parts[-1].shape) != (s.heads, q.shape[1]):
                raise ValueError(f"{p}: the gate projection has one row per head")
        self.w_qkv = torch.cat(parts, 0).to(self.m.device, self.m.torch_dtype).contiguous()   # [q | k | v (| gate logits), W]
        self.gate_col = s.heads * s.dim + s.kv_heads * (s.dim + s.vdim)
        self.w_o = self.w(get, p + "o", True)
        self.q_norm = self.w(get, p + "q.norm", False) if s.qk_norm else None
        self.k_norm = self.w(get, p + "k.norm", False) if s.qk_norm else None
        if s.qk_norm and (self.q_norm.numel(), self.k_norm.numel()) != ((s.dim, s.dim) if s.head_norm else (s.heads * s.dim, s.kv_heads * s.dim)):
            raise ValueError(f"{p}: query / key norm weights do not match the mixer's sizes")
        self.sink = self.w(get, p + "sink", False) if s.sink else None
        if s.sink and self.sink.numel() != s.heads:
            raise ValueError(f"{p}: one sink per head")
        if s.chunk and (s.window or s.keep_first):
            raise ValueError(f"{p}: chunks and a sliding window exclude each other")

    def carried(self):
        return (self.k_cache, self.v_cache)

    def kv_bytes_per_token(self) -> int:
        return self.k_cache.element_size() * self.s.kv_heads * (self.s.dim + self.s.vdim)

    def forward(self, h, x, b: RaggedBatch, accumulate: bool = True):
        s, m = self.s, self.m
        T = b.rows
        qkv = m.linear(h, self.w_qkv)
        q = torch.empty(T, s.heads * s.dim, dtype=m.torch_dtype, device=m.device)
        _call("mrs_hyb_qk_headnorm_rope_cache" if s.head_norm else "mrs_hyb_qk_norm_rope_cache", qkv, qkv.stride(0), self.q_norm, self.k_norm, self.freq, b.tok_pos,
              b.slot_mapping, q, self.k_cache, self.v_cache, T, s.heads, s.kv_heads, s.dim, s.vdim, s.rotary.dims if s.rotary else 0, m.block_size, m.spec.eps, m.dt)
        o = torch.empty(T, s.heads * s.vdim, dtype=m.torch_dtype, device=m.device)
        if s.chunk or s.sink or s.head_gate:
            if s.window or s.keep_first:
                raise NotImplementedError("a learned sink / a per-head gate beside a sliding window")
            scratch, splits = m.key_splits(b, s.heads, s.vdim, s.chunk)   # single-row steps deal a long chunk's keys to several workgroups
            _call("mrs_hyb_paged_attn_chunked", q, self.k_cache, self.v_cache, b.block_tables, b.tok_seq, b.tok_pos, o, T, s.heads, s.kv_heads, s.dim, s.vdim, m.block_size,
                  b.max_blocks, s.chunk, s.scale, m.dt, b.seg_entry, b.seg_row0, b.seg_len, b.segments, RaggedBatch.SEGMENT, 0.0, int(s.sink), self.sink,
                  qkv[:, self.gate_col:] if s.head_gate else None, qkv.stride(0), 1, scratch, splits)
        else:
            _call("mrs_hyb_paged_window_attn", q, self.k_cache, self.v_cache, b.block_tables, b.tok_seq, b.tok_pos, o, T, s.heads, s.kv_heads, s.dim, s.vdim, m.block_size,
                  b.max_blocks, s.window, s.keep_first, s.scale, m.dt, b.seg_entry, b.seg_row0, b.seg_len, b.segments, RaggedBatch.SEGMENT)
        m.linear(o, self.w_o, out=x, accumulate=accumulate)


class TalkSigmoidAttention(_Module):
    """q, k, v and the output projection with biases, the per-head gate logits in the same product.  No rotation: positions enter through a query temperature
    (q *= 1 + coef ln(floor((pos + 1) / every) + 1)) and a per-head distance bias.  Head g scores key j as scale (q_g . k_j) - 2^(-8 (g + 1) / heads) (i - j); the heads'
    scores are mixed by the [heads, heads] matrix `talk`; a key with 0 <= i - j < window weighs sigmoid(mixed + pb_h), un-normalised; head outputs are multiplied by
    sigmoid(gate logit), then projected.  With `kv_from` the layer has no key / value projections: it reads the K / V pages of that earlier layer (same block tables)."""
    KEY_SPLITS = 64      # at most this many workgroups share a row's keys
    SPLIT_ROWS = 128     # steps of at most this many rows may split

    def __init__(self, model, spec: TalkAttentionSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix
        if spec.heads % spec.kv_heads:
            raise ValueError(f"{prefix}: heads % kv_heads must be 0")
        dev, bs, nb = model.device, model.block_size, model.num_blocks
        self.k_cache = self.v_cache = None
        if spec.kv_from is None:
            self.k_cache = torch.zeros(nb, spec.kv_heads, bs, spec.dim, dtype=model.torch_dtype, device=dev)
            self.v_cache = torch.zeros(nb, spec.kv_heads, bs, spec.vdim, dtype=model.torch_dtype, device=dev)
        self.slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / spec.heads) for h in range(spec.heads)], dtype=torch.float64).to(dev, torch.float32)

    def carried(self):
        return (self.k_cache, self.v_cache) if self.k_cache is not None else ()

    def kv_bytes_per_token(self) -> int:
        return self.k_cache.element_size() * self.s.kv_heads * (self.s.dim + self.s.vdim) if self.k_cache is not None else 0

    def load(self, get):
        s, p, own = self.s, self.p, self.s.kv_from is None
        names = ["q", "k", "v"] if own else ["q"]
        parts = [get(p + n) for n in names] + [get(p + "g")]
        want = [s.heads * s.dim, s.kv_heads * s.dim, s.kv_heads * s.vdim][:len(names)] + [s.heads]
        if [t.shape[0] for t in parts] != want or any(t.shape[1] != self.m.spec.width for t in parts):
            raise ValueError(f"{p}: projection shapes do not match the mixer's sizes")
        self.w_in = torch.cat(parts, 0).to(self.m.device, self.m.torch_dtype).contiguous()     # [q | k | v | gate, W]
        self.gate_col = sum(want[:-1])
        self.qb = self.w(get, p + "q.b", False)
        self.kb = self.w(get, p + "k.b", False) if own else None
        self.vb = self.w(get, p + "v.b", False) if own else None
        self.w_o, self.out_bias = self.w(get, p + "o", True), self.w(get, p + "o.b", False)
        self.talk, self.pb = self.w(get, p + "talk", False), self.w(get, p + "pb", False)
        if tuple(self.talk.shape) != (s.heads, s.heads) or self.pb.numel() != s.heads or tuple(self.w_o.shape) != (self.m.spec.width, s.heads * s.vdim):
            raise ValueError(f"{p}: head-mixing / output shapes do not match the mixer's sizes")

    def forward(self, h, x, b: RaggedBatch, accumulate: bool = True):
        s, m = self.s, self.m
        T = b.rows
        u = m.linear(h, self.w_in)                                         # f32 [T, q | k | v | gate logits]
        q = torch.empty(T, s.heads * s.dim, dtype=m.torch_dtype, device=m.device)
        _call("mrs_hyb_qkv_bias_temp_cache", u, u.stride(0), self.qb, self.kb, self.vb, b.tok_pos, b.slot_mapping, q, self.k_cache, self.v_cache, T, s.heads, s.kv_heads,
              s.dim, s.vdim, m.block_size, s.temp_coef, s.temp_every, m.dt)
        src = self if s.kv_from is None else m.layers[s.kv_from].mixer      # that layer ran earlier in this step: its pages hold this step's rows already
        o = torch.empty(T, s.heads * s.vdim, dtype=m.torch_dtype, device=m.device)
        # a step of few rows deals every row's keys to several workgroups: room for their partial sums
        splits = min(self.KEY_SPLITS, -(-(min(s.window, b.max_blocks * m.block_size) if s.window > 0 else b.max_blocks * m.block_size) // 64)) if T <= self.SPLIT_ROWS else 0
        scratch = torch.empty(splits, T, s.heads * s.vdim, dtype=torch.float32, device=m.device) if splits > 1 else None
        _call("mrs_hyb_paged_talk_sigmoid_attn", q, src.k_cache, src.v_cache, b.block_tables, b.tok_pos, self.talk, self.pb, self.slopes, u[:, self.gate_col:], u.stride(0), o,
              T, s.heads, s.kv_heads, s.dim, s.vdim, m.block_size, b.max_blocks, s.window, s.scale, m.dt, b.seg_entry, b.seg_row0, b.seg_len, b.segments, b.seg_rows,
              scratch, splits)
        m.linear(o, self.w_o, out=x, accumulate=accumulate)


class SigmoidMoe(_Module):
    """Router logits in f32, scores = sigmoid, the `top` largest, un-renormalised; the score multiplies the expert's INPUT: out = sum_e expert_e(s_e h), expert =
    down(silu(gate h) * (up h)); plus sigmoid(sg . h) * shared(h).  All experts of a step run as grouped products over expert-sorted rows."""

    def __init__(self, model, spec: MoeSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix

    wants_f32_input = True

    def load(self, get):
        s, p, m = self.s, self.p, self.m
        dev, dt = m.device, m.torch_dtype
        self.w_gu = torch.stack([torch.cat([get(f"{p}e{e}.gate"), get(f"{p}e{e}.up")], 0) for e in range(s.experts)]).to(dev, dt).contiguous()   # [E, 2 ff, W]
        self.w_down = torch.stack([get(f"{p}e{e}.down") for e in range(s.experts)]).to(dev, dt).contiguous()                                      # [E, W, ff]
        if tuple(self.w_gu.shape[1:]) != (2 * s.ff, m.spec.width):
            raise ValueError(f"{p}: expert shapes do not match the layer's sizes")
        rows = [get(p + "router")]
        if s.shared_ff:
            rows.append(get(p + "shared.sg").reshape(1, -1))
            self.ws_gu = torch.cat([get(p + "shared.gate"), get(p + "shared.up")], 0).to(dev, dt).contiguous()
            self.ws_down = self.w(get, p + "shared.down", True)
        self.w_router = torch.cat(rows, 0).to(dev, torch.float32).contiguous()   # [E (+ 1), W] f32: router rows, then the shared expert's gate row

    def forward(self, h, h32, x, b: RaggedBatch, accumulate: bool = True):
        s, m = self.s, self.m
        T, W, dev = b.rows, m.spec.width, m.device
        if not accumulate:
            x.zero_()
        R = T * s.top
        ids = torch.empty(R, dtype=torch.int32, device=dev)
        wts = torch.empty(R, dtype=torch.float32, device=dev)
        gate = torch.empty(T, dtype=torch.float32, device=dev) if s.shared_ff else None
        _call("mrs_hyb_route_sigmoid_topk", h32, self.w_router, T, W, s.experts, s.top, int(bool(s.shared_ff)), ids, wts, gate)
        meta = torch.empty(s.experts + 1 + 3 * R, dtype=torch.int32, device=dev)
        bounds, sorted_route, route_pos, sorted_expert = meta[:s.experts + 1], meta[s.experts + 1:][:R], meta[s.experts + 1 + R:][:R], meta[s.experts + 1 + 2 * R:][:R]
        _call("mrs_hyb_moe_dispatch", ids, R, s.experts, bounds, sorted_route, route_pos, sorted_expert)
        f32 = dict(dtype=torch.float32, device=dev)
        if R <= m.GROUPED_GEMV_ROWS:
            # decode-sized steps: every route streams its expert's slabs; the scaled gather and the GLU happen in the consuming product's operand load (same roundings)
            gu = torch.empty(R, 2 * s.ff, **f32)
            _call("mrs_hyb_gemv", h32, self.w_gu, gu, R, 2 * s.ff, W, h32.stride(0), W, 2 * s.ff, m.dt, 0, sorted_expert, self.w_gu.stride(0), 2, sorted_route, wts, s.top)
            d = torch.empty(R, W, **f32)
            _call("mrs_hyb_gemv", gu, self.w_down, d, R, W, s.ff, 2 * s.ff, s.ff, W, m.dt, 0, sorted_expert, self.w_down.stride(0), 1, None, None, 1)
        else:
            xs = torch.empty(R, W, dtype=m.torch_dtype, device=dev)
            _call("mrs_hyb_moe_gather", h32, sorted_route, wts, s.top, xs, R, W, m.dt)
            gu = m.grouped_linear(xs, self.w_gu, bounds, sorted_expert)
            act = torch.empty(R, s.ff, dtype=m.torch_dtype, device=dev)
            _call("mrs_hyb_glu_silu", gu, act, R, s.ff, m.dt)
            d = m.grouped_linear(act, self.w_down, bounds, sorted_expert)
        sh = None
        if s.shared_ff:
            sgu = m.linear(h, self.ws_gu)
            if T <= m.GEMV_ROWS:
                sh = torch.empty(T, W, **f32)
                _call("mrs_hyb_gemv", sgu, self.ws_down, sh, T, W, s.shared_ff, 2 * s.shared_ff, s.shared_ff, W, m.dt, 0, None, 0, 1, None, None, 1)
            else:
                sact = torch.empty(T, s.shared_ff, dtype=m.torch_dtype, device=dev)
                _call("mrs_hyb_glu_silu", sgu, sact, T, s.shared_ff, m.dt)
                sh = m.linear(sact, self.ws_down)
        _call("mrs_hyb_moe_combine", x, d, route_pos, s.top, sh, gate, T, W)


class ClampedSoftmaxMoe(_Module):
    """Router logits in f32, scores = softmax over all experts, the `top` largest; weights = route_scale * score, un-renormalised, on the experts' OUTPUTS.  Expert (no
    biases): g = min(gate h, limit), u = clamp(up h, -limit, limit), down(g sigmoid(1.702 g) (u + 1)); a shared expert of the same form (its own size and limit) runs for
    every row with weight 1.  All experts of a step run as grouped products over expert-sorted rows."""
    ALPHA = 1.702
    wants_f32_input = True

    def __init__(self, model, spec: ClampedMoeSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix

    def load(self, get):
        s, p, m = self.s, self.p, self.m
        dev, dt = m.device, m.torch_dtype
        self.w_gu = torch.stack([torch.cat([get(f"{p}e{e}.gate"), get(f"{p}e{e}.up")], 0) for e in range(s.experts)]).to(dev, dt).contiguous()   # [E, 2 ff, W]
        self.w_down = torch.stack([get(f"{p}e{e}.down") for e in range(s.experts)]).to(dev, dt).contiguous()                                      # [E, W, ff]
        self.w_router = self.w(get, p + "router", False)
        if tuple(self.w_gu.shape[1:]) != (2 * s.ff, m.spec.width) or tuple(self.w_router.shape) != (s.experts, m.spec.width):
            raise ValueError(f"{p}: expert / router shapes do not match the layer's sizes")
        if s.shared_ff:
            self.ws_gu = torch.cat([get(p + "shared.gate"), get(p + "shared.up")], 0).to(dev, dt).contiguous()
            self.ws_down = self.w(get, p + "shared.down", True)
            if tuple(self.ws_gu.shape) != (2 * s.shared_ff, m.spec.width):
                raise ValueError(f"{p}: shared expert shapes do not match the layer's sizes")

    def forward(self, h, h32, x, b: RaggedBatch, accumulate: bool = True):
        s, m = self.s, self.m
        T, W, dev = b.rows, m.spec.width, m.device
        R = T * s.top
        ids = torch.empty(R, dtype=torch.int32, device=dev)
        wts = torch.empty(R, dtype=torch.float32, device=dev)
        _call("mrs_hyb_route_softmax_topk", h32, self.w_router, T, W, s.experts, s.top, s.route_scale, ids, wts)
        meta = torch.empty(s.experts + 1 + 3 * R, dtype=torch.int32, device=dev)
        bounds, sorted_route, route_pos, sorted_expert = meta[:s.experts + 1], meta[s.experts + 1:][:R], meta[s.experts + 1 + R:][:R], meta[s.experts + 1 + 2 * R:][:R]
        _call("mrs_hyb_moe_dispatch", ids, R, s.experts, bounds, sorted_route, route_pos, sorted_expert)
        f32 = dict(dtype=torch.float32, device=dev)
        if R <= m.GROUPED_GEMV_ROWS:
            # decode-sized steps: every route streams its expert's slabs; the row gather and the clamped GLU happen in the consuming product's operand load (same roundings)
            gu = torch.empty(R, 2 * s.ff, **f32)
            m.gemv_act(h32, self.w_gu, gu, R, 2 * s.ff, W, h32.stride(0), W, sorted_expert, self.w_gu.stride(0), 2, sorted_route, s.top)
            d = torch.empty(R, W, **f32)
            m.gemv_act(gu, self.w_down, d, R, W, s.ff, 2 * s.ff, s.ff, sorted_expert, self.w_down.stride(0), 3, p0=s.limit, p1=self.ALPHA)
        else:
            xs = torch.empty(R, W, dtype=m.torch_dtype, device=dev)
            _call("mrs_hyb_moe_gather", h32, sorted_route, None, s.top, xs, R, W, m.dt)
            gu = m.grouped_linear(xs, self.w_gu, bounds, sorted_expert)
            act = torch.empty(R, s.ff, dtype=m.torch_dtype, device=dev)
            _call("mrs_hyb_glu_clamped", gu, act, R, s.ff, s.limit, self.ALPHA, m.dt)
            d = m.grouped_linear(act, self.w_down, bounds, sorted_expert)
        sh = None
        if s.shared_ff:
            sgu = m.linear(h, self.ws_gu)
            if T <= m.GEMV_ROWS:
                sh = torch.empty(T, W, **f32)
                m.gemv_act(sgu, self.ws_down, sh, T, W, s.shared_ff, 2 * s.shared_ff, s.shared_ff, None, 0, 3, p0=s.shared_limit, p1=self.ALPHA)
            else:
                sact = torch.empty(T, s.shared_ff, dtype=m.torch_dtype, device=dev)
                _call("mrs_hyb_glu_clamped", sgu, sact, T, s.shared_ff, s.shared_limit, self.ALPHA, m.dt)
                sh = m.linear(sact, self.ws_down)
        _call("mrs_hyb_moe_combine_weighted", x, d, route_pos, wts, s.top, sh, T, W, int(accumulate))


class XieluFeedForward(_Module):
    """down(act(up h + b_up)) + b_down with act = xIELU: z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1 / 2 + softplus(q)) (e^z - 1 - z) + z / 2; p, q = the tensor `act`."""

    def __init__(self, model, spec: DenseSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix

    def load(self, get):
        s, p, W = self.s, self.p, self.m.spec.width
        self.w_up, self.w_down = self.w(get, p + "up", True), self.w(get, p + "down", True)
        self.b_up, self.out_bias = self.w(get, p + "up.b", False), self.w(get, p + "down.b", False)
        if tuple(self.w_up.shape) != (s.ff, W) or tuple(self.w_down.shape) != (W, s.ff):
            raise ValueError(f"{p}: projection shapes do not match the layer's sizes")
        pq = np.asarray(get(p + "act").to(torch.float32).cpu().numpy(), dtype=np.float32).reshape(-1)
        sp = lambda v: np.float32(max(v, np.float32(0))) + np.log1p(np.exp(-np.abs(np.float32(v)), dtype=np.float32), dtype=np.float32)
        self.ap, self.an = float(sp(pq[0])), float(np.float32(0.5) + sp(pq[1]))

    def forward(self, h, h32, x, b: RaggedBatch, accumulate: bool = True):
        s, m = self.s, self.m
        T = b.rows
        u = m.linear(h, self.w_up)
        if T <= m.GEMV_ROWS:   # decode-sized steps: bias and activation in the down product's operand load
            m.gemv_act(u, self.w_down, x, T, x.shape[1], s.ff, u.stride(0), s.ff, None, 0, 4, bias=self.b_up, p0=self.ap, p1=self.an, accumulate=accumulate)
            return
        a = torch.empty(T, s.ff, dtype=m.torch_dtype, device=m.device)
        _call("mrs_hyb_bias_xielu", u, u.stride(0), self.b_up, a, T, s.ff, self.ap, self.an, m.dt)
        m.linear(a, self.w_down, out=x, accumulate=accumulate)


class GatedSinkAttention(_Module):
    """q, k, v (with biases) and the gate logits in one product; an optional short causal convolution over every q / k / v channel (no bias, no activation; the last
    taps - 1 projected rows ride in the sequence's state slot); no rotation: positions enter through a query temperature (q *= 1 + coef ln(floor((pos + 1) / every) + 1)).
    Score s = scale (q . k), optionally cap tanh(s / cap); causal softmax with a sink, p_j = e^{s_j} / (1 + sum e^{s}); the concatenated heads times sigmoid(gate logits)
    element by element, then the output projection.  With `kv_from` the layer has no key / value projections: it reads the K / V pages of that earlier layer."""

    def __init__(self, model, spec: SinkAttentionSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix
        if spec.heads % spec.kv_heads:
            raise ValueError(f"{prefix}: heads % kv_heads must be 0")
        dev, bs, nb = model.device, model.block_size, model.num_blocks
        self.own = spec.kv_from is None
        self.k_cache = self.v_cache = None
        if self.own:
            self.k_cache = torch.zeros(nb, spec.kv_heads, bs, spec.dim, dtype=model.torch_dtype, device=dev)
            self.v_cache = torch.zeros(nb, spec.kv_heads, bs, spec.vdim, dtype=model.torch_dtype, device=dev)
        self.nq, self.nk, self.nv = spec.heads * spec.dim, spec.kv_heads * spec.dim, spec.kv_heads * spec.vdim
        self.channels = self.nq + (self.nk + self.nv if self.own else 0)
        self.conv_state = torch.zeros(model.state_slots, self.channels, spec.conv - 1, dtype=torch.float32, device=dev) if spec.conv > 1 else None

    def carried(self):
        return tuple(t for t in (self.k_cache, self.v_cache, self.conv_state) if t is not None)

    def kv_bytes_per_token(self) -> int:
        return self.k_cache.element_size() * self.s.kv_heads * (self.s.dim + self.s.vdim) if self.own else 0

    def state_bytes_per_slot(self) -> int:
        return 4 * self.conv_state[0].numel() if self.conv_state is not None else 0

    def load(self, get):
        s, p, W = self.s, self.p, self.m.spec.width
        names = ["q", "k", "v"] if self.own else ["q"]
        parts = [get(p + n) for n in names] + [get(p + "g")]
        want = [self.nq, self.nk, self.nv][:len(names)] + [s.heads * s.vdim]
        if [t.shape[0] for t in parts] != want or any(t.shape[1] != W for t in parts):
            raise ValueError(f"{p}: projection shapes do not match the mixer's sizes")
        self.w_in = torch.cat(parts, 0).to(self.m.device, self.m.torch_dtype).contiguous()     # [q | k | v | gate, W]
        self.gate_col = self.channels
        self.bias = torch.cat([get(p + n + ".b").reshape(-1) for n in names], 0).to(self.m.device, torch.float32).contiguous()   # [q | k | v]
        self.conv_w = None
        if s.conv:
            self.conv_w = torch.cat([get(p + n + ".conv") for n in names], 0).to(self.m.device, torch.float32).contiguous()     # [channels, taps]
            if tuple(self.conv_w.shape) != (self.channels, s.conv):
                raise ValueError(f"{p}: convolution shapes do not match the mixer's sizes")
        self.w_o = self.w(get, p + "o", True)
        if self.bias.numel() != self.channels or tuple(self.w_o.shape) != (W, s.heads * s.vdim):
            raise ValueError(f"{p}: bias / output shapes do not match the mixer's sizes")

    def forward(self, h, x, b: RaggedBatch, accumulate: bool = True):
        s, m = self.s, self.m
        T = b.rows
        u = m.linear(h, self.w_in)                                         # f32 [T, q | k | v | gate logits]
        q = torch.empty(T, self.nq, dtype=m.torch_dtype, device=m.device)
        if s.conv:   # bias, convolution, temperature and the page write in one launch (the slots' taps in a second one when a portion is in the batch)
            _call("mrs_hyb_conv_qkv_cache", u, u.stride(0), self.bias, self.conv_w, self.conv_state, b.tok_seq, b.seq_start, b.seq_pos0, b.seq_slot, b.tok_pos, b.slot_mapping, q,
                  self.k_cache, self.v_cache, T, b.entries, s.heads, s.kv_heads, s.dim, s.vdim, m.block_size, s.conv, s.temp_coef, s.temp_every, m.dt)
        else:
            qb = self.bias[:self.nq]
            kb, vb = (self.bias[self.nq:self.nq + self.nk], self.bias[self.nq + self.nk:]) if self.own else (None, None)
            _call("mrs_hyb_qkv_bias_temp_cache", u, u.stride(0), qb, kb, vb, b.tok_pos, b.slot_mapping, q, self.k_cache, self.v_cache, T, s.heads, s.kv_heads, s.dim, s.vdim,
                  m.block_size, s.temp_coef, s.temp_every, m.dt)
        src = self if self.own else m.layers[s.kv_from].mixer               # that layer ran earlier in this step: its pages hold this step's rows already
        o = torch.empty(T, s.heads * s.vdim, dtype=m.torch_dtype, device=m.device)
        _call("mrs_hyb_paged_attn_opts", q, src.k_cache, src.v_cache, b.block_tables, b.tok_seq, b.tok_pos, o, T, s.heads, s.kv_heads, s.dim, s.vdim, m.block_size, b.max_blocks,
              0, 0, s.scale, m.dt, b.seg_entry, b.seg_row0, b.seg_len, b.segments, RaggedBatch.SEGMENT, s.softcap, int(s.sink), u[:, self.gate_col:], u.stride(0),
              *m.key_splits(b, s.heads, s.vdim), 0)
        m.linear(o, self.w_o, out=x, accumulate=accumulate)


class RetentionMixer(_Module):
    """v | k | q | gate in one product (no biases); half-split rotary on the first `rot.dims` dimensions of every query and key head (angles from f32 positions), keys
    times dim^(-1/2); per head the f32 state S [dim, vdim] <- decay_h S + k v^T and o = S^T q, carried per sequence slot; o / rms(o) per head (no weight), times
    silu(gate), output projection.  The recurrence is the state-space scan with unit steps and fixed decays (segments of a long portion run in parallel)."""

    def __init__(self, model, spec: RetentionSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix
        if spec.rotary and spec.rotary.layout != "half":
            raise ValueError(f"{prefix}: retention rotates half-split pairs")
        dev = model.device
        self.state = torch.zeros(model.state_slots, spec.heads, spec.dim, spec.vdim, dtype=torch.float32, device=dev)
        self.decay = torch.tensor(spec.decay, dtype=torch.float64).to(dev, torch.float32)
        self.freq = torch.from_numpy(spec.rotary.frequencies()).to(dev) if spec.rotary else None
        self.k_mult = float(np.float32(spec.dim) ** np.float32(-0.5))

    def carried(self):
        return (self.state,)

    def state_bytes_per_slot(self) -> int:
        return 4 * self.state[0].numel()

    def load(self, get):
        s, p, W = self.s, self.p, self.m.spec.width
        parts = [get(p + n) for n in ("v", "k", "q", "g")]
        want = [s.heads * s.vdim, s.heads * s.dim, s.heads * s.dim, s.heads * s.vdim]
        if [t.shape[0] for t in parts] != want or any(t.shape[1] != W for t in parts):
            raise ValueError(f"{p}: projection shapes do not match the mixer's sizes")
        self.w_in = torch.cat(parts, 0).to(self.m.device, self.m.torch_dtype).contiguous()     # [v | k | q | gate, W]
        self.k_col, self.q_col, self.gate_col = want[0], want[0] + want[1], want[0] + 2 * want[1]
        self.w_o = self.w(get, p + "o", True)
        if tuple(self.w_o.shape) != (W, s.heads * s.vdim):
            raise ValueError(f"{p}: output shape does not match the mixer's sizes")

    def forward(self, h, x, b: RaggedBatch, accumulate: bool = True):
        s, m = self.s, self.m
        T, dev = b.rows, m.device
        u = m.linear(h, self.w_in)                                         # f32 [T, v | k | q | gate]
        _call("mrs_hyb_rotary_half", u, u.stride(0), self.q_col, self.k_col, s.heads, s.dim, s.rotary.dims if s.rotary else 0, self.freq, b.tok_pos, self.k_mult, T)
        y = torch.empty(T, s.heads * s.vdim, dtype=torch.float32, device=dev)
        steps = torch.empty(T, s.heads, 2, dtype=torch.float32, device=dev)
        carry = decay = None
        if b.segments > b.entries:   # some portion is longer than a segment: scratch for the segments' local end states
            carry = torch.empty(b.segments, s.heads, s.dim, s.vdim, dtype=torch.float32, device=dev)
            decay = torch.empty(b.segments, s.heads, dtype=torch.float32, device=dev)
        _call("mrs_hyb_decay_scan", u, u.stride(0), self.decay, self.state, y, b.seq_pos0, b.seq_slot, b.seg_entry, b.seg_row0, b.seg_len, b.ent_seg0, steps, carry, decay,
              T, b.entries, b.segments, s.heads, s.vdim, s.dim, s.heads)
        yn = m.norm(y, None, one_plus=False, parts=s.heads, gate=u[:, self.gate_col:], gate_after=True)   # per-head unit norm, then silu(gate)
        m.linear(yn, self.w_o, out=x, accumulate=accumulate)


class LatentAttention(_Module):
    """q | latent in one product; the latent row c = norm(W_dkv h) (plain weight) is the only thing paged.  Head h's keys W_uk,h c and values W_uv,h c are never
    materialised: q'_h = W_uk,h^T q_h scores against the cached rows (one shared key / value head of kv_rank dimensions for all query heads), the weighted sum of cached
    rows is expanded by W_uv,h afterwards -- the same sums, reassociated.  Causal softmax, s = scale (q . k); no positions."""

    def __init__(self, model, spec: LatentAttentionSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix
        self.c_cache = torch.zeros(model.num_blocks, 1, model.block_size, spec.kv_rank, dtype=model.torch_dtype, device=model.device)

    def carried(self):
        return (self.c_cache,)

    def kv_bytes_per_token(self) -> int:
        return self.c_cache.element_size() * self.s.kv_rank

    def load(self, get):
        s, p, W = self.s, self.p, self.m.spec.width
        dev, dt = self.m.device, self.m.torch_dtype
        q, dkv, uk, uv = (get(p + n) for n in ("q", "dkv", "uk", "uv"))
        if tuple(q.shape) != (s.heads * s.dim, W) or tuple(dkv.shape) != (s.kv_rank, W) or tuple(uk.shape) != (s.heads * s.dim, s.kv_rank) or \
                tuple(uv.shape) != (s.heads * s.vdim, s.kv_rank):
            raise ValueError(f"{p}: projection shapes do not match the mixer's sizes")
        self.w_in = torch.cat([q, dkv], 0).to(dev, dt).contiguous()                                       # [q | latent, W]
        self.w_ukT = uk.reshape(s.heads, s.dim, s.kv_rank).transpose(1, 2).to(dev, dt).contiguous()       # [H, kv_rank, dim]: q' = this . q
        self.w_uv = uv.reshape(s.heads, s.vdim, s.kv_rank).to(dev, dt).contiguous()                       # [H, vdim, kv_rank]
        self.w_uk = uk.to(dev, dt).contiguous()                                                           # [H * dim, kv_rank]: the keys themselves (prompt steps)
        self.c_norm = self.w(get, p + "dkv.norm", False)
        self.w_o = self.w(get, p + "o", True)
        if self.c_norm.numel() != s.kv_rank or tuple(self.w_o.shape) != (W, s.heads * s.vdim):
            raise ValueError(f"{p}: norm / output shapes do not match the mixer's sizes")

    def forward(self, h, x, b: RaggedBatch, accumulate: bool = True):
        s, m = self.s, self.m
        T, dev, dt = b.rows, m.device, m.torch_dtype
        H, D, Dv, R = s.heads, s.dim, s.vdim, s.kv_rank
        u = m.linear(h, self.w_in)                                         # f32 [T, q | latent]
        q = torch.empty(T, H * D, dtype=dt, device=dev)
        _call("mrs_hyb_latent_norm_cache", u, u.stride(0), H * D, R, self.c_norm, b.slot_mapping, q, self.c_cache, m.spec.eps, T, m.dt)
        if self.expands(b):
            # a step with prompt portions: the contexts' latent rows are gathered block by block and expanded into keys and values of `dim` / `vdim` per head (two products
            # on the matrix cores); attention then costs dim + vdim per (query, key) pair instead of 2 kv_rank
            tables, source, n = b.context_blocks()
            bs = m.block_size
            per = bs * R * self.c_cache.element_size() // 4
            c = torch.empty(n * bs, R, dtype=dt, device=dev)
            _call("mrs_hyb_gather_rows", self.c_cache, source, c, n, per)
            k = m.linear_rounded(c, self.w_uk)                              # [n * bs, H * dim]: block, slot, head -- the attention kernel's token-major layout
            v = m.linear_rounded(c, self.w_uv.view(H * Dv, R))
            ov = torch.empty(T, H * Dv, dtype=dt, device=dev)
            _call("mrs_hyb_paged_attn_opts", q, k, v, tables, b.tok_seq, b.tok_pos, ov, T, H, H, D, Dv, bs, b.max_blocks, 0, 0, s.scale, m.dt, b.seg_entry, b.seg_row0, b.seg_len,
                  b.segments, RaggedBatch.SEGMENT, 0.0, 0, None, 0, None, 0, 1)
        else:
            qa = m.batched_linear(q, self.w_ukT, H)                        # [T, H * kv_rank] in the serving dtype
            oa = torch.empty(T, H * R, dtype=dt, device=dev)
            _call("mrs_hyb_paged_attn_opts", qa, self.c_cache, self.c_cache, b.block_tables, b.tok_seq, b.tok_pos, oa, T, H, 1, R, R, m.block_size, b.max_blocks, 0, 0, s.scale,
                  m.dt, b.seg_entry, b.seg_row0, b.seg_len, b.segments, RaggedBatch.SEGMENT, 0.0, 0, None, 0, *m.key_splits(b, H, R), 0)
            ov = m.batched_linear(oa, self.w_uv, H)                        # [T, H * vdim]
        m.linear(ov, self.w_o, out=x, accumulate=accumulate)

    MATRIX_TO_VECTOR_RATE = 6.0   # products on the matrix cores against attention arithmetic on the vector ALU, per operation

    def expands(self, b: RaggedBatch) -> bool:
        """Whether this step materialises keys and values.  Reading latent rows directly costs 2 kv_rank multiply-adds per (query, key) pair and head, expanded ones dim + vdim
        plus the expansion of every context row (kv_rank (dim + vdim) per head, on the matrix cores).  With about rows / 2 queries per context row the expansion pays from
        rows > 2 kv_rank (dim + vdim) / (rate (2 kv_rank - dim - vdim)) on; steps of single rows never expand."""
        s = self.s
        gain = 2 * s.kv_rank - s.dim - s.vdim
        if b.seg_rows <= 1 or b.host_blocks is None or gain <= 0 or (self.m.block_size * s.kv_rank * self.c_cache.element_size()) % 4:
            return False
        return b.rows * self.MATRIX_TO_VECTOR_RATE * gain > 2 * s.kv_rank * (s.dim + s.vdim)


class GluFeedForward(_Module):
    """down(silu(gate h) * (up h)), no biases; gate | up are one product."""

    def __init__(self, model, spec: GluSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix

    def load(self, get):
        s, p, W = self.s, self.p, self.m.spec.width
        g, u = get(p + "gate"), get(p + "up")
        self.w_down = self.w(get, p + "down", True)
        if tuple(g.shape) != (s.ff, W) or tuple(u.shape) != (s.ff, W) or tuple(self.w_down.shape) != (W, s.ff):
            raise ValueError(f"{p}: projection shapes do not match the layer's sizes")
        self.w_gu = torch.cat([g, u], 0).to(self.m.device, self.m.torch_dtype).contiguous()

    def forward(self, h, h32, x, b: RaggedBatch, accumulate: bool = True):
        s, m = self.s, self.m
        T = b.rows
        gu = m.linear(h, self.w_gu)
        if T <= m.GEMV_ROWS:   # decode-sized steps: the GLU in the down product's operand load
            _call("mrs_hyb_gemv", gu, self.w_down, x, T, x.shape[1], s.ff, 2 * s.ff, s.ff, x.stride(0), m.dt, int(accumulate), None, 0, 1, None, None, 1)
            return
        a = torch.empty(T, s.ff, dtype=m.torch_dtype, device=m.device)
        _call("mrs_hyb_glu_silu", gu, a, T, s.ff, m.dt)
        m.linear(a, self.w_down, out=x, accumulate=accumulate)


class DeltaRuleMixer(_Module):
    """q, k (kv_heads x dim), v (heads x vdim), the write strengths and the first steps of the decay / gate projections are ONE product; q, k, v pass a short causal
    convolution + SiLU (taps carried per slot); q and k become unit vectors per head (q times dim^(-1/2)); beta = sigmoid; g = exp(-exp(A_log_h) softplus(a + dt_bias)) per
    head or per (head, key channel).  Per head the f32 state S [dim, vdim] (carried per slot): S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.
    o / rms(o) per head times the weight `norm` [vdim] times the gate, then the output projection.  Head h reads q / k head h // (heads / kv_heads)."""

    CHAIN_WAVES = int(os.environ.get("MRS_DELTA_CHAIN_WAVES", "256"))   # entries x heads x (value size / 16) below this: long portions run their segments in parallel
    LANES = int(os.environ.get("MRS_DELTA_LANES", "0"))                 # lanes per state column (4 | 16); 0: the launcher chooses
    SEGMENT = int(os.environ.get("MRS_DELTA_SEGMENT", "128"))           # rows per segment of that form: the carry between segments costs dim^2 vdim per segment

    def __init__(self, model, spec: DeltaRuleSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix
        if spec.heads % spec.kv_heads or spec.decay not in ("head", "channel") or spec.gate not in ("silu", "sigmoid_lowrank") or spec.conv < 1:
            raise ValueError(f"{prefix}: heads % kv_heads must be 0; decay head | channel; gate silu | sigmoid_lowrank; at least one tap")
        dev = model.device
        self.nqk, self.nv = spec.kv_heads * spec.dim, spec.heads * spec.vdim
        self.channels = 2 * self.nqk + self.nv
        self.per = spec.dim if spec.decay == "channel" else 1
        self.conv_state = torch.zeros(model.state_slots, self.channels, max(spec.conv - 1, 1), dtype=torch.float32, device=dev)
        self.state = torch.zeros(model.state_slots, spec.heads, spec.dim, spec.vdim, dtype=torch.float32, device=dev)

    def carried(self):
        return (self.conv_state, self.state)

    def state_bytes_per_slot(self) -> int:
        return 4 * (self.conv_state[0].numel() + self.state[0].numel())

    def load(self, get):
        s, p, W = self.s, self.p, self.m.spec.width
        dev, dt = self.m.device, self.m.torch_dtype
        lowrank_a, lowrank_g = s.decay == "channel", s.gate == "sigmoid_lowrank"
        parts = [get(p + n) for n in ("q", "k", "v", "b", "a1" if lowrank_a else "a", "g1" if lowrank_g else "g")]
        ndec = s.heads * self.per
        self.rank_a = parts[4].shape[0] if lowrank_a else 0
        self.rank_g = parts[5].shape[0] if lowrank_g else 0
        want = [self.nqk, self.nqk, self.nv, s.heads, self.rank_a or ndec, self.rank_g or self.nv]
        if [t.shape[0] for t in parts] != want or any(t.shape[1] != W for t in parts):
            raise ValueError(f"{p}: projection shapes do not match the mixer's sizes")
        self.w_in = torch.cat(parts, 0).to(dev, dt).contiguous()            # [q | k | v | beta | a (a1) | g (g1), W]
        self.b_col = self.channels
        self.a_col = self.b_col + s.heads
        self.g_col = self.a_col + want[4]
        self.w_a2 = self.w(get, p + "a2", True) if lowrank_a else None
        self.w_g2 = self.w(get, p + "g2", True) if lowrank_g else None
        self.w_ag2 = None
        if lowrank_a and lowrank_g:   # both second steps as ONE product on the adjacent first steps: a block-diagonal weight (the zeros add nothing, exactly)
            self.w_ag2 = torch.zeros(ndec + self.nv, self.rank_a + self.rank_g, dtype=dt, device=dev)
            self.w_ag2[:ndec, :self.rank_a], self.w_ag2[ndec:, self.rank_a:] = self.w_a2, self.w_g2
        self.conv_w = torch.cat([get(p + n + ".conv") for n in ("q", "k", "v")], 0).to(dev, torch.float32).contiguous()   # [channels, taps]
        self.A_log, self.dt_bias, self.norm = (self.w(get, p + n, False).reshape(-1) for n in ("A_log", "dt_bias", "norm"))
        self.w_o = self.w(get, p + "o", True)
        if tuple(self.conv_w.shape) != (self.channels, s.conv) or self.A_log.numel() != s.heads or self.dt_bias.numel() != ndec or self.norm.numel() != s.vdim or \
                tuple(self.w_o.shape) != (W, self.nv) or (lowrank_a and tuple(self.w_a2.shape) != (ndec, self.rank_a)) or \
                (lowrank_g and tuple(self.w_g2.shape) != (self.nv, self.rank_g)):
            raise ValueError(f"{p}: convolution / decay / gate / output shapes do not match the mixer's sizes")

    def forward(self, h, x, b: RaggedBatch, accumulate: bool = True):
        s, m = self.s, self.m
        T, dev = b.rows, m.device
        f32 = dict(dtype=torch.float32, device=dev)
        u = m.linear(h, self.w_in)                                          # f32 [T, q | k | v | beta | a | g]
        c = torch.empty(T, self.channels, **f32)
        a, gate = u[:, self.a_col:], u[:, self.g_col:]
        if self.w_ag2 is not None:
            ag = m.linear(m.round_cols(a, self.rank_a + self.rank_g), self.w_ag2)   # the second steps of decay and gate: one product on the rounded first steps
            a, gate = ag, ag[:, self.w_a2.shape[0]:]
        else:
            if self.w_a2 is not None:
                a = m.linear(m.round_cols(a, self.rank_a), self.w_a2)
            if self.w_g2 is not None:
                gate = m.linear(m.round_cols(gate, self.rank_g), self.w_g2)
        beta = torch.empty(T, s.heads, **f32)
        dec = torch.empty(T, s.heads * self.per, **f32)
        if T == b.entries and b.seg_rows == 1:   # every entry brings one row: convolution, tap shift and the operands in one launch
            _call("mrs_hyb_delta_step_prep", u, u.stride(0), self.conv_w, self.conv_state, c, c.stride(0), self.channels, s.conv, self.b_col, a, a.stride(0), self.A_log,
                  self.dt_bias, beta, dec, b.seq_start, b.seq_pos0, b.seq_slot, T, b.entries, s.heads, s.kv_heads, s.dim, self.per)
        else:
            _call("mrs_hyb_conv", u, u.stride(0), None, self.conv_w, None, self.conv_state, b.tok_seq, b.seq_start, b.seq_pos0, b.seq_slot, c, T, b.entries, self.channels,
                  s.conv, 1)
            _call("mrs_hyb_delta_prep", c, c.stride(0), u, u.stride(0), self.b_col, a, a.stride(0), self.A_log, self.dt_bias, beta, dec, T, s.heads, s.kv_heads, s.dim, self.per)
        y = torch.empty(T, self.nv, **f32)
        table, nseg, carry, trans = b.entry_table(), b.entries, None, None      # every entry one chain: entries x heads x columns fill the chip, or all are short
        if b.seg_rows > 1 and b.entries * s.heads * -(-s.vdim // 16) < self.CHAIN_WAVES:
            # long portions in a step that would leave most of the chip idle: their segments side by side (end states from zero and transitions, a carry, then the outputs)
            *cut, n = b.segment_table(self.SEGMENT)
            if n > b.entries:
                table, nseg = cut, n
                carry = torch.empty(nseg, s.heads, s.dim, s.vdim, **f32)
                trans = torch.empty(nseg, s.heads, s.dim, s.dim, **f32)
        _call("mrs_hyb_delta_scan", c, c.stride(0), beta, dec, self.state, y, b.seq_pos0, b.seq_slot, *table, carry, trans, T, b.entries, nseg, s.heads, s.kv_heads, s.dim,
              s.vdim, self.per, self.LANES)
        o = torch.empty(T, self.nv, dtype=m.torch_dtype, device=dev)
        _call("mrs_hyb_head_norm_gate", y, s.vdim, None, self.norm, 0, gate, gate.stride(0), 1 if self.w_g2 is not None else 2, o, T, s.heads, s.vdim, m.spec.eps, m.dt)
        m.linear(o, self.w_o, out=x, accumulate=accumulate)


class MlstmMixer(_Module):
    """v | k | q | gate | input-gate | forget-gate logits in one product; q times dim^(-1/2) (as the scan reads it); log gates i = cap tanh((.. + b) / cap), f = logsigmoid(cap tanh((.. + b) /
    cap)); with the running maximum m' = max(f + m, i) (m starts at 0): S <- e^{f + m - m'} S + e^{i - m'} k v^T, n likewise with k alone, o = S^T q / (max(|n . q|,
    e^{-m'}) + 1e-6).  n rides as one more column of the state (a value that is always 1), so the recurrence is the gated scan of the state-space mixers with step values
    from the gates: portions run their segments in parallel.  o / rms(o) per head, times `norm` [heads * vdim], times sigmoid(gate), output projection.  Carries S | n
    [heads, dim, vdim + 1] and m [heads] per slot, f32."""

    def __init__(self, model, spec: MlstmSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix
        dev = model.device
        self.state = torch.zeros(model.state_slots, spec.heads, spec.dim, spec.vdim + 1, dtype=torch.float32, device=dev)
        self.m_state = torch.zeros(model.state_slots, spec.heads, dtype=torch.float32, device=dev)
        self.q_mult = float(np.float32(spec.dim) ** np.float32(-0.5))

    def carried(self):
        return (self.state, self.m_state)

    def state_bytes_per_slot(self) -> int:
        return 4 * (self.state[0].numel() + self.m_state[0].numel())

    def load(self, get):
        s, p, W = self.s, self.p, self.m.spec.width
        parts = [get(p + n) for n in ("v", "k", "q", "g", "i", "f")]
        nv, nk = s.heads * s.vdim, s.heads * s.dim
        want = [nv, nk, nk, nv, s.heads, s.heads]
        if [t.shape[0] for t in parts] != want or any(t.shape[1] != W for t in parts):
            raise ValueError(f"{p}: projection shapes do not match the mixer's sizes")
        self.w_in = torch.cat(parts, 0).to(self.m.device, self.m.torch_dtype).contiguous()     # [v | k | q | gate | i | f, W]
        self.q_col, self.g_col, self.i_col, self.f_col = nv + nk, nv + 2 * nk, 2 * nv + 2 * nk, 2 * nv + 2 * nk + s.heads
        self.bi, self.bf, self.norm = (self.w(get, p + n, False).reshape(-1) for n in ("i.b", "f.b", "norm"))
        self.w_o = self.w(get, p + "o", True)
        if self.bi.numel() != s.heads or self.bf.numel() != s.heads or self.norm.numel() != nv or tuple(self.w_o.shape) != (W, nv):
            raise ValueError(f"{p}: gate bias / norm / output shapes do not match the mixer's sizes")

    def forward(self, h, x, b: RaggedBatch, accumulate: bool = True):
        s, m = self.s, self.m
        T, dev = b.rows, m.device
        f32 = dict(dtype=torch.float32, device=dev)
        u = m.linear(h, self.w_in)                                          # f32 [T, v | k | q | gate | i | f]
        steps = torch.empty(T, s.heads, 2, **f32)
        mbuf, mexp = torch.empty(T + b.entries, s.heads, **f32), torch.empty(T, s.heads, **f32)
        _call("mrs_hyb_exp_gates", u, u.stride(0), self.i_col, self.f_col, self.bi, self.bf, s.gate_cap, self.m_state, steps, mbuf, mexp, b.tok_seq, b.seq_start, b.seq_pos0,
              b.seq_slot, T, b.entries, s.heads)
        P = s.vdim + 1
        y = torch.empty(T, s.heads * P, **f32)
        carry = decay = None
        if b.segments > b.entries:   # some portion is longer than a segment: scratch for the segments' local end states
            carry = torch.empty(b.segments, s.heads, s.dim, P, **f32)
            decay = torch.empty(b.segments, s.heads, **f32)
        _call("mrs_hyb_gated_scan", u, u.stride(0), steps, self.state, y, b.seq_pos0, b.seq_slot, b.seg_entry, b.seg_row0, b.seg_len, b.ent_seg0, carry, decay, T, b.entries,
              b.segments, s.heads, s.vdim, s.dim, s.heads, 1, self.q_mult)
        o = torch.empty(T, s.heads * s.vdim, dtype=m.torch_dtype, device=dev)
        _call("mrs_hyb_head_norm_gate", y, P, mexp, self.norm, 1, u[:, self.g_col:], u.stride(0), 1, o, T, s.heads, s.vdim, m.spec.eps, m.dt)
        m.linear(o, self.w_o, out=x, accumulate=accumulate)


class ParallelMixer(_Module):
    """Two registered mixers (tensors under `left.` / `right.`) read the same input; result = (left / rms(left) * w_left + right / rms(right) * w_right) / 2, the norms over
    the model width with plain weights `left.out` / `right.out`.  Pages, taps and states are the sub-mixers' own."""

    def __init__(self, model, spec: ParallelSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix
        self.left = MIXERS[spec.left_kind](model, spec.left, prefix + "left.")
        self.right = MIXERS[spec.right_kind](model, spec.right, prefix + "right.")

    def carried(self):
        return tuple(self.left.carried()) + tuple(self.right.carried())

    def kv_bytes_per_token(self) -> int:
        return sum(c.kv_bytes_per_token() for c in (self.left, self.right) if hasattr(c, "kv_bytes_per_token"))

    def state_bytes_per_slot(self) -> int:
        return sum(c.state_bytes_per_slot() for c in (self.left, self.right) if hasattr(c, "state_bytes_per_slot"))

    def load(self, get):
        self.left.load(get)
        self.right.load(get)
        self.w_left, self.w_right = self.w(get, self.p + "left.out", False), self.w(get, self.p + "right.out", False)
        if self.w_left.numel() != self.m.spec.width or self.w_right.numel() != self.m.spec.width:
            raise ValueError(f"{self.p}: the output norms run over the model width")

    def share_from(self, other: "ParallelMixer") -> None:
        self.left.share_from(other.left)
        self.right.share_from(other.right)
        self.w_left, self.w_right = other.w_left, other.w_right

    def forward(self, h, x, b: RaggedBatch, accumulate: bool = True):
        m = self.m
        yl = torch.empty(b.rows, m.spec.width, dtype=torch.float32, device=m.device)
        yr = torch.empty_like(yl)
        self.left.forward(h, yl, b, accumulate=False)
        self.right.forward(h, yr, b, accumulate=False)
        _call("mrs_hyb_norm_pair_add", x, x.stride(0), yl, self.w_left, yr, self.w_right, b.rows, m.spec.width, m.spec.eps, 0.5, int(accumulate))


class TopkSoftmaxReluSqMoe(_Module):
    """Router logits (weight and bias) in f32; the `top` largest are chosen, their weights are the softmax over the chosen logits only, applied to the experts' OUTPUTS.
    Expert (no biases, no gate): down(max(up h, 0)^2).  All experts of a step run as grouped products over expert-sorted rows."""
    wants_f32_input = True

    def __init__(self, model, spec: TopkSoftmaxMoeSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix

    def load(self, get):
        s, p, m = self.s, self.p, self.m
        dev, dt = m.device, m.torch_dtype
        self.w_up = torch.stack([get(f"{p}e{e}.up") for e in range(s.experts)]).to(dev, dt).contiguous()       # [E, ff, W]
        self.w_down = torch.stack([get(f"{p}e{e}.down") for e in range(s.experts)]).to(dev, dt).contiguous()   # [E, W, ff]
        self.w_router, self.b_router = self.w(get, p + "router", False), self.w(get, p + "router.b", False).reshape(-1)
        if tuple(self.w_up.shape[1:]) != (s.ff, m.spec.width) or tuple(self.w_down.shape[1:]) != (m.spec.width, s.ff) or \
                tuple(self.w_router.shape) != (s.experts, m.spec.width) or self.b_router.numel() != s.experts:
            raise ValueError(f"{p}: expert / router shapes do not match the layer's sizes")

    def forward(self, h, h32, x, b: RaggedBatch, accumulate: bool = True):
        s, m = self.s, self.m
        T, W, dev = b.rows, m.spec.width, m.device
        R = T * s.top
        ids = torch.empty(R, dtype=torch.int32, device=dev)
        wts = torch.empty(R, dtype=torch.float32, device=dev)
        _call("mrs_hyb_route_topk_softmax", h32, self.w_router, self.b_router, T, W, s.experts, s.top, 1.0, ids, wts)
        meta = torch.empty(s.experts + 1 + 3 * R, dtype=torch.int32, device=dev)
        bounds, sorted_route, route_pos, sorted_expert = meta[:s.experts + 1], meta[s.experts + 1:][:R], meta[s.experts + 1 + R:][:R], meta[s.experts + 1 + 2 * R:][:R]
        _call("mrs_hyb_moe_dispatch", ids, R, s.experts, bounds, sorted_route, route_pos, sorted_expert)
        f32 = dict(dtype=torch.float32, device=dev)
        if R <= m.GROUPED_GEMV_ROWS:
            # decode-sized steps: every route streams its expert's slabs; the row gather and the squared ReLU happen in the consuming product's operand load (same roundings)
            up = torch.empty(R, s.ff, **f32)
            m.gemv_act(h32, self.w_up, up, R, s.ff, W, h32.stride(0), W, sorted_expert, self.w_up.stride(0), 2, sorted_route, s.top)
            d = torch.empty(R, W, **f32)
            m.gemv_act(up, self.w_down, d, R, W, s.ff, s.ff, s.ff, sorted_expert, self.w_down.stride(0), 5)
        else:
            xs = torch.empty(R, W, dtype=m.torch_dtype, device=dev)
            _call("mrs_hyb_moe_gather", h32, sorted_route, None, s.top, xs, R, W, m.dt)
            up = m.grouped_linear(xs, self.w_up, bounds, sorted_expert)
            act = torch.empty(R, s.ff, dtype=m.torch_dtype, device=dev)
            _call("mrs_hyb_relu_sq", up, act, R, s.ff, m.dt)
            d = m.grouped_linear(act, self.w_down, bounds, sorted_expert)
        _call("mrs_hyb_moe_combine_weighted", x, d, route_pos, wts, s.top, None, T, W, int(accumulate))


MIXERS: Dict[str, Callable] = {"delta_rule": DeltaRuleMixer, "mlstm": MlstmMixer, "parallel": ParallelMixer, "mamba2": Mamba2Mixer, "attention": WindowAttention, "talk_attention": TalkSigmoidAttention, "sink_attention": GatedSinkAttention,
                               "retention": RetentionMixer, "latent_attention": LatentAttention}
FEED_FORWARDS: Dict[str, Callable] = {"moe_topk_softmax_relu2": TopkSoftmaxReluSqMoe, "moe": SigmoidMoe, "moe_softmax_clamped": ClampedSoftmaxMoe, "dense_xielu": XieluFeedForward, "dense_glu_silu": GluFeedForward}


class _Layer:
    def __init__(self, model, ls: LayerSpec):
        self.spec = ls
        self.mixer = MIXERS[ls.kind](model, ls.mixer, ls.prefix + "mix.")
        self.ff = FEED_FORWARDS[ls.ff.kind](model, ls.ff, ls.prefix + "mlp.") if ls.ff else None
        self.norm1 = self.norm2 = self.norm1b = self.norm2b = None   # (weight, bias | None)
        self.hc1 = self.hc2 = None   # several residual streams: (in [S], out [S] times the residual multiplier, mix [S, S]) of the sublayer, f32


# ------------------------------------------------------------------------------------------------------------------ the model
class HybridDecoder:
    """`num_blocks` K / V pages of `block_size` tokens per attention layer and `state_slots` recurrent-state slots per state-space layer; which sequence uses which is
    the cache managers' business (KVCacheManager / StateSlotPool), the model only follows the tables in the batch."""

    GEMV_ROWS = 8          # at most this many rows share one streamed weight pass
    GROUPED_GEMV_ROWS = 32 # expert-sorted rows up to which every row streams its own expert slab

    def __init__(self, spec: HybridSpec, device, dtype: str = "bfloat16", num_blocks: int = 64, block_size: int = 32, state_slots: int = 4):
        if dtype not in DTYPES:
            raise ValueError(f"dtype must be one of {sorted(DTYPES)}")
        _lib.load("hybrid")
        self.spec, self.device, self.dtype = spec, torch.device(device), dtype
        self.dt, self.torch_dtype = DTYPES[dtype]
        self.num_blocks, self.block_size, self.state_slots = int(num_blocks), int(block_size), int(state_slots)
        self.layers = [_Layer(self, ls) for ls in spec.layers]
        self.trace_layers: Optional[list] = None   # set to a list: forward_batch appends the residual stream after every layer (debugging / tests)

    # ---- construction
    @property
    def has_recurrent_state(self) -> bool:
        return self.state_bytes_per_slot() > 0

    @property
    def has_paged_kv(self) -> bool:
        return self.kv_bytes_per_token() > 0

    def load_weights(self, get: Callable[[str], torch.Tensor]) -> None:
        sp = self.spec
        f32 = lambda n: get(n).to(self.device, torch.float32).contiguous()
        self.embed = get(sp.embed).to(self.device, self.torch_dtype).contiguous()
        self.head = self.embed if sp.head == sp.embed else get(sp.head).to(self.device, self.torch_dtype).contiguous()   # a head tied to the embedding is the same tensor
        norm = lambda n: (f32(n), f32(n + ".b") if sp.norm == "layer" else None)
        self.final_norm = norm(sp.final_norm)
        if tuple(self.embed.shape) != (sp.vocab, sp.width) or tuple(self.head.shape) != (sp.vocab, sp.width):
            raise ValueError("embedding / head shapes do not match vocab x width")
        self.embed_norm = norm(sp.embed_norm) if sp.embed_norm else None
        S = max(1, sp.streams)
        self.ones = torch.ones(S, dtype=torch.float32, device=self.device)

        def hyper(prefix):
            """(in, residual_mult * out, mix) of a sublayer; one plain stream: (1, residual_mult, 1)"""
            if not sp.streams:
                return self.ones, torch.full((1,), sp.residual_mult, dtype=torch.float32, device=self.device), self.ones.view(1, 1)
            w_in, w_out, mix = f32(prefix + ".in").reshape(-1), f32(prefix + ".out").reshape(-1), f32(prefix + ".mix")
            if w_in.numel() != S or w_out.numel() != S or tuple(mix.shape) != (S, S):
                raise ValueError(f"{prefix}: stream weights do not match the number of streams")
            return w_in, (w_out * np.float32(sp.residual_mult)).contiguous(), mix
        self.multi_stream = bool(sp.streams) or sp.residual_mult != 1.0
        for l in self.layers:
            if l.spec.weights_of is not None:
                continue
            if self.multi_stream:
                l.hc1 = hyper(l.spec.prefix + "hc1")
                l.hc2 = hyper(l.spec.prefix + "hc2") if l.ff else None
            l.norm1 = norm(l.spec.prefix + "norm1")
            l.norm1b = norm(l.spec.prefix + "norm1b") if sp.post_norms else None
            l.mixer.load(get)
            if l.ff:
                l.norm2 = norm(l.spec.prefix + "norm2")
                l.norm2b = norm(l.spec.prefix + "norm2b") if sp.post_norms else None
                l.ff.load(get)
        for l in self.layers:   # layers that use another layer's tensors: the same norms and feed-forward, the same mixer weights around pages / taps / states of their own
            if l.spec.weights_of is not None:
                o = self.layers[l.spec.weights_of]
                l.norm1, l.norm2, l.norm1b, l.norm2b, l.hc1, l.hc2, l.ff = o.norm1, o.norm2, o.norm1b, o.norm2b, o.hc1, o.hc2, o.ff
                l.mixer.share_from(o.mixer)

    @classmethod
    def from_pretrained(cls, path: str, device, dtype: str = "bfloat16", **kw) -> "HybridDecoder":
        """`path`: a folder with config.json and model.safetensors."""
        from safetensors import safe_open
        with open(os.path.join(path, "config.json")) as f:
            cfg = json.load(f)
        model = cls(SPEC_READERS[cfg["architecture"]](cfg), device, dtype, **kw)
        with safe_open(os.path.join(path, "model.safetensors"), "pt") as st:
            model.load_weights(st.get_tensor)
        return model

    # ---- building blocks on the current stream
    def norm(self, x, w, one_plus: bool, parts: int = 1, want32: bool = False, gate=None, gate_after: bool = False):
        """RMS norm of every row (in `parts` equal pieces; w None: no weight); gate [rows, >= width]: the row is multiplied by silu(gate) first, or (gate_after) the
        normed row is."""
        rows, width = x.shape
        out = torch.empty(rows, width, dtype=self.torch_dtype, device=self.device)
        out32 = torch.empty(rows, width, dtype=torch.float32, device=self.device) if want32 else None
        _call("mrs_hyb_rmsnorm", x, x.stride(0), w, out, out32, None, rows, width, parts, self.spec.eps, int(one_plus), self.dt, gate, gate.stride(0) if gate is not None else 0,
              int(gate_after))
        return (out, out32) if want32 else out

    def hyper_step(self, x, y, write, read, norm_w, want32: bool = False):
        """One launch between two sublayers of a design with residual streams x [rows, S, W]: `write` = (_, out, mix) of the sublayer that made y (mix None: the streams
        start as out[r] * y), `read` = the in-weights of the next reader, `norm_w` its one-plus norm weight (None: the read sum itself comes back in f32)."""
        rows, S, W = x.shape
        out = torch.empty(rows, W, dtype=self.torch_dtype, device=self.device) if norm_w is not None else None
        out32 = torch.empty(rows, W, dtype=torch.float32, device=self.device) if (want32 or norm_w is None) else None
        _call("mrs_hyb_hyper_step", x, y, write[2] if y is not None else None, write[1] if y is not None else None, read, norm_w, out, out32, rows, S, W, self.spec.eps, 1, self.dt)
        if norm_w is None:
            return out32
        return (out, out32) if want32 else out

    KEY_SPLIT_ROWS = 128   # steps of single rows up to this many rows split their keys
    KEYS_PER_SPLIT = 256   # at least this many keys (of the longest table in the batch) per workgroup
    KEY_SPLITS = 32

    def key_splits(self, b: RaggedBatch, heads: int, vdim: int, most_keys: int = 0):
        """(scratch, splits) for an attention launch over unwindowed keys: a step in which every entry brings one row deals each row's keys to several workgroups
        (one wave walking thousands of keys is latency-bound); (None, 0) otherwise.  most_keys > 0: no row reads more keys than that (a chunk, a window)."""
        if b.seg_rows != 1 or b.rows > self.KEY_SPLIT_ROWS:
            return None, 0
        keys = b.max_blocks * self.block_size
        splits = min(self.KEY_SPLITS, (min(keys, most_keys) if most_keys > 0 else keys) // self.KEYS_PER_SPLIT)
        if splits < 2:
            return None, 0
        return torch.empty(splits, b.rows, heads, vdim + 2, dtype=torch.float32, device=self.device), splits

    def linear_rounded(self, a, w):
        """a [M, K] . w [N, K]^T -> [M, N] in the serving dtype, rounded once: a product whose consumer is another product or the attention kernel."""
        M, K = a.shape
        out = torch.empty(M, w.shape[0], dtype=self.torch_dtype, device=self.device)
        _call("mrs_hyb_gemm_batched", a, w, out, M, w.shape[0], K, a.stride(0), w.stride(0), out.stride(0), self.dt, 0, 0, 0, 0, 1)
        return out

    def batched_linear(self, a, w, heads: int):
        """a [M, heads * K] (column block h = the operand of head h), w [heads, N, K] -> [M, heads * N] in the serving dtype, rounded once: per-head products whose
        consumer is another product or the attention kernel."""
        M = a.shape[0]
        _, N, K = w.shape
        out = torch.empty(M, heads * N, dtype=self.torch_dtype, device=self.device)
        _call("mrs_hyb_gemm_batched", a, w, out, M, N, K, a.stride(0), K, out.stride(0), self.dt, heads, K, N * K, N, 1)
        return out

    def layer_norm(self, x, wb, want32: bool = False):
        """(x - mean) / sqrt(var + eps) * w + b of every row, in the serving dtype (and in f32 with want32)."""
        rows, width = x.shape
        out = torch.empty(rows, width, dtype=self.torch_dtype, device=self.device)
        out32 = torch.empty(rows, width, dtype=torch.float32, device=self.device) if want32 else None
        _call("mrs_hyb_layernorm", x, x.stride(0), None, wb[0], wb[1], out, out32, None, 0, rows, width, self.spec.eps, self.dt)
        return (out, out32) if want32 else out

    def pre_norm(self, x, wb, want32: bool = False):
        """The norm in front of a sublayer (and of the head), of the kind the model's description names."""
        if self.spec.norm == "layer":
            return self.layer_norm(x, wb, want32)
        return self.norm(x, wb[0], one_plus=self.spec.norm == "rms_one_plus", want32=want32)

    def pre_norm_pair(self, x, wb1, wb2, want32: bool = False):
        """The norms in front of two sublayers that read the same rows: one pass, one root mean square, two weights.  Returns (first, second, second in f32 | None)."""
        if self.spec.norm == "layer":
            return (self.layer_norm(x, wb1),) + tuple(self.layer_norm(x, wb2, True) if want32 else (self.layer_norm(x, wb2), None))
        rows, width = x.shape
        o1 = torch.empty(rows, width, dtype=self.torch_dtype, device=self.device)
        o2 = torch.empty_like(o1)
        o32 = torch.empty(rows, width, dtype=torch.float32, device=self.device) if want32 else None
        _call("mrs_hyb_rmsnorm_pair", x, x.stride(0), wb1[0], wb2[0], o1, o2, o32, rows, width, self.spec.eps, int(self.spec.norm == "rms_one_plus"), self.dt)
        return o1, o2, o32

    def round_cols(self, u, n: int):
        """The first n columns of the f32 rows u, rounded once to the serving dtype and contiguous: a column block of one product as the operand of the next."""
        out = torch.empty(u.shape[0], n, dtype=self.torch_dtype, device=self.device)
        _call("mrs_hyb_round_cols", u, u.stride(0), out, u.shape[0], n, self.dt)
        return out

    def add_post_norm(self, x, y, in_bias, wb, then=None, want32: bool = False):
        """x += norm(y + in_bias): a sublayer's product (its bias still to be added) joins the f32 residual stream through the norm behind the sublayer.  `then` = the
        (weight, bias) of the norm in front of the next sublayer: the same launch norms the updated rows with it and returns them like `pre_norm`."""
        if self.spec.norm != "layer":
            raise NotImplementedError("norms behind a sublayer exist as layer norms only")
        rows, width = y.shape
        if then is None:
            _call("mrs_hyb_layernorm", y, y.stride(0), in_bias, wb[0], wb[1], None, None, x, x.stride(0), rows, width, self.spec.eps, self.dt)
            return None
        out = torch.empty(rows, width, dtype=self.torch_dtype, device=self.device)
        out32 = torch.empty(rows, width, dtype=torch.float32, device=self.device) if want32 else None
        _call("mrs_hyb_layernorm_pair", y, y.stride(0), in_bias, wb[0], wb[1], x, x.stride(0), then[0], then[1], out, out32, rows, width, self.spec.eps, self.dt)
        return (out, out32) if want32 else out

    def gemv_act(self, a, w, out, M, N, K, lda, ldw, row_group, wstride, in_mode, src_row=None, src_div=1, bias=None, p0=0.0, p1=0.0, accumulate=False, src_scale=None):
        """out [M, N] (+)= act(a) . w^T for at most GEMV_ROWS rows (or one weight slab per row with `row_group`), the activation evaluated in the operand load.  in_mode:
        0 plain, 1 silu(gate) * up of a = f32 [gate | up], 2 gathered (and scaled) f32 source rows, 3 clamped GLU of a = f32 [gate | up] (p0 = limit, p1 = the sigmoid's
        factor), 4 xIELU(a + bias) (p0, p1 = its two coefficients)."""
        _call("mrs_hyb_gemv_act", a, w, out, M, N, K, lda, ldw, out.stride(0), self.dt, int(accumulate), row_group, wstride, in_mode, src_row, src_scale, src_div, bias, p0, p1)

    def linear(self, a, w, out=None, accumulate: bool = False, dtype_code: Optional[int] = None):
        """out (f32 [M, N]) (+)= a [M, K] . w [N, K]^T"""
        M, K = a.shape
        N = w.shape[0]
        if out is None:
            out = torch.empty(M, N, dtype=torch.float32, device=self.device)
        dt = dtype_code or self.dt
        if M <= self.GEMV_ROWS:
            _call("mrs_hyb_gemv", a, w, out, M, N, K, a.stride(0), w.stride(0), out.stride(0), dt, int(accumulate), None, 0, 0, None, None, 1)
        else:
            _call("mrs_hyb_gemm", a, w, out, M, N, K, a.stride(0), w.stride(0), out.stride(0), dt, int(accumulate), None, 0, 0, 0)
        return out

    def grouped_linear(self, a, w, bounds, sorted_expert):
        """a [R, K] rows sorted by group, w [groups, N, K]: row r multiplies the slab of its group."""
        R, K = a.shape
        E, N = w.shape[0], w.shape[1]
        out = torch.empty(R, N, dtype=torch.float32, device=self.device)
        if R <= self.GROUPED_GEMV_ROWS:
            _call("mrs_hyb_gemv", a, w, out, R, N, K, a.stride(0), w.stride(1), out.stride(0), self.dt, 0, sorted_expert, w.stride(0), 0, None, None, 1)
        else:
            _call("mrs_hyb_gemm", a, w, out, R, N, K, a.stride(0), w.stride(1), out.stride(0), self.dt, 0, bounds, E, w.stride(0), R)
        return out

    # ---- the step
    def forward_batch(self, b: RaggedBatch) -> torch.Tensor:
        """Runs the batch's rows from the cache and state that earlier steps left; returns f32 logits [len(want), vocab] in the order of `want`."""
        global _step_stream
        _step_stream = torch.cuda.current_stream().cuda_stream
        try:
            return self._forward_batch(b)
        finally:
            _step_stream = None

    def _forward_batch(self, b: RaggedBatch) -> torch.Tensor:
        sp = self.spec
        T = b.rows
        if T == 0:
            return torch.empty(0, sp.vocab, dtype=torch.float32, device=self.device)
        x = torch.empty(T, sp.width, dtype=torch.float32, device=self.device)
        _call("mrs_hyb_embed", b.tokens, self.embed, x, T, sp.width, sp.vocab, self.dt)
        if self.embed_norm is not None:
            e = torch.empty_like(x)
            if sp.norm == "layer":
                _call("mrs_hyb_layernorm", x, x.stride(0), None, self.embed_norm[0], self.embed_norm[1], None, e, None, 0, T, sp.width, sp.eps, self.dt)
            else:
                _call("mrs_hyb_rmsnorm", x, x.stride(0), self.embed_norm[0], None, e, None, T, sp.width, 1, sp.eps, 1, self.dt, None, 0, 0)
            x = e
        if self.multi_stream:
            return self._forward_streams(b, x)
        y = torch.empty_like(x) if sp.post_norms else None   # a sublayer's product on its way through the norm behind it
        h_next = None                                         # post-norm designs: the next sublayer's input, normed by the launch that closed the previous sublayer
        for li, l in enumerate(self.layers):
            if sp.post_norms:
                l.mixer.forward(h_next if h_next is not None else self.pre_norm(x, l.norm1), y, b, accumulate=False)
                nxt = self.layers[li + 1].norm1 if li + 1 < len(self.layers) else None
                if l.ff:
                    h, h32 = self.add_post_norm(x, y, l.mixer.out_bias, l.norm1b, then=l.norm2, want32=True)
                    l.ff.forward(h, h32, y, b, accumulate=False)
                    h_next = self.add_post_norm(x, y, l.ff.out_bias, l.norm2b, then=nxt)
                else:
                    h_next = self.add_post_norm(x, y, l.mixer.out_bias, l.norm1b, then=nxt)
            elif sp.parallel_sublayers and l.ff:
                h1, h2, h32 = self.pre_norm_pair(x, l.norm1, l.norm2, want32=l.ff.wants_f32_input)   # both sublayers read the row as it is now; their sums join it in turn
                l.mixer.forward(h1, x, b)
                l.ff.forward(h2, h32, x, b)
            else:
                l.mixer.forward(self.pre_norm(x, l.norm1), x, b)
                if l.ff:
                    h, h32 = self.pre_norm(x, l.norm2, want32=True)
                    l.ff.forward(h, h32, x, b)
            if self.trace_layers is not None:
                self.trace_layers.append(x.clone())
        n = b.want.numel()
        if n == 0:
            return torch.empty(0, sp.vocab, dtype=torch.float32, device=self.device)
        xs = torch.empty(n, sp.width, dtype=torch.float32, device=self.device)
        _call("mrs_hyb_gather_rows", x, b.want, xs, n, sp.width)
        return self.linear(self.pre_norm(xs, self.final_norm), self.head)

    def _forward_streams(self, b: RaggedBatch, e: torch.Tensor) -> torch.Tensor:
        """Designs with scaled sublayer outputs and / or several residual streams: x [rows, S, W] f32.  Every sublayer's product goes to a scratch block; the launch that
        writes it into the streams also reads and norms the input of the NEXT sublayer, so a sublayer costs one launch besides its own."""
        sp = self.spec
        if sp.post_norms or sp.norm != "rms_one_plus":
            raise NotImplementedError("residual streams are built for one-plus RMS norms in front of the sublayers")
        T, W, S = b.rows, sp.width, max(1, sp.streams)
        subs = []   # (layer, module, (in, out, mix), norm weight, last sublayer of its layer)
        for l in self.layers:
            subs.append((l, l.mixer, l.hc1, l.norm1[0], l.ff is None))
            if l.ff:
                subs.append((l, l.ff, l.hc2, l.norm2[0], True))
        x = torch.empty(T, S, W, dtype=torch.float32, device=self.device)
        y = torch.empty(T, W, dtype=torch.float32, device=self.device)
        h = self.hyper_step(x, e, (None, self.ones, None), subs[0][2][0], subs[0][3], want32=subs[0][1].wants_f32_input)
        total = None
        for k, (l, mod, hc, _, closes) in enumerate(subs):
            if mod is l.mixer:
                mod.forward(h, y, b, accumulate=False)
            else:
                h, h32 = h if isinstance(h, tuple) else (h, None)
                mod.forward(h, h32, y, b, accumulate=False)
            if k + 1 < len(subs):
                nxt = subs[k + 1]
                h = self.hyper_step(x, y, hc, nxt[2][0], nxt[3], want32=nxt[1].wants_f32_input)
            else:
                total = self.hyper_step(x, y, hc, self.ones, None)   # the sum of the streams
            if closes and self.trace_layers is not None:
                self.trace_layers.append(x.sum(1))
        n = b.want.numel()
        if n == 0:
            return torch.empty(0, sp.vocab, dtype=torch.float32, device=self.device)
        xs = torch.empty(n, W, dtype=torch.float32, device=self.device)
        _call("mrs_hyb_gather_rows", total, b.want, xs, n, W)
        return self.linear(self.pre_norm(xs, self.final_norm), self.head)

    # ---- decode steps as a HIP graph
    def capture_decode(self, entries: int, max_blocks: int) -> "DecodeGraph":
        """One decode step for `entries` sequences (one row each), captured into a HIP graph over static batch buffers: replays cost one launch instead of one per kernel."""
        return DecodeGraph(self, entries, max_blocks)

    # ---- sizes
    def kv_bytes_per_token(self) -> int:
        return sum(l.mixer.kv_bytes_per_token() for l in self.layers if hasattr(l.mixer, "kv_bytes_per_token"))

    def state_bytes_per_slot(self) -> int:
        return sum(l.mixer.state_bytes_per_slot() for l in self.layers if hasattr(l.mixer, "state_bytes_per_slot"))


class DecodeGraph:
    """A captured decode step (role of pipeline/cuda_graph.rs in the reference): the batch description lives in static device buffers that `replay` refreshes with two
    small host -> device copies; every kernel argument besides those buffers (row counts, table width) is fixed at capture.  Logits of all rows come back as a view of a
    static buffer: consume them before the next replay."""

    def __init__(self, model: HybridDecoder, entries: int, max_blocks: int):
        self.m, self.n, self.mb = model, int(entries), int(max_blocks)
        dev, n, mb = model.device, self.n, self.mb
        self._ints = torch.zeros(3 * n + (n + 1) + 2 * n + n * mb, dtype=torch.int32, device=dev)
        self._slots = torch.zeros(n, dtype=torch.int64, device=dev)
        v, o = [], 0
        for k in (n, n, n, n + 1, n, n, n * mb):
            v.append(self._ints[o:o + k])
            o += k
        rows = torch.arange(n + 1, dtype=torch.int32, device=dev)   # one row = one segment per entry
        self.batch = RaggedBatch(n, n, mb, v[0], v[1], v[2], v[3], v[4], v[5], v[6].view(n, mb), self._slots, rows[:n].clone(), n, rows[:n], rows[:n],
                                 torch.ones(n, dtype=torch.int32, device=dev), rows, 1)
        self._host = np.zeros(self._ints.numel(), dtype=np.int32)
        self._host[3 * n:3 * n + n + 1] = np.arange(n + 1)          # seq_start: one row per entry
        self._host[2 * n:3 * n] = 1                                  # positions >= 1 during warm-up: the slots' states are read, nothing is reset
        self._host[n:2 * n] = np.arange(n)                           # tok_seq
        self._ints.copy_(torch.from_numpy(self._host))
        # warm-up outside capture (lazy module loads).  It really runs -- on state slot 0 and page slot 0, which may belong to a live sequence: put both back afterwards
        keep = []
        for l in model.layers:
            keep += [(t, t[0].clone()) for t in l.mixer.carried()]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            model.forward_batch(self.batch)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        for t, saved in keep:
            t[0].copy_(saved)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits = model.forward_batch(self.batch)

    def replay(self, entries: Sequence[dict]) -> torch.Tensor:
        """entries as for RaggedBatch.build, one token each (`pos0` = the token's position)."""
        n, mb, h = self.n, self.mb, self._host
        if len(entries) != n:
            raise ValueError(f"DecodeGraph: captured for {n} sequences, got {len(entries)}")
        slots = np.zeros(n, dtype=np.int64)
        bt = h[3 * n + (n + 1) + 2 * n:].reshape(n, mb)
        bs = self.m.block_size
        for s, e in enumerate(entries):
            p, blocks = int(e["pos0"]), e["blocks"]
            if len(e["tokens"]) != 1 or len(blocks) > mb or p // bs >= len(blocks):
                raise ValueError("DecodeGraph: one token per entry, its page inside the captured table width")
            h[s], h[2 * n + s] = e["tokens"][0], p
            h[3 * n + (n + 1) + s], h[3 * n + (n + 1) + n + s] = p, int(e.get("slot") or 0)
            bt[s, :len(blocks)] = blocks
            slots[s] = blocks[p // bs] * bs + p % bs
        self._ints.copy_(torch.from_numpy(h))
        self._slots.copy_(torch.from_numpy(slots))
        self.graph.replay()
        return self.logits


def synthetic_weights(spec: HybridSpec, device, seed: int = 0) -> Callable[[str], torch.Tensor]:
    """`get(name)` for HybridDecoder.load_weights that draws every tensor on the device when it is asked for (benchmarks: there is no network for checkpoints).
    Projections N(0, 1 / fan_in), norm weights around their neutral value, decays and step sizes in the range trained state-space models use."""
    W = spec.width
    g = torch.Generator(device=device).manual_seed(seed)
    shapes: Dict[str, tuple] = {spec.embed: (spec.vocab, W), spec.head: (spec.vocab, W), spec.final_norm: (W,)}
    norm_names = {spec.final_norm} | ({spec.embed_norm} if spec.embed_norm else set())
    def new_mixer_shapes(p, m) -> bool:
        """delta-rule, matrix-memory, parallel and chunked / gated attention mixers; False: `m` is of another kind"""
        if isinstance(m, ParallelSpec):
            shapes.update({p + "left.out": (W,), p + "right.out": (W,)})
            norm_like.update({p + "left.out", p + "right.out"})
            for side, sub in (("left.", m.left), ("right.", m.right)):
                if not new_mixer_shapes(p + side, sub):
                    raise ValueError("synthetic_weights: a parallel mixer's sides are attention, delta-rule or matrix-memory mixers")
        elif isinstance(m, DeltaRuleSpec):
            nqk, nv, rank = m.kv_heads * m.dim, m.heads * m.vdim, max(8, min(128, W // 16))
            for n, rows in (("q", nqk), ("k", nqk), ("v", nv)):
                shapes.update({p + n: (rows, W), p + n + ".conv": (rows, m.conv)})
            shapes.update({p + "b": (m.heads, W), p + "A_log": (m.heads,), p + "norm": (m.vdim,), p + "o": (W, nv)})
            if m.decay == "channel":
                shapes.update({p + "a1": (rank, W), p + "a2": (m.heads * m.dim, rank), p + "dt_bias": (m.heads * m.dim,)})
            else:
                shapes.update({p + "a": (m.heads, W), p + "dt_bias": (m.heads,)})
            shapes.update({p + "g1": (rank, W), p + "g2": (nv, rank)} if m.gate == "sigmoid_lowrank" else {p + "g": (nv, W)})
        elif isinstance(m, MlstmSpec):
            nk, nv = m.heads * m.dim, m.heads * m.vdim
            shapes.update({p + "q": (nk, W), p + "k": (nk, W), p + "v": (nv, W), p + "g": (nv, W), p + "o": (W, nv), p + "norm": (nv,), p + "i": (m.heads, W), p + "i.b": (m.heads,),
                           p + "f": (m.heads, W), p + "f.b": (m.heads,)})
        elif isinstance(m, AttentionSpec) and (m.head_norm or m.sink or m.head_gate):
            shapes.update({p + "q": (m.heads * m.dim, W), p + "k": (m.kv_heads * m.dim, W), p + "v": (m.kv_heads * m.vdim, W), p + "o": (W, m.heads * m.vdim),
                           p + "q.norm": (m.dim if m.head_norm else m.heads * m.dim,), p + "k.norm": (m.dim if m.head_norm else m.kv_heads * m.dim,)})
            if m.sink:
                shapes[p + "sink"] = (m.heads,)
            if m.head_gate:
                shapes[p + "g"] = (m.heads, W)
        else:
            return False
        return True

    norm_like = set()   # plain-weight norms besides the layers' own: drawn around one
    for ls in spec.layers:
        p, m = ls.prefix, ls.mixer
        if ls.weights_of is not None:
            continue
        for n in ["norm1"] + (["norm2"] if ls.ff else []) + ((["norm1b"] + (["norm2b"] if ls.ff else [])) if spec.post_norms else []):
            norm_names.add(p + n)
        if spec.streams:
            for q in ("hc1", "hc2") if ls.ff else ("hc1",):
                shapes.update({f"{p}{q}.in": (spec.streams,), f"{p}{q}.out": (spec.streams,), f"{p}{q}.mix": (spec.streams, spec.streams)})
        if new_mixer_shapes(p + "mix.", m):
            pass
        elif isinstance(m, SinkAttentionSpec):
            own = ["q", "k", "v"] if m.kv_from is None else ["q"]
            rows = {"q": m.heads * m.dim, "k": m.kv_heads * m.dim, "v": m.kv_heads * m.vdim}
            for n in own:
                shapes.update({f"{p}mix.{n}": (rows[n], W), f"{p}mix.{n}.b": (rows[n],)})
                if m.conv:
                    shapes[f"{p}mix.{n}.conv"] = (rows[n], m.conv)
            shapes.update({p + "mix.g": (m.heads * m.vdim, W), p + "mix.o": (W, m.heads * m.vdim)})
        elif isinstance(m, RetentionSpec):
            shapes.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.k": (m.heads * m.dim, W), p + "mix.v": (m.heads * m.vdim, W), p + "mix.g": (m.heads * m.vdim, W),
                           p + "mix.o": (W, m.heads * m.vdim)})
        elif isinstance(m, LatentAttentionSpec):
            shapes.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.dkv": (m.kv_rank, W), p + "mix.dkv.norm": (m.kv_rank,), p + "mix.uk": (m.heads * m.dim, m.kv_rank),
                           p + "mix.uv": (m.heads * m.vdim, m.kv_rank), p + "mix.o": (W, m.heads * m.vdim)})
        elif isinstance(m, TalkAttentionSpec):
            shapes.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.q.b": (m.heads * m.dim,), p + "mix.g": (m.heads, W), p + "mix.talk": (m.heads, m.heads),
                           p + "mix.pb": (m.heads,), p + "mix.o": (W, m.heads * m.vdim), p + "mix.o.b": (W,)})
            if m.kv_from is None:
                shapes.update({p + "mix.k": (m.kv_heads * m.dim, W), p + "mix.k.b": (m.kv_heads * m.dim,), p + "mix.v": (m.kv_heads * m.vdim, W), p + "mix.v.b": (m.kv_heads * m.vdim,)})
        elif isinstance(m, Mamba2Spec):
            shapes.update({p + "mix.in": (2 * m.inner + 2 * m.groups * m.state + m.heads, W), p + "mix.conv": (m.conv_channels, m.conv), p + "mix.conv.b": (m.conv_channels,),
                           p + "mix.dt_bias": (m.heads,), p + "mix.A_log": (m.heads,), p + "mix.D": (m.heads,), p + "mix.norm": (m.inner,), p + "mix.o": (W, m.inner)})
        else:
            shapes.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.k": (m.kv_heads * m.dim, W), p + "mix.v": (m.kv_heads * m.vdim, W), p + "mix.q.norm": (m.heads * m.dim,),
                           p + "mix.k.norm": (m.kv_heads * m.dim,), p + "mix.o": (W, m.heads * m.vdim)})
        if isinstance(ls.ff, GluSpec):
            shapes.update({p + "mlp.gate": (ls.ff.ff, W), p + "mlp.up": (ls.ff.ff, W), p + "mlp.down": (W, ls.ff.ff)})
        elif isinstance(ls.ff, DenseSpec):
            shapes.update({p + "mlp.up": (ls.ff.ff, W), p + "mlp.up.b": (ls.ff.ff,), p + "mlp.down": (W, ls.ff.ff), p + "mlp.down.b": (W,), p + "mlp.act": (2,)})
        elif isinstance(ls.ff, TopkSoftmaxMoeSpec):
            shapes.update({p + "mlp.router": (ls.ff.experts, W), p + "mlp.router.b": (ls.ff.experts,)})
            for e in range(ls.ff.experts):
                shapes.update({f"{p}mlp.e{e}.up": (ls.ff.ff, W), f"{p}mlp.e{e}.down": (W, ls.ff.ff)})
        elif ls.ff:
            f = ls.ff
            shapes[p + "mlp.router"] = (f.experts, W)
            for e in range(f.experts):
                shapes.update({f"{p}mlp.e{e}.gate": (f.ff, W), f"{p}mlp.e{e}.up": (f.ff, W), f"{p}mlp.e{e}.down": (W, f.ff)})
            if f.shared_ff:
                shapes.update({p + "mlp.shared.gate": (f.shared_ff, W), p + "mlp.shared.up": (f.shared_ff, W), p + "mlp.shared.down": (W, f.shared_ff)})
                if isinstance(f, MoeSpec):
                    shapes[p + "mlp.shared.sg"] = (1, W)
    for n in norm_names:
        shapes[n] = (W,)
        if spec.norm == "layer":
            shapes[n + ".b"] = (W,)

    def get(name: str) -> torch.Tensor:
        shape = shapes[name]
        r = torch.randn(*shape, device=device, generator=g)
        last = name.rsplit(".", 1)[-1]
        if name.endswith(("q.norm", "k.norm", "dkv.norm")) or last == "D" or name.endswith(("mix.norm", "left.norm", "right.norm")) or name in norm_like or \
                (name in norm_names and spec.norm in ("layer", "rms")):
            r = 1.0 + 0.1 * r
        elif name.endswith("f.b"):
            r = 3.0 + 0.5 * r      # forget gates mostly open
        elif last == "mix" and len(shape) == 2 and shape[0] == shape[1] == spec.streams:
            r = torch.eye(shape[0], device=device) + 0.1 * r
        elif last == "in" and shape == (spec.streams,):
            r = 1.0 / spec.streams + 0.1 * r
        elif last == "out" and shape == (spec.streams,):
            r = 1.0 + 0.1 * r
        elif name in norm_names:
            r = 0.1 * r
        elif last == "talk":
            r = torch.eye(shape[0], device=device) + 0.1 * r
        elif last == "pb":
            r = -3.0 + 0.5 * r     # un-normalised weights: most keys weigh little
        elif last == "act":
            r = 0.5 * r
        elif last == "dt_bias":
            r = -2.0 + 0.5 * r
        elif last == "A_log":
            r = 0.5 * r
        elif last == "b":
            r = 0.1 * r
        elif last == "conv":
            r = 0.4 * r
        elif name != spec.embed:
            r = r * (shape[-1] ** -0.5)
        return r.to(torch.bfloat16)
    return get


SPEC_READERS: Dict[str, Callable[[dict], HybridSpec]] = {"Gekilix": gekilix_spec, "Sobunex": sobunex_spec, "Setopel": setopel_spec, "Gifopel": gifopel_spec}


class HybridCache:
    """What live sequences hold between steps, for a HybridDecoder: K / V blocks from the paged `KVCacheManager` and one state slot each from `StateSlotPool`.
    `reserve` grows a request to `total_tokens` (admitting it on first use), `entry` describes its next rows for `RaggedBatch.build`, `release` gives everything back.
    Prefix caching stays off when the model has recurrent layers: a cached K / V block does not bring the recurrent state of its last token with it."""

    def __init__(self, model: HybridDecoder, enable_prefix_caching: bool = False):
        from .kv_cache_manager import KVCacheManager, StateSlotPool
        self.model = model
        self.kv = KVCacheManager(model.num_blocks, model.block_size, enable_prefix_caching and not model.has_recurrent_state, [0])
        self.slots = StateSlotPool(model.state_slots)

    def reserve(self, request_id: int, total_tokens: int) -> bool:
        if self.slots.allocate(request_id) is None:
            return False
        if self.kv.allocate_slots(request_id, total_tokens, []) is None:
            if not self.kv.has_request(request_id):
                self.slots.free(request_id)
            return False
        return True

    def entry(self, request_id: int, tokens: Sequence[int], pos0: int, want: Sequence[int] = ()) -> dict:
        return {"tokens": list(tokens), "pos0": pos0, "slot": self.slots.slot_of(request_id), "blocks": self.kv.get_block_ids(request_id) or [], "want": list(want)}

    def release(self, request_id: int) -> None:
        self.kv.free(request_id)
        self.slots.free(request_id)
