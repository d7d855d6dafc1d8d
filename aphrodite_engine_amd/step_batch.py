"""What one engine step hands to a model: a batch of SEGMENTS.  Segment s is ``q_len[s]`` consecutive rows of the token
batch -- a portion of a prompt or a single decoded token -- that continue a sequence of which ``ctx_len[s]`` tokens were
processed by earlier steps; its keys live in the pages of ``block_tables[s]``, its recurrent state in slot
``state_slots[s]``.  The same structure serves paged attention (through ``attention_metadata()``, the fields of the
reference's AttentionMetadata, attention/backends/abstract.py:96-135) and the recurrent mixers."""
from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import numpy as np
import torch


@dataclass
class StepBatch:
    num_tokens: int
    num_seqs: int
    input_ids: torch.Tensor          # int64 [T]
    positions: torch.Tensor          # int64 [T]
    q_start: torch.Tensor            # int32 [S] first row of each segment
    q_len: torch.Tensor              # int32 [S]
    ctx_len: torch.Tensor            # int32 [S] tokens of the sequence before this step
    seq_of_token: torch.Tensor       # int32 [T]
    block_tables: torch.Tensor       # int32 [S, max_blocks]
    slot_mapping: torch.Tensor       # int64 [T] block * block_size + offset of each row's key / value
    state_slots: torch.Tensor        # int32 [S]
    block_size: int
    q_lens: List[int] = field(default_factory=list)      # host copies
    ctx_lens: List[int] = field(default_factory=list)

    @staticmethod
    def build(tokens: Sequence[Sequence[int]], ctx_lens: Sequence[int], block_tables: Sequence[Sequence[int]],
              state_slots: Sequence[int], block_size: int, device) -> "StepBatch":
        """From host lists, one entry per segment.  Every index the kernels will follow is checked here."""
        S = len(tokens)
        q_lens = [len(t) for t in tokens]
        if S == 0 or min(q_lens) <= 0:
            raise ValueError("a step batch needs at least one segment and no empty one")
        T = sum(q_lens)
        starts = np.zeros(S, np.int32)
        starts[1:] = np.cumsum(q_lens)[:-1]
        width = max(1, max(len(b) for b in block_tables))
        bt = np.zeros((S, width), np.int32)
        pos = np.empty(T, np.int64)
        slots = np.empty(T, np.int64)
        seq_of = np.empty(T, np.int32)
        for s in range(S):
            n, c, a = q_lens[s], int(ctx_lens[s]), int(starts[s])
            need = (c + n + block_size - 1) // block_size
            if len(block_tables[s]) < need:
                raise ValueError(f"segment {s}: {len(block_tables[s])} pages for {c + n} tokens")
            bt[s, :len(block_tables[s])] = block_tables[s]
            p = np.arange(c, c + n, dtype=np.int64)
            pos[a:a + n] = p
            slots[a:a + n] = bt[s, p // block_size].astype(np.int64) * block_size + p % block_size
            seq_of[a:a + n] = s
        if len(set(int(x) for x in state_slots)) != S:
            raise ValueError("two segments of one step share a state slot")

        def dev(a):
            return torch.from_numpy(a).to(device)
        ids = np.concatenate([np.asarray(t, np.int64) for t in tokens])
        return StepBatch(num_tokens=T, num_seqs=S, input_ids=dev(ids), positions=dev(pos), q_start=dev(starts),
                         q_len=dev(np.asarray(q_lens, np.int32)), ctx_len=dev(np.asarray(ctx_lens, np.int32)),
                         seq_of_token=dev(seq_of), block_tables=dev(bt), slot_mapping=dev(slots),
                         state_slots=dev(np.asarray(state_slots, np.int32)), block_size=block_size, q_lens=q_lens,
                         ctx_lens=[int(c) for c in ctx_lens])

    def last_rows(self) -> List[int]:
        """Row of the last token of every segment."""
        out, a = [], 0
        for n in self.q_lens:
            a += n
            out.append(a - 1)
        return out

    def decode_split(self) -> int:
        """Number of leading segments that are prompt portions when the batch is ordered portions first, single tokens
        with a context last (the order the reference's metadata assumes); raises if it is not."""
        kinds = [n == 1 and c > 0 for n, c in zip(self.q_lens, self.ctx_lens)]
        k = kinds.index(True) if True in kinds else len(kinds)
        if not all(kinds[k:]):
            raise ValueError("segments are not ordered prompt portions first, decoded tokens last")
        return k

    def attention_metadata(self):
        """The same batch as MI355XAttentionMetadata (prefill rows first, decode rows after)."""
        from .attention.backend import MI355XAttentionMetadata
        k = self.decode_split()
        dev = self.input_ids.device
        seq_lens = [c + n for c, n in zip(self.ctx_lens, self.q_lens)]
        npt = sum(self.q_lens[:k])
        loc = np.zeros(k + 1, np.int32)
        loc[1:] = np.cumsum(self.q_lens[:k])
        sloc = np.zeros(k + 1, np.int32)
        sloc[1:] = np.cumsum(seq_lens[:k])
        return MI355XAttentionMetadata(
            num_prefills=k, num_prefill_tokens=npt, num_decode_tokens=self.num_tokens - npt, slot_mapping=self.slot_mapping,
            seq_lens=seq_lens, seq_lens_tensor=torch.tensor(seq_lens, dtype=torch.int32, device=dev),
            max_query_len=max(self.q_lens), max_prefill_seq_len=max(seq_lens[:k], default=0),
            max_decode_seq_len=max(seq_lens[k:], default=0),
            query_start_loc=torch.from_numpy(loc).to(dev), seq_start_loc=torch.from_numpy(sloc).to(dev),
            context_lens_tensor=self.ctx_len[:k] if k else self.ctx_len[:0], block_tables=self.block_tables,
            use_cuda_graph=False, max_context_len=max(self.ctx_lens[:k], default=0))
