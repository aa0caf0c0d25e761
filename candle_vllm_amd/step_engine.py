"""Step driver for models whose layers carry state from token to token (candle_vllm_amd.hybrid_model): the block engine's pages and
state slots, the block engine's input preparation, and the model's one step function.  A request is admitted with its first tokens,
may bring more prompt tokens (or decoded ones) at any later step, may sit a step out, and gives its pages and its slot back when it
ends.  Every entry of a step is one row group of the same launch: portions of prompts beside single decoded tokens.
The continuous-batching loop with the scheduler is candle_vllm_amd.engine.run_engine; this class is what drives a given schedule
(replaying a trace, tests of cache and state handling)."""
import numpy as np

from .block_engine import BlockEngine


class StepEngine:
    def __init__(self, model, max_tokens, block_size=None):
        """max_tokens: the most tokens live requests hold at any time, each request's count rounded up to the page size"""
        self.model = model
        self.block_size = int(block_size or model.block_size)
        self.num_blocks = max(1, -(-int(max_tokens) // self.block_size))
        self.be = BlockEngine(self.block_size, self.num_blocks, 0)
        self.be.state_init(model.state_slots)
        model.alloc_cache(self.num_blocks)
        self.seqs, self._next = {}, 0
        self.use_graph = True                 # short steps (decoding batches) replay a captured hipGraph

    def feed(self, rid, tokens):
        """admit `rid` with its first tokens, or append tokens to it; pages are taken for exactly what the sequence holds"""
        tokens = [int(t) for t in tokens]
        if not tokens:
            raise ValueError("an entry brings at least one token")
        s = self.seqs.get(rid)
        if s is None:
            s = self.seqs[rid] = self.be.new_sequence(self._next, tokens)
            self._next += 1
            try:
                self.be.allocate([s], chunk=len(tokens))
                self.be.state_acquire(s)
            except RuntimeError:
                del self.seqs[rid]
                self.be.free_sequence(s)
                self.be_remove(s)
                raise
        else:
            s.extend_prompt(tokens)
            if not self.be.can_append_prefill_chunk_to_seq_group([s], 0):
                raise RuntimeError("no free pages for the request's next tokens")
            self.be.append_prefill_chunk_slots_to_seq_group([s], 0)
        return s

    def be_remove(self, s):
        from ._lib import lib
        lib.mi355_be_seq_remove(self.be.h, s.id)

    def step(self, rids, want=None, trace=False):
        """run the not yet cached tokens of `rids` as one batch.  want: per request, the places among its new tokens whose logits
        are asked for (default: the last).  -> logits f32 [sum of wanted places, vocab] (torch, on the device)"""
        group = [self.seqs[r] for r in rids]
        pending = sum(s.get_len() - s.get_num_cached_tokens() for s in group)
        meta = self.be.prepare_prompt(group, chunk=0, tok_cap=max(16, pending))
        cu = np.asarray(meta["cu_seqlens_q"]).astype(np.int64)
        if want is None:
            rows = (cu[1:] - 1).tolist()
        else:
            rows = []
            for i, w in enumerate(want):
                for k in w:
                    if not 0 <= k < cu[i + 1] - cu[i]:
                        raise ValueError("a wanted place outside the entry's tokens")
                    rows.append(int(cu[i] + k))
        slots = [self.be.state_slot(s) for s in group]
        out = self.model.step(meta, slots, want_rows=rows, trace=trace, graph=self.use_graph)
        for s in group:
            s.set_num_cached_tokens(s.get_len())
        return out

    def finish(self, rid):
        """the request is done: its pages and its state slot go back to the pools"""
        s = self.seqs.pop(rid)
        self.be.free_sequence(s)
        self.be_remove(s)

    def free_pages(self):
        return self.be.get_num_free_blocks()
