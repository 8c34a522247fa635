"""Requests over one model: a pool of sequence states and batched steps (the host side of uzu_hip_model_step_batch).

`SequencePool` owns the HipStates of the live requests of an f32-stream model: a new request takes a state that a finished request gave back (reset) or a fresh
one; `step` runs the next tokens of any subset of the live requests as ONE batch of the engine -- prompts of unequal length, continued prompts and one-token decode
steps alike -- and returns the logits asked for and, on request, the token sampled from every request's last row.  `generate` decodes several prompts together
until each has its tokens or its stop token: requests leave the batch as they finish, the others go on.  bin/trace_run replays recorded steps through the same pool.
"""
from __future__ import annotations

from typing import Dict, Hashable, Iterable, List, Optional, Sequence

import numpy as np

from .engine import HipModel, HipState


class SequencePool:
    def __init__(self, model: HipModel):
        if not model.f32_stream:
            raise ValueError("batched steps of unequal sequences are a path of the f32-stream designs (HipModel.step_batch)")
        self.model = model
        self.live: Dict[Hashable, HipState] = {}
        self.free: List[HipState] = []

    def state(self, rid: Hashable) -> HipState:
        """the state of request `rid`; a request seen for the first time takes a recycled state or a new one (context length 0)"""
        st = self.live.get(rid)
        if st is None:
            st = self.free.pop() if self.free else self.model.new_state()
            self.live[rid] = st
        return st

    def finish(self, rid: Hashable):
        """what the request holds goes back to the pool"""
        st = self.live.pop(rid, None)
        if st is not None:
            st.reset()
            self.free.append(st)

    def step(self, entries: Sequence[dict], sample: bool = False):
        """entries: [{"id", "tokens", "want" (optional positions among the tokens)}] -> (logits f32 [wanted, vocab] in the order of the entries and of `want`,
        sampled token per entry or None)"""
        if not entries:
            return np.empty((0, self.model.vocab_size), dtype=np.float32), None
        states = [self.state(e["id"]) for e in entries]
        return self.model.step_batch(states, [e["tokens"] for e in entries], [e.get("want") or [] for e in entries], sample=sample)

    def generate(self, prompts: Dict[Hashable, Sequence[int]], max_tokens: int, stop_token_ids: Iterable[int] = ()) -> Dict[Hashable, List[int]]:
        """Prefill all prompts in one batch, then decode them together; returns the generated ids per request (a stop token ends a request and is not returned).
        Sampling follows the model's setting (HipModel.set_sampling; greedy by default)."""
        stops = set(int(t) for t in stop_token_ids)
        out: Dict[Hashable, List[int]] = {rid: [] for rid in prompts}
        live = list(prompts)
        _, sampled = self.step([{"id": rid, "tokens": list(prompts[rid])} for rid in live], sample=True)
        while live:
            nxt, go_on = {}, []
            for rid, tok in zip(live, sampled):
                tok = int(tok)
                if tok in stops:
                    self.finish(rid)
                    continue
                out[rid].append(tok)
                if len(out[rid]) >= max_tokens:
                    self.finish(rid)
                else:
                    nxt[rid] = tok
                    go_on.append(rid)
            live = go_on
            if live:
                _, sampled = self.step([{"id": rid, "tokens": [nxt[rid]]} for rid in live], sample=True)
        return out

    def close(self):
        for st in list(self.live.values()) + self.free:
            st.close()
        self.live.clear()
        self.free.clear()
