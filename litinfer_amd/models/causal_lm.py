"""The Python entry point, in the manner of the reference's
`llaisys.models.Qwen2` (python/llaisys/models/qwen2.py:23-501): a model folder
in, token ids in, token ids out.

    model = load(model_path)            # the class that the architecture's registry entry names
    tokens = model.generate(inputs, max_new_tokens=64, top_k=1, top_p=1.0, temperature=1.0)

Names and meanings of the options are the reference's.  `generate` is the
scheduler with one request; the `engine_*` calls are the scheduler itself.
Nothing here knows an architecture: the model is whatever config.json names in
the registry of architectures.
"""
from __future__ import annotations

import time
from pathlib import Path
from typing import Iterator, List, Optional, Sequence

from ..engine import Engine, Scheduler
from ..sampling import SamplingParams


def _is_greedy(top_k: int, top_p: float, temperature: float) -> bool:
    """The reference decodes greedily iff top_k == 1 and top_p >= 1 and
    temperature == 1 (python/llaisys/models/qwen2.py:378)."""
    return top_k == 1 and top_p >= 1.0 and temperature == 1.0


def _params(top_k: int, top_p: float, temperature: float, seed: int) -> SamplingParams:
    if _is_greedy(top_k, top_p, temperature):
        return SamplingParams()
    # a temperature <= 0 means "1" in the reference's sampling path (src/llaisys/models/qwen2.cpp:442)
    return SamplingParams(temperature=temperature if temperature > 0 else 1.0, top_k=int(top_k),
                          top_p=float(top_p), seed=int(seed))


class CausalLM:
    def __init__(self, model_path, device: str = "cuda:0", quantize: Optional[str] = None, *,
                 dtype: str = "bfloat16", page_size: int = 16, num_pages: Optional[int] = None,
                 max_tokens: Optional[int] = None, max_seqs: int = 64, max_batch_tokens: int = 2048,
                 chunk_size: int = 512, seed: int = 0, lookahead: bool = True, strict_weights: bool = False,
                 keep_stored_precision: bool = False):
        if quantize is not None:
            raise NotImplementedError("quantized weights are not supported")
        self.model_path = Path(model_path)
        print(f"[litinfer_amd] loading {self.model_path} ({dtype}) ...", flush=True)
        self.engine = Engine.from_dir(self.model_path, dtype=dtype, device=device, page_size=page_size,
                                      num_pages=num_pages, max_tokens=max_tokens, max_seqs=max_seqs,
                                      strict_weights=strict_weights, keep_stored_precision=keep_stored_precision,
                                      step_tokens=max_batch_tokens)
        self.meta = self.engine.config
        self.seed = int(seed)
        # lookahead: a step is started before the tokens of the one before have reached the host
        self._sched_args = dict(max_batch_tokens=max_batch_tokens, chunk_size=chunk_size,
                                lookahead=bool(lookahead))
        self._scheduler: Optional[Scheduler] = None
        print(f"[litinfer_amd] ready: {self.engine.spec.architecture}, "
              f"{self.engine.model.weight_bytes() / 2**20:.1f} MiB of weights", flush=True)

    @property
    def max_seq_len(self) -> int:
        return self.engine.spec.max_positions

    @property
    def end_tokens(self):
        return self.engine.spec.eos_token_ids

    # ---- single request ---------------------------------------------------
    def _check(self, inputs: Sequence[int], max_new_tokens: int, who: str) -> List[int]:
        tokens = [int(t) for t in inputs]
        if not tokens:
            raise ValueError(f"{who}: inputs must not be empty")
        if len(tokens) + max_new_tokens - 1 > self.max_seq_len:
            raise ValueError(f"{who}: requested prompt and output exceed model max sequence length "
                             f"({self.max_seq_len})")
        return tokens

    def generate(self, inputs: Sequence[int], max_new_tokens: Optional[int] = None, top_k: int = 1,
                 top_p: float = 1.0, temperature: float = 1.0) -> List[int]:
        """New tokens only; an end token stops and is not returned.  The first new
        token is always the argmax, as in the reference
        (python/llaisys/models/qwen2.py:359)."""
        return self.generate_profile(inputs, max_new_tokens, top_k, top_p, temperature)[0]

    def generate_profile(self, inputs, max_new_tokens=None, top_k=1, top_p=1.0, temperature=1.0):
        max_new_tokens = 1 if max_new_tokens is None else max_new_tokens
        zero = {"prefill_seconds": 0.0, "first_token_seconds": 0.0, "decode_seconds": 0.0,
                "decode_tokens": 0, "decode_tokens_per_second": 0.0,
                "time_per_decode_token_seconds": 0.0, "generated_tokens": 0}
        if max_new_tokens <= 0:
            return [], zero
        t0 = time.perf_counter()
        first_at = None
        out: List[int] = []
        for tok in self.generate_stream(inputs, max_new_tokens, top_k, top_p, temperature,
                                        _who="generate"):
            if first_at is None:
                first_at = time.perf_counter()
            out.append(tok)
        t1 = time.perf_counter()
        prefill = (first_at if first_at is not None else t1) - t0
        dec_tokens = max(len(out) - 1, 0)
        dec = t1 - first_at if first_at is not None else 0.0
        return out, {"prefill_seconds": prefill, "first_token_seconds": prefill, "decode_seconds": dec,
                     "decode_tokens": dec_tokens,
                     "decode_tokens_per_second": dec_tokens / dec if dec > 0 and dec_tokens else 0.0,
                     "time_per_decode_token_seconds": dec / dec_tokens if dec_tokens else 0.0,
                     "generated_tokens": len(out)}

    def generate_stream(self, inputs, max_new_tokens: int = 128, top_k: int = 1, top_p: float = 1.0,
                        temperature: float = 1.0, _who: str = "generate_stream") -> Iterator[int]:
        max_new_tokens = 1 if max_new_tokens is None else max_new_tokens
        tokens = self._check(inputs, max_new_tokens, _who)
        sched = Scheduler(self.engine, **self._sched_args)
        rid = sched.add_request(tokens, max_new_tokens, _params(top_k, top_p, temperature, self.seed),
                                first_token_greedy=True)
        try:
            while sched.has_unfinished():
                for _, tok in sched.step():
                    yield tok
            reason = sched.requests[rid].finish_reason or ""
            if reason.startswith("error"):
                raise RuntimeError(f"{_who}: {reason}")
        finally:
            sched.abort(rid)                         # gives back whatever is still held

    # ---- continuous batching ------------------------------------------------
    def engine_start(self) -> None:
        self._scheduler = Scheduler(self.engine, **self._sched_args)

    def _sched(self) -> Scheduler:
        if self._scheduler is None:
            self.engine_start()
        return self._scheduler

    def engine_add_request(self, inputs: Sequence[int], max_new_tokens: int = 128,
                           sampling: Optional[SamplingParams] = None) -> int:
        """Returns the request id.  Without `sampling` the options given to
        `engine_step` apply to the request, as in the reference."""
        return self._sched().add_request(inputs, max_new_tokens, sampling)

    def engine_step(self, top_k: int = 1, top_p: float = 1.0, temperature: float = 1.0) -> int:
        """One step of continuous batching; returns how many requests finished in
        it.  temperature <= 0 is greedy (src/llaisys/models/qwen2.cpp:893)."""
        s = self._sched()
        before = sum(1 for r in s.requests.values() if r.state == "finished")
        default = (SamplingParams() if temperature <= 0 or top_k == 1 else
                   SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p, seed=self.seed))
        s.step(default)
        return sum(1 for r in s.requests.values() if r.state == "finished") - before

    def engine_has_unfinished(self) -> bool:
        return self._sched().has_unfinished()

    def engine_num_seqs(self) -> int:
        return self._sched().num_requests()

    def engine_is_finished(self, seq_id) -> bool:
        return self._sched().is_finished(seq_id)

    def engine_get_output(self, seq_id) -> List[int]:
        return self._sched().output(seq_id)

    def engine_stop(self) -> None:
        if self._scheduler is not None:
            for rid, r in list(self._scheduler.requests.items()):
                self._scheduler.abort(rid)
        self._scheduler = None
