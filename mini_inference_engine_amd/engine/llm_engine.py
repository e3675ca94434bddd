"""The offline entry point: add requests, step until done.

Surface as the reference's (inference_engine/engine.py:17-24,35-37,123,181,232):
``LLMEngine(model, engine_config, dtype, load_tokenizer, verbose)``,
``add_request``, ``step`` (returns the requests that finished), ``generate``,
``RequestOutput``; attributes ``scheduler``, ``cfg``, ``model_cfg``,
``num_steps``, ``num_graph_steps``.  ``model`` is a folder (config.json and
safetensors); prompts are lists of token ids (strings only when a tokenizer
was loaded).
"""
from __future__ import annotations

import time
from dataclasses import dataclass, replace

import torch

from ..config.engine_config import EngineConfig
from ..sampling import Sampler, SamplingParams
from .batch import StepRow
from .runner import ModelRunner, parse_dtype
from .scheduler import Scheduler
from .sequence import PENDING, Sequence, Status


@dataclass
class RequestOutput:
    seq_id: int
    prompt_len: int
    output_ids: list
    text: str | None
    ttft: float | None          # seconds from arrival to the first generated token
    latency: float | None       # seconds from arrival to the end


@dataclass
class _StepInFlight:
    """A step that was started and whose chosen tokens the host has not read."""
    seqs: list                  # the requests a token is being chosen for, in sampling order
    places: list                # where in each request's token list that token goes
    chosen: object              # sampling.ChosenTokens, or None if no row wanted a token
    index_of: dict              # request -> its entry among the chosen tokens (for the next step's rows)


class LLMEngine:
    def __init__(self, model, engine_config: EngineConfig | None = None, dtype=torch.bfloat16,
                 load_tokenizer: bool = False, verbose: bool = True, *, device="cuda", backend=None, weights=None):
        self.cfg = engine_config or EngineConfig()
        self.verbose = verbose
        self.dtype = parse_dtype(dtype)
        cfg = self.cfg
        self.runner = ModelRunner(
            model, dtype=self.dtype, device=device, backend=backend, page_size=cfg.block_size,
            num_pages=cfg.num_blocks, memory_fraction=cfg.kv_cache_memory_fraction,
            reserve_bytes=cfg.activation_reserve_bytes, max_step_tokens=cfg.max_num_batched_tokens,
            max_rows=cfg.max_num_seqs, max_model_len=cfg.max_model_len, num_state_slots=cfg.num_state_slots,
            weights=weights, cast_float32_weights=cfg.cast_float32_weights,
            tune_library_products=cfg.tune_library_products)
        self.model_cfg = self.runner.model_cfg
        self.cfg.max_model_len = self.runner.max_model_len
        self.cache = self.runner.cache
        self.allocator = self.cache            # the name the reference's callers use
        if cfg.poison_freed_pages:
            self.cache.on_release = self.runner.storage.poison_pages
        self.scheduler = Scheduler(self.cfg, self.cache)
        self.sampler = Sampler(self.runner.device, cfg.max_num_seqs, out=self.runner.chosen_tokens)
        if cfg.trace_ranges and self.runner.device.type == "cuda":
            self.runner.ranges.on = True
        self._in_flight = None             # the step whose tokens the host has not read yet
        self.stop_token_ids = frozenset(self.runner.model.spec.stop_token_ids)
        if verbose:
            print(f"[mini_inference_engine_amd] cache: {self.runner.num_pages} pages x {cfg.block_size} tokens "
                  f"({self.runner.storage.num_bytes() / 2**30:.2f} GiB), weights "
                  f"{self.runner.model.weight_bytes() / 2**30:.2f} GiB, dtype {self.dtype}", flush=True)
        kept = self.runner.load_report.get("kept_float32", [])
        if kept:
            import warnings
            warnings.warn(f"{len(kept)} weight matrices are stored in float32 and stay so (first: {kept[0]}): their "
                          f"products run on the 32-bit kernels, much slower than bfloat16; save the checkpoint in "
                          f"bfloat16, or set EngineConfig.cast_float32_weights, for speed", stacklevel=2)
        self.tokenizer = None
        if load_tokenizer and isinstance(model, str):
            from transformers import AutoTokenizer      # text in and out only; never on the token path
            self.tokenizer = AutoTokenizer.from_pretrained(model)
        if cfg.use_hip_graphs and self.runner.device.type == "cuda":
            self.runner.capture_decode_graphs(cfg.graph_batch_sizes, verbose=verbose, sample=True)
            sizes = cfg.portion_graph_sizes
            if sizes is None:           # eighths of the token budget: a prompt runs in a step at most an eighth of it longer
                most = min(cfg.max_num_batched_tokens, self.runner.max_model_len)
                sizes = sorted({most * k // 8 for k in range(1, 9) if most * k // 8 >= 64} | ({most} if most >= 2 else set()))
            if cfg.enable_chunked_prefill and sizes:
                self.runner.capture_portion_graphs(sizes)
        self.graphs = self.runner.graphs
        self.num_steps = 0
        self.num_graph_steps = 0
        self._num_requests = 0

    # ---------------------------------------------------------------- requests
    def add_request(self, prompt, params: SamplingParams | None = None) -> Sequence:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("a text prompt needs a tokenizer (load_tokenizer=True); pass token ids instead")
            ids = self.tokenizer.encode(prompt)
        else:
            ids = list(prompt)
        params = params or SamplingParams()
        if len(ids) > self.cfg.max_model_len:
            raise ValueError(f"prompt of {len(ids)} tokens exceeds max_model_len {self.cfg.max_model_len}")
        vocab = self.runner.vocab_size
        bad = [t for t in ids if not 0 <= t < vocab]
        if bad:
            raise ValueError(f"token ids outside the vocabulary of {vocab}: {bad[:5]}")
        if len(ids) + params.max_tokens > self.cfg.max_model_len:
            params = replace(params, max_tokens=self.cfg.max_model_len - len(ids))
        seq = Sequence(ids, params)
        if params.seed is None:
            seq.seed = (self.cfg.seed << 32) ^ self._num_requests
        self._num_requests += 1
        self.scheduler.add(seq)
        return seq

    # ------------------------------------------------------------------- step
    def has_work(self) -> bool:
        return self._in_flight is not None or self.scheduler.has_work()

    def step(self) -> list[Sequence]:
        """Starts one step (schedule, forward, sampling) and then reads the tokens of the step before it,
        which ran on the device while this one was prepared.  Returns the requests which that earlier step
        finished.  With ``run_ahead`` off, the step started is also the one read.

        Running one step ahead: a request's next row is scheduled before its last token is known to the
        host; the device takes the token from where the sampling kernel left it.  What does not depend on
        the token's value (positions, pages, the end by max_tokens or length) is decided at once; an end
        by the stop token is seen one step late, and the row already started for that request is dropped."""
        started = self._start()
        if not self.cfg.run_ahead:
            return self._finish_step(started) if started is not None else []
        finished = self._finish_step(self._in_flight) if self._in_flight is not None else []
        self._in_flight = started
        return finished

    def drain(self) -> list[Sequence]:
        """Reads the tokens of the step that is still on its way, if any, without starting another."""
        if self._in_flight is None:
            return []
        finished = self._finish_step(self._in_flight)
        self._in_flight = None
        return finished

    def _start(self):
        with self.runner.ranges("schedule"):
            batch = self.scheduler.schedule()
        if not batch:
            return None
        taken = self._in_flight.index_of if self._in_flight is not None else {}
        rows, sample_seqs = [], []
        for seq, n in batch:
            nc = seq.num_computed
            last = nc + n == seq.num_tokens
            tokens = seq.token_ids[nc:nc + n]
            source = -1
            if tokens[-1] == PENDING:
                # only ever the one token the step in flight is choosing for this request
                if n != 1 or seq not in taken:
                    raise RuntimeError(f"request {seq.seq_id}: a token not yet known in a row of {n}")
                tokens, source = [0], taken[seq]
            rows.append(StepRow(seq.cache, tokens, nc, [n - 1] if last else [], taken_from=source))
            if last:
                sample_seqs.append(seq)

        # a captured graph when every row is a single token; the tokens are chosen in the step as well
        self.runner.forward_step(rows, sampling=self.sampler.sampling_inputs(sample_seqs) if sample_seqs else None)
        self.num_steps += 1
        self.num_graph_steps += self.runner.last_step_captured
        chosen = self.sampler.fetch_async(len(sample_seqs)) if sample_seqs else None

        # what is certain whatever the tokens turn out to be
        for seq, n in batch:
            self.scheduler.advance(seq, n)
        places = []
        for seq in sample_seqs:
            places.append(seq.num_tokens)
            seq.token_ids.append(PENDING)
            if seq.num_output_tokens >= seq.params.max_tokens or seq.num_tokens >= self.cfg.max_model_len:
                seq.ending = True              # its last token is on its way: not to be scheduled again
        return _StepInFlight(sample_seqs, places, chosen, {s: j for j, s in enumerate(sample_seqs)})

    def _finish_step(self, st) -> list[Sequence]:
        tokens = st.chosen.tolist() if st.chosen is not None else []
        now = time.perf_counter()
        finished = []
        for seq, place, tok in zip(st.seqs, st.places, tokens):
            if seq.status is Status.FINISHED:
                continue                       # ended by its stop token a step ago; this row was one too many
            seq.token_ids[place] = tok
            if seq.first_token_time is None:
                seq.first_token_time = now
            stopped = tok in self.stop_token_ids and not seq.params.ignore_eos
            if not (stopped or (seq.ending and place == seq.num_tokens - 1)):
                continue
            del seq.token_ids[place + 1:]      # a placeholder of the row started meanwhile, if any
            seq.finish_time = now
            if seq.status is Status.RUNNING:
                self.scheduler.finish(seq)
            else:                              # preempted while its last token was on its way
                self.scheduler.waiting.remove(seq)
                seq.status = Status.FINISHED
            finished.append(seq)
        return finished

    @property
    def eos_token_id(self):
        """The stop id, under the name the reference's engine has (inference_engine/engine.py:217); the first
        one if the model has several.  Assigning replaces them all by one id."""
        return min(self.stop_token_ids) if self.stop_token_ids else None

    @eos_token_id.setter
    def eos_token_id(self, token):
        self.stop_token_ids = frozenset() if token is None else frozenset([int(token)])

    # --------------------------------------------------------------- offline
    def generate(self, prompts, params: SamplingParams | list | None = None, decode_text: bool = True
                 ) -> list[RequestOutput]:
        if not isinstance(params, list):
            params = [params or SamplingParams()] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError(f"{len(prompts)} prompts but {len(params)} sampling params")
        seqs = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        while self.has_work():
            self.step()
        outs = []
        for s in seqs:
            text = None
            if decode_text and self.tokenizer is not None:
                text = self.tokenizer.decode(s.output_ids, skip_special_tokens=True)
            outs.append(RequestOutput(s.seq_id, s.prompt_len, s.output_ids, text,
                                      s.first_token_time - s.arrival_time, s.finish_time - s.arrival_time))
        return outs
