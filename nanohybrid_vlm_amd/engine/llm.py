"""The Python entry point: ``LLM(model, **options).generate(prompts, sampling_params)``.

Surface and meanings follow the reference (nanovllm/llm.py:4,
nanovllm/engine/llm_engine.py:176-993): ``add_request``, ``step``, ``is_finished``,
``generate``, ``exit``; a prompt is a string (needs the checkpoint's tokenizer) or a
list of token ids; ``generate`` returns ``[{"text", "token_ids"}]`` in the order of
the prompts. Options are the fields of ``EngineConfig``; an unknown option is an
error (the reference drops it silently, llm_engine.py:179-181).
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from itertools import count
from time import perf_counter

from ..config.engine_config import EngineConfig
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler, noise_key
from .runner import ModelRunner, StepEntry
from .scheduler import Scheduler
from .sequence import Sequence


@dataclass
class StepStats:
    """Tokens and wall time of one step (llm_engine.py:27-63). Decoded tokens and
    prompt portions run in one pass here, so both rates are over the same time."""

    num_prefill_tokens: int = 0
    num_decode_tokens: int = 0
    seconds: float = 0.0
    num_preempted: int = 0

    @property
    def prefill_throughput(self) -> float:
        return self.num_prefill_tokens / self.seconds if self.seconds > 0 else 0.0

    @property
    def decode_throughput(self) -> float:
        return self.num_decode_tokens / self.seconds if self.seconds > 0 else 0.0


@dataclass
class RequestMetrics:
    """Times of one request in seconds of ``perf_counter`` (llm_engine.py:66-174)."""

    seq_id: int
    num_prompt_tokens: int
    arrival: float
    first_scheduled: float | None = None
    first_token: float | None = None
    finished: float | None = None
    num_completion_tokens: int = 0

    @property
    def ttft_ms(self):
        return None if self.first_token is None else (self.first_token - self.arrival) * 1e3

    @property
    def e2e_ms(self):
        return None if self.finished is None else (self.finished - self.arrival) * 1e3

    @property
    def tpot_ms(self):
        if self.finished is None or self.first_token is None or self.num_completion_tokens < 2:
            return None
        return (self.finished - self.first_token) * 1e3 / (self.num_completion_tokens - 1)

    @property
    def queue_ms(self):
        return None if self.first_scheduled is None else (self.first_scheduled - self.arrival) * 1e3


def validate_token_ids(token_ids) -> None:
    """A prompt of token ids is a list with at least one entry, every entry a plain integer that is not
    negative (the reference checks the same four things, nanovllm/inputs.py:29-55)."""
    if not isinstance(token_ids, list):
        raise TypeError(f"a prompt of token ids is a list, not {type(token_ids).__name__}")
    if len(token_ids) == 0:
        raise ValueError("a prompt needs at least one token")
    for place, t in enumerate(token_ids):
        if isinstance(t, bool) or not isinstance(t, int):
            raise TypeError(f"token {place} of the prompt is {t!r}: token ids are integers")
        if t < 0:
            raise ValueError(f"token {place} of the prompt is {t}: token ids are not negative")


def _load_tokenizer(folder: str):
    path = os.path.join(folder, "tokenizer.json")
    if not os.path.isfile(path):
        return None
    from tokenizers import Tokenizer
    return Tokenizer.from_file(path)


def _tokenizer_eos(folder: str, tokenizer) -> int | None:
    """The id of the tokenizer's end-of-sequence token: ``tokenizer_config.json`` names the token (a string, or an
    object with ``content``), ``tokenizer.json`` knows its id. None if the folder does not say. Several end tokens
    are refused, as for the model's own (nanovllm/engine/llm_engine.py:217-220)."""
    import json
    path = os.path.join(folder, "tokenizer_config.json")
    if tokenizer is None or not os.path.isfile(path):
        return None
    with open(path) as f:
        token = json.load(f).get("eos_token")
    if isinstance(token, dict):
        token = token.get("content")
    if isinstance(token, (list, tuple)):
        raise NotImplementedError("several end-of-sequence tokens are not supported")
    if not isinstance(token, str):
        return None
    return tokenizer.token_to_id(token)


class LLM:
    def __init__(self, model, *, random_weights: int | None = None, built_model=None, poison_freed_pages: bool = False,
                 **kwargs):
        """``model``: folder with config.json, model.safetensors (and tokenizer.json for text prompts); or the
        contents of a config.json as a dict, together with ``random_weights=seed``: a model of that
        configuration with random weights drawn on the device.
        ``built_model``: (architecture, typed configuration, model with weights bound) made elsewhere;
        ``model`` is then only a label.
        ``poison_freed_pages``: a debugging aid of the runner (every page that a request gives back is filled
        with NaN, so that a read of a page its reader no longer owns shows in the logits)."""
        unknown = set(kwargs) - EngineConfig.field_names()
        if unknown:
            raise TypeError(f"unknown engine options: {sorted(unknown)}; known: {sorted(EngineConfig.field_names())}")
        if isinstance(model, dict):
            if built_model is not None:
                raise TypeError("give either a configuration with random_weights or built_model, not both")
            if random_weights is None:
                raise TypeError("a configuration in place of a model folder needs random_weights=SEED")
            from ..weights.random_init import build_random_model
            check = EngineConfig(model="random weights", **kwargs)           # (the options are checked before the weights are drawn)
            built_model = build_random_model(model, random_weights, check.dtype, check.device,
                                             options={"residual_float32": check.residual_dtype == "float32"})
            model = f"random weights ({built_model[0].name}, seed {random_weights})"
        elif random_weights is not None:
            raise TypeError("random_weights goes with a configuration (a dict), not with a model folder")
        self.config = cfg = EngineConfig(model=model, **kwargs)
        if built_model is None and not os.path.isdir(model):
            raise FileNotFoundError(f"model folder '{model}' does not exist")
        arch, typed, built = built_model if built_model is not None else (None, None, None)
        gemm_table, measure_gemms = self._gemm_choices_of(cfg)
        self.runner = ModelRunner(
            model, dtype=cfg.dtype, device=cfg.device, page_size=cfg.kvcache_block_size,
            num_pages=None if cfg.num_kvcache_blocks == -1 else cfg.num_kvcache_blocks,
            num_state_slots=cfg.max_num_seqs if cfg.num_state_slots == -1 else cfg.num_state_slots,
            gpu_memory_utilization=cfg.gpu_memory_utilization, max_num_batched_tokens=cfg.max_num_batched_tokens,
            model=built, arch=arch, cfg=typed, use_graphs=not cfg.enforce_eager, max_model_len=cfg.max_model_len,
            share_prefixes=cfg.enable_prefix_cache, max_graph_batch=cfg.max_graph_batch, max_graph_tokens=cfg.max_graph_tokens,
            residual_float32=cfg.residual_dtype == "float32", poison_freed_pages=poison_freed_pages,
            gemm_table=gemm_table, measure_gemms=measure_gemms, fuse_norms=cfg.fuse_norms)
        cfg.num_kvcache_blocks = self.runner.num_pages
        # max_model_len is capped by the model's positions (nanovllm/config.py:420-423); both, and the token that
        # ends a request, are facts of the built model (no field of an architecture's configuration is read here)
        cfg.max_model_len = min(cfg.max_model_len, self.runner.max_position)
        self.tokenizer = _load_tokenizer(model) if built_model is None else None
        if cfg.eos == -1:
            # the model's end token; a model that names none ends where its tokenizer does
            # (nanovllm/engine/llm_engine.py:207-223)
            eos = self.runner.eos_token_id
            if eos is None and built_model is None:
                eos = _tokenizer_eos(model, self.tokenizer)
            if eos is not None:
                cfg.eos = eos
        self.scheduler = Scheduler(self.runner.cache, cfg.max_num_seqs, cfg.max_num_batched_tokens, cfg.eos,
                                   cfg.max_model_len, cfg.scheduler_policy, cfg.max_prefill_wait_ms,
                                   release=self.runner.finish)
        self.sampler = Sampler(self.runner.vocab_size)
        self._ids = count()
        self._sequences: dict[int, Sequence] = {}
        self._metrics: dict[int, RequestMetrics] = {}
        self._completed_metrics: list[RequestMetrics] = []
        self._ahead = None               # a decoding step issued before its tokens were known to the host (see step)
        self.num_steps_ahead = 0         # steps that were already under way when their turn came
        if cfg.warm_up:
            self.warm_up()

    # ------------------------------------------------------------------ how matrix products are done
    @staticmethod
    def _gemm_choices_of(cfg: EngineConfig) -> tuple[dict | None, bool]:
        """(this engine's table of choices, whether shapes it lacks may be timed). With a table read from a file, or
        with measuring off, the same kernels run in every process: logits are the same bit for bit from start to
        start, and no step pays for a measurement. An engine with a file of choices, or with measuring off, has a
        table of its own; any other shares the process-wide table, in which a shape is timed once for all engines."""
        import json
        from ..native import ops
        backend = ops.backend()
        if not hasattr(backend, "parse_choices"):
            return None, False                         # (a stand-in for the kernels has nothing to choose)
        if cfg.gemm_choices and os.path.isfile(cfg.gemm_choices):
            with open(cfg.gemm_choices) as f:
                return backend.parse_choices(json.load(f)), False
        if cfg.gemm_choices or not cfg.measure_gemms:
            return {}, bool(cfg.measure_gemms)
        return None, True

    def gemm_choices(self) -> dict:
        """How each shape of matrix product that this engine's table holds is done ("M,N,K,float result,gated" ->
        -1 own kernel, -2 the rule, or a library algorithm's number)."""
        from ..native import ops
        backend = ops.backend()
        if not hasattr(backend, "choices_table"):
            return {}
        table = self.runner.gemm_table
        return backend.choices_table(backend.shared_chosen if table is None else table)

    def save_gemm_choices(self, path: str | None = None) -> str:
        """Writes the choices made so far to ``path`` (default: the engine option ``gemm_choices``); a later run
        started with ``gemm_choices=path`` does every product the same way and times nothing."""
        import json
        path = path or self.config.gemm_choices
        if not path:
            raise ValueError("no file named: pass a path or start the engine with gemm_choices=PATH")
        with open(path, "w") as f:
            json.dump(self.gemm_choices(), f, indent=1, sort_keys=True)
        return path

    # ------------------------------------------------------------------ before the first request
    def warm_up(self, batch_sizes=None, token_counts=None) -> dict:
        """Meets every size of step that replays a graph once, before any request does: the matrix products of each
        size are measured (which is what takes the time: a fraction of a second a size) and the graphs of single-token
        steps (for short contexts; one for longer contexts is recorded when they are met, without measuring again)
        and of short steps of any other make are recorded. The reference records its graphs when the engine starts
        (nanovllm/engine/model_runner.py:2559-2594); here it is asked for: engine option ``warm_up``, or this call.
        ``batch_sizes``, ``token_counts``: the sizes to meet (default: all that the engine's limits allow).
        Returns what was recorded. Nothing of it stays in the cache."""
        runner = self.runner
        if not runner.use_graphs or self.scheduler.running or self.scheduler.waiting:
            return {"graphs_recorded": [], "mixed_graphs_recorded": []}
        most = min(self.config.max_num_seqs, runner.cache.num_free_slots(), runner.num_pages)
        sizes = [b for b in (batch_sizes or runner.graph_buckets) if b <= most]
        for b in sizes:
            ids = [("warm up", i) for i in range(b)]
            runner.step([StepEntry(r, [0], []) for r in ids])              # a first token each, then a step of single tokens
            runner.step([StepEntry(r, [0], [0]) for r in ids])
            for r in ids:
                runner.finish(r)
        counts = token_counts if token_counts is not None else runner.mixed_token_buckets
        for t in counts:
            if t <= min(runner.max_graph_tokens, runner.max_model_len, runner.num_pages * runner.page_size):
                runner.step([StepEntry(("warm up", 0), [0] * (t - 1), [t - 2])])   # (a bucket holds steps of fewer tokens than its size)
                runner.finish(("warm up", 0))
        stats = runner.get_memory_stats()
        return {key: stats[key] for key in ("graphs_recorded", "mixed_graphs_recorded")}

    # ------------------------------------------------------------------ requests
    def add_request(self, prompt, sampling_params: SamplingParams | None = None) -> int:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("a text prompt needs a tokenizer.json in the model folder; pass token ids instead")
            token_ids = self.tokenizer.encode(prompt).ids
        else:
            validate_token_ids(prompt)
            token_ids = list(prompt)
        vocab = self.runner.vocab_size
        for t in token_ids:
            if t >= vocab:
                raise ValueError(f"token id {t} is outside the vocabulary of {vocab}")
        seq = Sequence(next(self._ids), token_ids, sampling_params)
        self.scheduler.add(seq)
        self._sequences[seq.seq_id] = seq
        self._metrics[seq.seq_id] = RequestMetrics(seq.seq_id, seq.num_prompt_tokens, perf_counter())
        return seq.seq_id

    def is_finished(self) -> bool:
        return self.scheduler.is_finished()

    # ------------------------------------------------------------------ one step
    def step(self):
        """Plans, runs and finishes one step. Returns ([(seq_id, completion token ids)
        of the requests that finished], StepStats)."""
        t0 = perf_counter()
        plan = self.scheduler.schedule()
        seqs = plan.seqs
        num_prefill_tokens, num_decode_tokens = plan.num_prefill_tokens, plan.num_decode_tokens
        entries, sampled_rows = [], []
        for seq in seqs:
            n = seq.num_scheduled_tokens
            start = seq.num_cached_tokens
            ends = start + n == seq.num_tokens
            entries.append(StepEntry(seq.seq_id, seq.token_ids[start:start + n], [n - 1] if ends else []))
            if ends:
                sampled_rows.append(seq)
            m = self._metrics[seq.seq_id]
            if m.first_scheduled is None:
                m.first_scheduled = t0
        ids = [e.request_id for e in entries]
        ahead, self._ahead = self._ahead, None
        issued = False
        if ahead is not None:
            if num_prefill_tokens == 0 and set(ids) <= set(ahead["requests"]):
                # the step issued ahead is this one (a request that ended meanwhile had its row in it for nothing;
                # one that lives on but is not planned now takes its token back)
                self.runner.undo_ahead(ahead, set(ahead["requests"]) - set(ids))
                logits = self.runner.logits_ahead(ahead, ids)
                issued = True
                self.num_steps_ahead += 1
            else:
                self.runner.undo_ahead(ahead, set(ahead["requests"]))       # the plan is another: as if never issued
        if not issued:
            logits = self.runner.step(entries, keep=False)                  # sampled from at once
        tokens_by_id = {}
        if sampled_rows:
            seed = self.config.seed
            temps = [s.temperature for s in sampled_rows]
            keys = [noise_key(seed if s.seed is None else s.seed, s.seq_id, s.num_completion_tokens)
                    for s in sampled_rows]
            launched = self.sampler.launch(logits, temps, keys)
            # While the host waits for the tokens, ends this step and plans the next, the GPU would wait: if the
            # next step is bound to be these requests' next tokens (nothing waits, nobody reaches max_tokens; only
            # an end-of-sequence token can still end one), it is issued now, fed from the tokens on the device.
            if (self.config.run_ahead and num_prefill_tokens == 0 and len(sampled_rows) == len(seqs)
                    and not self.scheduler.waiting
                    and all(s.num_completion_tokens + 1 < s.max_tokens for s in seqs)
                    and self.runner.can_step_ahead(ids)):
                self._ahead = self.runner.step_ahead(ids, launched["tokens"])
            tokens = self.sampler.finish(launched)
            tokens_by_id = {s.seq_id: t for s, t in zip(sampled_rows, tokens)}
        finished = self.scheduler.postprocess(seqs, [tokens_by_id.get(s.seq_id) for s in seqs])
        now = perf_counter()
        for s in sampled_rows:
            m = self._metrics[s.seq_id]
            if m.first_token is None:
                m.first_token = now
        outputs = []
        for s in finished:
            m = self._metrics.pop(s.seq_id)
            m.finished = now
            m.num_completion_tokens = s.num_completion_tokens
            self._completed_metrics.append(m)
            self._sequences.pop(s.seq_id, None)
            outputs.append((s.seq_id, s.completion_token_ids))
        stats = StepStats(num_prefill_tokens=num_prefill_tokens, num_decode_tokens=num_decode_tokens,
                          seconds=now - t0, num_preempted=len(plan.preempted_seq_ids))
        return outputs, stats

    # ------------------------------------------------------------------ many prompts
    def generate(self, prompts: list, sampling_params: SamplingParams | list[SamplingParams],
                 use_tqdm: bool = True) -> list[dict]:
        if not isinstance(sampling_params, list):
            sampling_params = [sampling_params] * len(prompts)
        if len(sampling_params) != len(prompts):
            raise ValueError(f"{len(prompts)} prompts but {len(sampling_params)} sampling_params")
        pbar = None
        if use_tqdm:
            from tqdm.auto import tqdm
            pbar = tqdm(total=len(prompts), desc="Generating", dynamic_ncols=True)
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, sampling_params)]
        outputs = {}
        prefill_tp = decode_tp = 0.0
        while not self.is_finished():
            done, stats = self.step()
            if stats.num_prefill_tokens:
                prefill_tp = stats.prefill_throughput
            if stats.num_decode_tokens:
                decode_tp = stats.decode_throughput
            for seq_id, token_ids in done:
                outputs[seq_id] = token_ids
                if pbar is not None:
                    pbar.update(1)
            if pbar is not None:
                pbar.set_postfix({"Prefill": f"{int(prefill_tp)}tok/s", "Decode": f"{int(decode_tp)}tok/s"})
        if pbar is not None:
            pbar.close()
        result = []
        for seq_id in ids:
            token_ids = outputs[seq_id]
            text = self.tokenizer.decode(token_ids) if self.tokenizer is not None else None
            result.append({"text": text, "token_ids": token_ids})
        return result

    def get_memory_stats(self) -> dict:
        stats = self.runner.get_memory_stats()
        stats["gemm_choices"] = self.gemm_choices()
        return stats

    def get_completed_request_metrics(self) -> list[RequestMetrics]:
        out, self._completed_metrics = self._completed_metrics, []
        return out

    def exit(self) -> None:
        """Lets go of the model and the cache."""
        self.runner = None
        self.scheduler = None
