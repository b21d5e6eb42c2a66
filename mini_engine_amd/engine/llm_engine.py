"""The Python entry point: add requests, step, generate (reference engine/llm_engine.py:11-64)."""
from __future__ import annotations

import os
from dataclasses import fields
from time import perf_counter

import torch

from ..cache.manager import CacheManager
from ..cache.pool import page_bytes
from ..config.engine_config import EngineConfig
from ..sampling.sampler import Sampler
from ..sampling.sampling_params import SamplingParams
from ..weights.loader import load_model
from .runner import ModelRunner, StepEntry
from .scheduler import Scheduler
from .sequence import Sequence

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def _load_tokenizer(model_dir: str):
    """The folder's tokenizer.json, if it has one; ids-in/ids-out works without."""
    path = os.path.join(model_dir, "tokenizer.json")
    if not os.path.isfile(path):
        return None
    try:
        from tokenizers import Tokenizer
        return Tokenizer.from_file(path)
    except Exception:
        return None


class _Launched:
    """A step that has been launched: who samples, where their tokens go, and the handle that fetches them."""

    def __init__(self, samplers, index_of, handle, num_prefill, num_decode):
        self.samplers, self.index_of, self.handle = samplers, index_of, handle
        self.num_prefill, self.num_decode = num_prefill, num_decode


class LLMEngine:
    def __init__(self, model: str, **kwargs):
        names = {f.name for f in fields(EngineConfig)}
        config = EngineConfig(model, **{k: v for k, v in kwargs.items() if k in names})
        self.config = config
        self.device = torch.device(kwargs.get("device", "cuda"))
        self.dtype = _DTYPES[config.dtype]
        self.model = load_model(config.model, self.device, self.dtype, config.max_model_len, config.model_config)
        plan = self.model.cache_plan()
        has_state = any(s is not None for s in plan.state_needs)
        if config.num_kvcache_blocks <= 0:
            config.num_kvcache_blocks = self._size_pool(plan)
        self.manager = CacheManager(config.num_kvcache_blocks, config.kvcache_block_size,
                                    ModelRunner.windows_of(self.model),
                                    num_state_slots=config.max_num_seqs if has_state else 0,
                                    enable_prefix_caching=config.enable_prefix_caching)
        self.runner = ModelRunner(self.model, self.manager, self.dtype, self.device, config.max_model_len,
                                  poison_cache=bool(kwargs.get("poison_cache", False)),
                                  use_graphs=config.use_graphs)
        self.tokenizer = _load_tokenizer(config.model)
        self.scheduler = Scheduler(config, self.manager)
        self.sampler = Sampler(self.runner, config.seed)
        self.run_ahead = bool(config.run_ahead)
        self._in_flight = None
        self._finishing = []
        self.steps_run_ahead = 0

    @classmethod
    def from_parts(cls, config, model, manager, runner, tokenizer=None):
        """An engine around an already loaded model and its runner (benchmarks that build random
        weights in memory). `config` needs the scheduler's fields and `seed`."""
        self = cls.__new__(cls)
        self.config, self.model, self.manager, self.runner = config, model, manager, runner
        self.device, self.dtype, self.tokenizer = runner.device, runner.dtype, tokenizer
        self.scheduler = Scheduler(config, manager)
        self.sampler = Sampler(runner, config.seed)
        self.run_ahead = bool(getattr(config, "run_ahead", True))
        self._in_flight = None
        self._finishing = []
        self.steps_run_ahead = 0
        return self

    def _size_pool(self, plan) -> int:
        """Pages per group from the memory that is free now (reference engine/model_runner.py:69-80
        sizes from a measured warm-up peak; here the step's working set is estimated instead)."""
        cfg = self.config
        free, total = torch.cuda.mem_get_info(self.device)
        item = torch.empty((), dtype=self.dtype).element_size()
        widths = sum(int(torch.tensor(spec.shape).prod()) // spec.shape[1]
                     for _, _, _, spec in self.model.named_specs() if len(spec.shape) == 2) // max(1, len(self.model.layers))
        vocab = getattr(self.model.embedding, "vocab_size", 0)
        working = cfg.max_num_batched_tokens * widths * item * 2 + 2 * cfg.max_num_seqs * vocab * 4 + (256 << 20)
        budget = int(total * cfg.gpu_memory_utilization) - (total - free) - working
        per_page = sum(page_bytes(plan, cfg.kvcache_block_size, self.dtype))
        pages = budget // max(1, per_page)
        most = -(-cfg.max_model_len // cfg.kvcache_block_size) * cfg.max_num_seqs   # more can never be held
        pages = min(pages, most)
        if pages <= 0:
            raise RuntimeError("no memory left for the cache: lower max_num_seqs / max_num_batched_tokens "
                               "or raise gpu_memory_utilization")
        return int(pages)

    # -- requests ----------------------------------------------------------------------------
    def add_request(self, prompt, sampling_params: SamplingParams, priority: int = 0,
                    sample_stream: int | None = None) -> int:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("this model folder has no tokenizer.json: give prompts as lists of token ids")
            prompt = self.tokenizer.encode(prompt).ids
        seq = Sequence(prompt, sampling_params, priority, sample_stream)
        self.scheduler.add(seq)
        return seq.seq_id

    def step(self):
        """One scheduler step. Returns (finished [(seq_id, completion ids)], prefill tokens run,
        decode requests run, ids of the requests that got a token).

        With `run_ahead`, while the requests only decode, the next step is launched before this one's
        tokens are fetched (it takes them from the device), so the GPU does not wait for the host's
        bookkeeping. A request that samples its end token then runs one step too far; that token is dropped."""
        if self._in_flight is None:
            self._in_flight = self._launch()
        current = self._in_flight
        self._in_flight = None
        if (self.run_ahead and current.num_prefill == 0 and self.runner.graphs is not None
                and self.scheduler.next_step_is_plain_decoding()
                and self.runner.graphs.takes(len(self.scheduler.running))):
            self._in_flight = self._launch()
            self.steps_run_ahead += 1
        return self._settle(current)

    def _launch(self):
        seqs = self.scheduler.schedule()
        # single-token requests first (as the scheduler has them), the longest context first among them:
        # the decode kernel starts its workgroups in row order, and a long context that starts last is
        # what the launch then waits for (256 contexts of 100-2,048 keys: 224 us as drawn, 206 us sorted).
        # Requests that decode together keep their order from step to step, so rows stay where they are.
        seqs.sort(key=lambda s: -(s.num_computed_tokens + 1) if s.num_scheduled_tokens == 1 else 1)
        num_decode = num_prefill = 0
        entries, index_of = [], []
        for s in seqs:
            a, n = s.num_computed_tokens, s.num_scheduled_tokens
            if n == 1:
                num_decode += 1
            else:
                num_prefill += n
            samples = a + n == len(s.token_ids)
            if samples:
                index_of.append(a + n)
            entries.append(StepEntry(s.seq_id, s.token_ids[a:a + n], a, [n - 1] if samples else []))
        logits = self.runner.step(entries)
        samplers = [s for s, e in zip(seqs, entries) if e.want]
        handle = self.sampler.launch(logits, samplers) if samplers else None
        self.scheduler.advance(seqs)
        return _Launched(samplers, index_of, handle, num_prefill, num_decode)

    def _settle(self, step):
        tokens = step.handle.tokens() if step.handle is not None else []
        emitted = self.scheduler.settle(step.samplers, tokens, step.index_of)
        # what finished requests hold goes back once no launched step writes to their pages any more:
        # those of the step before this one now, this one's at once unless a step is already in flight
        self.scheduler.release_finished(self._finishing)
        self._finishing = step.samplers if self._in_flight is not None else []
        if self._in_flight is None:
            self.scheduler.release_finished(step.samplers)
        # a request that ends by max_tokens is marked finished when its last step is launched; it is
        # reported when that step's token has arrived, not with the token before it
        outputs = [(s.seq_id, s.completion_token_ids) for s in emitted
                   if s.is_finished and s.token_ids[-1] != Scheduler.PLACEHOLDER]
        return outputs, step.num_prefill, step.num_decode, [s.seq_id for s in emitted]

    def is_finished(self) -> bool:
        return self._in_flight is None and self.scheduler.is_finished()

    def generate(self, prompts: list, sampling_params, use_tqdm: bool = True, priorities: list | None = None) -> list:
        """Run all prompts (strings or lists of token ids) to completion; results in submission
        order as {"text", "token_ids"}."""
        if not isinstance(sampling_params, list):
            sampling_params = [sampling_params] * len(prompts)
        priorities = priorities or [0] * len(prompts)
        ids = [self.add_request(p, sp, prio, sample_stream=i)
               for i, (p, sp, prio) in enumerate(zip(prompts, sampling_params, priorities))]
        pbar = None
        if use_tqdm:
            try:
                from tqdm.auto import tqdm
                pbar = tqdm(total=len(prompts), desc="Generating", dynamic_ncols=True)
            except Exception:
                pbar = None
        outputs = {}
        while not self.is_finished():
            t = perf_counter()
            out, num_prefill, num_decode, _ = self.step()
            dt = perf_counter() - t
            if pbar is not None:
                pbar.set_postfix({"prefill": num_prefill, "decode": num_decode,
                                  "tok/s": f"{(num_prefill + num_decode) / dt:.0f}"})
            for seq_id, toks in out:
                outputs[seq_id] = toks
                if pbar is not None:
                    pbar.update(1)
        if pbar is not None:
            pbar.close()
        result = []
        for seq_id in ids:
            toks = outputs[seq_id]
            text = self.tokenizer.decode(toks, skip_special_tokens=True) if self.tokenizer is not None else ""
            result.append({"text": text, "token_ids": toks})
        return result
