"""The Python entry point: add requests, step, generate (reference engine/llm_engine.py:11-64 for the
names and meanings of the calls)."""
from __future__ import annotations

import os
import sys
import time

import torch

from ..cache.manager import CacheManager
from ..cache.pool import page_bytes
from ..config.engine_config import EngineConfig
from ..sampling.sampler import Sampler
from ..sampling.sampling_params import SamplingParams
from ..weights.loader import load_model
from .request import Request
from .runner import ModelRunner, StepEntry
from .scheduler import UNKNOWN, Scheduler

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

    def __init__(self, sampling, places, handle, num_prefill, num_decode):
        self.sampling, self.places, self.handle = sampling, places, handle
        self.num_prefill, self.num_decode = num_prefill, num_decode


class _Progress:
    """Finished requests and the last step's rate on one line of stderr (through tqdm where it is installed)."""

    def __init__(self, total: int, enabled: bool):
        self.bar = None
        if enabled:
            try:
                from tqdm.auto import tqdm
                self.bar = tqdm(total=total, desc="Generating", dynamic_ncols=True, file=sys.stderr)
            except Exception:
                self.bar = None

    def step(self, finished: int, prompt_tokens: int, decoded: int, seconds: float) -> None:
        if self.bar is None:
            return
        rate = (prompt_tokens + decoded) / seconds if seconds > 0 else 0.0
        self.bar.set_postfix_str(f"prompt tokens {prompt_tokens}, decoding {decoded}, {rate:.0f} tok/s", refresh=False)
        self.bar.update(finished)

    def close(self) -> None:
        if self.bar is not None:
            self.bar.close()


class LLMEngine:
    def __init__(self, model: str, **options):
        """`options`: any field of EngineConfig (the reference's option names among them); beside those
        `device` and, for tests, `poison_cache`. Unknown names are ignored, as the reference does."""
        config = EngineConfig.from_options(model, options)
        self.config = config
        self.device = torch.device(options.get("device", "cuda"))
        self.dtype = _DTYPES[config.dtype]
        self.model = load_model(config.model, self.device, self.dtype, config.max_model_len, config.model_config,
                                random_weights=config.random_weights)
        plan = self.model.cache_plan()
        self._state_slots = config.max_num_seqs if any(s is not None for s in plan.state_needs) else 0
        self.reserved_bytes = 0
        if config.num_kvcache_blocks <= 0:
            config.num_kvcache_blocks = self._size_pool(plan)
        self.manager = CacheManager(config.num_kvcache_blocks, config.kvcache_block_size,
                                    ModelRunner.windows_of(self.model), num_state_slots=self._state_slots,
                                    enable_prefix_caching=config.enable_prefix_caching)
        self.runner = ModelRunner(self.model, self.manager, self.dtype, self.device, config.max_model_len,
                                  poison_cache=bool(options.get("poison_cache", False)),
                                  use_graphs=config.use_graphs, max_decode_rows=config.max_num_seqs)
        self.tokenizer = _load_tokenizer(config.model)
        self.scheduler = Scheduler(config, self.manager)
        self.sampler = Sampler(self.runner, config.seed)
        self.run_ahead = bool(config.run_ahead)
        self._in_flight = None
        self._ending = []            # requests of the last settled step that may still hold pages
        self.steps_run_ahead = 0

    def _size_pool(self, plan) -> int:
        """Pages per group from what the device has free after the engine's two largest steps have run
        once on a one-page pool (reference engine/model_runner.py:59-80: a warm-up with the largest
        prompt step and the largest decode step, then the pool from the allocator's peak).

        Kept free beside the pool: the measured peak of the larger of the two steps (activations,
        attention scratch; the library's workspace is allocated by then and counts as used), and for
        the captured graphs their memory pool (a captured step needs what the eager one needs: the same
        peak once more) and the logits buffer."""
        cfg = self.config
        if self.device.type != "cuda":
            raise RuntimeError("the cache pool can be sized from free memory only on a GPU: give num_kvcache_blocks")
        probe_manager = CacheManager(1, cfg.kvcache_block_size, ModelRunner.windows_of(self.model),
                                     num_state_slots=self._state_slots, enable_prefix_caching=False)
        probe = ModelRunner(self.model, probe_manager, self.dtype, self.device, cfg.max_model_len)
        step_peak, decode_peak = probe.measure_working_set(cfg.max_num_batched_tokens, cfg.max_num_seqs, cfg.max_model_len)
        del probe, probe_manager
        torch.cuda.empty_cache()
        vocab = getattr(self.model.embedding, "vocab_size", 0)
        graphs = step_peak + (cfg.max_num_seqs + 128) * vocab * 4 if cfg.use_graphs else 0
        self.reserved_bytes = step_peak + graphs
        free, total = torch.cuda.mem_get_info(self.device)
        budget = int(total * cfg.gpu_memory_utilization) - (total - free) - self.reserved_bytes
        per_page = sum(page_bytes(plan, cfg.kvcache_block_size, self.dtype))
        most = -(-cfg.max_model_len // cfg.kvcache_block_size) * cfg.max_num_seqs   # more can never be held
        pages = min(budget // max(1, per_page), most)
        if pages <= 0:
            raise RuntimeError("the engine's largest step leaves no memory for the cache: lower max_num_seqs / "
                               "max_num_batched_tokens or raise gpu_memory_utilization")
        return int(pages)

    # -- requests ----------------------------------------------------------------------------
    def add_request(self, prompt, sampling_params: SamplingParams, priority: int = 0,
                    sample_stream: int | None = None) -> int:
        """Queue a prompt (text, if the folder has a tokenizer, or token ids); returns the request's id."""
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("this model folder has no tokenizer.json: give prompts as lists of token ids")
            prompt = self.tokenizer.encode(prompt).ids
        req = Request(prompt, sampling_params, priority, sample_stream)
        self.scheduler.add(req)
        return req.id

    def step(self):
        """One scheduler step. Returns (finished [(request id, generated ids)], prompt tokens run,
        decode requests run, ids of the requests that got a token).

        With `run_ahead`, while the requests only decode, the next step is launched before this one's
        tokens are fetched (it takes them from the device), so the GPU does not wait for the host's
        bookkeeping. A request that samples its end token then runs one step too far; that token is dropped."""
        current = self._in_flight or self._launch()
        self._in_flight = None
        if (self.run_ahead and current.num_prefill == 0 and self.runner.graphs is not None
                and self.scheduler.next_step_is_plain_decoding()
                and self.runner.graphs.takes(len(self.scheduler.running))):
            self._in_flight = self._launch()
            self.steps_run_ahead += 1
        return self._settle(current)

    def _launch(self) -> _Launched:
        reqs = self.scheduler.schedule()
        # single-token requests first (as the scheduler has them), the longest context first among them:
        # the decode kernel starts its workgroups in row order, and a long context that starts last is
        # what the launch then waits for (256 contexts of 100-2,048 keys: 224 us as drawn, 206 us sorted).
        # Requests that decode together keep their order from step to step, so rows stay where they are.
        reqs.sort(key=lambda r: -(r.in_cache + 1) if r.portion == 1 else 1)
        num_decode = num_prefill = 0
        entries, places = [], []
        for r in reqs:
            first, n = r.in_cache, r.portion
            if n == 1:
                num_decode += 1
            else:
                num_prefill += n
            samples = first + n == len(r.tokens)
            if samples:
                places.append(first + n)
            entries.append(StepEntry(r.id, r.tokens[first:first + n], first, [n - 1] if samples else []))
        logits = self.runner.step(entries)
        sampling = [r for r, e in zip(reqs, entries) if e.want]
        handle = self.sampler.launch(logits, sampling) if sampling else None
        self.scheduler.advance(reqs)
        return _Launched(sampling, places, handle, num_prefill, num_decode)

    def _settle(self, step: _Launched):
        tokens = step.handle.tokens() if step.handle is not None else []
        got = self.scheduler.settle(step.sampling, tokens, step.places)
        # what ended requests hold goes back once no launched step writes to their pages any more:
        # those of the step before this one now, this one's at once unless a step is already in flight
        self.scheduler.release_finished(self._ending)
        self._ending = step.sampling if self._in_flight is not None else []
        if self._in_flight is None:
            self.scheduler.release_finished(step.sampling)
        # a request that ends by max_tokens is marked done when its last step is launched; it is
        # reported when that step's token has arrived, not with the token before it
        finished = [(r.id, r.generated) for r in got if r.done and r.tokens[-1] != UNKNOWN]
        return finished, step.num_prefill, step.num_decode, [r.id for r in got]

    def is_finished(self) -> bool:
        return self._in_flight is None and self.scheduler.is_finished()

    def generate(self, prompts: list, sampling_params, use_tqdm: bool = True, priorities: list | None = None) -> list:
        """Run all prompts (strings or lists of token ids) to completion; one {"text", "token_ids"} per
        prompt, in the order given. `sampling_params`: one for all, or one per prompt; `priorities`: one
        per prompt, lower first under the priority policy."""
        count = len(prompts)
        params = sampling_params if isinstance(sampling_params, list) else [sampling_params] * count
        ranks = priorities if priorities else [0] * count
        if len(params) != count or len(ranks) != count:
            raise ValueError("one SamplingParams (or one priority) per prompt, or a single one for all")
        # the place of a prompt in this call keys its sampling noise: results do not depend on earlier traffic
        place_of = {self.add_request(prompt, params[i], ranks[i], sample_stream=i): i for i, prompt in enumerate(prompts)}
        results = [None] * count
        progress = _Progress(count, use_tqdm)
        try:
            while not self.is_finished():
                began = time.perf_counter()
                finished, num_prefill, num_decode, _ = self.step()
                for request_id, token_ids in finished:
                    if request_id in place_of:
                        text = self.tokenizer.decode(token_ids, skip_special_tokens=True) if self.tokenizer else ""
                        results[place_of[request_id]] = {"text": text, "token_ids": token_ids}
                progress.step(len(finished), num_prefill, num_decode, time.perf_counter() - began)
        finally:
            progress.close()
        return results
