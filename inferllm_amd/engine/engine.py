"""The engine: a model folder (or a configuration and a seed) in, logits and
generated tokens out, on one GPU.

Python entry point of the library, in the role of the reference's `Model` facade
(include/model.h:27-59: load, init, prefill, decode, decode_iter, reset_token,
decode_summary) with batches of sequences in place of its single one.
"""
from __future__ import annotations

import warnings
from typing import Dict, List, Optional, Sequence, Union

import torch

from ..kernels import ops
from ..kernels.plan import Plan
from ..cache.manager import PAGE_SIZE, CacheManager, round_up
from ..cache.slots import CacheError, CacheFull
from ..config.registry import config_from_dict, load_config
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from ..weights.loader import load_named_tensors
from ..weights.random_init import random_tensors
from .generate import GenerationLoop, GenerationStats
from .model import DecoderModel
from .step import StepEntry, StepRunner

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16,
           torch.float32: torch.float32, torch.bfloat16: torch.bfloat16}


def parse_dtype(dtype) -> torch.dtype:
    """"float32" or "bfloat16" (the reference's strings are src/core/model_imp.h:17-33)."""
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {dtype!r}: use 'float32' or 'bfloat16'") from None


class Engine:
    """One model on one GPU with its cache, step function and generation loop.

    dtype "bfloat16": bfloat16 matrices, activations and cache, float32 residual
    stream, statistics and logits.  dtype "float32": everything in true
    float32 (own kernels: float32 operands, products and sums; no reduced-precision mode).

    `decode_copies`: keep a second copy of every matrix in the layout of the few-rows kernels
    (decoding reads that one, prompts the row-major one), or with "thin" of the down projections
    alone; default: all if they fit comfortably, else the thin ones if those do.

    `tune`, `plan`: some bfloat16 products have several equivalent ways that differ in speed by
    shape and in rounding.  By default the way is taken from fixed tables (`kernels.plan`), so the
    same request gives the same bits in every process and nothing is timed.  `tune=True` times
    the ways for shapes the tables lack (thin matrices now, many-row products at first use) and
    keeps the winners in `engine.plan`; `plan=` (a `Plan` or what its `to_dict()` gave) pins them.

    `step_rows`: a cache line that keeps a window of keys is a ring of pages with room for the
    window and this many rows more; a sequence that goes on from earlier tokens by more than
    that in one step has the step run in pieces.  Models without windows ignore it.

    Cache size: `max_tokens` is the most tokens live sequences hold together (each
    rounded up to 64), `max_batch` the most live sequences, `max_seq_len` the longest
    sequence (default: the model's max positions).
    """

    def __init__(self, config, tensors: Dict[str, torch.Tensor], dtype, device="cuda:0",
                 max_batch: int = 8, max_seq_len: Optional[int] = None,
                 max_tokens: Optional[int] = None, use_graphs: bool = True,
                 poison_freed: bool = False, decode_copies=None, tune: bool = False, plan=None,
                 step_rows: int = 512):
        self.config = config
        self.dtype = parse_dtype(dtype)
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise ValueError("the engine runs on a GPU only (device 'cuda:N')")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible; the engine has no CPU path")
        torch.cuda.set_device(self.device)
        self.spec = config.to_spec()
        self.model = DecoderModel(self.spec)
        if decode_copies is None:
            # a second copy of the matrices, laid out for the few-rows kernels of decoding, if it
            # takes no more than a quarter of the memory that is free now; else of the long thin
            # ones alone (the down projections) if that takes no more than a third
            sizes = [(t.numel() * t.element_size(), t.shape) for t in tensors.values() if t.dim() == 2]
            free, _total = torch.cuda.mem_get_info(self.device)
            thin = sum(n for n, shape in sizes if shape[1] >= 2 * shape[0])
            if self.dtype != torch.bfloat16:
                decode_copies = False
            elif sum(n for n, _ in sizes) <= free // 4:
                decode_copies = True
            else:
                decode_copies = "thin" if 0 < thin <= free // 3 else False
        if self.dtype != torch.bfloat16:
            decode_copies = False
        self.decode_copies = decode_copies if decode_copies == "thin" else bool(decode_copies)
        self.model.load(tensors, decode_copies=self.decode_copies)
        if isinstance(plan, dict):
            plan = Plan.from_dict(plan)
        self.plan: Plan = plan if plan is not None else Plan.fixed(measure=bool(tune))
        if self.plan.measure and self.dtype == torch.bfloat16:
            # what each part lists as having several ways (`Part.tunables`); the engine knows no
            # part's fields
            for part in self.model.every_part():
                for kind, w, geometry in part.tunables():
                    ops.tune_product(self.plan, kind, w, **geometry)
        limit = self.spec.max_positions
        self.max_seq_len = min(int(max_seq_len), limit) if max_seq_len else limit
        self.max_batch = int(max_batch)
        if max_tokens is None:
            max_tokens = self.max_batch * round_up(self.max_seq_len, PAGE_SIZE)
        self.cache = CacheManager(self.model.kv_lines(), self.model.state_lines(),
                                  max_tokens=int(max_tokens), max_slots=self.max_batch,
                                  max_seq_len=self.max_seq_len, dtype=self.dtype,
                                  device=self.device, poison_freed=poison_freed,
                                  step_rows=int(step_rows))
        self.runner = StepRunner(self.model, self.cache, self.dtype, self.device, use_graphs,
                                 plan=self.plan)
        self.last_stats: Optional[GenerationStats] = None

    # ------------------------------------------------------------ construction
    @classmethod
    def from_pretrained(cls, model_dir: str, dtype="bfloat16", device="cuda:0",
                        keep_stored: bool = False, **kw) -> "Engine":
        """From a folder with config.json and model.safetensors (or its shards).

        Matrices take the engine's dtype as they are loaded, whatever the file stores them in
        (float16 and float32 are rounded to bfloat16, to nearest even, in a bfloat16 engine; the
        reference gives a tensor the runtime type of its file code, src/core/graph.cpp:216-231).
        `keep_stored=True` keeps 32-bit and float16 matrices as float32 instead: their products
        then run on the float32 multiply-add kernel, at twice the memory and a fraction of the
        speed (a warning says so)."""
        config = load_config(model_dir)
        model = DecoderModel(config.to_spec())
        dt = parse_dtype(dtype)
        tensors = load_named_tensors(model_dir, model.wants(), dt, device,
                                     config.to_spec().ignored_tensor_suffixes, keep_stored)
        if keep_stored and dt == torch.bfloat16:
            wide = [n for n, t in tensors.items() if t.dim() == 2 and t.dtype == torch.float32]
            if wide:
                warnings.warn(f"{len(wide)} matrices stay float32 in a bfloat16 engine "
                              f"(keep_stored): their products run on the float32 kernel, not on "
                              f"the matrix cores")
        return cls(config, tensors, dtype, device, **kw)

    @classmethod
    def from_random(cls, config: Union[dict, object], seed: int = 0, dtype="bfloat16",
                    device="cuda:0", **kw) -> "Engine":
        """Seeded random weights drawn on the device (no folder is written)."""
        if isinstance(config, dict):
            config = config_from_dict(config)
        dt = parse_dtype(dtype)
        wants = DecoderModel(config.to_spec()).wants()
        tensors = dict(random_tensors(wants, seed, dt, device))
        return cls(config, tensors, dtype, device, **kw)

    # ------------------------------------------------------------ low level
    def alloc_slot(self) -> int:
        return self.cache.alloc_slot()

    def free_slot(self, slot: int) -> None:
        self.cache.free_slot(slot)

    def step(self, entries: Sequence[StepEntry], device_tokens: Optional[torch.Tensor] = None,
             borrow: bool = False) -> Optional[torch.Tensor]:
        """See `StepRunner.step`.  The returned tensor is the caller's; with `borrow` it may be
        memory that the next step writes again."""
        return self.runner.step(entries, device_tokens, borrow)

    def generation_loop(self, sampler: Sampler, on_token=None, max_step_tokens: Optional[int] = None,
                        ahead: bool = True) -> GenerationLoop:
        """The generation loop over this engine's step function, cache and `sampler`.  `ahead`:
        every step is started before the tokens of the step before it have been read."""
        step = lambda entries, device_tokens=None: self.runner.step(entries, device_tokens, borrow=True)
        return GenerationLoop(step, sampler, self.alloc_slot, self.free_slot,
                              max_batch=self.max_batch, max_tokens=self.cache.max_tokens,
                              max_seq_len=self.max_seq_len, page_size=self.cache.page_size,
                              sync=lambda: torch.cuda.synchronize(self.device), on_token=on_token,
                              draw=sampler.draw if ahead else None, max_step_tokens=max_step_tokens,
                              keep=lambda logits, row: logits[row].clone(), join=torch.stack,
                              rewind_slot=self.cache.rewind)

    def session(self, temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0,
                repeat_penalty: float = 1.0, repeat_last_n: int = 64, seed: int = 0,
                stop_token_ids: Optional[Sequence[int]] = None):
        """A conversation in one slot of the cache: `say(tokens)` feeds a turn after everything
        said so far and returns the answer, as the reference's chat keeps one context over its
        turns (application/chat.cpp:221-275).  Close it (or use it in a `with`) to give the slot
        back."""
        from .session import Session
        params = SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p,
                                repeat_penalty=repeat_penalty, repeat_last_n=repeat_last_n, seed=seed)
        return Session(self, params, stop_token_ids)

    def warm_up(self, batch_sizes: Optional[Sequence[int]] = None, longest: int = 1,
                prompt_tokens: int = 0) -> int:
        """Capture the decode graphs for these numbers of sequences (default: every size up to
        `max_batch` that has a graph of its own) with contexts up to `longest` keys, so that the
        first decode step of such a batch does not pay for the capture.  `prompt_tokens` > 0: also
        run a throwaway prompt of that many tokens in a slot that is given back at once, so that
        the first request does not pay for what a first prompt step sets up (at the LLaMA-2-7B
        sizes 200 ms against 10).  Returns how many graphs were captured."""
        if batch_sizes is None:
            batch_sizes = range(1, self.max_batch + 1)
        captured = self.runner.warm_up(batch_sizes, min(int(longest), self.max_seq_len))
        n = min(int(prompt_tokens), self.max_seq_len)
        if n > 0:
            try:
                slot = self.alloc_slot()
            except CacheError:
                return captured                  # every slot is in use: nothing to warm up with
            try:
                self.step([StepEntry(slot, [0] * n, [n - 1])])
            except CacheFull:
                pass                             # no room for a throwaway prompt now: skipped
            finally:
                self.free_slot(slot)
        return captured

    # ------------------------------------------------------------ generation
    def generate(self, prompts: Sequence[Sequence[int]], temperature: float = 0.0,
                 top_k: int = 0, top_p: float = 1.0, repeat_penalty: float = 1.0,
                 repeat_last_n: int = 64, seed: int = 0, max_new_tokens: int = 128,
                 stop_token_ids: Optional[Sequence[int]] = None,
                 include_stop: bool = False, on_token=None,
                 max_step_tokens: Optional[int] = None) -> List[List[int]]:
        """Generated token ids for every prompt (lists of token ids).

        `max_step_tokens`: most tokens a step of prompts may hold; a batch's prompts are then fed
        in several steps (models whose mixers can go on from the cache by several tokens).

        `stop_token_ids` defaults to the model's eos ids; a stop token ends its
        sequence and is left out of the result unless `include_stop`.  `on_token(request
        index, token)` is called for every token as it is generated (the reference prints
        tokens as they come, application/chat.cpp:232-236)."""
        params = SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p,
                                repeat_penalty=repeat_penalty, repeat_last_n=repeat_last_n,
                                seed=seed)
        sampler = Sampler(params, self.device)
        stops = list(self.spec.eos_token_ids) if stop_token_ids is None else list(stop_token_ids)
        vocab = self.spec.vocab_size
        for i, p in enumerate(prompts):
            for t in p:
                if not (0 <= int(t) < vocab):
                    raise ValueError(f"request {i}: token id {t} outside the vocabulary of {vocab}")
        if max_step_tokens is not None and self.model.one_token_mixers:
            raise ValueError("max_step_tokens: this model's " + ", ".join(self.model.one_token_mixers)
                             + " cannot go on from the cache by several tokens")
        loop = self.generation_loop(sampler, on_token, max_step_tokens)
        out = loop.run(prompts, params, max_new_tokens, stops, include_stop)
        self.last_stats = loop.stats
        return out
