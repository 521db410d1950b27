"""The Python entry point: a model folder (or a configuration and a seed) in, tokens out.

Named after the reference's binding (pytorch/src/mini_llm/native.py): ``EngineOptions``, an
engine object that is a context manager, ``forward_last``, sessions with ``prefill`` /
``decode``, and the four calls its scheduler drives (``try_take_cache``, ``release_cache``,
``prefill_greedy``, ``decode_batch``: pytorch/src/mini_llm/batch_api.py:33-70). Above them sits
this framework's own scheduler with ``submit`` / ``step`` / ``generate``."""

from __future__ import annotations

import collections
from dataclasses import dataclass

import numpy as np

from ..sampling import SamplingParams
from .batch import StepEntry
from .loading import DEFAULT_PAGE_SIZE, load_model, make_cache, random_model, tokens_for_memory
from .scheduler import Request, Scheduler
from .step import ModelRunner


@dataclass(frozen=True)
class EngineOptions:
    """How the engine is sized. ``max_sessions`` is the reference's name for the number of
    requests that can be live at once (native.py:31-38)."""

    dtype: str = "bfloat16"
    max_sessions: int = 64
    max_tokens: int | None = None        # cache capacity in tokens; None: max_sessions full contexts
    cache_gib: float | None = None       # or the capacity as memory: GiB of page pools (an MI355X has 288 GB to give)
    page_size: int = DEFAULT_PAGE_SIZE
    max_length: int | None = None        # longest sequence a request may reach: needed for a model without a position limit of its own, and narrows a model's own
    max_tokens_per_step: int = 2048      # token budget of one scheduler step
    use_graphs: bool = True              # replay decode steps from captured HIP graphs
    portion_graph_after: int | None = None   # a shape of batch with prompt portions is captured when it comes this often (None: the step function's default; 0: never)
    decode_lanes_from: int | None = None     # captured decode steps of at least so many requests run two halves of them side by side (None: the step function's default; 0: never)
    step_ahead: bool = True              # the scheduler launches a step before it has read the one before
    device: str = "cuda:0"


class _Executor:
    """The scheduler's view of the runner, the cache and the sampler."""

    def __init__(self, engine: "Engine"):
        self._engine = engine
        self.page_size = engine.cache.page_size

    def max_positions(self):
        """The longest sequence a request may reach: the model's own limit or the one the cache was made for."""
        return self._engine.runner.longest_sequence()

    def check_prompt(self, tokens):
        limit, vocab = self.max_positions(), self._engine.model.vocab_size
        if limit is not None and len(tokens) > limit:
            raise ValueError(f"the prompt has {len(tokens)} tokens; the model holds {limit}")
        try:
            array = np.asarray(tokens)
            if array.ndim == 1 and array.dtype.kind in "iu" and (array.size == 0 or (0 <= int(array.min()) and int(array.max()) < vocab)):
                return
        except (ValueError, TypeError, OverflowError):
            pass
        for token in tokens:   # something is wrong: token by token, to name it
            if not 0 <= int(token) < vocab:
                raise ValueError(f"token {token} is outside the vocabulary [0, {vocab})")

    def can_open(self):
        return self._engine.cache.can_open()

    def open(self, request_id):
        self._engine.cache.open(("scheduled", request_id))

    def close(self, request_id):
        self._engine.cache.close(("scheduled", request_id))

    def length(self, request_id):
        return self._engine.cache.length(("scheduled", request_id))

    def pages_needed(self, request_id, n_new):
        return self._engine.cache.pages_needed(("scheduled", request_id), n_new)

    def free_pages(self):
        return self._engine.cache.free_pages()

    def run(self, entries, sampling, steps):
        return self.collect(self.launch(entries, sampling, steps))

    # One step ahead: launch() queues the step, the sampling (each token also goes to its request's
    # last-token slot, where the next step finds it) and the copy of the tokens into pinned host
    # memory; collect() waits for that copy alone, not for what was launched after it.
    def launch(self, entries, sampling, steps):
        engine = self._engine
        entries = [StepEntry(("scheduled", e.request_id), e.tokens, e.want, e.from_slot) for e in entries]
        # the tokens are chosen inside the step, greedily or as each row's parameters say
        return engine.runner.step(entries, choose=True, sampling=(sampling, steps))

    def collect(self, handle):
        return [] if handle is None else handle.tolist()


class Session:
    """One sequence driven by hand: prefill a prompt (in one or several portions), then decode
    token by token; each call returns the logits after its last token (the reference's
    CachedSession, native.py:88-166)."""

    def __init__(self, engine: "Engine", handle):
        self._engine, self._handle = engine, handle

    def _active(self):
        if self._engine is None:
            raise RuntimeError("the session is closed")
        return self._engine

    def prefill(self, token_ids) -> np.ndarray:
        tokens = [int(t) for t in token_ids]
        logits = self._active().runner.step([StepEntry(self._handle, tokens, [len(tokens) - 1])])
        return logits[0].cpu().numpy()

    def decode(self, token_id: int) -> np.ndarray:
        return self.prefill([token_id])

    def length(self) -> int:
        return self._active().cache.length(self._handle)

    def close(self) -> None:
        if self._engine is not None:
            self._engine.release_cache(self._handle)
            self._engine = None

    def __enter__(self):
        return self

    def __exit__(self, *_):
        self.close()


class Engine:
    def __init__(self, model_dir=None, options: EngineOptions = EngineOptions(), *, model=None):
        """model_dir: folder with config.json and model.safetensors. ``model``: an already
        loaded model instead (see ``from_random``)."""
        import torch

        from ..ops import library
        from ..sampling import Sampler

        library()  # fails loudly here if the kernels are missing
        self.options = options
        self.model = model if model is not None else load_model(model_dir, options.dtype, options.device)
        # the longest sequence a request may reach: the model's own limit, narrowed by the caller's if one is given
        if options.max_length is not None and options.max_length < 1:
            raise ValueError(f"max_length must be at least 1, not {options.max_length}")
        limit = self.model.max_positions()
        if options.max_length is not None:
            limit = options.max_length if limit is None else min(limit, options.max_length)
        if options.max_tokens is not None and options.cache_gib is not None:
            raise ValueError("give the cache's capacity as max_tokens or as cache_gib, not both")
        if options.cache_gib is not None:
            element_size = torch.empty((), dtype=self.model.precision.compute).element_size()
            max_tokens = tokens_for_memory(self.model.cache_groups(), element_size, options.cache_gib, options.page_size)
        elif options.max_tokens is not None:
            max_tokens = options.max_tokens
        elif limit is not None:
            # max_sessions whole sequences: each takes whole pages
            max_tokens = options.max_sessions * (-(-limit // options.page_size) * options.page_size)
        else:
            raise ValueError("this model has no position limit of its own: give max_length (the cache then holds max_sessions "
                             "sequences of that length), or size the cache with max_tokens or cache_gib as well")
        if limit is None:
            # Block tables and the buffers of captured steps are as wide as the longest sequence: it has to be named,
            # not taken from the size of the pool (which may be millions of tokens).
            raise ValueError("this model has no position limit of its own: give max_length, the longest sequence a request may reach")
        self.cache = make_cache(self.model, max_tokens=max_tokens, page_size=options.page_size,
                                max_requests=options.max_sessions, device=options.device, max_length=limit)
        self.runner = ModelRunner(self.model, self.cache, options.device, use_graphs=options.use_graphs, portion_graph_after=options.portion_graph_after,
                                  lanes_from=options.decode_lanes_from)
        self.sampler = Sampler(self.runner.staging)
        self.scheduler = Scheduler(_Executor(self), max_batch=options.max_sessions, max_tokens_per_step=options.max_tokens_per_step,
                                   step_ahead=options.step_ahead)
        self._next_handle = 0
        self._queued = collections.deque()   # the chosen tokens of steps that were not taken yet

    @classmethod
    def from_random(cls, config, seed: int, options: EngineOptions = EngineOptions()):
        """An engine over random weights of the given typed configuration."""
        return cls(options=options, model=random_model(config, seed, options.dtype, options.device))

    @property
    def config(self):
        return self.model.config

    def __enter__(self):
        return self

    def __exit__(self, *_):
        self.close()

    def close(self) -> None:
        """Whatever is still live or waiting ends with an error; its pages go back, and so do the captured steps."""
        self.scheduler.shutdown()
        self.runner.drop_graphs()

    # --- one sequence at a time (native.py) ---------------------------------------------------------
    def forward_last(self, token_ids) -> np.ndarray:
        """Logits after the last token of a whole sequence; nothing is kept."""
        with self.open_session() as session:
            return session.prefill(token_ids)

    def open_session(self) -> Session:
        handle = self.try_take_cache()
        if handle is None:
            raise RuntimeError("all sessions are taken")
        return Session(self, handle)

    # --- the calls the reference's scheduler drives (batch_api.py) --------------------------------------
    def try_take_cache(self):
        """A handle for a new sequence, or None when all are taken. Never waits."""
        if not self.cache.can_open():
            return None
        handle = ("session", self._next_handle)
        self._next_handle += 1
        self.cache.open(handle)
        return handle

    def release_cache(self, handle) -> None:
        self.cache.close(handle)

    def prefill_greedy(self, handle, token_ids) -> int:
        """The prompt in one step; returns its greedy next token, which also stays in the sequence's last-token slot."""
        tokens = [int(t) for t in token_ids]
        if not tokens:
            raise RuntimeError("the prompt has no tokens")
        return self.runner.step([StepEntry(handle, tokens, [len(tokens) - 1])], choose=True).tolist()[0]

    def decode_batch(self, handles, tokens) -> list[int]:
        if len(handles) != len(tokens) or not handles:
            raise RuntimeError("a batch has one token per sequence and at least one sequence")
        return self.runner.step([StepEntry(h, [int(t)], [0]) for h, t in zip(handles, tokens)], choose=True).tolist()

    # --- queued decoding: step n+1 is launched before the host has read token n ------------------------
    # (the reference's enqueue / take: engine/src/gpt2_gpu_greedy.cu:80-123, native.py:123-155)
    MAX_QUEUED = 4

    def decode_batch_enqueue(self, handles) -> None:
        """Queues one greedy decode step for these sequences. Each sequence's input is the token
        its previous step (``prefill_greedy``, ``decode_batch`` or an earlier enqueue) chose, taken
        from its last-token slot on the device; the host need not have read it yet."""
        import torch

        if not handles:
            raise RuntimeError("a batch has at least one sequence")
        if len(self._queued) >= self.MAX_QUEUED:
            raise RuntimeError(f"{self.MAX_QUEUED} steps are queued already: take one first")
        self._queued.append(self.runner.step([StepEntry(h, [0], [0], from_slot=True) for h in handles], choose=True))

    def take(self) -> list[int]:
        """The tokens of the oldest queued step (waits for it)."""
        if not self._queued:
            raise RuntimeError("no step is queued")
        return self._queued.popleft().tolist()

    # --- continuous batching ------------------------------------------------------------------------------
    def submit(self, request: Request) -> None:
        self.scheduler.submit(request)

    def step(self) -> bool:
        return self.scheduler.step()

    def stats(self) -> dict:
        return self.scheduler.stats()

    def generate(self, prompts, max_new_tokens: int = 64, temperature: float = 0.0, top_p: float = 1.0,
                 seed: int = 0, eos_token_id: int | None = None) -> list[list[int]]:
        """Continues every prompt (a list of token ids) through the scheduler; returns the new
        tokens of each. A prompt too long for the model is cut from the left so that the new
        tokens fit, as the reference's script does (scripts/complete.py:92-110)."""
        limit = self.runner.longest_sequence()
        outputs: list[list[int]] = [[] for _ in prompts]
        errors: list[str | None] = [None] * len(prompts)
        for i, prompt in enumerate(prompts):
            tokens = [int(t) for t in prompt]
            if limit is not None and len(tokens) > max(1, limit - max_new_tokens):
                tokens = tokens[-max(1, limit - max_new_tokens):]

            def emit(token, finish, i=i):
                outputs[i].append(token)

            def fail(message, i=i):
                errors[i] = message

            self.submit(Request(tokens, on_token=emit, on_error=fail, max_new_tokens=max_new_tokens, eos_token_id=eos_token_id,
                                sampling=SamplingParams(temperature=temperature, top_p=top_p, seed=seed + i)))
        self.scheduler.run_until_idle()
        failed = [f"prompt {i}: {e}" for i, e in enumerate(errors) if e is not None]
        if failed:
            raise RuntimeError("generation failed: " + "; ".join(failed))
        return outputs
