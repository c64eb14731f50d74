"""The model-side contract and the Python entry point.

``InferenceServer`` has the shape of the reference's trait of that name
(crates/burn-lm-inference/src/server.rs:21-52: load / is_loaded / unload / run_job /
clear_state, with the options parsed from command-line flags or JSON) and of its Llama servers
(crates/burn-lm-llama/src/server/llama3.rs:400-577).  Options carry the reference's names,
meanings and defaults (llama3.rs:14-31): ``top_p`` 0.9, ``temperature`` 0.0 (0 = greedy),
``max_seq_len`` 8192 (the context the cache is built for), ``sample_len`` 4096 (JSON alias
``max_tokens``), ``seed`` 0 (0 = a fresh random seed for each request).  Download and delete are
not part of it: a model is a local folder.
"""
from __future__ import annotations

import json
import time
from dataclasses import asdict, dataclass, fields
from typing import Callable, List, Optional, Sequence

from .engine.generate import ContextLengthExceeded, generate
from .text.tokenizer import StreamingDecoder
from .engine.stats import Stats
from .sampling.sampler import Sampler


class ModelNotLoaded(RuntimeError):
    def __init__(self):
        super().__init__("Model has not been loaded.")


@dataclass
class ServerConfig:
    top_p: float = 0.9
    temperature: float = 0.0
    max_seq_len: int = 8192
    sample_len: int = 4096
    seed: int = 0

    ALIASES = {"max_tokens": "sample_len"}

    def update(self, **kw):
        names = {f.name for f in fields(self)}
        for k, v in kw.items():
            k = self.ALIASES.get(k, k)
            if k not in names:
                raise KeyError(f"unknown option {k!r}; options: {', '.join(sorted(names))}")
            if v is not None:
                setattr(self, k, type(getattr(self, k))(v))
        return self


def add_cli_flags(parser):
    """The reference's per-model flags (crates/burn-lm-macros/src/lib.rs:20-171 makes one
    ``--long`` flag per option)."""
    d = ServerConfig()
    parser.add_argument("--top-p", type=float, default=None, help=f"Top-p probability threshold [default: {d.top_p}]")
    parser.add_argument("--temperature", type=float, default=None,
                        help=f"Temperature value for controlling randomness in sampling [default: {d.temperature}]")
    parser.add_argument("--max-seq-len", type=int, default=None,
                        help=f"Maximum sequence length for input text [default: {d.max_seq_len}]")
    parser.add_argument("--sample-len", type=int, default=None,
                        help=f"The number of new tokens to generate [default: {d.sample_len}]")
    parser.add_argument("--seed", type=int, default=None,
                        help="The seed to use when generating random samples. If it is 0 then a random seed is "
                             f"used for each inference [default: {d.seed}]")


class InferenceServer:
    """One model folder behind the reference's server interface."""

    def __init__(self, folder: str, dtype: str = "bfloat16", config: Optional[ServerConfig] = None,
                 batch_size: int = 8, device: str = "cuda:0", model_name: Optional[str] = None,
                 cast_32bit: bool = False):
        self.folder, self.dtype, self.device = folder, dtype, device
        self.cast_32bit = cast_32bit
        self.config = config or ServerConfig()
        self.batch_size = batch_size
        self.engine = None
        self.tokenizer = None
        self._name = model_name

    # ---- metadata (crates/burn-lm-macros/src/lib.rs:296-301) ---------------------------------
    def model_name(self):
        return self._name or self.folder.rstrip("/").split("/")[-1]

    def model_cli_param_name(self):
        return self.model_name().lower().replace(" ", "-")

    # ---- options -----------------------------------------------------------------------------
    def parse_cli_config(self, args) -> None:
        self.config.update(**{f.name: getattr(args, f.name, None) for f in fields(ServerConfig)})

    def parse_json_config(self, text: str) -> None:
        self.config.update(**json.loads(text))

    # ---- life cycle --------------------------------------------------------------------------
    def is_loaded(self) -> bool:
        return self.engine is not None

    def load(self) -> Optional[Stats]:
        if self.is_loaded():
            return None
        from .engine.loading import load_engine, read_config
        t0 = time.perf_counter()
        _, cfg = read_config(self.folder)
        ctx = min(self.config.max_seq_len, cfg.max_position_embeddings)
        self.engine = load_engine(self.folder, dtype=self.dtype, max_tokens=ctx * self.batch_size,
                                  max_seqs=self.batch_size, max_context=ctx, device=self.device,
                                  cast_32bit=self.cast_32bit)
        st = Stats()
        st.model_loading_seconds = time.perf_counter() - t0
        self._load_seconds = st.model_loading_seconds
        return st

    def unload(self) -> Optional[Stats]:
        self.engine = None
        self.tokenizer = None
        import torch
        if torch.cuda.is_available():
            torch.cuda.empty_cache()
        return None

    def clear_state(self) -> None:
        if not self.is_loaded():
            raise ModelNotLoaded()
        self.engine.clear()

    # ---- work --------------------------------------------------------------------------------
    def stop_ids(self):
        """The configuration's end-of-sequence ids and the tokenizer's stop ids together."""
        ids = set(self.engine.model.plan.stop_ids)
        if self.tokenizer is not None:
            ids.update(self.tokenizer.stop_ids())
        return sorted(ids)

    def generate(self, prompts: Sequence[Sequence[int]], on_token: Optional[Callable[[int, int], None]] = None,
                 stop_ids: Optional[Sequence[int]] = None, **options):
        """Token-id prompts in, ``(list of Generation, Stats)`` out; options override the config."""
        first = self.load()
        cfg = ServerConfig(**asdict(self.config)).update(**options)
        sampler = Sampler(cfg.temperature, cfg.top_p, cfg.seed)
        results, stats = generate(self.engine, prompts, sampler, cfg.sample_len,
                                  stop_ids=self.stop_ids() if stop_ids is None else stop_ids,
                                  batch_size=self.batch_size, on_token=on_token)
        if first is not None:
            stats.model_loading_seconds = first.model_loading_seconds
        return results, stats

    def _tokenizer(self):
        if self.tokenizer is None:
            from .text.tokenizer import for_folder
            self.tokenizer = for_folder(self.folder, self.engine.vocab_size,
                                        self.engine.model.architecture.special_tokens)
        return self.tokenizer

    def prompt(self, messages) -> str:
        """The prompt text of a list of messages: the architecture's chat template (the reference's
        servers each carry their own, crates/burn-lm-llama/src/server/llama3.rs:561-576); an
        architecture without one gets the contents joined by newlines."""
        self.load()
        template = self.engine.model.architecture.chat_template
        if template is None:
            return "\n".join(m["content"] for m in messages)
        return template(messages)

    def _text_of(self, task) -> str:
        if isinstance(task, str):
            return task
        return self.prompt([task] if isinstance(task, dict) else list(task))

    def run_jobs(self, tasks, **options):
        """Several tasks (each as for run_job) as batches of unequal lengths -> (texts, Stats); a
        request that cannot run (longer than the context) gives its error as its text."""
        self.load()
        tok = self._tokenizer()
        ids = [tok.encode(self._text_of(t), False, False) for t in tasks]
        stop = set(self.stop_ids())
        results, stats = self.generate(ids, **options)
        texts = [f"error: {r.error}" if r.finish_reason == "error" else tok.decode([t for t in r.tokens if t not in stop])
                 for r in results]
        self.last_generations = results
        return texts, stats

    def run_job(self, task, on_text: Optional[Callable[[str], None]] = None, **options) -> Stats:
        """task: a prompt string, one message ``{"role", "content"}``, or a list of messages
        (InferenceTask::Prompt / Message / Context, crates/burn-lm-inference/src/job.rs:15-50)."""
        first = self.load()
        text = self._text_of(task)
        tok = self._tokenizer()
        ids = tok.encode(text, False, False)  # no BOS/EOS added (nn/llama/inference.rs:35-40)
        stop = set(self.stop_ids())
        pieces = StreamingDecoder(tok)

        def emit(_, t):
            if on_text is None or t in stop:
                return
            s = pieces.push(t)
            if s:
                on_text(s)

        results, stats = self.generate([ids], on_token=emit, **options)
        if on_text is not None:
            rest = pieces.flush()
            if rest:
                on_text(rest)
        r = results[0]
        if r.finish_reason == "error":
            if len(ids) > self.engine.max_context:
                raise ContextLengthExceeded(len(ids), self.engine.max_context)
            raise RuntimeError(r.error)
        self.last_generation = r
        if first is not None:
            stats.model_loading_seconds = first.model_loading_seconds
        return stats
