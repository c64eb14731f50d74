"""Figures of a run, printed as the reference prints them: a markdown table under the marker
``##### BurnLM Stats`` (crates/burn-lm-inference/src/stats.rs:4-95).  The reference divides the
generated tokens by the whole ``generate()`` time, prompt included
(crates/burn-lm-llama/src/generation/generate.rs:59,105-108); that figure is kept as "Tokens Per
Second", and prompt and decode speeds are given beside it."""
from __future__ import annotations

from dataclasses import dataclass

STATS_MARKER = "##### BurnLM Stats"


@dataclass
class Stats:
    prompt_tokens: int = 0
    prompt_seconds: float = 0.0
    generated_tokens: int = 0
    decode_tokens: int = 0       # generated tokens that came from one-token steps
    decode_seconds: float = 0.0
    inference_seconds: float = 0.0
    model_loading_seconds: float = None
    steps: int = 0

    @property
    def tokens_per_second(self):
        return self.generated_tokens / self.inference_seconds if self.inference_seconds > 0 else None

    @property
    def prompt_tokens_per_second(self):
        return self.prompt_tokens / self.prompt_seconds if self.prompt_seconds > 0 else None

    @property
    def decode_tokens_per_second(self):
        return self.decode_tokens / self.decode_seconds if self.decode_seconds > 0 else None

    def entries(self):
        def rate(v):
            return "N/A" if v is None else f"{v:.2f}"
        rows = [("Inference Duration", f"{self.inference_seconds:.2f}s")]
        if self.model_loading_seconds is not None:
            rows.append(("Model Loading Duration", f"{self.model_loading_seconds:.2f}s"))
        rows += [("Tokens Count", str(self.generated_tokens)),
                 ("Tokens Per Second", rate(self.tokens_per_second)),
                 ("Total Duration", f"{self.inference_seconds + (self.model_loading_seconds or 0.0):.2f}s"),
                 ("Prompt Tokens", str(self.prompt_tokens)),
                 ("Prompt Tokens Per Second", rate(self.prompt_tokens_per_second)),
                 ("Decode Tokens Per Second", rate(self.decode_tokens_per_second))]
        return rows

    def display_stats(self) -> str:
        rows = self.entries()
        w0 = max(len("Statistic Name"), *(len(r[0]) for r in rows))
        w1 = max(len("Value"), *(len(r[1]) for r in rows))
        lines = [f"| {'Statistic Name':<{w0}} | {'Value':>{w1}} |", f"|{'-' * (w0 + 2)}|{'-' * (w1 + 2)}|"]
        lines += [f"| {a:<{w0}} | {b:>{w1}} |" for a, b in rows]
        return "\n" + STATS_MARKER + "\n" + "\n".join(lines)
