"""How a bfloat16 run is compared with the plain float32 implementation.

Logits: the largest difference over a row, relative to the largest logit of the
sequence, stays under BF16_TOL (the worst seen over some thousands of seeded
tiny models is 8e-3).  Greedy tokens: each one is the plain model's argmax,
unless the plain model's two best logits lie closer together than twice that
tolerance allows a logit to move, and only a few tokens may use that excuse
(the reference's tests/test_paged.py:88-99 judges bfloat16 runs the same way:
mismatches only at near-ties, and only a few)."""

from __future__ import annotations

FP32_TOL = 1e-4
BF16_TOL = 1.5e-2
TOL = {"float32": FP32_TOL, "bfloat16": BF16_TOL}
MAX_EXCUSED = 0.10  # share of the generated tokens that may differ at a near-tie


class GreedyCheck:
    """Counts, over any number of requests, the tokens that were compared and
    those that differed from the plain argmax at a near-tie."""

    def __init__(self, plain, dtype: str):
        self.plain = plain
        self.exact = dtype == "float32"
        self.compared = 0
        self.excused = 0

    def request(self, prompt, generated) -> None:
        seq = list(prompt)
        for i, tok in enumerate(generated):
            row = self.plain.logits(seq)[-1]
            self.compared += 1
            if int(row.argmax()) != tok:
                top2 = row.topk(2).values
                gap = 0.0 if self.exact else 2 * BF16_TOL * float(row.abs().max())
                assert float(top2[0] - top2[1]) < gap, (
                    f"token {i}: engine chose {tok}, plain argmax {int(row.argmax())} at a clear "
                    f"margin ({float(top2[0] - top2[1]):.4f} against {gap:.4f})"
                )
                assert int(row.topk(2).indices[1]) == tok, (
                    f"token {i}: engine chose {tok}, which is not even the plain model's second choice"
                )
                self.excused += 1
            seq.append(tok)

    def finish(self) -> None:
        assert self.compared > 0
        assert self.excused <= MAX_EXCUSED * self.compared, (
            f"{self.excused} of {self.compared} tokens differ from the plain argmax: near-ties "
            "are not that common"
        )
