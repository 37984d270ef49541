"""Helpers that build replay traces and compare what a replay wrote with the
plain implementation."""
import json

import numpy as np

from conftest import assert_close, plain_logits


def ceil64(n):
    return -(-n // 64) * 64


class Trace:
    """Steps of {"step", "entries", "end"}; remembers which (request, position)
    each written row belongs to."""

    def __init__(self):
        self.steps, self.expect, self.fed, self.peak, self._live = [], {}, {}, 0, {}

    def add(self, entries, end=(), fork=()):
        """entries: [(id, tokens, want)]; fork: [(source, target)], done before the entries run"""
        index = len(self.steps)
        rows = []
        for source, target in fork:
            self.fed[target] = list(self.fed[source])
            self._live[target] = len(self.fed[target])
        for rid, tokens, want in entries:
            start = len(self.fed.setdefault(rid, []))
            self.fed[rid].extend(tokens)
            rows.extend((rid, start + w) for w in want)
            self._live[rid] = len(self.fed[rid])
        self.peak = max(self.peak, sum(ceil64(n) for n in self._live.values()))
        for rid in end:
            self._live.pop(rid)
        self.steps.append({"step": index, "entries": [{"id": r, "tokens": list(map(int, t)), "want": list(w)} for r, t, w in entries],
                           "end": list(end), **({"fork": [list(f) for f in fork]} if fork else {})})
        if rows:
            self.expect[index] = rows
        return index

    def lines(self):
        return [json.dumps(s) for s in self.steps]

    def check(self, folder, out_dir, dtype, vocab, sequences):
        """sequences: {id: full token list}.  Compares every written row."""
        per_request = {}
        for step, rows in self.expect.items():
            data = np.fromfile(out_dir / f"{step}.f32", dtype="<f4").reshape(len(rows), vocab)
            for row, (rid, pos) in zip(data, rows):
                per_request.setdefault(rid, []).append((pos, row))
        written = {int(p.stem) for p in out_dir.glob("*.f32")}
        assert written == set(self.expect), "a step without wanted rows wrote a file, or a wanted one is missing"
        for rid, items in per_request.items():
            ref = plain_logits(folder, sequences[rid])
            pos = [p for p, _ in items]
            assert_close(np.stack([r for _, r in items]), ref[pos], dtype, what=f"request {rid}")
        return per_request
