"""What the command line shows beside the generated text: the configuration in use, the prefill's progress
and the speeds at the end.

The reference draws panels, tables and a progress bar with a terminal library and has a plain mode that prints
the same facts as bare lines (cpmcu/common/display.py:57-115, 182-260; ``--plain-output``).  Here both modes
are written with nothing but the standard streams: plain mode prints one fact a line and nothing that moves;
formatted mode adds a rule above and below each group, colours when the stream is a terminal, and a progress
bar that redraws in place.  Everything goes to the diagnostic stream, so that standard output carries the
generated text alone.
"""
from __future__ import annotations

import sys
import time
from typing import List, Optional, Sequence, Tuple

_COLOURS = {"title": "1;32", "key": "36", "dim": "2", "bar": "32"}


class Display:
    def __init__(self, plain: bool = False, stream=None, width: int = 72):
        self.plain = bool(plain)
        self.stream = stream if stream is not None else sys.stderr
        self.width = width
        self.colour = not self.plain and hasattr(self.stream, "isatty") and self.stream.isatty()

    # ------------------------------------------------------------------
    def _paint(self, text: str, kind: str) -> str:
        return f"\033[{_COLOURS[kind]}m{text}\033[0m" if self.colour else text

    def line(self, text: str = ""):
        print(text, file=self.stream, flush=True)

    def table(self, title: str, rows: Sequence[Tuple[str, object, str]]):
        """A group of (name, value, unit) facts under a title."""
        rows = [(str(k), self._value(v), u) for k, v, u in rows]
        if self.plain:
            self.line(f"{title}:")
            for k, v, u in rows:
                self.line(f"  {k}: {v}{' ' + u if u else ''}")
            return
        rule = "-" * self.width
        head = f" {title} "
        self.line(self._paint(rule[:3] + head + rule[3 + len(head):], "title"))
        pad = max((len(k) for k, _, _ in rows), default=0)
        for k, v, u in rows:
            self.line(f"  {self._paint(k.ljust(pad), 'key')}  {v}{' ' + self._paint(u, 'dim') if u else ''}")
        self.line(self._paint(rule, "title"))

    @staticmethod
    def _value(v) -> str:
        if isinstance(v, bool):
            return "yes" if v else "no"
        if isinstance(v, float):
            return f"{v:.2f}"
        s = str(v)
        return s[:45] + "..." if len(s) > 50 else s

    # ------------------------------------------------------------------
    def configuration(self, args, sections: Sequence[Tuple[str, Sequence[Tuple[str, str]]]]):
        """The options in use, by sections of (attribute of ``args``, label); absent or unset ones are left out."""
        for title, fields in sections:
            rows = [(label, getattr(args, name), "") for name, label in fields
                    if getattr(args, name, None) is not None]
            if rows:
                self.table(title, rows)

    def performance(self, prefill_tokens: int, prefill_time: float, decode_tokens: int, decode_time: float):
        """The figures the reference ends with (cpmcu/common/display.py:95-115): lengths, times, speeds."""
        rows: List[Tuple[str, object, str]] = [("Prefill Length", prefill_tokens, "tokens")]
        if prefill_time > 0:
            rows += [("Prefill Time", prefill_time, "s"), ("Prefill Speed", f"{prefill_tokens / prefill_time:.1f}", "tokens/s")]
        rows.append(("Decode Length", decode_tokens, "tokens"))
        if decode_time > 0:
            rows += [("Decode Time", decode_time, "s"), ("Decode Speed", f"{decode_tokens / decode_time:.1f}", "tokens/s")]
        self.table("Performance Summary", rows)

    def progress(self, total_tokens: int) -> "Progress":
        return Progress(self, total_tokens)

    def progress_callback(self):
        """A callback for ``LLM.generate(progress_callback=)``: events 'begin' {total_tokens}, 'advance'
        {current_tokens}, 'finish' {total_time} (cpmcu/cli.py:82-97)."""
        state = {"bar": None}

        def callback(event: str, data: dict):
            if event == "begin":
                state["bar"] = self.progress(int(data["total_tokens"]))
                state["bar"].begin()
            elif event == "advance" and state["bar"] is not None:
                state["bar"].advance(int(data["current_tokens"]))
            elif event == "finish" and state["bar"] is not None:
                state["bar"].finish(data.get("total_time"))
                state["bar"] = None
        return callback


class Progress:
    """Prefill progress: a bar that redraws in place, or in plain mode a line at the start and one at the end."""

    def __init__(self, display: Display, total_tokens: int):
        self.d = display
        self.total = max(int(total_tokens), 1)
        self.t0 = 0.0
        self.shown = -1

    def begin(self):
        self.t0 = time.time()
        if self.d.plain:
            self.d.line(f"Prefilling: 0/{self.total} tokens")
        else:
            self._draw(0)

    def advance(self, current_tokens: int):
        if not self.d.plain:
            self._draw(min(current_tokens, self.total))

    def finish(self, total_time: Optional[float] = None):
        took = total_time if total_time is not None else time.time() - self.t0
        if self.d.plain:
            self.d.line(f"Prefill done: {self.total}/{self.total} tokens in {took:.2f} s")
        else:
            self._draw(self.total)
            self.d.stream.write(f"  {took:.2f} s\n")
            self.d.stream.flush()

    def _draw(self, done: int):
        cells = 30
        full = done * cells // self.total
        if full == self.shown and done != self.total:
            return
        self.shown = full
        bar = self.d._paint("#" * full, "bar") + "." * (cells - full)
        self.d.stream.write(f"\rPrefilling [{bar}] {done}/{self.total} tokens")
        self.d.stream.flush()
