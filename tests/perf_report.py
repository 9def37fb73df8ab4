"""Measured times, ratios and ceilings are reported by the tests, never asserted: a correct
library on a slow or noisy box must not fail the parity run.  `expect` prints the figure and
raises a warning (shown in pytest's summary) when it is outside what was seen before."""
import warnings


class PerfWarning(UserWarning):
    pass


def expect(ok: bool, what: str) -> bool:
    print(f"[perf] {'ok  ' if ok else 'SLOW'} {what}", flush=True)
    if not ok:
        warnings.warn(PerfWarning(what), stacklevel=2)
    return bool(ok)
