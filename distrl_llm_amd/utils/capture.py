"""Keeping Python's cyclic collector out of a hipGraph capture.

An engine and its captured decode steps refer to each other, so a dropped
engine is only freed when the cyclic collector runs, at a moment of its own
choosing. Destroying a captured graph while another stream capture is open
is an error that ends the process: collect what is garbage before the
capture starts and keep the collector off until it has ended.
"""

from __future__ import annotations

import gc
from contextlib import contextmanager


@contextmanager
def collector_paused():
    gc.collect()
    was_on = gc.isenabled()
    gc.disable()
    try:
        yield
    finally:
        if was_on:
            gc.enable()
