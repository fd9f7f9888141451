"""Front-end mode switch.

EXACT = False (default): everything is restated as the reference has it, including
behaviours that differ from the mathematics (see the module docstrings).
EXACT = True: gradients use correct VJPs and shared views are un-shared before
lowering; used for the training-step configurations, which the reference's own
rules cannot run to completion.
"""

import contextlib

EXACT = False


@contextlib.contextmanager
def exact_mode(on: bool = True):
    global EXACT
    old, EXACT = EXACT, on
    try:
        yield
    finally:
        EXACT = old
