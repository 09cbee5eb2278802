"""Backend selection: the plug-in boundary of the lazy front end.

Same rule as the reference (delayrepay/backend.py:3-11): the choice is made
once, at import, by the *presence* of an environment variable.  `DELAY_CPU`
selects the NumPy node-by-node evaluator; anything else selects the HIP
fusion backend for gfx950, which needs libdrhip.so and raises at import when
it is missing (there is no silent host fall-back).
"""
import os

if "DELAY_CPU" in os.environ:
    from . import cpu as _selected
else:
    from . import hip as _selected

backend = _selected
