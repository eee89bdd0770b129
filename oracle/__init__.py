"""CPU oracle for the paged KV-cache write + paged attention path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; the only callers are ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``, and there it is the checker / the timed
CPU baseline, never the thing that produces a result handed to a user.

Modules
-------
paged_ops   torch restatement of the reference's CPU branches
            (python_package/tt_torch/custom_ops.py:635-742, 962-1104, 1198-1443,
            GQA decode form :551-610), plus the sliding-window / attention-sink forms
            that the reference's CPU branches ignore: semantics specified here,
            PARITY UNPINNED against the reference.
bfp8_codec  numpy block-float-8 quantise / dequantise.  The reference holds no
            CPU codec for this format (it lives in un-vendored tt-metal), so the
            codec is specified here and pinned by invariants: PARITY UNPINNED
            against the reference.
"""

from . import paged_ops, bfp8_codec  # noqa: F401
