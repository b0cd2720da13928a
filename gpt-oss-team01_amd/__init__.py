"""gptoss_mi355: MI355X (gfx950) implementation of the GPT-OSS decode hot path behind a C ABI.

``lib`` binds the shared library, ``ops`` is a thin device-pointer front end for tests and
benchmarks, ``binfmt``/``synth`` read, write and synthesise the reference's flat ``.bin``
checkpoints."""
from . import binfmt, synth  # noqa: F401
