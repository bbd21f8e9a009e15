"""MI355X-native (gfx950) implementation of IsoExec's batch-invariant token-logprob path.

Layout mirrors the reference package ``skyrl/backends/skyrl_train/isoexec``: ``ops/<family>``
hold the op functions (same names and argument meaning) and ``_register.py`` declarations,
``core`` / ``contract`` / ``models`` hold the declaration API and the content-hashed execution
contract. The arithmetic lives in ``csrc/`` behind the C ABI of ``include/isoexec_hip.h``.
"""

ARCH = "gfx950"
