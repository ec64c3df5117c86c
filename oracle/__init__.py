"""CPU restatement of the reference's decode-step hot path -- TEST INFRASTRUCTURE ONLY.

Nothing under ``oracle/`` is part of the product: only ``tests/``, the smoke check and the
benchmark's CPU-baseline leg import it, and only as the checker.  Each function cites the
reference lines it restates.  What pins each function (golden vectors held by the
reference's own tests, library routines, closed forms, brute force) is listed in the
module docstrings and exercised by ``tests/test_oracle_*.py``.

Parity status: the paged attention arithmetic itself lives in the third-party ``flash-attn``
package (not vendored, not pinned by the reference; minimum 2.7.3 asserted at
megatron/core/transformer/attention.py:650-653) and no reference test holds numeric
vectors for it, so :mod:`oracle.paged_attention` restates the published algorithm
(softmax(QK^T * scale)V with flash-attn's bottom-right aligned causal mask) and is pinned by
library routines and invariants, not by reference-held vectors.
"""
