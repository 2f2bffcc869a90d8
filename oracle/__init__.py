"""CPU restatement of decode attention over a paged KV cache, its forest-cascade
decomposition, the log-sum-exp merge, shared-prefix discovery and the platform's
feature-flag parser.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this directory; it is
used by ``tests/``, by the smoke check and by the CPU-baseline leg of ``bench.py`` as the
checker.  Every function cites the reference lines whose behaviour it restates.

The forest cascade kernels themselves have no counterpart in the reference tree (they
live in an external, un-vendored package), so the value oracle is the reference's own
plain softmax attention with grouped KV heads, evaluated per sequence on gathered pages.

Parity pins (see tests/test_oracle.py): brute force vs ``F.scaled_dot_product_attention``
and ``torch.logsumexp``; closed forms (single token, constant V, score shift, distinct
constant V per KV head for the GQA mapping); merge invariants (partition independence,
associativity, empty partial is the identity); grouping literals from the reference's
``tests/zorro_train/test_dedup.py:76-104``; flag-parser cases.
"""
