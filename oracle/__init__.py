"""CPU oracle for the block-sparse attention path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package (``dkernel_amd``) may import this package: it is
the checker that the HIP path is compared against, never the thing that is
shipped or measured.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` use it.

Modules
-------
layout     numpy restatement of the reference's host LUT code
           (dkernel/utils.py): block mask, CSR/CSC with -1 padding,
           merge/split to kernel tiles, KV-cache-efficiency check.
attention  dense masked softmax attention in fp32 (restating
           tests/test_sparse_attn.py:486-537 of the reference), natural-log
           LSE, gradients through torch autograd, LSE merge of partitions
           (dkernel/interface.py:303-324).

Pinning status (what fixes each function independently of this file's own
formulae) is listed in each module's header.
"""
from . import layout, attention  # noqa: F401
