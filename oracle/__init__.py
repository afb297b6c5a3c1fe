"""CPU oracle for the KvsAll scoring / filtered-rank / top-k path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory: the only permitted users are ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``.  The product path calls the HIP
library through its C ABI and raises when that library is missing.

Contents
--------
``kge_oracle``      numpy restatement (fp64 by default) of the reference
                    arithmetic: query builders, Q.E^T scores, filtered-rank
                    counts, top-k, multi-hot BCE, bf16/int8 table emulation.
``torch_cpu_path``  restatement of the reference's *op sequence* on torch CPU
                    (several narrow ``mm``/``einsum`` calls, the per-row Python
                    mask loop, full ``torch.sort``, ``torch.topk``); this is
                    what ``bench.py`` times as ``cpu_baseline`` (kind "port").

Pinning status (what independent check each function has) is listed in the
header of ``kge_oracle``.
"""
