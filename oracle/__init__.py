"""CPU restatement of the reference's MXFP4 fused-MoE path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``pyhip_amd/`` imports this package: it is
the checker used by ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py``, never the thing that is shipped or measured.

Every function cites the reference file:line it restates (paths relative to the
tingqli/pyhip tree).  What pins each function (independent of the formula it
retypes) is listed in its module docstring; functions with no such pin are marked
"parity unpinned".
"""
