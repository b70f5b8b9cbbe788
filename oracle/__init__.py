"""CPU restatement of the reference's algorithms for the fused GEMM + collective path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``tileccl_amd/`` imports this package; it is used
by ``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py`` as the checker (and as the timed CPU port), never as the product path.

Every function cites the reference lines it restates.  How each part is pinned (which
known answers, closed forms or brute-force checks hold it in place) is listed in
``oracle/PINNING.md`` and exercised by ``tests/test_oracle_*.py``.

Parity status
    planning (tile groups, tables, specs, transport, wg)   pinned: closed-form known answers,
                                                            invariants, brute force on tiny shapes
    heap bump allocator / pointer translation               pinned: invariants + closed forms
    scatter / gather placement                              pinned: element-loop brute force
    reduce-scatter sum                                      pinned: exact fp32 two-addend sum,
                                                            textbook RTNE casts
    GEMM numerics                                           pinned to fp32 matmul within the
                                                            reference's own tolerance
                                                            (tests/test_gemm_allscatter_smoke.py:39-40)
    cost model                                              pinned: closed-form floats, exact
                                                            recovery of synthetic (alpha, beta)
    S0/S1/S2 kernel schedules, cost-model -> group-size rule
                                                            parity unpinned: the reference tree
                                                            does not contain them
"""
