"""CPU oracle for the landmark-attention hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this directory: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` use it,
and only as the checker.  It restates, in plain torch-on-CPU code, what the
reference computes on this path:

* ``s1``        closed form of landmark grouped-softmax causal attention
                (what ``llama/ltriton/flash_landmark_attention.py:6-305`` fuses)
* ``highlevel`` the scatter/gather grouped softmax the reference ships as its
                high-level path (``llama/llama_mem.py:168-243``,
                ``lm_benchmark/models/landmark.py:37-119,196-236``,
                ``llama/ltriton/test_flash_landmark_attention.py:105-125``)
* ``rotary``    half-split rotary embedding (``llama/llama_mem.py:95-149``)
* ``retrieval`` mem-cache scoring / top-k / gather / attend
                (``llama/llama_mem.py:318-430,447-477,807-815``)

Pinning.  The reference holds no golden vectors for this path (its only test
draws unseeded ``torch.rand``), so every function here is pinned by mathematics
in ``tests/test_oracle_*.py``: a literal per-row brute force in Python floats,
textbook causal softmax attention on the cases that reduce to it, rows of
weights summing to one, invariances (landmark value rows, permutations inside a
block), a hand-derived two-block closed form, finite differences for the
gradients, and agreement between the closed form and the independently written
scatter/gather restatement.  No function is left "parity unpinned".
"""
