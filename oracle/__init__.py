"""CPU restatement of the reference's algorithm for the batch-split MLP path.

THIS PACKAGE IS TEST INFRASTRUCTURE.  It is imported only by ``tests/``, by
``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py`` - as
the checker, never as the thing that is measured or shipped.  Nothing under
``dynaflow_amd/`` imports it.

Modules and what pins each of them (none of the reference's own files holds a
test, golden vector or fixture for this path, so every function is pinned by
closed forms, invariants, brute force or an independent second implementation;
see the tests named below):

    split_policy    pack_tokens, the trivial split, the balanced two-way cut
                    and the equal N-way cut.  Pinned by hand-derived cases
                    (tests/golden/split_cases.json), an O(n^2) brute-force
                    search with first-minimiser tie-break and structural
                    invariants  (tests/test_oracle_split.py).
    partition       Op / Mod / rule matching, partition numbering and tagging
                    on plain node records.  Pinned by hand-derived goldens
                    (tests/golden/partition_cases.json) and invariants
                    (tests/test_oracle_partition.py).
    schedule_trace  issue order of (sub-graph, nano-batch) launches and the
                    event chain for the round-robin and staggered schedules.
                    Pinned by the hand-derived traces in
                    tests/golden/schedule_traces.json and invariants
                    (tests/test_oracle_schedule.py).
    mlp             the arithmetic: split -> per-nano-batch SwiGLU MLP -> cat,
                    SiLU*mul, RMSNorm, e4m3 quantisation.  Pinned by the
                    row-independence identity (split == unsplit), a float64
                    closed form, and the independent C restatement mlp_ref.c
                    (tests/test_oracle_mlp.py).  PARITY UNPINNED against the
                    reference's own outputs: the reference ships none.
    decoder         one Llama-shaped decoder layer (embedding, RMSNorm, QKV,
                    RoPE, causal grouped-query attention, output projection,
                    residuals, SwiGLU MLP) in float64, written independently
                    of the product module: RoPE as a complex multiplication,
                    attention as an explicit masked softmax per head.  Pinned
                    by special cases (position 0 is the identity, rotation
                    preserves norms, one-token attention returns v, causal
                    prefix independence) and by torch's own attention routine
                    on the CPU  (tests/test_decoder_cpu.py).  PARITY UNPINNED
                    against reference outputs: the reference ships none.
    decode          one decode step (one new token per sequence) over stacked
                    layers with KV caches, float64, caches in the natural
                    layout, loops over tokens and heads.  Pinned by special
                    cases (a single position returns its value, constant V,
                    a dominated head), by token-by-token decoding == the
                    prefill oracle on the whole sequence, and by the product
                    module on the CPU  (tests/test_decode_cpu.py).  PARITY
                    UNPINNED against reference outputs: there are none.
"""
