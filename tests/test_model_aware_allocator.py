"""Model-aware activation planner (host logic, no GPU): the recipes of the reference's
core/allocator/bert_allocator_test.cpp:30-108 and model_aware_memory_scheduler.cpp:34-120.

The validity predicate is restated here in Python, independently of the C++ one: two records that
are live at the same time must not overlap inside a chunk, every record must lie inside its chunk.
"""
import itertools

import numpy as np
import pytest

import turbo_transformers

cxx = turbo_transformers.cxx

MiB = 1 << 20


def check_valid(records, chunk_sizes, placements):
    assert len(placements) == len(records)
    for (name, a0, a1, asz), (ac, ao) in zip(records, placements):
        assert 0 <= ac < len(chunk_sizes), name
        assert ao >= 0 and ao % 256 == 0 and ao + asz <= chunk_sizes[ac], name
    for ((na, a0, a1, asz), (ac, ao)), ((nb, b0, b1, bsz), (bc, bo)) in itertools.combinations(zip(records, placements), 2):
        if ac != bc or max(a0, b0) > min(a1, b1):
            continue
        assert max(ao, bo) >= min(ao + asz, bo + bsz), "%s and %s are live together and overlap" % (na, nb)


def test_bert_usage_records_shape_and_order():
    recs = cxx.bert_tensor_usage_records(2, 50, 12, 768, 12)
    names = [r[0] for r in recs]
    assert len(set(names)) == len(names)
    for want in ("BERTEmbedding/Reshape", "self/q/Reshape", "self/k/Reshape", "self/v/Reshape", "batch_gemm3/Reshape",
                 "batch_gemm4/Reshape", "gemm5/Reshape", "BertIntermediate/Reshape"):
        assert want in names
    sizes = [r[3] for r in recs]
    assert sizes == sorted(sizes, reverse=True)  # greedy by size needs the largest first
    by = {r[0]: r for r in recs}
    T, H = 100, 768
    assert by["gemm5/Reshape"][3] == T * H * 4
    assert by["BertIntermediate/Reshape"][3] == 4 * T * H * 4
    assert by["batch_gemm3/Reshape"][3] == 2 * 12 * 50 * 50 * 4
    assert by["self/v/Reshape"][3] == 2 * 56 * H * 4  # V may be stored transposed with seq padded to 8
    # the hidden states outlive every per-layer tensor; q and k die before the probabilities do
    assert by["BERTEmbedding/Reshape"][1] <= by["self/q/Reshape"][1] and by["BERTEmbedding/Reshape"][2] >= by["gemm5/Reshape"][2]
    assert by["self/q/Reshape"][2] < by["self/v/Reshape"][2]


@pytest.mark.parametrize("B,S", [(1, 40), (2, 50), (1, 100), (20, 128), (64, 512)])
def test_bert_plan_is_valid(B, S):
    """bert_allocator_test.cpp:68-83 ("bert-allocator-multiple-chunk")."""
    recs = cxx.bert_tensor_usage_records(B, S, 12, 768, 12)
    placements, chunks, used = cxx.plan_memory(recs, [])
    check_valid(recs, chunks, placements)
    assert cxx.placement_is_valid(recs, chunks, placements)
    assert all(used)
    # sharing by lifetime must beat one buffer per tensor, chunk slack (x1.2, 2 MiB minimum) included
    assert sum(chunks) < 1.2 * sum(r[3] for r in recs) + 2 * MiB * len(chunks)
    total_live_peak = max(sum(r[3] for r in recs if r[1] <= op <= r[2]) for op in range(13))
    assert sum(chunks) >= total_live_peak


def test_replanning_reuses_chunks():
    """bert_allocator_test.cpp:85-108 ("bert-allocator-multiple-allocation"): plans for a sequence of
    input shapes over one chunk list stay valid; old chunks are reused when they fit."""
    chunks = []
    history = []
    for B, S in [(2, 50), (1, 100), (2, 50), (4, 16), (1, 4)]:
        recs = cxx.bert_tensor_usage_records(B, S, 12, 768, 12)
        before = list(chunks)
        placements, chunks, used = cxx.plan_memory(recs, chunks)
        check_valid(recs, chunks, placements)
        assert chunks[:len(before)] == before  # existing chunks keep their size and index
        history.append((len(chunks), used))
        chunks = [c for c, u in zip(chunks, used) if u]  # what the allocator keeps (unused ones are freed)
    # the same shape planned twice into a list that already fits it adds no chunk
    recs = cxx.bert_tensor_usage_records(2, 50, 12, 768, 12)
    _, chunks1, _ = cxx.plan_memory(recs, [])
    _, chunks2, used2 = cxx.plan_memory(recs, chunks1)
    assert chunks2 == chunks1 and all(used2)


def test_planner_known_answers():
    # two tensors never live together share offset 0; a third that overlaps both goes behind the larger
    recs = [("a", 0, 1, 1000), ("b", 2, 3, 800), ("c", 1, 2, 500)]
    placements, chunks, used = cxx.plan_memory(recs, [])
    assert chunks == [2 * MiB] and used == [True]
    assert placements[0] == (0, 0) and placements[1] == (0, 0)
    assert placements[2] == (0, 1024)  # behind a (1000 rounded to the 256-byte placement grid)
    # best fit: the tightest gap between live neighbours wins
    recs = [("x", 0, 9, 4096), ("y", 0, 9, 4096), ("z", 0, 9, 4096), ("gapmaker", 5, 9, 256)]
    placements, chunks, _ = cxx.plan_memory(recs, [])
    assert [p[1] for p in placements] == [0, 4096, 8192, 12288]
    # a hole left by a tensor that is dead by then is reused rather than growing the chunk
    recs = [("a", 0, 9, 4096), ("b", 0, 3, 4096), ("c", 0, 9, 4096), ("d", 5, 9, 2048), ("e", 5, 9, 4096)]
    placements, chunks, _ = cxx.plan_memory(recs, [])
    assert placements[3] == (0, 4096)       # d sits in b's hole between a and c
    assert placements[4] == (0, 12288)      # e no longer fits there (d took half of it): behind c
    # a tensor larger than the default chunk opens a chunk of 1.2x its size
    big = 10 * MiB
    placements, chunks, _ = cxx.plan_memory([("big", 0, 0, big)], [])
    assert placements == [(0, 0)] and 1.2 * big <= chunks[0] <= 1.2 * big + 256
    # it does not fit an existing small chunk: the small one is reported unused
    placements, chunks, used = cxx.plan_memory([("big", 0, 0, big)], [2 * MiB])
    assert placements == [(1, 0)] and used == [False, True]


def test_planner_random_records_stay_valid():
    rng = np.random.default_rng(7)
    for trial in range(40):
        n = int(rng.integers(1, 40))
        recs = []
        for i in range(n):
            a = int(rng.integers(0, 12))
            recs.append(("t%d" % i, a, a + int(rng.integers(0, 6)), int(rng.integers(1, 6 * MiB))))
        recs.sort(key=lambda r: -r[3])
        placements, chunks, used = cxx.plan_memory(recs, [3 * MiB] if trial % 2 else [])
        check_valid(recs, chunks, placements)
        assert cxx.placement_is_valid(recs, chunks, placements)


def test_validity_predicate_rejects_overlap():
    recs = [("a", 0, 2, 1000), ("b", 1, 3, 1000)]
    assert cxx.placement_is_valid(recs, [4096], [(0, 0), (0, 1024)])
    assert not cxx.placement_is_valid(recs, [4096], [(0, 0), (0, 512)])     # live together, overlapping
    assert not cxx.placement_is_valid(recs, [4096], [(0, 0), (0, 3584)])    # runs past the chunk
    assert cxx.placement_is_valid([("a", 0, 1, 1000), ("b", 2, 3, 1000)], [4096], [(0, 0), (0, 0)])


def test_schema_names():
    assert cxx.allocator_schema() == "naive"
    with pytest.raises(RuntimeError, match="no schema"):
        turbo_transformers.reset_allocator_schema("greedy")
    turbo_transformers.reset_allocator_schema("model-aware")
    try:
        assert cxx.allocator_schema() == "model-aware"
    finally:
        turbo_transformers.reset_allocator_schema("naive")
    assert cxx.allocator_schema() == "naive"
