"""The step's batch as the kernels read it: the flat arrays and the block tables, packed on the host.  On the
CPU the builder's device is the host, so what a step would send can be read back."""

import numpy as np
import pytest
import torch

from rvllm_amd.cache.pages import BlockTable
from rvllm_amd.engine.batch import BatchBuilder, Portion


def build(builder, portions, tables):
    return builder.build(portions, tables, list(range(len(portions))))


def test_arrays_of_a_mixed_step():
    b = BatchBuilder("cpu", 32, 4, {"all": 8})
    portions = [Portion("a", [5, 6, 7], 10, want=[2]), Portion("b", [9], 40, want=[0]), Portion("c", [1, 2], 0)]
    step = build(b, portions, {"all": [[3, 4], [7, 8, 9, 2], [5]]})
    assert step.num_tokens == 6 and step.num_requests == 3 and step.max_portion == 3 and step.max_context == 41
    assert step.token_ids.tolist() == [5, 6, 7, 9, 1, 2]
    assert step.positions.tolist() == [10, 11, 12, 40, 0, 1]
    assert step.token_req.tolist() == [0, 0, 0, 1, 2, 2]
    assert step.q_start.tolist() == [0, 3, 4, 6] and step.chunk_start.tolist() == [10, 40, 0]
    assert step.context_len.tolist() == [13, 41, 2] and step.logit_rows.tolist() == [2, 3]
    table = step.block_tables["all"]
    assert table.shape == (4, 8)
    assert table[:3, :4].tolist() == [[3, 4, -1, -1], [7, 8, 9, 2], [5, -1, -1, -1]]


def test_a_shorter_step_after_a_longer_one_reads_no_page_of_the_earlier_one():
    """Only the step's requests by the entries of its longest table are sent.  Inside that rectangle every entry
    is the step's own: a row shorter than the longest ends in -1, whatever the step before left there."""
    b = BatchBuilder("cpu", 16, 3, {"all": 6, "window": 6})
    long_tables = {"all": [[1, 2, 3, 4, 5], [6, 7, 8]], "window": [BlockTable([-1, -1, 3, 4, 5]), BlockTable([6, 7, 8])]}
    build(b, [Portion("a", [1], 70), Portion("b", [1], 40)], long_tables)
    step = build(b, [Portion("c", [1], 20), Portion("d", [1, 2], 3)], {"all": [[9, 10], [11]], "window": [[9, 10], [11]]})
    for name in ("all", "window"):
        assert step.block_tables[name][:2, :2].tolist() == [[9, 10], [11, -1]]
    # the staging buffers take turns: a third step finds in its buffer what the first one left, and still sends its own
    step = build(b, [Portion("e", [4], 0)], {"all": [[2]], "window": [[2]]})
    assert step.block_tables["all"][0, 0].item() == 2 and step.block_tables["window"][0, 0].item() == 2


def test_tables_of_many_pages_match_a_plain_loop():
    rng = np.random.default_rng(3)
    width, n = 700, 5
    b = BatchBuilder("cpu", 64, 8, {"g": width})
    for _ in range(4):
        rows = [rng.integers(0, 10_000, size=int(rng.integers(1, width + 1))).tolist() for _ in range(n)]
        portions = [Portion(i, [1], len(rows[i]) * 16 - 1) for i in range(n)]
        step = build(b, portions, {"g": rows})
        longest = max(len(r) for r in rows)
        want = np.full((n, longest), -1)
        for i, r in enumerate(rows):
            want[i, : len(r)] = r
        assert np.array_equal(step.block_tables["g"][:n, :longest].numpy(), want)


def test_too_many_requests_tokens_or_pages_are_refused():
    b = BatchBuilder("cpu", 4, 2, {"g": 2})
    with pytest.raises(ValueError, match="3 requests"):
        build(b, [Portion(i, [1], 0) for i in range(3)], {"g": [[1]] * 3})
    with pytest.raises(ValueError, match="5 tokens"):
        build(b, [Portion("a", [1] * 5, 0)], {"g": [[1]]})
    with pytest.raises(ValueError, match="3 entries"):
        build(b, [Portion("a", [1], 40)], {"g": [[1, 2, 3]]})
    with pytest.raises(ValueError, match="wanted place"):
        build(b, [Portion("a", [1, 2], 0, want=[2])], {"g": [[1]]})
    assert isinstance(build(b, [], {"g": []}).block_tables["g"], torch.Tensor)


def test_graph_buckets_cover_every_context_and_widen_with_it():
    from rvllm_amd.engine.runner import ModelRunner

    last = 0
    edges = set()
    for context in range(1, 140_000, 7):
        edge = ModelRunner.context_bucket(context)
        assert edge >= context and edge >= last  # covers the context; never goes back
        assert edge - context < max(1024, context / 8 + 1)  # planned for at most an eighth more keys
        assert ModelRunner.context_bucket(edge) == edge
        last = edge
        edges.add(edge)
    assert ModelRunner.context_bucket(1) == 1024 and ModelRunner.context_bucket(16_385) == 18_432
    assert len(edges) <= 16 + 8 * 4
