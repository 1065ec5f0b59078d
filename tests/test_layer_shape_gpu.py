"""One layer with the sizes of the Qwen2.5-7B shape (width 3584, 28 query / 4
key-value heads of 128, feed-forward 18944; a small vocabulary so that the plain
implementation stays quick) against the plain implementation. The tiny models never
reach the code that only real sizes take: weight-streaming products with many column
tiles and eight-way splits along k, the library products of a long portion, attention
with seven query heads per key/value head, decode steps replayed from HIP graphs."""

from __future__ import annotations

import pytest
import torch

from helpers import TOL, first_bad, make_engine, plain_logits, random_ids, replay

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def layer_model(tmp_path_factory):
    import plain_qwen2 as P
    from pyre_amd.config import preset
    from pyre_amd.weights import write_random_model

    cfg = preset("qwen2.5-7b", num_hidden_layers=1, vocab_size=1536)
    d = tmp_path_factory.mktemp("layer7b")
    write_random_model(d, cfg, seed=5, std=0.02, gain_std=0.1)
    return d, (P.read_config(d), P.read_weights(d))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_layer_of_the_7b_shape(dtype, layer_model):
    folder, plain = layer_model
    vocab = plain[0]["vocab_size"]
    reqs = {"a": random_ids(vocab, 150, 1), "b": random_ids(vocab, 90, 2), "c": random_ids(vocab, 41, 3)}
    rounding = torch.bfloat16 if dtype == "bfloat16" else None
    want = {r: plain_logits(plain, ids, rounding) for r, ids in reqs.items()}
    eng = make_engine(folder, dtype, use_graphs=True, max_cached_tokens=512, max_num_seqs=4)
    a, b, c = reqs["a"], reqs["b"], reqs["c"]
    steps = [
        ([("a", a[:100], [0, 63, 99])], []),                       # a long portion: library products in 16 bits
        ([("a", a[100:130], [29]), ("b", b[:70], [69])], []),      # two portions in one step
    ]
    # decode a and b token by token beside portions of c, then c alone
    for i in range(20):
        entries = [("a", a[130 + i:131 + i], [0]), ("b", b[70 + i:71 + i], [0])]
        if i < 4:
            entries.append(("c", c[10 * i:10 * i + 10], [9]))
        steps.append((entries, ["a", "b"] if i == 19 else []))
    steps.append(([("c", c[40:41], [0])], ["c"]))
    got = replay(eng, steps)
    bad, worst = first_bad(got, want, TOL[dtype])
    assert bad is None, bad
    assert eng.graph_replays > 0
    assert eng.cache.page_groups[0].allocator.num_used == 0
