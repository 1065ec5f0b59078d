"""Two layers with the sizes of the Qwen2.5-7B shape (width 3584, 28 query / 4 key-value
heads of 128, feed-forward 18944) and its whole vocabulary of 152,064 against the plain
implementation. The tiny models never reach the code that only real sizes take:
weight-streaming products with many column tiles and splits along k, the head's product
over 152,064 rows in slices of 64 requests, the library products of a long portion,
attention with seven query heads per key/value head, decode steps of 17 to 64 requests
replayed from HIP graphs at their padded sizes.

The weights are drawn on the device (a file of this shape would take 3 GB) and the plain
implementation runs there too, in float64 (on the CPU it would take minutes)."""

from __future__ import annotations

import pytest
import torch

import plain_qwen2 as P
from helpers import (TOL, depth_tol, first_bad, first_layer_off, layer_report, make_engine_from_state, plain_logits,
                     random_ids, replay)

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def layers_7b():
    from pyre_amd.config import preset
    from pyre_amd.weights import model_tensor_specs, random_state

    cfg = preset("qwen2.5-7b", num_hidden_layers=2)
    assert cfg.vocab_size == 152064 and cfg.hidden_size == 3584 and cfg.intermediate_size == 18944
    state = random_state(model_tensor_specs(cfg), seed=5, std=0.02, gain_std=0.1, dtype="bfloat16", device=DEV)
    plain_cfg = {k: getattr(cfg, k) for k in ("hidden_size", "intermediate_size", "num_hidden_layers",
                                              "num_attention_heads", "num_key_value_heads", "vocab_size",
                                              "rms_norm_eps", "rope_theta", "tie_word_embeddings", "head_dim")}
    weights = {n: t.to(torch.float64) for n, t in state.items()}
    yield cfg, state, (plain_cfg, weights)
    weights.clear()
    state.clear()
    torch.cuda.empty_cache()


def _want(plain, reqs, dtype):
    rounding = torch.bfloat16 if dtype == "bfloat16" else None
    return {r: plain_logits(plain, ids, rounding) for r, ids in reqs.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_two_layers_of_the_7b_shape_with_the_whole_vocabulary(dtype, layers_7b):
    cfg, state, plain = layers_7b
    vocab = cfg.vocab_size
    reqs = {"a": random_ids(vocab, 150, 1), "b": random_ids(vocab, 90, 2), "c": random_ids(vocab, 41, 3)}
    want = _want(plain, reqs, dtype)
    eng = make_engine_from_state(cfg, state, dtype, use_graphs=True, max_cached_tokens=512, max_num_seqs=4)
    a, b, c = reqs["a"], reqs["b"], reqs["c"]
    steps = [
        ([("a", a[:100], [0, 63, 99])], []),                       # a long portion: library products in 16 bits
        ([("a", a[100:130], [29]), ("b", b[:70], list(range(70)))], []),   # two portions; 71 rows of logits at once
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_of_many_requests_at_the_7b_shape(dtype, layers_7b):
    """64, then 33, then 17 live requests, one token each per step, from HIP graphs: the
    weight-streaming products with two to four tiles of rows, the fused SiLU-gate product of
    17 to 64 rows, the decode attention's split rule at large batches, the head in slices."""
    cfg, state, plain = layers_7b
    vocab = cfg.vocab_size
    lengths = [5 + (7 * i) % 29 for i in range(64)]              # contexts that cross page ends at different steps
    reqs = {i: random_ids(vocab, n + 4, 100 + i) for i, n in enumerate(lengths)}
    want = _want(plain, reqs, dtype)
    eng = make_engine_from_state(cfg, state, dtype, use_graphs=True, max_cached_tokens=64 * 48, max_num_seqs=64,
                                 max_num_batched_tokens=2048)
    # prompts in two mixed steps, no logits; then four decode steps with fewer and fewer requests
    steps = [([(i, reqs[i][:lengths[i]], []) for i in range(0, 40)], []),
             ([(i, reqs[i][:lengths[i]], []) for i in range(40, 64)], [])]
    live = list(range(64))
    for k, keep in enumerate((64, 64, 33, 17)):
        live = live[:keep]
        steps.append(([(i, [reqs[i][lengths[i] + k]], [0]) for i in live], []))
    got = replay(eng, steps)
    assert len(got) == 64 + 64 + 33 + 17
    bad, worst = first_bad(got, want, TOL[dtype])
    assert bad is None, bad
    # the same again: steps that ran eagerly at their padded sizes (64, 48 for 33, 24 for 17) are now replayed
    for i in range(64):
        eng.finish(i)
    got2 = replay(eng, steps)
    assert eng.graph_replays > 0
    bad, worst = first_bad(got2, want, TOL[dtype])
    assert bad is None, bad
    for k in got:
        assert torch.equal(got[k], got2[k]), f"{k}: a replayed step differs from the eager one"


def test_captured_decode_steps_with_library_products_at_the_7b_shape(layers_7b):
    """100 live requests: a decode step of 128 rows, whose products are the BLAS library's,
    captured and replayed four times; every replay against the plain implementation."""
    cfg, state, plain = layers_7b
    vocab = cfg.vocab_size
    lengths = [3 + (5 * i) % 23 for i in range(100)]
    reqs = {i: random_ids(vocab, n + 6, 300 + i) for i, n in enumerate(lengths)}
    want = _want(plain, reqs, "bfloat16")
    eng = make_engine_from_state(cfg, state, "bfloat16", use_graphs=True, max_cached_tokens=100 * 48, max_num_seqs=100,
                                 max_num_batched_tokens=2048)
    steps = [([(i, reqs[i][:lengths[i]], []) for i in range(lo, lo + 50)], []) for lo in (0, 50)]
    for k in range(6):
        steps.append(([(i, [reqs[i][lengths[i] + k]], [0]) for i in range(100)], []))
    got = replay(eng, steps)
    assert len(got) == 600 and eng.graph_replays == 5
    bad, worst = first_bad(got, want, TOL["bfloat16"])
    assert bad is None, bad


def test_decode_steps_of_few_requests_at_the_1p5b_shape():
    """Two layers of the Qwen2.5-1.5B shape (width 1536, 12 query / 2 key-value heads, feed-forward
    8960, tied head): its products are so small that the weight-streaming kernel's blocks would
    not fill the chip, and the kernel that keeps the step's rows in a block takes them at every
    size, in blocks of 32 and 64 rows. Steps of 40, 8 and 1 requests from HIP graphs, twice."""
    from pyre_amd.config import preset
    from pyre_amd.parts.fast import mid_ksplit, skinny_ksplit
    from pyre_amd.weights import model_tensor_specs, random_state

    cfg = preset("qwen2.5-1.5b", num_hidden_layers=2)
    h, inter = cfg.hidden_size, cfg.intermediate_size
    for n_out, k in ((h + 2 * cfg.num_key_value_heads * cfg.head_dim, h), (h, h), (h, inter)):
        assert mid_ksplit(n_out, k) and -(-n_out // 64) * skinny_ksplit(8, n_out, k) < 256   # the rule of parts/fast.py
    state = random_state(model_tensor_specs(cfg), seed=6, std=0.02, gain_std=0.1, dtype="bfloat16", device=DEV)
    plain_cfg = {k: getattr(cfg, k) for k in ("hidden_size", "intermediate_size", "num_hidden_layers",
                                              "num_attention_heads", "num_key_value_heads", "vocab_size",
                                              "rms_norm_eps", "rope_theta", "tie_word_embeddings", "head_dim")}
    plain = (plain_cfg, {n: t.to(torch.float64) for n, t in state.items()})
    plain[1].setdefault("lm_head.weight", plain[1]["model.embed_tokens.weight"])    # the tied head, as the plain loader has it
    vocab = cfg.vocab_size
    lengths = [4 + (11 * i) % 27 for i in range(40)]
    reqs = {i: random_ids(vocab, n + 6, 700 + i) for i, n in enumerate(lengths)}
    want = _want(plain, reqs, "bfloat16")
    eng = make_engine_from_state(cfg, state, "bfloat16", use_graphs=True, max_cached_tokens=40 * 48, max_num_seqs=40,
                                 max_num_batched_tokens=2048)
    steps = [([(i, reqs[i][:lengths[i]], []) for i in range(40)], [])]
    live = list(range(40))
    for k, keep in enumerate((40, 40, 8, 8, 1, 1)):
        live = live[:keep]
        steps.append(([(i, [reqs[i][lengths[i] + k]], [0]) for i in live], []))
    got = replay(eng, steps)
    assert len(got) == 2 * (40 + 8 + 1) and eng.graph_replays == 3
    bad, worst = first_bad(got, want, TOL["bfloat16"])
    assert bad is None, bad
    # the same steps with the weight-streaming kernel for the narrow products, run eagerly
    eng2 = make_engine_from_state(cfg, state, "bfloat16", use_graphs=False, max_cached_tokens=40 * 48, max_num_seqs=40,
                                  max_num_batched_tokens=2048)
    eng2.runtime.options["mid_small"] = False
    got2 = replay(eng2, steps)
    bad, worst = first_bad(got2, want, TOL["bfloat16"])
    assert bad is None, bad
    plain[1].clear()
    state.clear()
    torch.cuda.empty_cache()


# ----------------------------------------------------------------------------- whole models

class _Widened(dict):
    """The bfloat16 tensors of a whole model, each widened to float64 when the plain implementation
    asks for it (61 GB of float64 copies at the 7B shape would fit, but nothing needs them at once)."""

    def __getitem__(self, name):
        return super().__getitem__(name).to(torch.float64)


@pytest.mark.parametrize("shape,dtype", [("qwen2.5-7b", "float32"), ("qwen2.5-7b", "bfloat16"),
                                         ("qwen2.5-1.5b", "float32"), ("qwen2.5-1.5b", "bfloat16")])
def test_every_layer_of_the_benchmarked_shapes(shape, dtype):
    """All 28 layers of the Qwen2.5-7B shape (the one that is benchmarked) and of the Qwen2.5-1.5B
    shape (tied head), the whole vocabulary: a prompt of 48 tokens whole with logits at every
    position, then the same prompt as a portion of 32 tokens and 16 single tokens, the single
    tokens from captured graphs from their third step on, every row against the plain
    implementation in float64 on the device. The bound was fixed before the first run
    (``helpers.depth_tol``). If a row is off, the message names the first layer whose hidden rows
    leave the bound (`scripts/diagnose_parity.py:103-120` of the reference walks its layers so)."""
    from pyre_amd.config import preset
    from pyre_amd.weights import model_tensor_specs, random_state

    cfg = preset(shape)
    assert cfg.num_hidden_layers == 28
    state = random_state(model_tensor_specs(cfg), seed=9, std=0.02, gain_std=0.1, dtype="bfloat16", device=DEV)
    plain_cfg = {k: getattr(cfg, k) for k in ("hidden_size", "intermediate_size", "num_hidden_layers",
                                              "num_attention_heads", "num_key_value_heads", "vocab_size",
                                              "rms_norm_eps", "rope_theta", "tie_word_embeddings", "head_dim")}
    weights = _Widened(state)
    if cfg.tie_word_embeddings:
        assert "lm_head.weight" not in state
        dict.__setitem__(weights, "lm_head.weight", state["model.embed_tokens.weight"])   # the tied head, as the plain loader has it
    plain = (plain_cfg, weights)
    ids = random_ids(cfg.vocab_size, 48, 77)
    rounding = torch.bfloat16 if dtype == "bfloat16" else None
    want = {r: plain_logits(plain, ids, rounding) for r in ("whole", "cut")}
    tol = depth_tol(dtype, cfg.num_hidden_layers)
    eng = make_engine_from_state(cfg, state, dtype, use_graphs=True, max_cached_tokens=256, max_num_seqs=2,
                                 max_num_batched_tokens=64, max_model_len=128)
    steps = [([("whole", ids, list(range(48)))], ["whole"]), ([("cut", ids[:32], list(range(32)))], [])]
    steps += [([("cut", ids[i:i + 1], [0])], ["cut"] if i == 47 else []) for i in range(32, 48)]
    got = replay(eng, steps)
    assert len(got) == 96 and eng.graph_replays >= 14
    bad, worst = first_bad(got, want, tol)
    if bad is not None:
        bad += " | " + first_layer_off(layer_report(eng, plain, ids, rounding), tol)
    assert bad is None, bad
    assert all(torch.isfinite(row).all() for row in got.values())
    # the walk through the layers itself: every layer's hidden rows within the same bound
    report = layer_report(eng, plain, ids, rounding)
    assert len(report) == 28 and all(d <= tol for _, d in report), first_layer_off(report, tol)
    print(f"{shape} {dtype}: worst row {worst:.2e} of the logit scale (bound {tol:.1e}); layers "
          f"{report[0][1]:.1e} .. {report[-1][1]:.1e}")
    weights.clear()
    state.clear()
    del eng
    torch.cuda.empty_cache()
