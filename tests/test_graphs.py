"""Decode steps replayed from a HIP graph give the logits of the eager step, replay after
replay, with the program's own eager work (prefill steps of other shapes, new requests)
between the replays."""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu

CFG = dict(H.TINY_A, num_hidden_layers=4, hidden_size=128, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
           intermediate_size=128, vocab_size=320)       # head size 64: the MFMA attention kernels run


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_graph_replays_equal_eager_steps(tmp_path, dtype):
    from spite_amd.engine.engine import Engine, StepEntry
    d = str(tmp_path / "m")
    H.make_model(d, CFG, seed=2, dtype=dtype)
    engines = [Engine(d, dtype=dtype, page_size=32, cache_tokens=1024, max_requests=4, graphs=g) for g in (True, False)]
    prompts = [H.random_tokens(CFG["vocab_size"], n, 20 + n) for n in (37, 5, 64)]
    late = H.random_tokens(CFG["vocab_size"], 45, 99)
    outs = []
    for eng in engines:
        rows = []
        slots = [eng.admit() for _ in prompts]
        logits = eng.step([StepEntry(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)])
        toks = logits.argmax(-1).tolist()
        rows.append(logits.cpu().numpy().copy())
        for step in range(40):
            if step == 17:                      # eager work of another shape between replays
                slots.append(eng.admit())
                lg = eng.step([StepEntry(slots[-1], late, [len(late) - 1])])
                rows.append(lg.cpu().numpy().copy())
                toks.append(int(lg.argmax(-1)[0]))
            logits = eng.step([StepEntry(s, [t], [0]) for s, t in zip(slots, toks)])
            toks = logits.argmax(-1).tolist()
            rows.append(logits.cpu().numpy().copy())
        outs.append(rows)
        eng.cache.check()
    assert engines[0].graph_replays >= 30 and engines[1].graph_replays == 0
    for a, b in zip(*outs):
        assert a.shape == b.shape and np.array_equal(a, b)


def test_a_graph_is_not_replayed_after_a_later_step_has_moved_the_workspaces(tmp_path):
    # a small decode shape is captured; the first decode step of a larger shape then grows the
    # scratch buffers (they start tiny here), which frees what the first graph points into; back
    # at the small shape the graph must be captured anew, not replayed
    from spite_amd.engine.engine import Engine, StepEntry
    d = str(tmp_path / "m")
    H.make_model(d, CFG, seed=4, dtype="bfloat16")
    prompts = [H.random_tokens(CFG["vocab_size"], 1 if i == 0 else 2, 70 + i) for i in range(7)]
    outs = []
    for graphs in (True, False):
        eng = Engine(d, dtype="bfloat16", page_size=32, cache_tokens=1024, max_requests=8, graphs=graphs,
                     workspace_bytes=1024)
        rows = []
        slots = [eng.admit()]
        tok = [int(eng.step([StepEntry(slots[0], prompts[0], [0])]).argmax(-1)[0])]
        for _ in range(6):                                   # seen, captured, replayed
            lg = eng.step([StepEntry(slots[0], [tok[0]], [0])])
            rows.append(lg.cpu().numpy().copy())
            tok = lg.argmax(-1).tolist()
        first = {k: v for k, v in eng._graphs.items() if v != "seen"}
        assert bool(first) == graphs
        for p in prompts[1:]:
            slots.append(eng.admit())
            tok.append(int(eng.step([StepEntry(slots[-1], p, [1])]).argmax(-1)[0]))
        before = eng._stamp()
        for _ in range(3):                                   # seven requests: seven rows of logits, more scratch
            lg = eng.step([StepEntry(s, [t], [0]) for s, t in zip(slots, tok)])
            rows.append(lg.cpu().numpy().copy())
            tok = lg.argmax(-1).tolist()
        if graphs:
            assert eng._stamp() != before, "the larger shape was meant to grow a workspace"
            assert all(eng._graphs.get(k) is not g for k, g in first.items()), "a stale graph was kept"
        for s in slots[1:]:
            eng.release(s)
        for _ in range(5):                                   # the small shape again
            lg = eng.step([StepEntry(slots[0], [tok[0]], [0])])
            rows.append(lg.cpu().numpy().copy())
            tok = [int(lg.argmax(-1)[0])]
        outs.append(rows)
        eng.cache.check()
    for a, b in zip(*outs):
        assert a.shape == b.shape and np.array_equal(a, b)
