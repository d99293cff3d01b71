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
