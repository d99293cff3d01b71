"""The engine says, once and on standard error, when a part will run a kernel far slower than the
one meant for it: a configuration one step off the sizes that the MFMA kernels take must not run
an order of magnitude slower without a word."""
import pytest

import helpers as H

pytestmark = pytest.mark.gpu


def build(tmp_path, name, dtype, page, **over):
    from spite_amd.engine.engine import Engine
    cfg = dict(H.CONFIGS[name], **over)
    folder = str(tmp_path / f"{name}_{dtype}_{page}")
    H.make_model(folder, cfg, seed=2, dtype=dtype)
    return Engine(folder, dtype=dtype, page_size=page, cache_tokens=256, max_requests=2)


def test_sizes_that_the_mfma_kernels_take_say_nothing(tmp_path, capfd):
    eng = build(tmp_path, "C", "bfloat16", 32)
    assert eng.slow_paths == {} and "slow path" not in capfd.readouterr().err


def test_a_head_size_or_a_page_size_off_the_kernels_is_reported(tmp_path, capfd):
    eng = build(tmp_path, "B", "bfloat16", 8)                  # head size 24, pages of 8
    err = capfd.readouterr().err
    notes = [n for n in eng.slow_paths if "attention runs on plain FMAs" in n]
    assert len(notes) == 1 and "head size 24" in notes[0] and "pages of 8" in notes[0]
    assert eng.slow_paths[notes[0]] == list(range(8)) and err.count("attention runs on plain FMAs") == 1
    eng = build(tmp_path, "C", "bfloat16", 16)                 # the right head size on pages of 16
    assert any("pages of 16" in n and "head size" not in n for n in eng.slow_paths)
    capfd.readouterr()
    # a 32-bit run has no fast path to fall off
    assert build(tmp_path, "B", "float32", 8).slow_paths == {} and "slow path" not in capfd.readouterr().err


def test_a_width_off_the_products_and_a_tensor_kept_wide_are_reported(tmp_path, capfd):
    eng = build(tmp_path, "C", "bfloat16", 32, hidden_size=132)          # 132 is no multiple of 8
    assert any("no multiple of 8" in n for n in eng.slow_paths)
    from spite_amd.engine.engine import Engine
    folder = str(tmp_path / "wide")
    H.make_model(folder, H.CONFIGS["C"], seed=2, dtype="bfloat16", keep_wide=("shared_expert",))
    eng = Engine(folder, dtype="bfloat16", page_size=32, cache_tokens=256, max_requests=2)
    assert any("shared expert" in n and "kept in 32-bit" in n for n in eng.slow_paths)
