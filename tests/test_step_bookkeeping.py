"""Everything around the kernels, checked without a GPU: the kernels' entry points
are replaced by torch stand-ins (tests/helpers/cpu_ops.py) and the replay regimes
are compared with the plain implementation.  A difference here is a fault of the
batch descriptor, the block tables or the page accounting."""

import numpy as np
import pytest
import torch

from helpers import configs, cpu_ops, models, traces


def _requests(vocab, lengths, seed=0):
    return {f"r{i}": traces.random_tokens(seed * 100 + i, n, vocab) for i, n in enumerate(lengths)}


@pytest.mark.parametrize("name,lengths", [("tiny_a", [5, 17, 33, 64]), ("tiny_b", [9, 40, 100, 57, 23]), ("tiny_c", [70, 41, 90])])
@pytest.mark.parametrize("regime", ["whole", "tail", "portions", "mixed"])
def test_regimes_against_plain(tmp_path, monkeypatch, name, lengths, regime):
    from cwm_amd.replay import Replayer

    cpu_ops.install(monkeypatch)
    folder = models.make_folder(tmp_path, name, seed=3, dtype="float32")
    vocab = configs.get(name)["vocab_size"]
    requests = _requests(vocab, lengths)
    steps = {
        "whole": traces.whole,
        "tail": lambda r: traces.tail_one_by_one(r, tail=8),
        "portions": traces.portions,
        "mixed": traces.mixed,
    }[regime](requests)
    max_tokens = traces.max_live_tokens(steps)
    rep = Replayer(folder, "float32", max_tokens, device="cpu", page_size=4 if regime == "mixed" else 16, poison_freed_pages=True)
    outputs = traces.run_in_process(rep, steps)
    got = traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab)
    want = models.plain_logits(folder, requests, dtype=torch.float32)
    for rid in requests:
        assert not np.isnan(got[rid]).any(), f"{rid}: missing or NaN logits"
        np.testing.assert_allclose(got[rid], want[rid], rtol=2e-4, atol=2e-5, err_msg=f"{name} {regime} {rid}")
    assert rep.manager.live_requests() == []
    assert all(f == g.pool.num_pages for f, g in zip(rep.manager.free_pages(), rep.manager.groups))


def test_a_step_whose_readable_pages_are_not_all_held_is_refused():
    """The descriptor is refused when a logical page that the step's queries read, or that its
    tokens are written to, has no page of the pool; a page that the window has passed may be gone."""
    from cwm_amd.cache import CacheManager
    from cwm_amd.engine.batch import BatchError, Portion, build_batch
    from cwm_amd.parts import PagedKVSpec

    specs = [PagedKVSpec(1, 16, None), PagedKVSpec(1, 16, 6)]
    manager = CacheManager(specs, 4, 16, 2)
    manager.admit("a")
    assert manager.extend("a", 20)
    manager.advance("a", 20)  # the window group has given back pages 0..2 (keys 0..11 lie before 20 - 5)
    assert manager.table(1, "a")[:3] == [-1, -1, -1]
    assert manager.extend("a", 3)
    device = torch.device("cpu")
    build_batch([Portion("a", [1, 2, 3], [2])], manager, device, 50)  # fine as it is
    # a hole where the first query of the portion still reads (key 15 = 20 - 5 lies in page 3)
    held = manager.table(1, "a")[3]
    manager.table(1, "a")[3] = -1
    with pytest.raises(BatchError, match="holds no page"):
        build_batch([Portion("a", [1, 2, 3], [2])], manager, device, 50)
    manager.table(1, "a")[3] = held
    # a hole in the keep-all group, far back
    held = manager.table(0, "a")[0]
    manager.table(0, "a")[0] = 99
    with pytest.raises(BatchError, match="holds no page"):
        build_batch([Portion("a", [1, 2, 3], [2])], manager, device, 50)
    manager.table(0, "a")[0] = held
    build_batch([Portion("a", [1, 2, 3], [2])], manager, device, 50)


def test_trace_run_options(tmp_path, monkeypatch, capsys):
    """The replay program with a configuration and a seed instead of a folder, pages of 8 tokens,
    the pools' sizes given outright, and the log of pages taken and given back: a window group
    gives pages back while its request runs, and no page is handed out while it is held."""
    import io
    import json
    import sys

    from cwm_amd import replay

    cpu_ops.install(monkeypatch)
    config = configs.get("tiny_b")
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(config))
    vocab = config["vocab_size"]
    requests = _requests(vocab, [40, 23], seed=5)
    steps = traces.portions(requests, sizes=[5, 3, 9])
    log = tmp_path / "pages.jsonl"
    out = tmp_path / "out"
    monkeypatch.setattr(sys, "stdin", io.StringIO("".join(json.dumps(s) + "\n" for s in steps)))
    rc = replay.main([
        "--random-config", str(cfg_path), "--seed", "3", "--std", "0.05", "--dtype", "float32", "--out", str(out), "--max-tokens", "64",
        "--device", "cpu", "--page-size", "8", "--pages", "all=6,8=3", "--page-log", str(log),
    ])
    assert rc == 0
    assert [l for l in capsys.readouterr().out.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    # the logits are those of the plain implementation on the same random weights
    from cwm_amd.weights import write_random_model

    folder = str(tmp_path / "same")
    write_random_model(folder, config, seed=3, std=0.05, norm_init="ones", dtype="float32")
    outputs = {s["step"]: np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(-1, vocab) for s in steps}
    got = traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab)
    want = models.plain_logits(folder, requests, dtype=torch.float32)
    for rid in requests:
        np.testing.assert_allclose(got[rid], want[rid], rtol=2e-4, atol=2e-5)
    # the log: what is taken was free, what is given back was held
    records = [json.loads(l) for l in log.read_text().splitlines()]
    assert len(records) == len(steps)
    held = {0: set(), 1: set()}
    sizes = {0: None, 1: None}
    gave_back_early = False
    for rec, st in zip(records, steps):
        for rid, by_group in rec["take"].items():
            for g, pages in by_group.items():
                assert not held[int(g)] & set(pages)
                held[int(g)] |= set(pages)
        for g, pages in rec["give"].items():
            assert set(pages) <= held[int(g)]
            held[int(g)] -= set(pages)
            if not st["end"]:
                gave_back_early = True
        assert len(rec["free"]) == 2
    assert gave_back_early  # the window of 8 keys passes pages of 8 tokens as the request goes on
    assert held == {0: set(), 1: set()}
    with pytest.raises(SystemExit):
        replay.main(["--dtype", "float32", "--out", str(out), "--max-tokens", "64"])
