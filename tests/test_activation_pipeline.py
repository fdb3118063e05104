"""Cached-activation files, reader, mask filter and batchler: the reference's own expectations
(tests/unit/test_activation_writer.py, tests/unit/test_activation_processors.py:92-124, 228-300) on CPU tensors."""

import json

import pytest
import torch
from safetensors.torch import load_file, save_file


def sample_data():
    # tests/unit/test_activation_writer.py:37-58
    return [
        {"tokens": torch.tensor([[1, 2, 3]]), "meta": [{"context_idx": 1}], "h0": torch.ones(1, 3, 4), "h1": torch.zeros(1, 3, 4)},
        {"tokens": torch.tensor([[4, 5, 6]]), "meta": [{"context_idx": 2}], "h0": torch.ones(1, 3, 4) * 2, "h1": torch.zeros(1, 3, 4) * 2},
        {"tokens": torch.tensor([[7, 8, 9]]), "meta": [{"context_idx": 3}], "h0": torch.ones(1, 3, 4) * 3, "h1": torch.zeros(1, 3, 4) * 3},
    ]


def test_writer_layout_pt_and_safetensors(pkg, tmp_path):
    cfg = pkg.ActivationWriterConfig(cache_dir=str(tmp_path / "pt"), hook_points=["h0", "h1"], n_samples_per_chunk=2, format="pt")
    w = pkg.ActivationWriter(cfg)
    assert (tmp_path / "pt" / "h0").is_dir() and (tmp_path / "pt" / "h1").is_dir()
    w.process(sample_data())
    for hp in ("h0", "h1"):
        c0 = torch.load(tmp_path / "pt" / hp / f"chunk-{0:08d}.pt", weights_only=True)
        assert (tmp_path / "pt" / hp / f"chunk-{1:08d}.pt").exists()
        assert set(c0) >= {"activation", "tokens", "meta"} and len(c0["meta"]) == 2
        assert c0["activation"].shape == (2, 1, 3, 4) and c0["tokens"].shape == (2, 1, 3)
    cfg = pkg.ActivationWriterConfig(cache_dir=str(tmp_path / "st"), hook_points=["h0", "h1"], n_samples_per_chunk=2,
                                     format="safetensors", num_workers=2)
    pkg.ActivationWriter(cfg).process(sample_data())
    c0 = tmp_path / "st" / "h0" / f"chunk-{0:08d}.safetensors"
    assert load_file(str(c0))["activation"].shape == (2, 1, 3, 4)
    meta = json.loads(c0.with_suffix(".meta.json").read_text())
    assert isinstance(meta, list) and len(meta) == 2 and meta[0][0]["context_idx"] == 1 and meta[1][0]["context_idx"] == 2
    # no batching: one chunk per sample
    cfg = pkg.ActivationWriterConfig(cache_dir=str(tmp_path / "nb"), hook_points=["h0", "h1"], format="pt")
    pkg.ActivationWriter(cfg).process(sample_data())
    for i, s in enumerate(sample_data()):
        c = torch.load(tmp_path / "nb" / "h1" / f"chunk-{i:08d}.pt", weights_only=True)
        assert c["meta"] == s["meta"] and c["activation"].shape == (1, 3, 4) and c["tokens"].shape == (1, 3)
    with pytest.raises(ValueError, match="Invalid format: invalid"):
        pkg.ActivationWriter(pkg.ActivationWriterConfig(cache_dir=str(tmp_path / "x"), hook_points=["h0", "h1"],
                                                        format="invalid")).process(sample_data())
    with pytest.raises(AssertionError):
        w.process([{"tokens": torch.tensor([[1]]), "h0": torch.ones(1, 1, 4)}])     # h1 missing


def test_chunk_names(pkg, tmp_path):
    from pathlib import Path

    c = pkg.ChunkInfo.from_path(Path("shard-3-chunk-00000007.safetensors"))
    assert (c.shard_id, c.chunk_id) == (3, 7)
    c = pkg.ChunkInfo.from_path(Path("chunk-12.pt"))
    assert (c.shard_id, c.chunk_id) == (0, 12)
    with pytest.raises(ValueError):
        pkg.ChunkInfo.from_path(Path("part-1.pt"))


def _write_cache(root, hooks, n_chunks, n_samples, n_ctx, d, seed=0, shard=None, fmt="safetensors"):
    g = torch.Generator().manual_seed(seed)
    want = []
    for c in range(n_chunks):
        tokens = torch.randint(0, 1000, (n_samples, n_ctx), generator=g)
        mask = (torch.rand(n_samples, n_ctx, generator=g) > 0.25).to(torch.int64)
        acts = {hp: torch.randn(n_samples, n_ctx, d, generator=g) for hp in hooks}
        for hp in hooks:
            (root / hp).mkdir(parents=True, exist_ok=True)
            name = f"chunk-{c:08d}" if shard is None else f"shard-{shard}-chunk-{c:08d}"
            payload = {"activation": acts[hp], "tokens": tokens, "mask": mask, "attention_mask": torch.ones_like(mask)}
            if fmt == "safetensors":
                save_file(payload, str(root / hp / f"{name}.safetensors"))
            else:
                torch.save(payload, str(root / hp / f"{name}.pt"))
        want.append((tokens, mask, acts))
    return want


def test_loader_streams_chunks_in_order_and_merges_hook_points(pkg, tmp_path):
    hooks = ["blocks.0.hook_resid", "blocks.1.hook_resid"]
    want = _write_cache(tmp_path, hooks, n_chunks=3, n_samples=2, n_ctx=5, d=8, shard=1)
    want0 = _write_cache(tmp_path, hooks, n_chunks=2, n_samples=2, n_ctx=5, d=8, seed=9, shard=0, fmt="pt")
    loader = pkg.CachedActivationLoader({hp: tmp_path / hp for hp in hooks}, device="cpu", dtype=torch.bfloat16)
    out = list(loader.process())
    assert len(out) == 5
    for got, (tokens, mask, acts) in zip(out, want0 + want):      # shard 0 before shard 1, chunk order inside
        assert torch.equal(got["tokens"], tokens) and torch.equal(got["mask"], mask)
        for hp in hooks:
            assert got[hp].dtype == torch.bfloat16 and torch.equal(got[hp], acts[hp].to(torch.bfloat16))
    # a hook point with a different number of chunks is an error, as is a missing directory
    (tmp_path / hooks[1] / "shard-1-chunk-00000002.safetensors").unlink()
    with pytest.raises(ValueError, match="different numbers of chunks"):
        list(loader.process())
    with pytest.raises(FileNotFoundError):
        list(pkg.CachedActivationLoader({"nope": tmp_path / "nope"}).process())


def test_loader_flattens_stacked_samples_and_checks_tokens(pkg, tmp_path):
    cfg = pkg.ActivationWriterConfig(cache_dir=str(tmp_path), hook_points=["h0", "h1"], n_samples_per_chunk=2, format="safetensors")
    data = [dict(s, mask=torch.ones(1, 3, dtype=torch.int64), attention_mask=torch.ones(1, 3, dtype=torch.int64)) for s in sample_data()]
    pkg.ActivationWriter(cfg).process(data)
    out = list(pkg.CachedActivationLoader({"h0": tmp_path / "h0", "h1": tmp_path / "h1"}).process())
    assert out[0]["tokens"].shape == (2, 3) and out[0]["h0"].shape == (2, 3, 4) and out[1]["h0"].shape == (1, 3, 4)
    assert out[0]["meta"] == [{"context_idx": 1}, {"context_idx": 2}]
    assert torch.equal(out[0]["h0"][1], torch.full((3, 4), 2.0))
    # tokens that disagree between hook points are refused
    bad = load_file(str(tmp_path / "h1" / "chunk-00000000.safetensors"))
    bad["tokens"] = bad["tokens"] + 1
    save_file(bad, str(tmp_path / "h1" / "chunk-00000000.safetensors"))
    with pytest.raises(AssertionError, match="tokens mismatch"):
        list(pkg.CachedActivationLoader({"h0": tmp_path / "h0", "h1": tmp_path / "h1"}).process())
    # a chunk without a required field is refused
    save_file({"activation": torch.ones(1, 3, 4), "tokens": torch.ones(1, 3)}, str(tmp_path / "h0" / "chunk-00000000.safetensors"))
    with pytest.raises(AssertionError, match="missing 'mask' field"):
        list(pkg.CachedActivationLoader({"h0": tmp_path / "h0"}).process())


def test_activation_transformer_reference_cases(pkg):
    # tests/unit/test_activation_processors.py:92-124
    acts = [{"tokens": torch.tensor([1, 3, 2]), "h0": torch.arange(9).reshape(3, 3), "h1": torch.arange(9, 18).reshape(3, 3)}]
    out = list(pkg.ActivationTransformer().process(acts, ignore_token_ids=[1, 2]))
    assert len(out) == 1 and torch.equal(out[0]["h0"], torch.tensor([[3, 4, 5]])) and torch.equal(out[0]["h1"], torch.tensor([[12, 13, 14]]))
    out = list(pkg.ActivationTransformer().process(acts, ignore_token_ids=[3]))
    assert torch.equal(out[0]["h0"], torch.tensor([[0, 1, 2], [6, 7, 8]])) and torch.equal(out[0]["h1"], torch.tensor([[9, 10, 11], [15, 16, 17]]))
    # default: the stored mask decides, (batch, context, d) -> (kept, d), meta dropped
    d = {"tokens": torch.tensor([[1, 2], [3, 4]]), "mask": torch.tensor([[1, 0], [1, 1]]), "h0": torch.arange(8.0).reshape(2, 2, 2), "meta": [{}, {}]}
    out = list(pkg.ActivationTransformer().process([d]))[0]
    assert "meta" not in out and torch.equal(out["tokens"], torch.tensor([1, 3, 4]))
    assert torch.equal(out["h0"], torch.tensor([[0.0, 1.0], [4.0, 5.0], [6.0, 7.0]]))


def _five_samples():
    return [{"h0": torch.tensor([[3, 4, 5]]) + i * 10, "h1": torch.tensor([[12, 13, 14]]) + i * 10, "tokens": torch.tensor([[1, 2, 3]])}
            for i in range(5)]


def test_activation_batchler_reference_cases(pkg, monkeypatch):
    # tests/unit/test_activation_processors.py:228-300
    result = list(pkg.ActivationBatchler(batch_size=2).process(_five_samples()))
    assert len(result) == 3
    assert torch.equal(result[0]["h0"], torch.tensor([[3, 4, 5], [13, 14, 15]])) and torch.equal(result[0]["h1"], torch.tensor([[12, 13, 14], [22, 23, 24]]))
    assert torch.equal(result[1]["h0"], torch.tensor([[23, 24, 25], [33, 34, 35]])) and torch.equal(result[1]["h1"], torch.tensor([[32, 33, 34], [42, 43, 44]]))
    assert torch.equal(result[2]["h0"], torch.tensor([[43, 44, 45]])) and torch.equal(result[2]["h1"], torch.tensor([[52, 53, 54]]))
    assert torch.equal(result[0]["tokens"], torch.tensor([[1, 2, 3], [1, 2, 3]]))

    monkeypatch.setattr(torch, "randperm", lambda *a, **k: torch.tensor([1, 0, 2]))
    result = list(pkg.ActivationBatchler(batch_size=2, buffer_size=3).process(_five_samples()))
    assert len(result) == 3
    assert torch.equal(result[0]["h0"], torch.tensor([[13, 14, 15], [3, 4, 5]])) and torch.equal(result[0]["h1"], torch.tensor([[22, 23, 24], [12, 13, 14]]))
    assert torch.equal(result[1]["h0"], torch.tensor([[33, 34, 35], [23, 24, 25]])) and torch.equal(result[1]["h1"], torch.tensor([[42, 43, 44], [32, 33, 34]]))
    assert torch.equal(result[2]["h0"], torch.tensor([[43, 44, 45]])) and torch.equal(result[2]["h1"], torch.tensor([[52, 53, 54]]))
    assert torch.equal(result[0]["tokens"], torch.tensor([[1, 2, 3], [1, 2, 3]]))

    monkeypatch.setattr(torch, "randperm", lambda *a, **k: torch.tensor([2, 0, 1]))
    cfg = pkg.BufferShuffleConfig(perm_seed=42, generator_device="cpu")
    result = list(pkg.ActivationBatchler(batch_size=2, buffer_size=3, buffer_shuffle_config=cfg).process(_five_samples()))
    assert len(result) == 3 and "h0" in result[0] and "h1" in result[0] and "tokens" in result[0]
    assert torch.equal(result[0]["h0"], torch.tensor([[23, 24, 25], [3, 4, 5]]))


def _reference_style_batches(chunks, batch_size, buffer_size, seed):
    """The reference's buffer algorithm written the slow way it is defined (concatenate, permute, slice):
    activation/processors/activation.py:96-164, 335-395."""
    gen = torch.Generator(); gen.manual_seed(seed)
    buf = None
    out = []
    cat = lambda a, b: b if a is None else {k: torch.cat([a[k], b[k]]) for k in a}  # noqa: E731
    n = lambda b: 0 if b is None else len(next(iter(b.values())))                      # noqa: E731
    for d in chunks:
        buf = cat(buf, d)
        if buffer_size is not None:
            if n(buf) >= buffer_size:
                perm = torch.randperm(n(buf), generator=gen)
                buf = {k: v[perm] for k, v in buf.items()}
                while n(buf) >= buffer_size // 2 and n(buf) >= batch_size:
                    out.append({k: v[:batch_size] for k, v in buf.items()}); buf = {k: v[batch_size:] for k, v in buf.items()}
        else:
            while n(buf) >= batch_size:
                out.append({k: v[:batch_size] for k, v in buf.items()}); buf = {k: v[batch_size:] for k, v in buf.items()}
    while n(buf) > 0:
        out.append({k: v[:batch_size] for k, v in buf.items()}); buf = {k: v[batch_size:] for k, v in buf.items()}
    return out


@pytest.mark.parametrize("batch_size,buffer_size", [(7, None), (16, 50), (5, 64), (32, 33), (3, 200)])
def test_batchler_equals_the_concatenate_and_permute_definition(pkg, batch_size, buffer_size):
    g = torch.Generator().manual_seed(3)
    chunks = []
    for i in range(9):
        n = int(torch.randint(0, 40, (1,), generator=g))
        chunks.append({"h": torch.randn(n, 6, generator=g), "tokens": torch.randint(0, 99, (n,), generator=g)})
    want = _reference_style_batches(chunks, batch_size, buffer_size, seed=11)
    got = list(pkg.ActivationBatchler(batch_size, buffer_size, pkg.BufferShuffleConfig(perm_seed=11)).process(chunks))
    assert len(got) == len(want)
    for a, b in zip(got, want):
        assert torch.equal(a["h"], b["h"]) and torch.equal(a["tokens"], b["tokens"])
    # every row comes out exactly once
    assert sorted(torch.cat([b["tokens"] for b in got]).tolist()) == sorted(torch.cat([c["tokens"] for c in chunks]).tolist())


def test_cached_activation_stream_end_to_end_on_cpu(pkg, tmp_path):
    hooks = ["in", "out"]
    want = _write_cache(tmp_path, hooks, n_chunks=4, n_samples=3, n_ctx=6, d=8)
    batches = list(pkg.cached_activation_stream(tmp_path, hooks, batch_size=10, device="cpu"))
    kept = torch.cat([acts["in"][mask.bool()] for _, mask, acts in want])
    got = torch.cat([b["in"] for b in batches])
    assert torch.equal(got, kept) and all(b["in"].shape[0] == 10 for b in batches[:-1])
    assert torch.equal(torch.cat([b["tokens"] for b in batches]), torch.cat([t[m.bool()] for t, m, _ in want]))


def test_staged_chunk_is_tied_to_the_consumer_stream(pkg):
    """A chunk copied on the side stream is handed over by waiting for the copy on the consumer's stream and by
    recording that stream on every tensor, so the allocator cannot recycle the blocks under queued readers."""
    calls = []

    class FakeStream:
        def wait_event(self, ev):
            calls.append(("wait", ev))

    class FakeTensor(torch.Tensor):
        def record_stream(self, stream):
            calls.append(("record", stream))

    consumer, done = FakeStream(), object()
    staged = {"a": torch.zeros(2).as_subclass(FakeTensor), "tokens": torch.zeros(2, dtype=torch.long).as_subclass(FakeTensor),
              "meta": [{"x": 1}]}
    out = pkg.activation.CachedActivationLoader._hand_over(staged, done, consumer)
    assert out is staged
    assert calls[0] == ("wait", done)
    assert [c for c in calls[1:]] == [("record", consumer), ("record", consumer)]
