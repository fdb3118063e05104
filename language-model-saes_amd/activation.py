"""Activation data either side of the train step: the cached-activation files, their reader, the mask filter
and the shuffling batchler that hands `[batch, d_model]` tensors to `Trainer.fit`.

File layout and processor semantics are the reference's
(`activation/writer.py:59-190`, `activation/processors/cached_activation.py:84-420`,
`activation/processors/activation.py:26-164, 228-395`):

    <cache_dir>/<hook_point>/chunk-00000000.safetensors            activation, tokens, mask, attention_mask
    <cache_dir>/<hook_point>/chunk-00000000.meta.json              (optional)
    <cache_dir>/<hook_point>/shard-3-chunk-00000007.pt             the sharded / torch.save variants

What differs is where the bytes live.  The reference's `ActivationBuffer` re-concatenates and permutes the
whole shuffle buffer for every refill and every batch; here the buffer is a fixed slab per key (in HBM when
the stream is on the GPU), a shuffle permutes row indices on the host, and a batch is one gather kernel
(`ops.gather_rows`, with the dtype override and a scale folded in).  Given the same `torch.randperm` draws
the batches are the reference's, row for row.  The reader stages each chunk through pinned host memory and
copies it on a side stream while the previous chunk is being consumed.
"""

from __future__ import annotations

import json
import os
import re
import threading
from dataclasses import dataclass
from pathlib import Path
from queue import Queue
from typing import Any, Iterable, Iterator, Literal, Mapping, Optional, Sequence

import torch
from pydantic import BaseModel

from . import ops


# ---- writer (activation/writer.py) ----------------------------------------------------------------

class ActivationWriterConfig(BaseModel):
    hook_points: list[str]
    total_generating_tokens: Optional[int] = None
    n_samples_per_chunk: Optional[int] = None
    cache_dir: str = "activations"
    format: str = "safetensors"      # "pt" | "safetensors"; anything else is rejected when a chunk is written
    num_workers: Optional[int] = None


class ActivationWriter:
    """Writes `{hook: [..., d], tokens, mask, ..., meta}` samples as chunk files the loader below (and the
    reference's loader) reads.  `n_samples_per_chunk` stacks that many samples into one chunk."""

    def __init__(self, cfg: ActivationWriterConfig):
        self.cfg = cfg
        self.cache_dir = Path(cfg.cache_dir)
        for hp in cfg.hook_points:
            (self.cache_dir / hp).mkdir(parents=True, exist_ok=True)

    def _write_chunk(self, hook_point: str, chunk_data: dict, chunk_name: str, meta=None) -> None:
        path = self.cache_dir / hook_point / f"{chunk_name}.{self.cfg.format}"
        if self.cfg.format == "pt":
            torch.save(chunk_data | ({"meta": meta} if meta is not None else {}), path)
        elif self.cfg.format == "safetensors":
            from safetensors.torch import save_file

            save_file({k: v.detach().cpu().contiguous() for k, v in chunk_data.items()}, str(path))
            if meta is not None:
                with open(path.with_suffix(".meta.json"), "w") as f:
                    json.dump(meta, f)
        else:
            raise ValueError(f"Invalid format: {self.cfg.format}")

    def process(self, data: Iterable[dict[str, Any]], *, start_shard: Optional[int] = None) -> None:
        def batched(it, n):
            group = []
            for x in it:
                group.append(x)
                if len(group) == n:
                    yield group
                    group = []
            if group:
                yield group

        def collate(group: Sequence[dict]) -> dict:
            assert all(k in d for k in group[0] for d in group), f"All samples must have the same keys: {group[0].keys()}"
            return {k: torch.stack([d[k] for d in group]) if isinstance(group[0][k], torch.Tensor) else [d[k] for d in group]
                    for k in group[0].keys()}

        if self.cfg.n_samples_per_chunk is not None:
            data = map(collate, batched(data, self.cfg.n_samples_per_chunk))
        written = 0
        pool = None
        if self.cfg.num_workers is not None:
            from concurrent.futures import ThreadPoolExecutor

            pool = ThreadPoolExecutor(max_workers=self.cfg.num_workers)
        futures = []
        try:
            for chunk_id, chunk in enumerate(data):
                assert all(k in chunk for k in self.cfg.hook_points), f"All samples must have the hook points: {self.cfg.hook_points}"
                name = f"chunk-{chunk_id:08d}" if start_shard is None else f"shard-{start_shard}-chunk-{chunk_id:08d}"
                for hp in self.cfg.hook_points:
                    payload = {"activation": chunk[hp]} | {k: v for k, v in chunk.items() if k not in ["meta", *self.cfg.hook_points]}
                    if pool is None:
                        self._write_chunk(hp, payload, name, chunk.get("meta"))
                    else:
                        futures.append(pool.submit(self._write_chunk, hp, payload, name, chunk.get("meta")))
                written += chunk["tokens"].numel()
                if self.cfg.total_generating_tokens is not None and written >= self.cfg.total_generating_tokens:
                    break
            for f in futures:
                f.result()
        finally:
            if pool is not None:
                pool.shutdown(wait=True)


# ---- reader (activation/processors/cached_activation.py) ---------------------------------------------

@dataclass
class ChunkInfo:
    path: Path
    shard_id: int
    chunk_id: int

    @classmethod
    def from_path(cls, path: Path) -> "ChunkInfo":
        m = re.match(r"shard-(\d+)-chunk-(\d+)\.(pt|safetensors)", path.name)
        if m:
            return cls(path=path, shard_id=int(m.group(1)), chunk_id=int(m.group(2)))
        m = re.match(r"chunk-(\d+)\.(pt|safetensors)", path.name)
        if m:
            return cls(path=path, shard_id=0, chunk_id=int(m.group(1)))
        raise ValueError(f"Invalid chunk filename format: {path.name}. "
                         "Expected 'shard-{N}-chunk-{N}.(pt|safetensors)' or 'chunk-{N}.(pt|safetensors)'")


_REQUIRED = ("activation", "tokens", "mask", "attention_mask")


class CachedActivationLoader:
    """Streams cached chunks in (shard, chunk) order; one output dict per chunk index with every hook point's
    activation under its name plus tokens / mask / attention_mask / meta, leading sample dims flattened
    until `tokens` is at most 2-D (cached_activation.py:318-420).  With a GPU `device`, chunk i + 1 is read
    from disk by a worker thread into pinned memory and copied on a side stream while chunk i is in use."""

    def __init__(self, cache_dirs: Mapping[str, str | Path], device: str = "cpu", dtype: Optional[torch.dtype] = None,
                 prefetch: int = 2):
        self.cache_dirs = {k: Path(v) for k, v in cache_dirs.items()}
        self.device = torch.device(device)
        self.dtype = dtype
        self.prefetch = max(1, int(prefetch))

    def _get_sorted_chunks(self, hook_point: str) -> list[ChunkInfo]:
        hook_dir = self.cache_dirs[hook_point]
        if not hook_dir.exists():
            raise FileNotFoundError(f"Hook point directory not found: {hook_dir}")
        chunks = [ChunkInfo.from_path(p)
                  for pattern in ["shard-*-chunk-*.pt", "shard-*-chunk-*.safetensors", "chunk-*.pt", "chunk-*.safetensors"]
                  for p in hook_dir.glob(pattern)]
        return sorted(chunks, key=lambda c: (c.shard_id, c.chunk_id))

    @staticmethod
    def _load_chunk(chunk_path: Path) -> dict[str, Any]:
        if chunk_path.suffix == ".safetensors":
            from safetensors.torch import load_file

            data: dict[str, Any] = load_file(str(chunk_path), device="cpu")
            meta_path = chunk_path.with_suffix(".meta.json")
            if meta_path.exists():
                with open(meta_path, "r") as f:
                    data = data | {"meta": json.load(f)}
            return data
        if chunk_path.suffix == ".pt":
            return torch.load(chunk_path, map_location="cpu", weights_only=True)
        raise ValueError(f"Invalid chunk file format: {chunk_path}. Expected .safetensors or .pt")

    def _read_chunk_index(self, i: int, hook_chunks: dict[str, list[ChunkInfo]]) -> dict[str, Any]:
        out: dict[str, Any] = {}
        for hp, chunks in hook_chunks.items():
            path = chunks[i].path
            data = self._load_chunk(path)
            assert isinstance(data, dict), f"Loading cached activation {path} error: returned {type(data)}"
            for field in _REQUIRED:
                assert field in data, f"Loading cached activation {path} error: missing '{field}' field"
            if not out:
                out = {"tokens": data["tokens"], "mask": data["mask"], "attention_mask": data["attention_mask"],
                       "meta": data.get("meta")}
            elif not torch.equal(data["tokens"], out["tokens"]):
                raise AssertionError(f"Loading cached activation error: tokens mismatch for chunk {i}")
            act = data["activation"]
            out[hp] = act.to(self.dtype) if self.dtype is not None else act
        while out["tokens"].ndim >= 3:
            out = {k: (v.flatten(0, 1) if isinstance(v, torch.Tensor) else ([a for b in v for a in b] if v is not None else None))
                   for k, v in out.items()}
        return out

    @staticmethod
    def _pin(chunk: dict[str, Any]) -> dict[str, Any]:
        """Copy the chunk's tensors into freshly allocated pinned host memory (runs on the reader thread)."""
        out = {}
        for k, v in chunk.items():
            if isinstance(v, torch.Tensor):
                pinned = torch.empty(v.shape, dtype=v.dtype, pin_memory=True)
                pinned.copy_(v)
                out[k] = pinned
            else:
                out[k] = v
        return out

    def _to_device(self, chunk: dict[str, Any], stream) -> tuple[dict[str, Any], Any]:
        staged = {}
        with torch.cuda.stream(stream):
            for k, v in chunk.items():
                if isinstance(v, torch.Tensor):
                    staged[k] = v.to(self.device, non_blocking=True)
                else:
                    staged[k] = v
            done = torch.cuda.Event()
            done.record(stream)
        return staged, (done, chunk)   # the pinned source stays referenced until the copy has been waited for

    @staticmethod
    def _hand_over(staged: dict[str, Any], done, consumer) -> dict[str, Any]:
        """Give a staged chunk to the stream that will read it.  The tensors were allocated on the copy stream, so
        the caching allocator would reuse their blocks for a later host-to-device copy as soon as the consumer drops
        them, while kernels queued on the consumer stream may still be reading: `record_stream(consumer)` defers that
        reuse until the consumer's queued work has passed."""
        consumer.wait_event(done)
        for v in staged.values():
            if isinstance(v, torch.Tensor):
                v.record_stream(consumer)
        return staged

    def process(self, data: None = None, **kwargs) -> Iterator[dict[str, Any]]:
        hook_chunks = {hp: self._get_sorted_chunks(hp) for hp in self.cache_dirs}
        counts = {hp: len(c) for hp, c in hook_chunks.items()}
        if len(set(counts.values())) != 1:
            raise ValueError(f"Hook points have different numbers of chunks: {counts}. "
                             "All hook points must have the same number of chunks.")
        n = next(iter(counts.values()))
        if self.device.type != "cuda":
            for i in range(n):
                yield self._read_chunk_index(i, hook_chunks)
            return

        q: Queue = Queue(maxsize=self.prefetch)
        stop = threading.Event()

        def reader():
            try:
                for i in range(n):
                    if stop.is_set():
                        return
                    q.put(("chunk", self._pin(self._read_chunk_index(i, hook_chunks))))
                q.put(("end", None))
            except BaseException as e:  # noqa: BLE001  (handed to the consumer, which re-raises)
                q.put(("error", e))

        t = threading.Thread(target=reader, daemon=True)
        t.start()
        copy_stream = torch.cuda.Stream(device=self.device)
        try:
            pending = None
            while True:
                kind, payload = q.get()
                if kind == "error":
                    raise payload
                nxt = self._to_device(payload, copy_stream) if kind == "chunk" else None
                if pending is not None:
                    staged, (done, _host) = pending
                    yield self._hand_over(staged, done, torch.cuda.current_stream(self.device))
                pending = nxt
                if kind == "end":
                    break
        finally:
            stop.set()
            while t.is_alive():
                try:
                    q.get_nowait()
                except Exception:  # noqa: BLE001
                    pass
                t.join(timeout=0.05)


# ---- mask filter (activation/processors/activation.py:228-288) ------------------------------------------

class ActivationTransformer:
    """Keeps the tokens whose `mask` is set (or whose id is not in `ignore_token_ids`), flattening
    (batch, context, d) to (kept tokens, d); non-tensor fields (meta) are dropped."""

    def process(self, data: Iterable[dict[str, Any]], *, ignore_token_ids: Optional[list[int]] = None, **kwargs):
        for d in data:
            assert "tokens" in d and isinstance(d["tokens"], torch.Tensor)
            tokens = d["tokens"]
            if ignore_token_ids is not None:
                mask = torch.isin(tokens, torch.tensor(ignore_token_ids).to(tokens.device), invert=True)
            else:
                mask = d["mask"].bool()
            yield {k: v[mask] for k, v in d.items() if isinstance(v, torch.Tensor)}


# ---- shuffling batchler (activation/processors/activation.py:18-164, 297-395) -----------------------------

class BufferShuffleConfig(BaseModel):
    perm_seed: int = 42
    generator_device: Optional[str] = None


class _RowStore:
    """Rows of one key in a fixed slab; logical order is kept by the batchler as a list of slab rows."""

    def __init__(self, like: torch.Tensor, capacity: int):
        self.data = torch.empty((capacity, *like.shape[1:]), dtype=like.dtype, device=like.device)

    def grow(self, capacity: int) -> None:
        if capacity > self.data.shape[0]:
            bigger = torch.empty((capacity, *self.data.shape[1:]), dtype=self.data.dtype, device=self.data.device)
            bigger[: self.data.shape[0]] = self.data
            self.data = bigger

    def put(self, rows: torch.Tensor, slots_host: torch.Tensor) -> None:
        n = rows.shape[0]
        first = int(slots_host[0])
        if int(slots_host[-1]) - first == n - 1:      # slots are handed out ascending: contiguous means a plain slice
            self.data[first:first + n] = rows
        else:
            self.data.index_copy_(0, slots_host.to(self.data.device), rows.to(self.data.dtype))

    def take(self, idx_host: torch.Tensor, out_dtype: Optional[torch.dtype], scale: float) -> torch.Tensor:
        d = self.data
        floaty = d.ndim == 2 and d.dtype in (torch.float32, torch.bfloat16)
        if d.is_cuda and floaty:
            return ops.gather_rows(d, idx_host.to(d.device), out_dtype=out_dtype or d.dtype, scale=scale)
        out = d.index_select(0, idx_host.to(d.device))
        if floaty or d.is_floating_point():
            if scale != 1.0:
                out = out * scale
            if out_dtype is not None:
                out = out.to(out_dtype)
        return out


class ActivationBatchler:
    """Batches (and optionally shuffles) token rows exactly as the reference's `ActivationBatchler`:
    with `buffer_size`, rows accumulate until the buffer holds that many, the buffer is shuffled, and batches
    are drawn until it is half empty; without, full batches are cut in arrival order; the tail is flushed in
    batches at the end.  `override_dtype` / `scale` apply to floating-point rows on the way out."""

    def __init__(self, batch_size: int, buffer_size: Optional[int] = None,
                 buffer_shuffle_config: Optional[BufferShuffleConfig] = None, override_dtype: Optional[torch.dtype] = None,
                 scale: float = 1.0):
        self.batch_size = batch_size
        self.buffer_size = buffer_size
        self.override_dtype = override_dtype
        self.scale = float(scale)
        self.perm_generator = torch.Generator()
        if buffer_shuffle_config is not None:
            self.perm_generator = torch.Generator(buffer_shuffle_config.generator_device)
            self.perm_generator.manual_seed(buffer_shuffle_config.perm_seed)

    def process(self, data: Iterable[dict[str, Any]], **kwargs) -> Iterator[dict[str, torch.Tensor]]:
        stores: dict[str, _RowStore] = {}
        lists: dict[str, list] = {}          # non-tensor fields travel in arrival order (no shuffling with them)
        order = torch.empty(0, dtype=torch.int64)   # slab rows in logical order
        free = torch.empty(0, dtype=torch.int64)    # slab rows not in use, ascending
        capacity = 0

        def alloc(n: int) -> torch.Tensor:
            """n free slab rows, ascending (the slabs grow when too few are free)."""
            nonlocal capacity, free
            if free.numel() < n:
                grown = capacity + max(n - free.numel(), capacity // 2, self.buffer_size or 0, self.batch_size)
                for s in stores.values():
                    s.grow(grown)
                free = torch.cat([free, torch.arange(capacity, grown, dtype=torch.int64)])
                capacity = grown
            slots, free = free[:n], free[n:]
            return slots

        def release(rows: torch.Tensor) -> None:
            nonlocal free
            if rows.numel():
                free = torch.cat([free, rows]).sort().values

        def take(n: int) -> dict[str, Any]:
            nonlocal order
            idx, order = order[:n], order[n:]
            batch: dict[str, Any] = {k: s.take(idx, self.override_dtype, self.scale) for k, s in stores.items()}
            for k in lists:
                batch[k], lists[k] = lists[k][:n], lists[k][n:]
            release(idx)
            return batch

        for d in data:
            n = len(d[next(iter(d.keys()))])
            assert all(len(d[k]) == n for k in d.keys()), (
                f"All tensors and lists must have the same batch size, {[(k, len(d[k])) for k in d.keys()]}")
            if n > 0:
                tensors = {k: v for k, v in d.items() if isinstance(v, torch.Tensor)}
                for k, v in tensors.items():
                    if k not in stores:
                        stores[k] = _RowStore(v, capacity)
                slots = alloc(n)
                for k, v in tensors.items():
                    stores[k].put(v, slots)
                for k, v in d.items():
                    if not isinstance(v, torch.Tensor):
                        lists.setdefault(k, []).extend(v)
                order = torch.cat([order, slots])
            if self.buffer_size is not None:
                if order.numel() >= self.buffer_size:
                    assert not lists, "All data must be tensors to perform shuffling"
                    perm = torch.randperm(order.numel(), generator=self.perm_generator, device=self.perm_generator.device)
                    order = order[perm.cpu()]
                    while order.numel() >= self.buffer_size // 2 and order.numel() >= self.batch_size:
                        yield take(self.batch_size)
            else:
                while order.numel() >= self.batch_size:
                    yield take(self.batch_size)
        while order.numel() > 0:
            yield take(self.batch_size)


def cached_activation_stream(cache_dir: str | Path, hook_points: Sequence[str], *, batch_size: int,
                             buffer_size: Optional[int] = None, buffer_shuffle_config: Optional[BufferShuffleConfig] = None,
                             device: str = "cuda", dtype: Optional[torch.dtype] = None,
                             override_dtype: Optional[torch.dtype] = None) -> Iterator[dict[str, torch.Tensor]]:
    """Loader -> mask filter -> batchler, the chain the reference's ActivationFactory builds for a cached
    source with a batch size (activation/factory.py:246-345): yields `{hook: [batch, d], tokens: [batch], ...}`."""
    loader = CachedActivationLoader({hp: os.path.join(str(cache_dir), hp) for hp in hook_points}, device=device, dtype=dtype)
    batchler = ActivationBatchler(batch_size, buffer_size, buffer_shuffle_config, override_dtype=override_dtype)
    return batchler.process(ActivationTransformer().process(loader.process()))
