"""Length-bucketed batching frontend for one device.

Host-side counterpart of the reference's ``queue_manager`` / ``batch_container``
(engine.py:12-130), ``optimize_batch`` / ``Batch_Packed`` / ``Tagged_line``
(utils.py:3-60) and the ordered writer of ``Engine._engine_postprocess``
(engine.py:303-372), reduced to a single process and a single device: the
reference's reader, model and writer processes and their multiprocessing queues
become three steps of one loop.

What is kept, because it determines the (batch, seq) shapes the engine sees:

* the useful length of a line is the position of its last mask 1 plus one
  (utils.py:46-52);
* bucket edges ``[0, start, start+step, ..., end, max_seq_length]``
  (engine.py:225-232); a line goes to the first bucket whose upper edge is not
  below its length (engine.py:83-88);
* a bucket emits a batch when it holds ``batch_size`` lines, or when it is
  flushed (end of input, or too many finished lines waiting for an earlier one);
* a batch is trimmed to its longest line (utils.py:3-13);
* among the buckets that have a batch ready the one holding the earliest input
  line goes first (engine.py:117-124);
* results leave in input order (engine.py:325-361).

Differences: ready batches of a bucket leave first-in first-out (the reference
pops the newest one while ranking buckets by their oldest, engine.py:58-61); a
line whose mask has no 1 at all has length 1 rather than 512.
"""
from __future__ import annotations

import sys
from collections import deque
from typing import Callable, Iterable, List, Optional, Sequence

import numpy as np


def generate_splits(max_seq_length: int, start_split: int = 50, end_split: int = 180, split_size: int = 2) -> List[int]:
    """Bucket edges, engine.py:225-232 (defaults from the reference's config comment, engine.py:196-198)."""
    edges = [0]
    edges.extend(range(start_split, end_split + split_size, split_size))
    edges.append(max_seq_length)
    return edges


class TaggedLine:
    """One tokenised input line (utils.py:33-60)."""

    __slots__ = ("num_line", "line_data", "input_ids", "input_mask", "segment_ids", "length", "output")

    def __init__(self, num_line: int, line_data, input_ids, input_mask, segment_ids):
        self.num_line = num_line
        self.line_data = line_data
        self.input_ids = np.asarray(input_ids, dtype=np.int32)
        self.input_mask = np.asarray(input_mask, dtype=np.int32)
        self.segment_ids = np.asarray(segment_ids, dtype=np.int32)
        if not (self.input_ids.shape == self.input_mask.shape == self.segment_ids.shape) or self.input_ids.ndim != 1:
            raise ValueError("input_ids, input_mask and segment_ids must be 1-D and of equal length")
        ones = np.flatnonzero(self.input_mask == 1)
        self.length = int(ones[-1]) + 1 if ones.size else 1
        self.output = None

    def get_tensor(self, index: int):
        return (self.input_ids, self.segment_ids, self.input_mask)[index]


def optimize_batch(lines: Sequence[TaggedLine]):
    """[ids, segments, mask], each int32 [len(lines), longest line] (utils.py:3-13)."""
    max_length = max(l.length for l in lines)
    batch = []
    for i in range(3):
        arr = np.empty((len(lines), max_length), dtype=np.int32)
        for j, l in enumerate(lines):
            arr[j] = l.get_tensor(i)[:max_length]
        batch.append(arr)
    return batch


class BatchPacked:
    """A batch and the lines it came from (utils.py:15-31)."""

    def __init__(self, lines_list: List[TaggedLine], tensor):
        self.lines_list = lines_list
        self.tensor = tensor
        self.output = None

    def set_output(self, output):
        self.output = output

    def write_line(self):
        for line, out in zip(self.lines_list, self.output):
            line.output = out


class BatchContainer:
    """Lines of one length bucket (engine.py:12-61)."""

    def __init__(self, base_length: int, top_length: int, batchsize: int):
        self.base_length = base_length
        self.top_length = top_length
        self.batchsize = batchsize
        self.temp: List[TaggedLine] = []
        self.prepare: deque = deque()

    def put(self, line: TaggedLine):
        self.temp.append(line)
        if len(self.temp) == self.batchsize:
            self._batch()

    def _batch(self):
        if not self.temp:
            return
        self.prepare.append(BatchPacked(list(self.temp), optimize_batch(self.temp)))
        self.temp.clear()

    def force_enqueue(self):
        self._batch()

    @property
    def min_index(self) -> int:
        return self.prepare[0].lines_list[0].num_line if self.prepare else sys.maxsize

    def pop(self) -> BatchPacked:
        return self.prepare.popleft()


class QueueManager:
    """Routes lines to their bucket and hands out ready batches (engine.py:63-130)."""

    def __init__(self, seq_length_split: Sequence[int], batchsize: int):
        if len(seq_length_split) < 2 or any(b <= a for a, b in zip(seq_length_split, seq_length_split[1:])):
            raise ValueError("bucket edges must be strictly increasing")
        self.boardlines = list(seq_length_split)
        self.containers = [BatchContainer(a, b, batchsize) for a, b in zip(self.boardlines, self.boardlines[1:])]

    def put(self, line: TaggedLine):
        if line.length > self.boardlines[-1]:
            raise ValueError("line %d has length %d, above max_seq_length %d" %
                             (line.num_line, line.length, self.boardlines[-1]))
        q = 0
        while line.length > self.boardlines[q + 1]:
            q += 1
        self.containers[q].put(line)

    def force_enqueue(self):
        for c in self.containers:
            c.force_enqueue()

    def ready(self) -> int:
        return sum(len(c.prepare) for c in self.containers)

    def get(self) -> Optional[BatchPacked]:
        """The ready batch that holds the earliest input line, or None."""
        best = min(self.containers, key=lambda c: c.min_index)
        return best.pop() if best.prepare else None


class OrderedWriter:
    """Releases per-line results in input order (engine.py:303-372)."""

    def __init__(self, sink: Callable[[object], None]):
        self.sink = sink
        self.next_line = 0
        self.waiting = {}

    def add(self, batch: BatchPacked):
        batch.write_line()
        for line in batch.lines_list:
            if line.num_line < self.next_line or line.num_line in self.waiting:
                raise RuntimeError("line index %d is written twice" % line.num_line)
            self.waiting[line.num_line] = line
        while self.next_line in self.waiting:
            self.sink(self.waiting.pop(self.next_line))
            self.next_line += 1

    @property
    def backlog(self) -> int:
        return len(self.waiting)


class Engine:
    """Single-device ``Engine.run`` (engine.py:377-403): tokenise -> bucket -> encode -> ordered output.

    tokenize(max_seq_length, line, index) -> (index, line_data, input_ids, input_mask, segment_ids)
        as the reference's ``tokenlizer_line`` callback (engine.py:291-292).
    encode([ids, segments, mask]) -> per-line outputs [batch, ...]   (``Cuda_BERT.encode`` plus,
        if wanted, the fine-tune layer; engine.py:258-260).
    output(line_data, line_output) -> what ``sink`` receives for the line (engine.py:338-339).
    """

    def __init__(self, encode, tokenize, output=lambda data, out: out, max_seq_length: int = 200,
                 batch_size: int = 128, start_split: int = 50, end_split: int = 180, split_size: int = 2,
                 alert_size: int = 1000000):
        self.encode, self.tokenize, self.output = encode, tokenize, output
        self.max_seq_length, self.batch_size, self.alert_size = max_seq_length, batch_size, alert_size
        self.splits = generate_splits(max_seq_length, start_split, end_split, split_size)
        self.batch_shapes: List[tuple] = []          # (batch, seq) of every batch sent to the device

    def _drain(self, manager: QueueManager, writer: OrderedWriter):
        while True:
            batch = manager.get()
            if batch is None:
                return
            self.batch_shapes.append(batch.tensor[0].shape)
            batch.set_output(self.encode(batch.tensor))
            writer.add(batch)

    def run(self, lines: Iterable[str], sink: Callable[[object], None]):
        manager = QueueManager(self.splits, self.batch_size)
        writer = OrderedWriter(lambda line: sink(self.output(line.line_data, line.output)))
        for index, text in enumerate(lines):
            manager.put(TaggedLine(*self.tokenize(self.max_seq_length, text, index)))
            self._drain(manager, writer)
            if writer.backlog > self.alert_size:      # finished lines pile up behind a half-full bucket
                manager.force_enqueue()
                self._drain(manager, writer)
        manager.force_enqueue()
        self._drain(manager, writer)
        if writer.backlog:
            raise RuntimeError("%d results were never released" % writer.backlog)
