"""Records -> token sequences.

A measured point is the dictionary of its CSP variables (``records.txt`` rows carry it as ``param``).  Each knob
(``P#ST:<stage>,AX:<axis>,PA:<name>``) and each derived variable (``V#ST:...,VA:<name>``) becomes one token
(kind, stage id, axis id, split depth, name id, ln(1 + value)); one-hot companions (``O#``) and loop lengths (``L#``)
are left out, as pretrain/dataset.py:95-129 of the reference does.  Ids come from a vocabulary that grows while a
training set is read and is frozen afterwards (unseen names map to 0).  The label of a point is its throughput relative
to the best point of its own task, so tasks of different sizes mix.
"""
import gzip
import json
import math
import os

import numpy as np

KIND_PAD, KIND_KNOB, KIND_VAR, KIND_OTHER = 0, 1, 2, 3
TOKEN_WIDTH = 6             # kind, stage, axis, split depth, name, value
SKIPPED_PREFIXES = ("O#", "L#")


class Vocabulary:
    """Name tables of stages, axes and variables; id 0 is 'none / unseen'."""

    def __init__(self, stages=(), axes=(), names=()):
        self.tables = {"stage": list(stages), "axis": list(axes), "name": list(names)}
        self.frozen = False

    def lookup(self, table, word):
        if word in (None, "None", ""):
            return 0
        words = self.tables[table]
        if word in words:
            return words.index(word) + 1
        if self.frozen:
            return 0
        words.append(word)
        return len(words)

    def size(self, table):
        return len(self.tables[table]) + 1

    def to_dict(self):
        return {k: list(v) for k, v in self.tables.items()}

    @classmethod
    def from_dict(cls, d):
        v = cls(d.get("stage", ()), d.get("axis", ()), d.get("name", ()))
        v.frozen = True
        return v


def _field(text, tag):
    return text.split(tag, 1)[1] if tag in text else None


def tokenize(param, vocab):
    """``param`` dictionary -> float32 array (tokens, TOKEN_WIDTH)."""
    rows = []
    for key, value in param.items():
        if key.startswith(SKIPPED_PREFIXES):
            continue
        if key.startswith(("P#", "V#")):
            kind = KIND_KNOB if key[0] == "P" else KIND_VAR
            stage, axis, name = key[2:].split(",", 2)
            axis_name = _field(axis, "AX:")
            depth = 0
            if axis_name not in (None, "None"):
                parts = axis_name.split(".")
                axis_name, depth = parts[0], min(len(parts) - 1, 5)
            rows.append((kind, vocab.lookup("stage", _field(stage, "ST:")), vocab.lookup("axis", axis_name), depth,
                         vocab.lookup("name", _field(name, "PA:" if kind == KIND_KNOB else "VA:")),
                         math.log1p(max(float(value), 0.0))))
        else:
            rows.append((KIND_OTHER, 0, 0, 0, vocab.lookup("name", key), math.log1p(max(float(value), 0.0))))
    return np.array(rows, dtype=np.float32).reshape(-1, TOKEN_WIDTH)


class RecordSet:
    """Per task: a list of token arrays and the relative-throughput labels of the same points."""

    def __init__(self, vocab=None):
        self.vocab = vocab or Vocabulary()
        self.tokens = {}
        self.labels = {}

    # ------------------------------------------------------------------ filling
    def add_rows(self, task, rows):
        """``rows``: parsed records ({"perf": ln(1/s), "param": {...}}); failed measurements (perf 0) are dropped."""
        rows = [r for r in rows if r.get("perf", 0) != 0]
        if not rows:
            return 0
        best = max(r["perf"] for r in rows)
        self.tokens.setdefault(task, []).extend(tokenize(r["param"], self.vocab) for r in rows)
        self.labels[task] = np.concatenate([self.labels.get(task, np.zeros(0, np.float32)),
                                            np.array([math.exp(r["perf"] - best) for r in rows], np.float32)])
        return len(rows)

    def add_file(self, task, path):
        """One records file: the tuner's ``records.txt`` or a gzip-compressed copy (``*.jsonl.gz``)."""
        opener = gzip.open if path.endswith(".gz") else open
        with opener(path, "rt") as f:
            return self.add_rows(task, [json.loads(line) for line in f if line.strip()])

    def add_tree(self, root):
        """Every ``<root>/**/<case>/records.txt`` (task name = the path below ``root``) and every ``*.jsonl.gz``
        (task name = the file's stem)."""
        count = 0
        for folder, _, files in sorted(os.walk(root)):
            for name in sorted(files):
                if name == "records.txt":
                    count += self.add_file(os.path.relpath(folder, root), os.path.join(folder, name))
                elif name.endswith(".jsonl.gz"):
                    count += self.add_file(name[:-len(".jsonl.gz")], os.path.join(folder, name))
        return count

    def add_samples(self, task, samples):
        """Unmeasured points of a search (labels are zeros): what ``predict`` is asked about."""
        self.tokens[task] = [tokenize(s.knob_manager.solved_knob_vals_phenotype, self.vocab) for s in samples]
        self.labels[task] = np.zeros(len(samples), np.float32)

    # ------------------------------------------------------------------ views
    def tasks(self):
        return list(self.tokens.keys())

    def __len__(self):
        return sum(len(v) for v in self.tokens.values())

    def max_tokens(self):
        return max((len(t) for seqs in self.tokens.values() for t in seqs), default=0)

    def subset(self, picks):
        """``picks``: task -> index array."""
        out = RecordSet(self.vocab)
        for task, idx in picks.items():
            idx = np.asarray(idx, dtype=np.int64)
            if len(idx):
                out.tokens[task] = [self.tokens[task][i] for i in idx]
                out.labels[task] = self.labels[task][idx]
        return out

    def split_within_tasks(self, ratio=0.9, rng=None):
        """Train / validation parts of every task (random ``ratio`` of its points for training)."""
        rng = rng or np.random.default_rng(0)
        train, valid = {}, {}
        for task in self.tasks():
            order = rng.permutation(len(self.tokens[task]))
            cut = max(1, int(ratio * len(order)))
            train[task], valid[task] = order[:cut], order[cut:]
        return self.subset(train), self.subset(valid)

    def split_by_task(self, held_out):
        """(all other tasks, the tasks named in ``held_out``)."""
        held = set(held_out)
        return (self.subset({t: np.arange(len(self.tokens[t])) for t in self.tasks() if t not in held}),
                self.subset({t: np.arange(len(self.tokens[t])) for t in self.tasks() if t in held}))

    def padded(self, task=None, length=None):
        """(tokens [points, length, TOKEN_WIDTH], labels [points]) of one task or of all; short sequences are padded
        with kind-0 tokens."""
        names = [task] if task is not None else self.tasks()
        seqs = [t for n in names for t in self.tokens[n]]
        labels = np.concatenate([self.labels[n] for n in names]) if names else np.zeros(0, np.float32)
        length = length or max((len(t) for t in seqs), default=1)
        out = np.zeros((len(seqs), length, TOKEN_WIDTH), np.float32)
        for i, t in enumerate(seqs):
            n = min(len(t), length)
            out[i, :n] = t[:n]
        return out, labels
