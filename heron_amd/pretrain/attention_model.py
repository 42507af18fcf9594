"""Attention cost model over tokenised points (the role of pretrain/cost_model/transformer_model.py:123-215).

Every token (one CSP variable of a point) is embedded from its kind, stage, axis, split depth and name plus its
value; one self-attention layer lets the variables of a point see each other (tile against wave grid against LDS
bytes ...), two residual blocks follow, a per-token head is averaged over the point's tokens and squashed to (0, 1):
the predicted throughput relative to the best point of the task.  There is no positional term: a point is a set of
named variables, not a sequence.  Training is plain regression (mean squared error, Adam, gradient clipping).
torch is used as a library here; the model is small enough to train on the CPU.
"""
import time

import numpy as np
import torch
from torch import nn

from .dataset import KIND_PAD, RecordSet, Vocabulary
from . import metric


class PointNet(nn.Module):
    """tokens [batch, length, 6] -> score [batch] in (0, 1)."""
    GAIN = 8.0

    def __init__(self, n_stage, n_axis, n_name, width=128, heads=8, blocks=2):
        super().__init__()
        self.kind = nn.Embedding(4, 8, padding_idx=KIND_PAD)
        self.stage = nn.Embedding(n_stage, 8)
        self.axis = nn.Embedding(n_axis, 8)
        self.depth = nn.Embedding(6, 4)
        self.name = nn.Embedding(n_name, 48)
        # the value enters as itself and through a few sinusoids, so that "is a power of two" and "is large" are both easy
        self.register_buffer("freq", torch.tensor([0.5, 1.0, 2.0, 4.0]) * (np.pi / np.log(2.0)))
        self.mix = nn.Sequential(nn.Linear(8 + 8 + 8 + 4 + 48 + 1 + 8, width), nn.ReLU(), nn.Linear(width, width), nn.ReLU())
        self.attention = nn.MultiheadAttention(width, heads, batch_first=True)
        self.norm = nn.LayerNorm(width)
        self.blocks = nn.ModuleList([nn.Sequential(nn.Linear(width, width), nn.ReLU()) for _ in range(blocks)])
        self.head = nn.Sequential(nn.Linear(width, width // 2), nn.ReLU(), nn.Linear(width // 2, 1))

    def forward(self, tokens, value_scale):
        ids = tokens[..., :5].long()
        pad = ids[..., 0] == KIND_PAD
        value = tokens[..., 5:6] / value_scale
        waves = tokens[..., 5:6] * self.freq
        x = torch.cat([self.kind(ids[..., 0]), self.stage(ids[..., 1].clamp(max=self.stage.num_embeddings - 1)),
                       self.axis(ids[..., 2].clamp(max=self.axis.num_embeddings - 1)), self.depth(ids[..., 3].clamp(max=5)),
                       self.name(ids[..., 4].clamp(max=self.name.num_embeddings - 1)), value,
                       torch.sin(waves), torch.cos(waves)], dim=-1)
        x = self.mix(x)
        seen, _ = self.attention(x, x, x, key_padding_mask=pad, need_weights=False)
        x = self.norm(x + seen)
        for block in self.blocks:
            x = x + block(x)
        per_token = self.head(x).squeeze(-1).masked_fill(pad, 0.0)
        # the mean over the point's tokens, not the sum: a hundred tokens would saturate the sigmoid from the first step
        live = (~pad).sum(dim=1).clamp(min=1)
        return torch.sigmoid(per_token.sum(dim=1) / live * self.GAIN)


class AttentionCostModel:
    """What ``Tuner.setPretrainedModel`` takes: ``predict(samples)`` for the search, ``fit`` / ``finetune`` /
    ``evaluate`` / ``save`` / ``load`` around it."""

    def __init__(self, device="cpu", width=128, lr=7e-4, weight_decay=1e-6, batch_size=256, grad_clip=0.5, seed=0):
        self.device = torch.device(device)
        self.width, self.lr, self.weight_decay = width, lr, weight_decay
        self.batch_size, self.grad_clip, self.seed = batch_size, grad_clip, seed
        self.vocab = None
        self.net = None
        self.value_scale = 1.0
        self.history = []

    # ------------------------------------------------------------------------------------------------ training
    def _build(self, vocab):
        torch.manual_seed(self.seed)
        # headroom in the tables: a later fine-tuning set may add a few names
        self.net = PointNet(vocab.size("stage") + 8, vocab.size("axis") + 8, vocab.size("name") + 64,
                            width=self.width).to(self.device)

    def _epochs(self, data, valid, n_epoch, verbose):
        tokens, labels = data.padded()
        x = torch.from_numpy(tokens).to(self.device)
        y = torch.from_numpy(labels).to(self.device)
        opt = torch.optim.Adam(self.net.parameters(), lr=self.lr, weight_decay=self.weight_decay)
        loss_fn = nn.MSELoss()
        gen = torch.Generator().manual_seed(self.seed)
        for epoch in range(n_epoch):
            started = time.time()
            self.net.train()
            order = torch.randperm(len(x), generator=gen)
            running = 0.0
            for at in range(0, len(order), self.batch_size):
                pick = order[at:at + self.batch_size].to(self.device)
                opt.zero_grad()
                loss = loss_fn(self.net(x[pick], self.value_scale), y[pick])
                loss.backward()
                nn.utils.clip_grad_norm_(self.net.parameters(), self.grad_clip)
                opt.step()
                running += loss.item() * len(pick)
            row = {"epoch": epoch, "train_rmse": float(np.sqrt(running / max(len(x), 1)))}
            if valid is not None and len(valid):
                row.update(self.evaluate(valid))
            self.history.append(row)
            if verbose and (epoch % verbose == 0 or epoch == n_epoch - 1):
                print("epoch %d  train rmse %.4f  %s  (%.1f s)" % (
                    epoch, row["train_rmse"], "  ".join("%s %.3f" % (k, v) for k, v in row.items()
                                                         if k not in ("epoch", "train_rmse", "tasks")), time.time() - started))

    def fit(self, train, valid=None, n_epoch=60, verbose=10):
        """Trains a fresh network on ``train`` (a RecordSet); its vocabulary is frozen and kept with the model."""
        self.vocab = train.vocab
        self.vocab.frozen = True
        tokens, _ = train.padded()
        self.value_scale = float(max(tokens[..., 5].max(), 1.0))
        self._build(self.vocab)
        self._epochs(train, valid, n_epoch, verbose)
        return self

    fit_base = fit          # the reference's name for it (transformer_model.py:218)

    def finetune(self, train, n_epoch=10, verbose=0):
        """Continues training on the records of a new task (its unseen names stay 'unknown')."""
        assert self.net is not None, "fit or load a model first"
        self._epochs(train, None, n_epoch, verbose)
        return self

    # ------------------------------------------------------------------------------------------------ inference
    def _scores(self, tokens):
        self.net.eval()
        out = []
        with torch.no_grad():
            for at in range(0, len(tokens), 4096):
                out.append(self.net(torch.from_numpy(tokens[at:at + 4096]).to(self.device), self.value_scale).cpu())
        return torch.cat(out).numpy() if out else np.zeros(0, np.float32)

    def predict(self, inp, output_margin=False):
        """A RecordSet, or the list of samples a tuner asks about -> {task: scores}."""
        if not isinstance(inp, RecordSet):
            samples = list(inp)
            if not samples:
                return np.zeros(0)
            data = RecordSet(self.vocab)
            data.add_samples(samples[0].task.name, samples)
            inp = data
        return {task: self._scores(inp.padded(task)[0]) for task in inp.tasks()}

    def evaluate(self, data):
        return metric.summary(self.predict(data), data.labels)

    def train(self, perf_buffer):            # Tuner hook: a pre-trained model is not re-fitted during the search
        return

    # ------------------------------------------------------------------------------------------------ files
    def save(self, path):
        """Tensors and plain Python values only, so that the file loads with ``weights_only=True``."""
        torch.save({"state": {k: v.cpu() for k, v in self.net.state_dict().items()}, "vocab": self.vocab.to_dict(),
                    "value_scale": self.value_scale, "width": self.width}, path)

    def load(self, path):
        blob = torch.load(path, map_location="cpu", weights_only=True)
        self.vocab = Vocabulary.from_dict(blob["vocab"])
        self.value_scale, self.width = float(blob["value_scale"]), int(blob["width"])
        self._build(self.vocab)
        self.net.load_state_dict(blob["state"])
        self.net.to(self.device)
        return self
