"""Attention cost model over tokenised records: tokeniser, metrics (hand-checked values), training, files, and its use
by the search loop (Tuner.run_with_pretrained).  Runs on the CPU; no GPU code is involved."""
import json
import os

import numpy as np
import pytest
import torch

from heron_amd.pretrain import AttentionCostModel, RecordSet, Vocabulary, metric
from heron_amd.pretrain.dataset import KIND_KNOB, KIND_OTHER, KIND_VAR, tokenize

HERE = os.path.dirname(os.path.abspath(__file__))
RECORDS = os.path.join(HERE, "pretrain", "records")


def test_tokeniser_and_vocabulary():
    v = Vocabulary()
    p = {"P#ST:dense,AX:None,PA:mfma": 16, "O#ST:dense,AX:None,PA:mfma_cand0": 1, "V#ST:dense,AX:i.outer.inner,VA:block_m": 255,
         "L#ST:dense,AX:i": 4096, "free": 0}
    t = tokenize(p, v)
    assert t.shape == (3, 6)                                   # the O# and L# entries are left out
    assert t[0, 0] == KIND_KNOB and t[1, 0] == KIND_VAR and t[2, 0] == KIND_OTHER
    assert t[0, 1] == t[1, 1] == 1 and t[2, 1] == 0            # stage 'dense' is id 1, no stage is 0
    assert t[0, 2] == 0 and t[1, 2] == 1 and t[1, 3] == 2      # axis 'i' with two split levels
    assert abs(t[0, 5] - np.log(17.0)) < 1e-6 and t[1, 5] == np.float32(np.log(256.0)) and t[2, 5] == 0
    assert v.tables["name"] == ["mfma", "block_m", "free"]
    v.frozen = True
    t2 = tokenize({"P#ST:other,AX:None,PA:unknown_knob": 3, "P#ST:dense,AX:None,PA:mfma": 32}, v)
    assert t2[0, 1] == 0 and t2[0, 4] == 0 and t2[1, 4] == 1   # unseen names map to 0 once frozen
    assert Vocabulary.from_dict(v.to_dict()).tables == v.tables


def test_metrics_known_answers():
    labels = np.array([1.0, 0.5, 0.25, 0.75])
    perfect, reverse = labels.copy(), -labels
    assert metric.rmse(perfect, labels) == 0 and metric.r_squared(perfect, labels) == 1
    assert abs(metric.rmse(labels + 0.5, labels) - 0.5) < 1e-12
    assert metric.r_squared(np.full(4, labels.mean()), labels) == 0
    assert metric.pairwise_accuracy(perfect, labels) == 1 and metric.pairwise_accuracy(reverse, labels) == 0
    assert metric.pairwise_accuracy(np.array([4.0, 1.0, 2.0, 3.0]), labels) == 5 / 6.0   # one of six pairs swapped
    assert metric.top_k_recall(perfect, labels, 2) == 1 and metric.top_k_recall(reverse, labels, 2) == 0
    assert metric.peak_score(perfect, labels, 1) == 1 and metric.peak_score(reverse, labels, 1) == 0.25
    # picks in predicted order measure 0.25, 0.5, 0.75: running best / best of all, averaged
    assert abs(metric.peak_score(reverse, labels, 3) - (0.25 + 0.5 + 0.75) / 3) < 1e-12
    s = metric.summary({"a": perfect, "b": reverse}, {"a": labels, "b": labels})
    assert s["tasks"] == 2 and s["pairwise accuracy"] == 0.5 and s["peak score@1"] == 0.625


def test_record_set_labels_and_splits():
    data = RecordSet()
    n = data.add_tree(RECORDS)
    assert n == len(data) == 1150 and len(data.tasks()) == 9
    for task in data.tasks():
        y = data.labels[task]
        assert y.max() == 1.0 and 0 < y.min() < 1 and len(y) == len(data.tokens[task])
    rows = [{"perf": 0, "param": {}}, {"perf": np.log(1 / 2e-3), "param": {"P#ST:s,AX:None,PA:k": 1}},
            {"perf": np.log(1 / 1e-3), "param": {"P#ST:s,AX:None,PA:k": 2}}]
    tiny = RecordSet()
    assert tiny.add_rows("t", rows) == 2                        # the failed measurement is dropped
    assert np.allclose(tiny.labels["t"], [0.5, 1.0])            # throughput relative to the task's best
    seen, unseen = data.split_by_task(["GEMM_F16_4096"])
    assert unseen.tasks() == ["GEMM_F16_4096"] and len(seen) + len(unseen) == 1150
    train, valid = seen.split_within_tasks(0.9)
    assert len(train) + len(valid) == len(seen) and set(valid.tasks()) <= set(train.tasks())
    x, y = train.padded()
    assert x.shape == (len(train), data.max_tokens(), 6) and y.shape == (len(train),)


@pytest.fixture(scope="module")
def trained():
    data = RecordSet()
    data.add_tree(RECORDS)
    seen, unseen = data.split_by_task(["GEMM_F16_4096"])
    model = AttentionCostModel().fit(seen, None, n_epoch=40, verbose=0)
    return model, seen, unseen


def test_training_learns_to_rank_a_task_it_never_saw(trained):
    model, seen, unseen = trained
    assert model.history[-1]["train_rmse"] < 0.6 * model.history[0]["train_rmse"]
    r = model.evaluate(unseen)
    # measured with this seed: pairwise accuracy 0.78, peak score@5 0.98; chance is 0.5 and about 0.8
    assert r["pairwise accuracy"] > 0.65 and r["peak score@5"] > 0.9, r
    assert model.evaluate(seen)["pairwise accuracy"] > 0.7


def test_save_and_load_give_the_same_scores(trained, tmp_path):
    model, _, unseen = trained
    path = str(tmp_path / "m.pt")
    model.save(path)
    blob = torch.load(path, map_location="cpu", weights_only=True)      # nothing in the file needs unpickling of code
    assert set(blob) == {"state", "vocab", "value_scale", "width"}
    again = AttentionCostModel().load(path)
    a, b = model.predict(unseen), again.predict(unseen)
    assert np.allclose(a["GEMM_F16_4096"], b["GEMM_F16_4096"], atol=1e-6)


def test_search_steered_by_the_pretrained_model(trained, tmp_path):
    """Env.tune with config.pretrained_model: the saved model scores the samples of a new task (dictionary by task
    name, as the reference's model returns) and run_with_pretrained measures its picks without re-training."""
    from test_tuner_cpu import make_env
    model, _, _ = trained
    path = str(tmp_path / "m.pt")
    model.save(path)
    env = make_env(tmp_path, method="CGA", trials=16, case=("gemm", [2048, 2048, 2048]))
    env.config.pretrained_model, env.config.search_generations = path, 2
    env.tune("T1")
    rows = [json.loads(l) for l in open(os.path.join(env.config.log_dir, "records.txt"))]
    assert 8 <= len(rows) <= 16
    tuner_model = env.tuner.cost_model
    assert isinstance(tuner_model, AttentionCostModel)
    samples = env.tuner.constrained_random_sample(env, 8)
    scores = tuner_model.predict(samples)
    assert list(scores) == ["T1"] and scores["T1"].shape == (len(samples),) and np.all((scores["T1"] > 0) & (scores["T1"] < 1))
    assert all(0 < s.predict < 1 for s in samples)
