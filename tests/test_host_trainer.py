"""Host logic of the trainer patches (src/art/local/train.py:19-31, 156-174):
`train` installs and restores `compute_loss` / `log`; `log` averages the step
metrics (floats or device scalars), prefixes them for evaluation logs, drops
the learning rate and clears the store.  CPU only."""
import asyncio
import collections

import torch

from art_amd import train as T


class FakeQueue:
    def __init__(self):
        self.items = []

    def put_nowait(self, x):
        self.items.append(x)


class FakeTrainer:
    def __init__(self):
        self._metrics = collections.defaultdict(list)
        self.compute_loss = "orig_loss"
        self.log = "orig_log"
        self.trained_with = None

    def train(self):
        self.trained_with = (self.compute_loss, self.log)
        raise RuntimeError("stop")


def test_log_fn_averages_and_clears():
    tr, q = FakeTrainer(), FakeQueue()
    log = T.get_log_fn(tr, q)
    tr._metrics["policy_loss"] += [torch.tensor(1.0), torch.tensor(3.0)]   # device scalars in the real run
    tr._metrics["kl_div"] += [0.5, 1.5]
    tr._metrics["learning_rate"] += [5e-6, 5e-6]
    log({"loss": 0.25, "grad_norm": 0.1})
    assert q.items == [{"loss": 0.25, "grad_norm": 0.1, "policy_loss": 2.0, "kl_div": 1.0}]
    assert all(isinstance(v, float) for v in q.items[0].values())
    assert len(tr._metrics) == 0
    tr._metrics["policy_loss"].append(4.0)
    log({"eval_loss": 1.0})
    assert q.items[1] == {"eval_loss": 1.0, "eval_policy_loss": 4.0}


def test_train_installs_and_restores_patches():
    tr, q = FakeTrainer(), FakeQueue()
    try:
        asyncio.run(T.train(tr, q))
    except RuntimeError as e:
        assert str(e) == "stop"
    assert callable(tr.trained_with[0]) and callable(tr.trained_with[1])
    assert (tr.compute_loss, tr.log) == ("orig_loss", "orig_log")
