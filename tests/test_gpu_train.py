"""End-to-end training loop on a small synthetic graph: every model family learns (the loss falls)
and the reference's result lines are produced.  The default mode (transposed lists in scheduling order: gradients
equal up to fp32 summation order) is what the first test pins; the second pins --deterministic 1 (bit-equal runs)."""
import importlib.util
import os

import pytest

from conftest import ROOT

pytestmark = pytest.mark.gpu


def load_train():
    spec = importlib.util.spec_from_file_location("fastgl_train", os.path.join(ROOT, "fastgl-ae_amd", "train.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("model", ["sage", "gcn", "gin", "gat"])
def test_training_reduces_the_loss(cuda, tmp_path, capsys, model):
    print("train %s" % model, flush=True)
    train = load_train()
    args = train.parse_args(["--model", model, "--nodes", "20000", "--draws", "200000", "--feat_dim", "32", "--classes", "4",
                             "--num_hidden", "32", "--batch_size", "512", "--fanout", "5", "5", "--num_epoch", "2",
                             "--train_frac", "0.4", "--dropout", "0.0", "--lr", "0.01", "--log_path", str(tmp_path)])
    result, losses = train.run(args)
    steps = len(losses) // 3
    first, last = sum(losses[:steps]) / steps, sum(losses[-steps:]) / steps
    assert last < first - 0.02, (first, last)  # mean loss of the last epoch vs the first (the linear GCN/GIN of the reference learn slowly)
    assert set(result) == {"sample_time", "copy_time", "forward_time", "backward_time", "epoch_time"}
    out = capsys.readouterr().out
    assert "test_result:epoch_time=" in out and "finish" in out
    logs = os.listdir(tmp_path)
    assert len(logs) == 1 and logs[0].startswith(model + "_rmat20000_2_32_512_1")


@pytest.mark.parametrize("model", ["sage", "gcn"])
def test_deterministic_training_is_bit_reproducible(cuda, model):
    """--deterministic 1: two runs from the same seed give the same losses bit for bit (sampling, numbering
    and the forward pass are deterministic in any mode; this mode also fixes the summation order of the
    backward gathers).  Dropout off, so that the comparison does not hinge on torch's generator state."""
    print("deterministic train %s" % model, flush=True)
    train = load_train()
    argv = ["--model", model, "--nodes", "20000", "--draws", "200000", "--feat_dim", "32", "--classes", "4",
            "--num_hidden", "32", "--batch_size", "512", "--fanout", "5", "5", "--num_epoch", "1", "--train_frac", "0.2",
            "--dropout", "0.0", "--deterministic", "1", "--prefetch", "0"]
    _, a = train.run(train.parse_args(argv))
    _, b = train.run(train.parse_args(argv))
    assert a == b and len(a) > 4
