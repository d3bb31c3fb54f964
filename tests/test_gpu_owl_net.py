"""owl.net on the GPU: the Caffe-like unit graph of the reference (owl/owl/net/net.py), its
builder from prototxt text, the momentum-SGD update, the snapshot layout of
owl/owl/net/net_helper.py:156-270, and one training step of the full Caffe-style AlexNet
(norm1 / norm2 LRN, drop6 / drop7) at batch 2 against the CPU oracle's graph of the same units."""
import os

import numpy as np
import pytest

from gpu_util import TOL, assert_bits_equal, normwise, say

pytestmark = pytest.mark.gpu

SMALL_NET = '''
name: "small"
layer { name: "data" type: "MemoryData" top: "data" top: "label"
  memory_data_param { batch_size: 6 channels: 2 height: 10 width: 10 } }
layer { name: "conv1" type: "Convolution" bottom: "data" top: "conv1"
  param { lr_mult: 1 decay_mult: 1 } param { lr_mult: 2 decay_mult: 0 }
  convolution_param { num_output: 8 kernel_size: 3 pad: 1
    weight_filler { type: "gaussian" std: 0.2 } bias_filler { type: "constant" value: 0.1 } } }
layer { name: "relu1" type: "ReLU" bottom: "conv1" top: "conv1" }
layer { name: "norm1" type: "LRN" bottom: "conv1" top: "norm1" lrn_param { local_size: 3 alpha: 0.01 beta: 0.75 } }
layer { name: "pool1" type: "Pooling" bottom: "norm1" top: "pool1" pooling_param { pool: MAX kernel_size: 3 stride: 2 } }
layer { name: "a/fc" type: "InnerProduct" bottom: "pool1" top: "fc1"
  inner_product_param { num_output: 16 weight_filler { type: "xavier" } } }
layer { name: "tanh1" type: "TanH" bottom: "fc1" top: "fc1" }
layer { name: "fc2" type: "InnerProduct" bottom: "fc1" top: "fc2"
  inner_product_param { num_output: 5 weight_filler { type: "uniform" min: -0.3 max: 0.3 } } }
layer { name: "loss" type: "SoftmaxWithLoss" bottom: "fc2" bottom: "label" top: "loss" }
layer { name: "accuracy" type: "Accuracy" bottom: "fc2" bottom: "label" top: "accuracy" include { phase: TEST } }
'''
SMALL_SOLVER = 'base_lr: 0.05 momentum: 0.9 weight_decay: 0.001 lr_policy: "step" gamma: 0.5 stepsize: 2 max_iter: 10'


@pytest.fixture(scope="module")
def owl():
    from minerva_amd import owl as front
    dev = front.create_gpu_device(0)
    front.set_device(dev)
    yield front
    front.close_devices()


def test_builder_graph_and_sizes(owl):
    from minerva_amd.owl import net as onet
    n = onet.Net()
    onet.NetBuilder(SMALL_SOLVER, SMALL_NET).build_net(n)
    n.compute_size("TRAIN")
    by = {u.name: u for u in n.units}
    assert n.batch_size == 6 and abs(n.base_lr - 0.05) < 1e-12 and n.momentum == 0.9
    # in-place ReLU / TanH are chained behind the unit that owns the blob
    assert by["relu1"].btm_names == ["conv1"] and by["norm1"].btm_names == ["relu1"]
    assert by["fc2"].btm_names == ["tanh1"]
    assert by["conv1"].out_shape == [10, 10, 8, 6] and by["conv1"].wshape == [3, 3, 2, 8]
    assert by["pool1"].out_shape == [5, 5, 8, 6]        # ceil((10 - 3) / 2) + 1
    assert by["a/fc"].wshape == [16, 200] and by["fc2"].bshape == [5, 1]
    assert by["conv1"].lr_mult_b == 2 and by["conv1"].decay_mult_b == 0 and by["fc2"].lr_mult_b == 1
    train = [n.units[u].name for u in n._toporder("TRAIN")]
    assert "accuracy" not in train and train.index("pool1") < train.index("a/fc")
    assert "accuracy" in [n.units[u].name for u in n._toporder("TEST")]
    with pytest.raises(ValueError):
        bad = SMALL_NET.replace('pad: 1', 'pad: 1 group: 2')
        onet.NetBuilder(SMALL_SOLVER, bad).build_net(onet.Net())


def test_training_reduces_the_loss_and_snapshots_round_trip(owl, tmp_path):
    from minerva_amd.owl import net as onet
    rng = np.random.default_rng(3)
    x = rng.standard_normal((6, 2, 10, 10)).astype(np.float32)
    y = rng.integers(0, 5, 6)
    solver = SMALL_SOLVER + ' snapshot_prefix: "%s" snapshot: 3' % tmp_path
    tr = onet.NetTrainer(solver, SMALL_NET, seed=5)
    net = tr.owl_net
    net.get_data_unit().set_batch(x, y)
    say("owl.net: 6 training iterations")
    net.forward("TRAIN")
    first = net.get_loss_units()[0].getloss()
    rate = tr.run(6)
    net.forward("TEST")
    last = net.get_loss_units()[0].getloss()
    assert last < 0.7 * first and rate > 0, (first, last)
    assert 0.0 <= net.get_accuracy_units()[0].acc <= 1.0
    assert abs(tr.learning_rate(0) - 0.05) < 1e-12 and abs(tr.learning_rate(5) - 0.0125) < 1e-12
    # the layout of the reference's snapshots
    folder = os.path.join(str(tmp_path), "snapshot2")
    names = sorted(os.listdir(folder))
    assert names == sorted("%s_%s.dat" % (l, s) for l in ("conv1", "a_fc", "fc2")
                           for s in ("weights", "weightdelta", "bias", "biasdelta"))
    assert os.path.getsize(os.path.join(folder, "conv1_weights.dat")) == 4 * 3 * 3 * 2 * 8
    # a second network initialised from the snapshot has the same bits and trains on alike
    state = {u.name: (u.weight.to_numpy(), u.weightdelta.to_numpy(), u.bias.to_numpy(), u.biasdelta.to_numpy())
             for u in (net.units[i] for i in net.get_weighted_unit_ids())}
    raw = np.fromfile(os.path.join(folder, "fc2_weights.dat"), np.float32)
    assert_bits_equal(raw, state["fc2"][0].ravel(), "raw float32 in the array's element order")
    tr2 = onet.NetTrainer(solver, SMALL_NET, snapshot=2, seed=99)
    for u in (tr2.owl_net.units[i] for i in tr2.owl_net.get_weighted_unit_ids()):
        for got, want, what in zip((u.weight, u.weightdelta, u.bias, u.biasdelta), state[u.name],
                                   ("weight", "weightdelta", "bias", "biasdelta")):
            assert_bits_equal(got.to_numpy(), want, "%s %s after loading the snapshot" % (u.name, what))
    for t in (tr, tr2):
        t.owl_net.get_data_unit().set_batch(x, y)
        t.step(6)
    for a, b in zip(net.get_weighted_unit_ids(), tr2.owl_net.get_weighted_unit_ids()):
        assert_bits_equal(tr2.owl_net.units[b].weight.to_numpy(), net.units[a].weight.to_numpy(),
                          "step after reload")
    # a snapshot of another network shape is reported, not loaded
    other = onet.NetTrainer(SMALL_SOLVER, SMALL_NET.replace("num_output: 16", "num_output: 12"), seed=1)
    missing = onet.init_net_from_file(other.owl_net, str(tmp_path), 2)
    assert "a/fc weight" in missing and "fc2 weight" in missing and "conv1 weight" not in missing


def test_caffe_alexnet_step_matches_oracle(owl):
    """Forward: every unit's output against the oracle's.  Backward: every gradient against the
    oracle's backward pass evaluated at the GPU's activations (same ReLU gates and pooling
    routes on both sides).  Update: the momentum / weight-decay rule on the GPU's gradients,
    bit for bit."""
    from minerva_amd.owl import net as onet
    from minerva_amd.owl.net import models
    from oracle import nets
    batch, classes, seed = 2, 1000, 777
    units = nets.caffe_alexnet_units(classes)
    tr = onet.NetTrainer(models.ALEXNET_SOLVER, models.alexnet_prototxt(batch, classes), seed=21)
    net = tr.owl_net
    rng = np.random.default_rng(22)
    data = rng.standard_normal(batch * 3 * 227 * 227).astype(np.float32)
    labels = rng.integers(0, classes, batch)
    net.get_data_unit().set_batch(data, labels)
    weighted = [net.units[i] for i in net.get_weighted_unit_ids()]
    before = {u.name: (u.weight.to_numpy().ravel().copy(), u.bias.to_numpy().ravel().copy()) for u in weighted}
    owl.set_random_seed(seed)
    say("owl.net Caffe AlexNet forward + backward b=2 (GPU)")
    net.current_lr = tr.learning_rate(0)
    net.forward("TRAIN")
    net.backward("TRAIN")
    owl.wait_for_all()
    order = [net.units[u] for u in net._toporder("TRAIN")]
    chain = [u for u in order if not isinstance(u, (onet.MemoryDataUnit, onet.SoftmaxUnit))]
    assert len(chain) == len(units)
    gpu_acts = [u.out.to_numpy().ravel() for u in chain]
    prob = net.get_loss_units()[0].ff_y.to_numpy().ravel()
    grads = {u.name: (u.weightgrad.to_numpy().ravel(), u.biasgrad.to_numpy().ravel()) for u in weighted}
    masks = nets.dropout_masks(batch, 0.5, seed)
    say("oracle forward (CPU)")
    ora_acts, ora_prob = nets.caffe_forward(units, before, data, batch, masks)
    worst = {"prob": normwise(prob, ora_prob)}
    for u, got, want in zip(chain, gpu_acts, ora_acts):
        worst["out " + u.name] = normwise(got, want)
    say("oracle backward at the GPU's activations (CPU)")
    ref = nets.caffe_backward(units, before, data, gpu_acts, prob, labels, batch, masks)
    for name, (gw, gb) in grads.items():
        worst["weightgrad " + name] = normwise(gw, ref[name][0])
        worst["biasgrad " + name] = normwise(gb, ref[name][1])
    say("  worst normwise error %.2e (%s)" % (max(worst.values()), max(worst, key=worst.get)))
    bad = {k: v for k, v in worst.items() if not v <= TOL}
    assert not bad, bad
    net.weight_update()
    owl.wait_for_all()
    for u in weighted:
        zero_w, zero_b = np.zeros_like(before[u.name][0]), np.zeros_like(before[u.name][1])
        w, dw = nets.caffe_update(before[u.name][0], zero_w, grads[u.name][0], 0.01, u.lr_mult_w,
                                  0.0005, u.decay_mult_w, 0.9, batch)
        b, db = nets.caffe_update(before[u.name][1], zero_b, grads[u.name][1], 0.01, u.lr_mult_b,
                                  0.0005, u.decay_mult_b, 0.9, batch)
        assert_bits_equal(u.weight.to_numpy().ravel(), w, "updated weight of " + u.name)
        assert_bits_equal(u.weightdelta.to_numpy().ravel(), dw, "momentum of " + u.name)
        assert_bits_equal(u.bias.to_numpy().ravel(), b, "updated bias of " + u.name)
        assert_bits_equal(u.biasdelta.to_numpy().ravel(), db, "bias momentum of " + u.name)


def _pattern_batches(count, batch, seed):
    """Synthetic digits a small CNN can learn in a few steps: class k lights a 6x6 patch whose
    position depends on k, on a noisy background."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        y = rng.integers(0, 10, batch)
        x = (rng.standard_normal((batch, 1, 28, 28)) * 0.3).astype(np.float32)
        for i, k in enumerate(y):
            r, c = 2 + 5 * (k // 5) * 2, 1 + 5 * (k % 5)
            x[i, 0, r:r + 6, c:c + 6] += 2.0
        out.append((x, y))
    return out


def test_mnist_cnn_test_phase_and_tester(owl, tmp_path):
    """trainer.py:156-169 (the TEST-phase pass every test_interval minibatches) and NetTester
    (trainer.py:247-329) on the MNIST CNN description: the accuracies they report are the
    share of arg-max predictions that hit the label, recomputed here from the probabilities."""
    from minerva_amd.owl import net as onet
    from minerva_amd.owl.net import models
    batch, test_batch = 32, 16
    solver = models.MNIST_CNN_SOLVER + 'snapshot_prefix: "%s" snapshot: 20\n' % tmp_path
    text = models.mnist_cnn_prototxt(batch, test_batch)
    train = _pattern_batches(20, batch, 1)
    test = _pattern_batches(3, test_batch, 2)
    tr = onet.NetTrainer(solver, text, seed=7)
    net = tr.owl_net
    assert net.get_data_unit("TRAIN") is not net.get_data_unit("TEST")
    assert net.get_data_unit("TEST").batch_size == test_batch
    say("owl.net: MNIST CNN, accuracy before training")
    before = tr.test(lambda i: test[i])
    logged = []
    say("owl.net: MNIST CNN, 20 minibatches with a TEST pass every 10")
    tr.run(20, lambda i: train[i], sync_freq=5, log=logged.append, next_test_batch=lambda i: test[i])
    assert [it for it, _ in tr.accuracies] == [10, 20]
    after = tr.accuracies[-1][1]
    assert after >= 0.9 and after > before + 0.3, (before, tr.accuracies)
    assert any(l.startswith("Testing Accuracy") for l in logged)
    # the reported accuracy is what the probabilities say, batch by batch
    hits = total = 0
    loss = net.get_units_by_name("loss")[0]
    for x, y in test:
        net.get_data_unit("TEST").set_batch(x, y)
        net.forward("TEST")
        prob = loss.ff_y.to_numpy().reshape(test_batch, 10)
        hits += int(np.sum(np.argmax(prob, axis=1) == y))
        total += test_batch
        assert abs(net.get_accuracy_units()[-1].acc - np.mean(np.argmax(prob, axis=1) == y)) < 1e-12
    assert abs(after - hits / total) < 1e-12
    # the tester on the snapshot written after 20 minibatches reports the same number
    tester = onet.NetTester(solver, "loss", "accuracy", 1, net_text=text)
    tester.build_net()
    lines = []
    assert abs(tester.run(lambda i: test[i], log=lines.append) - after) < 1e-12
    assert len(lines) == 4 and lines[-1].startswith("Testing Accuracy")
    # top-5 through the accuracy unit's top_k against a numpy ranking
    top5 = onet.NetTester(solver, "loss", "accuracy", 1,
                          net_text=models.mnist_cnn_prototxt(batch, test_batch, top_k=5))
    top5.build_net()
    got = top5.run(lambda i: test[i])
    want = 0
    for x, y in test:
        top5.owl_net.get_data_unit("TEST").set_batch(x, y)
        top5.owl_net.forward("TEST")
        prob = top5.owl_net.get_units_by_name("loss")[0].ff_y.to_numpy().reshape(test_batch, 10)
        want += sum(int(y[i] in np.argsort(prob[i])[::-1][:5]) for i in range(test_batch))
    assert abs(got - want / (3.0 * test_batch)) < 1e-12 and got >= after
