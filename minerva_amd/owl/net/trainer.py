"""Training and testing loops over a Net (reference owl/owl/net/trainer.py, one device):
NetTrainer (trainer.py:13-175): forward, backward, momentum-SGD update per weighted unit, the
solver's learning-rate policies, the periodic TEST-phase pass with its accuracy, periodic
snapshots.  NetTester (trainer.py:247-329): accuracy of a snapshot over `test_iter` batches,
top-1 or top-k.  Batches come from memory (`next_batch` callables); the reference's LMDB and
image-list providers, and with them the ten-crop "multiview" test, are not part of this
build."""
import time

import numpy as np

from .. import wait_for_all
from .net import Net
from .net_helper import NetBuilder, init_net_from_file, save_net_to_file


class NetTrainer(object):
    def __init__(self, solver_text, net_text=None, snapshot=0, seed=None):
        self.owl_net = Net()
        self.builder = NetBuilder(solver_text, net_text)
        self.snapshot_dir = self.builder.snapshot_dir
        self.snapshot = snapshot
        self.builder.build_net(self.owl_net)
        self.owl_net.compute_size()
        self.owl_net.init_weights(seed)
        if self.snapshot_dir:
            init_net_from_file(self.owl_net, self.snapshot_dir, self.snapshot)

    def learning_rate(self, iteridx):
        """trainer.py:96-100: "poly" and "step"; anything else keeps base_lr."""
        net, s = self.owl_net, self.owl_net.solver
        if net.lr_policy == "poly":
            return net.base_lr * pow(1 - float(iteridx) / s.max_iter, s.power)
        if net.lr_policy == "step":
            return net.base_lr * pow(s.gamma, iteridx // s.stepsize)
        return net.base_lr

    def step(self, iteridx=0):
        """One minibatch: forward, backward and the update of every weighted unit."""
        net = self.owl_net
        net.current_lr = self.learning_rate(iteridx)
        net.forward("TRAIN")
        net.backward("TRAIN")
        net.weight_update()

    def test(self, next_test_batch=None, iterations=None, log=None):
        """trainer.py:156-169: `iterations` (the solver's test_iter[0] by default) forward passes
        in the TEST phase; the accuracy is that of the LAST accuracy unit, weighted by batch
        size.  next_test_batch(i) -> (samples, labels) feeds the TEST-phase data unit."""
        net = self.owl_net
        if iterations is None:
            iterations = _first(net.solver.get("test_iter", 1))
        data = net.get_data_unit("TEST")
        acc_num, test_num = 0.0, 0
        for testiteridx in range(iterations):
            if next_test_batch is not None:
                data.set_batch(*next_test_batch(testiteridx))
            net.forward("TEST")
            accunit = net.get_accuracy_units()[-1]
            test_num += accunit.batch_size
            acc_num += accunit.batch_size * accunit.acc
            if log:
                log("Accuracy the %d mb: %f" % (testiteridx, accunit.acc))
        accuracy = float(acc_num) / max(test_num, 1)
        if log:
            log("Testing Accuracy: %f" % accuracy)
        return accuracy

    def run(self, iterations, next_batch=None, sync_freq=1, log=None, next_test_batch=None):
        """Trains for `iterations` minibatches.  next_batch(iteridx) -> (samples, labels) feeds
        the data unit (None: the batch already set is reused).  Every solver.test_interval
        minibatches (when the network has a TEST-phase data unit and next_test_batch or a batch
        set on it) the TEST-phase pass runs and its accuracy is appended to `self.accuracies`.
        Returns images per second over the whole run."""
        net = self.owl_net
        data = net.get_data_unit("TRAIN")
        every = net.solver.get("snapshot", 0)
        test_interval = net.solver.get("test_interval", 0)
        test_data = net.get_data_unit("TEST")
        has_test = test_data is not None and len(net.get_accuracy_units()) > 0 and \
            (next_test_batch is not None or test_data is not data)
        self.accuracies = []
        start = time.time()
        last = start
        for iteridx in range(iterations):
            if next_batch is not None:
                data.set_batch(*next_batch(iteridx))
            self.step(iteridx)
            if (iteridx + 1) % sync_freq == 0:
                wait_for_all()
                if log:
                    now = time.time()
                    log("finished %d minibatches (%.1f img/s, loss %.4f)" % (
                        iteridx + 1, net.batch_size * sync_freq / (now - last),
                        net.get_loss_units()[0].getloss()))
                    last = now
            if has_test and test_interval and (iteridx + 1) % test_interval == 0:
                self.accuracies.append((iteridx + 1, self.test(next_test_batch, log=log)))
            if every and self.snapshot_dir and (iteridx + 1) % every == 0:
                save_net_to_file(net, self.snapshot_dir, (iteridx + 1) // every)
        wait_for_all()
        return net.batch_size * iterations / (time.time() - start)


def _first(v):
    return v[0] if isinstance(v, (list, tuple)) else v


class NetTester(object):
    """trainer.py:247-329, single view: loads snapshot number `snapshot`, runs the solver's
    test_iter[0] TEST-phase batches and reports the mean accuracy of the named accuracy unit
    (its top_k decides top-1 or top-k), with the reference's running report per batch."""

    def __init__(self, solver_text, softmax_layer_name, accuracy_layer_name, snapshot, net_text=None):
        self.solver_text, self.net_text = solver_text, net_text
        self.softmax_layer_name = softmax_layer_name
        self.accuracy_layer_name = accuracy_layer_name
        self.snapshot = snapshot

    def build_net(self):
        self.owl_net = Net()
        self.builder = NetBuilder(self.solver_text, self.net_text)
        self.snapshot_dir = self.builder.snapshot_dir
        self.builder.build_net(self.owl_net)
        self.owl_net.compute_size("TEST")
        init_net_from_file(self.owl_net, self.snapshot_dir, self.snapshot)

    def run(self, next_test_batch=None, iterations=None, log=None):
        net = self.owl_net
        loss_unit = net.get_units_by_name(self.softmax_layer_name)[0]
        accunit = net.get_units_by_name(self.accuracy_layer_name)[0]
        data_unit = net.get_data_unit("TEST")
        assert data_unit is not None, "the network has no TEST-phase data unit"
        if iterations is None:
            iterations = _first(net.solver.get("test_iter", 1))
        acc_num, test_num = 0.0, 0
        for testiteridx in range(iterations):
            if next_test_batch is not None:
                data_unit.set_batch(*next_test_batch(testiteridx))
            net.forward("TEST")
            batch_size = accunit.batch_size
            correct = batch_size * accunit.acc
            test_num += batch_size
            acc_num += correct
            if log:
                log("Accuracy of the %d mb: %f, batch_size: %d, current mean accuracy: %f" % (
                    testiteridx, correct * 1.0 / batch_size, batch_size, float(acc_num) / test_num))
        self.predictions = np.asarray(loss_unit.ff_y.to_numpy())  # of the last batch
        accuracy = float(acc_num) / max(test_num, 1)
        if log:
            log("Testing Accuracy: %f" % accuracy)
        return accuracy
