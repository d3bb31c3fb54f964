"""Training loop over a Net (reference owl/owl/net/trainer.py:13-145, one device):
forward, backward, momentum-SGD update per weighted unit, the solver's learning-rate
policies, periodic snapshots."""
import time

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

    def run(self, iterations, next_batch=None, sync_freq=1, log=None):
        """Trains for `iterations` minibatches.  next_batch(iteridx) -> (samples, labels) feeds
        the data unit (None: the batch already set is reused).  Returns images per second over
        the whole run."""
        net = self.owl_net
        data = net.get_data_unit("TRAIN")
        every = net.solver.get("snapshot", 0)
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
            if every and self.snapshot_dir and (iteridx + 1) % every == 0:
                save_net_to_file(net, self.snapshot_dir, (iteridx + 1) // every)
        wait_for_all()
        return net.batch_size * iterations / (time.time() - start)
