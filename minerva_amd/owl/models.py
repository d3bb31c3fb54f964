"""The AlexNet-shaped single-group network of the reference's Python application
(owl/apps/imagenet_alexnet/alexnet.py:6-133) on the NArray front end: the same operator
sequence -- five convolutions with ReLU, three max-poolings, three fully connected layers
with drop6 / drop7, soft-max -- and the same momentum / weight-decay update."""
import numpy as np

from . import NArray, from_numpy, randb, randn, zeros
from . import conv as co
from . import elewise as ele


class AlexNet(object):
    CONVS = [(0, 0, 4, 4), (2, 2, 1, 1), (1, 1, 1, 1), (1, 1, 1, 1), (1, 1, 1, 1)]

    def __init__(self, classes=1000):
        self.classes = int(classes)
        self.convs = [co.Convolver(*c) for c in self.CONVS]
        self.poolings = [co.Pooler(3, 3, 2, 2, op=co.pool_op.max) for _ in range(3)]
        self.weight_shapes = [[11, 11, 3, 96], [5, 5, 96, 256], [3, 3, 256, 384], [3, 3, 384, 384],
                              [3, 3, 384, 256], [4096, 9216], [4096, 4096], [self.classes, 4096]]
        self.bias_shapes = [[96], [256], [384], [384], [256], [4096, 1], [4096, 1], [self.classes, 1]]
        self.num_weights = len(self.weight_shapes)
        self.weights = self.bias = self.weightsdelta = self.biasdelta = None
        self.keep_activations = False  # tests: train_one_mb leaves its activations in last_acts
        self.last_acts = None

    def _zero_deltas(self):
        self.weightsdelta = [zeros(s) for s in self.weight_shapes]
        self.biasdelta = [zeros(s) for s in self.bias_shapes]

    def init_random(self, std=0.01):
        self.weights = [randn(s, 0.0, std) for s in self.weight_shapes]
        self.bias = [zeros(s) for s in self.bias_shapes]
        self._zero_deltas()

    def load(self, weights, biases):
        """weights / biases: flat arrays in Minerva's element order, one per layer."""
        put = lambda a, s: from_numpy(np.asarray(a, np.float32).reshape(list(reversed(s))))
        self.weights = [put(a, s) for a, s in zip(weights, self.weight_shapes)]
        self.bias = [put(a, s) for a, s in zip(biases, self.bias_shapes)]
        self._zero_deltas()

    def train_one_mb(self, data, label, dropout_rate=None):
        """data {227,227,3,N}, label {classes,N} one-hot.  dropout_rate: probability with
        which an activation of fc6 / fc7 is KEPT (the application's convention: it is the
        parameter of the Bernoulli mask), or None for no dropout.  Returns (output
        probabilities, weight gradients, bias gradients)."""
        n = data.shape[-1]
        w, b, cv, pl = self.weights, self.bias, self.convs, self.poolings
        acts = [None] * 12
        acts[0] = data
        acts[1] = ele.relu(cv[0].ff(acts[0], w[0], b[0]))
        acts[2] = pl[0].ff(acts[1])
        acts[3] = ele.relu(cv[1].ff(acts[2], w[1], b[1]))
        acts[4] = pl[1].ff(acts[3])
        acts[5] = ele.relu(cv[2].ff(acts[4], w[2], b[2]))
        acts[6] = ele.relu(cv[3].ff(acts[5], w[3], b[3]))
        acts[7] = ele.relu(cv[4].ff(acts[6], w[4], b[4]))
        acts[8] = pl[2].ff(acts[7])
        flat8 = acts[8].reshape([int(np.prod(acts[8].shape[0:3])), n])
        acts[9] = ele.relu(w[5] * flat8 + b[5])
        mask6 = mask7 = None
        if dropout_rate is not None:
            mask6 = randb(acts[9].shape, dropout_rate)
            acts[9] = ele.mult(acts[9], mask6)
        acts[10] = ele.relu(w[6] * acts[9] + b[6])
        if dropout_rate is not None:
            mask7 = randb(acts[10].shape, dropout_rate)
            acts[10] = ele.mult(acts[10], mask7)
        acts[11] = w[7] * acts[10] + b[7]
        out = co.softmax(acts[11], co.soft_op.instance)
        if self.keep_activations:
            self.last_acts = list(acts)

        sens = [None] * 12
        sens[11] = out - label
        sens[10] = w[7].trans() * sens[11]
        if mask7 is not None:
            sens[10] = ele.mult(sens[10], mask7)
        sens[10] = ele.relu_back(sens[10], acts[10])
        sens[9] = w[6].trans() * sens[10]
        if mask6 is not None:
            sens[9] = ele.mult(sens[9], mask6)
        sens[9] = ele.relu_back(sens[9], acts[9])
        sens[8] = (w[5].trans() * sens[9]).reshape(acts[8].shape)
        sens[7] = ele.relu_back(pl[2].bp(sens[8], acts[8], acts[7]), acts[7])
        sens[6] = ele.relu_back(cv[4].bp(sens[7], acts[6], w[4]), acts[6])
        sens[5] = ele.relu_back(cv[3].bp(sens[6], acts[5], w[3]), acts[5])
        sens[4] = cv[2].bp(sens[5], acts[4], w[2])
        sens[3] = ele.relu_back(pl[1].bp(sens[4], acts[4], acts[3]), acts[3])
        sens[2] = cv[1].bp(sens[3], acts[2], w[1])
        sens[1] = ele.relu_back(pl[0].bp(sens[2], acts[2], acts[1]), acts[1])

        wgrad, bgrad = [None] * 8, [None] * 8
        wgrad[7] = sens[11] * acts[10].trans()
        wgrad[6] = sens[10] * acts[9].trans()
        wgrad[5] = sens[9] * flat8.trans()
        for k, (s, a) in zip((4, 3, 2, 1, 0), ((7, 6), (6, 5), (5, 4), (3, 2), (1, 0))):
            wgrad[k] = cv[k].weight_grad(sens[s], acts[a], w[k])
            bgrad[k] = cv[k].bias_grad(sens[s])
        for k, s in ((7, 11), (6, 10), (5, 9)):
            bgrad[k] = sens[s].sum(1)
        return out, wgrad, bgrad

    def update(self, weightsgrad, biasgrad, num_samples, mom, lr, wd):
        """Momentum SGD with weight decay, as the application applies it."""
        for k in range(self.num_weights):
            self.weightsdelta[k] = (mom * self.weightsdelta[k] - lr / num_samples * weightsgrad[k]
                                    - lr * wd * self.weights[k])
            self.biasdelta[k] = mom * self.biasdelta[k] - lr / num_samples * biasgrad[k]
            self.weights[k] += self.weightsdelta[k]
            self.bias[k] += self.biasdelta[k]

    def sgd(self, weightsgrad, biasgrad, num_samples, lr):
        """Plain SGD, w -= lr / num_samples * g (the step of the benchmark configuration)."""
        eps = float(np.float32(lr) / np.float32(num_samples))
        for k in range(self.num_weights):
            self.weights[k] -= eps * weightsgrad[k]
            self.bias[k] -= eps * biasgrad[k]
