"""Compute units and the network graph (reference owl/owl/net/net.py:24-1139).

A network is a DAG of ComputeUnits.  `forward` walks it in topological order handing every
unit the outputs of its bottom units (a dict name -> NArray), `backward` walks it in reverse
with the sensitivities, weighted units keep `weightgrad` / `biasgrad`, and `weight_update`
applies momentum SGD with weight decay.  Shapes follow Minerva: images are [W, H, C, N],
matrices [rows, N]."""
import collections

import numpy as np

from .. import conv as co
from .. import elewise as ele
from .. import from_numpy, randb, zeros, concat as _concat, slice as _slice

__all__ = ["ComputeUnit", "ComputeUnitSimple", "WeightedComputeUnit", "LinearUnit", "SigmoidUnit",
           "ReluUnit", "TanhUnit", "PoolingUnit", "DropoutUnit", "SoftmaxUnit", "AccuracyUnit",
           "LRNUnit", "ConcatUnit", "FullyConnection", "ConvConnection", "MemoryDataUnit", "Net"]


class ComputeUnit(object):
    """One node of the graph (net.py:24-103): `params` is the layer description, `btm_names` /
    `top_names` the blobs it reads and writes, `out_shape` is set by compute_size."""

    def __init__(self, params):
        self.params = params
        self.name = params.name
        self.btm_names = []
        self.top_names = []
        self.out = None
        self.out_shape = None
        # False for a unit fed by data units only: nobody uses the sensitivity of the input
        # images, so a weighted unit skips computing it (Caffe's propagate_down; the reference
        # computes it regardless, net.py:706-710)
        self.propagate_down = True

    def __str__(self):
        return "N/A unit"

    def compute_size(self, from_btm, to_top):
        pass

    def forward(self, from_btm, to_top, phase):
        pass

    def backward(self, from_top, to_btm, phase):
        pass

    def weight_update(self, base_lr, base_weight_decay, momentum, batch_size):
        pass


class ComputeUnitSimple(ComputeUnit):
    """A unit with one bottom and one top (net.py:105-152): subclasses write ff / bp."""

    def compute_size(self, from_btm, to_top):
        self.out_shape = list(from_btm[self.btm_names[0]])
        to_top[self.top_names[0]] = list(self.out_shape)

    def forward(self, from_btm, to_top, phase):
        to_top[self.top_names[0]] = self.ff(from_btm[self.btm_names[0]], phase)
        self.out = to_top[self.top_names[0]]

    def ff(self, act, phase):
        raise NotImplementedError

    def backward(self, from_top, to_btm, phase):
        to_btm[self.btm_names[0]] = self.bp(from_top[self.top_names[0]], phase)

    def bp(self, sen, phase):
        raise NotImplementedError


def _fill(filler, shape, fan_in, rng):
    """Caffe's fillers as the reference applies them (net.py:209-239)."""
    kind = filler.get("type", "constant")
    if kind == "constant":
        return np.ones(shape, np.float32) * np.float32(filler.get("value", 0.0))
    if kind == "gaussian":
        return rng.normal(filler.get("mean", 0.0), filler.get("std", 1.0), shape).astype(np.float32)
    if kind == "uniform":
        return rng.uniform(filler.get("min", 0.0), filler.get("max", 1.0), shape).astype(np.float32)
    if kind == "xavier":
        scale = np.sqrt(3.0 / fan_in)
        return rng.uniform(-scale, scale, shape).astype(np.float32)
    raise ValueError("unknown filler type %r" % kind)


class WeightedComputeUnit(ComputeUnitSimple):
    """A unit with weight and bias, their gradients and momentum terms (net.py:154-262)."""

    def __init__(self, params):
        super(WeightedComputeUnit, self).__init__(params)
        self.weight = self.weightdelta = self.weightgrad = None
        self.bias = self.biasdelta = self.biasgrad = None
        self.in_shape = self.fan_in = self.fan_out = None
        self.wshape = self.bshape = None
        mult = params.get_all("param")
        self.lr_mult_w = mult[0].get("lr_mult", 1.0) if len(mult) >= 1 else 1.0
        self.decay_mult_w = mult[0].get("decay_mult", 1.0) if len(mult) >= 1 else 1.0
        self.lr_mult_b = mult[1].get("lr_mult", 1.0) if len(mult) >= 2 else 1.0
        self.decay_mult_b = mult[1].get("decay_mult", 1.0) if len(mult) >= 2 else 0.0
        self.weight_filler = self.bias_filler = None

    def init_weights_with_filler(self, rng=None):
        rng = rng or np.random
        w = _fill(self.weight_filler, [int(np.prod(self.wshape))], self.fan_in, rng)
        b = _fill(self.bias_filler, [int(np.prod(self.bshape))], self.fan_in, rng)
        self.weight = from_numpy(w).reshape(self.wshape)
        self.bias = from_numpy(b).reshape(self.bshape)

    def weight_update(self, base_lr, base_weight_decay, momentum, batch_size):
        """delta = momentum * delta - (lr * lr_mult / batch) * grad - (lr * lr_mult * wd *
        decay_mult) * value; value += delta (net.py:241-262)."""
        if self.weightdelta is None:
            self.weightdelta = zeros(self.weightgrad.shape)
        self.weightdelta = (momentum * self.weightdelta
                            - (base_lr * self.lr_mult_w / batch_size) * self.weightgrad
                            - (base_lr * self.lr_mult_w * base_weight_decay * self.decay_mult_w) * self.weight)
        self.weight = self.weight + self.weightdelta
        self.weightgrad = None
        if self.biasdelta is None:
            self.biasdelta = zeros(self.biasgrad.shape)
        self.biasdelta = (momentum * self.biasdelta
                          - (base_lr * self.lr_mult_b / batch_size) * self.biasgrad
                          - (base_lr * self.lr_mult_b * base_weight_decay * self.decay_mult_b) * self.bias)
        self.bias = self.bias + self.biasdelta
        self.biasgrad = None


class LinearUnit(ComputeUnitSimple):
    def ff(self, x, phase):
        return x

    def bp(self, y, phase):
        return y

    def __str__(self):
        return "linear"


class SigmoidUnit(ComputeUnitSimple):
    def ff(self, x, phase):
        self.ff_y = ele.sigm(x)
        return self.ff_y

    def bp(self, y, phase):
        return ele.sigm_back(y, self.ff_y)

    def __str__(self):
        return "sigmoid"


class ReluUnit(ComputeUnitSimple):
    """net.py:289-299: the gradient is gated by the unit's input."""

    def ff(self, x, phase):
        self.ff_x = x
        return ele.relu(x)

    def bp(self, y, phase):
        return ele.relu_back(y, self.ff_x)

    def __str__(self):
        return "relu"


class TanhUnit(ComputeUnitSimple):
    def ff(self, x, phase):
        self.ff_y = ele.tanh(x)
        return self.ff_y

    def bp(self, y, phase):
        return ele.tanh_back(y, self.ff_y)

    def __str__(self):
        return "tanh"


class PoolingUnit(ComputeUnitSimple):
    """net.py:312-360; the output extent is Caffe's ceil rule, which is the library's."""

    def __init__(self, params):
        super(PoolingUnit, self).__init__(params)
        p = params.pooling_param
        self.kernel_size, self.stride, self.pad = p.get("kernel_size", 1), p.get("stride", 1), p.get("pad", 0)
        kind = co.pool_op.avg if p.get("pool", "MAX") == "AVE" else co.pool_op.max
        self.pooler = co.Pooler(self.kernel_size, self.kernel_size, self.stride, self.stride,
                                self.pad, self.pad, kind)

    def compute_size(self, from_btm, to_top):
        shp = list(from_btm[self.btm_names[0]])
        for d in (0, 1):
            ori = shp[d]
            shp[d] = int(np.ceil(float(ori + 2 * self.pad - self.kernel_size) / self.stride)) + 1
            if self.pad and (shp[d] - 1) * self.stride >= ori + self.pad:
                shp[d] -= 1
        self.out_shape = shp
        to_top[self.top_names[0]] = list(shp)

    def ff(self, x, phase):
        self.ff_x = x
        self.ff_y = self.pooler.ff(x)
        return self.ff_y

    def bp(self, y, phase):
        return self.pooler.bp(y, self.ff_y, self.ff_x)

    def __str__(self):
        return "pooling"


class DropoutUnit(ComputeUnitSimple):
    """net.py:362-391: in the TRAIN phase the activations are multiplied by a Bernoulli(keep)
    mask and by 1 / keep; other phases pass them through."""

    def __init__(self, params):
        super(DropoutUnit, self).__init__(params)
        ratio = params.dropout_param.get("dropout_ratio", 0.5)
        self.scale = 1.0 / (1.0 - ratio)
        self.keep_ratio = 1.0 - ratio
        self.dropmask = None

    def ff(self, x, phase):
        if phase == "TRAIN":
            self.dropmask = randb(x.shape, self.keep_ratio)
            return ele.mult(x, self.dropmask) * self.scale
        return x

    def bp(self, y, phase):
        if phase == "TRAIN":
            return ele.mult(y, self.dropmask) * self.scale
        return y

    def __str__(self):
        return "dropout"


class SoftmaxUnit(ComputeUnit):
    """Softmax with cross-entropy loss (net.py:393-441): bottoms are the scores and the integer
    labels; backward starts the chain with (probabilities - one-hot labels) * loss_weight."""

    def __init__(self, params):
        super(SoftmaxUnit, self).__init__(params)
        self.loss_weight = params.get_all("loss_weight")

    def compute_size(self, from_btm, to_top):
        self.out_shape = list(from_btm[self.btm_names[0]])
        to_top[self.top_names[0]] = list(self.out_shape)

    def forward(self, from_btm, to_top, phase):
        self.ff_y = co.softmax(from_btm[self.btm_names[0]], co.soft_op.instance)
        to_top[self.top_names[0]] = self.ff_y
        labels = np.asarray(from_btm[self.btm_names[1]]).astype(np.int64).ravel()
        onehot = np.zeros([self.ff_y.shape[1], self.ff_y.shape[0]], np.float32)
        onehot[np.arange(labels.size), labels] = 1
        self.y = from_numpy(onehot)
        self.out = self.ff_y

    def backward(self, from_top, to_btm, phase):
        sen = self.ff_y - self.y
        if len(self.loss_weight) == 1:
            sen = sen * float(self.loss_weight[0])
        to_btm[self.btm_names[0]] = sen

    def getloss(self):
        lossmat = ele.mult(ele.ln(self.ff_y), self.y)
        res = lossmat.sum(0).sum(1).to_numpy()
        return -float(res.ravel()[0]) / lossmat.shape[1]

    def __str__(self):
        return "softmax"


class AccuracyUnit(ComputeUnit):
    """Top-1 / top-5 accuracy (net.py:443-492); reads results back, so it is not lazy."""

    def __init__(self, params):
        super(AccuracyUnit, self).__init__(params)
        self.acc = 0
        self.batch_size = 0
        self.top_k = params.accuracy_param.get("top_k", 1)

    def compute_size(self, from_btm, to_top):
        self.out_shape = list(from_btm[self.btm_names[0]])
        to_top[self.top_names[0]] = list(self.out_shape)

    def forward(self, from_btm, to_top, phase):
        scores = from_btm[self.btm_names[0]]
        truth = np.asarray(from_btm[self.btm_names[1]]).astype(np.int64).ravel()
        self.batch_size = scores.shape[1]
        if self.top_k == 1:
            predict = scores.max_index(0)
            ground = from_numpy(truth.astype(np.float32)).reshape(predict.shape)
            self.acc = (predict - ground).count_zero() * 1.0 / self.batch_size
        else:
            top = np.argsort(scores.to_numpy(), axis=1)[:, ::-1][:, :self.top_k]
            self.acc = float(np.mean([truth[i] in top[i] for i in range(self.batch_size)]))

    def __str__(self):
        return "accuracy"


class LRNUnit(ComputeUnitSimple):
    """net.py:494-510"""

    def __init__(self, params):
        super(LRNUnit, self).__init__(params)
        p = params.lrn_param
        self.lrner = co.Lrner(p.get("local_size", 5), p.get("alpha", 1.0), p.get("beta", 0.75))
        self.scale = None

    def ff(self, x, phase):
        self.ff_x = x
        self.scale = zeros(x.shape)
        self.ff_y = self.lrner.ff(x, self.scale)
        return self.ff_y

    def bp(self, y, phase):
        return self.lrner.bp(self.ff_x, self.ff_y, self.scale, y)

    def __str__(self):
        return "lrn"


class ConcatUnit(ComputeUnit):
    """Concatenation along Caffe's concat_dim, counted from the slowest dimension
    (net.py:512-558); backward slices the sensitivity back apart."""

    def __init__(self, params):
        super(ConcatUnit, self).__init__(params)
        self.concat_dim_caffe = params.concat_param.get("concat_dim", 1)
        self.slice_count = []

    def compute_size(self, from_btm, to_top):
        shp = list(from_btm[self.btm_names[0]])
        self.concat_dim = len(shp) - 1 - self.concat_dim_caffe
        for name in self.btm_names[1:]:
            shp[self.concat_dim] += from_btm[name][self.concat_dim]
        self.out_shape = shp
        to_top[self.top_names[0]] = list(shp)

    def forward(self, from_btm, to_top, phase):
        arrays = [from_btm[n] for n in self.btm_names]
        self.concat_dim = len(arrays[0].shape) - 1 - self.concat_dim_caffe
        self.slice_count = [a.shape[self.concat_dim] for a in arrays]
        to_top[self.top_names[0]] = _concat(arrays, self.concat_dim)
        self.out = to_top[self.top_names[0]]

    def backward(self, from_top, to_btm, phase):
        st_off = 0
        for name, count in zip(self.btm_names, self.slice_count):
            to_btm[name] = _slice(from_top[self.top_names[0]], self.concat_dim, st_off, count)
            st_off += count

    def __str__(self):
        return "concat"


class FullyConnection(WeightedComputeUnit):
    """Inner product (net.py:560-637): weight [out, in], bias [out, 1]; an image batch is
    flattened to [W*H*C, N] first."""

    def __init__(self, params):
        super(FullyConnection, self).__init__(params)
        p = params.inner_product_param
        self.num_output = p.num_output
        self.weight_filler = p.get("weight_filler", {"type": "constant"})
        self.bias_filler = p.get("bias_filler", {"type": "constant"})

    def compute_size(self, from_btm, to_top):
        shp = list(from_btm[self.btm_names[0]])
        self.in_shape = [int(np.prod(shp[:-1])), shp[-1]] if len(shp) > 2 else shp
        self.out_shape = [self.num_output, 1]
        to_top[self.top_names[0]] = list(self.out_shape)
        self.wshape = [self.num_output, self.in_shape[0]]
        self.bshape = [self.num_output, 1]
        self.fan_out = self.num_output
        self.fan_in = int(np.prod(shp[:-1]))

    def _flat(self, act):
        shp = act.shape
        return act.reshape([int(np.prod(shp[:-1])), shp[-1]]) if len(shp) > 2 else act

    def ff(self, act, phase):
        self.ff_act = act
        if self.weight is None:
            self.init_weights_with_filler()
        return self.weight * self._flat(act) + self.bias

    def bp(self, sen, phase):
        a = self._flat(self.ff_act)
        self.weightgrad = sen * a.trans()
        self.biasgrad = sen.sum(1)
        if not self.propagate_down:
            return None
        s = self.weight.trans() * sen
        return s.reshape(self.ff_act.shape) if len(self.ff_act.shape) > 2 else s

    def __str__(self):
        return "fc"


class ConvConnection(WeightedComputeUnit):
    """Convolution (net.py:639-731): weight [k, k, Cin, Cout], bias [Cout]; one group only, as
    in the reference."""

    def __init__(self, params):
        super(ConvConnection, self).__init__(params)
        p = params.convolution_param
        self.conv_params = p
        self.kernel_size, self.stride, self.pad = p.kernel_size, p.get("stride", 1), p.get("pad", 0)
        self.num_output = p.num_output
        self.group = p.get("group", 1)
        if self.group != 1:
            raise ValueError("%s: multi-group convolution is not supported (use one group with "
                             "the feature maps doubled, as the reference advises)" % self.name)
        self.convolver = co.Convolver(self.pad, self.pad, self.stride, self.stride)
        self.weight_filler = p.get("weight_filler", {"type": "constant"})
        self.bias_filler = p.get("bias_filler", {"type": "constant"})

    def compute_size(self, from_btm, to_top):
        self.in_shape = list(from_btm[self.btm_names[0]])
        shp = list(self.in_shape)
        shp[0] = (shp[0] + 2 * self.pad - self.kernel_size) // self.stride + 1
        shp[1] = (shp[1] + 2 * self.pad - self.kernel_size) // self.stride + 1
        shp[2] = self.num_output
        self.out_shape = shp
        to_top[self.top_names[0]] = list(shp)
        self.wshape = [self.kernel_size, self.kernel_size, self.in_shape[2], self.num_output]
        self.bshape = [self.num_output]
        self.fan_out = self.kernel_size * self.kernel_size * self.num_output
        self.fan_in = self.kernel_size * self.kernel_size * self.in_shape[2]

    def ff(self, act, phase):
        self.ff_act = act
        if self.weight is None:
            self.init_weights_with_filler()
        return self.convolver.ff(act, self.weight, self.bias)

    def bp(self, sen, phase):
        self.weightgrad = self.convolver.weight_grad(sen, self.ff_act, self.weight)
        self.biasgrad = self.convolver.bias_grad(sen)
        if not self.propagate_down:
            return None
        return self.convolver.bp(sen, self.ff_act, self.weight)

    def __str__(self):
        return "conv"


class MemoryDataUnit(ComputeUnit):
    """The data unit of this build: batches set from memory with `set_batch` (Caffe's
    MemoryData layer) instead of the reference's LMDB / image-list providers
    (net.py:733-938).  tops: the image batch [W, H, C, N] and the integer labels."""

    def __init__(self, params):
        super(MemoryDataUnit, self).__init__(params)
        p = params.memory_data_param
        self.batch_size = p.batch_size
        self.shape = [p.width, p.height, p.channels, p.batch_size]
        self.samples = self.labels = None

    def set_batch(self, samples, labels):
        """samples: float32 of batch x channels x height x width elements (any shape);
        labels: batch integers."""
        samples = np.ascontiguousarray(samples, np.float32)
        if samples.size != int(np.prod(self.shape)):
            raise ValueError("%s: batch of %d values, expected %s" % (self.name, samples.size, self.shape))
        self.samples = from_numpy(samples.reshape(list(reversed(self.shape))))
        self.labels = np.asarray(labels).astype(np.int64).ravel()

    def compute_size(self, from_btm, to_top):
        self.out_shape = list(self.shape)
        to_top[self.top_names[0]] = list(self.shape)
        for name in self.top_names[1:]:
            to_top[name] = [1, self.batch_size]

    def forward(self, from_btm, to_top, phase):
        if self.samples is None:
            raise RuntimeError("%s: no batch set" % self.name)
        to_top[self.top_names[0]] = self.samples
        for name in self.top_names[1:]:
            to_top[name] = self.labels
        self.out = self.samples

    def __str__(self):
        return "memory_data"


class Net(object):
    """The graph (net.py:940-1139): units, adjacency lists, name -> unit ids, and the
    traversals."""

    def __init__(self):
        self.units = []
        self.adjacent = []
        self.reverse_adjacent = []
        self.base_lr = 0
        self.base_weight_decay = 0
        self.momentum = 0
        self.batch_size = 0
        self.name_to_uid = {}
        self.loss_uids = []
        self.accuracy_uids = []

    def add_unit(self, unit):
        uid = len(self.units)
        self.units.append(unit)
        self.adjacent.append([])
        self.reverse_adjacent.append([])
        self.name_to_uid.setdefault(unit.name, []).append(uid)
        return uid

    def connect(self, u1, u2):
        self.adjacent[u1].append(u2)
        self.reverse_adjacent[u2].append(u1)

    def get_units_by_name(self, name):
        return [self.units[uid] for uid in self.name_to_uid[name]]

    def get_loss_units(self):
        return [self.units[uid] for uid in self.loss_uids]

    def get_accuracy_units(self):
        return [self.units[uid] for uid in self.accuracy_uids]

    def get_data_unit(self, phase="TRAIN"):
        for uid, unit in enumerate(self.units):
            if isinstance(unit, MemoryDataUnit) and not self._is_excluded(uid, phase):
                return unit

    def get_weighted_unit_ids(self):
        return [i for i, u in enumerate(self.units) if isinstance(u, WeightedComputeUnit)]

    def _is_excluded(self, uid, phase):
        include = self.units[uid].params.get_all("include")
        return phase is not None and len(include) != 0 and include[0].get("phase") != phase

    def _order(self, phase, adjacent, reverse_adjacent):
        depcount = [len(r) for r in reverse_adjacent]
        for unit in range(len(depcount)):
            if self._is_excluded(unit, phase):
                for l in adjacent[unit]:
                    depcount[l] -= 1
        queue = collections.deque(u for u, c in enumerate(depcount) if c == 0)
        while queue:
            unit = queue.popleft()
            if self._is_excluded(unit, phase):
                continue
            yield unit
            for l in adjacent[unit]:
                depcount[l] -= 1
                if depcount[l] == 0:
                    queue.append(l)

    def _toporder(self, phase=None):
        return self._order(phase, self.adjacent, self.reverse_adjacent)

    def _reverse_toporder(self, phase=None):
        return self._order(phase, self.reverse_adjacent, self.adjacent)

    def compute_size(self, phase="TRAIN"):
        unit_to_tops = [{} for _ in self.units]
        for u in self._toporder(phase):
            from_btm = {}
            for btm in self.reverse_adjacent[u]:
                from_btm.update(unit_to_tops[btm])
            self.units[u].compute_size(from_btm, unit_to_tops[u])
            self.units[u].propagate_down = any(not isinstance(self.units[b], MemoryDataUnit)
                                               for b in self.reverse_adjacent[u])

    def forward(self, phase="TRAIN"):
        unit_to_tops = [{} for _ in self.units]
        for u in self._toporder(phase):
            from_btm = {}
            for btm in self.reverse_adjacent[u]:
                from_btm.update(unit_to_tops[btm])
            self.units[u].forward(from_btm, unit_to_tops[u], phase)

    def backward(self, phase="TRAIN"):
        """Sensitivities that reach a blob from several tops are added (net.py:1101-1116)."""
        unit_to_btms = [{} for _ in self.units]
        for u in self._reverse_toporder(phase):
            from_top = {}
            for top in self.adjacent[u]:
                for key, val in unit_to_btms[top].items():
                    if val is not None:
                        from_top[key] = from_top[key] + val if key in from_top else val
            self.units[u].backward(from_top, unit_to_btms[u], phase)

    def update(self, uid):
        self.units[uid].weight_update(self.current_lr, self.base_weight_decay, self.momentum,
                                      self.batch_size)

    def weight_update(self):
        for uid in self.get_weighted_unit_ids():
            self.update(uid)

    def init_weights(self, seed=None):
        """Applies every weighted unit's fillers (the reference does it lazily in the first
        forward pass, from numpy's global generator; a seed makes it repeatable)."""
        rng = np.random.RandomState(seed) if seed is not None else None
        for uid in self.get_weighted_unit_ids():
            self.units[uid].init_weights_with_filler(rng)

    def __str__(self):
        return "\n".join("%s (%s) <- %s" % (u.name, u, ",".join(u.btm_names)) for u in self.units)
