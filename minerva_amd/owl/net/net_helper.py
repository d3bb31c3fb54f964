"""Building a network from Caffe's solver / network description and saving / loading
snapshots (reference owl/owl/net/net_helper.py:11-270).

The reference parses the descriptions with Caffe's protobuf classes; here a small parser
reads the same prototxt TEXT into plain message objects, which is all the builder needs.
The snapshot layout is the reference's: a folder `<dir>/snapshot<idx>/` holding, per weighted
layer, `<layer>_weights.dat`, `<layer>_weightdelta.dat`, `<layer>_bias.dat` and
`<layer>_biasdelta.dat` as raw float32 in the arrays' element order ('/' in a layer name
becomes '_')."""
import os
import re

import numpy as np

from .. import from_numpy, zeros
from . import net as _net


class Message(object):
    """One prototxt message: fields by attribute (`msg.convolution_param.num_output`),
    `get(name, default)`, and `get_all(name)` for repeated fields.  A missing sub-message
    reads as an empty one, as protobuf does."""

    def __init__(self):
        object.__setattr__(self, "_fields", {})

    def add(self, key, value):
        self._fields.setdefault(key, []).append(value)

    def get_all(self, key):
        return list(self._fields.get(key, []))

    def get(self, key, default=None):
        vals = self._fields.get(key)
        return vals[-1] if vals else default

    def has(self, key):
        return key in self._fields

    def __getattr__(self, key):
        if key.startswith("_"):
            raise AttributeError(key)
        vals = self._fields.get(key)
        if vals:
            return vals[-1]
        if key.endswith("_param") or key.endswith("_filler"):
            return Message()
        raise AttributeError("field %r is not set" % key)

    def __repr__(self):
        return "Message(%r)" % (self._fields,)


_TOKEN = re.compile(r'"(?:[^"\\]|\\.)*"|\'(?:[^\'\\]|\\.)*\'|[{}:]|[^\s{}:]+')


def _scalar(tok):
    if tok[0] in "\"'":
        return tok[1:-1]
    if tok in ("true", "false"):
        return tok == "true"
    try:
        return int(tok)
    except ValueError:
        try:
            return float(tok)
        except ValueError:
            return tok  # an enum name: MAX, AVE, TRAIN, ...


def parse_prototxt(text):
    """Protobuf text format -> Message: `key: value` pairs and `key { ... }` blocks, repeated
    keys kept in order, '#' comments dropped."""
    text = re.sub(r"#[^\n]*", "", text)
    toks = _TOKEN.findall(text)
    pos = 0

    def block():
        nonlocal pos
        msg = Message()
        while pos < len(toks) and toks[pos] != "}":
            key = toks[pos]
            pos += 1
            if pos < len(toks) and toks[pos] == ":":
                pos += 1
                if toks[pos] == "{":
                    pos += 1
                    msg.add(key, block())
                    pos += 1
                else:
                    msg.add(key, _scalar(toks[pos]))
                    pos += 1
            elif pos < len(toks) and toks[pos] == "{":
                pos += 1
                msg.add(key, block())
                if pos >= len(toks):
                    raise ValueError("prototxt: unbalanced braces")
                pos += 1
            else:
                raise ValueError("prototxt: expected ':' or '{' after %r" % key)
        return msg

    msg = block()
    if pos != len(toks):
        raise ValueError("prototxt: unbalanced braces")
    return msg


_UNIT_TYPES = {
    "MemoryData": _net.MemoryDataUnit, "InnerProduct": _net.FullyConnection,
    "Convolution": _net.ConvConnection, "Pooling": _net.PoolingUnit, "ReLU": _net.ReluUnit,
    "Sigmoid": _net.SigmoidUnit, "SoftmaxWithLoss": _net.SoftmaxUnit, "TanH": _net.TanhUnit,
    "Dropout": _net.DropoutUnit, "LRN": _net.LRNUnit, "Concat": _net.ConcatUnit,
    "Accuracy": _net.AccuracyUnit,
}


class NetBuilder(object):
    """Builds a Net from a solver description and a network description in Caffe's text
    format (CaffeNetBuilder, net_helper.py:11-154).  In-place layers (bottom == top, e.g. a
    ReLU on a convolution's blob) are chained behind the layer that owns the blob, as the
    reference does."""

    def __init__(self, solver_text, net_text=None):
        self.solverconfig = parse_prototxt(solver_text)
        if net_text is None:
            with open(self.solverconfig.net) as f:
                net_text = f.read()
        self.netconfig = parse_prototxt(net_text)
        self.snapshot_dir = self.solverconfig.get("snapshot_prefix", "")

    def build_net(self, owl_net, num_gpu=1):
        s = self.solverconfig
        owl_net.base_lr = owl_net.current_lr = s.get("base_lr", 0.01)
        owl_net.base_weight_decay = s.get("weight_decay", 0.0)
        owl_net.momentum = s.get("momentum", 0.0)
        owl_net.solver = s
        owl_net.lr_policy = s.get("lr_policy", "fixed")
        stacked_layers, top_name_to_layer = {}, {}
        owl_net.data_layers = []
        for l in self.netconfig.get_all("layer"):
            cls = _UNIT_TYPES.get(l.type)
            if cls is None:
                raise ValueError("layer %r: type %r is not implemented" % (l.name, l.type))
            unit = cls(l)
            uid = owl_net.add_unit(unit)
            bottoms, tops = l.get_all("bottom"), l.get_all("top")
            if l.type == "MemoryData":
                owl_net.data_layers.append(l.name)
                include = l.get_all("include")
                if not include or include[0].get("phase") == "TRAIN":
                    owl_net.batch_size = unit.batch_size
            elif l.type == "SoftmaxWithLoss":
                owl_net.loss_uids.append(uid)
            elif l.type == "Accuracy":
                owl_net.accuracy_uids.append(uid)
            if len(bottoms) == 1 and len(tops) == 1 and bottoms[0] == tops[0]:
                # in place: reads the output of the last unit stacked on that blob and
                # publishes under its own name
                top_name_to_layer[l.name] = [uid]
                unit.top_names = [l.name]
                stack_to = bottoms[0]
                if stack_to not in stacked_layers:
                    stacked_layers[stack_to] = [top_name_to_layer[stack_to][0]]
                unit.btm_names = [owl_net.units[stacked_layers[stack_to][-1]].top_names[0]]
                stacked_layers[stack_to].append(uid)
            else:
                for top in tops:
                    top_name_to_layer.setdefault(top, []).append(uid)
                unit.top_names = list(tops)
                unit.btm_names = [owl_net.units[stacked_layers[b][-1]].top_names[0]
                                  if b in stacked_layers else b for b in bottoms]
        for uid, unit in enumerate(owl_net.units):
            for btm in unit.btm_names:
                for btm_uid in top_name_to_layer[btm]:
                    owl_net.connect(btm_uid, uid)


def _snapshot_dir(weightpath, snapshotidx):
    return os.path.join(weightpath, "snapshot%d" % snapshotidx)


def save_net_to_file(owl_net, weightpath, snapshotidx):
    """net_helper.py:233-270"""
    folder = _snapshot_dir(weightpath, snapshotidx)
    os.makedirs(folder, exist_ok=True)
    for uid in owl_net.get_weighted_unit_ids():
        unit = owl_net.units[uid]
        base = os.path.join(folder, unit.name.replace("/", "_"))
        for arr, ref, suffix in ((unit.weight, unit.weight, "weights"),
                                 (unit.weightdelta, unit.weight, "weightdelta"),
                                 (unit.bias, unit.bias, "bias"),
                                 (unit.biasdelta, unit.bias, "biasdelta")):
            if arr is None:  # no update yet: the momentum term is zero
                arr = zeros(ref.shape)
            arr.to_numpy().astype(np.float32).ravel().tofile("%s_%s.dat" % (base, suffix))


def init_net_from_file(owl_net, weightpath, snapshotidx):
    """net_helper.py:156-231: a layer whose file is missing or has another size keeps its
    state and is reported in the returned list ("need reinit")."""
    folder = _snapshot_dir(weightpath, snapshotidx)
    need_reinit = []
    for uid in owl_net.get_weighted_unit_ids():
        unit = owl_net.units[uid]
        base = os.path.join(folder, unit.name.replace("/", "_"))
        for attr, delta, shape, suffix in (("weight", "weightdelta", unit.wshape, "weights"),
                                           ("bias", "biasdelta", unit.bshape, "bias")):
            path = "%s_%s.dat" % (base, suffix)
            want = int(np.prod(shape))
            if not os.path.isfile(path) or os.path.getsize(path) != 4 * want:
                need_reinit.append("%s %s" % (unit.name, attr))
                continue
            setattr(unit, attr, from_numpy(np.fromfile(path, np.float32)).reshape(shape))
            dpath = "%s_%s.dat" % (base, delta)
            if os.path.isfile(dpath) and os.path.getsize(dpath) == 4 * want:
                setattr(unit, delta, from_numpy(np.fromfile(dpath, np.float32)).reshape(shape))
    return need_reinit
