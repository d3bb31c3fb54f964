"""Seeded host inputs of the benchmark configurations (parameters, one batch, one-hot
labels) for the three training graphs of the host layer: the MLP 784-256-10, the MNIST
CNN and the AlexNet-shaped network.  Weights ~ N(0, 0.01), biases 0, MNIST-like data
uniform[0, 1], AlexNet data ~ N(0, 1), labels uniform.  Shapes are Minerva extents
(dimension 0 fastest); the arrays are flat float32."""
import numpy as np

ALEXNET_CONVS = [  # C, K, R, S of conv1..conv5
    (3, 96, 11, 11), (96, 256, 5, 5), (256, 384, 3, 3), (384, 384, 3, 3), (384, 256, 3, 3)]


def param_shapes(kind, classes=None):
    if kind == "mlp":
        return {"w0": [256, 784], "b0": [256, 1], "w1": [10, 256], "b1": [10, 1]}
    if kind == "cnn":
        return {"w0": [5, 5, 1, 16], "b0": [16], "w1": [5, 5, 16, 32], "b1": [32],
                "w2": [10, 512], "b2": [10, 1]}
    if kind == "alexnet":
        classes = classes or 1000
        shapes = {}
        for i, (C, K, R, S) in enumerate(ALEXNET_CONVS):
            shapes["w%d" % i] = [S, R, C, K]
            shapes["b%d" % i] = [K]
        shapes.update({"w5": [4096, 9216], "w6": [4096, 4096], "w7": [classes, 4096],
                       "b5": [4096, 1], "b6": [4096, 1], "b7": [classes, 1]})
        return shapes
    raise ValueError(kind)


def make_inputs(kind, batch, seed=1000, classes=None):
    """(parameters by name, data, labels) of one configuration, from one seeded generator."""
    rng = np.random.default_rng(seed)
    if kind in ("mlp", "cnn"):
        classes = 10
        data = rng.random(784 * batch, dtype=np.float32)
    elif kind == "alexnet":
        classes = classes or 1000
        data = rng.standard_normal(227 * 227 * 3 * batch, dtype=np.float32)
    else:
        raise ValueError(kind)
    shapes = param_shapes(kind, classes)
    params = {}
    for name in sorted(shapes):
        n = int(np.prod(shapes[name]))
        params[name] = (np.zeros(n, np.float32) if name.startswith("b")
                        else (rng.standard_normal(n, dtype=np.float32) * np.float32(0.01)))
    lab = rng.integers(0, classes, size=batch)
    label = np.zeros((batch, classes), np.float32)
    label[np.arange(batch), lab] = 1.0
    return params, data, label.ravel()
