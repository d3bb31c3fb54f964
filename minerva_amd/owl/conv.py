"""Convolution, pooling, softmax and LRN wrappers with the interface of the reference's
owl/owl/conv.py:13-182 (`Convolver`, `Pooler`, `Lrner`, `softmax`, `soft_op`, `pool_op`)."""
from . import NArray


class _SoftmaxAlgo(object):
    """SoftmaxAlgorithm (reference narray/convolution_info.h:43-47)."""
    instance, channel = 0, 1


class _PoolingAlgo(object):
    """PoolingInfo::Algorithm (reference narray/convolution_info.h:19-23)."""
    max, avg = 0, 1


class _ActivationAlgo(object):
    """ActivationAlgorithm (reference narray/convolution_info.h:49-54)."""
    sigmoid, relu, tanh = 0, 1, 2


soft_op = _SoftmaxAlgo
pool_op = _PoolingAlgo
act_op = _ActivationAlgo


class ConvInfo(object):
    def __init__(self, pad_height=0, pad_width=0, stride_vertical=1, stride_horizontal=1):
        self.pad_height, self.pad_width = int(pad_height), int(pad_width)
        self.stride_vertical, self.stride_horizontal = int(stride_vertical), int(stride_horizontal)

    def params(self):
        return [self.pad_height, self.pad_width, self.stride_vertical, self.stride_horizontal]


class PoolingInfo(object):
    def __init__(self, height, width, stride_vertical, stride_horizontal, pad_height=0,
                 pad_width=0, algorithm=pool_op.max):
        self.algorithm = int(algorithm)
        self.height, self.width = int(height), int(width)
        self.stride_vertical, self.stride_horizontal = int(stride_vertical), int(stride_horizontal)
        self.pad_height, self.pad_width = int(pad_height), int(pad_width)

    def params(self):
        return [self.algorithm, self.height, self.width, self.stride_vertical,
                self.stride_horizontal, self.pad_height, self.pad_width]


def softmax(x, op=soft_op.instance):
    """Softmax over the instances of x, whose last dimension counts them; arrays of fewer
    than four dimensions are viewed as {d0, .., 1, 1, instances} (conv.py:13-30)."""
    if len(x.shape) == 4:
        return NArray.softmax_forward(x, op)
    ori = list(x.shape)
    four = ori[:-1] + [1] * (4 - len(ori)) + [ori[-1]]
    return NArray.softmax_forward(x.reshape(four), op).reshape(ori)


class Lrner(object):
    """Local response normalisation across channels (conv.py:32-71)."""

    def __init__(self, local_size, alpha, beta):
        self.local_size, self.alpha, self.beta = int(local_size), float(alpha), float(beta)

    def ff(self, x, scale):
        """x: {W,H,C,N}; scale: an array of the same shape that receives the window sums."""
        return NArray.lrn_forward(x, scale, self.local_size, self.alpha, self.beta)

    def bp(self, bottom_data, top_data, scale, top_diff):
        return NArray.lrn_backward(bottom_data, top_data, scale, top_diff, self.local_size,
                                   self.alpha, self.beta)


class Convolver(object):
    """Convolution with fixed padding and strides (conv.py:74-134)."""

    def __init__(self, pad_h, pad_w, stride_v, stride_h):
        self.param = ConvInfo(pad_h, pad_w, stride_v, stride_h)

    def ff(self, x, w, b):
        """x {W,H,C,N}, w {S,R,C,K}, b {K} -> {Wo,Ho,K,N}"""
        return NArray.conv_forward(x, w, b, self.param)

    def bp(self, y, x, w):
        """Gradient with respect to the input: y is the output's gradient, x the input."""
        return NArray.conv_backward_data(y, x, w, self.param)

    def weight_grad(self, y, x, w):
        return NArray.conv_backward_filter(y, x, w, self.param)

    def bias_grad(self, y):
        return NArray.conv_backward_bias(y)


class Pooler(object):
    """Pooling (conv.py:136-182)."""

    def __init__(self, h, w, stride_v, stride_h, pad_h=0, pad_w=0, op=pool_op.max):
        self.param = PoolingInfo(h, w, stride_v, stride_h, pad_h, pad_w, op)

    def ff(self, x):
        return NArray.pooling_forward(x, self.param)

    def bp(self, y, ff_y, ff_x):
        """y: gradient of the pooled output, ff_y: the pooled output, ff_x: the input."""
        return NArray.pooling_backward(y, ff_y, ff_x, self.param)
