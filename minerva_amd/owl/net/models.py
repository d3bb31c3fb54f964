"""Network descriptions in Caffe's text format for the benchmark and the tests."""


def _conv(name, bottom, num_output, kernel, stride=1, pad=0, std=0.01, bias=0.0):
    return '''
layer { name: "%s" type: "Convolution" bottom: "%s" top: "%s"
  param { lr_mult: 1 decay_mult: 1 } param { lr_mult: 2 decay_mult: 0 }
  convolution_param { num_output: %d kernel_size: %d stride: %d pad: %d
    weight_filler { type: "gaussian" std: %g } bias_filler { type: "constant" value: %g } } }
layer { name: "relu_%s" type: "ReLU" bottom: "%s" top: "%s" }''' % (
        name, bottom, name, num_output, kernel, stride, pad, std, bias, name, name, name)


def _fc(name, bottom, num_output, relu_dropout, std=0.005, bias=0.1):
    text = '''
layer { name: "%s" type: "InnerProduct" bottom: "%s" top: "%s"
  param { lr_mult: 1 decay_mult: 1 } param { lr_mult: 2 decay_mult: 0 }
  inner_product_param { num_output: %d
    weight_filler { type: "gaussian" std: %g } bias_filler { type: "constant" value: %g } } }''' % (
        name, bottom, name, num_output, std, bias)
    if relu_dropout:
        text += '''
layer { name: "relu_%s" type: "ReLU" bottom: "%s" top: "%s" }
layer { name: "drop_%s" type: "Dropout" bottom: "%s" top: "%s" dropout_param { dropout_ratio: 0.5 } }''' % (
            name, name, name, name, name, name)
    return text


def _pool(name, bottom):
    return '''
layer { name: "%s" type: "Pooling" bottom: "%s" top: "%s"
  pooling_param { pool: MAX kernel_size: 3 stride: 2 } }''' % (name, bottom, name)


def _lrn(name, bottom):
    return '''
layer { name: "%s" type: "LRN" bottom: "%s" top: "%s"
  lrn_param { local_size: 5 alpha: 0.0001 beta: 0.75 } }''' % (name, bottom, name)


def alexnet_prototxt(batch_size, classes=1000):
    """Caffe's reference AlexNet (conv1-relu-norm1-pool1, conv2-relu-norm2-pool2, conv3..5,
    pool5, fc6/fc7 with ReLU and dropout, fc8, softmax loss) with every convolution in ONE
    group (the reference's units do not support groups), fed from memory."""
    return ('name: "AlexNet"\n'
            'layer { name: "data" type: "MemoryData" top: "data" top: "label"\n'
            '  memory_data_param { batch_size: %d channels: 3 height: 227 width: 227 } }' % batch_size
            + _conv("conv1", "data", 96, 11, stride=4)
            + _lrn("norm1", "conv1") + _pool("pool1", "norm1")
            + _conv("conv2", "pool1", 256, 5, pad=2, bias=0.1)
            + _lrn("norm2", "conv2") + _pool("pool2", "norm2")
            + _conv("conv3", "pool2", 384, 3, pad=1)
            + _conv("conv4", "conv3", 384, 3, pad=1, bias=0.1)
            + _conv("conv5", "conv4", 256, 3, pad=1, bias=0.1)
            + _pool("pool5", "conv5")
            + _fc("fc6", "pool5", 4096, True) + _fc("fc7", "fc6", 4096, True)
            + _fc("fc8", "fc7", classes, False, std=0.01, bias=0.0)
            + '\nlayer { name: "loss" type: "SoftmaxWithLoss" bottom: "fc8" bottom: "label" top: "loss" }\n')


ALEXNET_SOLVER = '''
base_lr: 0.01 lr_policy: "step" gamma: 0.1 stepsize: 100000
momentum: 0.9 weight_decay: 0.0005 max_iter: 450000
'''


def mnist_cnn_prototxt(batch_size, test_batch_size=None, top_k=1):
    """The MNIST CNN of the reference's applications (owl/apps/mnist/mnist_cnn.py:17-47: conv 5x5
    16 - ReLU - max-pool 2x2/2 - conv 5x5 32 - ReLU - max-pool 2x2/2 - fully connected 10 -
    softmax, weights N(0, 0.1)) as a network description with a TRAIN-phase and a TEST-phase data
    unit and an accuracy unit in the TEST phase, the shape of the reference's prototxt networks."""
    test_batch_size = test_batch_size or batch_size
    data = ('layer { name: "mnist" type: "MemoryData" top: "data" top: "label" include { phase: %s }\n'
            '  memory_data_param { batch_size: %d channels: 1 height: 28 width: 28 } }\n')
    conv = ('layer { name: "%s" type: "Convolution" bottom: "%s" top: "%s"\n'
            '  convolution_param { num_output: %d kernel_size: 5 weight_filler { type: "gaussian" std: 0.1 } } }\n'
            'layer { name: "relu_%s" type: "ReLU" bottom: "%s" top: "%s" }\n')
    pool = ('layer { name: "%s" type: "Pooling" bottom: "%s" top: "%s"'
            ' pooling_param { pool: MAX kernel_size: 2 stride: 2 } }\n')
    return ('name: "MnistCnn"\n' + data % ("TRAIN", batch_size) + data % ("TEST", test_batch_size)
            + conv % ("conv1", "data", "conv1", 16, "conv1", "conv1", "conv1")
            + pool % ("pool1", "conv1", "pool1")
            + conv % ("conv2", "pool1", "conv2", 32, "conv2", "conv2", "conv2")
            + pool % ("pool2", "conv2", "pool2")
            + 'layer { name: "ip" type: "InnerProduct" bottom: "pool2" top: "ip"\n'
              '  inner_product_param { num_output: 10 weight_filler { type: "gaussian" std: 0.1 } } }\n'
              'layer { name: "loss" type: "SoftmaxWithLoss" bottom: "ip" bottom: "label" top: "loss" }\n'
              'layer { name: "accuracy" type: "Accuracy" bottom: "ip" bottom: "label" top: "accuracy"\n'
              '  accuracy_param { top_k: %d } include { phase: TEST } }\n' % top_k)


MNIST_CNN_SOLVER = (
    'base_lr: 0.05 lr_policy: "step" gamma: 0.5 stepsize: 1000 momentum: 0.9 weight_decay: 0.0001\n'
    'max_iter: 1000 test_iter: 3 test_interval: 10\n')
