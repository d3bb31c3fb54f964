"""Caffe-like network structure on the NArray front end, with the unit classes, graph
traversal, update rule and snapshot layout of the reference's owl.net package
(owl/owl/net/net.py, net_helper.py, trainer.py).  What is left out: the LMDB / image-list /
window data providers and Caffe's protobuf classes -- networks are described in Caffe's
prototxt TEXT, which a small parser here reads (no protobuf), and batches come from memory."""
from .net import *  # noqa: F401,F403
from .net_helper import NetBuilder, parse_prototxt, save_net_to_file, init_net_from_file  # noqa: F401
from .trainer import NetTrainer, NetTester  # noqa: F401
