"""MI355X-native leaky ring-attractor RNN time loop (forward + BPTT) behind the operator API of
chongxi/rnn_train_ring_attractor's cpp/ring_rnn_cuda.py."""
from .ring_rnn_cuda import RingRnnCudaFunc, ring_rnn_cuda_func  # noqa: F401
from .rnn_cuda import bwd_cuda, fwd_cuda  # noqa: F401
