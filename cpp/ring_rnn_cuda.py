"""Drop-in module path `cpp.ring_rnn_cuda` (the reference script does `from cpp.ring_rnn_cuda import *`)."""
import torch  # noqa: F401  (star-importers rely on this name)
from torch.autograd import Function  # noqa: F401
from rnn_train_ring_attractor_amd.rnn_cuda import fwd_cuda, bwd_cuda  # noqa: F401
from rnn_train_ring_attractor_amd.ring_rnn_cuda import ring_rnn_cuda_func, RingRnnCudaFunc  # noqa: F401
