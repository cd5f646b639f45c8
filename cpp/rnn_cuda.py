"""Drop-in module path `cpp.rnn_cuda` exporting `fwd_cuda` and `bwd_cuda`."""
from rnn_train_ring_attractor_amd.rnn_cuda import fwd_cuda, bwd_cuda  # noqa: F401
