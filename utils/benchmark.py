"""Module path `utils.benchmark`: the comparison and latency helpers the reference's scripts import."""
from rnn_train_ring_attractor_amd.bench_utils import set_seed, check_tensor_match, measure_latency_cuda  # noqa: F401
