"""MI355X-native leaky ring-attractor RNN time loop (forward + BPTT) behind the operator API of
chongxi/rnn_train_ring_attractor's cpp/ring_rnn_cuda.py."""

_EXPORTS = {
    "ring_rnn_cuda_func": "ring_rnn_cuda", "RingRnnCudaFunc": "ring_rnn_cuda",
    "fwd_cuda": "rnn_cuda", "bwd_cuda": "rnn_cuda",
    "ring_loss_pair": "loss_head", "RingLossPair": "loss_head",
    "ring_rnn_loss_func": "loss_head", "RingRnnLossFunc": "loss_head",
    "generate_inputs": "device_aux", "FusedClipAdam": "device_aux",
    "ring_gain_func": "gain", "RingGainFunc": "gain", "pack_gain_nets": "gain",
}


def __getattr__(name):          # resolved on first use so `python -m ...build` does not import torch
    if name in _EXPORTS:
        import importlib
        return getattr(importlib.import_module(f"{__name__}.{_EXPORTS[name]}"), name)
    raise AttributeError(name)
