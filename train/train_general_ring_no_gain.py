"""Module path `train.train_general_ring_no_gain`: the general ring without gain networks."""
from rnn_train_ring_attractor_amd.host import (  # noqa: F401
    GeneralizedRingAttractorNoGain, av_to_action_signal, av_to_action_signal_ND, plot_general_ring_matrices,
    AVIntegrationDataset, non_linear, create_initial_bump, cosine_similarity_loss, bump_amplitude_loss,
    decode_angle_from_population_vector, decode_angle_from_argmax, plot_ring_matrices)


def run_training_and_evaluation(action_dim=2, **kwargs):
    """The entry point of this module path with its defaults in the reference (train/train_general_ring_no_gain.py:
    185-330 there: 120 neurons, sequences of 120 steps); the loop itself is the root driver's."""
    import train_general_ring_no_gain as driver
    kwargs.setdefault("num_neurons", 120)
    kwargs.setdefault("seq_len", 120)
    return driver.run_training_and_evaluation(action_dim=action_dim, **kwargs)
