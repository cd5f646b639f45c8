"""Module path `train.train_general_ring_no_gain`: the general ring without gain networks."""
from rnn_train_ring_attractor_amd.host import (  # noqa: F401
    GeneralizedRingAttractorNoGain, av_to_action_signal, av_to_action_signal_ND, plot_general_ring_matrices,
    AVIntegrationDataset, non_linear, create_initial_bump, cosine_similarity_loss, bump_amplitude_loss,
    decode_angle_from_population_vector, decode_angle_from_argmax, plot_ring_matrices)
