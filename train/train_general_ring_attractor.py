"""Module path `train.train_general_ring_attractor`: the general ring with per-channel gain networks."""
from rnn_train_ring_attractor_amd.host import (  # noqa: F401
    GeneralizedRingAttractor, av_to_action_signal, plot_general_ring_matrices, AVIntegrationDataset, non_linear,
    create_initial_bump, cosine_similarity_loss, bump_amplitude_loss, decode_angle_from_population_vector,
    decode_angle_from_argmax, plot_ring_matrices)
from rnn_train_ring_attractor_amd.drivers import (  # noqa: F401,E402
    run_general_training_and_evaluation as run_training_and_evaluation)
