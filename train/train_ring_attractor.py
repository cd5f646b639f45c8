"""Module path `train.train_ring_attractor`: the helper names the CUDA-backed training script imports."""
from rnn_train_ring_attractor_amd.host import (  # noqa: F401
    non_linear, create_initial_bump, cosine_similarity_loss, bump_amplitude_loss,
    decode_angle_from_population_vector, decode_angle_from_argmax, plot_ring_matrices, LeakyRingAttractor)
from rnn_train_ring_attractor_amd.drivers import (  # noqa: F401,E402
    run_leaky_training_and_evaluation as run_training_and_evaluation, sanity_check_loss)
