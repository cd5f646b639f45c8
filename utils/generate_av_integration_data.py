"""Module path `utils.generate_av_integration_data`."""
from rnn_train_ring_attractor_amd.host import (  # noqa: F401
    AVIntegrationDataset, generate_av_integration_data_ultra_fast, generate_av_integration_data_chunked)
