"""Training driver with the reference script's import lines and call pattern (no plotting):
AV batches -> action signal -> initial bump -> ring_rnn_cuda_func -> loss pair -> clip -> Adam.
fused_loss=True computes the same loss pair with the fused HIP loss head instead of the chain of torch tensor ops
(one pass over the history instead of about a dozen) and lets the backward kernels form its gradient themselves."""
import numpy as np

from utils.generate_av_integration_data import AVIntegrationDataset
from train.train_ring_attractor import (
    create_initial_bump, cosine_similarity_loss, bump_amplitude_loss, decode_angle_from_population_vector)
from cpp.ring_rnn_cuda import *  # noqa: F401,F403  (also provides `torch`)
from rnn_train_ring_attractor_amd.host import GeneralizedRingAttractorNoGain, av_to_action_signal_ND


def run_training(action_dim=2, num_neurons=256, training_steps=1000, batch_size=128, seq_len=100, lr=1e-3,
                 activation="gelu", log_every=10, seed=0, fused_loss=False, fused_optimizer=False):
    torch.manual_seed(seed)
    device = torch.device("cuda")
    data = AVIntegrationDataset(num_samples=min(training_steps * batch_size, 200_000), seq_len=seq_len,
                                zero_padding_start_ratio=0.1, zero_ratios_in_rest=[0.2, 0.5, 0.8], device="cuda")
    model = GeneralizedRingAttractorNoGain(num_neurons, action_dim=action_dim, activation=activation).to(device)
    if fused_optimizer:       # clip_grad_norm_ + Adam.step() as three kernel launches
        from rnn_train_ring_attractor_amd import FusedClipAdam
        opt = FusedClipAdam(model.parameters(), lr=lr, max_norm=1.0)
    else:
        opt = torch.optim.Adam(model.parameters(), lr=lr)
    history = []
    for step in range(training_steps):
        av, target = data.generate_batch(batch_size)
        action = av_to_action_signal_ND(av, action_dim)
        r_init = create_initial_bump(target[:, 0], num_neurons, device=device)
        if fused_loss:
            total, loss, _, _ = model.loss_pair(action, target, r_init=r_init, bump_weight=0.2)
        else:
            wave, bump = model(action, r_init=r_init)
            loss = cosine_similarity_loss(wave, target)
            total = loss + 0.2 * bump_amplitude_loss(bump)
        opt.zero_grad()
        total.backward()
        if not fused_optimizer:
            torch.nn.utils.clip_grad_norm_(model.parameters(), 1.0)
        opt.step()
        history.append(float(total))
        if log_every and step % log_every == 0:
            print(f"Step {step}/{training_steps}, Total Loss: {history[-1]:.4f}, Main loss: {float(loss):.4f}")
    return model, history


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser(description="Train the ring attractor (no gain networks) on the HIP operator")
    ap.add_argument("--action_dim", type=int, default=16)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--fused_loss", action="store_true", help="loss pair and its gradient by the fused HIP loss head")
    ap.add_argument("--fused_optimizer", action="store_true", help="gradient clipping + Adam as one fused HIP step")
    a = ap.parse_args()
    run_training(action_dim=a.action_dim, training_steps=a.steps, fused_loss=a.fused_loss,
                 fused_optimizer=a.fused_optimizer)
