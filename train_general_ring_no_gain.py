"""Training driver with the reference script's import lines and call pattern (no plotting):
AV batches -> action signal -> initial bump -> ring_rnn_cuda_func -> loss pair -> clip -> Adam.
fused_loss=True computes the same loss pair with the fused HIP loss head instead of the chain of torch tensor ops
(one pass over the history instead of about a dozen) and lets the backward kernels form its gradient themselves."""
import numpy as np

from utils.generate_av_integration_data import AVIntegrationDataset
from train.train_ring_attractor import (
    create_initial_bump, cosine_similarity_loss, bump_amplitude_loss, decode_angle_from_population_vector,
    decode_angle_from_argmax)
from cpp.ring_rnn_cuda import *  # noqa: F401,F403  (also provides `torch`)
from rnn_train_ring_attractor_amd.host import (  # noqa: F401
    GeneralizedRingAttractorNoGain, av_to_action_signal, av_to_action_signal_ND, plot_general_ring_matrices)


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


def evaluate(model, action_dim, seq_len=100, seed=1):
    """The reference script's evaluation without its figure (train_general_ring_no_gain.py:345-376): one test trial
    (1 % leading zeros, 30 % of the rest zeroed), the model started from its default bump at pi, the target aligned
    to that start; returns the decoded angles and their mean absolute circular error against the aligned target."""
    torch.manual_seed(seed)
    test = AVIntegrationDataset(num_samples=1, seq_len=seq_len, zero_padding_start_ratio=0.01, zero_ratios_in_rest=[0.3],
                                device="cuda", fast_mode=True)
    av, target = test.generate_batch(1)
    action = av_to_action_signal_ND(av, action_dim)
    aligned = (target + (np.pi - target[:, 0].unsqueeze(1))) % (2 * np.pi)
    model.eval()
    with torch.no_grad():
        cos_activity, bump_activity = model(action)
    out = {"aligned_target": aligned, "cos_activity": cos_activity, "bump_activity": bump_activity}
    for name, dec in (("pv", decode_angle_from_population_vector), ("argmax", decode_angle_from_argmax)):
        angle = dec(cos_activity)
        err = torch.remainder(angle - aligned + np.pi, 2 * np.pi) - np.pi
        out[f"decoded_{name}"] = angle
        out[f"mean_abs_error_{name}"] = float(err.abs().mean())
    return out


def run_training_and_evaluation(action_dim=2, training_steps=1000, **train_kwargs):
    """The reference entry point's name and defaults (N = 256, 1000 steps of batch 128 x 100, gelu, Adam 1e-3):
    training, then `evaluate`.  Returns (model, loss history, evaluation dictionary)."""
    model, history = run_training(action_dim=action_dim, training_steps=training_steps, **train_kwargs)
    print("Training finished.")
    result = evaluate(model, action_dim, seq_len=train_kwargs.get("seq_len", 100))
    print(f"Mean absolute decoding error: population vector {result['mean_abs_error_pv']:.4f} rad, "
          f"argmax {result['mean_abs_error_argmax']:.4f} rad")
    return model, history, result


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser(description="Train the ring attractor (no gain networks) on the HIP operator")
    ap.add_argument("--action_dim", type=int, default=16)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--fused_loss", action="store_true", help="loss pair and its gradient by the fused HIP loss head")
    ap.add_argument("--fused_optimizer", action="store_true", help="gradient clipping + Adam as one fused HIP step")
    a = ap.parse_args()
    run_training_and_evaluation(action_dim=a.action_dim, training_steps=a.steps, fused_loss=a.fused_loss,
                                fused_optimizer=a.fused_optimizer)
