"""Training entry points of the two gain-network models, with the reference scripts' defaults and call pattern
(train/train_ring_attractor.py:301-452 and train/train_general_ring_attractor.py:203-340 there), minus the figures:
dataset of pre-generated AV trials -> initial bump -> model (gain networks + time loop on the HIP operators) -> loss
pair -> clip -> Adam, then one long evaluation trial decoded two ways.  `fused=True` runs the objective as chained HIP
operators (`model.loss_pair`) and the optimizer step as the fused clip + Adam; the default follows the reference's
chain of torch loss ops and `torch.optim.Adam`."""
import math

import torch

from . import host


def sanity_check_loss(batch_size=128, seq_len=120, num_neurons=360, seed=0):
    """The reference's own acceptance check (train/train_ring_attractor.py:327-348): the model with fixed cosine
    weights and no gain networks ('debug_perfect', N = 360, gelu) integrates angular velocity well enough that the
    cosine-similarity loss of its read-out stays below 0.5.  Returns that loss."""
    torch.manual_seed(seed)
    device = torch.device("cuda")
    data = host.AVIntegrationDataset(num_samples=batch_size, seq_len=seq_len, zero_padding_start_ratio=0.1,
                                     zero_ratios_in_rest=[0.2, 0.5, 0.8], device=device)
    model = host.LeakyRingAttractor(num_neurons, tau=10, dt=1, activation="gelu", initialization="debug_perfect").to(device)
    model.eval()
    av, target = data.generate_batch(batch_size)
    with torch.no_grad():
        wave, _ = model(av, r_init=host.create_initial_bump(target[:, 0], num_neurons, device=device))
        return float(host.cosine_similarity_loss(wave, target))


def _train(model, to_model_input, num_neurons, training_steps, batch_size, seq_len, lr, log_every, fused):
    device = torch.device("cuda")
    data = host.AVIntegrationDataset(num_samples=min(training_steps * batch_size, 200_000), seq_len=seq_len,
                                     zero_padding_start_ratio=0.1, zero_ratios_in_rest=[0.2, 0.5, 0.8], device=device)
    if fused:
        from .device_aux import FusedClipAdam
        opt = FusedClipAdam(model.parameters(), lr=lr, max_norm=1.0)
    else:
        opt = torch.optim.Adam(model.parameters(), lr=lr)
    history = []
    for step in range(training_steps):
        av, target = data.generate_batch(batch_size)
        r_init = host.create_initial_bump(target[:, 0], num_neurons, device=device)
        if fused:
            total, loss, bump_loss, _ = model.loss_pair(to_model_input(av), target, r_init=r_init, bump_weight=0.2)
        else:
            wave, bump = model(to_model_input(av), r_init=r_init)
            loss, bump_loss = host.cosine_similarity_loss(wave, target), host.bump_amplitude_loss(bump)
            total = loss + 0.2 * bump_loss
        opt.zero_grad()
        total.backward()
        if not fused:
            torch.nn.utils.clip_grad_norm_(model.parameters(), 1.0)
        opt.step()
        history.append(float(total.detach()))
        if log_every and step % log_every == 0:
            print(f"Step {step}/{training_steps}, Total Loss: {history[-1]:.4f}, Main loss: {float(loss.detach()):.4f}, "
                  f"Bump loss: {float(bump_loss.detach()):.4f}")
    print("Training finished.")
    return history


def _evaluate(model, to_model_input, seq_len, seed):
    """One test trial (1 % leading zeros, 30 % of the rest zeroed) from the model's default bump at pi, the target
    aligned to that start; decoded by population vector and by argmax."""
    torch.manual_seed(seed)
    test = host.AVIntegrationDataset(num_samples=1, seq_len=seq_len, zero_padding_start_ratio=0.01,
                                     zero_ratios_in_rest=[0.3], device="cuda")
    av, target = test.generate_batch(1)
    aligned = (target + (math.pi - target[:, 0].unsqueeze(1))) % (2 * math.pi)
    model.eval()
    with torch.no_grad():
        wave, bump = model(to_model_input(av))
    out = {"aligned_target": aligned, "cos_activity": wave, "bump_activity": bump}
    for name, decode in (("pv", host.decode_angle_from_population_vector), ("argmax", host.decode_angle_from_argmax)):
        angle = decode(wave)
        err = torch.remainder(angle - aligned + math.pi, 2 * math.pi) - math.pi
        out[f"decoded_{name}"], out[f"mean_abs_error_{name}"] = angle, float(err.abs().mean())
    print(f"Mean absolute decoding error: population vector {out['mean_abs_error_pv']:.4f} rad, "
          f"argmax {out['mean_abs_error_argmax']:.4f} rad")
    return out


def run_leaky_training_and_evaluation(num_neurons=120, training_steps=1000, batch_size=128, seq_len=120, lr=1e-3,
                                      activation="gelu", hidden_gain_neurons=3, log_every=10, seed=0, fused=False,
                                      sanity_check=True, eval_seq_len=200):
    """LeakyRingAttractor (two gain networks on the angular velocity).  Returns (model, loss history, evaluation)."""
    if sanity_check:
        loss = sanity_check_loss(batch_size, seq_len, seed=seed)
        print(f"Loss for the fixed-weight model: {loss:.6f} ({'passed' if loss < 0.5 else 'higher than expected'})")
    torch.manual_seed(seed)
    model = host.LeakyRingAttractor(num_neurons, tau=10, dt=1, activation=activation, initialization="random",
                                    hidden_gain_neurons=hidden_gain_neurons).to("cuda")
    history = _train(model, lambda av: av, num_neurons, training_steps, batch_size, seq_len, lr, log_every, fused)
    return model, history, _evaluate(model, lambda av: av, eval_seq_len, seed + 1)


def run_general_training_and_evaluation(action_dim=2, num_neurons=120, training_steps=1000, batch_size=128, seq_len=120,
                                        lr=1e-3, activation="gelu", hidden_gain_neurons=3, log_every=10, seed=0,
                                        fused=False, eval_seq_len=200):
    """GeneralizedRingAttractor (one gain network per action channel); the angular-velocity task always feeds it the
    two-channel (L, R) signal, as the reference does.  Returns (model, loss history, evaluation)."""
    if action_dim != 2:
        raise ValueError("the angular-velocity task drives the two-channel (L, R) action signal: action_dim must be 2")
    torch.manual_seed(seed)
    model = host.GeneralizedRingAttractor(num_neurons, action_dim=action_dim, tau=10, dt=1, activation=activation,
                                          initialization="random", hidden_gain_neurons=hidden_gain_neurons).to("cuda")
    history = _train(model, host.av_to_action_signal, num_neurons, training_steps, batch_size, seq_len, lr, log_every, fused)
    return model, history, _evaluate(model, host.av_to_action_signal, eval_seq_len, seed + 1)
