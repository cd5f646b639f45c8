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
                 activation="gelu", log_every=10, seed=0, fused_loss=False, fused_optimizer=False, hip_graph=False):
    """hip_graph=True records one training step (action signal, initial bump, time loop, loss head, backward, clipping
    and Adam) into a HIP graph after three eager steps and replays it for the rest of the run: one graph launch per
    step instead of some thirty kernel launches and the Python between them.  It needs both fused options (their
    kernels neither allocate through HIP nor read the device back, and the fused optimizer counts its steps on the
    device); the loss values stay on the device and are read only where they are printed and at the end."""
    torch.manual_seed(seed)
    device = torch.device("cuda")
    if hip_graph and not (fused_loss and fused_optimizer):
        raise ValueError("hip_graph=True records the fused loss head and the fused optimizer step: "
                         "pass fused_loss=True and fused_optimizer=True")
    data = AVIntegrationDataset(num_samples=min(training_steps * batch_size, 200_000), seq_len=seq_len,
                                zero_padding_start_ratio=0.1, zero_ratios_in_rest=[0.2, 0.5, 0.8], device="cuda")
    model = GeneralizedRingAttractorNoGain(num_neurons, action_dim=action_dim, activation=activation).to(device)
    if fused_optimizer:       # clip_grad_norm_ + Adam.step() as three kernel launches
        from rnn_train_ring_attractor_amd import FusedClipAdam
        opt = FusedClipAdam(model.parameters(), lr=lr, max_norm=1.0, capturable=hip_graph)
    else:
        opt = torch.optim.Adam(model.parameters(), lr=lr)

    def train_step(av, target):
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
        return total.detach(), loss.detach()

    def report(step, total, loss):
        if log_every and step % log_every == 0:
            print(f"Step {step}/{training_steps}, Total Loss: {float(total):.4f}, Main loss: {float(loss):.4f}")

    if not hip_graph:
        history = []
        for step in range(training_steps):
            total, loss = train_step(*data.generate_batch(batch_size))
            history.append(float(total))
            report(step, total, loss)
        return model, history

    # Graph mode: the batch lands in two static tensors, everything behind them is recorded once.
    static_av = torch.empty(batch_size, seq_len, device=device)
    static_target = torch.empty(batch_size, seq_len, device=device)
    totals = torch.zeros(training_steps, device=device)

    def load_batch():
        av, target = data.generate_batch(batch_size)
        static_av.copy_(av)
        static_target.copy_(target)

    eager_steps = min(3, training_steps)          # real training steps; they also settle the allocator
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for step in range(eager_steps):
            load_batch()
            total, loss = train_step(static_av, static_target)
            totals[step] = total
            report(step, total, loss)
    torch.cuda.current_stream().wait_stream(side)
    if eager_steps < training_steps:
        opt.zero_grad()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            g_total, g_loss = train_step(static_av, static_target)
        for step in range(eager_steps, training_steps):
            load_batch()
            graph.replay()
            totals[step] = g_total
            report(step, g_total, g_loss)
    return model, totals.tolist()


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
    ap.add_argument("--hip_graph", action="store_true",
                    help="record the training step into a HIP graph and replay it (implies both fused options)")
    a = ap.parse_args()
    run_training_and_evaluation(action_dim=a.action_dim, training_steps=a.steps, fused_loss=a.fused_loss or a.hip_graph,
                                fused_optimizer=a.fused_optimizer or a.hip_graph, hip_graph=a.hip_graph)
