"""Host-side companions of the operator: the helpers the reference training script imports next to
`ring_rnn_cuda_func` (initial bump, losses, decoders, action-signal builders, the AV dataset) and the
nn.Module that wraps the operator.  All plain torch; they run on whatever device their inputs are on.

Counterparts (reference paths): train/train_ring_attractor.py:10-52, 190-298;
utils/generate_av_integration_data.py:11-58, 111-215; train_general_ring_no_gain.py:21-118, 176-229.
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn


def non_linear(x, activation_name):
    fns = {"tanh": torch.tanh, "relu": torch.relu, "gelu": torch.nn.functional.gelu, "silu": torch.nn.functional.silu}
    if activation_name not in fns:
        raise ValueError(f"Activation function {activation_name} not supported")
    return fns[activation_name](x)


def create_initial_bump(initial_angles, num_neurons, bump_width_factor=10, device="cpu"):
    """Gaussian bump on the ring (circular index distance, sigma = N / factor), unit L2 norm per row."""
    ang = initial_angles.to(device)
    centre = (ang * num_neurons / (2 * math.pi)).unsqueeze(1)
    idx = torch.arange(num_neurons, device=device).unsqueeze(0)
    dist = (idx - centre).abs()
    dist = torch.minimum(dist, num_neurons - dist)
    sigma = num_neurons / bump_width_factor
    bump = torch.exp(-dist.pow(2) / (2 * sigma * sigma))
    return bump / bump.norm(dim=1, keepdim=True)


def _preferred_angles(n, like):
    return torch.linspace(0, 2 * math.pi, n, device=like.device)   # end point included, as the reference does


def cosine_similarity_loss(predicted_cosine_wave, true_angle):
    pa = _preferred_angles(predicted_cosine_wave.shape[-1], predicted_cosine_wave)
    x = (predicted_cosine_wave * torch.cos(pa)).sum(-1)
    y = (predicted_cosine_wave * torch.sin(pa)).sum(-1)
    theta = torch.atan2(y, x)
    return torch.mean((torch.cos(theta) - torch.cos(true_angle)) ** 2 + (torch.sin(theta) - torch.sin(true_angle)) ** 2)


def bump_amplitude_loss(bump_activity, target_amplitude=None):
    total = bump_activity.abs().sum(dim=2)
    if target_amplitude is None:
        target_amplitude = total[:, 0:1]
    return torch.mean((total - target_amplitude) ** 2)


def decode_angle_from_population_vector(activity):
    pa = _preferred_angles(activity.shape[-1], activity).view(1, 1, -1)
    x = (torch.cos(pa) * activity).sum(dim=2)
    y = (torch.sin(pa) * activity).sum(dim=2)
    return (torch.atan2(y, x) + 2 * math.pi) % (2 * math.pi)


def decode_angle_from_argmax(activity):
    pa = _preferred_angles(activity.shape[-1], activity)
    return pa[torch.argmax(activity, dim=2)]


def plot_ring_matrices(ring_rnn, title_prefix=""):
    """Plotting is outside the accelerated path; kept as a no-op so driver scripts need no edits."""
    return None


def av_to_action_signal(av_signal):
    return torch.stack([torch.relu(-av_signal), torch.relu(av_signal)], dim=2)


def av_to_action_signal_ND(av_signal, action_dim=16, zero_padding=True):
    if zero_padding:
        out = torch.zeros(*av_signal.shape, action_dim, device=av_signal.device, dtype=av_signal.dtype)
        out[:, :, 0] = torch.relu(-av_signal)
        out[:, :, 1] = torch.relu(av_signal)
        if action_dim > 2:
            # what this construction guarantees, for the operator: channels 2.. are identically zero
            from .ring_rnn_cuda import DRIVEN_ATTR
            setattr(out, DRIVEN_ATTR, (0, 1))
        return out
    scales = torch.linspace(-1, 1, action_dim, device=av_signal.device, dtype=av_signal.dtype)
    return torch.relu(av_signal.unsqueeze(-1) * scales)


def generate_av_integration_data_ultra_fast(num_trials, seq_len, zero_padding_start_ratio=0.1, zero_ratios_in_rest=None,
                                            max_av=0.1 * math.pi, device="cpu"):
    """Vectorised AV trials: leading zeros, then exactly len_rest - floor(len_rest*ratio) randomly placed
    U(-max_av, max_av) draws per trial; angle = initial + exclusive cumulative sum, modulo 2*pi."""
    ratios = [0.2, 0.5, 0.8] if zero_ratios_in_rest is None else list(zero_ratios_in_rest)
    n0 = int(seq_len * zero_padding_start_ratio)
    rest = seq_len - n0
    av = torch.zeros(num_trials, seq_len, device=device)
    angle0 = torch.rand(num_trials, device=device) * 2 * math.pi
    pick = torch.randint(0, len(ratios), (num_trials,), device=device)
    n_nonzero = rest - (rest * torch.tensor(ratios, device=device)[pick]).long()
    if rest > 0:
        values = (torch.rand(num_trials, rest, device=device) - 0.5) * 2 * max_av
        order = torch.rand(num_trials, rest, device=device).argsort(dim=1)
        av[:, n0:] = values * (order < n_nonzero.unsqueeze(1)).float()
    angle = torch.zeros(num_trials, seq_len, device=device)
    angle[:, 0] = angle0
    angle[:, 1:] = (angle0.unsqueeze(1) + torch.cumsum(av[:, :-1], dim=1)) % (2 * math.pi)
    return av, angle


def generate_av_integration_data_chunked(num_trials, seq_len, zero_padding_start_ratio=0.1, zero_ratios_in_rest=None,
                                         max_av=0.1 * math.pi, device="cpu", chunk_size=10000):
    """The same trials generated `chunk_size` at a time and concatenated (bounded temporaries for large sets;
    reference: utils/generate_av_integration_data.py:61-108)."""
    parts = [generate_av_integration_data_ultra_fast(min(chunk_size, num_trials - start), seq_len, zero_padding_start_ratio,
                                                     zero_ratios_in_rest, max_av, device)
             for start in range(0, num_trials, chunk_size)]
    return torch.cat([a for a, _ in parts]), torch.cat([g for _, g in parts])


class AVIntegrationDataset(torch.utils.data.Dataset):
    """Pre-generated AV trials with a shuffled batch cursor (generate_batch wraps and reshuffles)."""

    def __init__(self, num_samples, seq_len, zero_padding_start_ratio=0.1, zero_ratios_in_rest=None,
                 max_av=0.1 * math.pi, device="cpu", fast_mode=True, chunk_size=10000):
        self.num_samples, self.seq_len, self.device = num_samples, seq_len, torch.device(device)
        self.av_data, self.angle_data = generate_av_integration_data_chunked(
            num_samples, seq_len, zero_padding_start_ratio, zero_ratios_in_rest, max_av, device, chunk_size)
        self.current_index = 0
        self.shuffled_indices = torch.randperm(num_samples, device=device)

    def __len__(self):
        return self.num_samples

    def __getitem__(self, idx):
        if idx >= self.num_samples:
            raise IndexError(f"Index {idx} out of range for dataset of size {self.num_samples}")
        return self.av_data[idx], self.angle_data[idx]

    def reset_batch_iterator(self):
        self.current_index = 0
        self.shuffled_indices = torch.randperm(self.num_samples, device=self.device)

    def get_memory_usage_mb(self):
        """Megabytes held by the pre-generated trials (utils/generate_av_integration_data.py:206-211)."""
        return (self.av_data.element_size() * self.av_data.nelement()
                + self.angle_data.element_size() * self.angle_data.nelement()) / (1024 * 1024)

    def generate_batch(self, batch_size):
        if batch_size > self.num_samples:
            raise ValueError(f"Batch size {batch_size} cannot be larger than dataset size {self.num_samples}")
        end = self.current_index + batch_size
        if end <= self.num_samples:
            idx = self.shuffled_indices[self.current_index:end]
            self.current_index = end
        else:
            head = end - self.num_samples
            idx = torch.cat([self.shuffled_indices[self.current_index:], self.shuffled_indices[:head]])
            self.current_index = head
            if self.current_index > 0.8 * self.num_samples:
                self.reset_batch_iterator()
        return self.av_data[idx], self.angle_data[idx]


class GeneralizedRingAttractorNoGain(nn.Module):
    """r += alpha * (-r + F(J0*sum(r) + J1*Wo r + sum_c A_c Wa_c r)) through the HIP operator; returns the
    max-normalised cosine read-out and the raw bump, both [B,T,N]."""

    def __init__(self, num_neurons, action_dim=2, tau=10.0, dt=1.0, activation="tanh", initialization="random"):
        super().__init__()
        self.num_neurons, self.action_dim, self.activation_name = num_neurons, action_dim, activation
        idx = torch.arange(num_neurons, dtype=torch.float32)
        diff = 2 * math.pi * (idx[:, None] - idx[None, :]) / num_neurons
        self.register_buffer("W_delta7", torch.cos(diff))
        self.J0, self.J1 = -0.1, 0.1
        scale = 1.0 / math.sqrt(num_neurons)
        self.Wo = nn.Parameter(torch.randn(num_neurons, num_neurons) * scale)
        if initialization == "random":
            self.Wa = nn.Parameter(torch.randn(action_dim, num_neurons, num_neurons) * scale)
        elif initialization == "perfect":
            phases = [math.pi / 4, -math.pi / 4] if action_dim == 2 else [c * 2 * math.pi / action_dim for c in range(action_dim)]
            self.Wa = nn.Parameter(torch.stack([torch.cos(diff + ph) for ph in phases]))
        else:
            raise ValueError(f"Unknown initialization: {initialization}")

    def forward_history(self, action_signal, r_init=None):
        """bump_history [T,B,N] as the operator returns it (no read-out): the input of `ring_loss_pair`."""
        from .ring_rnn_cuda import ring_rnn_cuda_func
        batch_size, _, action_dim = action_signal.shape
        assert action_dim == self.action_dim, f"Expected action_dim {self.action_dim}, got {action_dim}"
        if r_init is None:
            angle = torch.full((batch_size,), math.pi, device=self.Wo.device)
            r_init = create_initial_bump(angle, self.num_neurons, device=self.Wo.device)
        return ring_rnn_cuda_func(action_signal=action_signal, Wa=self.Wa, J0=self.J0, J1=self.J1, Wo=self.Wo,
                                  r_init=r_init, alpha=0.15, activation=self.activation_name)

    def loss_pair(self, action_signal, target_angle, r_init=None, bump_weight=0.2):
        """(total, cos_loss, amp_loss, bump_history) of the training script's objective, time loop and loss head as
        one operator: its backward forms the loss gradient inside the BPTT kernel where the geometry allows."""
        from .loss_head import ring_rnn_loss_func
        batch_size, _, action_dim = action_signal.shape
        assert action_dim == self.action_dim, f"Expected action_dim {self.action_dim}, got {action_dim}"
        if r_init is None:
            angle = torch.full((batch_size,), math.pi, device=self.Wo.device)
            r_init = create_initial_bump(angle, self.num_neurons, device=self.Wo.device)
        return ring_rnn_loss_func(action_signal, self.Wa, self.J0, self.J1, self.Wo, r_init, 0.15, self.activation_name,
                                  target_angle, bump_weight)

    def forward(self, action_signal, r_init=None):
        bump = self.forward_history(action_signal, r_init).permute(1, 0, 2)
        proj = bump @ self.W_delta7
        return (proj / proj.max(dim=2, keepdim=True)[0]).clone(), bump.clone()


class GeneralizedRingAttractor(nn.Module):
    """The general ring with one learned input gain per action channel (reference:
    train/train_general_ring_attractor.py:22-153): A[b,t,c] = action[b,t,c] * gain_c(|action[b,t,c]|), each gain a
    1 -> h -> 1 MLP (GELU hidden, softplus output), then the leaky recurrence over `action_dim` action matrices
    through the HIP operator, which also returns dL/d action_signal for the gain networks.  Same constructor,
    parameter names (`gain_nets`, `Wo`, `Wa`) and return values as the reference."""

    def __init__(self, num_neurons, action_dim=2, tau=10.0, dt=1.0, activation="tanh", initialization="random",
                 hidden_gain_neurons=16):
        super().__init__()
        self.num_neurons, self.action_dim, self.tau, self.dt = num_neurons, action_dim, tau, dt
        self.activation_name, self.initialization = activation, initialization
        self.gain_nets = nn.ModuleList([
            nn.Sequential(nn.Linear(1, hidden_gain_neurons), nn.GELU(), nn.Linear(hidden_gain_neurons, 1), nn.Softplus())
            for _ in range(action_dim)])
        idx = torch.arange(num_neurons, dtype=torch.float32)
        diff = 2 * math.pi * (idx[:, None] - idx[None, :]) / num_neurons
        self.register_buffer("W_delta7", torch.cos(diff))
        self.J0, self.J1 = -0.1, 0.1
        scale = 1.0 / math.sqrt(num_neurons)
        self.Wo = nn.Parameter(torch.randn(num_neurons, num_neurons) * scale)
        if initialization == "random":
            self.Wa = nn.Parameter(torch.randn(action_dim, num_neurons, num_neurons) * scale)
        elif initialization == "perfect":
            phases = [math.pi / 4, -math.pi / 4] if action_dim == 2 else [c * 2 * math.pi / action_dim for c in range(action_dim)]
            self.Wa = nn.Parameter(torch.stack([torch.cos(diff + ph) for ph in phases]))
        else:
            raise ValueError(f"Unknown initialization: {initialization}")

    def gated_action_signal(self, action_signal):
        """[B,T,k] action signal -> action * gain(|action|) per channel.  On the GPU all gain networks run as one HIP
        operator (forward and backward); on the CPU (tests of the module itself) as the torch modules they are."""
        if action_signal.is_cuda:
            from .gain import pack_gain_nets, ring_gain_func
            return ring_gain_func(action_signal, pack_gain_nets(list(self.gain_nets)))
        gains = [net(action_signal[:, :, c:c + 1].abs()) for c, net in enumerate(self.gain_nets)]
        return action_signal * torch.cat(gains, dim=2)

    def forward_history(self, action_signal, r_init=None):
        """bump_history [T,B,N] as the operator returns it (gain networks, then the time loop; no read-out)."""
        from .ring_rnn_cuda import ring_rnn_cuda_func
        batch_size, _, action_dim = action_signal.shape
        assert action_dim == self.action_dim, f"Expected action_dim {self.action_dim}, got {action_dim}"
        if r_init is None:
            angle = torch.full((batch_size,), math.pi, device=self.Wo.device)
            r_init = create_initial_bump(angle, self.num_neurons, device=self.Wo.device)
        return ring_rnn_cuda_func(action_signal=self.gated_action_signal(action_signal), Wa=self.Wa, J0=self.J0,
                                  J1=self.J1, Wo=self.Wo, r_init=r_init, alpha=0.15, activation=self.activation_name)

    def loss_pair(self, action_signal, target_angle, r_init=None, bump_weight=0.2):
        """(total, cos_loss, amp_loss, bump_history) of the training objective with gain networks, time loop and loss
        head chained as HIP operators (see GeneralizedRingAttractorNoGain.loss_pair); the gain networks train through
        dL/d action_signal, which the fused backward returns."""
        from .loss_head import ring_rnn_loss_func
        batch_size, _, action_dim = action_signal.shape
        assert action_dim == self.action_dim, f"Expected action_dim {self.action_dim}, got {action_dim}"
        if r_init is None:
            angle = torch.full((batch_size,), math.pi, device=self.Wo.device)
            r_init = create_initial_bump(angle, self.num_neurons, device=self.Wo.device)
        return ring_rnn_loss_func(self.gated_action_signal(action_signal), self.Wa, self.J0, self.J1, self.Wo, r_init,
                                  0.15, self.activation_name, target_angle, bump_weight)

    def forward(self, action_signal, r_init=None):
        bump = self.forward_history(action_signal, r_init).permute(1, 0, 2)
        proj = bump @ self.W_delta7
        return (proj / proj.max(dim=2, keepdim=True)[0]).clone(), bump.clone()


def plot_general_ring_matrices(ring_rnn, title_prefix=""):
    """Plotting is outside the accelerated path; kept as a no-op so driver scripts need no edits."""
    return None


class LeakyRingAttractor(nn.Module):
    """The two-channel model with learned input gains (reference: train/train_ring_attractor.py:55-187):
    L = gain_l(relu(-av)) * relu(-av), R = gain_r(relu(av)) * relu(av), each gain a 1 -> h -> 1 MLP (GELU hidden,
    softplus output) applied per sample and step, then the leaky recurrence with [Wl, Wr] through the HIP operator.
    The operator returns dL/d action_signal, so the gain networks train through it.  Parameter names follow the
    reference (Wo, Wl, Wr, gain_r_net, gain_l_net); 'debug_perfect' fixes the weights and bypasses the gains."""

    def __init__(self, num_neurons, tau=10.0, dt=1.0, activation="tanh", initialization="random", hidden_gain_neurons=16):
        super().__init__()
        self.num_neurons, self.tau, self.dt = num_neurons, tau, dt
        self.activation_name, self.initialization = activation, initialization

        def gain_net():
            return nn.Sequential(nn.Linear(1, hidden_gain_neurons), nn.GELU(), nn.Linear(hidden_gain_neurons, 1),
                                 nn.Softplus())

        self.gain_r_net, self.gain_l_net = gain_net(), gain_net()
        idx = torch.arange(num_neurons, dtype=torch.float32)
        diff = 2 * math.pi * (idx[:, None] - idx[None, :]) / num_neurons
        self.register_buffer("W_delta7", torch.cos(diff))
        self.J0, self.J1 = -0.1, 0.1
        if initialization == "random":
            scale = 1.0 / math.sqrt(num_neurons)
            self.Wo = nn.Parameter(torch.randn(num_neurons, num_neurons) * scale)
            self.Wl = nn.Parameter(torch.randn(num_neurons, num_neurons) * scale)
            self.Wr = nn.Parameter(torch.randn(num_neurons, num_neurons) * scale)
        elif initialization in ("perfect", "debug_perfect"):
            learn = initialization == "perfect"
            if not learn:
                self.gain_r_net = self.gain_l_net = None
            self.Wo = nn.Parameter(torch.cos(diff), requires_grad=learn)
            self.Wl = nn.Parameter(torch.cos(diff + math.pi / 4), requires_grad=learn)
            self.Wr = nn.Parameter(torch.cos(diff - math.pi / 4), requires_grad=learn)
        else:
            raise ValueError(f"Unknown initialization type: {initialization}")

    def action_signal(self, av_signal):
        """[B,T] angular velocity -> [B,T,2] gated (L, R) channels.  On the GPU both gain networks run as one HIP
        operator (forward and backward); on the CPU (tests of the module itself) as the torch modules they are."""
        left, right = torch.relu(-av_signal).unsqueeze(2), torch.relu(av_signal).unsqueeze(2)
        if self.gain_l_net is None:
            return torch.cat([left, right], dim=2)
        if av_signal.is_cuda:
            from .gain import pack_gain_nets, ring_gain_func
            return ring_gain_func(torch.cat([left, right], dim=2), pack_gain_nets([self.gain_l_net, self.gain_r_net]))
        return torch.cat([self.gain_l_net(left) * left, self.gain_r_net(right) * right], dim=2)

    def forward_history(self, av_signal, r_init=None):
        """bump_history [T,B,N] as the operator returns it (gain networks, then the time loop; no read-out)."""
        from .ring_rnn_cuda import ring_rnn_cuda_func
        batch_size = av_signal.shape[0]
        if r_init is None:
            angle = torch.full((batch_size,), math.pi, device=self.Wo.device)
            r_init = create_initial_bump(angle, self.num_neurons, device=self.Wo.device)
        return ring_rnn_cuda_func(action_signal=self.action_signal(av_signal), Wa=torch.stack([self.Wl, self.Wr]),
                                  J0=self.J0, J1=self.J1, Wo=self.Wo, r_init=r_init, alpha=0.15,
                                  activation=self.activation_name)

    def loss_pair(self, av_signal, target_angle, r_init=None, bump_weight=0.2):
        """(total, cos_loss, amp_loss, bump_history) of the training objective (train/train_ring_attractor.py:275-298 of
        the reference: cosine-similarity loss of the read-out + bump_weight * bump-amplitude loss) with gain networks,
        time loop and loss head as HIP operators; the gain networks train through dL/d action_signal."""
        from .loss_head import ring_rnn_loss_func
        batch_size = av_signal.shape[0]
        if r_init is None:
            angle = torch.full((batch_size,), math.pi, device=self.Wo.device)
            r_init = create_initial_bump(angle, self.num_neurons, device=self.Wo.device)
        return ring_rnn_loss_func(self.action_signal(av_signal), torch.stack([self.Wl, self.Wr]), self.J0, self.J1,
                                  self.Wo, r_init, 0.15, self.activation_name, target_angle, bump_weight)

    def forward(self, av_signal, r_init=None):
        bump = self.forward_history(av_signal, r_init).permute(1, 0, 2)
        proj = bump @ self.W_delta7
        return proj / proj.max(dim=2, keepdim=True)[0], bump
