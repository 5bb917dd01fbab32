"""GPU integration: the drop-in API (GradSampleModule, ghost clipping, DPOptimizer,
PrivacyEngine.make_private) against the CPU oracle and plain autograd, on down-scaled
versions of the five benchmark configurations. Modelled on the reference's own tests
(opacus/tests/grad_samples/common.py, privacy_engine_test.py,
grad_sample_module_fast_gradient_clipping_test.py, randomness_test.py)."""

import copy
import math

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.utils.data import DataLoader, TensorDataset

from oracle import dp_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda"


@pytest.fixture(scope="module")
def A():
    import opacus_amd

    return opacus_amd


@pytest.fixture(autouse=True, params=[True, False], ids=["autograd_wgrads", "params_off"])
def weight_grad_mode(request, monkeypatch):
    """Every test of this file runs in both modes of the hooks: autograd's own (non-private) weight
    gradients kept, as in the reference and by default, and switched off during forward
    (``autograd_weight_grads=False``)."""
    from opacus_amd.grad_sample.grad_sample_module import GradSampleHooks

    monkeypatch.setattr(GradSampleHooks, "DEFAULT_AUTOGRAD_WEIGHT_GRADS", request.param)
    return request.param


def per_sample_grads_cpu(model, x, y, loss_fn, batch_dim=0):
    """Batch-of-one autograd on the CPU: the reference's microbatch oracle."""
    names = [k for k, p in model.named_parameters() if p.requires_grad]
    out = {k: [] for k in names}
    for i in range(x.shape[batch_dim]):
        model.zero_grad()
        xi = x.narrow(batch_dim, i, 1)
        loss_fn(model(xi), y[i : i + 1]).backward()
        for k, p in model.named_parameters():
            if p.requires_grad:
                out[k].append(p.grad.clone())
    model.zero_grad()
    return {k: torch.stack(v) for k, v in out.items()}


def close(got, want, rtol, atol, msg=""):
    torch.testing.assert_close(got.detach().float().cpu(), want.detach().float().cpu(), rtol=rtol, atol=atol, msg=lambda m: f"{msg}: {m}")


def test_small_model_step_in_one_launch_leaves_the_same_bits(A, monkeypatch):
    """DPOptimizer.step of a small model runs clip factors, clipped sum, noise and scaling as one kernel
    (optimizer.py:444-504 in one pass). p.grad and p.summed_grad must be bit for bit what the
    separate kernels leave, with and without noise (same generator seed: same Philox stream), for a
    parameter list with sizes that are and are not multiples of four; and virtual steps, which
    need the sum kept apart from the noise, must still take the separate kernels."""
    from opacus_amd.optimizers.optimizer import DPOptimizer

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.conv = nn.Conv2d(1, 6, 5, stride=2)
            self.fc1 = nn.Linear(6 * 12 * 12, 33)
            self.fc2 = nn.Linear(33, 10)

        def forward(self, x):
            return self.fc2(F.relu(self.fc1(F.relu(self.conv(x)).flatten(1))))

    torch.manual_seed(11)
    net = Net()
    n = 96
    x, y = torch.randn(n, 1, 28, 28).to(DEV), torch.randint(0, 10, (n,)).to(DEV)
    used = []
    real = DPOptimizer._fused_small_step

    def run(sigma, fused, skip_first=False):
        model = A.GradSampleModule(copy.deepcopy(net).to(DEV))
        g = torch.Generator(device=DEV).manual_seed(1234)
        opt = A.DPOptimizer(torch.optim.SGD(model.parameters(), lr=0.1), noise_multiplier=sigma, max_grad_norm=0.7,
                            expected_batch_size=n, generator=g)
        monkeypatch.setattr(DPOptimizer, "_fused_small_step", (lambda self: (used.append(real(self)), used[-1])[1]) if fused else (lambda self: False))
        out = []
        for step in range(2):
            opt.zero_grad()
            F.cross_entropy(model(x), y).backward()
            if skip_first and step == 0:
                opt.signal_skip_step(True)
            else:
                opt.signal_skip_step(False)
            opt.step()
            out.append([(p.grad.clone() if p.grad is not None else None, p.summed_grad.clone()) for p in model.parameters()])
        return out, g.get_offset()

    for sigma in (0.0, 1.3):
        used.clear()
        one, off1 = run(sigma, True)
        assert used == [True, True]
        sep, off2 = run(sigma, False)
        assert off1 == off2  # the generator moved by the same amount
        for s1, s2 in zip(one, sep):
            for (g1, sm1), (g2, sm2) in zip(s1, s2):
                assert torch.equal(g1, g2) and torch.equal(sm1, sm2)
        if sigma:
            assert not torch.equal(one[0][0][0], one[1][0][0])  # fresh noise every step
    # a skipped (virtual) step and the step that follows it keep the sum apart: separate kernels
    used.clear()
    one, _ = run(1.3, True, skip_first=True)
    assert used == [False, False]
    sep, _ = run(1.3, False, skip_first=True)
    for step, (s1, s2) in enumerate(zip(one, sep)):
        for (g1, sm1), (g2, sm2) in zip(s1, s2):
            assert torch.equal(sm1, sm2)
            if step == 1:  # (after the skipped step p.grad is whatever autograd's own pass left)
                assert torch.equal(g1, g2)


# ---- models (down-scaled versions of the benchmark configurations) -----------------------------
class SmallCNN(nn.Module):
    """Config 1: Conv(1,16,8,2,3) ReLU MaxPool Conv(16,32,4,2) ReLU MaxPool Linear(512,32) ReLU Linear(32,10)."""

    def __init__(self):
        super().__init__()
        self.conv1 = nn.Conv2d(1, 16, 8, 2, padding=3)
        self.conv2 = nn.Conv2d(16, 32, 4, 2)
        self.fc1 = nn.Linear(32 * 4 * 4, 32)
        self.fc2 = nn.Linear(32, 10)

    def forward(self, x):
        x = F.max_pool2d(F.relu(self.conv1(x)), 2, 1)
        x = F.max_pool2d(F.relu(self.conv2(x)), 2, 1)
        return self.fc2(F.relu(self.fc1(x.flatten(1))))


class ResBlock(nn.Module):
    """Config 4: two 3x3 convolutions with GroupNorm and a skip, then a small head."""

    def __init__(self, ch=16, groups=8):
        super().__init__()
        self.c1, self.g1 = nn.Conv2d(ch, ch, 3, padding=1), nn.GroupNorm(groups, ch)
        self.c2, self.g2 = nn.Conv2d(ch, ch, 3, padding=1), nn.GroupNorm(groups, ch)
        self.head = nn.Linear(ch, 10)

    def forward(self, x):
        h = F.relu(self.g1(self.c1(x)))
        h = F.relu(self.g2(self.c2(h)) + x)
        return self.head(h.mean(dim=(2, 3)))


class TinyLlama(nn.Module):
    """Config 5, down-scaled: embedding, RMSNorm, grouped-query attention with rotary
    embedding (no parameters), SwiGLU, untied LM head; all bias-free."""

    def __init__(self, vocab=50, d=32, heads=4, kv=2, ffn=48, layers=2):
        super().__init__()
        self.emb = nn.Embedding(vocab, d)
        self.heads, self.kv, self.hd = heads, kv, d // heads
        self.blocks = nn.ModuleList()
        for _ in range(layers):
            self.blocks.append(
                nn.ModuleDict(
                    dict(
                        n1=nn.RMSNorm(d, eps=1e-5),
                        q=nn.Linear(d, d, bias=False),
                        k=nn.Linear(d, kv * self.hd, bias=False),
                        v=nn.Linear(d, kv * self.hd, bias=False),
                        o=nn.Linear(d, d, bias=False),
                        n2=nn.RMSNorm(d, eps=1e-5),
                        gate=nn.Linear(d, ffn, bias=False),
                        up=nn.Linear(d, ffn, bias=False),
                        down=nn.Linear(ffn, d, bias=False),
                    )
                )
            )
        self.norm = nn.RMSNorm(d, eps=1e-5)
        self.lm_head = nn.Linear(d, vocab, bias=False)

    @staticmethod
    def rope(x):
        B, H, T, D = x.shape
        pos = torch.arange(T, device=x.device, dtype=torch.float32)
        inv = 1.0 / (10000 ** (torch.arange(0, D, 2, device=x.device, dtype=torch.float32) / D))
        ang = pos[:, None] * inv[None, :]
        cos, sin = ang.cos().to(x.dtype), ang.sin().to(x.dtype)
        x1, x2 = x[..., 0::2], x[..., 1::2]
        return torch.stack([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1).flatten(-2)

    def forward(self, ids):
        h = self.emb(ids)
        B, T, _ = h.shape
        for blk in self.blocks:
            a = blk["n1"](h)
            q = blk["q"](a).view(B, T, self.heads, self.hd).transpose(1, 2)
            k = blk["k"](a).view(B, T, self.kv, self.hd).transpose(1, 2)
            v = blk["v"](a).view(B, T, self.kv, self.hd).transpose(1, 2)
            q, k = self.rope(q), self.rope(k)
            rep = self.heads // self.kv
            k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
            att = F.scaled_dot_product_attention(q, k, v, is_causal=True)
            h = h + blk["o"](att.transpose(1, 2).reshape(B, T, -1))
            m = blk["n2"](h)
            h = h + blk["down"](F.silu(blk["gate"](m)) * blk["up"](m))
        return self.lm_head(self.norm(h))


def ce_sum(out, y):
    return F.cross_entropy(out, y, reduction="sum")


# ---- per-sample gradients through the hooks --------------------------------------------------
@pytest.mark.parametrize("loss_reduction", ["mean", "sum"])
def test_small_cnn_grad_samples(A, loss_reduction):
    torch.manual_seed(0)
    net = SmallCNN()
    n = 8
    x, y = torch.randn(n, 1, 28, 28), torch.randint(0, 10, (n,))
    want = per_sample_grads_cpu(net, x, y, ce_sum)
    gsm = A.GradSampleModule(copy.deepcopy(net).to(DEV), loss_reduction=loss_reduction)
    F.cross_entropy(gsm(x.to(DEV)), y.to(DEV), reduction=loss_reduction).backward()
    for k, p in gsm._module.named_parameters():
        assert p.grad_sample.shape == (n, *p.shape)
        close(p.grad_sample, want[k], 1e-4, 1e-5, k)  # the reference's own tolerance (common.py:50-51)
        # and the stricter bar of this build: relative to the tensor's scale
        assert (p.grad_sample.cpu() - want[k]).abs().max() <= 2e-5 * want[k].abs().max()


def test_res_block_grad_samples(A):
    torch.manual_seed(1)
    net = ResBlock()
    n = 5
    x, y = torch.randn(n, 16, 8, 8), torch.randint(0, 10, (n,))
    want = per_sample_grads_cpu(net, x, y, ce_sum)
    gsm = A.GradSampleModule(copy.deepcopy(net).to(DEV), loss_reduction="mean")
    F.cross_entropy(gsm(x.to(DEV)), y.to(DEV)).backward()
    for k, p in gsm._module.named_parameters():
        close(p.grad_sample, want[k], 1e-3, 1e-4, k)  # conv tolerance of the reference (conv2d_test.py:84-85)
        assert (p.grad_sample.cpu() - want[k]).abs().max() <= 5e-5 * want[k].abs().max(), k


def test_layer_norm_and_instance_norm_grad_samples(A):
    """LayerNorm and InstanceNorm have kernels of their own (no functorch fallback): per-sample
    gradients against batch-of-one autograd, as tests/grad_samples/layer_norm_test.py and
    instance_norm2d_test.py do."""

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.conv = nn.Conv2d(3, 6, 3, padding=1)
            self.inorm = nn.InstanceNorm2d(6, affine=True)
            self.ln = nn.LayerNorm([6, 5, 5])
            self.fc = nn.Linear(150, 4)

        def forward(self, x):
            return self.fc(self.ln(F.relu(self.inorm(self.conv(x)))).flatten(1))

    torch.manual_seed(5)
    net = Net()
    n = 6
    x, y = torch.randn(n, 3, 5, 5), torch.randint(0, 4, (n,))
    want = per_sample_grads_cpu(net, x, y, ce_sum)
    gsm = A.GradSampleModule(copy.deepcopy(net).to(DEV), loss_reduction="mean")
    from opacus_amd.grad_sample import GradSampleHooks

    assert nn.LayerNorm in GradSampleHooks.GRAD_SAMPLERS and nn.InstanceNorm2d in GradSampleHooks.GRAD_SAMPLERS
    F.cross_entropy(gsm(x.to(DEV)), y.to(DEV)).backward()
    for k, p in gsm._module.named_parameters():
        assert p.grad_sample.shape == (n, *p.shape), k
        close(p.grad_sample, want[k], 1e-3, 1e-5, k)


def test_conv3d_and_conv1d_grad_samples(A):
    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.c3 = nn.Conv3d(2, 4, (2, 3, 3), stride=(1, 2, 1), padding=(0, 1, 1), groups=2)
            self.c1 = nn.Conv1d(4, 5, 3, padding="same")
            self.fc = nn.Linear(5, 3)

        def forward(self, x):
            h = F.relu(self.c3(x))  # [n, 4, 3, 3, 6]
            h = F.relu(self.c1(h.flatten(2)))  # [n, 5, 54]
            return self.fc(h.mean(dim=2))

    torch.manual_seed(8)
    net = Net()
    n = 4
    x, y = torch.randn(n, 2, 4, 6, 6), torch.randint(0, 3, (n,))
    want = per_sample_grads_cpu(net, x, y, ce_sum)
    gsm = A.GradSampleModule(copy.deepcopy(net).to(DEV), loss_reduction="mean")
    F.cross_entropy(gsm(x.to(DEV)), y.to(DEV)).backward()
    for k, p in gsm._module.named_parameters():
        assert p.grad_sample.shape == (n, *p.shape), k
        close(p.grad_sample, want[k], 1e-3, 1e-5, k)


def test_embedding_bag_grad_samples(A):
    """nn.EmbeddingBag through the wrapper, with offsets and with a 2-D index tensor; bags hold
    distinct indices so that batch-of-one autograd is the reference."""

    class Net(nn.Module):
        def __init__(self, mode):
            super().__init__()
            self.bag = nn.EmbeddingBag(11, 6, mode=mode)
            self.fc = nn.Linear(6, 3)

        def forward(self, index, offsets=None):
            return self.fc(self.bag(index, offsets))

    for mode in ("sum", "mean"):
        torch.manual_seed(6)
        net = Net(mode)
        index2d = torch.stack([torch.randperm(11)[:4] for _ in range(5)])
        y = torch.randint(0, 3, (5,))
        gsm = A.GradSampleModule(copy.deepcopy(net).to(DEV), loss_reduction="mean")
        for flat in (False, True):
            gsm.zero_grad()
            if flat:
                out = gsm(index2d.reshape(-1).to(DEV), torch.arange(0, 20, 4).to(DEV))
            else:
                out = gsm(index2d.to(DEV))
            F.cross_entropy(out, y.to(DEV)).backward()
            for i in range(5):
                net.zero_grad()
                F.cross_entropy(net(index2d[i : i + 1]), y[i : i + 1], reduction="sum").backward()
                close(gsm._module.bag.weight.grad_sample[i], net.bag.weight.grad, 1e-5, 1e-7, f"{mode} bag {i}")
                close(gsm._module.fc.weight.grad_sample[i], net.fc.weight.grad, 1e-5, 1e-7)


@pytest.mark.parametrize("batch_first", [True, False])
def test_sequence_model_grad_samples(A, batch_first):
    """Embedding -> Linear over [batch, seq]; also with the batch in dimension 1."""
    torch.manual_seed(2)

    class Seq(nn.Module):
        def __init__(self):
            super().__init__()
            self.emb = nn.Embedding(20, 12)
            self.fc = nn.Linear(12, 7)

        def forward(self, ids):
            return self.fc(torch.tanh(self.emb(ids)))

    net = Seq()
    n, T = 6, 9
    ids = torch.randint(0, 20, (n, T) if batch_first else (T, n))
    tgt = torch.randn(n, T, 7) if batch_first else torch.randn(T, n, 7)
    bdim = 0 if batch_first else 1

    def loss_i(out, t):
        return (out - t).pow(2).sum()

    names = [k for k, _ in net.named_parameters()]
    want = {k: [] for k in names}
    for i in range(n):
        net.zero_grad()
        loss_i(net(ids.narrow(bdim, i, 1)), tgt.narrow(bdim, i, 1)).backward()
        for k, p in net.named_parameters():
            want[k].append(p.grad.clone())
    want = {k: torch.stack(v) for k, v in want.items()}
    gsm = A.GradSampleModule(copy.deepcopy(net).to(DEV), loss_reduction="sum", batch_first=batch_first)
    loss_i(gsm(ids.to(DEV)), tgt.to(DEV)).backward()
    for k, p in gsm._module.named_parameters():
        close(p.grad_sample, want[k], 1e-4, 1e-5, k)


class RecurrentNet(nn.Module):
    """A recurrent layer and a Linear head on its last output (batch-first tensors), or on the
    final hidden state for packed input."""

    def __init__(self, rnn):
        super().__init__()
        self.rnn = rnn
        self.head = nn.Linear(rnn.hidden_size * (2 if rnn.bidirectional else 1), 3)

    def forward(self, x):
        out, state = self.rnn(x)
        if isinstance(out, torch.nn.utils.rnn.PackedSequence):
            h = state[0] if isinstance(state, tuple) else state
            last = torch.cat([h[-2], h[-1]], dim=1) if self.rnn.bidirectional else h[-1]
        else:
            last = out.mean(dim=1 if self.rnn.batch_first else 0)  # every step feeds the loss
        return self.head(last)


@pytest.mark.parametrize("kind", ["lstm", "gru", "rnn"])
@pytest.mark.parametrize("packed", [False, True])
def test_recurrent_layers_grad_samples_and_ghost_norms(A, kind, packed):
    """dp_rnn_test.py / grad_samples/dp_rnn_test.py: DPLSTM, DPGRU, DPRNN produce torch.nn's
    outputs from torch.nn's state dict, and their per-sample gradients (input projection
    contracted over time in one call, recurrent projection over its stacked uses) equal
    batch-of-one autograd through the torch.nn module; two layers, bidirectional, packed
    sequences of unsorted lengths (row i of every gradient is sample i of the caller's batch,
    also for the recurrent parameters); ghost norms equal the norms of those gradients."""
    from torch.nn.utils.rnn import pack_padded_sequence

    from opacus_amd.layers import DPGRU, DPLSTM, DPRNN

    torch.manual_seed(31 + packed)
    DP, NN = {"lstm": (DPLSTM, nn.LSTM), "gru": (DPGRU, nn.GRU), "rnn": (DPRNN, nn.RNN)}[kind]
    kw = dict(num_layers=2, bidirectional=True, batch_first=True)
    ref = RecurrentNet(NN(5, 6, **kw))
    net = RecurrentNet(DP(5, 6, **kw))
    assert [k for k, _ in net.named_parameters()] == [k for k, _ in ref.named_parameters()]
    net.load_state_dict(ref.state_dict())
    n, T = 5, 7
    x, y = torch.randn(n, T, 5), torch.randn(n, 3)
    lengths = torch.tensor([4, 7, 2, 7, 5])

    def feed(xx, ll, dev="cpu"):
        if not packed:
            return xx.to(dev)
        return pack_padded_sequence(xx, ll, batch_first=True, enforce_sorted=False).to(dev)

    want = {k: [] for k, _ in ref.named_parameters()}
    for i in range(n):
        ref.zero_grad()
        (ref(feed(x[i : i + 1], lengths[i : i + 1])) - y[i : i + 1]).pow(2).sum().backward()
        for k, p in ref.named_parameters():
            want[k].append(p.grad.clone())
    want = {k: torch.stack(v) for k, v in want.items()}
    close(net(feed(x, lengths)), ref(feed(x, lengths)), 1e-5, 1e-6, "forward on the CPU")

    gsm = A.GradSampleModule(copy.deepcopy(net).to(DEV), loss_reduction="sum")
    out = gsm(feed(x, lengths, DEV))
    close(out, ref(feed(x, lengths)), 1e-4, 1e-5, "forward")
    (out - y.to(DEV)).pow(2).sum().backward()
    for k, p in gsm._module.named_parameters():
        assert p.grad_sample.shape == want[k].shape, k
        close(p.grad_sample, want[k], 1e-4, 1e-5, k)
    # a second pass must start clean (pending uses and counters were consumed)
    gsm.zero_grad()
    (gsm(feed(x, lengths, DEV)) - y.to(DEV)).pow(2).sum().backward()
    for k, p in gsm._module.named_parameters():
        close(p.grad_sample, want[k], 1e-4, 1e-5, f"second pass {k}")

    ghost = A.GradSampleModuleFastGradientClipping(copy.deepcopy(net).to(DEV), loss_reduction="sum", max_grad_norm=1.0)
    (ghost(feed(x, lengths, DEV)) - y.to(DEV)).pow(2).sum().backward()
    for k, p in ghost._module.named_parameters():
        assert p.grad_sample is None
        close(p._norm_sample, want[k].flatten(1).norm(dim=1), 1e-4, 1e-6, f"ghost {k}")


@pytest.mark.parametrize("batch_first", [False, True])
def test_multihead_attention_grad_samples(A, batch_first):
    """grad_samples/dp_multihead_attention_test.py: per-sample gradients of the four projections
    and of the key/value sequence biases equal batch-of-one autograd through
    torch.nn.MultiheadAttention holding the same state."""
    from opacus_amd.layers import DPMultiheadAttention

    torch.manual_seed(41)
    E, H, N, L, S = 8, 2, 4, 5, 6
    ref = nn.MultiheadAttention(E, H, add_bias_kv=True, add_zero_attn=True, batch_first=batch_first)
    dp = DPMultiheadAttention(E, H, add_bias_kv=True, add_zero_attn=True, batch_first=batch_first)
    dp.load_state_dict(ref.state_dict())
    bdim = 0 if batch_first else 1
    q = torch.randn(N, L, E) if batch_first else torch.randn(L, N, E)
    kv = torch.randn(N, S, E) if batch_first else torch.randn(S, N, E)
    tgt = torch.randn_like(q)
    want = {k: [] for k, _ in ref.named_parameters()}
    for i in range(N):
        ref.zero_grad()
        qi, kvi = q.narrow(bdim, i, 1), kv.narrow(bdim, i, 1)
        (ref(qi, kvi, kvi)[0] - tgt.narrow(bdim, i, 1)).pow(2).sum().backward()
        for k, p in ref.named_parameters():
            want[k].append(p.grad.clone())
    want = {k: torch.stack(v) for k, v in want.items()}
    wq, wk, wv = want["in_proj_weight"].chunk(3, dim=1)
    bq, bk, bv = want["in_proj_bias"].chunk(3, dim=1)
    mapped = {
        "qlinear.weight": wq, "klinear.weight": wk, "vlinear.weight": wv,
        "qlinear.bias": bq, "klinear.bias": bk, "vlinear.bias": bv,
        "out_proj.weight": want["out_proj.weight"], "out_proj.bias": want["out_proj.bias"],
        "seq_bias_k.bias": want["bias_k"].reshape(N, E), "seq_bias_v.bias": want["bias_v"].reshape(N, E),
    }
    gsm = A.GradSampleModule(dp.to(DEV), loss_reduction="sum", batch_first=batch_first)
    out, _ = gsm(q.to(DEV), kv.to(DEV), kv.to(DEV))
    close(out, ref(q, kv, kv)[0], 1e-4, 1e-5, "forward")
    (out - tgt.to(DEV)).pow(2).sum().backward()
    got = dict(gsm._module.named_parameters())
    assert set(got) == set(mapped)
    for k, w in mapped.items():
        close(got[k].grad_sample, w, 1e-4, 1e-5, k)


def test_accumulation_tied_parameters_and_functorch_fallback(A):
    torch.manual_seed(3)

    class Tied(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = nn.Linear(6, 6)
            self.ln = nn.LayerNorm(6)  # no kernel here: generic fallback

        def forward(self, x):
            return self.ln(self.fc(torch.relu(self.fc(x))))

    net = Tied()
    x, y = torch.randn(4, 6), torch.randn(4, 6)

    def mse(out, t):
        return (out - t).pow(2).sum()

    want = per_sample_grads_cpu(net, x, y, mse)
    gsm = A.GradSampleModule(copy.deepcopy(net).to(DEV), loss_reduction="sum")
    mse(gsm(x.to(DEV)), y.to(DEV)).backward()
    for k, p in gsm._module.named_parameters():
        assert isinstance(p.grad_sample, torch.Tensor)
        close(p.grad_sample, want[k], 1e-4, 1e-5, k)
    # a second backward without zero_grad stacks a list; the optimizer concatenates it
    mse(gsm(x.to(DEV)), y.to(DEV)).backward()
    assert all(isinstance(p.grad_sample, list) and len(p.grad_sample) == 2 for p in gsm.parameters())
    opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=0.0), noise_multiplier=0.0, max_grad_norm=1e20, expected_batch_size=4)
    assert opt.accumulated_iterations == 2
    opt.step()
    for k, p in gsm._module.named_parameters():
        close(p.grad, 2 * want[k].sum(0) / (4 * 2), 1e-4, 1e-5, k)


# ---- DPOptimizer ------------------------------------------------------------------------------
def _train(A, net, batches, *, private, sigma=0.0, C=1e20, lr=0.1, seed=None, generator=None, secure=False):
    net = copy.deepcopy(net).to(DEV)
    opt = torch.optim.SGD(net.parameters(), lr=lr)
    model = net
    if private:
        model = A.GradSampleModule(net, loss_reduction="mean")
        opt = A.DPOptimizer(opt, noise_multiplier=sigma, max_grad_norm=C, expected_batch_size=batches[0][0].shape[0], generator=generator, secure_mode=secure)
    if seed is not None:
        torch.manual_seed(seed)
    for x, y in batches:
        opt.zero_grad()
        F.cross_entropy(model(x.to(DEV)), y.to(DEV)).backward()
        opt.step()
    return [p.detach().cpu() for p in net.parameters()]


def test_private_equals_vanilla_when_nothing_clips(A):
    """sigma = 0, C = 1e20 (privacy_engine_test.py:220-273: atol 1e-7 one step, 1e-4 three, rtol 1e-3)."""
    torch.manual_seed(4)
    net = SmallCNN()
    batches = [(torch.randn(8, 1, 28, 28), torch.randint(0, 10, (8,))) for _ in range(3)]
    for steps, atol in ((1, 1e-7), (3, 1e-4)):
        van = _train(A, net, batches[:steps], private=False)
        prv = _train(A, net, batches[:steps], private=True)
        for v, p in zip(van, prv):
            torch.testing.assert_close(p, v, atol=atol, rtol=1e-3)
    clipped = _train(A, net, batches[:1], private=True, C=0.01)
    noised = _train(A, net, batches[:1], private=True, sigma=1.0, C=1.0)
    assert not torch.allclose(clipped[0], van[0]) and not torch.allclose(noised[0], van[0])


def test_flat_clipping_batch_of_one_has_norm_C(A):
    """privacy_engine_test.py:302-327."""
    torch.manual_seed(5)
    C = 0.5
    gsm = A.GradSampleModule(SmallCNN().to(DEV), loss_reduction="mean")
    opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=C, expected_batch_size=1)
    F.cross_entropy(gsm(torch.randn(1, 1, 28, 28, device=DEV)), torch.tensor([3], device=DEV)).backward()
    opt.clip_and_accumulate()
    total = math.sqrt(sum(p.summed_grad.double().pow(2).sum().item() for p in gsm.parameters()))
    assert round(total, 3) == C


def test_clipped_sum_matches_oracle_and_sumsq_cache_is_guarded(A):
    torch.manual_seed(6)
    net = ResBlock()
    n, C = 6, 0.3
    x, y = torch.randn(n, 16, 8, 8), torch.randint(0, 10, (n,))
    want_gs = per_sample_grads_cpu(net, x, y, ce_sum)
    names = list(want_gs)
    norms, clip, summed = O.clip_and_accumulate([want_gs[k] for k in names], C)
    gsm = A.GradSampleModule(copy.deepcopy(net).to(DEV), loss_reduction="sum")
    opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=C, expected_batch_size=n, loss_reduction="sum")
    ce_sum(gsm(x.to(DEV)), y.to(DEV)).backward()
    # tamper with one per-sample gradient in place: the squared norms its kernel left behind
    # are stale now and must not be used
    w = gsm._module.c1.weight
    assert getattr(w.grad_sample, "_dpk_sumsq", None) is not None
    w.grad_sample.mul_(3.0)
    want_gs["c1.weight"] = want_gs["c1.weight"] * 3.0
    norms, clip, summed = O.clip_and_accumulate([want_gs[k] for k in names], C)
    opt.clip_and_accumulate()
    for (k, p), s in zip(gsm._module.named_parameters(), summed):
        assert (p.summed_grad.cpu() - s).abs().max() <= 5e-5 * s.abs().max(), k
    with pytest.raises(ValueError, match="haven't been cleared"):
        opt.clip_and_accumulate()  # same grad samples twice


def test_virtual_steps_accumulate_summed_grad(A):
    torch.manual_seed(7)
    net = nn.Linear(10, 4)
    xs = [torch.randn(5, 10) for _ in range(2)]
    ys = [torch.randint(0, 4, (5,)) for _ in range(2)]
    C = 0.2
    gsm = A.GradSampleModule(copy.deepcopy(net).to(DEV), loss_reduction="mean")
    opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=1.0), noise_multiplier=0.0, max_grad_norm=C, expected_batch_size=10)
    opt.signal_skip_step(True)
    opt.signal_skip_step(False)
    results = []
    for x, y in zip(xs, ys):
        opt.zero_grad()
        F.cross_entropy(gsm(x.to(DEV)), y.to(DEV)).backward()
        results.append(opt.step())
    assert results[0] is None
    total = None
    for x, y in zip(xs, ys):
        gs = per_sample_grads_cpu(net, x, y, ce_sum)
        _, _, summed = O.clip_and_accumulate([gs["weight"], gs["bias"]], C)
        total = summed if total is None else [a + b for a, b in zip(total, summed)]
    close(gsm._module.weight.grad, total[0] / 10, 1e-4, 1e-6)
    close(gsm._module.bias.grad, total[1] / 10, 1e-4, 1e-6)


def test_batch_memory_manager_equals_one_large_batch(A):
    """Logical batches of 12 run as physical batches of at most 5 give the update of the
    undivided batch (sigma = 0), and the model only moves at the end of a logical batch
    (the reference's tests/batch_memory_manager_test.py checks the same two things)."""
    from opacus_amd.utils.batch_memory_manager import BatchMemoryManager

    torch.manual_seed(11)
    net = nn.Sequential(nn.Linear(6, 8), nn.ReLU(), nn.Linear(8, 3))
    x, y = torch.randn(24, 6), torch.randint(0, 3, (24,))
    dl = DataLoader(TensorDataset(x, y), batch_size=12, shuffle=False)

    def make():
        gsm = A.GradSampleModule(copy.deepcopy(net).to(DEV), loss_reduction="mean")
        opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=0.5), noise_multiplier=0.0, max_grad_norm=0.3, expected_batch_size=12)
        return gsm, opt

    whole, opt_w = make()
    for xb, yb in dl:
        opt_w.zero_grad()
        F.cross_entropy(whole(xb.to(DEV)), yb.to(DEV)).backward()
        opt_w.step()

    pieces, opt_p = make()
    moved = []
    with BatchMemoryManager(data_loader=dl, max_physical_batch_size=5, optimizer=opt_p) as dl2:
        for xb, yb in dl2:
            assert len(xb) <= 5
            before = pieces._module[0].weight.detach().clone()
            opt_p.zero_grad()
            F.cross_entropy(pieces(xb.to(DEV)), yb.to(DEV), reduction="sum").div(len(xb)).backward()
            opt_p.step()
            moved.append(not torch.equal(before, pieces._module[0].weight.detach()))
    assert moved == [False, False, True, False, False, True]
    for pw, pp in zip(whole.parameters(), pieces.parameters()):
        close(pp, pw, 1e-5, 1e-6, "parameters after two logical batches")


def test_per_layer_clipping_matches_oracle(A):
    """perlayeroptimizer.py:58-76 through ``make_private(clipping="per_layer")``: every parameter
    clipped on its own norm, all of them in one launch with a [K, n] factor table."""
    torch.manual_seed(21)
    net = SmallCNN()
    x, y = torch.randn(6, 1, 28, 28), torch.randint(0, 10, (6,))
    bounds = [0.05, 0.5, 0.02, 1e3, 0.3, 0.01, 0.2, 0.4]
    gs = per_sample_grads_cpu(net, x, y, ce_sum)
    names = [k for k, _ in net.named_parameters()]
    _, want = O.per_layer_clip_and_accumulate([gs[k] for k in names], bounds)
    model = copy.deepcopy(net).to(DEV)
    engine = A.PrivacyEngine()
    dl = DataLoader(TensorDataset(x, y), batch_size=6)
    gsm, opt, _ = engine.make_private(
        module=model, optimizer=torch.optim.SGD(model.parameters(), lr=0.0), data_loader=dl, noise_multiplier=0.0,
        max_grad_norm=bounds, poisson_sampling=False, clipping="per_layer",
    )
    assert type(opt).__name__ == "DPPerLayerOptimizer"
    opt.zero_grad()
    F.cross_entropy(gsm(x.to(DEV)), y.to(DEV)).backward()
    opt.step()
    for (k, p), w in zip(gsm._module.named_parameters(), want):
        close(p.grad, w / 6, 2e-4, 1e-7, f"per-layer clipped mean gradient of {k}")
    # a second, accumulated step (virtual batch) adds into summed_grad with the same table form
    opt.signal_skip_step(True)
    opt.zero_grad()
    F.cross_entropy(gsm(x.to(DEV)), y.to(DEV)).backward()
    assert opt.step() is None
    opt.zero_grad()
    F.cross_entropy(gsm(x.to(DEV)), y.to(DEV)).backward()
    opt.step()
    for (k, p), w in zip(gsm._module.named_parameters(), want):
        close(p.grad, 2 * w / 6, 2e-4, 1e-7, f"accumulated per-layer gradient of {k}")


def test_adaptive_clipping_counts_and_updates_the_bound(A):
    """adaclipoptimizer.py: unclipped count from the clip factors, bound update after a full step."""
    torch.manual_seed(22)
    net = nn.Linear(12, 5)
    x, y = torch.randn(16, 12), torch.randint(0, 5, (16,))
    gs = per_sample_grads_cpu(net, x, y, ce_sum)
    C = float(torch.sqrt(gs["weight"].flatten(1).pow(2).sum(1) + gs["bias"].pow(2).sum(1)).median())
    _, clip, summed = O.clip_and_accumulate([gs["weight"], gs["bias"]], C)
    count, new_bound = O.adaclip_update(clip, C, 0.7, 0.2, 0.01, 100.0)
    assert 0 < count < 16
    gsm = A.GradSampleModule(copy.deepcopy(net).to(DEV), loss_reduction="mean")
    opt = A.optimizers.AdaClipDPOptimizer(
        torch.optim.SGD(gsm.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=C, expected_batch_size=16,
        target_unclipped_quantile=0.7, clipbound_learning_rate=0.2, max_clipbound=100.0, min_clipbound=0.01,
        unclipped_num_std=1e-4,
    )
    opt.zero_grad()
    F.cross_entropy(gsm(x.to(DEV)), y.to(DEV)).backward()
    opt.pre_step()
    assert opt.sample_size == 16 and abs(opt.unclipped_num - count) < 1e-2
    assert abs(opt.max_grad_norm - new_bound) < 1e-3 * new_bound
    close(gsm._module.weight.grad, summed[0] / 16, 2e-4, 1e-7)
    # with noise the gradient noise uses the adjusted multiplier of Theorem 1
    opt2 = A.optimizers.AdaClipDPOptimizer(
        torch.optim.SGD(gsm.parameters(), lr=0.1), noise_multiplier=1.0, max_grad_norm=2.0, expected_batch_size=16,
        target_unclipped_quantile=0.5, clipbound_learning_rate=0.2, max_clipbound=100.0, min_clipbound=0.01,
        unclipped_num_std=2.0,
    )
    assert abs(opt2._noise_std() - 2.0 * (1 - 1 / 16) ** -0.5) < 1e-9


def test_noise_level(A):
    """privacy_engine_test.py:676-739: with zero gradients, after k steps sum p^2 ~ k P (sigma C lr / B)^2."""
    torch.manual_seed(8)
    net = nn.Linear(300, 200)
    P = sum(p.numel() for p in net.parameters())
    for p in net.parameters():
        p.data.zero_()
    sigma, C, lr, B, k = 1.5, 0.8, 0.5, 4, 3
    gsm = A.GradSampleModule(net.to(DEV), loss_reduction="mean")
    opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=lr), noise_multiplier=sigma, max_grad_norm=C, expected_batch_size=B)
    for _ in range(k):
        opt.zero_grad()
        (gsm(torch.zeros(B, 300, device=DEV)).sum() * 0.0).backward()
        opt.step()
    energy = sum(p.double().pow(2).sum().item() for p in net.parameters())
    expected = k * P * (sigma * C * lr / B) ** 2
    assert abs(energy / expected - 1) < 0.05


def test_noise_determinism_rules(A):
    """randomness_test.py:199-255: same global seed or same generator seed => same weights; else different."""
    torch.manual_seed(9)
    net = nn.Linear(20, 5)
    batches = [(torch.randn(4, 20), torch.randint(0, 5, (4,))) for _ in range(2)]
    a = _train(A, net, batches, private=True, sigma=1.0, C=1.0, seed=123)
    b = _train(A, net, batches, private=True, sigma=1.0, C=1.0, seed=123)
    c = _train(A, net, batches, private=True, sigma=1.0, C=1.0, seed=124)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    assert not torch.equal(a[0], c[0])
    for gdev in ("cuda", "cpu"):
        g1 = torch.Generator(device=gdev).manual_seed(7)
        g2 = torch.Generator(device=gdev).manual_seed(7)
        g3 = torch.Generator(device=gdev).manual_seed(8)
        d = _train(A, net, batches, private=True, sigma=1.0, C=1.0, generator=g1)
        e = _train(A, net, batches, private=True, sigma=1.0, C=1.0, generator=g2)
        f = _train(A, net, batches, private=True, sigma=1.0, C=1.0, generator=g3)
        assert all(torch.equal(x, y) for x, y in zip(d, e)), gdev
        assert not torch.equal(d[0], f[0]), gdev
    s = _train(A, net, batches, private=True, sigma=1.0, C=1.0, seed=123, secure=True)
    assert not torch.equal(a[0], s[0])
    # noise per parameter is independent of the other parameters' noise
    torch.manual_seed(1)
    n1 = A.optimizers.optimizer._generate_noise(1.0, torch.zeros(100000, device=DEV))
    n2 = A.optimizers.optimizer._generate_noise(1.0, torch.zeros(100000, device=DEV))
    assert abs(torch.corrcoef(torch.stack([n1, n2]))[0, 1].item()) < 0.02
    assert A.optimizers.optimizer._generate_noise(0.0, torch.ones(5, device=DEV)).abs().sum() == 0


def test_zero_std_leaves_the_generator_alone(A):
    net = nn.Linear(4, 2).to(DEV)
    gsm = A.GradSampleModule(net, loss_reduction="mean")
    gen = torch.Generator(device="cuda").manual_seed(11)
    opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=1.0, expected_batch_size=2, generator=gen)
    before = gen.get_offset()
    gsm(torch.randn(2, 4, device=DEV)).sum().backward()
    opt.step()
    assert gen.get_offset() == before


# ---- ghost clipping ----------------------------------------------------------------------------
class PerSampleMSE(nn.Module):
    def __init__(self, reduction="mean"):
        super().__init__()
        self.reduction = reduction

    def forward(self, out, tgt):
        l = (out - tgt).pow(2).flatten(1).mean(1)
        if self.reduction == "none":
            return l
        return l.mean() if self.reduction == "mean" else l.sum()


@pytest.mark.parametrize("loss_reduction", ["mean", "sum"])
def test_ghost_norms_and_step_match_hooks_mode(A, loss_reduction):
    """grad_sample_module_fast_gradient_clipping_test.py:129-280: per-parameter norms and the
    weights after one step agree between ghost clipping and materialised clipping."""
    torch.manual_seed(10)
    mlp = nn.Sequential(nn.Linear(24, 40), nn.GELU(), nn.Linear(40, 12))  # config 3, down-scaled
    n, T, C = 6, 33, 0.05
    x, y = torch.randn(n, T, 24), torch.randn(n, T, 12)
    crit = PerSampleMSE(loss_reduction)

    hooks = A.GradSampleModule(copy.deepcopy(mlp).to(DEV), loss_reduction=loss_reduction)
    hopt = A.DPOptimizer(torch.optim.SGD(hooks.parameters(), lr=0.5), noise_multiplier=0.0, max_grad_norm=C, expected_batch_size=n, loss_reduction=loss_reduction)
    crit(hooks(x.to(DEV)), y.to(DEV)).backward()
    want_norms = [p.grad_sample.double().flatten(1).norm(dim=1).cpu() for p in hooks.parameters()]
    hopt.step()

    ghost = A.GradSampleModuleFastGradientClipping(copy.deepcopy(mlp).to(DEV), loss_reduction=loss_reduction, max_grad_norm=C)
    gopt = A.DPOptimizerFastGradientClipping(torch.optim.SGD(ghost.parameters(), lr=0.5), noise_multiplier=0.0, max_grad_norm=C, expected_batch_size=n, loss_reduction=loss_reduction)
    dpl = A.DPLossFastGradientClipping(ghost, gopt, PerSampleMSE(loss_reduction), loss_reduction)
    gopt.zero_grad()
    dpl(ghost(x.to(DEV)), y.to(DEV)).backward()
    for p, w in zip(ghost.parameters(), want_norms):
        assert p.grad_sample is None
        close(p._norm_sample, w, 1e-4, 1e-7)
    total = torch.stack(want_norms).norm(dim=0)
    close(ghost.per_sample_gradient_norms, total, 1e-4, 1e-7)
    assert (total > C).all()  # the test clips every sample
    gopt.step()
    for pg, ph in zip(ghost.parameters(), hooks.parameters()):
        close(pg, ph, 1e-4, 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ghost_tiny_llama_norms(A, dtype):
    """Config 5, down-scaled: Embedding (ghost, id dedupe), RMSNorm (gradient formed and reduced
    at once), Linear (Gram contraction), sequence-level loss via shape=."""
    torch.manual_seed(11)
    net = TinyLlama()
    n, T, V = 4, 16, 50
    ids = torch.randint(0, V, (n, T))
    ids[0, :8] = 3  # repeated ids inside a sample
    tgt = torch.randint(0, V, (n, T))

    def seq_loss(logits, t):
        return F.cross_entropy(logits.flatten(0, 1).float(), t.flatten(), reduction="none").view(1, -1).mean(1).sum()

    want = per_sample_grads_cpu(net, ids, tgt, seq_loss)
    want_norm = torch.sqrt(sum(v.double().flatten(1).pow(2).sum(1) for v in want.values()))

    gnet = copy.deepcopy(net).to(DEV).to(dtype)
    ghost = A.GradSampleModuleFastGradientClipping(gnet, loss_reduction="mean", max_grad_norm=1.0)
    gopt = A.DPOptimizerFastGradientClipping(torch.optim.SGD(ghost.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=1.0, expected_batch_size=n)
    dpl = A.DPLossFastGradientClipping(ghost, gopt, nn.CrossEntropyLoss(), "mean")
    logits = ghost(ids.to(DEV))
    loss = dpl(logits.flatten(0, 1).float(), tgt.flatten().to(DEV), shape=(n, T, V))
    loss.backward()
    rtol = 1e-3 if dtype == torch.float32 else 5e-2
    close(ghost.per_sample_gradient_norms, want_norm, rtol, 1e-6)
    if dtype == torch.float32:
        coef = (1.0 / (want_norm + 1e-6)).clamp(max=1.0).float()
        gopt.step()  # lr 0.1, mean over n
        for (k, p0), p1 in zip(net.named_parameters(), gnet.parameters()):
            g = (coef.view(-1, *[1] * (want[k].dim() - 1)) * want[k]).sum(0) / n
            close(p1, p0 - 0.1 * g, 1e-3, 1e-5, k)


def test_ghost_tied_embedding_and_lm_head(A):
    """Config 5 as written (tied embeddings), down-scaled. The reference raises for tied
    parameters under ghost clipping; here an Embedding table shared with the LM head takes the
    two ghost norms plus the cross term. Checked against batch-of-one autograd, whose gradient
    of the shared table is the sum of both uses, and against the materialising hooks path."""
    torch.manual_seed(14)
    net = TinyLlama()
    net.lm_head.weight = net.emb.weight
    assert len(list(net.parameters())) == len(list(TinyLlama().parameters())) - 1
    n, T, V = 4, 16, 50
    ids = torch.randint(0, V, (n, T))
    ids[0, :8] = 3
    tgt = torch.randint(0, V, (n, T))

    def seq_loss(logits, t):
        return F.cross_entropy(logits.flatten(0, 1).float(), t.flatten(), reduction="none").view(1, -1).mean(1).sum()

    want = per_sample_grads_cpu(net, ids, tgt, seq_loss)
    want_norm = torch.sqrt(sum(v.double().flatten(1).pow(2).sum(1) for v in want.values()))

    gnet = copy.deepcopy(net).to(DEV)
    assert gnet.lm_head.weight is gnet.emb.weight
    ghost = A.GradSampleModuleFastGradientClipping(gnet, loss_reduction="mean", max_grad_norm=1.0)
    gopt = A.DPOptimizerFastGradientClipping(torch.optim.SGD(ghost.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=1.0, expected_batch_size=n)
    dpl = A.DPLossFastGradientClipping(ghost, gopt, nn.CrossEntropyLoss(), "mean")
    for _ in range(2):  # the second pass must find no leftovers of the first
        gopt.zero_grad()
        logits = ghost(ids.to(DEV))
        dpl(logits.flatten(0, 1).float(), tgt.flatten().to(DEV), shape=(n, T, V)).backward()
        close(gnet.emb.weight._norm_sample, want["emb.weight"].flatten(1).norm(dim=1), 1e-3, 1e-7, "shared table")
        close(ghost.per_sample_gradient_norms, want_norm, 1e-3, 1e-6)
    coef = (1.0 / (want_norm + 1e-6)).clamp(max=1.0).float()
    gopt.step()
    for (k, p0), p1 in zip(net.named_parameters(), gnet.parameters()):
        g = (coef.view(-1, *[1] * (want[k].dim() - 1)) * want[k]).sum(0) / n
        close(p1, p0 - 0.1 * g, 1e-3, 1e-5, k)

    # the same weight used by two Linear layers is still refused
    class TwoHeads(nn.Module):
        def __init__(self):
            super().__init__()
            self.a, self.b = nn.Linear(6, 6, bias=False), nn.Linear(6, 6, bias=False)
            self.b.weight = self.a.weight

        def forward(self, x):
            return self.b(self.a(x))

    with pytest.raises(NotImplementedError, match="tying"):
        A.GradSampleModuleFastGradientClipping(TwoHeads().to(DEV))(torch.randn(2, 6, device=DEV))


def test_ghost_bf16_mlp(A):
    """Config 3, down-scaled, bf16 parameters with fp32 accumulation inside the kernels."""
    torch.manual_seed(12)
    mlp = nn.Sequential(nn.Linear(64, 128), nn.GELU(), nn.Linear(128, 64))
    n, T = 4, 70
    x, y = torch.randn(n, T, 64), torch.randn(n, T, 64)
    ghost = A.GradSampleModuleFastGradientClipping(copy.deepcopy(mlp).to(DEV).bfloat16(), loss_reduction="mean", max_grad_norm=1.0)
    gopt = A.DPOptimizerFastGradientClipping(torch.optim.SGD(ghost.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=1.0, expected_batch_size=n)
    dpl = A.DPLossFastGradientClipping(ghost, gopt, PerSampleMSE("mean"), "mean")
    dpl(ghost(x.to(DEV).bfloat16()), y.to(DEV).bfloat16()).backward()
    # oracle: the same bf16 model evaluated sample by sample with autograd (bf16 forward)
    ref = copy.deepcopy(mlp).bfloat16()
    norms = []
    for i in range(n):
        ref.zero_grad()
        PerSampleMSE("sum")(ref(x[i : i + 1].bfloat16()), y[i : i + 1].bfloat16()).backward()
        norms.append(torch.sqrt(sum(p.grad.double().pow(2).sum() for p in ref.parameters())))
    close(ghost.per_sample_gradient_norms, torch.stack(norms), 2e-2, 1e-6)
    for p in ghost.parameters():
        assert p._norm_sample.dtype == torch.float32 and p.grad.dtype == torch.bfloat16
    gopt.step()


def _ghost_grads(A, net, batch, loss_call, *, single, steps=2, C=0.05, reduction="mean"):
    """p.grad after `steps` forward / DP-backward rounds (the last one's), plus the module."""
    ghost = A.GradSampleModuleFastGradientClipping(
        copy.deepcopy(net).to(DEV), loss_reduction=reduction, max_grad_norm=C, single_backward=single
    )
    n = batch[0].shape[0]
    opt = A.DPOptimizerFastGradientClipping(
        torch.optim.SGD(ghost.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=C, expected_batch_size=n, loss_reduction=reduction
    )
    for _ in range(steps):  # a second round must find no leftovers of the first
        opt.zero_grad()
        loss_call(ghost, opt, [t.to(DEV) for t in batch]).backward()
    return [p.grad.detach().clone() for p in ghost.parameters()], ghost


@pytest.mark.parametrize("case", ["mlp_mean", "mlp_sum", "llama", "llama_tied", "cnn", "lstm", "norm_twice"])
def test_ghost_single_backward_leaves_the_second_pass_gradients(A, case):
    """single_backward=True forms the clipped gradient sum from what the hooks kept of the first
    backward pass. It must equal what the reference's second pass of sum_n coef[n] loss[n]
    (fast_gradient_clipping_utils.py:193-201) leaves in p.grad: Linear with and without a
    sequence dimension and bias, Embedding with repeated ids, RMSNorm / GroupNorm / Conv2d
    through their grad samplers, a table tied to the LM head, a layer whose uses are
    stacked (the recurrent projection of an LSTM), and a LayerNorm applied twice in one pass
    (its two per-sample gradients are kept apart and both counted once)."""
    torch.manual_seed(21)
    reduction = "sum" if case == "mlp_sum" else "mean"
    if case.startswith("mlp"):
        net = nn.Sequential(nn.Linear(24, 40), nn.GELU(), nn.Linear(40, 12))
        batch = (torch.randn(6, 33, 24), torch.randn(6, 33, 12))

        def loss_call(model, opt, b):
            return A.DPLossFastGradientClipping(model, opt, PerSampleMSE(reduction), reduction)(model(b[0]), b[1])

    elif case.startswith("llama"):
        net = TinyLlama()
        if case == "llama_tied":
            net.lm_head.weight = net.emb.weight
        n, T, V = 4, 16, 50
        ids = torch.randint(0, V, (n, T))
        ids[0, :8] = 3
        batch = (ids, torch.randint(0, V, (n, T)))

        def loss_call(model, opt, b):
            crit = A.DPLossFastGradientClipping(model, opt, nn.CrossEntropyLoss(), "mean")
            return crit(model(b[0]).flatten(0, 1).float(), b[1].flatten(), shape=(n, T, V))

    elif case == "cnn":
        net = nn.Sequential(
            nn.Conv2d(3, 8, 3, padding=1), nn.GroupNorm(2, 8), nn.ReLU(), nn.Conv2d(8, 8, 3, stride=2), nn.ReLU(),
            nn.Flatten(), nn.Linear(8 * 3 * 3, 5),
        )
        batch = (torch.randn(7, 3, 8, 8), torch.randint(0, 5, (7,)))

        def loss_call(model, opt, b):
            return A.DPLossFastGradientClipping(model, opt, nn.CrossEntropyLoss(), "mean")(model(b[0]), b[1])

    elif case == "norm_twice":

        class TwoUses(nn.Module):
            def __init__(self):
                super().__init__()
                self.ln = nn.LayerNorm(12)
                self.fc = nn.Linear(12, 12)

            def forward(self, x):
                return self.ln(self.fc(self.ln(x)))

        net = TwoUses()
        batch = (torch.randn(6, 5, 12), torch.randn(6, 5, 12))

        def loss_call(model, opt, b):
            return A.DPLossFastGradientClipping(model, opt, PerSampleMSE("mean"), "mean")(model(b[0]), b[1])

    else:
        from opacus_amd.layers import DPLSTM

        class Tagger(nn.Module):
            def __init__(self):
                super().__init__()
                self.rnn = DPLSTM(6, 10, num_layers=1, batch_first=True, bidirectional=True)
                self.out = nn.Linear(20, 4)

            def forward(self, x):
                return self.out(self.rnn(x)[0])

        net = Tagger()
        batch = (torch.randn(5, 9, 6), torch.randn(5, 9, 4))

        def loss_call(model, opt, b):
            return A.DPLossFastGradientClipping(model, opt, PerSampleMSE("mean"), "mean")(model(b[0]), b[1])

    two, _ = _ghost_grads(A, net, batch, loss_call, single=False, reduction=reduction)
    one, ghost = _ghost_grads(A, net, batch, loss_call, single=True, reduction=reduction)
    assert ghost._kept_passes == []
    assert (ghost.per_sample_gradient_norms > 0.05).any()  # some sample is clipped
    for (name, _), g1, g2 in zip(ghost.named_parameters(), one, two):
        scale = g2.abs().max().item() + 1e-12
        close(g1 / scale, g2 / scale, 1e-4, 2e-6, f"{case} {name}")


@pytest.mark.parametrize("extra", ["regulariser", "functional_use"])
def test_ghost_loss_terms_outside_the_hooked_layers_keep_their_gradient(A, extra):
    """A loss with a term that reaches trainable parameters other than through a hooked layer
    (criterion + regulariser, the ``loss + tensor`` arithmetic of DPTensorFastGradientClipping;
    a functional use of a layer's weight): the reference's second pass differentiates it with the
    rest of sum_n coef[n] loss[n] (fast_gradient_clipping_utils.py:193-201). The default
    (single_backward=True) must leave the same p.grad as single_backward=False: its guard sends
    such a step through both passes. Checked against fp64 autograd of the weighted loss."""
    torch.manual_seed(5)
    net = nn.Sequential(nn.Linear(12, 20), nn.GELU(), nn.Linear(20, 6))
    x, y = torch.randn(6, 9, 12), torch.randn(6, 9, 6)
    C = 0.05

    def extra_term(model, xb):
        if extra == "regulariser":
            return 0.3 * sum(p.pow(2).sum() for p in model.parameters())
        inner = model._module if hasattr(model, "_module") else model
        return 0.2 * F.linear(xb, inner[0].weight).pow(2).flatten(1).mean(1)  # per sample

    def loss_call(model, opt, b):
        dp_loss = A.DPLossFastGradientClipping(model, opt, PerSampleMSE("mean"), "mean")(model(b[0]), b[1])
        return dp_loss + extra_term(model, b[0])

    import warnings as _w

    with _w.catch_warnings():
        _w.simplefilter("ignore")
        two, _ = _ghost_grads(A, net, (x, y), loss_call, single=False, C=C)
        one, ghost = _ghost_grads(A, net, (x, y), loss_call, single=True, C=C)
    assert ghost.single_backward is True and ghost._kept_passes == []
    # fp64: coefficients from the per-sample norms of the criterion alone (what the hooks see),
    # then the gradient of sum_n coef[n] * (loss[n] + extra)
    ref = copy.deepcopy(net).double()
    gs = per_sample_grads_cpu(ref, x.double(), y.double(), lambda out, t: PerSampleMSE("sum")(out, t))
    norms = torch.sqrt(sum(g.flatten(1).pow(2).sum(1) for g in gs.values()))
    coef = (C / (norms + 1e-6)).clamp(max=1.0)
    ref.zero_grad()
    per_sample = PerSampleMSE("none")(ref(x.double()), y.double()) + extra_term(ref, x.double())
    (coef * per_sample).sum().backward()
    for (name, _), g1, g2, p in zip(ghost.named_parameters(), one, two, ref.parameters()):
        scale = p.grad.abs().max().item() + 1e-12
        close(g1 / scale, g2 / scale, 1e-4, 2e-6, f"{extra} {name}: default against two passes")
        close(g1.double() / scale, p.grad / scale, 1e-4, 1e-5, f"{extra} {name}: against fp64 autograd")
    # without the extra term the same model takes the single pass (nothing is kept afterwards, no warning)
    with _w.catch_warnings():
        _w.simplefilter("error")
        _ghost_grads(A, net, (x, y), lambda m, o, b: A.DPLossFastGradientClipping(m, o, PerSampleMSE("mean"), "mean")(m(b[0]), b[1]),
                     single=True, C=C)


@pytest.mark.parametrize("bias", [True, False])
def test_ghost_single_backward_bf16_weighted_contraction(A, bias):
    """A bf16 MLP on sequences whose Linear layers the weighted contraction takes (whole k tiles of
    32 positions, widths above 64): the single-pass clipped sum, with the coefficients applied
    inside the kernel, against the two-pass gradients of the same model (bf16 autograd, whose
    weighted backprops are rounded to bf16 on the way) and against fp64 on the CPU."""
    from opacus_amd import kernels

    torch.manual_seed(31)
    n, T = 8, 64
    net = nn.Sequential(nn.Linear(128, 256, bias=bias), nn.GELU(), nn.Linear(256, 128, bias=bias))
    x, y = torch.randn(n, T, 128), torch.randn(n, T, 128) * torch.logspace(-0.7, 0.7, n).view(n, 1, 1)  # norms a decade apart
    half = copy.deepcopy(net).bfloat16()
    assert kernels.linear_weighted_sum_takes(torch.empty(n, T, 256, device=DEV, dtype=torch.bfloat16), torch.empty(n, T, 128, device=DEV, dtype=torch.bfloat16))

    def loss_call(model, opt, b):
        return A.DPLossFastGradientClipping(model, opt, PerSampleMSE("mean"), "mean")(model(b[0]), b[1])

    batch = (x.bfloat16(), y.bfloat16())
    C = 0.2
    two, _ = _ghost_grads(A, half, batch, loss_call, single=False, steps=1, C=C)
    one, ghost = _ghost_grads(A, half, batch, loss_call, single=True, steps=1, C=C)
    norms = ghost.per_sample_gradient_norms.double().cpu()
    assert (norms > C).any() and (norms < C).any(), norms  # clipped and unclipped samples
    # fp64 on the CPU from the same bf16 weights and inputs; the coefficients as the GPU run found them
    ref = copy.deepcopy(half).double()
    want = per_sample_grads_cpu(ref, batch[0].double(), batch[1].double(), lambda out, t: PerSampleMSE("sum")(out, t))
    coef = (C / (norms + 1e-6)).clamp(max=1.0)
    for (name, _), g1, g2 in zip(ghost.named_parameters(), one, two):
        scale = g2.float().abs().max().item() + 1e-12
        close(g1.float() / scale, g2.float() / scale, 2e-2, 2e-2, f"{name} against two passes")
        w = want[name[len('_module.'):]]
        g = (coef.view(-1, *[1] * (w.dim() - 1)) * w).sum(0)  # before the optimizer divides by n
        close(g1.double().cpu() / scale, g / scale, 2e-2, 2e-2, f"{name} against fp64")


def test_ghost_tied_parameters_raise(A):
    class Tied(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = nn.Linear(6, 6)

        def forward(self, x):
            return self.fc(self.fc(x))

    ghost = A.GradSampleModuleFastGradientClipping(Tied().to(DEV))
    with pytest.raises(NotImplementedError, match="tying"):
        ghost(torch.randn(2, 6, device=DEV))


@pytest.mark.parametrize("single", [False, True])
def test_ghost_adaptive_clipping_engine_step_matches_oracle(A, monkeypatch, single):
    """adaptive_clipping_utils.py:77-121 end to end: the norms of backward #1 feed the bound
    update, and the clipped sum of backward #2 (or, with single_backward, the sum formed from
    backward #1) equals sum_n coeff[n] * g[n] with the oracle's coefficients of the new bound
    (sigma = 0, count noise pinned to zero)."""
    from opacus_amd.utils.adaptive_clipping import DPLossFastGradientAdaptiveClipping, PrivacyEngineAdaptiveClipping

    torch.manual_seed(21)
    mlp = nn.Sequential(nn.Linear(24, 40), nn.GELU(), nn.Linear(40, 12))
    n, T, C = 12, 9, 0.3
    x, y = torch.randn(n, T, 24), torch.randn(n, T, 12)
    x[: n // 2] *= 0.05  # small inputs, small gradients: some samples end up under the bound
    ds = TensorDataset(x, y)
    dl = DataLoader(ds, batch_size=n)

    # per-sample gradients and norms by the materialising path
    hooks = A.GradSampleModule(copy.deepcopy(mlp).to(DEV), loss_reduction="mean")
    PerSampleMSE("mean")(hooks(x.to(DEV)), y.to(DEV)).backward()
    gs = [p.grad_sample.double().cpu() for p in hooks.parameters()]
    norms = torch.stack([g.flatten(1).norm(dim=1) for g in gs]).norm(dim=0)
    want_bound, want_sigma, coeff = O.ghost_adaptive_update(norms, C, 0.6, 0.3, 1e-4, 10.0, 0.0)
    assert 0 < (norms <= C).sum() < n and want_bound != C

    monkeypatch.setattr(torch, "normal", lambda **kw: torch.zeros(kw["size"]))  # the count's noise
    net = copy.deepcopy(mlp).to(DEV)
    engine = PrivacyEngineAdaptiveClipping()
    model, opt, crit, _ = engine.make_private(
        module=net, optimizer=torch.optim.SGD(net.parameters(), lr=1.0), criterion=PerSampleMSE("mean"), data_loader=dl,
        noise_multiplier=0.0, max_grad_norm=C, poisson_sampling=False, grad_sample_mode="ghost",
        target_unclipped_quantile=0.6, min_clipbound=1e-4, max_clipbound=10.0, clipbound_learning_rate=0.3,
    )
    assert isinstance(crit, DPLossFastGradientAdaptiveClipping)
    model.single_backward = single
    before = [p.detach().double().cpu().clone() for p in net.parameters()]
    opt.zero_grad()
    crit(model(x.to(DEV)), y.to(DEV)).backward()
    close(model.per_sample_gradient_norms, norms, 1e-4, 1e-8)
    assert model.max_grad_norm == opt.max_grad_norm == pytest.approx(want_bound, rel=1e-5)
    assert opt._adjusted_noise_multiplier == 0.0
    opt.step()
    for p, b, g in zip(net.parameters(), before, gs):
        want = b - (coeff.double().view(-1, *[1] * (g.dim() - 1)) * g).sum(0) / n
        close(p, want, 1e-4, 1e-6)


# ---- make_private end to end ----------------------------------------------------------------------
@pytest.mark.parametrize("mode", ["hooks", "ghost"])
def test_make_private_trains(A, mode):
    torch.manual_seed(13)
    net = ResBlock().to(DEV)
    ds = TensorDataset(torch.randn(16, 16, 8, 8), torch.randint(0, 10, (16,)))
    dl = DataLoader(ds, batch_size=8)
    engine = A.PrivacyEngine()
    out = engine.make_private(
        module=net, optimizer=torch.optim.SGD(net.parameters(), lr=0.05), data_loader=dl, noise_multiplier=1.0,
        max_grad_norm=1.0, poisson_sampling=False, grad_sample_mode=mode,
    )
    model, opt = out[0], out[1]
    crit = out[2] if mode == "ghost" else nn.CrossEntropyLoss()
    before = [p.detach().clone() for p in net.parameters()]
    for x, y in dl:
        opt.zero_grad()
        crit(model(x.to(DEV)), y.to(DEV)).backward()
        opt.step()
    assert len(engine.accountant) == 2 and engine.accountant.history[0][:2] == (1.0, 0.5)
    assert all(not torch.equal(b, p) for b, p in zip(before, net.parameters()))
    assert all(torch.isfinite(p).all() for p in net.parameters())


@pytest.mark.parametrize("mode", ["hooks", "ghost"])
def test_make_private_with_poisson_batches_including_empty_ones(A, mode):
    """The default ``poisson_sampling=True``: batch sizes vary and some draws are empty
    (sample rate 1/8 over 12 items); every step must go through, empty ones adding pure noise."""
    torch.manual_seed(14)
    net = nn.Sequential(nn.Linear(6, 8), nn.ReLU(), nn.Linear(8, 3)).to(DEV)
    ds = TensorDataset(torch.randn(12, 6), torch.randint(0, 3, (12,)))
    dl = DataLoader(ds, batch_size=1, generator=torch.Generator().manual_seed(3))
    engine = A.PrivacyEngine()
    out = engine.make_private(
        module=net, optimizer=torch.optim.SGD(net.parameters(), lr=0.05), data_loader=DataLoader(ds, batch_size=2),
        noise_multiplier=0.5, max_grad_norm=1.0, grad_sample_mode=mode,
        noise_generator=torch.Generator(device=DEV).manual_seed(1),
    )
    model, opt, loader = out[0], out[1], out[-1]
    crit = out[2] if mode == "ghost" else nn.CrossEntropyLoss()
    loader.batch_sampler.generator = torch.Generator().manual_seed(5)
    sizes = []
    for _ in range(6):
        for x, y in loader:
            sizes.append(len(y))
            opt.zero_grad()
            crit(model(x.to(DEV)), y.to(DEV)).backward()
            opt.step()
    assert 0 in sizes and max(sizes) >= 3, sizes
    assert len(engine.accountant) == len(sizes) == 36
    assert all(torch.isfinite(p).all() for p in net.parameters())


def test_mixed_precision_dtypes(A):
    """mixed_precision_test.py:107-213 checks dtypes only: fp32 parameters under bf16 autocast keep
    fp32 grads; bf16 parameters give bf16 grads."""
    net = nn.Sequential(nn.Linear(16, 32), nn.ReLU(), nn.Linear(32, 4)).to(DEV)
    gsm = A.GradSampleModule(net, loss_reduction="mean")
    opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=0.1), noise_multiplier=1.0, max_grad_norm=1.0, expected_batch_size=4)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = gsm(torch.randn(4, 16, device=DEV))
        assert out.dtype == torch.bfloat16
        out.float().sum().backward()
    opt.step()
    for p in net.parameters():
        assert p.grad.dtype == torch.float32 and p.summed_grad.dtype == torch.float32
    low = nn.Linear(16, 4).to(DEV).bfloat16()
    gl = A.GradSampleModule(low, loss_reduction="mean")
    ol = A.DPOptimizer(torch.optim.SGD(gl.parameters(), lr=0.1), noise_multiplier=1.0, max_grad_norm=1.0, expected_batch_size=4)
    gl(torch.randn(4, 16, device=DEV).bfloat16()).sum().backward()
    ol.step()
    for p in low.parameters():
        assert p.grad.dtype == torch.bfloat16 and p.grad_sample.dtype == torch.bfloat16


class _HalfNet(nn.Module):
    """Embedding, Linear on sequences, LayerNorm, a convolution with GroupNorm: one layer of each
    kind of sampler."""

    def __init__(self):
        super().__init__()
        self.emb = nn.Embedding(20, 16)
        self.fc = nn.Linear(16, 24)
        self.ln = nn.LayerNorm(24)
        self.conv = nn.Conv1d(24, 8, 3, padding=1)
        self.gn = nn.GroupNorm(2, 8)
        self.head = nn.Linear(8, 5)

    def forward(self, ids):
        h = self.ln(F.relu(self.fc(self.emb(ids))))  # [n, T, 24]
        h = F.relu(self.gn(self.conv(h.transpose(1, 2))))  # [n, 8, T]
        return self.head(h.mean(2))


@pytest.mark.parametrize("mode", ["hooks", "ghost"])
def test_float16_low_precision(A, mode):
    """mixed_precision_test.py:164-213 with dtype=float16: a float16 model gives float16 gradients
    and per-sample gradients. Values: against batch-of-one autograd of the same float16 model
    taken in float64 (the samplers run on the float32 kernels from widened operands)."""
    torch.manual_seed(7)
    net = _HalfNet()
    n, T = 6, 12
    ids, y = torch.randint(0, 20, (n, T)), torch.randint(0, 5, (n,))
    half = copy.deepcopy(net).half()
    ref = copy.deepcopy(half).double()  # the float16 weights, exactly
    want = per_sample_grads_cpu(ref, ids, y, lambda out, t: F.cross_entropy(out, t, reduction="sum"))
    norms = torch.sqrt(sum(v.flatten(1).pow(2).sum(1) for v in want.values()))
    C = float(norms.median())
    coef = (C / (norms + 1e-6)).clamp(max=1.0)
    gnet = half.to(DEV)
    if mode == "hooks":
        gsm = A.GradSampleModule(gnet, loss_reduction="mean")
        opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=0.0), noise_multiplier=0.0, max_grad_norm=C, expected_batch_size=n)
        F.cross_entropy(gsm(ids.to(DEV)).float(), y.to(DEV)).backward()
        for k, p in gnet.named_parameters():
            assert p.grad_sample.dtype == torch.float16
            close(p.grad_sample.double().cpu(), want[k], 2e-2, 2e-3, k)  # float16 forward and backward
    else:
        gsm = A.GradSampleModuleFastGradientClipping(gnet, loss_reduction="mean", max_grad_norm=C)
        opt = A.DPOptimizerFastGradientClipping(torch.optim.SGD(gsm.parameters(), lr=0.0), noise_multiplier=0.0, max_grad_norm=C, expected_batch_size=n)
        dpl = A.DPLossFastGradientClipping(gsm, opt, nn.CrossEntropyLoss(), "mean")
        dpl(gsm(ids.to(DEV)).float(), y.to(DEV)).backward()
        close(gsm.per_sample_gradient_norms.double().cpu(), norms, 1e-2, 1e-4)
    opt.step()
    for k, p in gnet.named_parameters():
        assert p.grad.dtype == torch.float16, k
        g = (coef.view(-1, *[1] * (want[k].dim() - 1)) * want[k]).sum(0) / n
        close(p.grad.double().cpu(), g, 2e-2, 1e-3, k)


def test_float16_autocast_and_noise(A):
    """mixed_precision_test.py:107-162 with dtype=float16: float32 parameters under float16
    autocast keep float32 gradients; a float16 model takes a noisy step."""
    torch.manual_seed(8)
    net = nn.Sequential(nn.Linear(16, 32), nn.ReLU(), nn.Linear(32, 4)).to(DEV)
    gsm = A.GradSampleModule(net, loss_reduction="mean")
    opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=0.1), noise_multiplier=1.0, max_grad_norm=1.0, expected_batch_size=4)
    with torch.autocast("cuda", dtype=torch.float16):
        out = gsm(torch.randn(4, 16, device=DEV))
        assert out.dtype == torch.float16
        out.float().sum().backward()
    for p in net.parameters():
        assert p.grad_sample.dtype in (torch.float16, torch.float32)
    opt.step()
    for p in net.parameters():
        assert p.grad.dtype == torch.float32 and p.summed_grad.dtype == torch.float32
    low = nn.Linear(16, 4).to(DEV).half()
    gl = A.GradSampleModule(low, loss_reduction="mean")
    ol = A.DPOptimizer(torch.optim.SGD(gl.parameters(), lr=0.1), noise_multiplier=1.0, max_grad_norm=1.0, expected_batch_size=4)
    gl(torch.randn(4, 16, device=DEV).half()).sum().backward()
    ol.step()
    for p in low.parameters():
        assert p.grad.dtype == torch.float16 and p.grad_sample.dtype == torch.float16 and torch.isfinite(p).all()


# ---- what backward() leaves behind, and activation checkpointing --------------------------------
def test_p_grad_after_backward_is_the_non_private_sum_by_default(A, weight_grad_mode):
    """grad_sample_module.py:291-365 adds hooks and leaves autograd alone: after ``backward()`` a
    caller finds the plain summed gradient in ``p.grad`` until ``DPOptimizer.step`` replaces it.
    That is the default here as well; ``autograd_weight_grads=False`` leaves ``None`` there."""
    torch.manual_seed(3)
    net = SmallCNN()
    x, y = torch.randn(6, 1, 28, 28), torch.randint(0, 10, (6,))
    plain = copy.deepcopy(net).to(DEV)
    F.cross_entropy(plain(x.to(DEV)), y.to(DEV)).backward()
    gsm = A.GradSampleModule(net.to(DEV))
    opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=1e9, expected_batch_size=6)
    F.cross_entropy(gsm(x.to(DEV)), y.to(DEV)).backward()
    for (k, p), q in zip(gsm._module.named_parameters(), plain.parameters()):
        assert p.grad_sample is not None and p.grad_sample.shape[0] == 6
        if weight_grad_mode:
            close(p.grad, q.grad, 1e-4, 1e-6, k)
        else:
            assert p.grad is None, k
    opt.step()  # either way the step writes the (here unclipped) mean of the per-sample gradients
    for (k, p), q in zip(gsm._module.named_parameters(), plain.parameters()):
        close(p.grad, q.grad, 1e-4, 1e-6, k)


def test_hooked_layers_under_activation_checkpointing(A):
    """A block run through ``torch.utils.checkpoint`` (the re-entrant form, whose first forward runs
    without grad so that the hooks see the block once, in the recomputation): per-sample gradients
    and the step's gradient equal those of the same model without checkpointing."""
    from torch.utils.checkpoint import checkpoint

    class Net(nn.Module):
        def __init__(self, ckpt):
            super().__init__()
            self.inp = nn.Linear(12, 16)
            self.block = nn.Sequential(nn.Linear(16, 32), nn.GELU(), nn.LayerNorm(32), nn.Linear(32, 16))
            self.out = nn.Linear(16, 5)
            self.ckpt = ckpt

        def forward(self, x):
            h = torch.tanh(self.inp(x))
            h = checkpoint(self.block, h, use_reentrant=True) if self.ckpt else self.block(h)
            return self.out(h)

    torch.manual_seed(11)
    base = Net(False)
    x, y = torch.randn(7, 9, 12), torch.randint(0, 5, (7,))
    results = []
    for ckpt in (False, True):
        net = copy.deepcopy(base)
        net.ckpt = ckpt
        gsm = A.GradSampleModule(net.to(DEV))
        opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=0.5, expected_batch_size=7)
        F.cross_entropy(gsm(x.to(DEV)).mean(1), y.to(DEV)).backward()
        gs = [p.grad_sample.detach().clone() for p in net.parameters()]
        opt.step()
        results.append((gs, [p.grad.detach().clone() for p in net.parameters()]))
        assert all(p.requires_grad for p in net.parameters())
    want = per_sample_grads_cpu(base, x, y, lambda out, t: F.cross_entropy(out.mean(1), t, reduction="sum"))
    for (k, w), g0, g1, s0, s1 in zip(want.items(), results[0][0], results[1][0], results[0][1], results[1][1]):
        close(g0, w, 1e-4, 1e-5, f"{k} without checkpointing")
        close(g1, w, 1e-4, 1e-5, f"{k} with checkpointing")
        close(s1, s0, 1e-4, 1e-6, f"{k} step gradient")


# ---- convolutions under ghost clipping: norms without stored per-sample gradients ---------------
@pytest.mark.parametrize("single", [False, True])
def test_ghost_cnn_norms_and_clipped_sum_against_batch_of_one_autograd(A, single):
    """The reference forms and drops every conv per-sample gradient under fast gradient clipping
    (grad_sample_module_fast_gradient_clipping.py:226-250). Here a convolution's norm comes from
    the conv kernel's norm-only mode (early layers: many positions) or from the Gram route on
    the unfolded input (late layers: few positions, many channels); a conv layer used twice in
    one pass falls back to materialising; Conv1d and asymmetric "same" padding included. Norms and
    the clipped mean gradient against CPU autograd on one sample at a time."""

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.c1 = nn.Conv2d(3, 8, 3, padding=1)  # 12 x 12 positions, 27 kernel elements: direct route
            self.c2 = nn.Conv2d(8, 32, 4, stride=3, padding="valid")  # 3 x 3 positions, 128 elements, 32 channels: Gram route
            self.c3 = nn.Conv2d(32, 32, 2, padding="same")  # asymmetric padding, 3 x 3 positions: Gram route
            self.twice = nn.Conv2d(32, 32, 1)  # used twice: materialised
            self.c1d = nn.Conv1d(32, 16, 3, padding=1)  # 9 positions
            self.fc = nn.Linear(16 * 9, 5)

        def forward(self, x):
            h = F.relu(self.c1(x))
            h = F.relu(self.c2(h))
            h = F.relu(self.c3(h))
            h = self.twice(F.relu(self.twice(h)))
            h = F.relu(self.c1d(h.flatten(2)))
            return self.fc(h.flatten(1))

    torch.manual_seed(31)
    net, n, C = Net(), 6, 0.3
    x, y = torch.randn(n, 3, 12, 12), torch.randint(0, 5, (n,))
    want = per_sample_grads_cpu(net, x, y, lambda out, t: F.cross_entropy(out, t, reduction="sum"))
    flat = torch.cat([g.flatten(1) for g in want.values()], dim=1)
    norms = flat.norm(dim=1)
    coef = (C / (norms + 1e-6)).clamp(max=1.0)
    assert (coef < 1).any() and (norms > 0).all()
    ghost = A.GradSampleModuleFastGradientClipping(copy.deepcopy(net).to(DEV), max_grad_norm=C, single_backward=single)
    opt = A.DPOptimizerFastGradientClipping(
        torch.optim.SGD(ghost.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=C, expected_batch_size=n
    )
    crit = A.DPLossFastGradientClipping(ghost, opt, nn.CrossEntropyLoss(), "mean")
    opt.zero_grad()
    crit(ghost(x.to(DEV)), y.to(DEV)).backward()
    close(ghost.per_sample_gradient_norms, norms, 1e-4, 1e-6, "per-sample norms")
    for (k, p), g in zip(ghost._module.named_parameters(), want.values()):
        assert not hasattr(p, "grad_sample") or p.grad_sample is None, k  # nothing materialised is kept
        close(p._norm_sample, g.flatten(1).norm(dim=1), 1e-4, 1e-6, f"norm of {k}")
    opt.pre_step()
    for (k, p), g in zip(ghost._module.named_parameters(), want.values()):
        close(p.grad, torch.einsum("n,n...->...", coef, g) / n, 1e-4, 1e-6, f"clipped mean gradient of {k}")
