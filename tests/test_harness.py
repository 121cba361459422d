"""The reference's example networks on this package's layers (s2cnn_amd/harness.py): parameter names and shapes as the
reference's scripts produce them (so state dicts interchange, examples/shrec17/train.py:123, test.py:49), a state-dict
round trip, and training steps on synthetic data."""
import io

import pytest
import torch

from s2cnn_amd import harness


def _bn(prefix, n):
    return {prefix + ".weight": (n,), prefix + ".bias": (n,), prefix + ".running_mean": (n,), prefix + ".running_var": (n,),
            prefix + ".num_batches_tracked": ()}


def test_state_dict_names_and_shapes_follow_the_reference_scripts():
    # examples/mnist/run.py:55-98: conv1 (S2, 1 -> 20, 24-point grid), conv2 (SO3, 20 -> 40, 192-point grid), out_layer
    want = {"conv1.kernel": (1, 20, 24), "conv1.bias": (1, 20, 1, 1, 1), "conv2.kernel": (20, 40, 192), "conv2.bias": (1, 40, 1, 1, 1),
            "out_layer.weight": (10, 40), "out_layer.bias": (10,)}
    got = {k: tuple(v.shape) for k, v in harness.S2ConvNet_original().state_dict().items()}
    assert got == want
    # examples/shrec17/model.py:7-48: nn.Sequential(S2Conv, BN, ReLU, SO3Conv, BN, ReLU), equatorial grids of 2 b_in points
    want = {"sequential.0.kernel": (6, 100, 128), "sequential.0.bias": (1, 100, 1, 1, 1), **_bn("sequential.1", 100),
            "sequential.3.kernel": (100, 100, 32), "sequential.3.bias": (1, 100, 1, 1, 1), **_bn("sequential.4", 100),
            "out_layer.weight": (55, 100), "out_layer.bias": (55,)}
    got = {k: tuple(v.shape) for k, v in harness.Shrec17Model(55).state_dict().items()}
    assert got == want
    # examples/shrec17/model_original.py:7-50: features 6, 50, 70, 350; bandwidths 128, 32, 22, 7; BatchNorm1d(affine=False) + Linear
    want = {"sequential.0.kernel": (6, 50, 256), "sequential.0.bias": (1, 50, 1, 1, 1), **_bn("sequential.1", 50),
            "sequential.3.kernel": (50, 70, 64), "sequential.3.bias": (1, 70, 1, 1, 1), **_bn("sequential.4", 70),
            "sequential.6.kernel": (70, 350, 44), "sequential.6.bias": (1, 350, 1, 1, 1), **_bn("sequential.7", 350),
            "out_layer.0.running_mean": (350,), "out_layer.0.running_var": (350,), "out_layer.0.num_batches_tracked": (),
            "out_layer.1.weight": (55, 350), "out_layer.1.bias": (55,)}
    got = {k: tuple(v.shape) for k, v in harness.Shrec17ModelOriginal(55).state_dict().items()}
    assert got == want


def test_state_dict_round_trip_on_the_host():
    torch.manual_seed(3)
    a = harness.Shrec17Model(55)
    buf = io.BytesIO()
    torch.save(a.state_dict(), buf)            # examples/shrec17/train.py:123
    buf.seek(0)
    torch.manual_seed(4)
    b = harness.Shrec17Model(55)
    assert not torch.equal(a.sequential[0].kernel, b.sequential[0].kernel)
    b.load_state_dict(torch.load(buf, weights_only=True))      # examples/shrec17/test.py:49
    for (ka, va), (kb, vb) in zip(a.state_dict().items(), b.state_dict().items()):
        assert ka == kb and torch.equal(va, vb), ka
    assert a.sequential[0].scaling == b.sequential[0].scaling  # the normalisation is not a parameter: it is rebuilt from the sizes


@pytest.mark.gpu
def test_digit_network_trains_and_reloads(hip):
    """examples/mnist/run.py:211-223 on a fixed synthetic batch: the loss falls, and a reloaded state dict reproduces the
    network's outputs bit for bit; the same network with the activations inside the layers gives the same losses."""
    model, losses, _ = harness.train_steps("mnist", batch=32, steps=12, warmup=0, lr=0.05)
    print("digit network losses:", ["%.4f" % l for l in losses], flush=True)
    assert all(l == l for l in losses) and losses[-1] < 0.98 * losses[0]     # random labels: it can only memorise, slowly
    x, _ = harness.synthetic_batch("mnist", 32, "cuda:0")
    model.eval()
    with torch.no_grad():
        want = model(x)
    buf = io.BytesIO()
    torch.save(model.state_dict(), buf)
    buf.seek(0)
    twin = harness.S2ConvNet_original().cuda()
    twin.load_state_dict(torch.load(buf, weights_only=True))
    twin.eval()
    with torch.no_grad():
        assert torch.equal(twin(x), want)
    torch.manual_seed(0)                       # the seed train_steps builds its own network under: same initial weights
    fused_net = harness.S2ConvNet_original(fused_activation=True)
    _, fused, _ = harness.train_steps("mnist", batch=32, steps=4, warmup=0, lr=0.05, model=fused_net)
    assert max(abs(a - b) for a, b in zip(fused, losses)) < 1e-4 * abs(losses[0])


@pytest.mark.gpu
@pytest.mark.parametrize("name,batch", [("shrec17", 4), ("shrec17_original", 2)])
def test_shape_networks_train_and_reload(hip, name, batch):
    """examples/shrec17/train.py:70-82 (nll_loss on log_softmax, SGD with momentum) on a fixed synthetic batch: finite, falling
    loss; BatchNorm3d between the layers; equatorial kernel grids with 2 b_in points on one ring; state-dict round trip."""
    model, losses, _ = harness.train_steps(name, batch=batch, steps=6, warmup=0, lr=0.02)
    print(name, "losses:", ["%.4f" % l for l in losses], flush=True)
    assert all(l == l and l < 1e3 for l in losses) and min(losses[1:]) < losses[0]
    x, _ = harness.synthetic_batch(name, batch, "cuda:0")
    model.eval()
    with torch.no_grad():
        want = model(x)
    buf = io.BytesIO()
    torch.save(model.state_dict(), buf)
    buf.seek(0)
    twin = harness.NETWORKS[name][0]().cuda()
    twin.load_state_dict(torch.load(buf, weights_only=True))
    twin.eval()
    with torch.no_grad():
        assert torch.equal(twin(x), want)


@pytest.mark.gpu
def test_digit_network_step_replayed_from_a_hip_graph(hip):
    """The training step of the digit network captured into one HIP graph: the replayed steps continue the eager
    warm-up steps with the losses an all-eager run of the same length gives."""
    _, eager, _ = harness.train_steps("mnist", batch=16, steps=5, warmup=3, lr=0.05)
    _, replayed, _ = harness.train_steps_replayed("mnist", batch=16, steps=5, warmup=3, lr=0.05)
    print("eager", ["%.5f" % l for l in eager[3:]], "replayed", ["%.5f" % l for l in replayed], flush=True)
    assert max(abs(a - b) for a, b in zip(eager[3:], replayed)) < 1e-5 * abs(eager[0])


@pytest.mark.gpu
def test_shape_network_step_replayed_from_a_hip_graph(hip):
    """The training step of the SHREC17 network with the normalisations inside the transforms, captured into one HIP
    graph (statistics, running averages and the step counter of the BatchNorm3d modules included): the replayed steps
    continue the eager ones with the same losses, and the buffers end where the all-eager run's do."""
    torch.manual_seed(0)
    eager_net = harness.Shrec17Model(55, fused_norm=True)
    torch.manual_seed(0)
    replay_net = harness.Shrec17Model(55, fused_norm=True)
    _, eager, _ = harness.train_steps("shrec17", batch=4, steps=4, warmup=3, lr=0.02, model=eager_net)
    _, replayed, _ = harness.train_steps_replayed("shrec17", batch=4, steps=4, warmup=3, lr=0.02, model=replay_net)
    print("eager", ["%.5f" % l for l in eager[3:]], "replayed", ["%.5f" % l for l in replayed], flush=True)
    assert max(abs(a - b) for a, b in zip(eager[3:], replayed)) < 1e-5 * abs(eager[0])
    for (name, a), (_, b) in zip(eager_net.named_buffers(), replay_net.named_buffers()):
        assert torch.allclose(a.float(), b.float(), rtol=1e-5, atol=1e-6), name
