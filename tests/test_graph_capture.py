"""The kernels are plain launches on the caller's stream: a forward + backward can be captured into a HIP graph and
replayed.  Every replay (with the program's own eager work and synchronisations in between) must reproduce the eager
result for the inputs then present in the captured buffers."""

import pytest
import torch

from cuequivariance_amd import cue

pytestmark = pytest.mark.gpu


def _capture(step, warmup=3):
    side = torch.cuda.Stream()  # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(warmup):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        results = step()
    return graph, results


def test_triangle_update_replays(device):
    from cuequivariance_amd import cuet

    g = torch.Generator(device=device).manual_seed(0)
    n, D = 64, 64
    dtype = torch.bfloat16

    def r(*shape, scale=1.0):
        return (torch.randn(*shape, device=device, generator=g) * scale).to(dtype)

    kw = dict(mask=(torch.rand(1, n, n, device=device, generator=g) < 0.9).to(dtype),
              p_in_weight=r(2 * D, D, scale=D ** -0.5), g_in_weight=r(2 * D, D, scale=D ** -0.5),
              p_out_weight=r(D, D, scale=D ** -0.5), g_out_weight=r(D, D, scale=D ** -0.5))
    x = r(1, n, n, D).requires_grad_(True)
    cot = r(1, n, n, D)

    def step():
        out = cuet.triangle_multiplicative_update(x, "outgoing", **kw)
        (gx,) = torch.autograd.grad(out, [x], cot)
        return out, gx

    graph, (out_g, gx_g) = _capture(step)
    for trial in range(3):
        with torch.no_grad():
            x.copy_(r(1, n, n, D))
            cot.copy_(r(1, n, n, D))
        graph.replay()
        torch.cuda.synchronize()
        got = (out_g.clone(), gx_g.clone())
        want = step()  # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), trial


def test_indexed_channelwise_replays(device):
    from cuequivariance_amd import cuet

    irreps1, irreps2 = cue.Irreps("O3", "32x0e+32x1o+32x2e"), cue.Irreps("O3", "0e+1o+2e")
    m = cuet.ChannelWiseTensorProduct(irreps1, irreps2, ["0e", "1o", "2e"], layout=cue.ir_mul, shared_weights=False,
                                      internal_weights=False, device=device, dtype=torch.float32)
    N, E = 50, 700
    g = torch.Generator(device=device).manual_seed(1)
    node = torch.randn(N, irreps1.dim, device=device, generator=g, requires_grad=True)
    sh = torch.randn(E, irreps2.dim, device=device, generator=g, requires_grad=True)
    w = torch.randn(E, m.weight_numel, device=device, generator=g, requires_grad=True)
    snd = torch.randint(0, N, (E,), device=device, generator=g, dtype=torch.int32)
    rcv = torch.sort(torch.randint(0, N, (E,), device=device, generator=g, dtype=torch.int32))[0]
    cot = torch.randn(N, m.irreps_out.dim, device=device, generator=g)

    def step():
        out = m(node, sh, w, indices_1=snd, indices_out=rcv, size_out=N)
        return (out,) + torch.autograd.grad(out, [node, sh, w], cot)

    graph, static = _capture(step)
    for trial in range(3):
        with torch.no_grad():
            node.copy_(torch.randn(N, irreps1.dim, device=device, generator=g))
            w.copy_(torch.randn(E, m.weight_numel, device=device, generator=g))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in static]
        want = step()
        torch.cuda.synchronize()
        for a, b in zip(got, want):  # the node gradient is a floating-point atomic sum: order may differ
            torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-5 * float(b.abs().max()))


@pytest.mark.parametrize("N,E", [(40, 500), (3000, 70_000)])
def test_indexed_channelwise_replays_with_new_graph_indices(device, N, E):
    """The grouping of edges by receiver is part of the captured graph: copying other senders / receivers (unsorted,
    so the sort really runs) into the static index buffers between replays must give what eager mode gives for them.
    Two sizes: the library sort behind the grouping picks different kernels for short and long inputs."""
    from cuequivariance_amd import cuet

    irreps1, irreps2 = cue.Irreps("O3", "32x0e+32x1o+32x2e"), cue.Irreps("O3", "0e+1o+2e")
    m = cuet.ChannelWiseTensorProduct(irreps1, irreps2, ["0e", "1o", "2e"], layout=cue.ir_mul, shared_weights=False,
                                      internal_weights=False, device=device, dtype=torch.float32)
    g = torch.Generator(device=device).manual_seed(2)
    node = torch.randn(N, irreps1.dim, device=device, generator=g, requires_grad=True)
    sh = torch.randn(E, irreps2.dim, device=device, generator=g, requires_grad=True)
    w = torch.randn(E, m.weight_numel, device=device, generator=g, requires_grad=True)
    snd = torch.randint(0, N, (E,), device=device, generator=g, dtype=torch.int32)
    rcv = torch.sort(torch.randint(0, N, (E,), device=device, generator=g, dtype=torch.int32))[0]
    cot = torch.randn(N, m.irreps_out.dim, device=device, generator=g)

    def step(s=snd, r=rcv):
        out = m(node, sh, w, indices_1=s, indices_out=r, size_out=N)
        return (out,) + torch.autograd.grad(out, [node, sh, w], cot)

    graph, static = _capture(step)
    for trial in range(3):
        new_snd = torch.randint(0, N, (E,), device=device, generator=g, dtype=torch.int32)
        new_rcv = torch.randint(0, N // (trial + 1), (E,), device=device, generator=g, dtype=torch.int32)  # unsorted, rows left empty
        with torch.no_grad():
            snd.copy_(new_snd)
            rcv.copy_(new_rcv)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in static]
        want = step(new_snd.clone(), new_rcv.clone())  # fresh tensors: eager mode builds (and checks) their grouping
        torch.cuda.synchronize()
        assert torch.equal(got[0], want[0]), trial  # the forward sums each receiver's edges in edge order: bit-exact
        for a, b in zip(got[1:], want[1:]):
            torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-5 * float(b.abs().max()))


def test_index_tensors_made_in_inference_mode(device):
    """Index tensors created under torch.inference_mode() carry no version counter; the grouping cache must not ask."""
    from cuequivariance_amd import cuet

    irreps1, irreps2 = cue.Irreps("O3", "32x0e+32x1o+32x2e"), cue.Irreps("O3", "0e+1o+2e")
    m = cuet.ChannelWiseTensorProduct(irreps1, irreps2, ["0e", "1o", "2e"], layout=cue.ir_mul, shared_weights=False,
                                      internal_weights=False, device=device, dtype=torch.float32)
    N, E = 30, 200
    g = torch.Generator(device=device).manual_seed(3)
    node = torch.randn(N, irreps1.dim, device=device, generator=g)
    sh = torch.randn(E, irreps2.dim, device=device, generator=g)
    w = torch.randn(E, m.weight_numel, device=device, generator=g)
    snd = torch.randint(0, N, (E,), device=device, generator=g, dtype=torch.int32)
    rcv = torch.randint(0, N, (E,), device=device, generator=g, dtype=torch.int32)
    want = m(node, sh, w, indices_1=snd, indices_out=rcv, size_out=N)
    with torch.inference_mode():
        got = m(node, sh, w, indices_1=snd.clone(), indices_out=rcv.clone(), size_out=N)
    assert torch.equal(got, want)
