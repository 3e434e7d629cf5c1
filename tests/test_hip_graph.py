"""A step captured in a HIP graph.

The step scalars (debiased betas, decay factor) are formed on the host from a CPU step counter,
as in the reference, so a captured launch carries the scalars of the step it was captured at:
the optimizers without step-dependent scalars - Lion and SGD - replay correctly, and that is
what is held here.  Every replay is checked against an eager optimizer fed the same gradients,
with eager work and a synchronisation between replays; short lists (kernel-argument table, no
device tables) and lists of more than 16 tensors (device tables, uploaded before the capture).
"""

import pytest
import torch

import golden_util as G
import optimi_amd

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n_tensors", [4, 20], ids=["kernel_argument_table", "device_tables"])
@pytest.mark.parametrize("name", ["lion", "sgd"])
def test_captured_step_replays_like_eager_steps(name, n_tensors, hip_device):
    cls, kw = {"lion": (optimi_amd.Lion, dict(lr=1e-4, weight_decay=0.1)),
               "sgd": (optimi_amd.SGD, dict(lr=1e-2, momentum=0.9, weight_decay=1e-2, decouple_wd=True))}[name]
    pattern = [(300, 70), (8200,), (5,), (4096, 64), (513,)]
    shapes = [pattern[i % len(pattern)] for i in range(n_tensors)]
    gen = torch.Generator().manual_seed(11)
    captured = [torch.nn.Parameter((torch.randn(s, generator=gen) * 0.02).bfloat16().to(hip_device)) for s in shapes]
    eager = [torch.nn.Parameter(p.detach().clone()) for p in captured]
    static_grads = [torch.zeros_like(p) for p in captured]
    opt_c, opt_e = cls(captured, **kw), cls(eager, **kw)

    def fresh():
        return [(torch.randn(s, generator=gen) * 1e-3).bfloat16().to(hip_device) for s in shapes]

    def feed(gs):
        for sg, g in zip(static_grads, gs):
            sg.copy_(g)
        for p, g in zip(eager, gs):
            p.grad = g.clone()

    for p, sg in zip(captured, static_grads):
        p.grad = sg
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # eager warm-up on a side stream: states, first-step set-up, device tables
        for _ in range(2):
            feed(fresh())
            side.wait_stream(torch.cuda.current_stream())
            opt_c.step()
            opt_e.step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        opt_c.step()
    for replay in range(4):
        feed(fresh())
        graph.replay()
        opt_e.step()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(captured, eager)):
            G.assert_bits_equal(a, b, f"{name} replay {replay} tensor {i}")
            G.assert_bits_equal(opt_c.state[a]["exp_avg"], opt_e.state[b]["exp_avg"], f"{name} replay {replay} exp_avg {i}")

    # and eager steps on the default stream afterwards: the capture left nothing of its own in the
    # optimizer's launch workspace (no event recorded inside the capture to wait for)
    for it in range(2):
        feed(fresh())
        opt_c.step()
        opt_e.step()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(captured, eager)):
            G.assert_bits_equal(a, b, f"{name} eager step {it} after the replays, tensor {i}")
    graph.replay()  # and the graph still replays after eager use
    for p, g in zip(eager, static_grads):
        p.grad = g.clone()
    opt_e.step()
    torch.cuda.synchronize()
    for i, (a, b) in enumerate(zip(captured, eager)):
        G.assert_bits_equal(a, b, f"{name} replay after eager steps, tensor {i}")
    del graph


def test_a_table_upload_under_capture_is_refused(hip_device):
    """A list of more than 16 tensors whose tables are not on the device yet cannot be stepped under
    capture: the upload would be baked into the graph, reading a staging slot that later uploads
    overwrite.  The call returns OPTIMI_ERR_CAPTURE and launches nothing; the same list, stepped once
    before the capture, is accepted."""
    from optimi_amd import cabi

    L = cabi.lib()
    n = 20
    ps = [torch.zeros(1000 + i, dtype=torch.bfloat16, device=hip_device) for i in range(n)]
    gs = [torch.full_like(p, 1e-3) for p in ps]
    ms = [torch.zeros_like(p) for p in ps]
    ks = [torch.zeros_like(p) for p in ps]
    cols = [cabi.ptr_array(t.data_ptr() for t in col) for col in (ps, gs, ms, ks)]
    numel = cabi.i64_array(p.numel() for p in ps)
    scratch = torch.zeros(8, device=hip_device)

    def call(group):
        return L.optimi_hip_lion_multi(group.handle, n, *cols, numel, cabi.BF16, 1e-4, 0.1, 0.01, 0.0,
                                       cabi.KAHAN | cabi.UPDATE, torch.cuda.current_stream().cuda_stream)

    cold, warm = cabi.Group(), cabi.Group()
    assert call(warm) == 0
    torch.cuda.synchronize()
    launches = L.optimi_hip_launch_count()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        scratch.add_(1)  # the graph is not empty whatever happens below
        rc_cold = call(cold)
        rc_warm = call(warm)
    assert rc_cold == -9 and b"capturing" in L.optimi_hip_error_string(-9)
    assert rc_warm == 0
    assert L.optimi_hip_launch_count() - launches == 1
    before = ps[0].clone()
    graph.replay()
    torch.cuda.synchronize()
    assert not torch.equal(ps[0], before)
    assert call(cold) == 0  # eagerly it is fine
    torch.cuda.synchronize()
    del graph
    cold.close()
    warm.close()
