"""A module's whole step (forward + backward, with the delayed-scaling update in front) captured into a HIP graph
and replayed.  The tables of the captured launches are copied to the device by a captured kernel, which reads its
source again at every replay: they live in page-locked memory that is handed out once and never recycled
(backend._CaptureArena, allocated by fp8gmm_host_alloc, which works while a stream is capturing)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kind", ["linear", "mlp"])
def test_captured_step_replays_like_eager_steps(dev, kind):
    """Four replays with new inputs, each followed by eager work of the program's own and a synchronisation, against
    an eager twin that takes the same steps: outputs, all gradients and the scaling state (scale, amax history of
    both directions) bit for bit, every time.  The graph holds the casts, the GEMMs (large and small tiles, tail
    sharing with its second launch), the table uploads and the scaling updates."""
    import fp8_gmm_amd as pkg
    from fp8_gmm_amd import backend

    sizes = [137, 0, 59, 403, 1, 700, 300, 448]
    e, h, f = len(sizes), 512, 768
    tokens = sum(sizes)
    out_features = h if kind == "mlp" else f
    g = torch.Generator(device=dev).manual_seed(31)
    make = (lambda: pkg.GroupedMlp(h, f, e, torch.bfloat16, device=dev)) if kind == "mlp" else \
        (lambda: pkg.GroupedLinear(h, f, e, torch.bfloat16, device=dev))
    captured_module, eager_module = make(), make()
    eager_module.load_state_dict(captured_module.state_dict())
    gs = torch.tensor(sizes, dtype=torch.int64)
    recipe = pkg.DelayedScaling(amax_history_len=4)
    xs = [torch.randn(tokens, h, generator=g, device=dev).to(torch.bfloat16) for _ in range(6)]
    dys = [(torch.randn(tokens, out_features, generator=g, device=dev) * 1e-2).to(torch.bfloat16) for _ in range(6)]
    backend.warm_up(dev)

    def step(module, x, dy):
        for p in module.parameters():
            p.grad = None
        x.grad = None
        with pkg.fp8_autocast(enabled=True, fp8_recipe=recipe):
            out = module(x, gs)
        out.backward(dy)
        return out

    static_x, static_dy = xs[0].clone().requires_grad_(), dys[0].clone()
    eager_x = xs[0].clone().requires_grad_()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(2):   # two steps before the capture: the scaling update is then part of every later step
            static_x.data.copy_(xs[i]), static_dy.copy_(dys[i])
            step(captured_module, static_x, static_dy)
    torch.cuda.current_stream().wait_stream(side)
    for i in range(2):
        eager_x.data.copy_(xs[i])
        step(eager_module, eager_x, dys[i])
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = step(captured_module, static_x, static_dy)
    torch.cuda.synchronize()

    for i in range(2, 6):
        static_x.data.copy_(xs[i]), static_dy.copy_(dys[i])
        graph.replay()
        eager_x.data.copy_(xs[i])
        eager_out = step(eager_module, eager_x, dys[i])
        torch.randn(1 << 20, device=dev).sum().item()   # eager work and a synchronisation between the replays
        torch.cuda.synchronize()
        pairs = [("out", static_out, eager_out), ("grad_input", static_x.grad, eager_x.grad)]
        pairs += [("grad of " + name, p.grad, q.grad) for (name, p), (_, q) in
                  zip(captured_module.named_parameters(), eager_module.named_parameters())]
        for name, a, b in pairs:
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), f"replay {i - 1}: {name}"
        for direction in ("scaling_fwd", "scaling_bwd"):
            a, b = captured_module.fp8_meta[direction], eager_module.fp8_meta[direction]
            assert torch.equal(a.scale, b.scale) and torch.equal(a.amax_history, b.amax_history), \
                f"replay {i - 1}: {direction}"


def test_host_memory_for_captured_tables(dev):
    """fp8gmm_host_alloc: page-locked memory that the device reads (through fp8gmm_upload), also when asked for while
    a stream is capturing."""
    import ctypes

    import numpy as np

    from fp8_gmm_amd import _lib

    L = _lib.load()
    _lib.init(dev.index)
    assert L.fp8gmm_host_alloc(0) is None
    graph = torch.cuda.CUDAGraph()
    out = torch.zeros(4096, dtype=torch.uint8, device=dev)
    with torch.cuda.graph(graph):
        address = L.fp8gmm_host_alloc(4096)
        assert address
        stream = torch.cuda.current_stream(dev).cuda_stream
        _lib.check(L.fp8gmm_upload(out.data_ptr(), address, 4096, stream))
    host = np.ctypeslib.as_array((ctypes.c_uint8 * 4096).from_address(address))
    for value in (7, 201):   # the captured copy reads what the memory holds at the time of the replay
        host[:] = value
        graph.replay()
        torch.cuda.synchronize()
        assert (out == value).all()
    del graph
    L.fp8gmm_host_free(address)
