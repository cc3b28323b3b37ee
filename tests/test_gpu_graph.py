"""The hot-path entry points only enqueue kernels (no allocation, no memset, no synchronisation), so a caller
may capture them into a HIP graph. A captured chain of layers is replayed several times, with eager work and
synchronisations of the same context between the replays, and every replay must equal the eager result bit for bit.
Run on the GPU box: pytest -m gpu."""
import numpy as np
import pytest

from helpers import bf16_tensor, bits_of, make_layer, to_ff_offsets

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("one_call", [False, True, "shared_inside", "shared8_inside"],
                         ids=["router_then_verify", "route_verify", "shared_expert_inside", "shared_expert_int8_inside"])
def test_router_verify_and_dense_chain_in_a_graph(oracle, one_call):
    """`route_verify`: the router, the select and gate/up share one launch whose blocks hand the logits and routes
    to each other through words stamped with an epoch that lives in device memory and is advanced by the call's
    last launch - a replayed graph (same kernel arguments every time) and eager calls in between must still never
    take a previous call's words for this call's."""
    import torch
    import fieldfare_moe as ff
    ff.lib()
    d, f, e, k, layers, t = 256, 128, 32, 8, 3, 16
    ctx = ff.Context(d, f, e, k, n_layers=layers, max_tokens=64)
    dense = ff.Context(d, 2 * f, 1, 1, n_layers=layers, max_tokens=64)
    rng = np.random.default_rng(5)
    for layer in range(layers):
        _, pool, router = make_layer(oracle, 40 + layer, d, f, e)
        ctx.upload_layer(layer, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
        ctx.upload_router_bf16(layer, router)
        if one_call == "shared8_inside":
            # the shared expert held 8-bit: the same calls serve it
            parts8 = tuple(oracle.quantize_int8(rng.uniform(-0.2, 0.2, (r, c)).astype(np.float32))
                           for r, c in ((2 * f, d), (2 * f, d), (d, 2 * f)))
            dense.upload_expert_parts(layer, 0, *parts8, int8=True)
            continue
        _, dpool, _ = make_layer(oracle, 70 + layer, d, 2 * f, 1)
        dense.upload_layer(layer, dpool.bytes, dpool.stride, to_ff_offsets(ff, dpool.offsets))
    x = bf16_tensor(torch, oracle.bf16_bits(rng.normal(0, 1, (t, d)).astype(np.float32)))
    ws = [bf16_tensor(torch, oracle.bf16_bits(rng.uniform(0.5, 1.5, d).astype(np.float32))) for _ in range(5)]
    hidden0 = bf16_tensor(torch, oracle.bf16_bits(rng.normal(0, 1, (t, d)).astype(np.float32)))
    hidden = hidden0.clone()
    idx = torch.empty((t, k), dtype=torch.int32, device="cuda")
    w = torch.empty((t, k), dtype=torch.bfloat16, device="cuda")
    outs = tuple(torch.empty((t, d), dtype=torch.bfloat16, device="cuda") for _ in range(3))
    h1 = torch.empty((t, d), dtype=torch.bfloat16, device="cuda")
    h2 = torch.empty((t, d), dtype=torch.bfloat16, device="cuda")

    def chain():
        # one decoder-layer MoE block per layer: setup -> (shared expert, router -> routed experts) -> tail
        for layer in range(layers):
            ctx.post_attn_setup(hidden, x, ws[0], ws[1], ws[2], out=outs)
            if one_call in ("shared_inside", "shared8_inside"):
                # the shared expert inside the routed experts' launches, both combined in the tail: the call's last launch
                # (the down projection) moves the epoch on
                i_, w_ = ctx.route_verify_shared(dense, layer, layer, outs[2], outs[1], outs[0])
                idx.copy_(i_)
                w.copy_(w_)
                ctx.layer_tail_routed_shared(dense, w, hidden, ws[3], ws[4], 0.9)
                continue
            dense.dense_ffn(layer, outs[0], out=h1)
            if one_call:
                _, i_, w_ = ctx.route_verify(layer, outs[2], outs[1], out=h2)
                idx.copy_(i_)
                w.copy_(w_)
            else:
                i_, w_ = ctx.router(layer, outs[2])
                idx.copy_(i_)
                w.copy_(w_)
                ctx.verify(layer, outs[1], idx, w, out=h2)
            ctx.layer_tail(h2, h1, hidden, ws[3], ws[4], 0.9)

    chain()
    torch.cuda.synchronize()
    eager = bits_of(hidden)
    assert np.isfinite(oracle.bf16_to_float(eager)).all()

    # warm the allocator on the capture stream, then capture
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        hidden.copy_(hidden0)
        chain()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    hidden.copy_(hidden0)
    with torch.cuda.graph(graph, stream=side):
        chain()
    for replay in range(4):
        hidden.copy_(hidden0)
        h2.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(bits_of(hidden), eager), f"replay {replay}"
        # eager work of the same contexts between replays
        ctx.verify(replay % layers, x, idx, w)
        if one_call:
            for _ in range(replay + 1):     # moves the epoch by a different amount before every replay
                ctx.route_verify(replay % layers, x, x)
        dense.dense_ffn(replay % layers, x)
        torch.cuda.synchronize()
    assert ctx.last_live_experts() > 0
    assert ctx.handover_giveups() == 0      # on a GPU of its own no wave of the one-launch form had to help itself
    ctx.close()
    dense.close()


def test_two_streams_on_one_context_run_one_after_the_other(oracle):
    """Calls on a context from two streams, no synchronisation between them on the caller's side: the later call's
    stream waits on the device for the earlier one's, so the context's scratch (plan, activation rows, hand-over
    words) is never used by two calls at once. Each result equals the same call made alone. The static-scratch entry
    point, whose array every context on the GPU shares, is held to the same."""
    import ctypes as C
    import torch
    import fieldfare_moe as ff
    L = ff.lib()
    d, f, e, k, t = 2816, 704, 128, 8, 16
    ctx = ff.Context(d, f, e, k, n_layers=1, max_tokens=16)
    _, pool, router = make_layer(oracle, 3, d, f, e)
    ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
    ctx.upload_router_bf16(0, router)
    g = torch.Generator(device="cuda")
    g.manual_seed(77)
    xs = [torch.randn((t, d), device="cuda", generator=g).to(torch.bfloat16) for _ in range(6)]
    alone = []
    for x in xs:
        y, idx, w = ctx.route_verify(0, x, x)
        alone.append((y.clone(), idx.clone(), w.clone()))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = []
    for i, x in enumerate(xs):
        with torch.cuda.stream(streams[i % 2]):
            outs.append(ctx.route_verify(0, x, x))
    torch.cuda.synchronize()
    for (y, idx, w), (y0, idx0, w0) in zip(outs, alone):
        assert torch.equal(idx, idx0) and torch.equal(w.view(torch.int16), w0.view(torch.int16))
        assert torch.equal(y.view(torch.int16), y0.view(torch.int16))
    assert ctx.handover_giveups() == 0
    # the static array, from a second context on the same GPU as well
    other = ff.Context(d, f, e, k, n_layers=1, max_tokens=16)
    other.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
    ys = [torch.empty((t, d), dtype=torch.bfloat16, device="cuda") for _ in xs]
    for i, x in enumerate(xs):
        with torch.cuda.stream(streams[i % 2]):
            err = C.c_char_p()
            stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
            rc = L.ffmoe_verify_static((ctx if i % 3 else other)._h, stream, 0, C.c_void_p(x.data_ptr()), d, t,
                                       C.c_void_p(alone[i][1].data_ptr()), C.c_void_p(alone[i][2].data_ptr()), None,
                                       C.c_void_p(ys[i].data_ptr()), C.byref(err))
            assert rc == 0, err.value
    torch.cuda.synchronize()
    for y, (y0, _, _) in zip(ys, alone):
        assert torch.equal(y.view(torch.int16), y0.view(torch.int16))
    ctx.close()
    other.close()
