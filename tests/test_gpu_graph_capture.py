"""The function-level calls are plain kernel launches on the caller's stream (no allocation, no memset, no host
wait), so a forward + backward can be captured into a HIP graph and replayed on new data.  Each case replays the
graph several times, with eager work and synchronisations in between, and checks every replay against the eager
result of the same inputs."""

import numpy as np
import pytest
import torch

from speech_amd.rnnt_loss import rnnt

from gpu_utils import DEV, make_lengths

pytestmark = pytest.mark.gpu


def eager_and_graph(kind, B, T, U, V, extra, seed):
    rng = np.random.RandomState(seed)
    D = len(extra.get("durations", []))
    acts = torch.zeros(B, T, U, V + D, device=DEV)
    labels = torch.tensor(rng.randint(0, V - 1 - len(extra.get("big", [])), size=(B, U - 1)), device=DEV)
    al, ll = make_lengths(rng, B, T, U, 2, 0)
    al, ll = torch.tensor(al, device=DEV), torch.tensor(ll, device=DEV)
    scale = torch.ones(B, device=DEV)
    ws = rnnt.new_workspace(acts, D if D else len(extra.get("big", [])))

    def run(costs, grads):
        if kind == "rnnt":
            rnnt.rnnt_forward(acts, labels, al, ll, costs, V - 1, 0.01, True, ws)
            rnnt.rnnt_backward(acts, labels, al, ll, grads, scale, V - 1, 0.01, 0.5, ws)
        elif kind == "tdt":
            rnnt.tdt_forward(acts, labels, al, ll, costs, V - 1, extra["durations"], 0.0, 0.05, False, True, ws)
            rnnt.tdt_backward(acts, labels, al, ll, grads, scale, V - 1, extra["durations"], 0.0, 0.0, 0.05, False, ws)
        else:
            rnnt.multiblank_forward(acts, labels, al, ll, costs, V - 1, extra["big"], 0.0, 0.05, True, ws)
            rnnt.multiblank_backward(acts, labels, al, ll, grads, scale, V - 1, extra["big"], 0.0, 0.0, 0.05, ws)

    costs_e, grads_e = torch.empty(B, device=DEV), torch.empty_like(acts)
    costs_g, grads_g = torch.empty(B, device=DEV), torch.empty_like(acts)
    acts.copy_(torch.tensor(rng.randn(*acts.shape), dtype=torch.float32))
    run(costs_e, grads_e)  # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(costs_g, grads_g)
    for replay in range(4):
        acts.copy_(torch.tensor(rng.randn(*acts.shape) * (1 + replay), dtype=torch.float32))
        scale.copy_(torch.tensor(rng.rand(B) + 0.5, dtype=torch.float32))
        costs_g.fill_(-1.0)
        grads_g.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        run(costs_e, grads_e)  # the program's own eager work between replays
        filler = (grads_e * 2).sum()
        torch.cuda.synchronize()
        assert torch.isfinite(filler)
        assert torch.equal(costs_g, costs_e), (kind, replay)
        assert torch.equal(grads_g, grads_e), (kind, replay)


def test_rnnt_forward_backward_in_a_graph():
    eager_and_graph("rnnt", 3, 19, 8, 300, {}, 0)


def test_rnnt_long_rows_in_a_graph():
    eager_and_graph("rnnt", 2, 9, 5, 5001, {}, 1)


def test_tdt_forward_backward_in_a_graph():
    eager_and_graph("tdt", 3, 17, 6, 65, {"durations": [0, 1, 2, 3, 4]}, 2)


def test_multiblank_forward_backward_in_a_graph():
    eager_and_graph("multiblank", 3, 17, 6, 40, {"big": [2, 4]}, 3)


def test_fused_joint_forward_and_backward_replay_from_a_graph():
    """The fused joint's step reads nothing back from the device (its row buffers are sized by a bound the host
    knows, the tiles in use are counted and consumed on the device), so the C-level forward, backward and reduction
    can be captured and replayed on new inputs -- with other lengths, i.e. another number of tiles in use."""
    import ctypes

    from speech_amd import _native
    from speech_amd.joint import fused

    lib = _native.lib()
    B, T, U, H, V = 4, 23, 9, 640, 130
    rng = np.random.RandomState(5)
    f = torch.zeros(B, T, H, dtype=torch.bfloat16, device=DEV)
    g = torch.zeros(B, U, H, dtype=torch.bfloat16, device=DEV)
    W = torch.tensor(rng.randn(V, H) / np.sqrt(H), dtype=torch.float32, device=DEV)
    bias = torch.tensor(rng.randn(V) * 0.3, dtype=torch.float32, device=DEV)
    labels = torch.tensor(rng.randint(0, V - 1, size=(B, U - 1)), device=DEV)
    al = torch.full((B,), T, dtype=torch.int64, device=DEV)
    ll = torch.full((B,), U - 1, dtype=torch.int64, device=DEV)
    ws = fused.joint_workspace(B, T, U, H, V, DEV)
    tiles = lib.mi_joint_tile_bound(B, T, U)
    NP = lib.mi_joint_padded_vocabulary(V)
    slices = 8
    logits = torch.empty(tiles * 128, NP, dtype=torch.float16, device=DEV)
    acts = torch.empty(tiles * 128, H + 16, dtype=torch.bfloat16, device=DEV)
    d_hidden = torch.empty(tiles * 128, H, dtype=torch.bfloat16, device=DEV)
    scale = torch.ones(B, device=DEV)

    def run(out):
        costs, dw, db, df, dg = out
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        args = (B, T, U, H, V, V - 1)
        st = lib.mi_joint_rnnt_forward(f.data_ptr(), g.data_ptr(), W.data_ptr(), bias.data_ptr(), _native.DTYPE_F32,
                                       labels.data_ptr(), al.data_ptr(), ll.data_ptr(), costs.data_ptr(), None, 0.0, 0, 0,
                                       *args, 0.01, 1, logits.data_ptr(), acts.data_ptr(), tiles, ws.data_ptr(),
                                       ws.numel(), stream)  # fmt: skip
        assert st == _native.SUCCESS
        st = lib.mi_joint_rnnt_backward(labels.data_ptr(), al.data_ptr(), ll.data_ptr(), logits.data_ptr(), acts.data_ptr(),
                                        d_hidden.data_ptr(), dw.data_ptr(), db.data_ptr(), slices, tiles, scale.data_ptr(),
                                        1, 1.0, *args, 0.01, 0.0, ws.data_ptr(), ws.numel(), stream)  # fmt: skip
        assert st == _native.SUCCESS
        st = lib.mi_joint_reduce_hidden(d_hidden.data_ptr(), f.data_ptr(), g.data_ptr(), al.data_ptr(), ll.data_ptr(),
                                        df.data_ptr(), dg.data_ptr(), None, 0, tiles, 0.0, 0, 0, B, T, U, H, V, 0, 0,
                                        ws.data_ptr(), ws.numel(), stream)  # fmt: skip
        assert st == _native.SUCCESS

    def outputs():
        return (torch.empty(B, device=DEV), torch.empty(slices, NP, H, device=DEV), torch.empty(slices, NP, device=DEV),
                torch.empty(B, T, H, device=DEV), torch.empty(B, U, H, device=DEV))

    eager, captured = outputs(), outputs()
    f.copy_(torch.tensor(rng.randn(B, T, H), dtype=torch.bfloat16))
    g.copy_(torch.tensor(rng.randn(B, U, H), dtype=torch.bfloat16))
    run(eager)  # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(captured)
    for replay in range(4):
        f.copy_(torch.tensor(rng.randn(B, T, H) * (1 + 0.5 * replay), dtype=torch.bfloat16))
        g.copy_(torch.tensor(rng.randn(B, U, H), dtype=torch.bfloat16))
        a, l = make_lengths(rng, B, T, U, 2, 0)
        al.copy_(torch.tensor(a))
        ll.copy_(torch.tensor(l))
        scale.copy_(torch.tensor(rng.rand(B) + 0.5, dtype=torch.float32))
        for x in captured:
            x.fill_(-3.0)
        graph.replay()
        torch.cuda.synchronize()
        run(eager)  # the program's own eager work between replays
        torch.cuda.synchronize()
        for name, x, y in zip(("costs", "dw", "db", "df", "dg"), captured, eager):
            assert torch.equal(x, y), (name, replay)
