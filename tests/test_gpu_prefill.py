"""Riders of the lattice launch: given the gradient buffer, a forward call zero-fills padded cells of it while the
lattice recursion runs, as far as it gets, and the backward call with padding_zeroed = 2 skips what was done.
Whatever the riders managed (nothing on a small problem whose lattice ends before they start, everything beside a
long TDT lattice), forward + backward must leave exactly what the plain calls leave, the forward call must touch
padded cells only, and a workspace full of junk must not change any of it."""

import numpy as np
import pytest
import torch

from speech_amd import MultiblankRNNTLossNumba, RNNTLossNumba, TDTLossNumba, _native, synthetic
from speech_amd.rnnt_loss import rnnt, rnnt_pytorch

from gpu_utils import DEV

pytestmark = pytest.mark.gpu

# (a forward call that is handed a gradient buffer takes riders whatever the size of the problem: whether that pays is
# the caller's decision -- the modules and the combined entry points decide by the size of the gradient)

DURATIONS = [0, 1, 2, 3]
BIG_BLANKS = [2, 4]


def make(seed, B, T, U, V, dtype, full=False):
    rng = np.random.RandomState(seed)
    acts = torch.tensor(rng.randn(B, T, U, V), dtype=torch.float32).to(dtype).to(DEV)
    labels = torch.tensor(rng.randint(0, max(V - 6, 1), size=(B, U - 1)), dtype=torch.int64, device=DEV)
    al, ll = rng.randint(1, T + 1, size=B), rng.randint(0, U, size=B)
    al[0], ll[-1] = T, U - 1
    if full:
        al[:], ll[:] = T, U - 1
    return acts, labels, torch.tensor(al, device=DEV), torch.tensor(ll, device=DEV)


def run(kind, acts, labels, al, ll, prefill, ws=None, scale=None, mode=None):
    """(costs, grads, buffer as the forward call left it) through the function-level seam."""
    B, T, U, V = acts.shape
    D = {"rnnt": 0, "tdt": len(DURATIONS), "multiblank": len(BIG_BLANKS)}[kind]
    ws = rnnt.new_workspace(acts, D) if ws is None else ws
    costs = torch.empty(B, dtype=torch.float32, device=DEV)
    grads = torch.full_like(acts, float("nan"))
    pre = grads if prefill else None
    mode = (2 if prefill else 0) if mode is None else mode
    if kind == "rnnt":
        rnnt.rnnt_forward(acts, labels, al, ll, costs, V - 1, 0.01, True, ws, pre)
        after_forward = grads.clone()
        rnnt.rnnt_backward(acts, labels, al, ll, grads, scale, V - 1, 0.01, 0.0, ws, padding_zeroed=mode)
    elif kind == "tdt":
        rnnt.tdt_forward(acts, labels, al, ll, costs, V - D - 1, DURATIONS, 0.0, 0.05, False, True, ws, pre)
        after_forward = grads.clone()
        rnnt.tdt_backward(acts, labels, al, ll, grads, scale, V - D - 1, DURATIONS, 0.0, 0.0, 0.05, False, ws,
                          padding_zeroed=mode)  # fmt: skip
    else:
        rnnt.multiblank_forward(acts, labels, al, ll, costs, V - 1, BIG_BLANKS, 0.0, 0.05, True, ws, pre)
        after_forward = grads.clone()
        rnnt.multiblank_backward(acts, labels, al, ll, grads, scale, V - 1, BIG_BLANKS, 0.0, 0.0, 0.05, ws,
                                 padding_zeroed=mode)  # fmt: skip
    torch.cuda.synchronize()
    return costs, grads, after_forward


def check_forward_touched_padding_only(after_forward, al, ll, ws=None, D=0):
    touched = ~torch.isnan(after_forward.float())
    assert torch.all(after_forward[touched] == 0)
    for b in range(after_forward.shape[0]):
        assert not touched[b, : int(al[b]), : int(ll[b]) + 1].any(), "a rider wrote into a valid cell"
    if ws is not None:  # the record names exactly the cells that were filled (whole rows)
        B, T, U, V = after_forward.shape
        said = rnnt.prefilled_cells(ws, al, ll, B, T, U, V, after_forward.element_size(), D)
        assert torch.equal(said, touched.all(dim=-1)) and torch.equal(said, touched.any(dim=-1))


# V: rows of one vector up to rows that take a workgroup of 1024 threads (one row per item), odd and even starts
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V", [29, 257, 1025, 4100, 16385])
@pytest.mark.parametrize("kind", ["rnnt", "tdt", "multiblank"])
def test_prefilled_gradient_equals_the_plain_gradient(kind, V, dtype):
    B, T, U = 3, 21, 11  # U is no multiple of the eight rows of an item
    acts, labels, al, ll = make(V, B, T, U, V, dtype)
    scale = torch.tensor([0.5, 1.0, 2.0], device=DEV)
    c0, g0, _ = run(kind, acts, labels, al, ll, False, scale=scale)
    c1, g1, after_forward = run(kind, acts, labels, al, ll, True, scale=scale)
    assert torch.isfinite(g0.float()).all()
    assert torch.equal(c0, c1) and torch.equal(g0, g1)
    check_forward_touched_padding_only(after_forward, al, ll)


@pytest.mark.parametrize("kind", ["rnnt", "tdt", "multiblank"])
def test_riders_fill_padding_beside_a_long_lattice(kind):
    """A lattice of several hundred anti-diagonals gives the riders time: they must have filled some padding, only
    padding, and the result must not change."""
    B, T, U, V = 4, 300, 40, 257 if kind != "tdt" else 257 + len(DURATIONS)
    acts, labels, al, ll = make(7, B, T, U, V, torch.float32)
    al[1], al[2] = 40, 150  # one long utterance keeps the lattice going while the short ones leave padding
    c0, g0, _ = run(kind, acts, labels, al, ll, False)
    D = {"rnnt": 0, "tdt": len(DURATIONS), "multiblank": len(BIG_BLANKS)}[kind]
    ws = rnnt.new_workspace(acts, D)
    c1, g1, after_forward = run(kind, acts, labels, al, ll, True, ws=ws)
    assert torch.equal(c0, c1) and torch.equal(g0, g1)
    check_forward_touched_padding_only(after_forward, al, ll, ws, D)
    assert (~torch.isnan(after_forward)).any(), "the riders filled nothing beside a lattice of 340 anti-diagonals"


@pytest.mark.parametrize("kind", ["rnnt", "tdt", "multiblank"])
@pytest.mark.parametrize("junk", ["nan", "ff", "zero"])
def test_junk_in_the_workspace_does_not_reach_the_result(kind, junk):
    B, T, U, V = 3, 60, 13, 300
    acts, labels, al, ll = make(11, B, T, U, V, torch.float32)
    c0, g0, _ = run(kind, acts, labels, al, ll, False)
    D = {"rnnt": 0, "tdt": len(DURATIONS), "multiblank": len(BIG_BLANKS)}[kind]
    ws = rnnt.new_workspace(acts, D)
    if junk == "nan":
        ws.view(torch.float32)[: ws.numel() // 4] = float("nan")
    elif junk == "ff":
        ws.fill_(255)
    else:
        ws.zero_()
    c1, g1, after_forward = run(kind, acts, labels, al, ll, True, ws=ws)
    assert torch.equal(c0, c1) and torch.equal(g0, g1)
    check_forward_touched_padding_only(after_forward, al, ll, ws, D)
    # the same workspace again: what the first call left (its riders' words, its epoch) is not mistaken for news
    c2, g2, after_forward = run(kind, acts, labels, al, ll, True, ws=ws)
    assert torch.equal(c0, c2) and torch.equal(g0, g2)
    check_forward_touched_padding_only(after_forward, al, ll)


def test_no_padding_and_batches_too_large_for_riders():
    # nothing to fill
    acts, labels, al, ll = make(3, 2, 30, 9, 257, torch.float32, full=True)
    c0, g0, _ = run("rnnt", acts, labels, al, ll, False)
    c1, g1, after_forward = run("rnnt", acts, labels, al, ll, True)
    assert torch.equal(c0, c1) and torch.equal(g0, g1) and torch.isnan(after_forward).all()
    # more lattice workgroups than the record has room for: no riders, the record is cleared, same result
    acts, labels, al, ll = make(4, 150, 6, 5, 40, torch.float32)
    c0, g0, _ = run("rnnt", acts, labels, al, ll, False)
    c1, g1, after_forward = run("rnnt", acts, labels, al, ll, True)
    assert torch.equal(c0, c1) and torch.equal(g0, g1) and torch.isnan(after_forward).all()


def test_invalid_padding_mode_and_prefill_buffer():
    acts, labels, al, ll = make(5, 2, 8, 5, 40, torch.float32)
    ws = rnnt.new_workspace(acts)
    costs = torch.empty(2, dtype=torch.float32, device=DEV)
    grads = torch.empty_like(acts)
    rnnt.rnnt_forward(acts, labels, al, ll, costs, 39, 0.0, True, ws)
    with pytest.raises(RuntimeError):
        rnnt.rnnt_backward(acts, labels, al, ll, grads, None, 39, 0.0, 0.0, ws, padding_zeroed=3)
    with pytest.raises(ValueError):
        rnnt.rnnt_forward(acts, labels, al, ll, costs, 39, 0.0, True, ws, grads[:, :-1])
    with pytest.raises(ValueError):
        rnnt.rnnt_forward(acts, labels, al, ll, costs, 39, 0.0, True, ws, grads.to(torch.bfloat16))


@pytest.mark.parametrize("kind", ["rnnt", "tdt", "multiblank"])
def test_module_with_and_without_prefill(kind, monkeypatch):
    """The modules hand the lattice launch their gradient buffer by default on problems this size; switched off they
    must return the same costs and gradients, also from a logits view that starts off a 16-byte boundary, and a
    second backward call through a retained graph must not reuse the prefilled buffer."""
    index = {"rnnt": 1, "tdt": 3, "multiblank": 5}[kind]
    cfg, acts, labels, al, ll = synthetic.make_inputs(index, device=DEV, generate_on_device=True)
    B = 4  # a slice of the benchmark batch: ragged lengths, a lattice of several hundred anti-diagonals
    flat = torch.empty(acts[:B].numel() + 1, dtype=acts.dtype, device=DEV)
    view = flat[1:].view(acts[:B].shape)
    view.copy_(acts[:B])
    labels, al, ll = labels[:B].contiguous(), al[:B].clone(), ll[:B].clone()
    al[0], ll[B - 1] = acts.shape[1], acts.shape[2] - 1  # (the modules insist on one utterance of full length each way)
    if kind == "rnnt":
        loss = RNNTLossNumba(blank=cfg.blank, reduction="none", fastemit_lambda=0.001)
    elif kind == "tdt":
        loss = TDTLossNumba(blank=cfg.blank, durations=cfg.durations, reduction="none", sigma=cfg.sigma)
    else:
        loss = MultiblankRNNTLossNumba(blank=cfg.blank, big_blank_durations=cfg.big_blank_durations, reduction="none",
                                       sigma=cfg.sigma)  # fmt: skip
    out = {}
    for mode in ("0", "1"):
        monkeypatch.setattr(rnnt_pytorch, "_PREFILL_ENV", mode)
        a = view.detach().requires_grad_(True)
        costs = loss(a, labels, al, ll)
        (g1,) = torch.autograd.grad(costs.sum(), a, retain_graph=True)
        (g2,) = torch.autograd.grad((2.0 * costs).sum(), a)
        torch.cuda.synchronize()
        out[mode] = (costs.detach().clone(), g1.clone(), g2.clone())
    assert torch.equal(out["0"][0], out["1"][0])
    assert torch.equal(out["0"][1], out["1"][1]) and torch.equal(out["0"][2], out["1"][2])
    assert torch.isfinite(out["1"][1]).all() and out["1"][1].abs().sum() > 0
    for b in range(B):
        assert torch.all(out["1"][1][b, int(al[b]) :] == 0) and torch.all(out["1"][1][b, :, int(ll[b]) + 1 :] == 0)


@pytest.mark.parametrize("kind", ["rnnt", "tdt", "multiblank"])
def test_replayed_from_a_graph(kind):
    """Captured once and replayed, the launch's epoch is the same every time: the riders must still tell this replay's
    lattice from the last one's (they did nothing on replays when they could not), and every replay must give the
    eager result."""
    B, T, U, V = 4, 300, 40, 257 if kind != "tdt" else 257 + len(DURATIONS)
    D = {"rnnt": 0, "tdt": len(DURATIONS), "multiblank": len(BIG_BLANKS)}[kind]
    acts, labels, al, ll = make(9, B, T, U, V, torch.float32)
    al[1], al[2] = 40, 150
    c0, g0, _ = run(kind, acts, labels, al, ll, False)
    ws = rnnt.new_workspace(acts, D)
    costs = torch.empty(B, dtype=torch.float32, device=DEV)
    grads = torch.full_like(acts, float("nan"))

    def step():
        if kind == "rnnt":
            rnnt.rnnt_forward(acts, labels, al, ll, costs, V - 1, 0.01, True, ws, grads)
            rnnt.rnnt_backward(acts, labels, al, ll, grads, None, V - 1, 0.01, 0.0, ws, padding_zeroed=2)
        elif kind == "tdt":
            rnnt.tdt_forward(acts, labels, al, ll, costs, V - D - 1, DURATIONS, 0.0, 0.05, False, True, ws, grads)
            rnnt.tdt_backward(acts, labels, al, ll, grads, None, V - D - 1, DURATIONS, 0.0, 0.0, 0.05, False, ws,
                              padding_zeroed=2)  # fmt: skip
        else:
            rnnt.multiblank_forward(acts, labels, al, ll, costs, V - 1, BIG_BLANKS, 0.0, 0.05, True, ws, grads)
            rnnt.multiblank_backward(acts, labels, al, ll, grads, None, V - 1, BIG_BLANKS, 0.0, 0.0, 0.05, ws,
                                     padding_zeroed=2)  # fmt: skip

    step()
    torch.cuda.synchronize()
    assert torch.equal(g0, grads)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for replay in range(4):
        grads.fill_(float("nan"))  # eager work between the replays
        costs.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(c0, costs) and torch.equal(g0, grads), f"replay {replay}"
        said = rnnt.prefilled_cells(ws, al, ll, B, T, U, V, 4, D)
        assert said.any(), f"the riders did nothing on replay {replay}"


def test_combined_entry_point_decides_by_size_unless_told():
    """mi_rnnt_loss with riders = AUTO launches none for a gradient below 32 MiB (the record stays empty), ON fills
    padding beside a lattice of several hundred anti-diagonals, OFF never does; the results are the same bits."""
    import ctypes

    B, T, U, V = 4, 300, 40, 129
    acts, labels, al, ll = make(7, B, T, U, V, torch.float32)
    al[1], al[2] = 40, 150
    assert acts.numel() * 4 < (32 << 20)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {}
    for riders in (_native.RIDERS_AUTO, _native.RIDERS_OFF, _native.RIDERS_ON):
        ws = rnnt.new_workspace(acts)
        ws.fill_(255)
        costs = torch.empty(B, dtype=torch.float32, device=DEV)
        grads = torch.full_like(acts, float("nan"))
        st = _native.lib().mi_rnnt_loss(acts.data_ptr(), 0, labels.data_ptr(), al.data_ptr(), ll.data_ptr(),
                                        costs.data_ptr(), grads.data_ptr(), None, 0, 1.0, B, T, U, V, V - 1, 0.01, 0.0,
                                        riders, ws.data_ptr(), ws.numel(), stream)  # fmt: skip
        assert st == _native.SUCCESS
        torch.cuda.synchronize()
        out[riders] = (costs, grads, rnnt.prefilled_cells(ws, al, ll, B, T, U, V, 4))
    assert not out[_native.RIDERS_AUTO][2].any() and not out[_native.RIDERS_OFF][2].any()
    assert out[_native.RIDERS_ON][2].any(), "riders = ON filled nothing beside a lattice of 340 anti-diagonals"
    for riders in (_native.RIDERS_OFF, _native.RIDERS_ON):
        assert torch.equal(out[riders][0], out[_native.RIDERS_AUTO][0])
        assert torch.equal(out[riders][1], out[_native.RIDERS_AUTO][1])
    assert torch.isfinite(out[_native.RIDERS_ON][1]).all()


def test_riders_fill_something_at_the_benchmark_shape():
    """B=16, T=375, U=121, V=1025 fp32 through the module: the riders of its lattice launch must fill part of the
    padding -- a driver or firmware that parks every rider would otherwise only show as a slower step."""
    cfg, acts, labels, al, ll = synthetic.make_inputs(1, device=DEV, generate_on_device=True)
    assert rnnt_pytorch._prefill_wanted(acts)
    ws = rnnt.new_workspace(acts)
    costs = torch.empty(cfg.B, dtype=torch.float32, device=DEV)
    grads = torch.empty_like(acts)
    filled = []
    for _ in range(3):
        rnnt.rnnt_forward(acts, labels, al, ll, costs, cfg.blank, 0.0, True, ws, grads)
        filled.append(int(rnnt.prefilled_cells(ws, al, ll, cfg.B, cfg.T, cfg.U, cfg.V, 4).sum()))
    assert max(filled) > 0, filled


@pytest.mark.parametrize("omega", [0.0, 1.0])
def test_function_level_seams_take_riders_by_themselves(omega):
    """rnnt_loss_gpu / tdt_loss_gpu (the reference's signatures: split token logits and duration log-probs, also its
    plain-RNNT branch) / combined_tdt_loss_gpu / multiblank_rnnt_loss_gpu hand their gradient buffer to the lattice
    launch on their own: with riders forced on and off the results must be the same bits."""
    B, T, U, V, D = 4, 200, 30, 130, len(DURATIONS)
    acts, labels, al, ll = make(13, B, T, U, V + D, torch.float32)
    al[1], al[2] = 30, 90
    label_acts = acts[..., :V].contiguous()
    duration_acts = torch.log_softmax(acts[..., V:], dim=-1).contiguous()
    mb_acts = acts[..., : V + len(BIG_BLANKS)].contiguous()
    out = {}
    for riders in (True, False):
        res = []
        costs, grads = torch.empty(B, device=DEV), torch.full_like(label_acts, float("nan"))
        rnnt.rnnt_loss_gpu(label_acts, labels, al, ll, costs, grads, V - 1, 0.01, 0.0, riders=riders)
        res += [costs, grads]
        costs, lg, dg = torch.empty(B, device=DEV), torch.full_like(label_acts, float("nan")), torch.full_like(duration_acts, float("nan"))
        rnnt.tdt_loss_gpu(label_acts, duration_acts, labels, al, ll, costs, lg, dg, V - 1, DURATIONS, 0.0, 0.0, 0, 0.05, omega,
                          riders=riders)  # fmt: skip
        res += [costs, lg, dg]
        costs, grads = torch.empty(B, device=DEV), torch.full_like(acts, float("nan"))
        rnnt.combined_tdt_loss_gpu(acts, labels, al, ll, costs, grads, V - 1, DURATIONS, 0.0, 0.0, 0, 0.05, omega > 0.5,
                                   riders=riders)  # fmt: skip
        res += [costs, grads]
        costs, grads = torch.empty(B, device=DEV), torch.full_like(mb_acts, float("nan"))
        rnnt.multiblank_rnnt_loss_gpu(mb_acts, labels, al, ll, costs, grads, V + len(BIG_BLANKS) - 1, BIG_BLANKS, 0.0, 0.0, 0,
                                      0.05, riders=riders)  # fmt: skip
        res += [costs, grads]
        torch.cuda.synchronize()
        out[riders] = res
    for a, b in zip(out[True], out[False]):
        assert torch.isfinite(a).all() and torch.equal(a, b)


def test_random_shapes_with_and_without_riders():
    """Seeded random shapes, lengths, dtypes and vocabulary sizes of every row-length class through the function-level
    seam: with riders the costs and gradients are bit-identical to the plain calls, and the forward call touched
    padding only."""
    rng = np.random.RandomState(20240607)
    Vs = [5, 17, 65, 129, 257, 513, 1025, 2049, 4097, 8193, 16385]
    for it in range(45):
        kind = ["rnnt", "tdt", "multiblank"][it % 3]
        B, T, U = int(rng.randint(1, 6)), int(rng.randint(1, 200)), int(rng.randint(2, 60))
        V = Vs[(it // 3) % len(Vs)] + {"rnnt": 0, "tdt": len(DURATIONS), "multiblank": len(BIG_BLANKS)}[kind]
        if B * T * U * V > 2.0e7:
            T = max(1, int(2.0e7 / (B * U * V)))
        dtype = [torch.float32, torch.bfloat16, torch.float16][(it // 3) % 3]
        acts, labels, al, ll = make(1000 + it, B, T, U, V, dtype)
        case = "%s B=%d T=%d U=%d V=%d %s" % (kind, B, T, U, V, dtype)
        plain = run(kind, acts, labels, al, ll, prefill=False)
        ws = rnnt.new_workspace(acts, {"rnnt": 0, "tdt": len(DURATIONS), "multiblank": len(BIG_BLANKS)}[kind])
        ridden = run(kind, acts, labels, al, ll, prefill=True, ws=ws)
        assert torch.equal(plain[0], ridden[0]), case
        assert torch.equal(plain[1], ridden[1]), case
        assert torch.isfinite(ridden[1].float()).all(), case
        check_forward_touched_padding_only(ridden[2], al, ll)


@pytest.mark.parametrize("kind", ["rnnt", "tdt", "multiblank"])
def test_a_record_of_an_earlier_call_is_not_believed(kind):
    """A workspace whose last call had riders serves a forward call without a gradient buffer; a backward call that is
    nevertheless told to consult the record must find it empty and write every padded cell itself."""
    V = 1025 + {"rnnt": 0, "tdt": len(DURATIONS), "multiblank": len(BIG_BLANKS)}[kind]
    acts, labels, al, ll = make(77, 4, 120, 40, V, torch.float32)
    ws = rnnt.new_workspace(acts, {"rnnt": 0, "tdt": len(DURATIONS), "multiblank": len(BIG_BLANKS)}[kind])
    first = run(kind, acts, labels, al, ll, prefill=True, ws=ws)
    assert (~torch.isnan(first[2])).any(), "the riders of the first call were expected to fill something"
    plain = run(kind, acts, labels, al, ll, prefill=False)
    again = run(kind, acts, labels, al, ll, prefill=False, ws=ws, mode=2)
    assert torch.isnan(again[2]).all()  # no riders: the forward call left the buffer alone
    assert torch.equal(plain[0], again[0]) and torch.equal(plain[1], again[1])
