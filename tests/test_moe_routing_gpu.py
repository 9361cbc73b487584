"""MoE routing kernels against the CPU oracle: ids, sorted slots and offsets bit-exact; softmax
weights to 1e-6 relative (expf vs float64 exp), sigmoid-routing weights bit-exact."""
import numpy as np
import pytest
import torch

from oracle import moe as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _topk_softmax(hk, logits, k):
    T = logits.shape[0]
    lg = torch.from_numpy(logits).to(DEV)
    ids = torch.full((T, k), -1, dtype=torch.int32, device=DEV)
    w = torch.zeros((T, k), dtype=torch.float32, device=DEV)
    hk.tk_kernel.dispatch_moe_topk_softmax(lg, ids, w)
    torch.cuda.synchronize()
    return ids.cpu().numpy(), w.cpu().numpy()


@pytest.mark.parametrize("T,E,k", [(4096, 128, 4), (1, 128, 4), (7, 8, 8), (513, 256, 8), (33, 512, 6), (100, 40, 3)])
def test_topk_softmax(hk, T, E, k):
    rng = np.random.default_rng(T + E + k)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    if T > 5:
        logits[2, :] = 1.0                       # all tied
        logits[3, E - 1] = logits[3, 0] = 9.0    # tie between first and last
        logits[4, 1] = -0.0; logits[4, 0] = 0.0  # signed zeros tie
        logits[4, 2:] = -1.0
    ids, w = _topk_softmax(hk, logits, k)
    rid, rw = O.topk_softmax(logits, k)
    assert np.array_equal(ids, rid)
    assert np.allclose(w, rw, rtol=2e-6, atol=1e-9)


@pytest.mark.parametrize("T,E,k,G,KG,use_bias", [(8192, 256, 8, 8, 4, False), (300, 256, 8, 8, 4, True),
                                                 (65, 64, 6, 4, 2, True), (9, 32, 4, 32, 8, False),
                                                 (17, 128, 8, 1, 1, True), (50, 192, 5, 4, 3, True),
                                                 (1000, 128, 4, 8, 2, False), (33, 64, 16, 16, 16, True),
                                                 (21, 96, 3, 3, 2, False)])
def test_topk_grouped_sigmoid(hk, T, E, k, G, KG, use_bias):
    rng = np.random.default_rng(T + E)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[0, :] = 0.5  # all tied
    if T > 2:
        logits[1, :] = np.linspace(-40, 40, E, dtype=np.float32)  # saturating sigmoid
    bias = (rng.standard_normal(E) * 0.05).astype(np.float32) if use_bias else None
    lg = torch.from_numpy(logits).to(DEV)
    bt = torch.from_numpy(bias).to(DEV) if use_bias else None
    ids = torch.full((T, k), -1, dtype=torch.int32, device=DEV)
    w = torch.zeros((T, k), dtype=torch.float32, device=DEV)
    hk.tk_kernel.dispatch_moe_topk_grouped_sigmoid(lg, bt, ids, w, G, KG, 2.5)
    torch.cuda.synchronize()
    rid, rw = O.topk_grouped_sigmoid(logits, bias, k, G, KG, 2.5)
    assert np.array_equal(ids.cpu().numpy(), rid)
    assert np.array_equal(w.cpu().numpy(), rw)


def _sort(hk, ids_np, E):
    T, k = ids_np.shape
    ids = torch.from_numpy(ids_np).to(DEV)
    ss = torch.full((T * k,), -1, dtype=torch.int32, device=DEV)
    off = torch.full((E + 1,), -1, dtype=torch.int32, device=DEV)
    inv = torch.full((T * k,), -1, dtype=torch.int32, device=DEV)
    ws = torch.empty(hk.tk_kernel.moe_sort_workspace_bytes(T, k, E), dtype=torch.uint8, device=DEV)
    hk.tk_kernel.dispatch_moe_sort(ids, ss, off, inv, ws)
    torch.cuda.synchronize()
    return ss.cpu().numpy(), off.cpu().numpy(), inv.cpu().numpy()


# up to 16384 slots: one workgroup does the whole sort; above: count / scan / scatter launches, with the
# scan in one workgroup up to 64 chunks of 1024 slots
@pytest.mark.parametrize("T,k,E", [(4096, 4, 128), (8192, 8, 256), (1, 1, 1), (3, 2, 512), (1000, 3, 7), (257, 4, 16),
                                   (16384, 1, 512), (16385, 1, 512), (4097, 4, 128), (2048, 8, 3), (65, 1, 2),
                                   (1023, 16, 300), (40000, 2, 100)])
def test_moe_sort(hk, T, k, E):
    rng = np.random.default_rng(T * 7 + k)
    ids = np.stack([rng.permutation(E)[:k] if k <= E else rng.integers(0, E, k) for _ in range(T)]).astype(np.int32)
    ss, off, inv = _sort(hk, ids, E)
    ro, roff, rinv = O.moe_sort(ids, E)
    assert np.array_equal(off, roff)
    assert np.array_equal(ss, ro)
    assert np.array_equal(inv, rinv)


def test_moe_sort_skewed_and_empty_experts(hk):
    T, k, E = 5000, 2, 64
    ids = np.zeros((T, k), dtype=np.int32)
    ids[:, 0] = 5          # everything on expert 5 ...
    ids[:, 1] = 63         # ... and 63; all others empty
    ids[::97, 1] = 0
    ss, off, inv = _sort(hk, ids, E)
    ro, roff, rinv = O.moe_sort(ids, E)
    assert np.array_equal(off, roff) and np.array_equal(ss, ro) and np.array_equal(inv, rinv)


@pytest.mark.parametrize("T,k,E", [(3000, 4, 128), (20000, 4, 512), (70000, 2, 100), (300, 2, 5)])
def test_moe_sort_drops_ids_outside_the_expert_range(hk, T, k, E):
    """Ids outside [0, E) (masked or padded tokens: -1, E, a large value) take no part on either
    launch path (one launch up to 16384 slots; count / scan / scatter above): the valid slots are
    sorted as if the others were absent, the tail of sorted_slots and the dropped slots' slot_to_pos
    keep the caller's contents, and nothing outside the outputs is written."""
    print(f"moe_sort invalid ids T={T} k={k} E={E}", flush=True)
    rng = np.random.default_rng(T + k + E)
    ids = rng.integers(0, E, size=(T, k)).astype(np.int32)
    bad = rng.random((T, k)) < 0.1
    ids[bad] = rng.choice(np.array([-1, E, E + 7, 511, 512, 2 ** 31 - 1, -2 ** 31], dtype=np.int64),
                          size=int(bad.sum())).astype(np.int32)
    bad = (ids < 0) | (ids >= E)
    ss, off, inv = _sort(hk, ids, E)
    flat = ids.reshape(-1)
    valid = np.nonzero(~bad.reshape(-1))[0].astype(np.int32)
    order = valid[np.argsort(flat[valid], kind="stable")]
    counts = np.bincount(flat[valid], minlength=E)
    assert np.array_equal(off, np.concatenate([[0], np.cumsum(counts)]).astype(np.int32))
    n = valid.size
    assert np.array_equal(ss[:n], order)
    assert np.all(ss[n:] == -1)                       # untouched (the test pre-fills -1)
    want_inv = np.full(T * k, -1, dtype=np.int32)
    want_inv[order] = np.arange(n, dtype=np.int32)
    assert np.array_equal(inv, want_inv)


def test_routing_rejects_bad_arguments(hk):
    lg = torch.zeros((4, 1024), dtype=torch.float32, device=DEV)
    ids = torch.zeros((4, 2), dtype=torch.int32, device=DEV)
    w = torch.zeros((4, 2), dtype=torch.float32, device=DEV)
    with pytest.raises(RuntimeError):
        hk.tk_kernel.dispatch_moe_topk_softmax(lg, ids, w)  # E > 512
    lg = torch.zeros((4, 30), dtype=torch.float32, device=DEV)
    with pytest.raises(RuntimeError):
        hk.tk_kernel.dispatch_moe_topk_grouped_sigmoid(lg, None, ids, w, 4, 2)  # E % n_group
