"""Seeded random sweep of the prepared call and of the layer's form against the oracle: shapes, epilogue, output type,
alignment of B and every hook of the C ABI drawn at random; integer operands, so every result must match bit for bit."""
import numpy as np
import pytest
import torch

import oracle
from onebitsparsemul_amd import _native, synthetic

pytestmark = pytest.mark.gpu


def _reset():
    _native.set_tile_config(-1)
    _native.set_skinny_enabled(True)
    _native.set_skinny_rows(-1)
    _native.set_split_k(-1)
    _native.set_pad_b(True)


@pytest.fixture(autouse=True)
def _defaults():
    _reset()
    yield
    _reset()


@pytest.mark.parametrize("seed", range(6))
def test_random_cases_match_the_oracle(seed):
    rng = np.random.default_rng(1000 + seed)
    for case in range(25):
        m = 64 * int(rng.integers(1, 24))
        k = 32 * int(rng.integers(1, 60)) if rng.random() < 0.85 else 32 * int(rng.integers(60, 300))
        n = int(rng.choice([1, 3, 4, 7, 8, 15, 16, 17, 24, 32, 33, 48, 64, 65, 72, 100, 128, 136, 200, 264]))
        alpha = float(rng.choice([1.0, 2.0, -1.0]))
        beta = float(rng.choice([0.0, 1.0]))
        out_dtype = torch.float32 if rng.random() < 0.5 else torch.float16
        hooks = dict(skinny=bool(rng.random() < 0.8), rows=int(rng.choice([-1, 32, 64, 128])),
                     split=int(rng.choice([-1, -1, 1, 2, 3, 5])), tile=int(rng.choice([-1, -1, -1] + list(range(16)))),
                     pad=bool(rng.random() < 0.8))
        offset = int(rng.choice([0, 0, 1, 4, 8]))  # halves: B 2, 8 or 16 bytes past a 16-byte boundary
        static = bool(rng.random() < 0.4)          # the entry point whose buffers live in the fixed device array
        _native.set_skinny_enabled(hooks["skinny"])
        _native.set_skinny_rows(hooks["rows"])
        _native.set_split_k(hooks["split"])
        _native.set_tile_config(hooks["tile"])
        _native.set_pad_b(hooks["pad"])
        what = (f"seed {seed} case {case}: m={m} n={n} k={k} alpha={alpha} beta={beta} {out_dtype} {hooks} offset={offset} "
                f"static={static}")
        a, meta = synthetic.make_weight(m, k, seed=int(rng.integers(1 << 30)))
        dense = oracle.decompress_operands(a.numpy(), meta.numpy(), m, k)
        bi = synthetic.make_b(k, n, seed=case, kind="int")
        ci = synthetic.make_c(m, n, seed=case + 1, dtype=torch.float32).round() if beta else None
        exact = oracle.host_gemm(dense, bi.numpy(), c=ci.numpy() if beta else None, alpha=alpha, beta=beta,
                                 d_dtype=oracle.F32, acc="f32")
        want = exact if out_dtype == torch.float32 else exact.astype(np.float16)
        prep = _native.prepare(a.cuda(), meta.cuda(), m, k)
        storage = torch.zeros(k * n + 16, dtype=torch.float16, device="cuda")
        bd = storage[offset:offset + k * n].view(k, n)
        bd.copy_(bi.cuda())
        d = torch.full((m, n), float("nan"), dtype=out_dtype, device="cuda")
        _native.matmul_prepared(prep, bd, d, m, n, k, c=ci.cuda() if beta else None, alpha=alpha, beta=beta,
                                static_scratch=static)
        torch.cuda.synchronize()
        assert np.array_equal(d.cpu().numpy(), want), what
        # the layer's form of the same product (tiles without a token-major variant: automatic choice)
        if hooks["tile"] not in (-1, 4, 6, 9, 10, 11, 12, 13, 14, 15):
            _native.set_tile_config(-1)
        plain = oracle.host_gemm(dense, bi.numpy(), d_dtype=oracle.F32, acc="f32")
        bias = synthetic.make_b(1, m, seed=case + 2, kind="int").reshape(m)
        y = torch.full((n, m), float("nan"), dtype=out_dtype, device="cuda")
        _native.linear_prepared(prep, bi.T.contiguous().cuda(), y, m, k, bias=bias.cuda())
        torch.cuda.synchronize()
        want_y = plain.T + bias.numpy().astype(np.float32)[None, :]
        assert np.array_equal(y.cpu().numpy(), want_y.astype(np.float32 if out_dtype == torch.float32 else np.float16)), what
