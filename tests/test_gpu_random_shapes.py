"""Random shapes and expert-size distributions: every fast path against the generic kernel (one thread per output
element, fp32 accumulation in k order), which the other GPU tests pin against the oracle. Covers what fixed cases
miss: tile tables with many experts, empty experts, sizes around the tile edges, N and K that are not multiples
of the tiles. Bar: the grouped-GEMM bar of the parity tests, 1e-2 + 1e-2 |ref| on bf16 results (the two sides
round the same fp32 sums, accumulated in different orders)."""
import random

import pytest
import torch

pytestmark = pytest.mark.gpu

GENERIC, PINGPONG, AUTO = 4, 0, -1


def sizes_for(rng, G, M):
    kind = rng.choice(["even", "rand", "zipf", "sparse"])
    if kind == "even":
        ms = [M // G] * G
    elif kind == "rand":
        cuts = sorted(rng.randint(0, M) for _ in range(G - 1))
        ms = [b - a for a, b in zip([0] + cuts, cuts + [M])]
    elif kind == "zipf":
        w = [1.0 / (i + 1) ** 1.2 for i in range(G)]
        ms = [int(M * v / sum(w)) for v in w]
    else:
        ms = [0] * G
        for _ in range(max(1, G // 4)):
            ms[rng.randrange(G)] += M // max(1, G // 4)
    rng.shuffle(ms)
    return ms


def close(a, b, tol=1e-2):
    d = (a.float() - b.float()).abs()
    return bool((d <= tol + tol * b.float().abs()).all()), float(d.max()) if d.numel() else 0.0


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_fast_paths_against_the_generic_kernel(seed):
    import applied_ai_amd as A
    from applied_ai_amd import _lib

    L = _lib.lib()
    rng = random.Random(seed)
    gen = torch.Generator(device="cuda").manual_seed(seed)
    try:
        for it in range(12):
            G = rng.choice([1, 2, 3, 8, 17, 64, 200])
            M = rng.choice([1, 77, 256, 300, 1000, 2049, 5000])
            N = rng.choice([8, 64, 72, 256, 264, 520, 1024, 1536])
            K = rng.choice([64, 128, 192, 448, 1024])
            ms = sizes_for(rng, G, M)
            R, pad = sum(ms), rng.choice([0, 0, 5])
            print(f"seed {seed} case {it}: G={G} rows={R}+{pad} N={N} K={K}", flush=True)
            x = (torch.randn(R + pad, K, device="cuda", generator=gen) / 4).bfloat16()
            w = (torch.randn(G * N, K, device="cuda", generator=gen) / 4).bfloat16()
            m = torch.tensor(ms, dtype=torch.int32, device="cuda")
            L.moe_gg_set_variant(0, GENERIC)
            ref = A.grouped_gemm(x, w, m)[:R]
            for variant in (PINGPONG, AUTO):
                L.moe_gg_set_variant(0, variant)
                ok, worst = close(A.grouped_gemm(x, w, m)[:R], ref)
                assert ok, (variant, G, R, N, K, worst)
            if N % 16 == 0 and R > 0:
                L.moe_gg_set_variant(0, GENERIC)
                two = A.silu_and_mul(A.grouped_gemm(x, w, m))[:R]
                L.moe_gg_set_variant(0, AUTO)
                ok, worst = close(A.grouped_gemm_swiglu(x, w, m)[:R], two, 2e-2)
                assert ok, ("swiglu", G, R, N, K, worst)
            if N % 4 == 0 and K % 4 == 0 and R > 0:
                go = (torch.randn(R + pad, N, device="cuda", generator=gen) / 4).bfloat16()
                L.moe_gg_set_variant(0, GENERIC)
                gx0, gw0 = A.grouped_gemm_backward(go, x, w, m)
                for variant in (AUTO, PINGPONG):
                    L.moe_gg_set_variant(0, variant)
                    gx, gw = A.grouped_gemm_backward(go, x, w, m)
                    ok, worst = close(gx, gx0, 2e-2)
                    assert ok, ("grad_x", variant, G, R, N, K, worst)
                    ok, worst = close(gw, gw0, 2e-2)
                    assert ok, ("grad_w", variant, G, R, N, K, worst)
    finally:
        L.moe_gg_set_variant(0, AUTO)


@pytest.mark.parametrize("seed", [21, 22])
def test_long_reductions_with_few_low_tiles(seed):
    """K >= 8192 and at most 32 experts: the automatic choice may leave the low tiles (an expert's few rows beyond
    its last full 256-row tile) to the small-M kernel, a decision both kernels take on the device. Random expert
    sizes around whole rounds of tiles, where that decision flips; reference = the ping-pong kernel alone."""
    import ctypes

    import applied_ai_amd as A
    from applied_ai_amd import _lib

    L = _lib.lib()
    rng = random.Random(seed)
    gen = torch.Generator(device="cuda").manual_seed(seed)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    nwg = cus - cus % 8
    apart = 0
    try:
        for it in range(8):
            N = rng.choice([256, 512, 1024, 2048])
            K = rng.choice([8192, 8320])
            G = rng.choice([2, 5, 8, 16, 32])
            ntn = N // 256
            # row tiles: about one round of long tiles, dealt to the experts; then tails
            tiles = [0] * G
            for _ in range(nwg // ntn + rng.choice([0, 0, 0, -3, 2])):
                tiles[rng.randrange(G)] += 1
            ms = []
            for t in tiles:
                kind = rng.choice(["full", "low", "low", "long"])
                if kind == "low":
                    ms.append(t * 256 + rng.choice([1, 7, 16, 31, 32, 33, 64, 100, 127]))
                elif kind == "long" and t > 0:
                    ms.append(t * 256 - rng.randint(1, 127))
                else:
                    ms.append(t * 256)
            R = sum(ms)
            arr = (ctypes.c_int32 * G)(*ms)
            hit = L.moe_gg_host_tails_apart(arr, G, R, N, K, nwg)
            apart += hit
            print(f"seed {seed} case {it}: G={G} rows={R} N={N} K={K} apart={hit} m_sizes={ms}", flush=True)
            x = (torch.randn(R, K, device="cuda", generator=gen) / 8).bfloat16()
            w = (torch.randn(G * N, K, device="cuda", generator=gen) / 8).bfloat16()
            m = torch.tensor(ms, dtype=torch.int32, device="cuda")
            L.moe_gg_set_variant(0, PINGPONG)
            ref = A.grouped_gemm(x, w, m)
            L.moe_gg_set_variant(0, AUTO)
            got = A.grouped_gemm(x, w, m)
            ok, worst = close(got, ref)
            assert ok, (G, R, N, K, ms, worst)
            del x, w, ref, got
        assert apart >= 2 or cus != 256, "the cases no longer reach the two-kernel path"
    finally:
        L.moe_gg_set_variant(0, AUTO)
