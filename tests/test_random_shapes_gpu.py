"""A seeded sweep over irregular problems -- ragged rows and reductions, odd group sizes, every
mode, both weight widths, both element types, 1-16 activation rows -- so that every launch rule
(k split, tile walks, which matrix-core kernel, how many tiles share a stage) meets shapes it
was not tuned on.  Same bars as the other GPU tests."""
import numpy as np
import pytest

from helpers import PER_COLUMN, SCALE_AND_ZEROS, SCALE_ONLY, DeviceProblem, Problem, bf16_ulp_report, error_report

pytestmark = pytest.mark.gpu


def _cases():
    rng = np.random.default_rng(20240611)
    out = []
    # (n_out range, k range): mostly small, a few with many tiles and a short reduction
    families = [((4, 600), (32, 4096), 22), ((600, 4096), (32, 2048), 10), ((10880, 23000), (64, 640), 6)]
    for (n_lo, n_hi), (k_lo, k_hi), count in families:
        for _ in range(count):
            bits = int(rng.choice([4, 4, 8]))
            chunk = 32 if bits == 4 else 16
            n_out = int(rng.integers(n_lo // 4, n_hi // 4 + 1)) * 4
            k = int(rng.integers(max(1, k_lo // chunk), k_hi // chunk + 1)) * chunk
            qop = int(rng.choice([PER_COLUMN, SCALE_ONLY, SCALE_AND_ZEROS, SCALE_AND_ZEROS]))
            groups = [g for g in range(64, k + 1, 32) if k % g == 0]
            if qop != PER_COLUMN and not groups:
                qop = PER_COLUMN
            group = int(rng.choice(groups[:6])) if qop != PER_COLUMN else 0
            m_batch = int(rng.choice([1, 1, 2, 3, 4, 5, 6, 8, 9, 12, 16]))
            if n_out * k * m_batch > 40_000_000:      # keep the CPU oracle quick
                m_batch = 1
            element = "bf16" if rng.random() < 0.35 else "f16"
            out.append((f"r{len(out)}_{n_out}x{k}_i{bits}_q{qop}_g{group}_m{m_batch}_{element}",
                        n_out, k, bits, qop, group, m_batch, bool(rng.integers(0, 2)), element))
    # per-column mode with reductions that are a multiple of 8 only (utils/preprocess.h:324-327)
    for _ in range(8):
        bits = int(rng.choice([4, 8]))
        n_out = int(rng.integers(1, 200)) * 4
        k = int(rng.integers(1, 400)) * 8
        m_batch = int(rng.choice([1, 2, 4, 5, 8, 16]))
        element = "bf16" if rng.random() < 0.35 else "f16"
        out.append((f"r{len(out)}_{n_out}x{k}_i{bits}_q1_g0_m{m_batch}_{element}", n_out, k, bits, PER_COLUMN, 0, m_batch,
                    bool(rng.integers(0, 2)), element))
    # enough tiles for 8 of them to share one 16-row activation stage, and for 2 to share 8 rows
    out.append(("fixed_21780x160_i4_q3_g160_m13_f16", 21780, 160, 4, SCALE_AND_ZEROS, 160, 13, True, "f16"))
    out.append(("fixed_22000x128_i4_q2_g64_m16_bf16", 22000, 128, 4, SCALE_ONLY, 64, 16, False, "bf16"))
    out.append(("fixed_6000x544_i8_q3_g544_m7_f16", 6000, 544, 8, SCALE_AND_ZEROS, 544, 7, True, "f16"))
    return out


CASES = _cases()


@pytest.mark.parametrize("cfg", CASES, ids=[c[0] for c in CASES])
def test_random_shape_parity(gpu, cfg):
    tag, n_out, k, bits, qop, group, m_batch, bias, element = cfg
    prob = Problem(tag, n_out, k, bits, qop, group, m_batch=m_batch, bias=bias, element=element,
                   x_dist="normal" if n_out % 8 else "uniform")
    dev = DeviceProblem(prob, gpu)
    if n_out * k <= 4_000_000:
        got, want = dev.dequant(), prob.oracle_dequant()
        assert int((got.view(np.uint16) != want.view(np.uint16)).sum()) == 0, "dequantised weights differ"
    y = dev.run()
    ref = prob.oracle_gemv(threads=16)
    if element == "bf16":
        ulp, differing = bf16_ulp_report(y, ref)
        assert ulp <= 1.0 + 1e-6 and differing <= 0.02, (ulp, differing)
    else:
        _, rel, _ = error_report(y, ref)
        assert np.isfinite(y.astype(np.float32)).all() and rel <= 2e-3, rel


def _k_stationary_cases():
    """The fp16 problems of the sweep above that fit the k-stationary matrix-core kernel (one wave per k step:
    at most 16 k steps), each with a seeded cap on the workgroups, so that walks of every length, ragged last
    tiles and ragged last k steps meet that kernel too, whatever the launch rules would have picked."""
    rng = np.random.default_rng(977)
    out = []
    for cfg in CASES:
        tag, n_out, k, bits, qop, group, m_batch, bias, element = cfg
        ksteps = -(-k // (512 if bits == 4 else 256))
        if element != "f16" or ksteps > 16:
            continue
        rows = m_batch if m_batch > 1 else int(rng.choice([2, 3, 7, 11, 16]))
        if n_out * k * rows > 40_000_000:
            rows = 2
        cap = int(rng.choice([0, 0, 8, 16, 40, 104]))
        out.append((f"{tag}_rows{rows}_cap{cap}", cfg, rows, cap))
    return out


KS_CASES = _k_stationary_cases()


@pytest.mark.parametrize("case", KS_CASES, ids=[c[0] for c in KS_CASES])
def test_random_shape_parity_on_the_k_stationary_kernel(gpu, case):
    import mixed_gemv_amd as mg
    _, (tag, n_out, k, bits, qop, group, _, bias, _), rows, cap = case
    prob = Problem(tag + "_ks", n_out, k, bits, qop, group, m_batch=rows, bias=bias, x_dist="normal" if n_out % 8 else "uniform")
    dev = DeviceProblem(prob, gpu)
    mg.set_matrix_core_threshold(1)
    mg.set_matrix_core_variant(mg.MATRIX_CORE_K_STATIONARY)
    mg.set_launch_override(0, 0, 0, cap)
    try:
        plan = mg.query_launch(n_out, rows, k, bits, prob.group_size)
        assert plan["matrix_core"] == 3, plan
        cov = mg.plan_coverage(n_out, rows, k, bits, prob.group_size)
        assert cov["tiles_miscovered"] == 0 and cov["bad_waves"] == 0, cov
        y = dev.run()
    finally:
        mg.set_launch_override(0, 0, 0, 0)
        mg.set_matrix_core_variant(mg.MATRIX_CORE_AUTO)
        mg.set_matrix_core_threshold(0)
    _, rel, _ = error_report(y, prob.oracle_gemv(threads=16))
    assert np.isfinite(y.astype(np.float32)).all() and rel <= 2e-3, rel
