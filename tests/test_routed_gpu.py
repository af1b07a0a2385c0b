"""Routed launch over an expert stack (mgemv_gemv_routed): problem b of a launch takes the weights, scales,
zeros and bias of entry route[b] of the stack, x and y stay with the problem.  The reference only steps
through a stack at a fixed stride (gemv/kernel/mixed_gemv.h:140-149), so the check is against its own
semantics applied per problem: one ordinary launch on the routed matrix, which must give the same bits
(same kernel, same launch plan, same summation order), and the oracle for the values."""
import numpy as np
import pytest

import mixed_gemv_amd as mg
from helpers import PER_COLUMN, SCALE_AND_ZEROS, SCALE_ONLY, Problem, bf16_ulp_report, error_report

pytestmark = pytest.mark.gpu

REL_TOL = 2e-3
NAN_PATTERN = 0x7E00

# tag, n_out, k, bits, quant mode, group, activation rows, bias, element, forced matrix-core variant, kind expected
# (kind: 0 VALU, 1 register-operand, 2 LDS-staged, 3 k-stationary matrix-core kernel)
CASES = [
    ("valu_one_row", 80, 1024, 4, SCALE_AND_ZEROS, 128, 1, True, "f16", None, 0),
    ("valu_three_rows_scale_only", 64, 1536, 4, SCALE_ONLY, 64, 3, False, "f16", None, 0),
    ("valu_int8_per_column", 48, 768, 8, PER_COLUMN, 0, 1, True, "f16", None, 0),
    ("valu_bf16", 64, 1024, 4, SCALE_AND_ZEROS, 128, 2, True, "bf16", None, 0),
    ("lds_staged_eight_rows", 96, 2048, 4, SCALE_AND_ZEROS, 128, 8, True, "f16", mg.MATRIX_CORE_LDS_STAGED, 2),
    ("lds_staged_bf16", 64, 1024, 4, SCALE_AND_ZEROS, 64, 6, False, "bf16", mg.MATRIX_CORE_LDS_STAGED, 2),
    ("register_operand_eight_rows", 64, 1024, 4, SCALE_AND_ZEROS, 128, 8, True, "f16",
     mg.MATRIX_CORE_REGISTER_OPERAND, 1),
    ("k_stationary_four_rows", 80, 2048, 4, SCALE_AND_ZEROS, 128, 4, True, "f16", mg.MATRIX_CORE_K_STATIONARY, 3),
    ("k_stationary_int8", 64, 2048, 8, SCALE_ONLY, 128, 5, False, "f16", mg.MATRIX_CORE_K_STATIONARY, 3),
]

ENTRIES = 5
ROUTE = [3, 0, 3, 4, 1, 1]   # repeats, an entry nobody takes (2), first and last entry


class Stack:
    """ENTRIES matrices of one shape, preprocessed as one 3-D stack (utils/preprocess.h:134-136), plus one
    set of activation rows per routed problem."""

    def __init__(self, case, device, problems):
        import torch
        tag, n_out, k, bits, qop, g, m, bias, element, _, _ = case
        self.case = case
        self.experts = [Problem(f"{tag}/e{i}", n_out, k, bits, qop, g, m_batch=m, bias=bias, element=element)
                        for i in range(ENTRIES)]
        self.tokens = [Problem(f"{tag}/t{b}", n_out, k, bits, qop, g, m_batch=m, element=element).x
                       for b in range(problems)]
        qt = mg.QuantType.W4_A16 if bits == 4 else mg.QuantType.W8_A16
        raw = np.concatenate([p.w_raw for p in self.experts])
        self.one = mg.preprocessed_size((k, n_out), qt)
        as_dev = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).to(device)  # noqa: E731
        self.w = torch.from_numpy(mg.MixedGemvWeightPreprocessor.run(raw, (ENTRIES, k, n_out),
                                                                     mg.LayoutType.kColumnMajor, qt)).to(device)
        self.scale = as_dev(np.stack([p.scale for p in self.experts]))
        self.zero = as_dev(np.stack([p.zero_add for p in self.experts])) if qop == SCALE_AND_ZEROS else None
        self.bias = as_dev(np.stack([p.bias for p in self.experts])) if bias else None
        self.x = as_dev(np.stack(self.tokens))
        self.groups = k // self.experts[0].group_size
        self.device = device

    def strides(self, shared_x=False):
        _, n_out, k, _, _, _, m, _, _, _, _ = self.case
        return (self.one, 0 if shared_x else m * k, self.groups * n_out, n_out, m * n_out)

    def routed(self, route, shared_x=False):
        import torch
        _, n_out, k, bits, qop, _, m, _, element, _, _ = self.case
        r = torch.tensor(route, dtype=torch.int32, device=self.device)
        y = torch.full((len(route), m, n_out), NAN_PATTERN, dtype=torch.int16, device=self.device)
        mg.device_gemv_routed(self.w, self.x, self.scale, self.zero, self.bias, y, r, ENTRIES, len(route), n_out, m, k,
                              self.experts[0].group_size, self.strides(shared_x), qop, bits, element=element)
        torch.cuda.synchronize()
        return y.cpu().numpy().view(np.uint16)

    def single(self, entry, token):
        """One ordinary launch: the matrix `entry` of the stack on the activations of problem `token`."""
        import torch
        _, n_out, k, bits, qop, _, m, _, element, _, _ = self.case
        y = torch.full((m, n_out), NAN_PATTERN, dtype=torch.int16, device=self.device)
        w = self.w[entry * self.one:(entry + 1) * self.one]
        mg.device_gemv(w, self.x[token], self.scale[entry], None if self.zero is None else self.zero[entry],
                       None if self.bias is None else self.bias[entry], y, 1, n_out, m, k,
                       self.experts[0].group_size, qop, bits, element=element)
        torch.cuda.synchronize()
        return y.cpu().numpy().view(np.uint16)

    def oracle(self, entry, token):
        p = self.experts[entry]
        p.x = self.tokens[token]
        return p.oracle_gemv(threads=4)


@pytest.fixture()
def forced_variant():
    def force(variant):
        if variant is not None:
            mg.set_matrix_core_variant(variant)
            if variant == mg.MATRIX_CORE_K_STATIONARY:
                mg.set_matrix_core_threshold(1)
    yield force
    mg.set_matrix_core_variant(mg.MATRIX_CORE_AUTO)
    mg.set_matrix_core_threshold(0)


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_routed_launch_equals_one_launch_per_problem(gpu, forced_variant, case):
    tag, n_out, k, bits, _, _, m, _, element, variant, kind = case
    forced_variant(variant)
    assert mg.query_launch(n_out, m, k, bits, element=element)["matrix_core"] == kind, tag
    stack = Stack(case, gpu, len(ROUTE))
    got = stack.routed(ROUTE)
    for b, entry in enumerate(ROUTE):
        assert np.array_equal(got[b], stack.single(entry, b)), (tag, b, entry)
    for b in (0, 3):   # the values themselves, against the oracle
        ref = stack.oracle(ROUTE[b], b)
        if element == "bf16":
            worst, differing = bf16_ulp_report(got[b], ref)
            assert worst <= 1.0 and differing <= 0.01, (tag, b, worst, differing)
        else:
            assert error_report(got[b].view(np.float16), ref)[1] <= REL_TOL, (tag, b)


@pytest.mark.parametrize("case", [CASES[0], CASES[4], CASES[7]], ids=[CASES[i][0] for i in (0, 4, 7)])
def test_one_token_and_its_chosen_experts(gpu, forced_variant, case):
    """stride_x = 0: every problem of the launch reads the same activations (a decode step's top-k)."""
    forced_variant(case[9])
    stack = Stack(case, gpu, 1)
    route = [4, 2]
    got = stack.routed(route, shared_x=True)
    for b, entry in enumerate(route):
        assert np.array_equal(got[b], stack.single(entry, 0)), (case[0], b)


@pytest.mark.parametrize("case", [CASES[0], CASES[4], CASES[6], CASES[7]], ids=[CASES[i][0] for i in (0, 4, 6, 7)])
def test_an_index_outside_the_stack_leaves_its_outputs_alone(gpu, forced_variant, case):
    forced_variant(case[9])
    stack = Stack(case, gpu, 4)
    route = [-1, 2, ENTRIES, 0]
    got = stack.routed(route)
    assert np.all(got[0] == NAN_PATTERN) and np.all(got[2] == NAN_PATTERN)
    assert np.array_equal(got[1], stack.single(2, 1))
    assert np.array_equal(got[3], stack.single(0, 3))


def test_a_captured_launch_follows_the_route_it_finds_at_replay(gpu):
    """The kernel reads the indices, so a HIP graph captured once serves every later routing decision: the
    route is rewritten in place between replays (by device-side work, as a router would)."""
    import torch
    case = CASES[0]
    _, n_out, k, bits, qop, g, m, _, element, _, _ = case
    stack = Stack(case, gpu, 3)
    routes = [[0, 1, 2], [4, 4, 3], [2, 0, 4], [1, 3, 0]]
    route = torch.tensor(routes[0], dtype=torch.int32, device=gpu)
    y = torch.full((3, m, n_out), NAN_PATTERN, dtype=torch.int16, device=gpu)

    def launch():
        mg.device_gemv_routed(stack.w, stack.x, stack.scale, stack.zero, stack.bias, y, route, ENTRIES, 3, n_out, m, k,
                              g, stack.strides(), qop, bits, element=element)

    launch()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            launch()
    torch.cuda.current_stream().wait_stream(side)
    for r in routes:
        route.copy_(torch.tensor(r, dtype=torch.int32, device=gpu))
        y.fill_(NAN_PATTERN)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = y.cpu().numpy().view(np.uint16)
        for b, entry in enumerate(r):
            assert np.array_equal(got[b], stack.single(entry, b)), (r, b)


def test_identity_route_is_the_batched_launch(gpu):
    import torch
    case = CASES[0]
    _, n_out, k, bits, qop, g, m, _, _, _, _ = case
    stack = Stack(case, gpu, ENTRIES)
    got = stack.routed(list(range(ENTRIES)))
    y = torch.full((ENTRIES, m, n_out), NAN_PATTERN, dtype=torch.int16, device=gpu)
    mg.device_gemv(stack.w, stack.x, stack.scale, stack.zero, stack.bias, y, ENTRIES, n_out, m, k, g, qop, bits,
                   batch_strides=stack.strides())
    torch.cuda.synchronize()
    assert np.array_equal(got, y.cpu().numpy().view(np.uint16))
