"""fp32 and complex64 GEMM through the C ABI against the CPU oracle and float64.

Tolerance 1e-4 relative per tensor (fp32; the accumulation order differs from the reference's
lane-strided dot product, matmul_op.mojo:181-199: MFMA sums K in pairs, tile by tile)."""
import numpy as np
import pytest

from conftest import assert_close
from endia_amd import _lib as L
from oracle import endia_ref as R

pytestmark = pytest.mark.gpu


def run_sgemm(dev, A, B, ta, tb, M, N, K, epi=L.EPI_NONE, act=L.OP_IDENTITY, bias=None, aux=None, want_z=False,
              C0=None, batch=1, sA=0, sB=0):
    dA, dB = dev.put(A), dev.put(B)
    dC = dev.put(C0) if C0 is not None else dev.alloc(max(batch * M * N * 4, 4))
    dbias = dev.put(bias) if bias is not None else None
    daux = dev.put(aux) if aux is not None else None
    dz = dev.alloc(max(M * N * 4, 4)) if want_z else None
    lda = A.shape[-1] if A.ndim >= 2 else 1
    ldb = B.shape[-1] if B.ndim >= 2 else 1
    dev.call("endia_hip_sgemm", ta, tb, M, N, K, dA, lda, dB, ldb, dC, N, batch, sA, sB, M * N, epi, act, dbias, daux, dz)
    C = dev.get(dC, (batch, M, N) if batch > 1 else (M, N))
    return (C, dev.get(dz, (M, N))) if want_z else C


SHAPES = [(128, 128, 32), (256, 384, 72), (132, 260, 100), (37, 53, 19), (4, 4, 4), (1, 1, 1), (128, 1, 32),
          (1, 32, 128), (300, 200, 8), (64, 64, 1024), (64, 96, 8192), (128, 200, 5000), (72, 64, 2052),
          (32, 1, 128), (3, 5, 1000), (40, 50, 64), (1, 1, 4096),  # few outputs, long reduction: one work-group per output
          (128, 128, 128), (128, 64, 96), (64, 128, 36), (132, 68, 124), (128, 32, 132)]  # reductions of 1-4 K tiles, and just past


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_sgemm_modes_vs_oracle(dev, M, N, K, ta, tb):
    rng = np.random.default_rng(M * 7 + N * 3 + K + ta * 2 + tb)
    A = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
    B = rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    C = run_sgemm(dev, A, B, ta, tb, M, N, K)
    opA, opB = (A.T if ta else A), (B.T if tb else B)
    assert_close(C, R.matmul(opA, opB), what="vs oracle")
    assert_close(C, opA.astype(np.float64) @ opB.astype(np.float64), what="vs float64")


def _embedded(rng, rows, cols, ld, off):
    """A rows x cols matrix inside a larger host buffer: `off` floats in front, leading dimension ld >= cols, the
    padding filled with large values that a read past an edge would drag into the result."""
    buf = np.full(off + rows * ld + 3, 1.0e6, np.float32)
    view = buf[off:off + rows * ld].reshape(rows, ld)
    view[:, :cols] = rng.standard_normal((rows, cols)).astype(np.float32)
    return buf, view[:, :cols]


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("M,N,K,pad_a,pad_b,off_a,off_b", [
    (30 * 4, 50, 40, 1, 0, 0, 0),     # odd leading dimension of A only (the shapes of the reference's own matmul test, rows x 4)
    (129, 131, 67, 0, 0, 0, 0),       # every extent odd, leading dimensions = extents
    (200, 72, 96, 0, 0, 1, 3),        # aligned shapes, bases 4 and 12 bytes off a 16-byte boundary
    (64, 64, 33, 3, 1, 2, 1),         # one tile, K one past a K tile, padded rows
    (256, 130, 515, 2, 3, 0, 1),      # few tiles and a long reduction: K is split inside the launch
    (1000, 10, 300, 0, 0, 0, 0),      # a classifier head: ten columns
    (70, 300, 9, 1, 1, 1, 1),         # shortest reduction the matrix-core path takes
])
def test_sgemm_unaligned_operands_on_the_matrix_cores(dev, M, N, K, pad_a, pad_b, off_a, off_b, ta, tb):
    """Operands whose base address, leading dimension or extents are not multiples of four floats (the reference's
    matmul takes any view: matmul_op.mojo:93-199) run the MFMA tiles with 4-byte loads. All four forms, every epilogue,
    accumulation, the bias gradient riding along, against the oracle and float64; repeated runs give the same bits."""
    rng = np.random.default_rng(M + 3 * N + 5 * K + 7 * ta + 11 * tb)
    ar, ac = (K, M) if ta else (M, K)
    br, bc = (N, K) if tb else (K, N)
    bufA, A = _embedded(rng, ar, ac, ac + pad_a, off_a)
    bufB, B = _embedded(rng, br, bc, bc + pad_b, off_b)
    B *= 1.0 / np.sqrt(K)
    dA, dB = dev.put(bufA) + 4 * off_a, dev.put(bufB) + 4 * off_b
    lda, ldb = ac + pad_a, bc + pad_b
    opA, opB = (A.T if ta else A), (B.T if tb else B)
    ref64 = opA.astype(np.float64) @ opB.astype(np.float64)
    ref = R.matmul(np.ascontiguousarray(opA), np.ascontiguousarray(opB))

    def run(epi=L.EPI_NONE, act=L.OP_IDENTITY, bias=None, aux=None, C0=None, aux_out=None):
        dC = dev.put(C0) if C0 is not None else dev.alloc(M * N * 4)
        dev.call("endia_hip_sgemm", ta, tb, M, N, K, dA, lda, dB, ldb, dC, N, 1, 0, 0, 0, epi, act,
                 dev.put(bias) if bias is not None else None, dev.put(aux) if aux is not None else None, aux_out)
        return dev.get(dC, (M, N))

    first = run()
    assert_close(first, ref, what="vs oracle")
    assert_close(first, ref64, what="vs float64")
    for _ in range(2):
        np.testing.assert_array_equal(run(), first)
    bias = rng.standard_normal(N).astype(np.float32)
    aux = rng.standard_normal((M, N)).astype(np.float32)
    assert_close(run(L.EPI_BIAS, bias=bias), ref64 + bias, what="bias")
    dz = dev.alloc(M * N * 4)
    assert_close(run(L.EPI_BIAS_ACT, L.OP_TANH, bias=bias, aux_out=dz), np.tanh(ref64 + bias), what="bias + tanh")
    assert_close(dev.get(dz, (M, N)), ref64 + bias, what="stored pre-activation")
    assert_close(run(L.EPI_ACT_GRAD, L.OP_SIN, aux=aux), ref64 * np.cos(aux.astype(np.float64)), what="sin gradient epilogue")
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    assert_close(run(L.EPI_NONE | L.GEMM_ACCUMULATE, C0=C0), C0 + ref64, what="accumulate")
    if not tb and pad_b == 0:  # the column sums of B (a bias gradient) from the same call
        dsum = dev.alloc(N * 4)
        assert_close(run(L.EPI_NONE | L.GEMM_COLSUM_B, aux_out=dsum), ref64, what="product with column sums")
        assert_close(dev.get(dsum, (N,)), B.astype(np.float64).sum(0), what="column sums of B")


@pytest.mark.parametrize("tb", [0, 1])
@pytest.mark.parametrize("M,N,K,pad_a,pad_b", [(4096, 10, 4096, 0, 0), (1000, 7, 1028, 4, 0), (256, 16, 512, 0, 0), (300, 1, 2052, 8, 0),
                                               (2049, 3, 640, 0, 0), (1000, 10, 1028, 0, 4), (520, 13, 4100, 4, 8)])
def test_sgemm_few_output_columns(dev, M, N, K, pad_a, pad_b, tb):
    """A classifier head: at most 16 output columns over a long reduction (matmul_op.mojo:93-199 takes any shape). One pass
    over A with the reduction cut across the waves of a work-group; ragged M and K, padded rows of A, B stored either way
    and, stored [K, N], both without padding (the rows of a piece fetched as one run of memory) and with it, every epilogue
    and accumulation, against the oracle and float64; repeated runs give the same bits."""
    rng = np.random.default_rng(M + 3 * N + 5 * K + tb)
    bufA, A = _embedded(rng, M, K, K + pad_a, 0)
    bufB, B = _embedded(rng, N if tb else K, K if tb else N, (K if tb else N) + pad_b, 0)
    bufB /= np.float32(np.sqrt(K))
    dA, dB = dev.put(bufA), dev.put(bufB)
    opB = B.T if tb else B
    ref64 = A.astype(np.float64) @ opB.astype(np.float64)
    ref = R.matmul(np.ascontiguousarray(A), np.ascontiguousarray(opB))

    def run(epi=L.EPI_NONE, act=L.OP_IDENTITY, bias=None, aux=None, C0=None, aux_out=None):
        dC = dev.put(C0) if C0 is not None else dev.alloc(M * N * 4)
        dev.call("endia_hip_sgemm", 0, tb, M, N, K, dA, K + pad_a, dB, B.shape[1] + pad_b, dC, N, 1, 0, 0, 0, epi, act,
                 dev.put(bias) if bias is not None else None, dev.put(aux) if aux is not None else None, aux_out)
        return dev.get(dC, (M, N))

    first = run()
    assert_close(first, ref, what="vs oracle")
    assert_close(first, ref64, what="vs float64")
    for _ in range(2):
        np.testing.assert_array_equal(run(), first)
    bias = rng.standard_normal(N).astype(np.float32)
    aux = rng.standard_normal((M, N)).astype(np.float32)
    assert_close(run(L.EPI_BIAS, bias=bias), ref64 + bias, what="bias")
    dz = dev.alloc(M * N * 4)
    assert_close(run(L.EPI_BIAS_ACT, L.OP_TANH, bias=bias, aux_out=dz), np.tanh(ref64 + bias), what="bias + tanh")
    assert_close(dev.get(dz, (M, N)), ref64 + bias, what="stored pre-activation")
    assert_close(run(L.EPI_ACT_GRAD, L.OP_SIN, aux=aux), ref64 * np.cos(aux.astype(np.float64)), what="sin gradient epilogue")
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    assert_close(run(L.EPI_NONE | L.GEMM_ACCUMULATE, C0=C0), C0 + ref64, what="accumulate")


def _grouped(dev, members):
    """members: dicts with ta, tb, A, B (host arrays as stored), optional bias, C0 (accumulate). Runs them through
    endia_hip_sgemm_grouped and returns the outputs."""
    import ctypes
    descs = (L.SgemmDesc * len(members))()
    outs = []
    for d, m in zip(descs, members):
        A, B, ta, tb = m["A"], m["B"], m["ta"], m["tb"]
        M, K = (A.shape[1], A.shape[0]) if ta else A.shape
        N = B.shape[0] if tb else B.shape[1]
        dC = dev.put(m["C0"]) if m.get("C0") is not None else dev.alloc(max(M * N * 4, 4))
        d.transA, d.transB, d.M, d.N, d.K = ta, tb, M, N, K
        d.A, d.lda, d.B, d.ldb, d.C, d.ldc = dev.put(A), A.shape[1], dev.put(B), B.shape[1], dC, N
        d.epilogue = (L.EPI_BIAS if m.get("bias") is not None else L.EPI_NONE) | (L.GEMM_ACCUMULATE if m.get("C0") is not None else 0)
        d.bias = dev.put(m["bias"]) if m.get("bias") is not None else None
        outs.append((dC, (M, N)))
    dev.call("endia_hip_sgemm_grouped", len(members), descs, -1, None)
    return [dev.get(p, shape) for p, shape in outs]


def _member(rng, ta, tb, M, N, K, bias=False, acc=False):
    m = {"ta": ta, "tb": tb, "A": rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32),
         "B": (rng.standard_normal((N, K) if tb else (K, N)) / np.sqrt(K)).astype(np.float32)}
    if bias:
        m["bias"] = rng.standard_normal(N).astype(np.float32)
    if acc:
        m["C0"] = rng.standard_normal((M, N)).astype(np.float32)
    return m


def _member_ref(m):
    opA, opB = (m["A"].T if m["ta"] else m["A"]), (m["B"].T if m["tb"] else m["B"])
    ref = opA.astype(np.float64) @ opB.astype(np.float64)
    if m.get("bias") is not None:
        ref = ref + m["bias"]
    if m.get("C0") is not None:
        ref = ref + m["C0"]
    return ref


@pytest.mark.parametrize("case", ["four_forms", "two_wide", "mixed_lengths", "ragged", "leftovers", "small_and_odd"])
def test_sgemm_grouped(dev, case):
    """endia_hip_sgemm_grouped: independent products that share one launch of the 256 x 128 tile (one tile per CU), in
    every transpose form, with the bias epilogue and accumulation, ragged edges, members of different reduction lengths,
    and members that no shared launch takes (they run as endia_hip_sgemm would run them). Against float64 and, bit for
    bit, against a second run."""
    rng = np.random.default_rng(len(case))
    if case == "four_forms":      # 4 x 64 tiles = one per CU, all four forms, one with bias, one accumulating
        ms = [_member(rng, 0, 0, 1024, 2048, 512, bias=True), _member(rng, 0, 1, 1024, 2048, 512), _member(rng, 1, 0, 1024, 2048, 512, acc=True),
              _member(rng, 1, 1, 1024, 2048, 512)]
    elif case == "two_wide":      # 2 x 128 tiles
        ms = [_member(rng, 1, 0, 2048, 2048, 256), _member(rng, 0, 0, 2048, 2048, 256, acc=True, bias=True)]
    elif case == "mixed_lengths":  # 2 x 64 long tiles and 2 x 128 tiles half as long: the short ones fill in behind
        ms = [_member(rng, 1, 0, 2048, 2048, 256), _member(rng, 0, 1, 1024, 2048, 512), _member(rng, 0, 0, 2048, 2048, 256),
              _member(rng, 0, 0, 1024, 2048, 512, bias=True)]
    elif case == "ragged":        # extents that are not multiples of the tile or of the K tile
        ms = [_member(rng, 0, 0, 1000, 2040, 500), _member(rng, 0, 1, 1020, 2000, 516, acc=True), _member(rng, 1, 0, 1016, 1944, 260),
              _member(rng, 1, 1, 1024, 2048, 300, bias=True)]
    elif case == "leftovers":     # five equal members: four share a launch, the fifth runs alone
        ms = [_member(rng, i % 2, 0, 1024, 2048, 512, acc=(i == 4)) for i in range(5)]
    else:                          # nothing here fits the shared launch: too small, unaligned, too short a reduction
        ms = [_member(rng, 0, 0, 64, 64, 64), _member(rng, 0, 1, 129, 131, 67, bias=True), _member(rng, 1, 0, 1024, 2048, 128),
              _member(rng, 0, 0, 4, 4, 4, acc=True)]
    got = _grouped(dev, ms)
    for k, (c, m) in enumerate(zip(got, ms)):
        assert_close(c, _member_ref(m), what="%s member %d" % (case, k))
    again = _grouped(dev, ms)
    for a, b in zip(got, again):
        np.testing.assert_array_equal(a, b)
    with pytest.raises(L.EndiaHipError):  # an epilogue the grouped call does not take
        ms[0]["bias"] = None
        descs = (L.SgemmDesc * 1)()
        descs[0].epilogue = L.EPI_ACT_GRAD
        dev.call("endia_hip_sgemm_grouped", 1, descs, -1, None)


def test_sgemm_grouped_runs_what_is_needed_and_its_company(dev):
    """need = i: member i runs together with the members that make its launch a better one, the others are left to
    the caller (their outputs untouched), and `launched` says which is which. Three products of 1024 x 2048 x 512 and
    two of 2048 x 2048 x 256 are offered; whatever subset runs, a second call with need = -1 finishes the job."""
    import ctypes
    rng = np.random.default_rng(3)
    ms = [_member(rng, 0, 0, 1024, 2048, 512), _member(rng, 1, 0, 2048, 2048, 256), _member(rng, 0, 1, 1024, 2048, 512),
          _member(rng, 1, 0, 2048, 2048, 256), _member(rng, 0, 0, 1024, 2048, 512), _member(rng, 0, 0, 8, 8, 8)]
    descs = (L.SgemmDesc * len(ms))()
    outs = []
    for d, m in zip(descs, ms):
        A, B, ta, tb = m["A"], m["B"], m["ta"], m["tb"]
        M, K = (A.shape[1], A.shape[0]) if ta else A.shape
        N = B.shape[0] if tb else B.shape[1]
        dC = dev.put(np.full((M, N), -7.0, np.float32))
        d.transA, d.transB, d.M, d.N, d.K = ta, tb, M, N, K
        d.A, d.lda, d.B, d.ldb, d.C, d.ldc, d.epilogue, d.bias = dev.put(A), A.shape[1], dev.put(B), B.shape[1], dC, N, L.EPI_NONE, None
        outs.append((dC, (M, N)))
    done = (ctypes.c_int32 * len(ms))()
    dev.call("endia_hip_sgemm_grouped", len(ms), descs, 2, done)
    flags = list(done)
    assert flags[2] == 1 and flags[5] == 0, flags      # the needed member ran; the tiny one shares no launch and was not needed
    assert sum(flags) >= 2, flags                      # and it found company
    for k, ((p, shape), m) in enumerate(zip(outs, ms)):
        got = dev.get(p, shape)
        if flags[k]:
            assert_close(got, _member_ref(m), what="member %d (launched)" % k)
        else:
            assert np.all(got == -7.0), "member %d was reported as not launched but its output changed" % k
    rest = [k for k in range(len(ms)) if not flags[k]]
    sub = (L.SgemmDesc * len(rest))(*[descs[k] for k in rest])
    dev.call("endia_hip_sgemm_grouped", len(rest), sub, -1, None)
    for k, ((p, shape), m) in enumerate(zip(outs, ms)):
        assert_close(dev.get(p, shape), _member_ref(m), what="member %d" % k)
    with pytest.raises(L.EndiaHipError):
        dev.call("endia_hip_sgemm_grouped", len(ms), descs, len(ms), done)


def test_sgemm_few_outputs_batched_accumulate(dev):
    """The one-group-per-output kernel with a batch, a broadcast operand and accumulation into C."""
    rng = np.random.default_rng(77)
    M, N, K, batch = 4, 6, 300, 3
    A = rng.standard_normal((batch, K, M)).astype(np.float32)   # used transposed
    B = rng.standard_normal((K, N)).astype(np.float32)          # shared by the batch
    C0 = rng.standard_normal((batch, M, N)).astype(np.float32)
    dA, dB, dC = dev.put(A), dev.put(B), dev.put(C0)
    dev.call("endia_hip_sgemm", 1, 0, M, N, K, dA, M, dB, N, dC, N, batch, K * M, 0, M * N, L.EPI_NONE | L.GEMM_ACCUMULATE,
             L.OP_IDENTITY, None, None, None)
    want = C0 + np.einsum("bkm,kn->bmn", A.astype(np.float64), B.astype(np.float64))
    assert_close(dev.get(dC, (batch, M, N)), want, what="batched accumulate")


def test_sgemm_golden(dev, golden):
    g = golden("matmul")
    a, b = g["a"], g["b"]
    # (2,30,40) @ (40,50): batch of 2 with a broadcast right operand (batch stride 0)
    C = run_sgemm(dev, a, b, 0, 0, 30, 50, 40, batch=2, sA=30 * 40, sB=0)
    assert_close(C, g["out"], what="batched forward")
    # the square VJP pair: dA = G B^T (NT), dB = A^T G (TN)
    assert_close(run_sgemm(dev, g["sg"], g["sb"], 0, 1, 64, 64, 64), g["dsa"], what="dA")
    assert_close(run_sgemm(dev, g["sa"], g["sg"], 1, 0, 64, 64, 64), g["dsb"], what="dB")


@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (50, 30, 7), (130, 70, 36),
                                   (128, 32, 1), (128, 1, 32), (40, 50, 3), (16, 8, 100), (128, 64, 128)])  # thin K, few outputs, short K
@pytest.mark.parametrize("act", ["relu", "tanh", "sin", "identity"])
def test_sgemm_epilogues(dev, M, N, K, act):
    rng = np.random.default_rng(5)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    aux = rng.standard_normal((M, N)).astype(np.float32)
    code = {"relu": L.OP_RELU, "tanh": L.OP_TANH, "sin": L.OP_SIN, "identity": L.OP_IDENTITY}[act]
    z_ref = R.binary("add", R.matmul(A, B), bias)
    # x @ W + b
    assert_close(run_sgemm(dev, A, B, 0, 0, M, N, K, L.EPI_BIAS, L.OP_IDENTITY, bias=bias), z_ref, what="bias")
    # act(x @ W + b), also storing the pre-activation
    C, Z = run_sgemm(dev, A, B, 0, 0, M, N, K, L.EPI_BIAS_ACT, code, bias=bias, want_z=True)
    assert_close(Z, z_ref, what="stored pre-activation")
    assert_close(C, R.unary(act, z_ref), what="bias+act")
    # (dZ W^T) * act'(aux) with aux = pre-activation
    g_ref = R.unary_vjp(act, aux, R.matmul(A, B))
    assert_close(run_sgemm(dev, A, B, 0, 0, M, N, K, L.EPI_ACT_GRAD, code, aux=aux), g_ref, what="act grad from input")
    if act in ("relu", "tanh"):
        out = R.unary(act, aux)
        assert_close(run_sgemm(dev, A, B, 0, 0, M, N, K, L.EPI_ACT_GRAD, code | L.ACT_FROM_OUTPUT, aux=out), g_ref,
                     what="act grad from output")
    # accumulate into C
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    assert_close(run_sgemm(dev, A, B, 0, 0, M, N, K, L.EPI_NONE | L.GEMM_ACCUMULATE, C0=C0),
                 C0 + R.matmul(A, B), what="accumulate")


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0)])
@pytest.mark.parametrize("M,N,K", [(512, 512, 512), (256, 192, 1000), (64, 64, 4096), (128, 256, 260), (1024, 1024, 512),
                                   (200, 136, 768)])
def test_sgemm_reduction_split_inside_the_launch(dev, M, N, K, ta, tb):
    """Products with few tiles per CU and K >= 256: K is cut into slices whose partial sums the last group of each
    tile adds up. Every epilogue, accumulation and a padded C go through that path; results repeat bit for bit."""
    rng = np.random.default_rng(M + 3 * N + 7 * K + ta + 2 * tb)
    A = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
    B = (rng.standard_normal((N, K) if tb else (K, N)) / np.sqrt(K)).astype(np.float32)
    opA, opB = (A.T if ta else A), (B.T if tb else B)
    ref = opA.astype(np.float64) @ opB.astype(np.float64)
    first = run_sgemm(dev, A, B, ta, tb, M, N, K)
    assert_close(first, R.matmul(opA, opB), what="vs oracle")
    assert_close(first, ref, what="vs float64")
    for _ in range(3):  # the arrival counters are back at zero after every launch, and the order of the sum is fixed
        np.testing.assert_array_equal(run_sgemm(dev, A, B, ta, tb, M, N, K), first)
    bias = rng.standard_normal(N).astype(np.float32)
    aux = rng.standard_normal((M, N)).astype(np.float32)
    C, Z = run_sgemm(dev, A, B, ta, tb, M, N, K, L.EPI_BIAS_ACT, L.OP_TANH, bias=bias, want_z=True)
    assert_close(Z, ref + bias, what="stored pre-activation")
    assert_close(C, np.tanh(ref + bias), what="bias + tanh")
    assert_close(run_sgemm(dev, A, B, ta, tb, M, N, K, L.EPI_ACT_GRAD, L.OP_RELU, aux=aux), ref * (aux > 0), what="relu gradient")
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    assert_close(run_sgemm(dev, A, B, ta, tb, M, N, K, L.EPI_NONE | L.GEMM_ACCUMULATE, C0=C0), C0 + ref, what="accumulate")
    # C with a leading dimension larger than N: the columns past N keep their contents
    ldc = N + 12
    wide = rng.standard_normal((M, ldc)).astype(np.float32)
    dA, dB, dC = dev.put(A), dev.put(B), dev.put(wide)
    dev.call("endia_hip_sgemm", ta, tb, M, N, K, dA, A.shape[1], dB, B.shape[1], dC, ldc, 1, 0, 0, 0, L.EPI_BIAS, L.OP_IDENTITY,
             dev.put(bias), None, None)
    got = dev.get(dC, (M, ldc))
    assert_close(got[:, :N], ref + bias, what="padded C")
    np.testing.assert_array_equal(got[:, N:], wide[:, N:])


def test_sgemm_edge_cases(dev):
    A = np.ones((4, 4), np.float32)
    # K = 0: the empty sum
    C = run_sgemm(dev, np.zeros((4, 0), np.float32), np.zeros((0, 4), np.float32), 0, 0, 4, 4, 0,
                  C0=np.full((4, 4), 7, np.float32))
    np.testing.assert_array_equal(C, np.zeros((4, 4), np.float32))
    # M = 0 / N = 0: nothing to do, no error
    dev.call("endia_hip_sgemm", 0, 0, 0, 4, 4, None, 4, None, 4, None, 4, 1, 0, 0, 0, 0, L.OP_IDENTITY, None, None, None)
    # errors are reported, not executed
    lib = L.lib()
    dA = dev.put(A)
    assert lib.endia_hip_sgemm(0, 0, 4, 4, 4, dA, 2, dA, 4, dA, 4, 1, 0, 0, 0, 0, L.OP_IDENTITY, None, None, None) == L.ERR_INVALID
    assert b"leading dimension" in lib.endia_hip_last_error()
    assert lib.endia_hip_sgemm(0, 0, 4, 4, 4, None, 4, dA, 4, dA, 4, 1, 0, 0, 0, 0, L.OP_IDENTITY, None, None, None) == L.ERR_INVALID
    assert lib.endia_hip_sgemm(0, 0, -1, 4, 4, dA, 4, dA, 4, dA, 4, 1, 0, 0, 0, 0, L.OP_IDENTITY, None, None, None) == L.ERR_INVALID
    assert lib.endia_hip_sgemm(0, 0, 4, 4, 4, dA, 4, dA, 4, dA, 4, 1, 0, 0, 0, L.EPI_BIAS, L.OP_IDENTITY, None, None, None) == L.ERR_INVALID
    assert lib.endia_hip_sgemm(0, 0, 4, 4, 4, dA, 4, dA, 4, dA, 4, 1, 0, 0, 0, 0, L.OP_COS, None, None, None) == L.ERR_INVALID


def test_sgemm_unaligned_views(dev):
    # operands that start in the middle of a buffer with odd leading dimensions take the unaligned path
    rng = np.random.default_rng(9)
    big = rng.standard_normal((70, 67)).astype(np.float32)
    dbig = dev.put(big)
    A = big[3:3 + 40, 5:5 + 33]
    B = rng.standard_normal((33, 21)).astype(np.float32)
    dB = dev.put(B)
    dC = dev.alloc(40 * 21 * 4)
    dev.call("endia_hip_sgemm", 0, 0, 40, 21, 33, dbig + 4 * (3 * 67 + 5), 67, dB, 21, dC, 21, 1, 0, 0, 0, 0,
             L.OP_IDENTITY, None, None, None)
    assert_close(dev.get(dC, (40, 21)), R.matmul(A, B), what="strided view")


@pytest.mark.parametrize("algo,tol", [(L.CGEMM_4M, 1e-4), (L.CGEMM_3M, 1e-4)])
@pytest.mark.parametrize("ta,ca,tb,cb", [(0, 0, 0, 0), (0, 0, 1, 0), (1, 0, 0, 0), (0, 0, 1, 1), (1, 1, 0, 0)])
def test_cgemm(dev, algo, tol, ta, ca, tb, cb):
    rng = np.random.default_rng(11)
    M, N, K = 96, 72, 40
    A = (rng.standard_normal((K, M) if ta else (M, K)) + 1j * rng.standard_normal((K, M) if ta else (M, K))).astype(np.complex64)
    B = (rng.standard_normal((N, K) if tb else (K, N)) + 1j * rng.standard_normal((N, K) if tb else (K, N))).astype(np.complex64)
    dA, dB, dC = dev.put(A), dev.put(B), dev.alloc(M * N * 8)
    dev.call("endia_hip_cgemm", ta, ca, tb, cb, M, N, K, dA, A.shape[1], dB, B.shape[1], dC, N, 1, 0, 0, 0, algo, 0)
    C = dev.get(dC, (M, N), np.complex64)
    opA = (A.T if ta else A)
    opB = (B.T if tb else B)
    opA = np.conj(opA) if ca else opA
    opB = np.conj(opB) if cb else opB
    assert_close(C, R.matmul(opA, opB), tol, what="vs oracle")
    assert_close(C, opA.astype(np.complex128) @ opB.astype(np.complex128), tol, what="vs complex128")


def test_cgemm_golden_and_accumulate(dev, golden):
    g = golden("matmul")
    ca, cb = g["ca"], g["cb"]
    dA, dB, dC = dev.put(ca), dev.put(cb), dev.alloc(2 * 30 * 50 * 8)
    dev.call("endia_hip_cgemm", 0, 0, 0, 0, 30, 50, 40, dA, 40, dB, 50, dC, 50, 2, 30 * 40, 0, 30 * 50, L.CGEMM_4M, 0)
    out = dev.get(dC, (2, 30, 50), np.complex64)
    assert_close(out, g["cout"], what="complex batched forward")
    dev.call("endia_hip_cgemm", 0, 0, 0, 0, 30, 50, 40, dA, 40, dB, 50, dC, 50, 2, 30 * 40, 0, 30 * 50, L.CGEMM_4M, 1)
    assert_close(dev.get(dC, (2, 30, 50), np.complex64), 2 * g["cout"], what="accumulate")


def test_sgemm_large_properties(dev):
    """Full-size check (4096^3, the wide-MLP shape) through properties that need no CPU GEMM:
    linearity in A, and agreement of row/column probes with float64 dot products."""
    rng = np.random.default_rng(21)
    n = 4096
    A = rng.standard_normal((n, n)).astype(np.float32)
    B = (rng.standard_normal((n, n)) / 64).astype(np.float32)
    for ta, tb in [(0, 0), (0, 1), (1, 0)]:
        C = run_sgemm(dev, A, B, ta, tb, n, n, n)
        opA, opB = (A.T if ta else A), (B.T if tb else B)
        rows = [0, 1, 127, 128, 2049, 4095]
        cols = [0, 31, 32, 1000, 4095]
        ref = opA[rows].astype(np.float64) @ opB[:, cols].astype(np.float64)
        assert_close(C[np.ix_(rows, cols)], ref, what="probes ta=%d tb=%d" % (ta, tb))
        # checksum of checksums: 1^T C 1 = (1^T A)(B 1)
        total = opA.astype(np.float64).sum(0) @ opB.astype(np.float64).sum(1)
        got = C.astype(np.float64).sum()
        assert abs(got - total) <= 1e-4 * np.abs(opA).astype(np.float64).sum(0) @ np.abs(opB).astype(np.float64).sum(1)
        dev.release()


@pytest.mark.parametrize("algo", [L.CGEMM_4M, L.CGEMM_3M])
@pytest.mark.parametrize("M,N,K,pad", [(96, 72, 40, 0), (64, 128, 64, 4), (33, 21, 17, 3)])
def test_cgemm_all_flag_combinations(dev, algo, M, N, K, pad):
    """Every transpose / conjugate combination, leading dimensions larger than the rows, accumulation into C,
    sizes that take the aligned MFMA path and sizes that take the unaligned one."""
    rng = np.random.default_rng(M + N + K)

    def cplx(*shape):
        return (rng.standard_normal(shape) + 1j * rng.standard_normal(shape)).astype(np.complex64)

    for ta in (0, 1):
        for ca in (0, 1):
            for tb in (0, 1):
                for cb in (0, 1):
                    a_shape = (K, M) if ta else (M, K)
                    b_shape = (N, K) if tb else (K, N)
                    Ap, Bp, Cp = cplx(a_shape[0], a_shape[1] + pad), cplx(b_shape[0], b_shape[1] + pad), cplx(M, N + pad)
                    A, B, C0 = Ap[:, :a_shape[1]], Bp[:, :b_shape[1]], Cp[:, :N]
                    dA, dB, dC = dev.put(Ap), dev.put(Bp), dev.put(Cp)
                    opA = np.conj(A.T if ta else A) if ca else (A.T if ta else A)
                    opB = np.conj(B.T if tb else B) if cb else (B.T if tb else B)
                    want = opA.astype(np.complex128) @ opB.astype(np.complex128)
                    dev.call("endia_hip_cgemm", ta, ca, tb, cb, M, N, K, dA, Ap.shape[1], dB, Bp.shape[1], dC, N + pad,
                             1, 0, 0, 0, algo, 1)
                    got = dev.get(dC, Cp.shape, np.complex64)
                    what = "ta=%d ca=%d tb=%d cb=%d" % (ta, ca, tb, cb)
                    assert_close(got[:, :N], want + C0, what=what)
                    np.testing.assert_array_equal(got[:, N:], Cp[:, N:], err_msg=what + ": padding columns of C touched")
                    dev.release()


@pytest.mark.parametrize("M,N,K", [(128, 128, 128), (64, 96, 40), (256, 384, 520), (32, 1, 128), (3, 5, 1000), (128, 200, 5000),
                                   (37, 53, 19), (64, 64, 4096)])
def test_sgemm_colsum_b(dev, M, N, K):
    """ENDIA_GEMM_COLSUM_B: C = A^T B as before, and aux_out[n] = sum_k B[k][n] from the same call, whichever
    kernel the shape selects (fused in the MFMA kernels, a separate reduction on the other paths and under split-K)."""
    rng = np.random.default_rng(M + N + K)
    A = rng.standard_normal((K, M)).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    dA, dB = dev.put(A), dev.put(B)
    dC, dsum = dev.put(np.full((M, N), np.nan, np.float32)), dev.put(np.full(N, np.nan, np.float32))
    dev.call("endia_hip_sgemm", 1, 0, M, N, K, dA, M, dB, N, dC, N, 1, 0, 0, 0, L.EPI_NONE | L.GEMM_COLSUM_B, L.OP_IDENTITY,
             None, None, dsum)
    assert_close(dev.get(dC, (M, N)), A.astype(np.float64).T @ B.astype(np.float64), what="C")
    assert_close(dev.get(dsum, (N,)), B.astype(np.float64).sum(0), tol=1e-5, what="column sums")
    assert_close(dev.get(dsum, (N,)), R.reduce_add(B, [0]).reshape(-1), tol=1e-5, what="column sums vs oracle")
    for bad in [(1, 1), (0, 0)]:   # transB = 1, or a fused epilogue, is refused
        with pytest.raises(L.EndiaHipError):
            dev.call("endia_hip_sgemm", 1, bad[0], M, N, K, dA, M, dB, N if not bad[0] else K, dC, N, 1, 0, 0, 0,
                     (L.EPI_NONE if bad[0] else L.EPI_BIAS) | L.GEMM_COLSUM_B, L.OP_IDENTITY, dsum, None, dsum)


@pytest.mark.parametrize("B,K,N", [(128, 128, 128), (128, 32, 64), (128, 64, 32), (64, 128, 96), (8, 4, 8), (128, 128, 132),
                                   (256, 64, 64), (128, 1, 32), (128, 30, 64), (100, 36, 20)])
@pytest.mark.parametrize("act", ["relu", "tanh", "none"])
def test_linear_bwd(dev, B, K, N, act):
    """endia_hip_linear_bwd against float64 for layers that take the one-launch path (B, N <= 128, aligned) and for
    ones that do not (large, unaligned, 1-wide): dx = (g W^T) * act'(aux), dW = x^T g, db = column sums of g;
    also with outputs left out."""
    rng = np.random.default_rng(B * 5 + K * 3 + N + len(act))
    x = rng.standard_normal((B, K)).astype(np.float32)
    W = rng.standard_normal((K, N)).astype(np.float32)
    g = rng.standard_normal((B, N)).astype(np.float32)
    aux = np.maximum(x, 0) if act == "relu" else np.tanh(x).astype(np.float32)   # the layer below's stored OUTPUT
    dmask = {"relu": (aux > 0).astype(np.float64), "tanh": 1 - aux.astype(np.float64) ** 2, "none": 1.0}[act]
    want_dx = (g.astype(np.float64) @ W.astype(np.float64).T) * dmask
    want_dW = x.astype(np.float64).T @ g.astype(np.float64)
    want_db = g.astype(np.float64).sum(0)
    flags = {"relu": L.OP_RELU | L.ACT_FROM_OUTPUT, "tanh": L.OP_TANH | L.ACT_FROM_OUTPUT, "none": L.OP_IDENTITY}[act]
    dxp, dWp, dbp = (dev.put(np.full(s, np.nan, np.float32)) for s in ((B, K), (K, N), (N,)))
    px, pW, pg, paux = dev.put(x), dev.put(W), dev.put(g), dev.put(aux)
    dev.call("endia_hip_linear_bwd", B, K, N, px, pW, pg, flags, paux if act != "none" else None, dxp, dWp, dbp)
    assert_close(dev.get(dxp, (B, K)), want_dx, what="dx")
    assert_close(dev.get(dWp, (K, N)), want_dW, what="dW")
    assert_close(dev.get(dbp, (N,)), want_db, tol=1e-5, what="db")
    # outputs left out: only dW and db (first layer of a model), only dx
    dW2, db2, dx2 = (dev.put(np.full(s, np.nan, np.float32)) for s in ((K, N), (N,), (B, K)))
    dev.call("endia_hip_linear_bwd", B, K, N, px, pW, pg, L.OP_IDENTITY, None, None, dW2, db2)
    assert_close(dev.get(dW2, (K, N)), want_dW, what="dW alone")
    assert_close(dev.get(db2, (N,)), want_db, tol=1e-5, what="db alone")
    dev.call("endia_hip_linear_bwd", B, K, N, px, pW, pg, flags, paux if act != "none" else None, dx2, None, None)
    assert_close(dev.get(dx2, (B, K)), want_dx, what="dx alone")


def test_sgemm_random_shapes_and_flags(dev):
    """Seeded sweep over the dispatch boundaries (tiled / short-reduction / few-outputs / thin-K / generic kernels,
    aligned and unaligned extents, every transpose and epilogue, accumulate, column sums): 240 cases against float64."""
    rng = np.random.default_rng(2024)
    picks = [1, 2, 3, 4, 5, 8, 16, 31, 32, 33, 63, 64, 65, 96, 127, 128, 129, 132, 200, 256, 260]
    for case in range(240):
        M, N = (int(rng.choice(picks)) for _ in range(2))
        K = int(rng.choice([0, 1, 2, 4, 5, 8, 16, 28, 32, 36, 64, 100, 128, 132, 256, 515, 1024]))
        if case % 3 == 0:  # favour the aligned, vectorised paths
            M, N, K = (max(4, v // 4 * 4) for v in (M, N, max(K, 4)))
        ta, tb = int(rng.integers(2)), int(rng.integers(2))
        epi = int(rng.choice([L.EPI_NONE, L.EPI_NONE, L.EPI_BIAS, L.EPI_BIAS_ACT, L.EPI_ACT_GRAD]))
        act = int(rng.choice([L.OP_RELU, L.OP_TANH, L.OP_SIN, L.OP_IDENTITY]))
        accumulate = epi == L.EPI_NONE and case % 5 == 0
        colsum = epi == L.EPI_NONE and not tb and not accumulate and case % 2 == 0
        A = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
        B = rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
        bias = rng.standard_normal(N).astype(np.float32)
        aux = rng.standard_normal((M, N)).astype(np.float32)
        C0 = rng.standard_normal((M, N)).astype(np.float32)
        opA = (A.T if ta else A).astype(np.float64)
        opB = (B.T if tb else B).astype(np.float64)
        want = opA @ opB
        if epi in (L.EPI_BIAS, L.EPI_BIAS_ACT):
            want = want + bias
        if epi == L.EPI_BIAS_ACT:
            want = {L.OP_RELU: lambda z: np.maximum(z, 0), L.OP_TANH: np.tanh, L.OP_SIN: np.sin, L.OP_IDENTITY: lambda z: z}[act](want)
        if epi == L.EPI_ACT_GRAD:
            a64 = aux.astype(np.float64)
            want = want * {L.OP_RELU: (a64 > 0) * 1.0, L.OP_TANH: 1 - np.tanh(a64) ** 2, L.OP_SIN: np.cos(a64), L.OP_IDENTITY: 1.0}[act]
        if accumulate:
            want = want + C0
        dA, dB, dC = dev.put(A), dev.put(B), dev.put(C0)
        dsum = dev.put(np.full(max(N, 1), np.nan, np.float32))
        flags = epi | (L.GEMM_ACCUMULATE if accumulate else 0) | (L.GEMM_COLSUM_B if colsum else 0)
        dev.call("endia_hip_sgemm", ta, tb, M, N, K, dA, M if ta else max(K, 1), dB, K if tb and K else (max(K, 1) if tb else N), dC, N,
                 1, 0, 0, 0, flags, act, dev.put(bias) if epi in (L.EPI_BIAS, L.EPI_BIAS_ACT) else None,
                 dev.put(aux) if epi == L.EPI_ACT_GRAD else None, dsum if colsum else None)
        what = "case %d: M=%d N=%d K=%d ta=%d tb=%d epi=%d act=%d acc=%d colsum=%d" % (case, M, N, K, ta, tb, epi, act, accumulate, colsum)
        got = dev.get(dC, (M, N))
        scale = max(float(np.abs(want).max()), 1e-30)
        assert np.abs(got - want).max() <= 2e-5 * scale * max(1.0, np.sqrt(K)), what
        if colsum:
            s = dev.get(dsum, (N,))
            assert np.abs(s - B.astype(np.float64).sum(0)).max() <= 2e-5 * max(1.0, np.sqrt(K)) * max(1.0, float(np.abs(B).max()) if K else 1.0), what + " (column sums)"
        dev.release()


@pytest.mark.parametrize("M,N,K", [(256, 256, 32), (256, 512, 64), (300, 520, 70), (516, 260, 1000), (1024, 768, 4100), (260, 1028, 36),
                                   (128, 64, 512), (512, 1024, 1100), (256, 256, 31), (320, 256, 97)])
def test_sgemm_every_tile_forced(dev, M, N, K):
    """endia_hip_gemm_force_tile: the weight-gradient form (A stored K x M, B stored K x N) through the 64, 128, 256 x 256
    and 256 x 128 tiles on shapes with ragged edges in M, N and K (the two one-wave-per-SIMD tiles are otherwise only
    chosen for products that fill every CU with one): every tile against the oracle and float64, plain and accumulating,
    a padded C, a batch; all four forms and every fused epilogue (also sin with the stored pre-activation, and cos as its
    gradient, the Hessian-vector benchmark's epilogues) through the 128, 256 x 256 and 256 x 128 tiles."""
    rng = np.random.default_rng(M + 3 * N + 7 * K)
    A = rng.standard_normal((K, M)).astype(np.float32)
    B = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32)
    ref = A.T.astype(np.float64) @ B.astype(np.float64)
    want = R.matmul(np.ascontiguousarray(A.T), B)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    try:
        for tile in (64, 128, 256, 256128):
            dev.call("endia_hip_gemm_force_tile", tile)
            got = run_sgemm(dev, A, B, 1, 0, M, N, K)
            assert_close(got, want, what="tile %d vs oracle" % tile)
            assert_close(got, ref, what="tile %d vs float64" % tile)
            np.testing.assert_array_equal(run_sgemm(dev, A, B, 1, 0, M, N, K), got)
            assert_close(run_sgemm(dev, A, B, 1, 0, M, N, K, L.EPI_NONE | L.GEMM_ACCUMULATE, C0=C0), C0 + ref, what="tile %d accumulate" % tile)
            ldc = N + 12
            wide = rng.standard_normal((M, ldc)).astype(np.float32)
            dA, dB, dC = dev.put(A), dev.put(B), dev.put(wide)
            dev.call("endia_hip_sgemm", 1, 0, M, N, K, dA, M, dB, N, dC, ldc, 1, 0, 0, 0, L.EPI_NONE, L.OP_IDENTITY, None, None, None)
            out = dev.get(dC, (M, ldc))
            assert_close(out[:, :N], ref, what="tile %d padded C" % tile)
            np.testing.assert_array_equal(out[:, N:], wide[:, N:])
        # a batch of two through the 256 tile (second entry: the operands swapped in sign), and the other forms untouched
        A2, B2 = np.stack([A, -A]), np.stack([B, B])
        dA, dB, dC = dev.put(A2), dev.put(B2), dev.put(np.zeros((2, M, N), np.float32))
        dev.call("endia_hip_sgemm", 1, 0, M, N, K, dA, M, dB, N, dC, N, 2, K * M, K * N, M * N, L.EPI_NONE, L.OP_IDENTITY, None, None, None)
        out = dev.get(dC, (2, M, N))
        assert_close(out[0], ref, what="batch entry 0")
        assert_close(out[1], -ref, what="batch entry 1")
        # all forms and the fused epilogues through the 128 and 256 tiles (tiles inside the matrix take bodies of their own)
        At, Bt = np.ascontiguousarray(A.T), np.ascontiguousarray(B.T)
        bias = rng.standard_normal(N).astype(np.float32)
        aux = rng.standard_normal((M, N)).astype(np.float32)
        for tile, ta, tb, a, b in [(t,) + f for t in (128, 256, 256128) for f in ((0, 0, At, B), (0, 1, At, Bt), (1, 1, A, Bt), (1, 0, A, B))]:
            if K % 4 and (not ta or tb):
                continue  # a K-major operand needs K in whole 16-byte pieces for the matrix-core path
            dev.call("endia_hip_gemm_force_tile", tile)
            what = "form (%d, %d) on the %d tile: " % (ta, tb, tile)
            assert_close(run_sgemm(dev, a, b, ta, tb, M, N, K), ref, what=what + "plain")
            assert_close(run_sgemm(dev, a, b, ta, tb, M, N, K, L.EPI_BIAS, bias=bias), ref + bias, what=what + "bias")
            Cz, Z = run_sgemm(dev, a, b, ta, tb, M, N, K, L.EPI_BIAS_ACT, L.OP_TANH, bias=bias, want_z=True)
            assert_close(Z, ref + bias, what=what + "stored pre-activation")
            assert_close(Cz, np.tanh(ref + bias), what=what + "bias + tanh")
            assert_close(run_sgemm(dev, a, b, ta, tb, M, N, K, L.EPI_ACT_GRAD, L.OP_RELU, aux=aux), ref * (aux > 0), what=what + "relu gradient")
            assert_close(run_sgemm(dev, a, b, ta, tb, M, N, K, L.EPI_ACT_GRAD, L.OP_TANH | L.ACT_FROM_OUTPUT, aux=np.tanh(aux)),
                         ref * (1 - np.tanh(aux.astype(np.float64)) ** 2), what=what + "tanh gradient from the output")
            Cs, Zs = run_sgemm(dev, a, b, ta, tb, M, N, K, L.EPI_BIAS_ACT, L.OP_SIN, bias=bias, want_z=True)
            assert_close(Zs, ref + bias, what=what + "stored pre-activation (sin)")
            assert_close(Cs, np.sin(ref + bias), tol=2e-4 if K > 2000 else 1e-4, what=what + "bias + sin")  # (sin of sums of size sqrt(K))
            assert_close(run_sgemm(dev, a, b, ta, tb, M, N, K, L.EPI_ACT_GRAD, L.OP_SIN, aux=aux), ref * np.cos(aux.astype(np.float64)),
                         what=what + "sin gradient from the pre-activation")
        dev.call("endia_hip_gemm_force_tile", 256)
        # the column sums of B from the same call (the bias gradient beside the weight gradient), small and large B
        dC, dsum = dev.put(np.full((M, N), np.nan, np.float32)), dev.put(np.full(N, np.nan, np.float32))
        dev.call("endia_hip_sgemm", 1, 0, M, N, K, dev.put(A), M, dev.put(B), N, dC, N, 1, 0, 0, 0, L.EPI_NONE | L.GEMM_COLSUM_B,
                 L.OP_IDENTITY, None, None, dsum)
        assert_close(dev.get(dC, (M, N)), ref, what="C beside the column sums")
        assert_close(dev.get(dsum, (N,)), B.astype(np.float64).sum(0), tol=1e-5, what="column sums")
    finally:
        dev.call("endia_hip_gemm_force_tile", 0)
    assert L.lib().endia_hip_gemm_force_tile(96) == L.ERR_INVALID
