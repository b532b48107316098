"""Host-side planning of the launches (which kernel, how chains are cut, how much workspace),
read through ``ftc_causal_dot_plan``: nothing is launched, no GPU is needed.

The figures pinned here are the planner's rules as documented where the planner lives
(csrc/ftc_mfma.hip): one workgroup per chain segment on up to 256 CUs, chains of up to 64
chunks cut without an exchange at multiples of four chunks with later segments shorter,
longer chains on few CUs with an exchange, everything the MFMA kernels do not cover on the
generic kernel."""
import re

import pytest

from fast_transformers_amd import _native


def lines(q, v, **kw):
    return [l for l in _native.plan(q, v, **kw).split("\n") if l]


def field(line, pattern):
    m = re.search(pattern, line)
    assert m, (pattern, line)
    return m.group(1)


def test_headline_shape():
    fwd = lines((10, 8, 1000, 64), (10, 8, 1000, 64))
    assert len(fwd) == 1 and fwd[0].startswith("scan_tph_kernel:")
    assert "3 segments" in fwd[0] and "cuts at chunks 0,20,28,32" in fwd[0]
    assert "240 workgroups" in fwd[0] and "workspace 0 bytes" in fwd[0]
    bwd = lines((10, 8, 1000, 64), (10, 8, 1000, 64), backward=True)
    assert len(bwd) == 1 and bwd[0].startswith("scan_tph_kernel: 3 scans")
    assert "1 segment " in bwd[0] and "240 workgroups" in bwd[0]


def test_long_chains_exchange_their_segment_sums():
    fwd = lines((1, 16, 65536, 64), (1, 16, 65536, 64))
    assert fwd[0].startswith("scan_tph_kernel (exchange):")
    assert "16 segments of 4096 rows" in fwd[0] and "256 workgroups" in fwd[0]
    need = int(field(fwd[0], r"workspace (\d+) bytes"))
    lib = _native.load()
    assert 0 < need <= lib.ftc_causal_dot_product_workspace_bytes(1, 16, 65536, 64, 64, 0)
    # three scans of 16 chains: one round of workgroups would need segments of 412 chunks, so
    # just under two rounds of shorter ones
    bwd = lines((1, 16, 65536, 64), (1, 16, 65536, 64), backward=True)
    assert bwd[0].startswith("scan_tph_kernel (exchange): 3 scans")
    assert "10 segments of 6656 rows" in bwd[0] and "480 workgroups" in bwd[0]
    need = int(field(bwd[0], r"workspace (\d+) bytes"))
    assert 0 < need <= lib.ftc_causal_dot_backward_workspace_bytes(1, 16, 65536, 64, 64, 0)
    # more workgroups than CUs: three rounds for 32 chains of 2048 chunks
    bwd = lines((2, 16, 65536, 64), (2, 16, 65536, 64), backward=True)
    assert bwd[0].startswith("scan_tph_kernel (exchange): 3 scans")
    assert "8 segments of 8192 rows" in bwd[0] and "768 workgroups" in bwd[0]
    # chains of 257 to 1024 chunks on 112 workgroups or more are walked whole, in any number of
    # rounds; on fewer they exchange
    bwd = lines((4, 16, 16384, 64), (4, 16, 16384, 64), backward=True)
    assert bwd[0].startswith("scan_tph_kernel: 3 scans") and "1 segment of 16384 rows" in bwd[0]
    assert lines((4, 16, 16384, 64), (4, 16, 16384, 64))[0].startswith("scan_tph_kernel (exchange):")
    assert lines((3, 64, 16384, 64), (3, 64, 16384, 64), backward=True)[0].startswith("scan_tph_kernel: 3 scans")
    assert lines((3, 64, 16384, 64), (3, 64, 16384, 64))[0].startswith("scan_tph_kernel: 1 scan")
    assert lines((1, 36, 16384, 64), (1, 36, 16384, 64), backward=True)[0].startswith("scan_tph_kernel (exchange)")
    assert lines((4, 64, 40000, 64), (4, 64, 40000, 64), backward=True)[0].startswith("scan_dma_kernel")
    assert lines((8, 16, 8192, 64), (8, 16, 8192, 64), backward=True)[0].startswith("scan_tph_kernel:")
    # two segments of up to 64 chunks: chains cut in two without an exchange instead
    assert lines((1, 96, 4096, 64), (1, 96, 4096, 64))[0].startswith("scan_tph_kernel: 1 scan")
    assert "cuts at chunks 0,92,128" in lines((1, 32, 4096, 64), (1, 32, 4096, 64), backward=True)[0]
    assert lines((1, 96, 8192, 64), (1, 96, 8192, 64))[0].startswith("scan_tph_kernel (exchange):")
    # config 4's operator shape
    op = lines((10, 8, 4096, 64), (10, 8, 4096, 64))
    assert op[0].startswith("scan_tph_kernel (exchange):") and "3 segments of 1408 rows" in op[0]


def test_what_the_chain_parallel_kernel_leaves_to_the_others():
    # rows that lie too far apart for one 32-bit descriptor per chain
    far = (144 * 8192 * 65536, 8192 * 65536, 65536, 1)
    out = lines((1, 144, 8192, 64), (1, 144, 8192, 64), strides=(far, far, far))
    assert not out[0].startswith("scan_tp_kernel")
    # more chains than two rounds of workgroups
    many = lines((64, 16, 128, 64), (64, 16, 128, 64))
    assert many[0].startswith("scan_dma_kernel")
    # ... which chains of 16 chunks or more fill without losing to them
    assert lines((64, 16, 512, 64), (64, 16, 512, 64), backward=True)[0].startswith("scan_tph_kernel: 3 scans")
    assert lines((64, 16, 256, 64), (64, 16, 256, 64), backward=True)[0].startswith("scan_dma_kernel")
    assert lines((32, 16, 256, 64), (32, 16, 256, 64), backward=True)[0].startswith("scan_tph_kernel: 3 scans")
    # other state sizes and element types
    assert lines((10, 8, 1000, 32), (10, 8, 1000, 32))[0].startswith("scan_dma_kernel")
    # (32 rows or columns: the chain-parallel kernel on whole chains unless both are 32,
    # the kernels that split L where it would need an exchange)
    assert lines((10, 8, 1000, 32), (10, 8, 1000, 128))[0].startswith("scan_tph_kernel:")
    assert lines((4, 16, 16384, 32), (4, 16, 16384, 128))[0].startswith("scan_dma_kernel")
    # few chains too short for an exchange: cut or whole on the chain-parallel kernel all the same
    assert lines((1, 3, 500, 128), (1, 3, 500, 128))[0].startswith("scan_mfma_kernel")
    assert lines((1, 3, 500, 128), (1, 3, 500, 128), backward=True)[0].startswith("scan_tp_kernel: 3 scans")
    assert lines((1, 8, 640, 64), (1, 8, 640, 64))[0].startswith("scan_tph_kernel: 1 scan")
    # bf16 rows: a single scan stays with the kernels that multiply such rows as they are
    # until the chain-parallel kernel has workgroups for about half of the CUs, and wherever
    # it would need an exchange; the three scans of a backward call, and widths that those
    # kernels would only take as padded copies, go to the chain-parallel kernel
    bf16 = dict(dtype=_native.FTC_BF16)
    assert lines((4, 8, 1000, 64), (4, 8, 1000, 64), **bf16)[0].startswith("scan_mfma_kernel")
    assert lines((1, 8, 2048, 64), (1, 8, 2048, 64), **bf16)[0].startswith("scan_mfma_kernel")
    assert lines((1, 8, 2048, 64), (1, 8, 2048, 64), backward=True, **bf16)[0] \
        .startswith("scan_tph_kernel (exchange): 3 scans")
    whole = lines((1, 64, 16384, 64), (1, 64, 16384, 64), backward=True, **bf16)[0]
    assert whole.startswith("scan_tph_kernel: 3 scans") and "1 segment of 16384 rows" in whole
    assert lines((1, 43, 16384, 64), (1, 43, 16384, 64), backward=True, **bf16)[0].startswith("scan_mfma_kernel")
    assert lines((10, 8, 1000, 64), (10, 8, 1000, 64), **bf16)[0].startswith("scan_mfma_kernel")
    assert lines((14, 8, 1000, 64), (14, 8, 1000, 64), **bf16)[0].startswith("scan_tph_kernel:")
    assert lines((16, 8, 1000, 64), (16, 8, 1000, 64), **bf16)[0].startswith("scan_tph_kernel:")
    assert lines((16, 8, 4096, 64), (16, 8, 4096, 64), **bf16)[0].startswith("scan_mfma_kernel")
    assert lines((24, 8, 4096, 64), (24, 8, 4096, 64), **bf16)[0].startswith("scan_tph_kernel:")
    assert lines((16, 16, 1000, 64), (16, 16, 1000, 64), **bf16)[0].startswith("scan_tph_kernel:")
    # config 5: the dV scan (fp32 values, a state of 32 rows) walks its chains whole, however
    # long; the forward and the scans with a state of 128 rows stay where they were
    cfg5 = lines((4, 32, 16384, 32), (4, 32, 16384, 128), backward=True, **bf16)
    assert len(cfg5) == 3 and sum(l.startswith("scan_mfma_kernel") for l in cfg5) == 2
    dv = [l for l in cfg5 if l.startswith("scan_tph_kernel:")]
    assert len(dv) == 1 and "state 32 x 128" in dv[0] and "1 segment of 16384 rows" in dv[0]
    assert lines((4, 32, 16384, 32), (4, 32, 16384, 128), **bf16)[0].startswith("scan_mfma_kernel")
    assert all(l.startswith("scan_mfma_kernel")
               for l in lines((2, 32, 16384, 32), (2, 32, 16384, 128), backward=True, **bf16))
    assert lines((10, 8, 1000, 64), (10, 8, 1000, 64), backward=True, **bf16)[0] \
        .startswith("scan_tph_kernel: 3 scans")
    assert lines((6, 8, 257, 48), (6, 8, 257, 40), **bf16)[0].startswith("scan_tph_kernel:")
    assert lines((8, 8, 130, 20), (8, 8, 130, 20), **bf16)[0].startswith("scan_tph_kernel:")
    # (rows of 128 values: no fp16-piece form, and the bf16-piece form takes fp32 rows only)
    assert lines((10, 8, 1000, 128), (10, 8, 1000, 128), backward=True, **bf16)[0] \
        .startswith("scan_mfma_kernel")
    # odd widths: zero-padded dense copies for the matrix-core kernels when there are enough
    # rows to pay for the extra launches; states of more than 128 rows stay generic
    # (queries and keys are copied, the values and the product stay where they are; in the
    # backward the two copies serve all three scans, and dQ and dK are copied back)
    odd = lines((8, 16, 4096, 25), (8, 16, 4096, 64))
    assert odd[0].startswith("pad_rows_kernel: 2 operands") and "0 results" in odd[0]
    assert odd[1].startswith("scan_tph_kernel") and "state 32 x 64" in odd[1]
    odd = lines((8, 16, 4096, 25), (8, 16, 4096, 64), backward=True)
    assert odd[0].startswith("pad_rows_kernel: 2 operands") and "2 results" in odd[0]
    assert odd[1].startswith("scan_tph_kernel: 2 scans") and "state 64 x 32" in odd[1]
    wide = lines((8, 16, 4096, 99), (8, 16, 4096, 101), backward=True)
    assert wide[0].startswith("pad_rows_kernel: 4 operands") and "3 results" in wide[0]
    assert wide[1].startswith("scan_tp_kernel: 3 scans") and "state 128 x 128" in wide[1]
    assert lines((2, 2, 40, 10), (2, 2, 40, 3))[0].startswith("generic_scan_kernel")
    # (bf16 rows of such a scan are converted into fp32 copies on the way)
    assert lines((1, 2, 8192, 300), (1, 2, 8192, 64), dtype=_native.FTC_BF16)[0] \
        .startswith("pad_rows_kernel: 3 operands")
    assert lines((1, 2, 100, 300), (1, 2, 100, 64), dtype=_native.FTC_BF16)[0] \
        .startswith("generic_scan_kernel")   # (too few rows for the copies)
    # states of 129 to 512 rows: up to four scans over a split of the rows, the later ones'
    # rows added to the first one's
    three = lines((1, 2, 8192, 300), (1, 2, 8192, 64))
    assert [l.split(":")[0].split(" ")[0] for l in three] == \
        ["scan_tp_kernel", "scan_tp_kernel", "add_rows_kernel", "scan_tph_kernel", "add_rows_kernel"]
    assert "state 128 x 64" in three[0] and "state 128 x 64" in three[1] and "state 44 x 64" in three[3]
    two = lines((1, 2, 8192, 200), (1, 2, 8192, 64))
    assert "state 128 x 64" in two[0] and "state 72 x 64" in two[1] and two[2].startswith("add_rows_kernel: 1 result")
    two = lines((4, 8, 1000, 200), (4, 8, 1000, 200), backward=True)
    assert two[0].startswith("scan_tp_kernel: 3 scans") and "state 128 x 200" in two[0]
    assert "state 72 x 200" in two[1] and two[2].startswith("add_rows_kernel: 3 results")
    odd = lines((2, 4, 700, 255), (2, 4, 700, 129))
    assert odd[0].startswith("pad_rows_kernel: 3 operands") and "state 128 x 160" in odd[1]
    odd = lines((2, 4, 700, 255), (2, 4, 700, 129), backward=True)
    assert odd[0].startswith("pad_rows_kernel: 4 operands") and "3 results" in odd[0]
    # nothing to do
    assert lines((0, 8, 100, 64), (0, 8, 100, 64)) == []


@pytest.mark.parametrize("L", [33, 129, 500, 1000, 1500, 2048])
@pytest.mark.parametrize("chains", [(2, 8), (5, 8), (10, 8), (30, 4)])
def test_cut_chains(chains, L):
    """Cuts at multiples of four chunks, the last one at the end, at most 256 workgroups, and
    the longest workgroup (a chunk walked for its state alone counted as 0.6 of a full one)
    no longer than with equal segments (of whole groups of four chunks)."""
    N, H = chains
    line = lines((N, H, L, 64), (N, H, L, 64))[0]
    if not line.startswith("scan_tph_kernel:"):
        return
    cuts = [int(x) for x in field(line, r"cuts at chunks ([\d,]*\d)").split(",")]
    nseg = int(field(line, r"(\d+) segments? of"))
    assert len(cuts) == nseg + 1 and cuts[0] == 0 and cuts[-1] == (L + 31) // 32
    assert all(c % 4 == 0 for c in cuts[:-1])
    lengths = [b - a for a, b in zip(cuts, cuts[1:])]
    assert all(x > 0 for x in lengths)
    longest = max(0.6 * a + (b - a) for a, b in zip(cuts, cuts[1:]))
    step = -(-(-(-cuts[-1] // nseg)) // 4) * 4   # equal segments of whole groups of four
    equal = [min(i * step, cuts[-1]) for i in range(nseg + 1)]
    assert longest <= max(0.6 * a + (b - a) for a, b in zip(equal, equal[1:])) + 1e-9
    assert N * H * nseg <= 256 and int(field(line, r"(\d+) workgroups")) == N * H * nseg


def test_wide_states_on_the_chain_parallel_kernel():
    """fp32 states of more than 32 and up to 128 rows and columns, widths multiples of 4: two
    blocks of rows per chunk, a workgroup per block of 64 output columns."""
    fwd = lines((8, 16, 4096, 128), (8, 16, 4096, 128))
    assert len(fwd) == 1 and fwd[0].startswith("scan_tp_kernel: 1 scan")
    assert "state 128 x 128" in fwd[0] and "256 workgroups" in fwd[0] and "workspace 0 bytes" in fwd[0]
    bwd = lines((8, 16, 4096, 128), (8, 16, 4096, 128), backward=True)
    assert len(bwd) == 1 and bwd[0].startswith("scan_tp_kernel: 3 scans") and "768 workgroups" in bwd[0]
    # widths that leave the last block partly empty need no copies
    odd = lines((8, 16, 4096, 100), (8, 16, 4096, 68), backward=True)
    assert [l.split(":")[0] for l in odd] == ["scan_tp_kernel", "scan_tp_kernel"]
    assert "2 scans" in odd[0] and "state 68 x 100" in odd[0] and "state 100 x 68" in odd[1]
    # one block of columns: as many workgroups as chains
    assert "256 workgroups" in lines((16, 16, 4000, 128), (16, 16, 4000, 64))[0]
    # long chains: segment sums are exchanged, also with more workgroups than CUs
    long = lines((4, 16, 16384, 128), (4, 16, 16384, 128), backward=True)
    assert long[0].startswith("scan_tp_kernel (exchange): 3 scans") and "2 segments of 8192 rows" in long[0]
    need = int(field(long[0], r"workspace (\d+) bytes"))
    assert need == 65536 + 2 * 4 * 768 * 128 * 16 * 4
    # more workgroups than CUs: segments chosen so that the rounds of 256 are full
    rounds = lines((1, 16, 20000, 128), (1, 16, 20000, 128), backward=True)
    assert "8 segments of 2560 rows" in rounds[0] and "768 workgroups" in rounds[0]
    # few chains: shapes that the kernels which split L also take go to those below half
    # the CUs, the others go to the chain-parallel kernel at any size
    assert lines((1, 8, 512, 128), (1, 8, 512, 128))[0].startswith("scan_mfma_kernel")
    assert lines((1, 8, 256, 128), (1, 8, 256, 128))[0].startswith("scan_tp_kernel: 1 scan")
    assert lines((1, 8, 512, 128), (1, 8, 512, 128), backward=True)[0].startswith("scan_tp_kernel: 3 scans")
    assert lines((1, 40, 16384, 128), (1, 40, 16384, 32))[0].startswith("scan_mfma_kernel")
    # ... unless four or more segments of every chain fit one round of workgroups: an exchange
    # from 24 chunks on, in segments of down to four chunks
    few = lines((1, 8, 2048, 128), (1, 8, 2048, 128))[0]
    assert few.startswith("scan_tp_kernel (exchange):") and "16 segments of 128 rows" in few
    few = lines((1, 16, 2048, 64), (1, 16, 2048, 64))[0]
    assert few.startswith("scan_tph_kernel (exchange):") and "16 segments of 128 rows" in few
    assert lines((1, 16, 1024, 64), (1, 16, 1024, 64), backward=True)[0].startswith("scan_tph_kernel: 3 scans")
    assert lines((1, 16, 2048, 64), (1, 16, 2048, 64), backward=True)[0].startswith("scan_tph_kernel (exchange)")
    assert lines((1, 1, 2048, 64), (1, 1, 2048, 64))[0].startswith("scan_dma_kernel")
    assert lines((1, 4, 500, 100), (1, 4, 500, 100))[0].startswith("scan_tp_kernel: 1 scan")
    assert lines((1, 4, 1000, 100), (1, 4, 1000, 100))[0].startswith("scan_tp_kernel (exchange): 1 scan")
    # thousands of chains of one or two chunks with a small state, 32-wide shapes on more
    # than two rounds of workgroups: the other routes
    assert lines((512, 16, 64, 20), (512, 16, 64, 20))[0].startswith("pad_rows_kernel")
    assert lines((512, 16, 64, 32), (512, 16, 64, 128))[0].startswith("scan_dma_kernel")
    assert lines((512, 16, 64, 100), (512, 16, 64, 100))[0].startswith("scan_tp_kernel")
    # 32-wide shapes on few workgroups: the kernels that split L unless the chains are short
    assert lines((1, 32, 4096, 32), (1, 32, 4096, 128))[0].startswith("scan_dma_kernel")
    assert lines((1, 32, 1024, 32), (1, 32, 1024, 128))[0].startswith("scan_tph_kernel:")
    assert lines((1, 64, 4096, 32), (1, 64, 4096, 128))[0].startswith("scan_tph_kernel:")
    cut = lines((1, 64, 8192, 32), (1, 64, 8192, 128))[0]
    assert cut.startswith("scan_tph_kernel:") and "2 segments" in cut
    assert lines((1, 128, 4096, 128), (1, 128, 4096, 32))[0].startswith("scan_mfma_kernel")
    assert lines((1, 256, 4096, 128), (1, 256, 4096, 32))[0].startswith("scan_tp_kernel:")
    assert lines((1, 64, 512, 128), (1, 64, 512, 32))[0].startswith("scan_tp_kernel:")
    assert lines((1, 128, 4096, 64), (1, 128, 4096, 32))[0].startswith("scan_tph_kernel:")
    assert lines((1, 64, 2048, 64), (1, 64, 2048, 32))[0].startswith("scan_dma_kernel")
    assert lines((1, 16, 2048, 32), (1, 16, 2048, 96))[0].startswith("scan_tph_kernel:")
    # ... and long ones where whole chains fill three quarters of the CUs
    assert lines((1, 128, 16384, 32), (1, 128, 16384, 128))[0].startswith("scan_tph_kernel: 1 scan")
    # bf16 rows and widths that are not multiples of 4 go the other ways
    assert lines((8, 16, 4096, 128), (8, 16, 4096, 128), dtype=_native.FTC_BF16)[0] \
        .startswith("scan_mfma_kernel")
    assert lines((8, 16, 4096, 98), (8, 16, 4096, 128))[0].startswith("pad_rows_kernel")


SWEEP = [(N, H, L, E, M) for (N, H) in [(1, 1), (1, 16), (2, 8), (10, 8), (64, 16)]
         for L in [1, 64, 1000, 4096, 20000] for (E, M) in [(64, 64), (32, 128), (96, 64), (25, 70), (128, 128), (100, 36), (200, 64), (255, 129), (511, 300)]]


@pytest.mark.parametrize("backward", [False, True])
def test_the_workspace_query_covers_every_launch(backward):
    lib = _native.load()
    query = lib.ftc_causal_dot_backward_workspace_bytes if backward \
        else lib.ftc_causal_dot_product_workspace_bytes
    for dtype in (_native.FTC_F32, _native.FTC_BF16):
        for N, H, L, E, M in SWEEP:
            granted = query(N, H, L, E, M, dtype)
            assert granted >= 0
            for line in lines((N, H, L, E), (N, H, L, M), dtype=dtype, backward=backward):
                need = int(field(line, r"workspace (\d+) bytes")) if "workspace" in line else 0
                assert need <= granted, (N, H, L, E, M, dtype, line, granted)


@pytest.mark.parametrize("dtype", [_native.FTC_F32, _native.FTC_BF16], ids=["f32", "bf16"])
def test_workspace_queries_cover_every_plan(dtype):
    """Whatever route the planner takes, no launch of the plan needs more workspace than the
    query of its entry point answers: widths on either side of every limit of the planner (32,
    64, 128 rows; multiples of 4 and of 32 and neither), also bf16 rows whose two state shapes
    call for copies of different element types."""
    lib = _native.load()
    widths = [10, 25, 32, 33, 48, 64, 65, 96, 100, 128, 129, 132, 200, 255, 256, 300]
    worst = 0.0
    for (N, H, L) in [(10, 8, 2048), (2, 3, 700), (1, 2, 8192), (40, 16, 64)]:
        for E in widths:
            for M in widths:
                for backward in (False, True):
                    text = lines((N, H, L, E), (N, H, L, M), backward=backward, dtype=dtype)
                    need = max([int(x) for l in text for x in re.findall(r"workspace (\d+) bytes", l)]
                               or [0])
                    query = (lib.ftc_causal_dot_backward_workspace_bytes if backward else
                             lib.ftc_causal_dot_product_workspace_bytes)(N, H, L, E, M, dtype)
                    assert need <= query, ((N, H, L, E, M), backward, need, query, text)
                    if query:
                        worst = max(worst, need / query)
    assert worst > 0.5   # (the queries are not wildly generous either)


def test_rows_of_more_than_512_values_are_cut_into_pieces():
    """fp32 rows wider than 512: column slices of v and out, row parts of a and b whose results
    are added; every piece is planned like a scan of its own and the queries cover the lot."""
    lib = _native.load()
    fwd = lines((1, 2, 300, 600), (1, 2, 300, 520))
    # two row parts of 300 for each of two column slices of 288 and 232
    assert sum("state 128 x 288" in l for l in fwd) == 4 and sum("state 44 x 232" in l for l in fwd) == 2
    assert sum(l.startswith("add_rows_kernel: rows 300 ..") for l in fwd) == 2
    for (N, H, L, E, M) in [(1, 2, 300, 600, 520), (2, 2, 100, 513, 33), (1, 1, 64, 1100, 40),
                            (1, 2, 256, 64, 1030), (3, 4, 2048, 700, 900)]:
        for backward in (False, True):
            text = lines((N, H, L, E), (N, H, L, M), backward=backward)
            need = max(int(x) for l in text for x in re.findall(r"workspace (\d+) bytes", l))
            query = (lib.ftc_causal_dot_backward_workspace_bytes if backward else
                     lib.ftc_causal_dot_product_workspace_bytes)(N, H, L, E, M, _native.FTC_F32)
            assert 0 < need <= query, ((N, H, L, E, M), backward, need, query)
    # bf16 rows of that width: refused, by the queries as by the calls
    assert lib.ftc_causal_dot_product_workspace_bytes(1, 2, 300, 600, 520, _native.FTC_BF16) < 0
    assert b"fp32" in lib.ftc_last_error()
