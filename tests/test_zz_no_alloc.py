"""varq_quant_pack_static -- the entry point that allocates nothing -- against
varq_quant_pack with a caller workspace: same words, codes, scales and zero-points,
bit for bit, on two calls in a row of which the second is smaller (the static scratch
keeps the first call's partial results)."""
import pytest
import torch

from gpu_util import note
from var_q_amd import _lib

pytestmark = pytest.mark.gpu


def _both(x, mask, bits, asym, pack, dev):
    lib = _lib.load()
    shape = list(x.shape)
    sh = _lib.i64arr(shape)
    sshape = [1 if (mask >> d) & 1 else shape[d] for d in range(4)]
    last = shape[3] * bits // 32 if pack else shape[3]
    res = []
    for static in (False, True):
        q = torch.full((*shape[:3], last), -7, dtype=torch.int32 if pack else torch.int8, device=dev)
        scale = torch.full(sshape, -1.0, dtype=torch.float32, device=dev)
        zp = torch.full(sshape, -1.0, dtype=torch.float32, device=dev) if asym else None
        words, codes = (q.data_ptr(), None) if pack else (None, q.data_ptr())
        stream = torch.cuda.current_stream().cuda_stream
        dt = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}[x.dtype]
        if static:
            rc = lib.varq_quant_pack_static(x.data_ptr(), dt, sh, mask, bits, int(asym), 1e-12, words, codes,
                                            scale.data_ptr(), zp.data_ptr() if asym else None, None, stream)
            _lib.check(rc, 'varq_quant_pack_static')
        else:
            n = lib.varq_quant_workspace_bytes(sh, mask)
            ws = torch.empty(max(n, 8), dtype=torch.uint8, device=dev)
            rc = lib.varq_quant_pack(x.data_ptr(), dt, sh, mask, bits, int(asym), 1e-12, words, codes,
                                     scale.data_ptr(), zp.data_ptr() if asym else None, None, ws.data_ptr(), ws.numel(),
                                     stream)
            _lib.check(rc, 'varq_quant_pack')
        torch.cuda.synchronize()
        res.append((q, scale, zp))
    return res


# reduce masks of the reference's methods on a [B,H,L,c] tensor (VAR_Q/quant.py:78-95)
MASKS = {'G_SCALE_HEAD_DIM': 0b0101, 'G_TENSOR': 0b1111, 'G_TOKEN': 0b1011, 'G_TOKEN_HEAD': 0b1001}


@pytest.mark.parametrize('method', sorted(MASKS))
@pytest.mark.parametrize('bits,asym,pack', [(8, False, True), (4, True, True), (2, True, True), (8, False, False)])
def test_static_scratch_matches_workspace_entry(dev, method, bits, asym, pack):
    mask = MASKS[method]
    g = torch.Generator().manual_seed(11)
    # the second call is smaller: whatever the first left in the scratch must not leak into it
    for shape, dtype in (([4, 6, 333, 64], torch.bfloat16), ([2, 3, 41, 64], torch.float32)):
        note('static scratch', method, bits, asym, pack, shape, dtype)
        x = (torch.randn(shape, generator=g) * 3 + 0.5).to(dtype).to(dev)
        (q0, s0, z0), (q1, s1, z1) = _both(x, mask, bits, asym, pack, dev)
        assert torch.equal(q0, q1) and torch.equal(s0, s1)
        assert (z0 is None and z1 is None) or torch.equal(z0, z1)
        assert float(s1.min()) > 0          # outputs were written, not left at the fill value


def test_scalar_kernels_share_the_scratch_too(dev):
    """A channel count that is not a multiple of 8 takes the kernels that start from a
    filled scratch (ordered-integer atomics): large call, then a small one."""
    g = torch.Generator().manual_seed(12)
    for shape in ([3, 5, 77, 30], [1, 2, 9, 30]):
        note('static scratch, scalar kernels', shape)
        x = torch.randn(shape, generator=g).to(dev)
        (q0, s0, z0), (q1, s1, z1) = _both(x, 0b0101, 8, True, False, dev)
        assert torch.equal(q0, q1) and torch.equal(s0, s1) and torch.equal(z0, z1)


def test_static_scratch_rejects_what_does_not_fit(dev):
    lib = _lib.load()
    cap = lib.varq_quant_static_scratch_bytes()
    assert cap == 16 << 20
    sh = _lib.i64arr([8, 4096, 16, 128])           # only the batch is reduced: 8.4 million groups, several words each
    assert lib.varq_quant_workspace_bytes(sh, 0b0001) > cap
    x = torch.zeros(8, dtype=torch.float32, device=dev)     # never read: the call is rejected on the host
    rc = lib.varq_quant_pack_static(x.data_ptr(), 0, sh, 0b0001, 8, 0, 1e-12, x.data_ptr(), None, x.data_ptr(), None,
                                    None, None)
    assert rc == -4 and b'static' in lib.varq_last_error()


def test_static_entry_recorded_into_a_graph(dev):
    """The entry point under HIP graph capture, its named use: the scratch address is looked up
    by the warm-up call before the capture, the capture records kernel launches only, and every
    replay on new input equals the eager result bit for bit."""
    lib = _lib.load()
    assert lib.varq_quant_static_scratch_bytes() >= (8 << 20)      # the warm-up call, outside capture
    B, H, L, c, bits, mask = 2, 6, 77, 64, 4, 0b0101
    gen = torch.Generator(device=dev).manual_seed(17)
    x = torch.randn(B, H, L, c, device=dev, generator=gen).bfloat16()
    sh = _lib.i64arr([B, H, L, c])
    words = torch.zeros(B, H, L, c * bits // 32, dtype=torch.int32, device=dev)
    scale, zp = torch.zeros(1, H, 1, c, device=dev), torch.zeros(1, H, 1, c, device=dev)

    def run(stream):
        _lib.check(lib.varq_quant_pack_static(x.data_ptr(), 1, sh, mask, bits, 1, 1e-12, words.data_ptr(), None,
                                              scale.data_ptr(), zp.data_ptr(), None, stream), 'varq_quant_pack_static')

    note('no-alloc graph: warm-up on a side stream')
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    note('no-alloc graph: capture')
    with torch.cuda.graph(graph):
        run(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for rep in range(3):
        x.normal_(generator=gen)
        note('no-alloc graph: eager', rep)
        run(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        want = [t.clone() for t in (words, scale, zp)]
        for t in (words, scale, zp):
            t.zero_()
        note('no-alloc graph: replay', rep)
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(want, (words, scale, zp)):
            assert torch.equal(a, b), f'replay {rep}: the graph and the eager call differ'
