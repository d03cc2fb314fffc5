"""The bare streaming probe (tt_stream_probe) moves bytes exactly: bit-exact copy / xor, ragged
sizes included, and refuses what it documents as unsupported."""
import pytest
import torch

from test_gpu_parity import DEV

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n_packs", [1, 63, 512, 513, 256 * 512 * 2 + 77, 3_000_001])
def test_stream_probe_copy_and_xor(n_packs):
    from teletron_amd import cabi
    g = torch.Generator().manual_seed(n_packs)
    a = torch.randint(-2**31, 2**31 - 1, (n_packs * 4 + 4,), generator=g, dtype=torch.int32).to(DEV)
    b = torch.randint(-2**31, 2**31 - 1, (n_packs * 4 + 4,), generator=g, dtype=torch.int32).to(DEV)
    out = torch.full_like(a, 7)
    stream = torch.cuda.current_stream().cuda_stream
    cabi.call("tt_stream_probe", out.data_ptr(), a.data_ptr(), None, n_packs * 16, stream)
    assert torch.equal(out[:n_packs * 4], a[:n_packs * 4])
    assert torch.all(out[n_packs * 4:] == 7)           # nothing past the end is touched
    cabi.call("tt_stream_probe", out.data_ptr(), a.data_ptr(), b.data_ptr(), n_packs * 16, stream)
    assert torch.equal(out[:n_packs * 4], a[:n_packs * 4] ^ b[:n_packs * 4])
    assert torch.all(out[n_packs * 4:] == 7)


@pytest.mark.parametrize("n_packs", [1, 511, 512 * 256 * 4 + 5, 3_000_001])
def test_stream_probe_write_only_and_read_only(n_packs):
    from teletron_amd import cabi
    out = torch.full((n_packs * 4 + 4,), 7, dtype=torch.int32, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    cabi.call("tt_stream_probe", out.data_ptr(), None, None, n_packs * 16, stream)     # writes on their own
    want = torch.arange(n_packs, dtype=torch.int32, device=DEV).repeat_interleave(4)
    assert torch.equal(out[:n_packs * 4], want)
    assert torch.all(out[n_packs * 4:] == 7)
    before = out.clone()
    cabi.call("tt_stream_probe", None, out.data_ptr(), None, n_packs * 16, stream)     # reads on their own
    torch.cuda.synchronize()
    assert torch.equal(out, before)


@pytest.mark.parametrize("n_packs", [1, 255, 1024, 1025, 256 * 4 * 256 + 77, 3_000_001])
def test_stream_probe_two_outputs(n_packs):
    from teletron_amd import cabi
    g = torch.Generator().manual_seed(n_packs)
    a = torch.randint(-2**31, 2**31 - 1, (n_packs * 4 + 4,), generator=g, dtype=torch.int32).to(DEV)
    out0, out1 = torch.full_like(a, 7), torch.full_like(a, 9)
    stream = torch.cuda.current_stream().cuda_stream
    cabi.call("tt_stream_probe_two_outputs", out0.data_ptr(), out1.data_ptr(), a.data_ptr(), n_packs * 16, stream)
    assert torch.equal(out0[:n_packs * 4], a[:n_packs * 4])
    assert torch.equal(out1[:n_packs * 4], ~a[:n_packs * 4])
    assert torch.all(out0[n_packs * 4:] == 7) and torch.all(out1[n_packs * 4:] == 9)
    lib = cabi.load()
    assert lib.tt_stream_probe_two_outputs(out0.data_ptr(), None, a.data_ptr(), 64, None) == cabi.TT_ERR_INVALID_ARGUMENT
    assert lib.tt_stream_probe_two_outputs(out0.data_ptr(), out1.data_ptr(), a.data_ptr(), 24, None) == cabi.TT_ERR_UNSUPPORTED


def test_stream_probe_errors():
    from teletron_amd import cabi
    lib = cabi.load()
    a = torch.zeros(64, dtype=torch.int32, device=DEV)
    out = torch.zeros_like(a)
    assert lib.tt_stream_probe(out.data_ptr(), a.data_ptr(), None, 0, None) == cabi.TT_OK
    assert lib.tt_stream_probe(None, None, None, 64, None) == cabi.TT_ERR_INVALID_ARGUMENT
    assert lib.tt_stream_probe(None, a.data_ptr(), a.data_ptr(), 64, None) == cabi.TT_ERR_INVALID_ARGUMENT
    assert lib.tt_stream_probe(out.data_ptr(), None, a.data_ptr(), 64, None) == cabi.TT_ERR_INVALID_ARGUMENT
    assert lib.tt_stream_probe(out.data_ptr(), a.data_ptr(), None, 24, None) == cabi.TT_ERR_UNSUPPORTED
    assert lib.tt_stream_probe(out.data_ptr() + 4, a.data_ptr(), None, 64, None) == cabi.TT_ERR_UNSUPPORTED
