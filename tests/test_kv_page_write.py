"""K/V page writer and device FP8 codec: the oracle restatement against the reference's expected bytes (CPU), and the
HIP kernels against the oracle, bit for bit (GPU).  Vectors follow kv_page_write.rs:285-398 of the reference."""
import numpy as np
import pytest

from khalamari_amd import _lib
from khalamari_amd._lib import DTYPE_BF16, DTYPE_FP8_E4M3FN, ReplayU32
from oracle import gqa_oracle as oracle


def _reference_vectors():
    """test_replay_matches_page_reference_across_active_counts (kv_page_write.rs:306-395): 8 writes, 2 slots, 4 pages."""
    flat_k = oracle.f32_to_bf16_bits(np.array([1.0 + i * 0.125 for i in range(16)], dtype=np.float32)).reshape(8, 1, 2)
    flat_v = oracle.f32_to_bf16_bits(np.array([-1.0 - i * 0.125 for i in range(16)], dtype=np.float32)).reshape(8, 1, 2)
    req_slots = np.array([0, 1, 0, 1, 0, 1, 0, 1], dtype=np.uint32)
    tokens = np.array([0, 0, 1, 1, 2, 2, 3, 3], dtype=np.uint32)
    page_ids = np.array([0, 1, 2, 3], dtype=np.uint32)
    return flat_k, flat_v, req_slots, tokens, page_ids


def test_oracle_page_write_matches_the_reference_layout_arithmetic():
    """Independent reconstruction exactly as the reference test builds `expected` (kv_page_write.rs:371-392)."""
    flat_k, flat_v, req_slots, tokens, page_ids = _reference_vectors()
    page_values, num_pages, head_dim, tokens_per_page, num_blocks = 16, 4, 2, 4, 2
    for active in [1, 8, 3, 7, 2, 6, 4, 5]:
        pages = np.full(num_pages * page_values, 0x55, dtype=np.uint8)
        got = oracle.kv_page_write(pages, flat_k, flat_v, req_slots, tokens, page_ids, active, 0, 1, num_blocks, 1, 1, head_dim,
                                   tokens_per_page, page_values, True)
        expected = np.full(num_pages * page_values, 0x55, dtype=np.uint8)
        kv_values_per_page = tokens_per_page * head_dim
        for write in range(active):
            slot, token = int(req_slots[write]), int(tokens[write])
            page = int(page_ids[slot * num_blocks + token // tokens_per_page])
            for dim in range(head_dim):
                offset = (token % tokens_per_page) * head_dim + dim
                expected[page * page_values + offset] = oracle.bf16_bits_to_fp8(flat_k[write, 0, dim:dim + 1])[0]
                expected[page * page_values + kv_values_per_page + offset] = oracle.bf16_bits_to_fp8(flat_v[write, 0, dim:dim + 1])[0]
        assert np.array_equal(got, expected), active


def test_oracle_page_write_special_values():
    """test_fp8_replay_matches_page_reference (kv_page_write.rs:397-420): -0, 2^-10, 2^-9, ties, 400, 448, 449, inf;
    the expected codes are the fixed encodings of fp8.rs:70-100."""
    k_values = np.array([-0.0, 2.0 ** -10, 2.0 ** -9, 1.0625, 1.1875, 400.0, 448.0, 449.0, np.inf], dtype=np.float32)
    expected_k = np.array([0x80, 0x00, 0x01, 0x38, 0x3A, 0x7C, 0x7E, 0x7E, 0x7E], dtype=np.uint8)
    assert np.array_equal(oracle.bf16_bits_to_fp8(oracle.f32_to_bf16_bits(k_values)), expected_k)
    n = len(k_values)
    # one write at token 1 of a two-token page, one head of n dims: K lands in the second row of the K plane
    pages = np.zeros(4 * n, dtype=np.uint8)
    got = oracle.kv_page_write(pages, oracle.f32_to_bf16_bits(k_values), oracle.f32_to_bf16_bits(-k_values), np.array([0], dtype=np.uint32),
                               np.array([1], dtype=np.uint32), np.array([0], dtype=np.uint32), 1, 0, 1, 1, 1, 1, n, 2, 4 * n, True)
    assert np.array_equal(got[n:2 * n], expected_k)
    assert np.array_equal(got[3 * n:], expected_k ^ 0x80)
    assert not got[:n].any() and not got[2 * n:3 * n].any()


def test_page_write_validation_without_a_gpu():
    from khalamari_amd import kv_page_write as kpw

    with pytest.raises(_lib.KhmError, match="divisible"):
        kpw.Config(2, 2, 15).num_tokens_per_page()
    assert kpw.Config(8, 128, 32 * 1024).num_tokens_per_page() == 16                        # the reference's 32 KiB FP8 page
    assert kpw.Config(8, 128, 64 * 1024, kv_dtype=DTYPE_BF16).num_tokens_per_page() == 16


# ---------------------------------------------------------------------------------------------- GPU


def _device():
    import torch

    assert torch.cuda.is_available()
    return torch.device("cuda:0")


@pytest.mark.gpu
def test_gpu_fp8_codec_matches_the_host_codec_exhaustively():
    import torch

    from khalamari_amd import kv_page_write as kpw

    device = _device()
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8).to(device)
    decoded = torch.zeros(256, dtype=torch.int16, device=device)
    kpw.fp8_decode_device(codes, decoded, 256)
    got = decoded.cpu().numpy().view(np.uint16)
    want = oracle.fp8_decode_table()
    finite = (np.arange(256) & 0x7F) != 0x7F
    assert np.array_equal(got[finite], want[finite])
    for code in (0x7F, 0xFF):   # NaN stays NaN; the payload is the hardware's
        assert (got[code] & 0x7F80) == 0x7F80 and (got[code] & 0x7F) != 0
    every_bf16 = torch.from_numpy(np.arange(65536, dtype=np.int32).astype(np.uint16).view(np.int16)).to(device)
    encoded = torch.zeros(65536, dtype=torch.uint8, device=device)
    kpw.fp8_encode_device(every_bf16, encoded, 65536)
    assert np.array_equal(encoded.cpu().numpy(), oracle.bf16_bits_to_fp8(np.arange(65536, dtype=np.uint32).astype(np.uint16)))
    # the device encoder converts eight elements at a time (pairs and a single element at the end of an odd count): every
    # pattern in every position of a group, and counts that leave 7 .. 1 elements to the tail paths
    every = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    for shift in range(1, 9):
        rolled = np.roll(every, shift)[:65536 - shift]
        encoded = torch.full((65536,), 0xAA, dtype=torch.uint8, device=device)
        kpw.fp8_encode_device(torch.from_numpy(rolled.view(np.int16).copy()).to(device), encoded, rolled.size)
        got = encoded.cpu().numpy()
        assert np.array_equal(got[:rolled.size], oracle.bf16_bits_to_fp8(rolled)), shift
        assert np.all(got[rolled.size:] == 0xAA), shift


def _run_page_write(device, config, shape, pages, flat_k, flat_v, req_slots, tokens, page_ids, active, layer=0, parameters=None):
    import torch

    from khalamari_amd import kv_page_write as kpw

    to = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy()).to(device)  # noqa: E731
    d_pages = to(pages)
    kpw.Compute(config).invoke(shape, pages=d_pages, flat_k=to(flat_k), flat_v=to(flat_v), req_slots=to(req_slots), flat_token_indices=to(tokens),
                               page_ids=to(page_ids), num_active_token_writes=active, page_table_index=ReplayU32.fixed(layer),
                               replay_parameters=parameters)
    torch.cuda.synchronize()
    return d_pages.cpu().numpy()


@pytest.mark.gpu
def test_gpu_page_write_reference_vectors_across_active_counts():
    import torch

    from khalamari_amd import kv_page_write as kpw

    device = _device()
    flat_k, flat_v, req_slots, tokens, page_ids = _reference_vectors()
    config = kpw.Config(1, 2, 16)
    shape = kpw.Shape(8, kpw.PageTableLayout(2, 1, 2, 1))
    block = torch.zeros(4, dtype=torch.int32, device=device)
    for active in [1, 8, 3, 7, 2, 6, 4, 5]:
        block[2] = active
        pages = np.full(64, 0x55, dtype=np.uint8)
        got = _run_page_write(device, config, shape, pages, flat_k, flat_v, req_slots, tokens, page_ids, ReplayU32.parameter(2), parameters=block)
        want = oracle.kv_page_write(pages, flat_k, flat_v, req_slots, tokens, page_ids, active, 0, 1, 2, 1, 1, 2, 4, 16, True)
        assert np.array_equal(got, want), active


@pytest.mark.gpu
def test_gpu_page_write_special_values():
    from khalamari_amd import kv_page_write as kpw

    device = _device()
    k_values = np.array([-0.0, 2.0 ** -10, 2.0 ** -9, 1.0625, 1.1875, 400.0, 448.0, 449.0, np.inf], dtype=np.float32)
    n = len(k_values)
    flat_k, flat_v = oracle.f32_to_bf16_bits(k_values), oracle.f32_to_bf16_bits(-k_values)
    config = kpw.Config(1, n, 4 * n)
    shape = kpw.Shape(1, kpw.PageTableLayout(1, 1, 1, 1))
    one = np.array([0], dtype=np.uint32)
    got = _run_page_write(device, config, shape, np.zeros(4 * n, dtype=np.uint8), flat_k, flat_v, one, np.array([1], dtype=np.uint32), one,
                          ReplayU32.fixed(1))
    want = oracle.kv_page_write(np.zeros(4 * n, dtype=np.uint8), flat_k, flat_v, one, [1], one, 1, 0, 1, 1, 1, 1, n, 2, 4 * n, True)
    assert np.array_equal(got, want)
    assert np.array_equal(got[n:2 * n], np.array([0x80, 0x00, 0x01, 0x38, 0x3A, 0x7C, 0x7E, 0x7E, 0x7E], dtype=np.uint8))


@pytest.mark.gpu
@pytest.mark.parametrize("kv_dtype", [DTYPE_FP8_E4M3FN, DTYPE_BF16])
@pytest.mark.parametrize("heads,dim", [(8, 128), (4, 256), (2, 65)])
def test_gpu_page_write_production_shapes(kv_dtype, heads, dim):
    """Real head geometries, several layers and page ids per block, scattered tokens, poisoned pages elsewhere."""
    from khalamari_amd import kv_page_write as kpw

    device = _device()
    rng = np.random.default_rng(heads * 1000 + dim + kv_dtype)
    element = 1 if kv_dtype == DTYPE_FP8_E4M3FN else 2
    tokens_per_page, layers, blocks, per_block, slots, writes = 16, 2, 3, 2, 3, 41
    page_bytes = 2 * heads * tokens_per_page * dim * element
    num_pages = slots * layers * blocks * per_block
    page_ids = rng.permutation(num_pages).astype(np.uint32)
    req_slots = rng.integers(0, slots, size=writes).astype(np.uint32)
    # distinct (slot, token) pairs so that no two writes race for one row
    pairs = rng.permutation(slots * blocks * per_block * tokens_per_page)[:writes]
    req_slots = (pairs % slots).astype(np.uint32)
    tokens = (pairs // slots).astype(np.uint32)
    flat_k = oracle.f32_to_bf16_bits((rng.standard_normal((writes, heads, dim)) * 4).astype(np.float32))
    flat_v = oracle.f32_to_bf16_bits((rng.standard_normal((writes, heads, dim)) * 4).astype(np.float32))
    pages = rng.integers(0, 256, size=num_pages * page_bytes, dtype=np.uint8)
    config = kpw.Config(heads, dim, page_bytes, kv_dtype=kv_dtype)
    shape = kpw.Shape(writes, kpw.PageTableLayout(slots, layers, blocks, per_block))
    active = writes - 4
    got = _run_page_write(device, config, shape, pages, flat_k, flat_v, req_slots, tokens, page_ids, ReplayU32.fixed(active), layer=1)
    want = oracle.kv_page_write(pages, flat_k, flat_v, req_slots, tokens, page_ids, active, 1, layers, blocks, per_block, heads, dim,
                                tokens_per_page, page_bytes, kv_dtype == DTYPE_FP8_E4M3FN)
    assert np.array_equal(got, want)


@pytest.mark.gpu
def test_gpu_page_write_rejects_bad_arguments():
    import torch

    from khalamari_amd import kv_page_write as kpw

    device = _device()
    config = kpw.Config(1, 2, 16)
    shape = kpw.Shape(8, kpw.PageTableLayout(2, 1, 2, 1))
    small = torch.zeros(4, dtype=torch.uint8, device=device)
    big = torch.zeros(256, dtype=torch.uint8, device=device)
    with pytest.raises(_lib.KhmError, match="flat_k buffer"):
        kpw.Compute(config).invoke(shape, pages=big, flat_k=small, flat_v=big, req_slots=big, flat_token_indices=big, page_ids=big,
                                   num_active_token_writes=ReplayU32.fixed(1), page_table_index=ReplayU32.fixed(0))
    with pytest.raises(_lib.KhmError, match="replay domain"):
        kpw.Compute(config).invoke(shape, pages=big, flat_k=big, flat_v=big, req_slots=big, flat_token_indices=big, page_ids=big,
                                   num_active_token_writes=ReplayU32.fixed(9), page_table_index=ReplayU32.fixed(0))
