"""K RMSNorm + RoPE fused with the K/V page write (khm_k_norm_rope_page_write): the pages must receive exactly the bytes
that khm_rms_norm_rope followed by khm_kv_page_write leave there (the order GQA::record enqueues them in,
crates/inference-executor-metal/src/attn/gqa/backend.rs:382-412), and what the oracle's chain of both steps gives."""
import numpy as np
import pytest

from khalamari_amd import _lib
from khalamari_amd._lib import DTYPE_BF16, DTYPE_F32, DTYPE_FP8_E4M3FN, ReplayU32
from oracle import gqa_oracle as oracle

YARN = dict(factor=32.0, attention_factor=float(np.float32(1.0) + np.float32(0.1) * np.log(np.float32(32.0))), beta_fast=32.0,
            beta_slow=1.0, original_max_position_embeddings=8192, truncate=True)


def _device():
    import torch

    assert torch.cuda.is_available()
    return torch.device("cuda:0")


def _case(heads, dim, rope_dim, kv_dtype, seed, writes=41, scale=4.0):
    rng = np.random.default_rng(seed)
    element = 1 if kv_dtype == DTYPE_FP8_E4M3FN else 2
    tokens_per_page, layers, blocks, per_block, slots = 16, 2, 3, 2, 3
    page_bytes = 2 * heads * tokens_per_page * dim * element
    num_pages = slots * layers * blocks * per_block
    pairs = rng.permutation(slots * blocks * per_block * tokens_per_page)[:writes]   # distinct (slot, token): no two writes share a row
    return dict(heads=heads, dim=dim, rope_dim=rope_dim, kv_dtype=kv_dtype, tokens_per_page=tokens_per_page, layers=layers, blocks=blocks,
                per_block=per_block, slots=slots, writes=writes, page_bytes=page_bytes,
                page_ids=rng.permutation(num_pages).astype(np.uint32), req_slots=(pairs % slots).astype(np.uint32),
                tokens=(pairs // slots).astype(np.uint32),
                k=oracle.f32_to_bf16_bits((rng.standard_normal((writes, heads, dim)) * scale).astype(np.float32)),
                v=oracle.f32_to_bf16_bits((rng.standard_normal((writes, heads, dim)) * scale).astype(np.float32)),
                weight=(0.75 + rng.random(dim) * 0.5).astype(np.float32),
                pages=rng.integers(0, 256, size=num_pages * page_bytes, dtype=np.uint8))


def _configs(case, weight_dtype, yarn):
    from khalamari_amd import kv_page_write as kpw
    from khalamari_amd import rms_norm_rope as rnr

    norm = rnr.Config.bf16(case["heads"], case["dim"], case["rope_dim"], 1e-6, 10_000_000.0).with_norm_weight_dtype(weight_dtype)
    if yarn:
        norm = norm.with_rope_scaling(rnr.Yarn(**YARN))
    page = kpw.Config(case["heads"], case["dim"], case["page_bytes"], kv_dtype=case["kv_dtype"])
    shape = kpw.Shape(case["writes"], kpw.PageTableLayout(case["slots"], case["layers"], case["blocks"], case["per_block"]))
    return norm, page, shape


def _weight_bytes(case, weight_dtype):
    return oracle.f32_to_bf16_bits(case["weight"]) if weight_dtype == DTYPE_BF16 else case["weight"]


def _run_fused(device, case, weight_dtype, yarn, active, layer, parameters=None):
    import torch

    from khalamari_amd import k_norm_rope_page_write as fused

    norm, page, shape = _configs(case, weight_dtype, yarn)
    to = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy()).to(device)  # noqa: E731
    pages = to(case["pages"])
    fused.Compute(norm, page).invoke(shape, pages=pages, k=to(case["k"]), v=to(case["v"]), norm_weight=to(_weight_bytes(case, weight_dtype)),
                                     req_slots=to(case["req_slots"]), flat_token_indices=to(case["tokens"]), page_ids=to(case["page_ids"]),
                                     num_active_tokens=active, page_table_index=ReplayU32.fixed(layer), replay_parameters=parameters)
    torch.cuda.synchronize()
    return pages.cpu().numpy()


def _run_two_kernels(device, case, weight_dtype, yarn, active, layer, parameters=None):
    import torch

    from khalamari_amd import kv_page_write as kpw
    from khalamari_amd import rms_norm_rope as rnr

    norm, page, shape = _configs(case, weight_dtype, yarn)
    to = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy()).to(device)  # noqa: E731
    pages, tokens = to(case["pages"]), to(case["tokens"])
    k_rows = torch.zeros(case["k"].nbytes, dtype=torch.uint8, device=device)
    rnr.Compute(norm).invoke(rnr.Shape(case["writes"]), input=to(case["k"]), norm_weight=to(_weight_bytes(case, weight_dtype)),
                             flat_token_indices=tokens, output=k_rows, num_active_tokens=active, replay_parameters=parameters)
    kpw.Compute(page).invoke(shape, pages=pages, flat_k=k_rows, flat_v=to(case["v"]), req_slots=to(case["req_slots"]), flat_token_indices=tokens,
                             page_ids=to(case["page_ids"]), num_active_token_writes=active, page_table_index=ReplayU32.fixed(layer),
                             replay_parameters=parameters)
    torch.cuda.synchronize()
    return pages.cpu().numpy()


def _oracle_chain(case, weight_dtype, yarn, active, layer):
    k_rows = oracle.rms_norm_rope(case["k"], _weight_bytes(case, weight_dtype), case["tokens"], case["heads"], case["dim"], case["rope_dim"],
                                  1e-6, 10_000_000.0, yarn=YARN if yarn else None, io_bf16=True, weight_bf16=weight_dtype == DTYPE_BF16)
    return oracle.kv_page_write(case["pages"], k_rows, case["v"], case["req_slots"], case["tokens"], case["page_ids"], active, layer,
                                case["layers"], case["blocks"], case["per_block"], case["heads"], case["dim"], case["tokens_per_page"],
                                case["page_bytes"], case["kv_dtype"] == DTYPE_FP8_E4M3FN)


@pytest.mark.gpu
@pytest.mark.parametrize("kv_dtype", [DTYPE_FP8_E4M3FN, DTYPE_BF16])
@pytest.mark.parametrize("heads,dim,rope_dim,weight_dtype,yarn", [(8, 128, 128, DTYPE_BF16, False), (4, 256, 64, DTYPE_BF16, False),
                                                                  (4, 256, 256, DTYPE_F32, True), (2, 64, 64, DTYPE_F32, False),
                                                                  (1, 512, 128, DTYPE_BF16, True), (3, 128, 32, DTYPE_BF16, False)])
def test_gpu_fused_pages_equal_the_two_kernel_sequence_byte_for_byte(kv_dtype, heads, dim, rope_dim, weight_dtype, yarn):
    import torch

    device = _device()
    case = _case(heads, dim, rope_dim, kv_dtype, seed=heads * 7919 + dim + rope_dim + kv_dtype)
    block = torch.zeros(4, dtype=torch.int32, device=device)
    for active, layer in [(case["writes"], 0), (case["writes"] - 4, 1), (1, 1)]:
        print(f"fused K norm/rope page write heads={heads} dim={dim} rope={rope_dim} kv_dtype={kv_dtype} active={active}", flush=True)
        fused = _run_fused(device, case, weight_dtype, yarn, ReplayU32.fixed(active), layer)
        separate = _run_two_kernels(device, case, weight_dtype, yarn, ReplayU32.fixed(active), layer)
        assert np.array_equal(fused, separate)
        changed = np.flatnonzero(fused != case["pages"])
        assert changed.size > 0
        # against the oracle's chain: the same pages except where sine, cosine and 1/sqrt round a K element the other way
        want = _oracle_chain(case, weight_dtype, yarn, active, layer)
        assert np.mean(fused == want) > 0.995
        untouched = want == case["pages"]
        assert np.array_equal(fused[untouched & (fused == case["pages"])], want[untouched & (fused == case["pages"])])
    # the active count as a replay parameter
    block.copy_(torch.tensor([0, 7, 0, 0], dtype=torch.int32))
    fused = _run_fused(device, case, weight_dtype, yarn, ReplayU32.parameter(1), 0, parameters=block)
    separate = _run_two_kernels(device, case, weight_dtype, yarn, ReplayU32.parameter(1), 0, parameters=block)
    assert np.array_equal(fused, separate)


@pytest.mark.gpu
def test_gpu_fused_write_of_rows_the_norm_leaves_alone_gives_the_page_writer_reference_bytes():
    """K rows of +-1 with unit weights at position 0 come out of RMSNorm + RoPE unchanged (x / sqrt(1 + 1e-6) rounds back
    to +-1 in bf16, the rotation is the identity), so the fused call must write what the plain page writer writes for
    them, whose FP8 codes are the reference's fixed encodings (kv_page_write.rs:397-420, fp8.rs:70-100): 0x38 / 0xB8 for
    +-1 in K, and in V the special values -0, 2^-10, 2^-9, the ties, 400, 448, 449 and infinity."""
    device = _device()
    v_special = np.array([-0.0, 2.0 ** -10, 2.0 ** -9, 1.0625, 1.1875, 400.0, 448.0, 449.0], dtype=np.float32)
    v_codes = np.array([0x80, 0x00, 0x01, 0x38, 0x3A, 0x7C, 0x7E, 0x7E], dtype=np.uint8)
    v_special, v_codes = np.tile(v_special, 2), np.tile(v_codes, 2)
    case = _case(1, 16, 16, DTYPE_FP8_E4M3FN, seed=3, writes=1)
    signs = np.array([1, -1, -1, 1, 1, 1, -1, 1, -1, -1, 1, -1, 1, 1, -1, -1], dtype=np.float32)
    case.update(k=oracle.f32_to_bf16_bits(signs).reshape(1, 1, 16), v=oracle.f32_to_bf16_bits(v_special).reshape(1, 1, 16),
                weight=np.ones(16, dtype=np.float32), tokens=np.array([0], dtype=np.uint32), req_slots=np.array([1], dtype=np.uint32),
                pages=np.zeros_like(case["pages"]))
    got = _run_fused(device, case, DTYPE_BF16, False, ReplayU32.fixed(1), 0)
    page = int(case["page_ids"][(1 * case["layers"] + 0) * case["blocks"] * case["per_block"]])
    base = page * case["page_bytes"]
    assert np.array_equal(got[base:base + 16], np.where(signs > 0, 0x38, 0xB8).astype(np.uint8))
    v_plane = base + case["tokens_per_page"] * 16
    assert np.array_equal(got[v_plane:v_plane + 16], v_codes)
    assert np.count_nonzero(got) == 16 + np.count_nonzero(v_codes)


def test_fused_write_validation_without_a_gpu():
    import ctypes

    from khalamari_amd import kv_page_write as kpw
    from khalamari_amd import rms_norm_rope as rnr
    from khalamari_amd._lib import Buffer, KNormRopePageWriteBuffers

    lib = _lib.lib()
    page = kpw.Config(2, 128, 2 * 2 * 16 * 128).as_struct()
    shape = kpw.Shape(4, kpw.PageTableLayout(1, 1, 1, 1)).as_struct()
    fake = Buffer(ctypes.c_void_p(4096), 1 << 30)
    buffers = KNormRopePageWriteBuffers(fake, fake, fake, fake, fake, fake, fake)

    def call(norm, fixed=4):
        return lib.khm_k_norm_rope_page_write(ctypes.byref(norm), ctypes.byref(page), ctypes.byref(shape), ctypes.byref(buffers),
                                              ReplayU32.fixed(fixed), ReplayU32.fixed(0), None, None)

    assert call(rnr.Config.bf16(3, 128, 128, 1e-6, 1e6).as_struct()) == _lib.KHM_ERR_INVALID_ARGUMENT
    assert b"do not match the page writer" in lib.khm_last_error()
    assert call(rnr.Config.f32(2, 128, 128, 1e-6, 1e6).as_struct()) == _lib.KHM_ERR_INVALID_ARGUMENT
    assert b"BF16 K and V rows" in lib.khm_last_error()
    assert call(rnr.Config.bf16(2, 128, 128, 1e-6, 1e6).as_struct(), fixed=5) == _lib.KHM_ERR_INVALID_ARGUMENT
    assert b"replay domain" in lib.khm_last_error()
    odd_page = kpw.Config(2, 12, 2 * 2 * 16 * 12).as_struct()
    status = lib.khm_k_norm_rope_page_write(ctypes.byref(rnr.Config.bf16(2, 12, 4, 1e-6, 1e6).as_struct()), ctypes.byref(odd_page), ctypes.byref(shape),
                                            ctypes.byref(buffers), ReplayU32.fixed(4), ReplayU32.fixed(0), None, None)
    assert status == _lib.KHM_ERR_UNSUPPORTED and b"khm_rms_norm_rope and khm_kv_page_write" in lib.khm_last_error()
