"""The device-side producer of q_offset / q_mask against the host restatement of
``metadata_for_lazy_attention`` (scheduler.py:758-787) and the reference's own known answer
(tests/core/test_scheduler.py:36-61)."""
import pytest
import torch

from oracle import deferred_rope as orc
from lazy_amd.core.sched import metadata as md

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _pad(lens, bs):
    return [((l + bs - 1) // bs) * bs for l in lens]


def test_known_answer_from_the_reference_tests():
    print("case: metadata KAT", flush=True)
    lens, padded = [[6, 15, 8, 2]], [[8, 16, 8, 8]]
    qo = torch.full((1, 9), 7, dtype=torch.int32, device=DEV); qm = torch.full_like(qo, 7)
    mx = torch.zeros(1, dtype=torch.int32, device=DEV)
    md.build_rotation_metadata_device(lens, padded, 8, qo, qm, max_offset=mx)
    assert qo[0].tolist() == [10, 16, 16, 31, 39, 1, 0, 0, 0]
    assert qm[0].tolist() == [2, 0, 1, 0, 6, 0, 0, 0, 0]
    assert int(mx[0]) == 39 == md.max_rotation_offset(lens[0], padded[0])
    md.build_rotation_metadata_device(lens, padded, 8, qo, qm, mepic=True)
    assert qo[0].tolist() == [0] * 9 and qm[0].tolist() == [2, 0, 1, 0, 6, 0, 0, 0, 0]


def test_random_batches_match_the_host_function():
    print("case: metadata random batches", flush=True)
    g = torch.Generator().manual_seed(0)
    for bs in (8, 16, 32):
        lens = [[int(x) for x in torch.randint(1, 700, (int(n),), generator=g)]
                for n in torch.randint(0, 400, (17,), generator=g)]
        lens[3] = []                                              # a request without documents
        padded = [_pad(l, bs) for l in lens]
        row_len = max(sum(p) // bs + 1 for p in padded) + 3
        qo = torch.full((17, row_len), -1, dtype=torch.int32, device=DEV); qm = torch.full_like(qo, -1)
        mx = torch.zeros(17, dtype=torch.int32, device=DEV)
        md.build_rotation_metadata_device(lens, padded, bs, qo, qm, max_offset=mx)
        for b in range(17):
            ro, rm = orc.metadata_for_lazy_attention(lens[b], padded[b], bs)
            ro = ro + [0] * (row_len - len(ro)); rm = rm + [0] * (row_len - len(rm))
            assert qo[b].tolist() == ro and qm[b].tolist() == rm, (bs, b)
            assert int(mx[b]) == orc.max_rotation_offset(lens[b], padded[b])


def test_buffers_too_small_is_refused_on_the_host():
    qo = torch.zeros(1, 4, dtype=torch.int32, device=DEV); qm = torch.zeros_like(qo)
    with pytest.raises(ValueError):
        md.build_rotation_metadata_device([[100]], [[112]], 16, qo, qm)


def test_packed_block_table_full_and_delta():
    print("case: packed block table", flush=True)
    from lazy_amd.attention.ops.chunked_prefill_paged_decode import unpack_block_table
    g = torch.Generator().manual_seed(2)
    bt = torch.randint(0, 2 ** 31 - 1, (9, 40), generator=g, dtype=torch.int32)
    qo = torch.randint(0, 0x10000, (9, 40), generator=g, dtype=torch.int32)
    qm = torch.randint(0, 17, (9, 40), generator=g, dtype=torch.int32)
    want = (bt.long() << 32) | (qo.long() << 16) | qm.long()          # gpu_model_runner.py:325-331
    packed = torch.zeros(9, 40, dtype=torch.int64, device=DEV)
    md.pack_block_table_device(bt.to(DEV), qo.to(DEV), qm.to(DEV), packed)
    assert torch.equal(packed.cpu(), want)
    blk, off, msk = unpack_block_table(packed)
    assert torch.equal(blk.cpu(), bt) and torch.equal(off.cpu(), qo) and torch.equal(msk.cpu(), qm)
    packed.zero_()
    md.pack_block_table_device(bt.to(DEV), qo.to(DEV), qm.to(DEV), packed, rows=[7, 2])
    got = packed.cpu()
    assert torch.equal(got[[7, 2]], want[[7, 2]]) and int(got[[0, 1, 3, 4, 5, 6, 8]].abs().sum()) == 0
