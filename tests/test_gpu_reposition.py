"""GPU parity of the block copy + key re-rotation launch (``lazyattn_reposition_blocks``) against the
CPU restatement of ``block_attn_vllm/utils.py:48-95``."""
import pytest
import torch

from oracle import deferred_rope as orc
from lazy_amd.block_attn import utils as ba

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _caches(dtype, d, hkv, nb, bs=16, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = 16 // torch.empty(0, dtype=dtype).element_size()
    kc = torch.randn(nb, hkv, d // x, bs, x, generator=g).to(dtype)
    vc = torch.randn(nb, hkv, d, bs, generator=g).to(dtype)
    table = orc.build_cos_sin_table(8192, d, 500000.0).to(dtype)
    return kc, vc, table


@pytest.mark.parametrize("dtype,d,tol", [(torch.bfloat16, 128, 4e-2), (torch.float32, 64, 2e-5), (torch.float16, 128, 5e-3)])
def test_copy_and_reposition_many_blocks(dtype, d, tol):
    print(f"case: reposition {dtype} d={d}", flush=True)
    kc, vc, table = _caches(dtype, d, 8 if d == 128 else 2, 40)
    g = torch.Generator().manual_seed(1)
    olds = torch.randperm(20, generator=g)[:11]
    items = [(20 + i, int(o), int(torch.randint(0, 3000, (1,), generator=g)), int(torch.randint(0, 8000, (1,), generator=g)))
             for i, o in enumerate(olds)]
    items.append((7, 7, 16, 2048))                                # in place
    items = [it for it in items if it[1] != 7 or it[0] == 7]
    kr, vr = kc.clone(), vc.clone()
    orc.reposition_blocks(kr, vr, items, table)
    kg, vg = kc.to(DEV), vc.to(DEV)
    ba.reposition_blocks(kg, vg, items, table.to(DEV))
    assert torch.equal(vg.cpu(), vr)                              # V is copied: bit-exact
    err = (kg.cpu().float() - kr.float()).abs().max().item()
    assert err < tol, err
    touched = {it[0] for it in items}
    rest = [b for b in range(40) if b not in touched]
    assert torch.equal(kg.cpu()[rest], kc[rest])                  # nothing else moved


def test_single_block_in_place_and_fp32_table():
    print("case: reposition one block, fp32 table", flush=True)
    kc, vc, table = _caches(torch.bfloat16, 128, 8, 6, seed=3)
    kr, vr = kc.clone(), vc.clone()
    orc.reposition_blocks(kr, vr, [(2, 2, 100, 37)], table.float())
    kg, vg = kc.to(DEV), vc.to(DEV)
    ba.place_paged_block_keys(kg, vg, 2, table.float().to(DEV), 100, 37)
    assert (kg.cpu().float() - kr.float()).abs().max() < 4e-2
    assert torch.equal(vg.cpu(), vc)


def test_moving_a_document_equals_encoding_it_at_the_target():
    """What the operation is for: keys cached at local positions, moved to their slot in the assembled
    sequence, equal (to bf16 accuracy) the keys rotated at the target positions directly."""
    print("case: reposition == direct rotation", flush=True)
    d, hkv, bs = 128, 2, 16
    g = torch.Generator().manual_seed(5)
    table = orc.build_cos_sin_table(4096, d, 500000.0).to(torch.bfloat16)
    raw = torch.randn(3 * bs, hkv, d, generator=g)
    local = orc.rotate_at(raw, torch.arange(3 * bs), table.float()).to(torch.bfloat16)
    kc = torch.zeros(8, hkv, d // 8, bs, 8, dtype=torch.bfloat16); vc = torch.zeros(8, hkv, d, bs, dtype=torch.bfloat16)
    for pg in range(3):
        kc[pg + 1] = local[pg * bs:(pg + 1) * bs].reshape(bs, hkv, d // 8, 8).permute(1, 2, 0, 3)
    kg, vg = kc.to(DEV), vc.to(DEV)
    ba.reposition_blocks(kg, vg, [(5 + pg, 1 + pg, pg * bs, 1000 + pg * bs) for pg in range(3)], table.to(DEV))
    want = orc.rotate_at(raw, 1000 + torch.arange(3 * bs), table.float())
    got = torch.cat([kg.cpu()[5 + pg].permute(2, 0, 1, 3).reshape(bs, hkv, d) for pg in range(3)]).float()
    assert (got - want).abs().max() < 8e-2                        # two bf16 table rows and two roundings apart
