"""The streaming GEMM variants ("_s2x4": one workgroup per compute unit walks its share of the output tiles, the operand
ring running on from tile to tile, the epilogue in registers) against the CPU oracle (cpu_gemm,
cutile-examples/examples/persistent_gemm.rs:140-152, on bf16 / f16 operands) and against the one-tile-per-workgroup
kernel on the same inputs: both accumulate the same K tiles in the same order and round once, so they agree bit for
bit.  Shapes: fewer tiles than compute units, more (a workgroup then computes two or three tiles and the ring crosses
tile boundaries at different phases of its six-tile cycle), the smallest K the variant takes, z through the caches and
past them, z as the initial accumulator and not."""
import numpy as np
import pytest
import torch

import oracle
from util import normal_bf16_bits, normal_f16_bits, rel_l2, to_dev_bf16, to_dev_f16

pytestmark = pytest.mark.gpu

CASES = [
    # m, n, k, accumulate
    (512, 512, 192, True),          # 4 tiles, 3 K tiles: the least the variant takes
    (512, 768, 256, False),
    (2048, 4096, 448, True),        # 128 tiles, 7 K tiles: one tile per workgroup
    (4352, 4352, 320, True),        # 289 tiles: some workgroups compute two; 5 K tiles: boundaries at odd phases
    (4352, 4352, 320, False),
    (8192, 4096, 512, True),        # 512 tiles, two per workgroup; z of 64 MiB: read and stored past the caches
    (6144, 8192, 704, False),       # 768 tiles, three per workgroup; 11 K tiles
]


def _run(ct, z, a, b, k, accumulate, variant):
    ct.gemm(ct.partition(z, [256, 256]), a, b, k, accumulate=accumulate, variant=variant)
    torch.cuda.synchronize()


@pytest.mark.parametrize("m,n,k,accumulate", CASES)
def test_gemm_stream_bf16(ct, dev, m, n, k, accumulate):
    print(f"gemm stream bf16 {m}x{n}x{k} acc={accumulate}", flush=True)
    a, b = normal_bf16_bits((m, k), 7000 + m, k ** -0.5), normal_bf16_bits((k, n), 7001 + n, k ** -0.5)
    z0 = normal_bf16_bits((m, n), 7002 + k, 0.5) if accumulate else np.zeros((m, n), np.uint16)
    ad, bd = to_dev_bf16(a, dev), to_dev_bf16(b, dev)
    z = to_dev_bf16(z0, dev).clone()
    if not accumulate:
        z.fill_(float("nan"))                       # every element must be written
    _run(ct, z, ad, bd, k, accumulate, "bf16_256x256x64_s2x4")
    assert ct.last_resolved()["variant"] == "bf16_256x256x64_s2x4"
    want = to_dev_bf16(z0, dev).clone()
    _run(ct, want, ad, bd, k, accumulate, "bf16_256x256x64_q2x4")
    assert torch.equal(z.view(torch.int16), want.view(torch.int16))
    ref = oracle.gemm_bf16(a, b, f32out=True) + (oracle.bf16_bits_to_f32(z0) if accumulate else 0.0)
    assert rel_l2(z.float().cpu().numpy(), ref) <= 1e-2


@pytest.mark.parametrize("m,n,k,accumulate", [(1024, 512, 256, True), (4352, 4352, 192, False)])
def test_gemm_stream_f16(ct, dev, m, n, k, accumulate):
    print(f"gemm stream f16 {m}x{n}x{k} acc={accumulate}", flush=True)
    a, b = normal_f16_bits((m, k), 7100 + m, k ** -0.5), normal_f16_bits((k, n), 7101 + n, k ** -0.5)
    z0 = normal_f16_bits((m, n), 7102 + k, 0.5) if accumulate else np.zeros((m, n), np.uint16)
    ad, bd = to_dev_f16(a, dev), to_dev_f16(b, dev)
    z = to_dev_f16(z0, dev).clone()
    _run(ct, z, ad, bd, k, accumulate, "f16_256x256x64_s2x4")
    want = to_dev_f16(z0, dev).clone()
    _run(ct, want, ad, bd, k, accumulate, "f16_256x256x64_q2x4")
    assert torch.equal(z.view(torch.int16), want.view(torch.int16))
    ref = oracle.f16_bits_to_f32(a).astype(np.float64) @ oracle.f16_bits_to_f32(b).astype(np.float64)
    ref = ref + (oracle.f16_bits_to_f32(z0) if accumulate else 0.0)
    assert rel_l2(z.float().cpu().numpy(), ref) <= 1e-2


def test_gemm_stream_is_not_offered_for_ragged_shapes(ct, dev):
    """partial tiles or fewer than three K tiles: the variant does not fit and the launcher says so (a K that is not a
    multiple of 64 runs k / 64 whole K tiles, as the tile program does, and fits)"""
    bf = torch.bfloat16
    for m, n, k in ((500, 512, 256), (512, 520, 256), (512, 512, 128), (512, 512, 160)):
        z = torch.zeros(m, n, dtype=bf, device=dev)
        a, b = torch.zeros(m, k, dtype=bf, device=dev), torch.zeros(k, n, dtype=bf, device=dev)
        with pytest.raises(ct.CutileError, match="does not fit these arguments"):
            ct.gemm(ct.partition(z, [256, 256]), a, b, k, variant="bf16_256x256x64_s2x4")
    # and a member of the family is not a variant a caller can name
    z = torch.zeros(512, 512, dtype=bf, device=dev)
    a, b = torch.zeros(512, 256, dtype=bf, device=dev), torch.zeros(256, 512, dtype=bf, device=dev)
    with pytest.raises(ct.CutileError, match="does not fit these arguments"):
        ct.gemm(ct.partition(z, [256, 256]), a, b, 256, variant="bf16_256x256x64_s2x4+new")


def test_gemm_persistent_stream_matches_the_tile_kernel(ct, dev):
    """the persistent GEMM over a mapped partition on the streaming body: the reference's grouped schedule
    (GROUP_SIZE_M = 8), 96 tile blocks over 17 x 17 tiles, against the plain launch from zero accumulators"""
    m = n = 4352
    k = 448
    a, b = normal_bf16_bits((m, k), 7200, k ** -0.5), normal_bf16_bits((k, n), 7201, k ** -0.5)
    ad, bd = to_dev_bf16(a, dev), to_dev_bf16(b, dev)
    z = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ct.gemm_persistent(ct.mapped(ct.partition(z, [256, 256]), [8, 1], 96), ad, bd, variant="bf16_256x256x64_s2x4")
    torch.cuda.synchronize()
    want = torch.zeros(m, n, dtype=torch.bfloat16, device=dev)
    _run(ct, want, ad, bd, k, False, "bf16_256x256x64_q2x4")
    assert torch.equal(z.view(torch.int16), want.view(torch.int16))
