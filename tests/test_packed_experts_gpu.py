"""A written .gturbo packed_experts directory -> layout -> parallel reader -> pinned staging -> HBM pool,
then the decode layer on the loaded pool: the cells hold the file's bytes and the layer's output equals,
byte for byte, the one from a pool filled by direct uploads of the same blobs."""
import numpy as np
import pytest

from shrike_amd import capi, host
from shrike_amd import synth as S
from tests.helpers import Layer
from tests.test_decode_gpu import DeviceLayer

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("d,f,ne,k,bits,additive,staged_blobs", [
    (256, 128, 12, 4, 4, False, 3),      # a staging buffer of three blobs: halves of one blob each
    (512, 256, 16, 8, 8, False, 8),
    (256, 192, 8, 4, 4, True, 2),        # gpt-oss style additive biases in the blob
])
def test_pool_loaded_from_a_packed_experts_directory(gpu, tmp_path, d, f, ne, k, bits, additive, staged_blobs):
    L = Layer(0x5EED0041, d, f, ne, k, bits=bits, additive_biases=additive)
    kw = dict(moe_kwargs=dict(additive_biases=True, activation=capi.ACT_CLAMPED_SWIGLU)) if additive else {}
    direct = DeviceLayer(gpu, L, **kw)
    direct.moe.encode_decode_layer(direct.layer_args())
    want = (direct.y.download(np.uint16, d), direct.acts.download(np.uint16, k * f), direct.out_idx.download(np.uint32, k))

    # layer 0 is dense (no file), layer 1 holds the experts at permuted physical ranks
    rank_of = {e: int(r) for e, r in enumerate(np.random.default_rng(3).permutation(ne))}
    S.write_packed_experts(str(tmp_path), [[], L.blobs], d, f, bits, additive, physical_rank=lambda l, e: rank_of[e])
    layout = host.PackedExpertsLayout.load(str(tmp_path))
    assert (layout.num_layers, layout.experts_per_layer) == (2, ne)
    assert layout.layer(0)["expert_count"] == 0
    stride = layout.expert_stride
    assert stride % 16384 == 0 and stride >= L.stride
    off = layout.expert_offsets(1, additive)
    assert bytes(off) == bytes(direct.off), "offsets from the file differ from the packer's"

    from_file = DeviceLayer(gpu, L, resident=[], **kw)
    pool = gpu.ExpertPool(ne, stride, ne)
    from_file.pool = pool
    reader = host.ParallelExpertReader(str(tmp_path / "packed_experts" / layout.layer(1)["file"]), stride, threads=4,
                                       batch_depth=2)
    staging = gpu.PinnedBuffer(staged_blobs * stride)
    cells = [(e * 5 + 1) % ne if np.gcd(5, ne) == 1 else e for e in range(ne)]
    entries = [layout.expert(1, e) for e in range(ne)]
    assert [x["physical_rank"] for x in entries] == [rank_of[e] for e in range(ne)]
    stream = gpu.Stream()
    pool.fetch_experts(reader, [x["offset"] for x in entries], cells, stride, staging, stream)
    for e, cell in enumerate(cells):
        pool.publish(e, cell, capi.RESIDENT, stream)
    stream.synchronize()
    for e in (0, ne // 2, ne - 1):
        got = np.empty(L.stride, np.uint8)
        capi.check(capi.load().shrike_hip_memcpy_d2h(got.ctypes.data, pool.cell_ptr(cells[e]), got.nbytes), "memcpy_d2h")
        assert np.array_equal(got, L.blobs[e]), f"cell of expert {e} does not hold its blob"

    args = from_file.layer_args()
    args.offsets = off
    from_file.moe.encode_decode_layer(args)
    assert np.array_equal(from_file.out_idx.download(np.uint32, k), want[2])
    assert np.array_equal(from_file.acts.download(np.uint16, k * f), want[1])
    assert np.array_equal(from_file.y.download(np.uint16, d), want[0])

    # argument errors come back as errors
    with pytest.raises(capi.ShrikeError, match="two blobs"):
        pool.fetch_experts(reader, [0], [0], stride, gpu.PinnedBuffer(stride), stream)
    with pytest.raises(capi.ShrikeError, match="out of range"):
        pool.fetch_experts(reader, [0], [ne], stride, staging, stream)
    with pytest.raises(capi.ShrikeError, match="expert read failed"):
        pool.fetch_experts(reader, [ne * stride], [0], stride, staging, stream)
