"""The entry point that allocates nothing (redmetal_ffn_pool_execute_expert_noalloc): same computation as
redmetal_ffn_pool_execute_expert, on device pointers and a stream, with its activations in an array that is part of the library's
device image. Checked bit for bit against the existing entry point (same kernels, same order of operations), on two calls in a
row of which the second is the smaller one, so stale contents of the shared scratch would show."""
import numpy as np
import pytest

import oracle_lib as orc
from dwarfstar_red_lite_amd import expert_type_word, synth
from gpu_common import REL_L2_TOL, T_IQ2, T_IQ3, T_Q6K, rel_l2

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def test_noalloc_matches_execute_expert_on_two_calls_in_a_row(tmp_path):
    from dwarfstar_red_lite_amd import RedHipError
    from dwarfstar_red_lite_amd.redmetal_ffn import ExpertLayout, RedMetalFfnPool
    rng = np.random.default_rng(707)
    # a large expert and a small one (the second call's ffn is half the first's), different formats
    shapes = [(1024, 512, T_IQ2, T_IQ3), (512, 256, T_Q6K, T_Q6K), (768, 256, T_IQ2, T_IQ2)]
    parts, off, lays = [np.zeros(10, np.uint8)], 10, []
    for H, F, gu, dn in shapes:
        mats = [synth.quant_rows(rng, gu, F, H), synth.quant_rows(rng, gu, F, H), synth.quant_rows(rng, dn, H, F)]
        rng_off = []
        for mtx in mats:
            b = mtx.reshape(-1)
            rng_off += [off, b.size]
            parts.append(b)
            off += b.size
        lays.append(ExpertLayout(*rng_off))
    blob = np.concatenate(parts)
    path = tmp_path / "experts.bin"
    blob.tofile(path)
    slot_bytes = max(l.gate_bytes + l.up_bytes + l.down_bytes for l in lays)
    stream = torch.cuda.Stream()
    with RedMetalFfnPool(str(path), 4 * (slot_bytes + 4096), slot_bytes, slots_per_slab=2) as pool:
        xs = [synth.normed_x(rng, 1, H)[0] for H, _, _, _ in shapes]
        # a slot that was never loaded has no memory behind it, and this call will not make any
        with pytest.raises(RedHipError, match="holds no expert"):
            pool.execute_noalloc(0, lays[0], expert_type_word(T_IQ2, T_IQ3), 1024, 512, 0, 1024, torch.zeros(1024, device="cuda").data_ptr(),
                                 torch.zeros(1024, device="cuda").data_ptr(), stream.cuda_stream)
        # nor does a slot whose slab exists (slot 0 shares it) but which itself was never loaded pass
        pool.load(0, lays[0])
        with pytest.raises(RedHipError, match="holds no expert"):
            pool.execute_noalloc(1, lays[1], expert_type_word(T_Q6K, T_Q6K), 512, 256, 0, 512, torch.zeros(512, device="cuda").data_ptr(),
                                 torch.zeros(512, device="cuda").data_ptr(), stream.cuda_stream)
        for slot, lay in enumerate(lays):
            pool.load(slot, lay)
        want = [pool.execute(slot, lays[slot], expert_type_word(gu, dn), H, F, 0, H, xs[slot])[0] for slot, (H, F, gu, dn) in enumerate(shapes)]
        # (the existing entry point against the CPU path, so that "equal to it" means "right")
        for slot, (H, F, gu, dn) in enumerate(shapes):
            l = lays[slot]
            ref = orc.expert_ffn(gu, dn, blob[l.gate_offset:l.gate_offset + l.gate_bytes], blob[l.up_offset:l.up_offset + l.up_bytes],
                                 blob[l.down_offset:l.down_offset + l.down_bytes], H, F, xs[slot])
            assert rel_l2(want[slot], ref) <= REL_L2_TOL
        xd = [torch.from_numpy(x).cuda() for x in xs]
        outs = [torch.full((H,), float("nan"), device="cuda") for H, _, _, _ in shapes]
        torch.cuda.synchronize()
        # two (three) calls in a row on one stream, large first, nothing between them
        for slot, (H, F, gu, dn) in enumerate(shapes):
            pool.execute_noalloc(slot, lays[slot], expert_type_word(gu, dn), H, F, 0, H, xd[slot].data_ptr(), outs[slot].data_ptr(), stream.cuda_stream)
        stream.synchronize()
        for slot in range(len(shapes)):
            assert np.array_equal(outs[slot].cpu().numpy(), want[slot]), slot
        # again in the other order, with a row window on the large one
        win = torch.full((12,), float("nan"), device="cuda")
        small = torch.full((512,), float("nan"), device="cuda")
        pool.execute_noalloc(1, lays[1], expert_type_word(T_Q6K, T_Q6K), 512, 256, 0, 512, xd[1].data_ptr(), small.data_ptr(), stream.cuda_stream)
        pool.execute_noalloc(0, lays[0], expert_type_word(T_IQ2, T_IQ3), 1024, 512, 1000, 12, xd[0].data_ptr(), win.data_ptr(), stream.cuda_stream)
        stream.synchronize()
        assert np.array_equal(small.cpu().numpy(), want[1]) and np.array_equal(win.cpu().numpy(), want[0][1000:1012])
        # the limit of the static scratch is checked before anything is launched
        big = lays[0]._replace(gate_bytes=16640 * 264, up_bytes=16640 * 264)
        with pytest.raises(RedHipError, match="exceeds the static scratch"):
            pool.execute_noalloc(0, big, T_IQ2, 1024, 16640, 0, 1024, xd[0].data_ptr(), outs[0].data_ptr(), stream.cuda_stream)
        with pytest.raises(RedHipError, match="invalid FFN dimensions"):
            pool.execute_noalloc(0, lays[0], expert_type_word(T_IQ2, T_IQ3), 1024, 512, 1024, 1, xd[0].data_ptr(), outs[0].data_ptr(), stream.cuda_stream)
