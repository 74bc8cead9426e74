"""Host-side allocators the attention mirror takes from its callers (no GPU needed: the buffers
are CPU tensors here): the bump allocator of a step (serenitymojo/autograd_v2/step_slab.mojo:39-90)
and the scratch ring with marks (serenitymojo/scratch_ring.mojo:27-215)."""
import pytest

from mojodiffusion_amd import attention_sage as A


def test_step_slab_bumps_aligned_views_and_rewinds():
    slab = A.StepSlab(4096, device="cpu")
    a = slab.alloc(10)
    b = slab.alloc(300)
    assert a.data_ptr() % 256 == 0 and b.data_ptr() % 256 == 0
    assert b.data_ptr() >= a.data_ptr() + 10
    assert slab.used_bytes() >= 310 and slab.peak_bytes() == slab.used_bytes() and slab.n_allocs == 2
    with pytest.raises(A.Error, match="StepSlab: out of space"):
        slab.alloc(4096)
    slab.reset()
    assert slab.used_bytes() == 0 and slab.peak_bytes() >= 310
    assert slab.alloc(10).data_ptr() == a.data_ptr()


def test_scratch_ring_marks_and_slabs():
    ring = A.ScratchRingAllocator(4096, device="cpu")
    assert ring.capacity_bytes() == 0 and ring.used_bytes() == 0
    a = ring.alloc(100)
    m = ring.mark()
    b = ring.alloc(2000)
    assert a.data_ptr() % 256 == 0 and b.data_ptr() % 256 == 0
    c = ring.alloc(3000)                    # does not fit the first slab any more: a second one
    assert len(ring.slabs) == 2 and ring.capacity_bytes() == 8192
    assert ring.used_bytes() == 4096 + (c.data_ptr() - ring.slabs[1].data_ptr()) + 3000
    ring.rewind(m)
    assert ring.used_bytes() == (a.data_ptr() - ring.slabs[0].data_ptr()) + 100
    assert ring.alloc(2000).data_ptr() == b.data_ptr()       # the same memory again, no new slab
    assert len(ring.slabs) == 2
    ahead = ring.mark()
    ring.rewind(m)
    with pytest.raises(A.Error, match="ahead of the allocator"):
        ring.rewind(ahead)
    with pytest.raises(A.Error, match="exceeds the slab size"):
        ring.alloc(5000)
    ring.reset()
    assert ring.used_bytes() == 0 and c.numel() == 3000
