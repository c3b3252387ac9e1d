"""The PSH bucketing entry point that allocates nothing (f3d_batch_psh_scatter_pad_hash_noalloc: scratch memory in a
fixed array inside the library) against the allocating entry point, through the C ABI: every output bit for bit, on
calls in a row that share the array, each smaller than the one before."""
import numpy as np
import pytest
import torch

from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


def _run(coords, seps, bucket_size, hash_op, no_alloc):
    from flash3dtransformer_amd.lib import pshattn
    from flash3dtransformer_amd.psh import psh_main
    nb, div, mx = psh_main.bucket_geometry(seps, bucket_size)
    n = coords.shape[0]
    pad_to = -(-n // bucket_size) * bucket_size
    buf = psh_main.BucketScatterBuffers.create_buffers(coords, seps, bucket_size, pad_to, nb)
    bb_min, bb_max = coords.min(0)[0].contiguous(), coords.max(0)[0].contiguous()
    torch.cuda.synchronize()
    # free device memory as the driver counts it: sees a hipMalloc / hipFree inside the library, which torch's own
    # allocation counter does not (the allocating entry point may grow the library's workspace: not held to this)
    free_before = torch.cuda.mem_get_info()[0]
    before = torch.cuda.memory_allocated()
    pshattn.batch_psh_scatter_pad_hash(coords, buf.bucket_id, buf.bucket_cntr, buf.bucket_offs, seps, mx, nb, div,
                                       bucket_size, 0xFFFF, bb_min, bb_max, buf.probe_offs, buf.bucket_cumsum,
                                       buf.scattered_coord, 0.0, hash_op, no_alloc=no_alloc)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    if no_alloc:
        assert torch.cuda.mem_get_info()[0] == free_before, "the entry point that allocates nothing changed free device memory"
    return buf


def _same(a, b):
    for name in ("bucket_id", "bucket_cntr", "bucket_offs", "bucket_cumsum", "scattered_coord"):
        x, y = getattr(a, name), getattr(b, name)
        bits = {2: torch.int16, 4: torch.int32}[x.element_size()]
        assert torch.equal(x.view(bits), y.view(bits)), name


def test_no_alloc_entry_point_matches_the_allocating_one_on_calls_in_a_row():
    import bench_workloads as configs
    synth = configs
    from flash3dtransformer_amd.lib import pshattn
    pshattn.DeviceManagerSingleton.instance().init_dev_info(0)
    pshattn.DeviceManagerSingleton.instance().set_psh_rebalance(1)
    g = torch.Generator().manual_seed(11)
    cases = []
    # 64 clouds x 65,536 uniform points: the 8192-point-tile configuration, 512 tiles
    cases.append(((torch.rand(64 * 65536, 3, generator=g) * 51.2).to(torch.float16).to(DEV),
                  (torch.arange(1, 65, dtype=torch.int32) * 65536).to(DEV).view(torch.uint32), 512, 1))
    # 4 LiDAR sweeps x 120,000 points (overflowing buckets: rebalance plan in use), then ragged small clouds, then one
    coords, seps, _ = configs.lidar_batch(4, 120_000, 1004)
    cases.append(configs.to_device(coords, seps, DEV) + (512, 2))
    rng = np.random.default_rng(5)
    coords, seps = synth.batch_of([rng.normal(0, 10, (m, 3)).astype(np.float32) for m in (20000, 17001, 30011)])
    cases.append(configs.to_device(coords, seps, DEV) + (256, 3))
    coords, seps = synth.batch_of([synth.uniform_cube(32768, 51.2, 1001)])
    cases.append(configs.to_device(coords, seps, DEV) + (512, 4))
    want = [_run(c, s, bs, h, False) for c, s, bs, h in cases]
    got = [_run(c, s, bs, h, True) for c, s, bs, h in cases]          # back to back on the shared array
    for a, b in zip(got, want):
        _same(a, b)
    # and interleaved with the allocating entry point, smallest first this time
    for (c, s, bs, h), w in reversed(list(zip(cases, want))):
        _same(_run(c, s, bs, h, True), w)


def test_no_alloc_entry_point_says_when_a_batch_does_not_fit():
    from flash3dtransformer_amd.lib import pshattn
    from flash3dtransformer_amd.psh import psh_main
    # 256 clouds x 262,144 points: 256 x 32 tiles x 512 buckets of histogram (16 MiB) exceed the array
    n_c, b = 262144, 256
    coords = torch.zeros(n_c * b, 3, dtype=torch.float16, device=DEV)
    seps = (torch.arange(1, b + 1, dtype=torch.int32) * n_c).to(DEV).view(torch.uint32)
    nb, div, mx = psh_main.bucket_geometry(seps, 512)
    buf = psh_main.BucketScatterBuffers.create_buffers(coords, seps, 512, n_c * b, nb)
    bb = torch.zeros(3, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="scratch"):
        pshattn.batch_psh_scatter_pad_hash(coords, buf.bucket_id, buf.bucket_cntr, buf.bucket_offs, seps, mx, nb, div,
                                           512, 0xFFFF, bb, bb + 1, buf.probe_offs, buf.bucket_cumsum,
                                           buf.scattered_coord, 0.0, 1, no_alloc=True)


def test_no_alloc_entry_point_in_a_captured_graph_replays_to_the_eager_result():
    """A caller that captures its stream (the kind of caller the entry point is for): the call sits in a HIP graph next
    to the fill kernel that clears the counters; every replay, with eager work and synchronisations of the program in
    between, leaves exactly what the eager call leaves."""
    import bench_workloads as configs
    from flash3dtransformer_amd.lib import pshattn
    from flash3dtransformer_amd.psh import psh_main
    pshattn.DeviceManagerSingleton.instance().init_dev_info(0)
    pshattn.DeviceManagerSingleton.instance().set_psh_rebalance(1)
    # the optional synchronisation around every op stays switched on, as earlier tests leave it: the library must not
    # synchronise a stream that is being captured
    mgr = pshattn.DeviceManagerSingleton.instance()
    was_syncing = mgr.get_sync_stream()
    mgr.set_sync_stream(True)
    try:
        _graph_replays(configs, pshattn, psh_main)
    finally:
        mgr.set_sync_stream(was_syncing)


def _graph_replays(configs, pshattn, psh_main):
    coords, seps, _ = configs.lidar_batch(2, 60_000, 1010)
    coords, seps = configs.to_device(coords, seps, DEV)
    nb, div, mx = psh_main.bucket_geometry(seps, 512)
    pad_to = -(-coords.shape[0] // 3072) * 3072
    buf = psh_main.BucketScatterBuffers.create_buffers(coords, seps, 512, pad_to, nb)
    bb_min, bb_max = coords.min(0)[0].contiguous(), coords.max(0)[0].contiguous()

    def run():
        buf.bucket_cntr.zero_()
        pshattn.batch_psh_scatter_pad_hash(coords, buf.bucket_id, buf.bucket_cntr, buf.bucket_offs, seps, mx, nb, div,
                                           512, 0xFFFF, bb_min, bb_max, buf.probe_offs, buf.bucket_cumsum,
                                           buf.scattered_coord, 0.0, 2, no_alloc=True)
    names = ("bucket_id", "bucket_cntr", "bucket_offs", "bucket_cumsum", "scattered_coord")
    run()
    torch.cuda.synchronize()
    want = {n: getattr(buf, n).clone() for n in names}
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        run()                                      # warm-up on the capture stream
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            run()
    torch.cuda.synchronize()
    for _ in range(4):
        for n in ("bucket_id", "bucket_offs", "bucket_cumsum", "scattered_coord"):
            getattr(buf, n).view(torch.int16).fill_(0x3C00)         # stale contents the replay must overwrite
        x = torch.randn(512, 512, device=DEV)
        assert torch.isfinite((x @ x).sum()).item()                 # eager work and a synchronisation in between
        graph.replay()
        torch.cuda.synchronize()
        for n in names:
            bits = {2: torch.int16, 4: torch.int32}[want[n].element_size()]
            assert torch.equal(getattr(buf, n).view(bits), want[n].view(bits)), n
