"""The optimizer block of the reference's checkpoint, written from and read into the device arena
(include/anni_adam.h: anni_adam_export_mv / import_mv / write_state / read_state) against the
reference's own writer and loader (lang/lm_serialize.c:263-331,526-587) compiled from its tree:
byte for byte against lm_save_checkpoint, and read back by lm_load_checkpoint."""
import os
import struct

import numpy as np
import pytest

from helpers import same_bits

pytestmark = pytest.mark.gpu

F32, BF16 = 0, 1
DECAY, TWIN = 1, 2
RAGGED = [(5000, 3), (3, 0), (4096, 3), (1, 2), (0, 3), (8191, 1), (12288, 3), (7, 0), (4097, 3)]
CHUNK = 1 << 21      # lm_serialize.c:261


def make(tensors, **kw):
    from anni_amd.lm_adam import LmAdam
    return LmAdam(tensors, **kw)


def random_state(n, seed):
    rng = np.random.default_rng(seed)
    m = (rng.standard_normal(n) * 1e-2).astype(np.float32)
    v = (rng.standard_normal(n) ** 2 * 1e-4).astype(np.float32)
    return m, v


def test_export_is_the_interleave_of_m_and_v(gpu):
    opt = make(RAGGED, grad_slots=1)
    n = opt.n
    m, v = random_state(n, 1)
    opt.upload("m", m)
    opt.upload("v", v)
    pairs = opt.export_mv()
    assert pairs.shape == (n, 2) and same_bits(pairs[:, 0].copy(), m) and same_bits(pairs[:, 1].copy(), v)
    # a ragged inner range, odd start
    sub = opt.export_mv(first=4097, count=9001)
    assert same_bits(sub[:, 0].copy(), m[4097:4097 + 9001]) and same_bits(sub[:, 1].copy(), v[4097:4097 + 9001])
    assert opt.export_mv(first=n, count=0).shape == (0, 2)
    with pytest.raises(RuntimeError):
        opt.export_mv(first=n - 1, count=2)          # past the end
    opt.free()


def test_import_scatters_pairs_and_leaves_the_rest(gpu):
    opt = make(RAGGED, grad_slots=1)
    n = opt.n
    m, v = random_state(n, 2)
    opt.upload("m", m)
    opt.upload("v", v)
    m2, v2 = random_state(777, 3)
    opt.import_mv(np.stack([m2, v2], axis=1), first=1001)
    m[1001:1778], v[1001:1778] = m2, v2
    assert same_bits(opt.download("m"), m) and same_bits(opt.download("v"), v)
    with pytest.raises(RuntimeError):
        opt.import_mv(np.zeros((2, 2), np.float32), first=n - 1)
    opt.free()


def test_bf16_moments_widen_exactly_and_round_to_nearest_even(gpu, oracle):
    opt = make(RAGGED, moment_type=BF16, grad_slots=1)
    n = opt.n
    m, v = random_state(n, 4)
    # ties and specials: exactly half way between two bf16 values, both parities; zeros; a denormal
    m[:6] = np.array([0x3f808000, 0x3f818000, 0xbf808000, 0x00000000, 0x80000000, 0x00010000],
                     np.uint32).view(np.float32)
    opt.import_mv(np.stack([m, v], axis=1))
    mh, vh = oracle.bf16_rne(m), oracle.bf16_rne(v)
    assert (opt.download("m") == mh).all() and (opt.download("v") == vh).all()
    assert list(mh[:3]) == [0x3f80, 0x3f82, 0xbf80]       # ties to even
    pairs = opt.export_mv()
    assert same_bits(pairs[:, 0].copy(), oracle.bf16_widen(mh))
    assert same_bits(pairs[:, 1].copy(), oracle.bf16_widen(vh))
    opt.free()


def test_more_slots_than_two_staging_chunks(gpu):
    """2 chunks + a ragged third: both staging buffers are reused."""
    n = 2 * CHUNK + 12345
    opt = make([(n - 5, DECAY | TWIN), (5, 0)], grad_slots=1)
    m, v = random_state(n, 5)
    opt.import_mv(np.stack([m, v], axis=1))
    assert same_bits(opt.download("m"), m) and same_bits(opt.download("v"), v)
    pairs = opt.export_mv()
    assert same_bits(pairs[:, 0].copy(), m) and same_bits(pairs[:, 1].copy(), v)
    # a range crossing the chunk boundary from an odd start
    sub = opt.export_mv(first=CHUNK - 3, count=CHUNK + 7)
    assert same_bits(sub[:, 1].copy(), v[CHUNK - 3:2 * CHUNK + 4])
    opt.free()


def test_block_layout_and_resume(gpu, oracle, tmp_path):
    """write_state -> the five int32 and the pairs; read_state into a fresh arena; both continue
    with the same gradients to identical bits (t restored, so bias correction continues)."""
    opt = make(RAGGED, grad_slots=1, beta2=0.95, weight_decay=0.1, grad_clip=1.0)
    n = opt.n
    rng = np.random.default_rng(6)
    opt.upload("param", rng.standard_normal(n).astype(np.float32))
    for t in range(3):
        opt.upload("grad", rng.standard_normal(n).astype(np.float32))
        opt.step_scaled(1e-3, 0.5)
    path = str(tmp_path / "state.bin")
    fd = os.open(path, os.O_WRONLY | os.O_CREAT | os.O_TRUNC, 0o600)
    opt.write_state(fd, 2, 1234)
    os.close(fd)
    raw = open(path, "rb").read()
    assert len(raw) == 20 + 8 * n
    assert struct.unpack("=5i", raw[:20]) == (1, 2, 1234, 3, n)
    pairs = np.frombuffer(raw, np.float32, offset=20).reshape(n, 2)
    assert same_bits(pairs[:, 0].copy(), opt.download("m")) and same_bits(pairs[:, 1].copy(), opt.download("v"))

    res = make(RAGGED, grad_slots=1, beta2=0.95, weight_decay=0.1, grad_clip=1.0)
    res.upload("param", opt.download("param"))
    fd = os.open(path, os.O_RDONLY)
    assert res.read_state(fd) == (2, 1234) and res.t == 3
    os.close(fd)
    for t in range(2):
        g = rng.standard_normal(n).astype(np.float32)
        for o in (opt, res):
            o.upload("grad", g)
            o.step_scaled(1e-3, 0.5)
    for w in ("param", "m", "v"):
        assert same_bits(opt.download(w), res.download(w))
    assert opt.t == res.t == 5

    # what lm_load_checkpoint refuses (lm_serialize.c:546-562): has_adam != 1, another slot count, a short file
    def attempt(blob):
        p = str(tmp_path / "bad.bin")
        open(p, "wb").write(blob)
        fd = os.open(p, os.O_RDONLY)
        try:
            with pytest.raises(ValueError):
                res.read_state(fd)
        finally:
            os.close(fd)
    attempt(struct.pack("=5i", 0, 2, 1234, 3, n) + raw[20:])
    attempt(struct.pack("=5i", 1, 2, 1234, 3, n + 1) + raw[20:])
    attempt(raw[:20 + 8 * (n // 2)])
    attempt(raw[:12])
    opt.free()
    res.free()


def test_block_equals_reference_checkpoint_and_reference_loads_ours(gpu, oracle, tmp_path):
    """The reference's real model (its compile-time sizes; the byte vocabulary of lm_create, which
    is what its loader expects of a file without a tokenizer) trained two steps on this backend
    and saved by its own lm_save_checkpoint: the arena, given the same m / v / t, writes the same optimizer block byte for byte.  Then the other direction: the reference's
    weights section followed by a block written from a different arena state is a file the
    reference's lm_load_checkpoint accepts, and the m / v / t / epoch / step it loads are ours."""
    if not oracle.ref_hip_available():
        pytest.skip("oracle/_ref/libanni_ref_hip.so not built (reference tree absent at build time)")
    M = oracle.RefModelOnBackend(1, beta2=0.95, weight_decay=0.1, grad_clip=1.0)
    n = M.n
    rng = np.random.default_rng(8)
    for t in range(2):
        M.set_grads(rng.standard_normal(n, dtype=np.float32) * np.float32(1e-3))
        gpu.gpu_device_sync()
        M.step(3e-4, 1.0)
    assert M.on_device and M.t == 2
    ref_path = str(tmp_path / "ref_ckpt.bin")
    M.save_checkpoint(ref_path, 3, 4321)
    size = os.path.getsize(ref_path)
    head_len = size - (20 + 8 * n)
    assert head_len > 0
    m, v = M.moments()
    tensors = [(cnt, (DECAY | TWIN) if is_mat else DECAY) for _off, cnt, is_mat in M.segs()]
    M.close()
    gpu.gpu_adam_set_weight_decay(0.0)
    print("reference checkpoint: %d slots, weights section %d bytes" % (n, head_len), flush=True)

    opt = make(tensors, grad_slots=0, layout=1)
    assert opt.n == n
    opt.import_mv(np.stack([m, v], axis=1))
    opt.o.t = 2
    ours = str(tmp_path / "ours.bin")
    fd = os.open(ours, os.O_WRONLY | os.O_CREAT | os.O_TRUNC, 0o600)
    opt.write_state(fd, 3, 4321)
    os.close(fd)
    assert os.path.getsize(ours) == 20 + 8 * n
    with open(ref_path, "rb") as fr, open(ours, "rb") as fo:
        fr.seek(head_len)
        while True:
            a, b = fr.read(1 << 24), fo.read(1 << 24)
            assert a == b
            if not a:
                break
    print("optimizer block identical to lm_save_checkpoint's (%d bytes)" % (20 + 8 * n), flush=True)

    # the other direction
    m2, v2 = random_state(n, 9)
    opt.import_mv(np.stack([m2, v2], axis=1))
    opt.o.t = 77
    mixed = str(tmp_path / "mixed.bin")
    with open(ref_path, "rb") as fr, open(mixed, "wb") as fw:
        left = head_len
        while left:
            blk = fr.read(min(left, 1 << 24))
            fw.write(blk)
            left -= len(blk)
        fw.flush()
        opt.write_state(fw.fileno(), 5, 99)
    opt.free()
    os.remove(ref_path)
    os.remove(ours)
    L, ep, st = oracle.RefModelOnBackend.load_checkpoint(mixed, backend="cpu")
    assert (ep, st) == (5, 99) and L.t == 77 and L.n == n
    lm_, lv_ = L.moments()
    assert same_bits(lm_, m2) and same_bits(lv_, v2)
    L.close()
    print("lm_load_checkpoint read the arena's block: t, epoch, step, m, v as written", flush=True)
