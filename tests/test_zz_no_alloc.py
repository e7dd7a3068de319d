"""dn_attention_decode_static: the split decode attention for callers that cannot allocate device
memory.  Called through ctypes, it must give what dn_attention_decode gives with a workspace that
the caller brought, bit for bit, on two calls in a row (the second with a smaller input, so that the
library's own array still holds the first call's results), and refuse what its array cannot hold."""
import ctypes
import math
from ctypes import c_float, c_int, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

SCRATCH_FLOATS = 256 * 1024      # DN_DECODE_STATIC_SCRATCH_FLOATS of csrc/kernels/attention.h
ERR_SCRATCH = -3


def library():
    from denno_beta_amd.build import load_library
    lib = ctypes.CDLL(load_library("attention")._name)      # a handle of this test's own: no declared signatures
    P, I, F = c_void_p, c_int, c_float
    lib.dn_attention_decode.argtypes = [P, I, P, I, P, P, P, I, P, P, P, I, P, I, I, I, I, I, I, I, F, I, P]
    lib.dn_attention_decode_static.argtypes = [P, I, P, I, P, P, P, I, P, P, P, I, I, I, I, I, I, I, I, F, I, P]
    lib.dn_attention_decode.restype = lib.dn_attention_decode_static.restype = c_int
    return lib


def case(seq_lens, H, Hkv, dh, ps, seed):
    """A cache of random keys and values for requests of these lengths on shuffled pages, and the
    tables of a step in which each brings one row."""
    g = torch.Generator().manual_seed(seed)
    blocks = [-(-n // ps) for n in seq_lens]
    n_pages = sum(blocks) + 2
    perm = torch.randperm(n_pages, generator=g).tolist()
    k = torch.randn(n_pages, Hkv, ps, dh, generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn(n_pages, Hkv, dh, ps, generator=g).to(torch.bfloat16).to(DEV)
    bt = torch.full((len(seq_lens), max(blocks)), -1, dtype=torch.int32)
    for s in range(len(seq_lens)):
        for b in range(blocks[s]):
            bt[s, b] = perm.pop()
    S = len(seq_lens)
    tiles = torch.tensor([list(range(S)), list(range(S)), [1] * S, [n - 1 for n in seq_lens]], dtype=torch.int32)
    q = torch.randn(S, H * dh, generator=g).to(torch.bfloat16).to(DEV)
    return q, k, v, bt.to(DEV), tiles.to(DEV).contiguous()


def both(lib, seq_lens, H, Hkv, dh, ps, waves, n_splits, seed):
    q, k, v, bt, tiles = case(seq_lens, H, Hkv, dh, ps, seed)
    S = len(seq_lens)
    chunks = -(-(-(-max(seq_lens) // (waves * 64))) // n_splits)
    assert n_splits > 1 and n_splits * chunks * waves * 64 >= max(seq_lens)
    base = tiles.data_ptr()
    stream = torch.cuda.current_stream().cuda_stream
    scale = 1.0 / math.sqrt(dh)
    common = (q.data_ptr(), q.stride(0))
    tables = (k.data_ptr(), v.data_ptr(), bt.data_ptr(), bt.shape[1], base, base + 4 * S, base + 12 * S, S)
    rest = (n_splits, chunks, waves, H, Hkv, dh, ps, scale, 0, stream)
    want = torch.zeros(S, H * dh, dtype=torch.bfloat16, device=DEV)
    part = torch.full((S * H * n_splits * (dh + 2),), float("nan"), dtype=torch.float32, device=DEV)
    assert lib.dn_attention_decode(*common, want.data_ptr(), want.stride(0), *tables, part.data_ptr(), *rest) == 0
    got = torch.zeros(S, H * dh, dtype=torch.bfloat16, device=DEV)
    free_before = torch.cuda.mem_get_info()[0]
    assert lib.dn_attention_decode_static(*common, got.data_ptr(), got.stride(0), *tables, *rest) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the call took or gave back device memory"
    assert bool(want.float().abs().sum() > 0) and not bool(torch.isnan(want.float()).any())
    assert torch.equal(got, want), (seq_lens, n_splits)


def test_two_calls_in_a_row_the_second_smaller():
    lib = library()
    # contexts on both sides of a split's edge; a request whose last splits are empty
    both(lib, [1000, 257, 640, 30, 1024], H=5, Hkv=5, dh=64, ps=16, waves=4, n_splits=4, seed=1)
    both(lib, [300, 513], H=3, Hkv=1, dh=32, ps=32, waves=4, n_splits=3, seed=2)
    both(lib, [1000, 257, 640, 30, 1024], H=5, Hkv=5, dh=64, ps=16, waves=4, n_splits=2, seed=3)


def test_it_refuses_more_than_its_array_holds():
    lib = library()
    q, k, v, bt, tiles = case([64], 2, 2, 64, 16, 0)
    base = tiles.data_ptr()
    out = torch.full((1, 128), 7.0, dtype=torch.bfloat16, device=DEV)
    # n_tiles * H * n_splits * (dh + 2) floats beyond the array: nothing may be launched
    n_tiles = SCRATCH_FLOATS // (2 * 2 * 66) + 1
    rc = lib.dn_attention_decode_static(q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), k.data_ptr(),
                                        v.data_ptr(), bt.data_ptr(), bt.shape[1], base, base + 4, base + 12, n_tiles,
                                        2, 1, 4, 2, 2, 64, 16, 0.125, 0, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == ERR_SCRATCH and bool((out == 7.0).all())
