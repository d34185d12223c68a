"""The entry point that allocates nothing (csrc/no_alloc.h), called through ctypes as a
foreign caller would: its output equals the existing entry point's, on two calls in a row,
the second with a smaller input; a call beyond the static buffer is refused."""
import ctypes
from ctypes import c_float, c_int, c_void_p

import numpy as np
import pytest
import torch

import plain_llama as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NH, NKV, DH = 8, 2, 128


def _case(lens, seed):
    """A paged cache with shuffled pages that holds every key and value of the sequences, and
    one rotated query row per sequence."""
    from transformer_amd import kernels
    r = np.random.default_rng(seed)
    B = len(lens)
    need = [-(-n // 64) for n in lens]
    n_pages = sum(need) + 3
    order = [int(x) for x in r.permutation(n_pages)]
    table = np.zeros((B, max(need)), dtype=np.int32)
    k = P.round_bf16(r.normal(size=(n_pages, NKV, 64, DH)))
    v = P.round_bf16(r.normal(size=(n_pages, NKV, 64, DH)))
    q = P.round_bf16(r.normal(size=(B, NH, DH)))
    at = 0
    for b in range(B):
        table[b, :need[b]] = order[at:at + need[b]]
        at += need[b]
    units, seq_units = kernels.uniform_key_units(lens, 2, table)      # several units per sequence
    want = []
    for b in range(B):
        pages = table[b, :need[b]]
        kk = k[pages].transpose(0, 2, 1, 3).reshape(-1, NKV, DH)[:lens[b]]
        vv = v[pages].transpose(0, 2, 1, 3).reshape(-1, NKV, DH)[:lens[b]]
        want.append(P.attention(q[b:b + 1], kk, vv, DH ** -0.5, first_pos=lens[b] - 1)[0])
    t = lambda a, dt: torch.tensor(np.ascontiguousarray(a), dtype=dt, device=DEV)
    return dict(
        q=t(q.reshape(B, NH * DH), torch.bfloat16), k=t(k, torch.bfloat16),
        v=t(v.transpose(0, 1, 3, 2), torch.bfloat16),                  # value pages are [dh][64]
        table=t(table, torch.int32), pos0=t([n - 1 for n in lens], torch.int32),
        cu=t(list(range(B + 1)), torch.int32), units=t(units, torch.int32),
        seq_units=t(seq_units, torch.int32), want=np.stack(want).reshape(B, NH * DH), lens=lens)


def _no_alloc(lib, c, out, n_units=None):
    p = lambda x: c_void_p(x.data_ptr() if x is not None else 0)
    B = c["q"].shape[0]
    return lib.ta_attention_keys_bf16_noalloc(
        c_void_p(torch.cuda.current_stream().cuda_stream), p(c["q"]), c_int(c["q"].stride(0)), p(None), p(None),
        c_int(0), p(None), p(out), c_int(out.stride(0)), p(c["k"]), p(c["v"]), p(c["table"]),
        c_int(c["table"].shape[1]), p(c["pos0"]), c_int(B), c_int(NH), c_int(NKV), c_int(DH),
        c_float(DH ** -0.5), c_int(0), p(c["units"]), p(c["seq_units"]),
        c_int(c["units"].shape[0] if n_units is None else n_units), c_int(0))


def test_attention_without_allocation_equals_the_existing_entry_point():
    from transformer_amd import kernels
    lib = kernels.library()
    lib.ta_noalloc_scratch_floats.restype = ctypes.c_longlong
    room = lib.ta_noalloc_scratch_floats()
    assert room == 1 << 20
    for lens, seed in (([700, 65, 300, 1, 512], 1), ([130, 64], 2)):        # the second is smaller
        c = _case(lens, seed)
        assert c["units"].shape[0] > len(lens)                                # scratch is really used
        assert c["units"].shape[0] * NH * (DH + 2) <= room
        ref = torch.full((len(lens), NH * DH), float("nan"), dtype=torch.bfloat16, device=DEV)
        kernels.attention_keys(c["q"], ref, c["k"], c["v"], c["table"], c["cu"], c["pos0"], max(lens),
                               NH, NKV, DH, DH ** -0.5, units=c["units"], seq_units=c["seq_units"])
        out = torch.full_like(ref, float("nan"))
        free_before = torch.cuda.mem_get_info()[0]
        rc = _no_alloc(lib, c, out)
        torch.cuda.synchronize()
        assert rc == 0, lib.ta_last_error().decode()
        assert torch.cuda.mem_get_info()[0] == free_before                    # nothing was allocated
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
        assert np.abs(out.float().cpu().numpy() - c["want"]).max() < 2e-2
    # beyond the static buffer: refused with a message, nothing launched, out untouched
    out.fill_(7.0)
    too_many = room // (NH * (DH + 2)) + 1
    rc = _no_alloc(lib, c, out, n_units=too_many)
    torch.cuda.synchronize()
    assert rc != 0 and "static buffer" in lib.ta_last_error().decode()
    assert (out == 7.0).all()
