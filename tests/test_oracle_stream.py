"""The numpy statement of the load-time weight stream (oracle.stream_pack / stream_unpack): a
bijection of the reference buffers, with every code in the slot the kernel's masks expect.  CPU only."""
import numpy as np
import pytest

from oracle import cherryq_oracle as orc


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("k,n,gs", [(512, 48, 128), (1024, 24, 128), (4096, 64, 128), (2304, 40, 256), (4104, 16, 128)])
def test_round_trip(bits, k, n, gs):
    p = orc.synthetic_packed_fast(k, n, bits, gs, seed=k + n + bits)
    c = p["cherry_indices"].shape[0]
    st = orc.stream_pack(p, bits, gs, k)
    g = orc.stream_geometry(bits, k, n, c)
    assert st.size == g["hdr_bytes"] + g["ntiles"] * g["record_bytes"] and g["record_bytes"] % 256 == 0
    back = orc.stream_unpack(st, bits, gs, k, n, c)
    for name in p:
        np.testing.assert_array_equal(back[name], p[name], err_msg=name)


@pytest.mark.parametrize("bits", [3, 4])
def test_every_code_sits_where_one_mask_isolates_it(bits):
    """Brute force over the 32 slots of a lane: set ONE code to all ones, everything else zero, and
    decode the lane's dwords the way the kernel does (mask in place, fields at bit p <= 8 of a
    16-bit half read as code * 2^p; the 3-bit left-over bits recombined).  Exactly slot q must
    answer, with the full code."""
    k, n = 128 + 0, 16   # one unit, one tile, no cherries
    full = 2 ** bits - 1
    for q in range(32):
        for kq in range(4):
            codes = np.zeros((128, n), dtype=np.uint8)
            codes[32 * kq + q, 5] = full
            p = {"cherry_indices": np.zeros(0, np.int16), "cherry_weight": np.zeros((0, n), np.float16),
                 "qweight": orc.pack_codes(codes, bits), "scales": np.ones((1, n), np.float16)}
            st = orc.stream_pack(p, bits, 128, k)
            g = orc.stream_geometry(bits, k, n, 0)
            units = st[g["hdr_bytes"] + g["off_units"]:].view(np.uint32).reshape(64, bits)
            w = units[kq * 16 + 5].astype(np.uint64)
            got = {}
            if bits == 4:
                y = w >> 8
                ops = [(w[0], 0), (y[0], 0), (w[1], 0), (y[1], 0), (w[2], 0), (y[2], 0), (w[3], 0), (y[3], 0),
                       (w[0], 4), (y[0], 4), (w[1], 4), (y[1], 4), (w[2], 4), (y[2], 4), (w[3], 4), (y[3], 4)]
                for i, (v, pbit) in enumerate(ops):
                    m = 0x000f000f << pbit
                    f = int(v) & m
                    got[2 * i] = (f & 0xffff) >> pbit
                    got[2 * i + 1] = (f >> 16) >> pbit
            else:
                y = w >> 9
                z = (int(y[0]) & 0x00400040) | ((int(y[1]) & 0x00400040) << 1) | ((int(y[2]) & 0x00400040) << 2)
                ops = ([(w[0], 0), (w[1], 0), (w[2], 0), (y[0], 0)] + [(w[0], 3), (w[1], 3), (w[2], 3), (y[0], 3)]
                       + [(w[0], 6), (w[1], 6), (w[2], 6), (z, 6)] + [(y[1], 0), (y[2], 0)] + [(y[1], 3), (y[2], 3)])
                for i, (v, pbit) in enumerate(ops):
                    f = int(v) & (0x00070007 << pbit)
                    got[2 * i] = (f & 0xffff) >> pbit
                    got[2 * i + 1] = (f >> 16) >> pbit
            assert got[q] == full, (q, kq)
            assert sum(got.values()) == full, (q, kq)
    # other lanes stay empty
    assert np.count_nonzero(units) <= 3


def test_header_is_the_gather_table():
    k, n, bits = 4096, 16, 4
    p = orc.synthetic_packed_fast(k, n, bits, 128, seed=1)
    idx = p["cherry_indices"].astype(np.int64)
    c = idx.shape[0]
    st = orc.stream_pack(p, bits, 128, k)
    g = orc.stream_geometry(bits, k, n, c)
    normal = orc.normal_indices(k, idx)
    tab = st[:g["knp512"]].reshape(-1, 64, 8)     # block, lane, j -> position block*512 + 64 j + lane
    for blk in range(tab.shape[0]):
        for lane in (0, 1, 17, 63):
            for j in range(8):
                pos = blk * 512 + 64 * j + lane
                if pos < g["kn"]:
                    assert pos + int(tab[blk, lane, j]) == normal[pos]
                else:
                    assert int(tab[blk, lane, j]) == c and pos + c >= k   # reads the zeros behind x
    cols = st[g["knp512"]:g["knp512"] + 2 * g["cp"]].view(np.uint16)
    np.testing.assert_array_equal(cols[:c], idx)
    assert (cols[c:] == k).all()
