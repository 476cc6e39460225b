"""The rule that picks the rows walked one per sub-wave, as the tests' mirror states it (no GPU needed):
spelled out on hand-made groups of rows."""
import gpu_api
import graphs


def test_the_rule_on_hand_made_groups():
    """The mirror's rule, spelled out on the groups above for K=32 (8 rows per group, 8 gathers in flight)."""
    g = graphs.boundary_graph()
    p = gpu_api.packed_rows(g, g["rows"], 32, 32, 4096)
    grp = lambda i: p[8 * i:8 * i + 8]
    assert grp(0).all()                    # 8 rows of 64: 8 batches either way
    assert not grp(1).any()                # one row of 65: too long for one sub-wave's share
    assert not grp(2).any()                # a lone row of 64: 8 batches packed, 1 unpacked
    assert grp(3).all() and not grp(4).any()     # a lone row: up to 8 edges is one batch either way
    assert grp(5).all() and not grp(6).any()     # two rows: up to 16 edges each
    assert not grp(7).any()                # all empty: nothing to pack (zeros are stored by the row loop)
    assert grp(8).all() and grp(9).all() and grp(10).all()
    assert gpu_api.packed_rows(g, g["rows"], 32, 32, 4096, pack=False).sum() == 0
    assert gpu_api.packed_rows(g, g["rows"], 128, 32, 4096).sum() == 0          # sub-waves of 32 lanes: never
    assert gpu_api.packed_rows(g, g["rows"], 33, 32, 4096, vec_ok=False).sum() == 0   # 4-byte layout: never
    p64 = gpu_api.packed_rows(g, g["rows"], 64, 32, 4096)                        # K=64: groups of 4, at most 32 edges
    assert p64[8 * 11:8 * 11 + 4].all() and not p64[8 * 12:8 * 12 + 4].any() and p64[8 * 12 + 4:8 * 12 + 8].all()
    assert not gpu_api.packed_rows(g, g["rows"], 32, 32, 20)[:8].any()           # rows that are split are never packed
    pd = gpu_api.packed_rows(g, g["rows"], 32, 64, 4096)                         # double: 4 gathers in flight
    assert not pd[:8].any() and pd[8 * 11:8 * 11 + 8].sum() == 0 and pd[8 * 9:8 * 9 + 8].all()
