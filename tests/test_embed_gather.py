"""Op::EmbedGather (crates/infr-core/src/graph.rs:853-865; CPU arm crates/infr-cpu/src/lib.rs:2084-2111).
The oracle's gather is pinned on tables whose decoded rows are known without any decoder (F32 rows
that hold their own index, a BF16 / F16 table built from exact values) and on the already pinned
host decode; the device kernel must equal the oracle bit for bit for every table format."""
import numpy as np
import pytest

from oracle import oracle as orc

FORMATS = [orc.F32, orc.F16, orc.BF16, orc.Q8_0, orc.Q4_0, orc.Q4_1, orc.Q5_0, orc.Q5_1, orc.Q4_K, orc.Q5_K,
           orc.Q6_K, orc.IQ4_NL, orc.Q2_0, orc.Q2_K, orc.Q3_K, orc.IQ4_XS, orc.MXFP4, orc.NVFP4, orc.TQ2_0, orc.TQ1_0]


def table_bytes(dtype, rows, ne, seed):
    if dtype == orc.F32:
        return orc.det_x(rows * ne, seed).view(np.uint8)
    if dtype == orc.F16:
        return orc.det_x(rows * ne, seed).astype(np.float16).view(np.uint8)
    if dtype == orc.BF16:
        return (orc.det_x(rows * ne, seed).view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
    return orc.synth_weight(dtype, rows * ne, seed)


def test_oracle_gather_indexing_and_scale():
    ne, rows = 8, 5
    table = np.repeat(np.arange(rows, dtype=np.float32), ne).reshape(rows, ne) + np.arange(ne, dtype=np.float32) / 16
    got = orc.embed_gather(orc.F32, table, rows * ne, [4, 0, 4, 2], ne, scale=0.5)
    assert np.array_equal(got, table[[4, 0, 4, 2]] * np.float32(0.5))
    with pytest.raises(ValueError):
        orc.embed_gather(orc.F32, table, rows * ne, [5], ne)            # the reference panics here
    with pytest.raises(ValueError):
        orc.embed_gather(orc.F32, table, rows * ne, [-1], ne)


def test_oracle_bf16_and_f16_tables_decode_exactly():
    vals = np.array([1.0, -2.5, 0.15625, 3.0e4, -1.0e-3, 0.0, 65504.0, 1.0e-7], np.float32)
    bf = (vals.view(np.uint32) >> 16).astype(np.uint16)
    want_bf = (bf.astype(np.uint32) << 16).view(np.float32)             # truncation is what the bits say
    assert np.array_equal(orc.embed_gather(orc.BF16, bf.view(np.uint8), 8, [0], 8)[0], want_bf)
    f16 = vals.astype(np.float16)
    assert np.array_equal(orc.embed_gather(orc.F16, f16.view(np.uint8), 8, [0], 8)[0], f16.astype(np.float32))


@pytest.mark.parametrize("dtype", FORMATS)
def test_oracle_gather_is_the_host_decode_of_the_selected_rows(dtype):
    e, b = orc.block_layout(dtype)
    ne, rows = max(e, 1) * (3 if e > 1 else 96), 7
    table = table_bytes(dtype, rows, ne, 11)
    ids = [6, 0, 3, 3]
    got = orc.embed_gather(dtype, table, rows * ne, ids, ne, scale=1.75)
    bpr = table.size // rows
    for r, t in enumerate(ids):
        want = orc.dequant_block(dtype, table[t * bpr:(t + 1) * bpr]) * np.float32(1.75)
        assert np.array_equal(got[r].view(np.uint32), want.view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", FORMATS)
def test_device_gather_equals_the_oracle_bit_for_bit(be, dtype):
    e, b = orc.block_layout(dtype)
    ne = 768 if e <= 64 else 1024
    rows_in_table, n_ids = 50, 33
    table = table_bytes(dtype, rows_in_table, ne, 3 + dtype)
    ids = ((np.arange(n_ids) * 7919) % rows_in_table).astype(np.int32)
    ids[:3] = [rows_in_table - 1, 0, 0]
    dst = be.alloc(n_ids * ne * 4)
    be.embed_gather(dtype, be.upload_new(table), rows_in_table * ne, be.upload_new(ids), n_ids, ne, dst,
                    scale=float(np.sqrt(np.float32(ne))))
    got = be.download(dst, np.empty((n_ids, ne), np.float32))
    want = orc.embed_gather(dtype, table, rows_in_table * ne, ids, ne, scale=float(np.sqrt(np.float32(ne))))
    assert np.abs(want).max() > 0
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.gpu
def test_device_gather_out_of_range_id_is_nan_not_a_fault(be):
    ne, rows = 256, 4
    table = orc.synth_weight(orc.Q4_K, rows * ne, 5)
    ids = np.array([1, 4, -1, 3], np.int32)
    dst = be.alloc(4 * ne * 4)
    be.embed_gather(orc.Q4_K, be.upload_new(table), rows * ne, be.upload_new(ids), 4, ne, dst)
    got = be.download(dst, np.empty((4, ne), np.float32))
    assert np.isnan(got[1]).all() and np.isnan(got[2]).all()
    want = orc.embed_gather(orc.Q4_K, table, rows * ne, [1, 3], ne)
    assert np.array_equal(got[[0, 3]], want)


@pytest.mark.gpu
def test_gather_feeds_a_linear_inside_a_plan(be):
    """token ids -> EmbedGather -> RmsNorm -> Linear, replayed with new ids."""
    from infr_amd import Bindings, DType, EmbedGather, Graph, Linear, RmsNorm, TensorDesc, synth_normal_f32, synth_weight
    ne, vocab, out_f, rows = 1024, 64, 96, 1
    g = Graph()
    ids = g.input(TensorDesc((rows,), DType.I32))
    table = g.weight(TensorDesc((vocab, ne), DType.Q6K))
    nw = g.weight(TensorDesc((ne,), DType.F32))
    w = g.weight(TensorDesc((out_f, ne), DType.Q4K))
    emb = g.internal(TensorDesc((rows, ne), DType.F32)) if hasattr(g, "internal") else g.output(TensorDesc((rows, ne), DType.F32))
    xn = g.output(TensorDesc((rows, ne), DType.F32))
    y = g.output(TensorDesc((rows, out_f), DType.F32))
    g.push(EmbedGather(ids, table, emb, rows, ne, 2.0))
    g.push(RmsNorm(emb, nw, xn, rows, ne, 1e-6))
    g.push(Linear(xn, w, y, rows, ne, out_f))
    tb = synth_weight(DType.Q6K, 1, vocab, ne)
    nwv = synth_normal_f32(2, ne, mean=1.0, sigma=0.1)
    wv = synth_weight(DType.Q4K, 3, out_f, ne)
    idb, yb = be.alloc(4), be.alloc(out_f * 4)
    binds = (Bindings().bind(ids, idb).bind(table, be.upload_new(tb)).bind(nw, be.upload_new(nwv))
             .bind(w, be.upload_new(wv)).bind(emb, be.alloc(ne * 4)).bind(xn, be.alloc(ne * 4)).bind(y, yb))
    plan = be.compile(g)
    for tok in (5, 63, 0):
        be.upload(idb, np.array([tok], np.int32))
        be.execute(plan, binds)
        got = be.download(yb, np.empty((1, out_f), np.float32))
        e = orc.embed_gather(orc.Q6_K, tb, vocab * ne, [tok], ne, scale=2.0)
        xnv = orc.rms_norm(e, nwv, 1, ne, 1e-6)
        want = orc.linear(orc.Q4_K, wv, xnv, 1, ne, out_f)
        rel = np.linalg.norm(got - want) / np.linalg.norm(want)
        assert rel <= 1e-4, rel
