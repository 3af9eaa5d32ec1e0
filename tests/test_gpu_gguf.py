"""Weights read from a GGUF file and uploaded by the reader feed Op::Linear / Op::MoeFfn and give
what the CPU oracle gives on the same file bytes. The files are written here from synthetic banks;
the layout mimics a real checkpoint (projections of one decoder block under their GGUF names, mixed
Q4_K / Q6_K / Q8_0, a two-file shard set)."""
import numpy as np
import pytest

import infr_amd.gguf as G
from infr_amd import DType, InfrError, synth_normal_f32, synth_weight
from oracle import oracle as orc
from tests.test_gpu_linear import gate

pytestmark = pytest.mark.gpu

NE, NFF = 1024, 3072
BLOCK = [  # name, dtype, in_f, out_f
    ("blk.0.attn_q.weight", DType.Q4K, NE, NE),
    ("blk.0.attn_k.weight", DType.Q4K, NE, 256),
    ("blk.0.attn_v.weight", DType.Q6K, NE, 256),
    ("blk.0.ffn_gate.weight", DType.Q4K, NE, NFF),
    ("blk.0.ffn_up.weight", DType.Q4K, NE, NFF),
    ("blk.0.ffn_down.weight", DType.Q6K, NFF, NE),
    ("output.weight", DType.Q8_0, NE, 512),
]


def block_tensors():
    return [(n, (in_f, out_f), int(dt), synth_weight(dt, 100 + i, out_f, in_f))
            for i, (n, dt, in_f, out_f) in enumerate(BLOCK)]


@pytest.mark.parametrize("m", [1, 5])
def test_linear_on_uploaded_gguf_tensors(be, tmp_path, m):
    p = tmp_path / "block.gguf"
    G.write_gguf(p, {"general.architecture": "qwen3", "qwen3.embedding_length": NE}, block_tensors())
    with G.Gguf.open(p) as g:
        assert g.metadata().u64("qwen3.embedding_length") == NE
        for t in g.tensors():
            in_f, out_f = t.shape
            w = g.upload(be, t.name)
            assert w.len_bytes() == t.nbytes
            x = synth_normal_f32(7 + out_f, m * in_f)
            y = be.alloc(m * out_f * 4)
            be.linear(t.dtype, w, be.upload_new(x), y, m, in_f, out_f)
            got = be.download(y, np.empty((m, out_f), np.float32))
            want = orc.linear(t.dtype, g.tensor_bytes(t.name), x, m, in_f, out_f)
            if m == 1 and t.dtype in (DType.Q4K, DType.Q6K):
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), t.name
            else:
                gate(got, want)
        with pytest.raises(InfrError):
            g.upload(be, "blk.9.nope.weight")


def test_concatenated_upload_is_addressed_by_w_off(be, tmp_path):
    """Same-typed tensors land back to back in one buffer and Op::Linear reaches each through its
    element offset, as the reference does for fused q/k/v (crates/infr-core/src/graph.rs:177-191)."""
    p = tmp_path / "block.gguf"
    G.write_gguf(p, {}, block_tensors())
    names = ["blk.0.attn_q.weight", "blk.0.attn_k.weight", "blk.0.ffn_gate.weight"]
    with G.Gguf.open(p) as g:
        buf, offs = g.upload_concat(be, names)
        infos = [g.tensor(n) for n in names]
        assert offs == [0, infos[0].nbytes, infos[0].nbytes + infos[1].nbytes]
        assert buf.len_bytes() == sum(t.nbytes for t in infos)
        x = synth_normal_f32(3, NE)
        xb = be.upload_new(x)
        for t, off in zip(infos, offs):
            in_f, out_f = t.shape
            y = be.alloc(out_f * 4)
            be.linear(DType.Q4K, buf, xb, y, 1, in_f, out_f, w_off=off // 144 * 256)
            want = orc.linear(DType.Q4K, g.tensor_bytes(t.name), x, 1, in_f, out_f)
            got = be.download(y, np.empty((1, out_f), np.float32))
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), t.name
        with pytest.raises(InfrError, match="ggml type"):
            g.upload_concat(be, ["blk.0.attn_q.weight", "blk.0.attn_v.weight"])


def test_weights_from_a_shard_set(be, tmp_path):
    ts = block_tensors()
    split = {"split.count": (2, 2), "split.tensors.count": (5, len(ts))}
    G.write_gguf(tmp_path / "m-00001-of-00002.gguf",
                 {"general.architecture": "qwen3", "split.no": (2, 0), **split}, ts[:4])
    G.write_gguf(tmp_path / "m-00002-of-00002.gguf", {"split.no": (2, 1), **split}, ts[4:])
    with G.Gguf.open(tmp_path / "m-00002-of-00002.gguf") as g:
        assert [t.name for t in g.tensors()] == [n for n, *_ in BLOCK] and len(g.shards()) == 2
        for name, dt, in_f, out_f in (BLOCK[1], BLOCK[5]):      # one tensor from each file
            w = g.upload(be, name)
            x = synth_normal_f32(9, in_f)
            y = be.alloc(out_f * 4)
            be.linear(dt, w, be.upload_new(x), y, 1, in_f, out_f)
            want = orc.linear(dt, next(d for n, _, _, d in ts if n == name), x, 1, in_f, out_f)
            got = be.download(y, np.empty((1, out_f), np.float32))
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), name


def test_moe_banks_from_gguf(be, tmp_path):
    """Expert banks stored as 3-D tensors [in, out, n_expert], the router as F32."""
    ne, nff, n_expert, n_used = 512, 256, 8, 2
    router = synth_normal_f32(1, n_expert * ne).astype(np.float32)
    gate_w = synth_weight(DType.Q4K, 2, n_expert * nff, ne)
    up_w = synth_weight(DType.Q4K, 3, n_expert * nff, ne)
    down_w = synth_weight(DType.Q6K, 4, n_expert * ne, nff)
    p = tmp_path / "moe.gguf"
    G.write_gguf(p, {"qwen3moe.expert_count": n_expert, "qwen3moe.expert_used_count": n_used}, [
        ("blk.0.ffn_gate_inp.weight", (ne, n_expert), 0, router),
        ("blk.0.ffn_gate_exps.weight", (ne, nff, n_expert), 12, gate_w),
        ("blk.0.ffn_up_exps.weight", (ne, nff, n_expert), 12, up_w),
        ("blk.0.ffn_down_exps.weight", (nff, ne, n_expert), 14, down_w),
    ])
    with G.Gguf.open(p) as g:
        md = g.metadata()
        assert g.tensor("blk.0.ffn_down_exps.weight").shape == (nff, ne, n_expert)
        bufs = [g.upload(be, n) for n in ("blk.0.ffn_gate_inp.weight", "blk.0.ffn_gate_exps.weight",
                                          "blk.0.ffn_up_exps.weight", "blk.0.ffn_down_exps.weight")]
        for rows in (1, 4):
            x = synth_normal_f32(20 + rows, rows * ne)
            dst = be.alloc(rows * ne * 4)
            be.moe_ffn(be.upload_new(x), *bufs, dst, rows=rows, ne=ne, n_expert=md.u64("qwen3moe.expert_count"),
                       n_used=md.u64("qwen3moe.expert_used_count"), n_ff_exp=nff, down_dtype=DType.Q6K)
            got = be.download(dst, np.empty((rows, ne), np.float32))
            want, _, _ = orc.moe_ffn(x, router, gate_w, up_w, down_w, ne=ne, n_expert=n_expert, n_used=n_used,
                                     n_ff_exp=nff, down_dtype=orc.Q6_K)
            gate(got, want)
