"""CPU tests of the host-side mirror of the reference interface: block input construction, bank
metadata helpers, the cache container and configuration (no GPU, no HIP calls)."""
import pytest
import torch

from msa_amd import cache as mcache
from msa_amd import config as mconfig
from msa_amd import prefill
from oracle import closed_form as cf


def _docs(lens, P):
    return [prefill.Document(doc=f"d{i}", doc_id=100 + i, num_chunks=prefill.num_chunks(n, P), input_ids=list(range(n)))
            for i, n in enumerate(lens)]


def test_prepare_block_inputs_matches_oracle_layout():
    P, lens, head = 8, [5, 8, 17, 1], [11, 12, 13]
    inp = prefill.prepare_block_inputs(_docs(lens, P), head, P)
    assert inp.doc_ids[0].tolist() == [-2] * 3 + [1] * 5 + [2] * 8 + [3] * 17 + [4]
    assert inp.position_ids[0].tolist() == cf.doc_positions(lens, 3).tolist()      # restart at 0 per document
    assert inp.chunk_sizes == [1, 1, 3, 1] and inp.num_chunks == 6
    assert inp.doc_attention_mask.sum() == 3 + sum(lens)
    assert inp.doc_input_ids[0, :3].tolist() == head
    _, dco, _, _, _ = cf.chunk_table(lens, P, 3)
    assert dco[-1] == inp.num_chunks
    bad = _docs(lens, P)
    bad[2].num_chunks = 2
    with pytest.raises(AssertionError, match="pre calculated chunk"):
        prefill.prepare_block_inputs(bad, head, P)
    with pytest.raises(ValueError):
        prefill.prepare_block_inputs([prefill.Document(doc_id=1)], head, P)


def test_split_docs_budget_and_order():
    docs = _docs([64, 64, 200, 8, 8, 8], 8)           # chunks 8, 8, 25, 1, 1, 1
    blocks = prefill.split_docs(docs, 16)
    assert [[d.doc_id for d in b] for b in blocks] == [[100, 101], [102], [103, 104, 105]]
    assert prefill.split_docs(docs, 1000) == [docs]
    assert prefill.split_docs([], 16) == []


def test_query_positions_rule():
    assert prefill.query_position_ids(3, 16) == [19, 20, 21]
    assert prefill.query_position_ids(2, 16, left_pad=3) == [19, 19, 19, 19, 20]
    assert prefill.query_position_ids(4, 16, 3, 1) == cf.query_positions(4, 16, 3, 1).tolist()


def test_cumulative_concat_and_block_desc():
    from msa_amd.msa_service import BlockDesc, cumulative_concat
    a, b, c = torch.tensor([1, 1, 2, 3, 3]), torch.tensor([1, 2, 2]), torch.tensor([1])
    assert cumulative_concat([a, b, c]).tolist() == [1, 1, 2, 3, 3, 4, 5, 5, 6]
    desc = BlockDesc()
    desc.init_docs(_docs([5, 8, 17], 8), "cpu")
    assert desc.doc_ids_cpu.tolist() == [0, 100, 101, 102]
    assert desc.doc_lens_cpu.tolist() == [0, 1, 1, 3]
    assert desc.doc_offsets_cpu.tolist() == [0, 0, 1, 2]
    assert desc.chunks() == 5 and desc.nr_docs == 3
    assert desc.create_global_doc_ids(torch.tensor([[3, 1]])).tolist() == [[102, 100]]


def test_cache_container():
    c = mcache.create_cache()
    c.record_kwargs(2, {"stage": "prefill_stage1"})
    c.record_kwargs(2, {"x": 1})
    assert c.cache_kwargs[2] == {"stage": "prefill_stage1", "x": 1} and c.get_layer_length() == 1
    k1, v1 = torch.ones(1, 2, 3, 4), torch.zeros(1, 2, 3, 4)
    c.update(k1, v1, 2)
    c.update(2 * k1, v1, 2)
    k, v = c.get_kvcache(2)
    assert k.shape == (1, 2, 6, 4) and k[0, 0, 3, 0] == 2 and c.get_seq_length(2) == 6 and c.get_seq_length(0) == 0
    assert c.get_router_kcache(2) is None
    c.update_router_kcache(k1, 2)
    assert c.get_router_kcache(2).shape == (1, 2, 3, 4) and c.get_router_kcache(0) is None
    c.record_kwargs(2, {"compacked_key_cache": 1, "compacked_value_cache": 2, "recall_topk": 3})
    c.clear_query()
    assert "compacked_key_cache" not in c.cache_kwargs[2] and "recall_topk" not in c.cache_kwargs[2]
    c.clear_kvcache()
    assert c.key_cache == [] and c.get_seq_length(2) == 0


def test_configs():
    g = mconfig.GenerateConfig(devices=[0], template="QWEN3_INSTRUCT_TEMPLATE")
    assert g.world == 1 and "{prompt}" in g.template["prompt"]
    with pytest.raises(ValueError):
        mconfig.GenerateConfig(template="NOPE")
    m = mconfig.ModelConfig()
    assert (m.doc_top_k, m.pooling_kernel_size, m.template_token_id, m.template_id_num) == (16, 64, -2, 3)
    assert mconfig.MemoryConfig().slice_chunk_size == 16384
    cfg = mconfig.MSAConfig(msa_config={"top_k_docs": 4})
    assert cfg.msa_config.top_k_docs == 4 and cfg.msa_config.missing is None
    d = mconfig.MSAConfig()
    assert d.msa_config.router_layer_idx.split(",")[0] == "18" and d.num_key_value_heads == 8


def test_bank_files_round_trip(tmp_path):
    """The on-disk bank format: raw arrays + JSON header, memory-mapped back bit for bit."""
    from msa_amd import bank_io
    g = torch.Generator().manual_seed(0)
    off = [0, 2, 5, 6]
    C, Hkv, D = 6, 2, 128
    for dtype in (torch.bfloat16, torch.float32):
        mk = lambda: torch.randn((C, Hkv, D), generator=g).to(dtype)
        rk, k, v = {3: mk(), 5: mk()}, {3: mk(), 5: mk()}, {3: mk(), 5: mk()}
        prefix = {l: (torch.randn((1, Hkv, 3, D), generator=g).to(dtype), torch.randn((1, Hkv, 3, D), generator=g).to(dtype))
                  for l in range(6)}
        path = str(tmp_path / f"bank_{dtype}".replace(".", "_"))
        bank_io.save_bank(path, {"pooling_kernel_size": 64, "aux_loss_method": "INFONCE"}, off, [10, 11, 12], rk, k, v, prefix)
        f = bank_io.BankFiles(path)
        assert f.header["chunks"] == C and f.header["router_layers"] == [3, 5] and f.header["pooling_kernel_size"] == 64
        assert f.doc_chunk_off.tolist() == off and f.doc_global_id.tolist() == [10, 11, 12]
        for layer in (3, 5):
            for tag, store in (("rk", rk), ("k", k), ("v", v)):
                dst = torch.empty((C, Hkv, D), dtype=dtype)
                f.copy_into(layer, tag, dst, rows_per_step=4)
                assert torch.equal(dst, store[layer])
        back = f.prefix()
        assert sorted(back) == list(range(6))
        assert torch.equal(back[4][0], prefix[4][0]) and torch.equal(back[4][1], prefix[4][1])
    # a truncated layer file is refused, and so is a missing header
    with open(f"{path}/layer_3.k.bin", "r+b") as fh:
        fh.truncate(100)
    with pytest.raises(ValueError, match="bytes, expected"):
        bank_io.BankFiles(path).layer(3, "k")
    import os
    os.remove(f"{path}/bank.json")
    with pytest.raises(FileNotFoundError):
        bank_io.BankFiles(path)


def test_source_block_positions_follow_the_reference_formula():
    """src/msa/generate.py:235-236: arange(W) + position_ids + sum(attention_mask) - W + 1 on the columns that hold
    tokens; the padding columns in front are floored at 0."""
    import torch
    from msa_amd import prefill as pf
    last = [25, 40, 3]
    n = [5, 2, 1]
    W = 5
    got = torch.tensor(pf.source_block_position_ids(last, n, W))
    mask = torch.tensor([[1] * 5, [0, 0, 0, 1, 1], [0, 0, 0, 0, 1]])
    ref = torch.arange(W).unsqueeze(0).expand(3, -1) + torch.tensor(last).unsqueeze(1) + mask.sum(dim=1, keepdim=True) - W + 1
    assert torch.equal(got[mask.bool()], ref[mask.bool()])
    assert got[0].tolist() == [26, 27, 28, 29, 30] and got[1].tolist()[3:] == [41, 42] and got[2, 4] == 4
    assert (got >= 0).all() and got[2].tolist() == [0, 1, 2, 3, 4]
    assert torch.equal(got[1, :3], ref[1, :3])                     # in front of real tokens the same expression runs on


def test_prefill_worker_block_inputs_and_split():
    from msa_amd import prefill as pf
    docs = [pf.Document(doc_id=10 + i, num_chunks=pf.num_chunks(n, 8), input_ids=list(range(1, n + 1))) for i, n in enumerate([9, 16, 3, 30])]
    w = pf.PrefillStage1Worker(0, None, [7, 8, 9], 8)
    blocks = w.split_docs(docs, 5)
    assert [[d.doc_id for d in b] for b in blocks] == [[10, 11, 12], [13]]      # 2 + 2 + 1 chunks fill a block of 5
    inp = w._prepare_block_inputs(blocks[0])
    assert inp.doc_ids[0, :3].tolist() == [-2, -2, -2] and inp.doc_ids[0, 3:12].tolist() == [1] * 9
    assert inp.position_ids[0, 3:12].tolist() == list(range(9)) and inp.position_ids[0, 12] == 0
    assert inp.chunk_sizes == [2, 2, 1]


def test_reference_bank_files_convert_to_the_native_format(tmp_path):
    """A bank directory in the reference's file layout (tests/golden/make_reference_style_bank.py) is read without
    its meta.pt, transposed to chunk-major, and converts to the native format bit for bit."""
    from types import SimpleNamespace
    from msa_amd import bank_io
    from tests.golden import make_reference_style_bank as mk
    src, dst = str(tmp_path / "ref"), str(tmp_path / "native")
    mk.write(src)
    layers, prefix = mk.expected()
    assert bank_io.reference_bank_layers(src) == mk.LAYERS
    rk, k, v = bank_io.read_reference_layer(src, 19)
    C = sum(mk.DOC_CHUNKS)
    assert rk.shape == (C, mk.HKV, mk.D) and rk.is_contiguous()
    assert torch.equal(rk, layers[19]["rk"][0].transpose(0, 1))
    assert torch.equal(k[5, 1], layers[19]["k"][0, 1, 5]) and torch.equal(v[2, 0], layers[19]["v"][0, 0, 2])
    docs = [SimpleNamespace(doc_id=i, num_chunks=n, doc=f"text {i}") for i, n in zip(mk.DOC_IDS, mk.DOC_CHUNKS)]
    bank_io.convert_reference_bank(src, dst, docs, {"pooling_kernel_size": 64, "aux_loss_method": "INFONCE"})
    files = bank_io.BankFiles(dst)
    assert files.header["router_layers"] == mk.LAYERS and files.shape == (C, mk.HKV, mk.D)
    assert files.doc_chunk_off.tolist() == [0, 3, 4, 8, 10] and files.doc_global_id.tolist() == mk.DOC_IDS
    for l in mk.LAYERS:
        for tag in ("rk", "k", "v"):
            got = torch.empty(files.shape, dtype=torch.bfloat16)
            files.copy_into(l, tag, got)
            assert torch.equal(got, layers[l][tag][0].transpose(0, 1))
    back = files.prefix()
    assert sorted(back) == sorted(prefix)
    assert all(torch.equal(back[l][0], prefix[l][0]) and torch.equal(back[l][1], prefix[l][1]) for l in prefix)
    assert [r["doc"] for r in bank_io.load_docs(dst)] == [d.doc for d in docs]
    # documents that do not add up to the stored chunks are refused
    with pytest.raises(ValueError, match="add up"):
        bank_io.convert_reference_bank(src, str(tmp_path / "bad"), docs[:-1], {})


def test_concatenated_projection_weights_follow_their_sources():
    """The [router_k | q | k | v | router_q] copy the fused projection multiplies by is rebuilt when a source weight
    is updated in place, replaced by a loaded state dict, or converted to another dtype; otherwise it is reused."""
    from msa_amd import memory_sparse_attention as msa
    cfg = mconfig.MSAConfig(hidden_size=64, num_hidden_layers=2, num_attention_heads=2, num_key_value_heads=1, head_dim=128,
                            intermediate_size=64, vocab_size=50,
                            msa_config=dict(mconfig.default_msa_config(), router_layer_idx="1"))
    layer = msa.MemorySparseAttention(cfg, 1)
    dev = torch.device("cpu")

    def want():
        return torch.cat([layer.router_k_proj[0].weight, layer.q_proj.weight, layer.k_proj.weight, layer.v_proj.weight,
                          layer.router_q_proj[0].weight])
    first = layer._all_weight(dev)
    assert torch.equal(first, want()) and layer._all_weight(dev) is first
    with torch.no_grad():
        layer.k_proj.weight.mul_(2.0)                                     # in-place update (an optimizer step)
    assert torch.equal(layer._all_weight(dev), want()) and layer._all_weight(dev) is not first
    state = {k: torch.randn_like(v) for k, v in layer.state_dict().items()}
    layer.load_state_dict(state)                                          # copy_ into the same storage
    assert torch.equal(layer._all_weight(dev), want())
    layer.bfloat16()                                                      # new dtype
    got = layer._all_weight(dev)
    assert got.dtype == torch.bfloat16 and torch.equal(got, want())
    assert torch.equal(layer._fused_weight(dev), torch.cat([layer.q_proj.weight, layer.k_proj.weight, layer.v_proj.weight]))


def test_compact_cache_in_the_reference_layout():
    """[B, Lcap, Hkv, D] + lengths -> the reference's left-padded [B, Hkv, maxL, D] + mask, against a loop."""
    g = torch.Generator().manual_seed(3)
    B, Lcap, Hkv, D = 3, 9, 2, 4
    kc, vc = torch.randn((B, Lcap, Hkv, D), generator=g), torch.randn((B, Lcap, Hkv, D), generator=g)
    lens = torch.tensor([5, 0, 7], dtype=torch.int32)
    k, v, mask = mcache.compact_cache_reference_layout(kc, vc, lens)
    assert k.shape == v.shape == (B, Hkv, 7, D) and mask.shape == (B, 7)
    for b in range(B):
        n = int(lens[b])
        assert mask[b].tolist() == [False] * (7 - n) + [True] * n
        assert float(k[b, :, :7 - n].abs().max() if n < 7 else 0.0) == 0.0
        for i in range(n):
            assert torch.equal(k[b, :, 7 - n + i], kc[b, i]) and torch.equal(v[b, :, 7 - n + i], vc[b, i])
    # the reference's own fill (boolean-mask assignment of the packed rows) gives the same tensors
    want = torch.zeros((B, Hkv, 7, D))
    want.permute(0, 2, 1, 3)[mask] = torch.cat([kc[b, :int(lens[b])] for b in range(B)])
    assert torch.equal(k, want)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU's throughput: a request for several exits with a message that says so, before
    anything touches a device."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)
