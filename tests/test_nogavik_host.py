"""Host side of the Nogavik model class, without a GPU: the loader (norm weights stored around zero kept as 1 + w, the state-space input projection kept in
its three parts, every layer's part of the side table as a table of its own, q / k / v of the delta branch as one projection, parameter vectors of unequal
lengths one after the other), what it refuses, the plain reference's own pieces, and the graph the engine builds for a mixed batch (which layer's cache a
layer with shared rows reads, which nodes exist)."""
import ctypes as C
import json

import numpy as np
import pytest

import llama_box_amd as L
import nogavik_ref as R


def small_cfg():
    return R.make_config(40, 53, [
        R.latent_layer(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=10, q_rank=6, scale=0.3, mlp=R.dense(16), base=100.0),
        R.state_space_layer(heads=4, vdim=6, state=5, groups=2, norm_groups=2, conv=3, mlp=None),
        R.latent_layer(heads=2, dim=12, rot_dim=4, vdim=8, kv_rank=10, q_rank=7, scale=0.25, mlp=R.dense(8), base=100.0, kv_from=0),
        R.parallel_layer(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.3, r_heads=2, r_kv_heads=1, r_dim=10, r_vdim=6, conv=4, mlp=R.dense(24), rank=5),
    ], side_dim=3, eps=1e-5)


def _get(H, m, name):
    t = H.llm_model_tensor(m, name.encode())
    assert t, name
    raw = np.empty(H.ggml_nbytes(t), np.uint8)
    H.ggml_backend_tensor_get(t, raw.ctypes.data_as(C.c_void_p), 0, raw.nbytes)
    tt = t.contents
    a = (raw.view(np.uint16).astype(np.uint32) << 16).view(np.float32) if tt.type == L.BF16 else raw.view(np.float32)
    return a.reshape([tt.ne[3], tt.ne[2], tt.ne[1], tt.ne[0]])[0]


def test_loader_reads_a_checkpoint_folder(H, tmp_path):
    cfg = small_cfg()
    W = R.random_weights(cfg, 3)
    R.save_model(cfg, W, str(tmp_path))
    for wtype in (L.BF16, L.F32):
        m = H.llm_model_load_dir(str(tmp_path).encode(), H.ggml_backend_cpu_buffer_type(), wtype)
        assert m
        hp = H.llm_model_hparams(m).contents
        assert (hp.arch, hp.n_layer, hp.n_embd, hp.n_vocab) == (b"nogavik", 4, 40, 53)
        # the model's norms are stored around zero and kept as 1 + w; the plain-weight norms are kept as they are
        for name, src in (("blk.0.attn_norm.weight", "l0.norm1"), ("blk.3.ffn_norm.weight", "l3.norm2"), ("output_norm.weight", "final.norm")):
            assert np.array_equal(_get(H, m, name).reshape(-1), (np.float32(1.0) + W[src].astype(np.float32)))
        assert np.array_equal(_get(H, m, "blk.0.attn_kv_a_norm.weight").reshape(-1), W["l0.mix.dkv.norm"])
        assert np.array_equal(_get(H, m, "blk.3.mix_left_norm.weight").reshape(-1), W["l3.mix.left.out"])
        assert not H.llm_model_tensor(m, b"blk.1.ffn_norm.weight")  # a layer without a feed-forward has no second norm
        # the state-space input projection [z | x, B, C | dt] in its three parts
        inner, ch = 24, 24 + 2 * 2 * 5
        w_in = W["l1.mix.in"]
        assert np.array_equal(_get(H, m, "blk.1.ssm_in_z.weight")[0], w_in[:inner])
        assert np.array_equal(_get(H, m, "blk.1.ssm_in_xbc.weight")[0], w_in[inner:inner + ch])
        assert np.array_equal(_get(H, m, "blk.1.ssm_in_dt.weight")[0], w_in[inner + ch:])
        assert np.array_equal(_get(H, m, "blk.1.ssm_params.weight").reshape(-1), np.concatenate([W["l1.mix.A_log"], W["l1.mix.dt_bias"], W["l1.mix.D"]]))
        assert np.array_equal(_get(H, m, "blk.1.ssm_conv1d.bias").reshape(-1), W["l1.mix.conv.b"])
        # every layer's part of the side table
        for il in range(4):
            assert np.array_equal(_get(H, m, "blk.%d.side_embd.weight" % il)[0], W["side.embed"][:, 3 * il:3 * il + 3])
        # the delta branch: q, k, v as one projection, their taps likewise; A_log of the heads in front of the per-channel offsets
        assert np.array_equal(_get(H, m, "blk.3.attn_qkv.weight")[0], np.concatenate([W["l3.mix.right.q"], W["l3.mix.right.k"], W["l3.mix.right.v"]]))
        assert np.array_equal(_get(H, m, "blk.3.ssm_conv1d.weight")[0], np.concatenate([W["l3.mix.right.q.conv"], W["l3.mix.right.k.conv"], W["l3.mix.right.v.conv"]]))
        assert np.array_equal(_get(H, m, "blk.3.attn_gates.param").reshape(-1), np.concatenate([W["l3.mix.right.A_log"], W["l3.mix.right.dt_bias"]]))
        assert _get(H, m, "blk.3.delta_a1.weight")[0].shape == (5, 40)  # the inner size of the decay's matrices comes from the checkpoint
        # W_uk is kept per head with its rows along dim 0; a layer with shared rows has no down projection
        uk = _get(H, m, "blk.2.attn_k_b_t.weight")  # [head][rank][dk]
        assert np.array_equal(uk[1], W["l2.mix.uk"].reshape(2, 12, 10)[1].T)
        assert H.llm_model_tensor(m, b"blk.0.attn_kv_a.weight") and not H.llm_model_tensor(m, b"blk.2.attn_kv_a.weight")
        assert np.allclose(_get(H, m, "blk.0.rope_freq.weight").reshape(-1), [1.0, 100.0 ** -0.5])
        assert not H.llm_model_tensor(m, b"output.weight")  # the output matrix is the embedding table
        H.llm_model_free(m)


@pytest.mark.parametrize("breakage", ["shape", "missing", "heads", "kv_from_later", "kv_from_rank", "kv_from_chain", "mixer", "kind", "norm_groups", "rot_dims", "in_rows", "side"])
def test_loader_refuses_what_it_cannot_serve(H, tmp_path, breakage):
    cfg = small_cfg()
    W = R.random_weights(cfg, 4)
    if breakage == "shape":
        W["l3.mix.right.k.conv"] = W["l3.mix.right.k.conv"][:, :-1]
    elif breakage == "missing":
        del W["l3.mix.left.q.norm"]
    elif breakage == "heads":
        cfg["layers"][3]["mixer"]["left"]["kv_heads"] = 3
    elif breakage == "kv_from_later":
        cfg["layers"][2]["mixer"]["kv_from"] = 3
    elif breakage == "kv_from_rank":
        cfg["layers"][2]["mixer"]["kv_rank"] = 12
    elif breakage == "kv_from_chain":
        cfg["layers"].append(R.latent_layer(heads=2, dim=12, rot_dim=4, vdim=8, kv_rank=10, q_rank=7, scale=0.25, mlp=None, base=100.0, kv_from=2))
    elif breakage == "mixer":
        cfg["layers"][1]["type"] = "something_else"
    elif breakage == "kind":
        cfg["layers"][0]["mlp"]["kind"] = "moe"
    elif breakage == "norm_groups":
        cfg["layers"][1]["mixer"]["norm_groups"] = 5
    elif breakage == "rot_dims":
        cfg["layers"][0]["mixer"]["rot"]["dims"] = 2
    elif breakage == "in_rows":
        W["l1.mix.in"] = W["l1.mix.in"][:-1]
    elif breakage == "side":
        W["side.embed"] = W["side.embed"][:, :-1]
    if breakage == "kv_from_chain":
        W = R.random_weights(cfg, 4)
    R.save_model(cfg, W, str(tmp_path))
    assert not H.llm_model_load_dir(str(tmp_path).encode(), H.ggml_backend_cpu_buffer_type(), L.F32)


def test_reference_pieces():
    # neighbouring pairs: (x0, x1) turns by pos * f0, (x2, x3) by pos * f1; entries beyond dims pass
    x = np.array([[[1.0, 0.0, 1.0, 0.0, 7.0]]])
    y = R.rotate_pairs(x, [3], 4, 100.0)
    assert np.allclose(y[0, 0], [np.cos(3), np.sin(3), np.cos(0.3), np.sin(0.3), 7.0])
    # the convolution: last column is the token's own, zeros before the start, the bias after the sum
    u = np.arange(1.0, 5.0)[:, None]
    assert np.allclose(R.short_conv(u, np.array([[100.0, 10.0, 1.0]]), np.array([0.5]))[:, 0], [1.5, 12.5, 123.5, 234.5])
    # one step of the two recurrences by hand
    o = R.delta_rule_channel_decay(np.array([[[1.0, 0.0]]]), np.array([[[1.0, 0.0]]]), np.array([[[2.0]]]), np.array([[0.5]]), np.array([[[0.3, 0.9]]]))
    assert np.allclose(o, 1.0)  # S starts at zero: u = beta v, o = (k . q) u
    y = R.state_space_scan(np.array([[[2.0]], [[0.0]]]), np.ones((2, 1, 1)), np.ones((2, 1, 1)), np.array([[0.5], [1.0]]), np.array([np.log(2.0)]), np.array([3.0]))
    assert np.allclose(y[:, 0, 0], [1.0 + 6.0, 0.5])  # dt B x, then its decay exp(-ln 2)
    assert np.allclose(R.norm_one_plus(np.array([[3.0, 4.0]]), np.array([0.0, 1.0]), 0.0), [[3.0 / np.sqrt(12.5), 8.0 / np.sqrt(12.5)]])
    assert abs(R.gelu_tanh(np.array([1.0]))[0] - 0.841192) < 1e-6
    # a layer with shared rows sees the first layer's latent, not its own input's
    cfg = R.make_config(16, 11, [R.latent_layer(2, 4, 2, 4, 6, 5, 0.5, None), R.latent_layer(2, 4, 2, 4, 6, 5, 0.5, None, kv_from=0)], side_dim=0)
    W = R.random_weights(cfg, 1)
    assert "l1.mix.dkv" not in W and "l0.mix.dkv" in W
    a = R.forward(cfg, W, [1, 2, 3])
    W2 = dict(W)
    W2["l0.mix.dkv"] = W["l0.mix.dkv"] * 2.0
    W2["l0.mix.o"] = W["l0.mix.o"] * 0.0
    W1 = dict(W)
    W1["l0.mix.o"] = W["l0.mix.o"] * 0.0
    assert np.abs(R.forward(cfg, W2, [1, 2, 3]) - R.forward(cfg, W1, [1, 2, 3])).max() > 1e-6  # (layer 0's output is off: only the shared rows carry the change)
    assert np.isfinite(a).all()


def _probe(H, m, n_ctx, steps, n_ubatch=64, n_seq=4):
    """llm_decode with a compute callback that records the nodes of every graph (host memory here)"""
    seen = []

    def comp(g, _n):
        gg = g.contents
        nodes = []
        for i in range(gg.n_nodes):
            t = gg.nodes[i].contents
            srcs = [t.src[s].contents.name.decode() if t.src[s] else None for s in range(10)]
            nodes.append((H.ggml_op_name(t.op).decode(), t.name.decode(), srcs, list(t.ne)))
        seen.append(nodes)
        return 0

    fn = L.COMPUTE_FN(comp)
    cp = L.ContextParams(n_ctx, n_ubatch, 1, 0, 1, 0, 0, n_seq)
    c = H.llm_context_new(m, None, fn, C.byref(cp))
    assert c
    for toks, pos, seq in steps:
        n = len(toks)
        assert H.llm_decode(c, n, (C.c_int32 * n)(*toks), (C.c_int32 * n)(*pos), (C.c_int32 * n)(*seq), None) == 0
    caches = [bool(H.llm_context_cache_tensor(c, il, 0)) for il in range(4)]
    H.llm_context_free(c)
    return seen, caches


def test_graph_of_a_mixed_batch(H):
    cfg = small_cfg()
    m = H.llm_model_synth_config(json.dumps(cfg).encode(), 7, H.ggml_backend_cpu_buffer_type(), L.BF16)
    assert m
    seen, caches = _probe(H, m, 256, [([5, 6], [0, 1], [2, 2]), ([20, 21, 30, 22], [0, 1, 2, 2], [0, 0, 2, 0])])
    nodes = seen[-1]
    ops = {}
    for op, *_ in nodes:
        ops[op] = ops.get(op, 0) + 1
    # two latent layers and one attention: three attentions; one state-space and one delta recurrence, each behind a convolution with its store
    assert ops["FLASH_ATTN_EXT"] == 3 and ops["GATED_LINEAR_ATTN"] == 2 and ops["SSM_CONV"] == 4 and ops["ROPE"] == 3
    # cells exist for the latent layer with rows of its own and for the attention branch; the state-space layer and the layer with shared rows have none
    assert caches == [True, False, False, True]
    fa = [n for n in nodes if n[0] == "FLASH_ATTN_EXT"]
    assert fa[0][2][1].startswith("cache_k_l-0") and fa[1][2][1].startswith("cache_k_l-0") and fa[2][2][1].startswith("cache_k_l-3")
    stores = [n[1] for n in nodes if n[0] == "SET_ROWS"]
    assert stores == ["kv_store-0", "k_store-3", "v_store-3"]
    # the recurrences: kinds, the bias of the state-space convolution, beta as an operand of its own
    rec = [n for n in nodes if n[0] == "GATED_LINEAR_ATTN"]
    assert rec[0][1] == "ssd-1" and rec[1][1] == "delta_channel-3" and rec[1][2][8] == "delta_b_pre-3" and rec[0][2][8] is None
    conv = [n for n in nodes if n[0] == "SSM_CONV" and not n[1].startswith("conv_store")]
    assert conv[0][2][4] == "blk.1.ssm_conv1d.bias" and conv[1][2][4] is None
    # the two branches' norms, factors and sum follow one another (the backend runs the seven nodes as one launch)
    names = [n[1] for n in nodes]
    at = names.index("mix_left_rnorm-3")
    assert names[at:at + 7] == ["mix_left_rnorm-3", "mix_left_normed-3", "mix_left-3", "mix_right_rnorm-3", "mix_right_normed-3", "mix_right-3", "mix_sum-3"]
    # ... as do the gate's activation and its product with the side rows, and the state-space gate, its norm in parts and the weight (views between them)
    at = names.index("side_gelu-0")
    assert names[at + 1] == "side_gated-0"
    at = names.index("ssm_z_silu-1")
    assert [x for x, n in zip(names[at:at + 8], nodes[at:at + 8]) if n[0] not in ("RESHAPE", "VIEW")][:4] == ["ssm_z_silu-1", "ssm_gated-1", "ssm_rnorm-1", "ssm_normed-1"]
    # the side input: one small table per layer, read by token
    assert [n[2][0] for n in nodes if n[1].startswith("side_embd")] == ["blk.%d.side_embd.weight" % il for il in range(4)]
    # the last layer goes on with the wanted rows only: here all of them
    assert [n for n in nodes if n[1] == "result_output"][0][3][:2] == [53, 4]
    H.llm_model_free(m)


def test_sequence_ids_beyond_the_state_rows_are_refused(H):
    cfg = small_cfg()
    m = H.llm_model_synth_config(json.dumps(cfg).encode(), 9, H.ggml_backend_cpu_buffer_type(), L.F32)
    fn = L.COMPUTE_FN(lambda g, n: 0)
    cp = L.ContextParams(256, 64, 1, 0, 1, 0, 0, 2)
    c = H.llm_context_new(m, None, fn, C.byref(cp))
    assert H.llm_decode(c, 1, (C.c_int32 * 1)(1), (C.c_int32 * 1)(0), (C.c_int32 * 1)(2), None) == -1
    assert H.llm_decode(c, 1, (C.c_int32 * 1)(1), (C.c_int32 * 1)(0), (C.c_int32 * 1)(1), None) == 0
    H.llm_context_free(c)
    H.llm_model_free(m)
