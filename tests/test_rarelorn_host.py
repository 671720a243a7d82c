"""Host side of the Rarelorn model class, without a GPU: the loader (q, k, v of a mixer as one projection, scalar norm weights kept as rows,
token-shift factors kept as 2-tap convolution weights, experts' gate and up rows in one tensor), what it refuses, the plain reference's own
pieces, and what the scheduler uploads for a mixed batch — where every token finds its predecessors, where the new state rows come from,
the batch rows grouped by sequence — checked against what the sequences' histories say."""
import ctypes as C
import json

import numpy as np
import pytest

import llama_box_amd as L
import rarelorn_ref as R


def small_cfg():
    return R.make_config(40, 53, [
        R.delta_layer(heads=4, kv_heads=2, dim=8, vdim=12, conv=3, mlp=R.moe_cfg(16, 6, 2, count=3, keep=2, scale=1.5)),
        R.mlstm_layer(heads=2, dim=12, vdim=8, mlp=None, gate_cap=9.0),
        R.parallel_layer(heads=4, kv_heads=2, dim=8, vdim=12, conv=4, size=5, rot_dims=4, scale=0.3, softcap=6.0, r_heads=2, r_dim=10, mlp=R.moe_cfg(8, 4, 1), base=100.0,
                         left_scale=1.1, right_scale=0.8, rank=5),
    ], loop=(1, 3, 2), eps=1e-5)


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
        assert (hp.arch, hp.n_layer, hp.n_embd, hp.n_vocab) == (b"rarelorn", 3, 40, 53)
        # q, k, v of unequal heights follow one another in ONE projection; so do their convolution taps
        assert np.array_equal(_get(H, m, "blk.0.attn_qkv.weight")[0], np.concatenate([W["l0.mix.q"], W["l0.mix.k"], W["l0.mix.v"]]))
        assert np.array_equal(_get(H, m, "blk.0.ssm_conv1d.weight")[0], np.concatenate([W["l0.mix.q.conv"], W["l0.mix.k.conv"], W["l0.mix.v.conv"]]))
        assert np.array_equal(_get(H, m, "blk.0.attn_gates.weight")[0], np.concatenate([W["l0.mix.b"], W["l0.mix.a"]]))
        assert np.array_equal(_get(H, m, "blk.0.attn_gates.param").reshape(-1), np.concatenate([W["l0.mix.A_log"], W["l0.mix.dt_bias"]]))
        assert np.array_equal(_get(H, m, "blk.1.attn_gates.bias").reshape(-1), np.concatenate([W["l1.mix.i.b"], W["l1.mix.f.b"]]))
        # a norm's ONE number becomes a row
        assert np.array_equal(_get(H, m, "blk.1.attn_norm.weight").reshape(-1), np.full(40, W["l1.norm1"]))
        assert np.array_equal(_get(H, m, "output_norm.weight").reshape(-1), np.full(40, W["final.norm"]))
        # token-shift factors as 2-tap weights (mu for the previous token, 1 - mu for the token's own), one set per reader
        taps = _get(H, m, "blk.2.time_mix_taps.weight")  # [5][E][2]
        for k, s in enumerate("rkvgw"):
            mu = W["l2.mix.right.mu." + s].astype(np.float32)
            assert np.array_equal(taps[k, :, 0], mu) and np.array_equal(taps[k, :, 1], np.float32(1.0) - mu)
        assert np.array_equal(_get(H, m, "blk.2.time_mix_rkvg.weight"), np.stack([W["l2.mix.right." + s] for s in "rkvg"]))
        assert _get(H, m, "blk.2.time_mix_w1.weight")[0].shape == (5, 40)  # the inner size of the decay's matrices comes from the checkpoint
        assert np.array_equal(_get(H, m, "blk.2.attn_fb.weight")[0], np.stack([W["l2.mix.left.temp"], W["l2.mix.left.pb"]]))
        gu = _get(H, m, "blk.0.ffn_gate_up_exps.weight")  # [expert][gate rows, then up rows][E]
        assert np.array_equal(gu[4], np.concatenate([W["l0.mlp.e4.gate"], W["l0.mlp.e4.up"]]))
        assert H.llm_model_tensor(m, b"blk.0.ffn_gate_inp.weight").contents.type == L.F32
        assert not H.llm_model_tensor(m, b"blk.1.ffn_gate_inp.weight")  # a layer without a feed-forward has none
        H.llm_model_free(m)


@pytest.mark.parametrize("breakage", ["shape", "missing", "heads", "loop", "mixer", "kind", "groups", "top", "norm"])
def test_loader_refuses_what_it_cannot_serve(H, tmp_path, breakage):
    cfg = small_cfg()
    W = R.random_weights(cfg, 4)
    if breakage == "shape":
        W["l0.mix.k.conv"] = W["l0.mix.k.conv"][:, :-1]
    elif breakage == "missing":
        del W["l2.mix.left.pb"]
    elif breakage == "heads":
        cfg["layers"][0]["mixer"]["kv_heads"] = 3
    elif breakage == "loop":
        cfg["loop"]["stop"] = 7
    elif breakage == "mixer":
        cfg["layers"][1]["type"] = "something_else"
    elif breakage == "kind":
        cfg["layers"][2]["mlp"]["kind"] = "dense"
    elif breakage == "groups":
        cfg["layers"][0]["mlp"]["router"]["groups"]["count"] = 4  # six experts do not form four equal groups
    elif breakage == "top":
        cfg["layers"][0]["mlp"]["router"]["groups"]["keep"] = 1
        cfg["layers"][0]["mlp"]["router"]["top"] = 3              # more than the kept groups hold
    elif breakage == "norm":
        W["l1.norm1"] = np.ones(40)                               # this design's norms have one number
    R.save_model(cfg, W, str(tmp_path))
    assert not H.llm_model_load_dir(str(tmp_path).encode(), H.ggml_backend_cpu_buffer_type(), L.BF16)


def test_reference_pieces():
    """The plain reference itself at places where a slip would not show in random data."""
    y = R.short_conv(np.arange(1.0, 5.0)[:, None], np.array([[100.0, 10.0, 1.0]]))  # the last tap is the token's own; zeros before the start
    assert y[:, 0].tolist() == [1.0, 12.0, 123.0, 234.0]
    assert R.window_visible(8, 3)[7].nonzero()[0].tolist() == [5, 6, 7] and R.window_visible(8, 3)[1].nonzero()[0].tolist() == [0, 1]
    x = R.rotate_half(np.ones((1, 1, 6)), [3], 4, 100.0)  # pairs (0, 2) and (1, 3) with frequencies 1 and 0.1; entries 4, 5 pass
    assert np.allclose(x[0, 0], [np.cos(3) - np.sin(3), np.cos(0.3) - np.sin(0.3), np.cos(3) + np.sin(3), np.cos(0.3) + np.sin(0.3), 1, 1])
    h = np.arange(6.0).reshape(3, 2)
    assert np.allclose(R.token_shift_mix(h, np.array([1.0, 0.5])), [[0, 0.5], [0, 2], [2, 4]])
    # the router: scores over ALL experts; only the best groups may be chosen from; weights are the scores themselves, scaled
    z = np.log(np.array([[0.30, 0.02, 0.05, 0.25, 0.20, 0.18]]))
    sel, w = R.router_choice(z, dict(experts=6, top=2, scale=2.0, groups=dict(count=3, keep=1)))
    assert sel.tolist() == [[0, 1]] and np.allclose(w, [[0.6, 0.04]])
    sel, w = R.router_choice(z, dict(experts=6, top=3, scale=1.0, groups=dict(count=3, keep=2)))
    assert sel.tolist() == [[0, 3, 2]] and np.allclose(w, [[0.30, 0.25, 0.05]])
    sel, _ = R.router_choice(z, dict(experts=6, top=3, scale=1.0, groups=dict(count=1, keep=1)))
    assert sel.tolist() == [[0, 3, 4]]
    assert [r[0] for r in R.layer_runs(small_cfg())] == [0, 1, 2, 1, 2]
    assert [(r[1], r[2]) for r in R.layer_runs(small_cfg())][1:] == [(0, True), (0, False), (1, True), (1, False)]


def _probe(H, m, n_ctx, steps, n_ubatch=64, n_seq=4):
    """llm_decode with a compute callback that records op counts and the named inputs the engine filled (host memory here)."""
    seen = []
    want = (b"KQ_mask", b"seq_hist", b"seq_upd", b"seq_tok", b"seq_info", b"k_idxs", b"inp_pos")

    def comp(g, _n):
        gg = g.contents
        ops, inputs = {}, {}
        for i in range(gg.n_nodes):
            t = gg.nodes[i].contents
            name = H.ggml_op_name(t.op).decode()
            ops[name] = ops.get(name, 0) + 1
            for s in range(10):
                if t.src[s] and t.src[s].contents.name.startswith(want):
                    mt = t.src[s].contents
                    ct = {L.F32: C.c_float, L.I32: C.c_int32, L.I64: C.c_int64}[mt.type]
                    inputs[mt.name.decode()] = np.ctypeslib.as_array(C.cast(mt.data, C.POINTER(ct)), shape=(mt.ne[1], mt.ne[0])).copy()
        seen.append((ops, inputs))
        return 0

    fn = L.COMPUTE_FN(comp)
    cp = L.ContextParams(n_ctx, n_ubatch, 1, 0, 1, 0, 0, n_seq)
    c = H.llm_context_new(m, None, fn, C.byref(cp))
    assert c
    for toks, pos, seq in steps:
        n = len(toks)
        assert H.llm_decode(c, n, (C.c_int32 * n)(*toks), (C.c_int32 * n)(*pos), (C.c_int32 * n)(*seq), None) == 0
    H.llm_context_free(c)
    return seen


def _where(code, rows_of, fed_before):
    """a history code -> the position it names in its sequence (None: before the start); rows_of: batch row -> position; fed_before: slot -> positions fed before this batch"""
    if code == -1:
        return None
    if code >= 0:
        return ("row", rows_of[code])
    cd = -2 - code
    slot, age = cd >> 6, cd & 63
    return ("state", slot, fed_before[slot] - 1 - age)


def test_scheduler_inputs_of_a_mixed_batch(H):
    cfg = small_cfg()
    m = H.llm_model_synth_config(json.dumps(cfg).encode(), 7, H.ggml_backend_cpu_buffer_type(), L.BF16)
    assert m
    # sequence 2: positions 0..1 as one portion; then sequence 0 (0..6) beside three more tokens of sequence 2, interleaved
    s1 = ([5, 6], [0, 1], [2, 2])
    toks2 = [20, 21, 30, 22, 23, 31, 24, 25, 26, 32]
    seq2 = [0, 0, 2, 0, 0, 2, 0, 0, 0, 2]
    pos2 = [0, 1, 2, 2, 3, 3, 4, 5, 6, 4]
    seen = _probe(H, m, 256, [s1, (toks2, pos2, seq2)])
    ops, inp = seen[-1]
    # five layer runs: delta, then (mlstm, parallel) twice — convolutions and their stores (the parallel mixer has two of each), recurrences, one attention per parallel run
    assert ops["SSM_CONV"] == 2 * (1 + 2 * 2) and ops["GATED_LINEAR_ATTN"] == 3 and ops["RWKV_WKV6"] == 2 and ops["FLASH_ATTN_EXT"] == 2
    assert len([k for k in inp if k.startswith("KQ_mask")]) == 1
    hs = 3  # the longest look-back: four taps
    hist = inp["seq_hist"]
    assert hist.shape == (len(toks2), hs)
    fed_before = {0: 0, 2: 2}
    for i, (s, p) in enumerate(zip(seq2, pos2)):
        for d in range(1, hs + 1):
            got = _where(int(hist[i, d - 1]), pos2, fed_before)
            if p - d < 0:
                assert got is None
            elif p - d >= fed_before[s]:  # a row of this batch: of the same sequence, at the right position
                assert got == ("row", p - d) and seq2[int(hist[i, d - 1])] == s
            else:
                assert got == ("state", s, p - d)
    info = inp["seq_info"]
    assert info.tolist() == [[0, 7, 0, 1], [7, 3, 2, 0]]  # (first entry, count, slot, starts here)
    assert inp["seq_tok"].reshape(-1).tolist() == [0, 1, 3, 4, 6, 7, 8, 2, 5, 9]
    upd = inp["seq_upd"]
    assert upd.shape == (2, hs)
    assert [_where(int(c), pos2, fed_before) for c in upd[0]] == [("row", 6), ("row", 5), ("row", 4)] and [int(c) for c in upd[0]] == [8, 7, 6]
    assert [int(c) for c in upd[1]] == [9, 5, 2]
    H.llm_model_free(m)


def test_micro_batches_carry_the_state(H):
    """a prompt cut into micro-batches by the engine: the first tokens of the second micro-batch find their predecessors in the state, and short sequences keep older rows"""
    cfg = small_cfg()
    m = H.llm_model_synth_config(json.dumps(cfg).encode(), 9, H.ggml_backend_cpu_buffer_type(), L.F32)
    seen = _probe(H, m, 256, [(list(range(1, 12)), list(range(11)), [1] * 11)], n_ubatch=8)
    assert len(seen) == 2
    first, second = seen[0][1], seen[1][1]
    assert first["seq_hist"][0].tolist() == [-1, -1, -1] and first["seq_hist"][2].tolist() == [1, 0, -1] and first["seq_info"].tolist() == [[0, 8, 1, 1]]
    st = lambda age: -2 - (1 * 64 + age)
    assert second["seq_hist"].tolist() == [[st(0), st(1), st(2)], [0, st(0), st(1)], [1, 0, st(0)]] and second["seq_info"].tolist() == [[0, 3, 1, 0]]
    assert second["seq_upd"].tolist() == [[2, 1, 0]]
    # one more token for a sequence that has fed two: the state keeps the older row, and what lies before the start stays nothing
    seen = _probe(H, m, 256, [([3, 4], [0, 1], [0, 0]), ([5], [2], [0])])
    assert seen[1][1]["seq_upd"].tolist() == [[0, -2 - 0, -2 - 1]] and seen[1][1]["seq_hist"].tolist() == [[-2 - 0, -2 - 1, -1]]
    H.llm_model_free(m)


def test_a_model_without_attention_has_no_masks_and_no_cell_indices(H):
    cfg = R.make_config(24, 31, [R.mlstm_layer(2, 8, 8, None), R.delta_layer(2, 1, 8, 4, 1, R.moe_cfg(8, 2, 1))])
    m = H.llm_model_synth_config(json.dumps(cfg).encode(), 9, H.ggml_backend_cpu_buffer_type(), L.F32)
    assert m
    ops, inp = _probe(H, m, 256, [([1, 2, 3], [0, 1, 2], [0, 0, 0])])[0]
    assert "FLASH_ATTN_EXT" not in ops and "SET_ROWS" not in ops and not [k for k in inp if k.startswith(("KQ_mask", "k_idxs", "inp_pos"))]
    assert ops["SSM_CONV"] == 1  # one tap: a convolution without history has no state to store
    H.llm_model_free(m)


def test_sequence_ids_beyond_the_state_slots_are_refused(H):
    m = H.llm_model_synth_config(json.dumps(small_cfg()).encode(), 9, H.ggml_backend_cpu_buffer_type(), L.F32)
    fn = L.COMPUTE_FN(lambda g, n: 0)
    cp = L.ContextParams(256, 64, 1, 0, 1, 0, 0, 2)
    c = H.llm_context_new(m, None, fn, C.byref(cp))
    one = (C.c_int32 * 1)
    assert H.llm_decode(c, 1, one(3), one(0), one(1), None) == 0
    assert H.llm_decode(c, 1, one(3), one(0), one(2), None) == -1
    H.llm_context_free(c)
    H.llm_model_free(m)
