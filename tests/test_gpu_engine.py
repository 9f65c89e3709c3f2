"""GPU parity of the UV-50M engine (fused kernels + attention + sampler through the C ABI) against the torch-CPU oracle
that is itself pinned by golden vectors from the reference.  Restates tests/test_math_kernels.py:152-189 and
tests/test_math_model.py:303-323 of the reference."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _setup(name="uv-test", dtype=torch.float32, seed=0, perturb=0.06, **over):
    from oracle.model import OracleModel
    from ultraviolet_amd.engine import UVEngine, UVWeights, make_config, random_params
    cfg = make_config(name, **over)
    params = random_params(cfg, seed, perturb=perturb)
    eng = UVEngine(UVWeights(cfg, params, dtype, DEV), max_tokens=2048)
    return cfg, params, eng, OracleModel


def _prompts(cfg, lens, seed=0):
    rng = np.random.default_rng(seed)
    return [rng.integers(1, cfg.vocab_size, size=int(n)).tolist() for n in lens]


def _teacher_forced(eng, prompts, cont, max_len):
    from ultraviolet_amd.engine import KVState
    B = len(prompts)
    st = KVState(eng.cfg, B, max_len, DEV)
    outs = [eng.logits(eng.prefill(prompts, list(range(B)), st)).cpu()]
    for t in range(cont.shape[1]):
        outs.append(eng.logits(eng.decode_step(torch.as_tensor(cont[:, t]).to(DEV), st)).cpu())
    torch.cuda.synchronize()
    return torch.stack(outs, 1).numpy(), st


def _oracle_teacher_forced(m, prompts, cont, max_len):
    from oracle.model import OracleState
    B = len(prompts)
    st = OracleState(m.cfg, B, max_len)
    outs = [m.logits(m.prefill(prompts, list(range(B)), st)).numpy()]
    for t in range(cont.shape[1]):
        outs.append(m.logits(m.decode_step(cont[:, t], st)).numpy())
    return np.stack(outs, 1), st


def test_fp32_engine_matches_oracle_logits_and_cache():
    """Through ring wrap (window 16) and left padding: logits close, int8 cache bytes and scales equal up to isolated
    rounding ties, positions exact."""
    cfg, params, eng, OracleModel = _setup(window=16)
    prompts = _prompts(cfg, (5, 12, 9, 20, 1, 17))
    cont = np.random.default_rng(1).integers(1, cfg.vocab_size, size=(6, 30))
    lg, st = _teacher_forced(eng, prompts, cont, 64)
    ref, ost = _oracle_teacher_forced(OracleModel(cfg, params, torch.float32), prompts, cont, 64)
    assert np.isfinite(lg).all()
    assert np.abs(lg - ref).max() < 2e-2                      # fp16 q in the attention kernel, fp16 P
    assert (lg.argmax(-1) == ref.argmax(-1)).mean() > 0.98
    assert np.array_equal(st.pos.cpu().numpy(), ost.pos) and np.array_equal(st.starts.cpu().numpy(), ost.starts)
    nb = nd = 0
    for l in range(cfg.n_layers):
        for mine, o in ((st.k[l], ost.k[l]), (st.v[l], ost.v[l])):
            # only slots a real token was written to are comparable (the oracle's padded prefill also writes pad slots)
            d = np.abs(mine.cpu().numpy().astype(np.int32) - o.astype(np.int32))
            valid = np.zeros(d.shape[:3], bool)
            S = d.shape[2]
            for b in range(d.shape[0]):
                for t in range(int(ost.starts[b]), int(ost.pos[b])):
                    if cfg.is_global(l) or t >= int(ost.pos[b]) - S:
                        valid[b, :, t if cfg.is_global(l) else t % S] = True
            nb += int(valid.sum()) * d.shape[3]
            nd += int((d[valid] != 0).sum())
            assert d[valid].max() <= 2
    # deeper layers see activations that differ at the 1e-3 level (fp16 q and P in the attention kernel), which moves
    # codes near a rounding boundary by one step; the quantizer itself is checked bit-exactly on identical inputs in
    # test_gpu_kernels.py and on layer 0 below
    assert nd < 0.15 * nb, (nd, nb)


def test_first_layer_cache_is_bit_exact():
    """Layer 0 sees only embedding -> norm -> QKV GEMM -> QK-norm / RoPE before the quantizer; with fp32 GEMMs its int8
    bytes and fp16 scales must equal the oracle's (GEMM summation order can flip a tie: none does on this case)."""
    cfg, params, eng, OracleModel = _setup(window=16)
    prompts = _prompts(cfg, (16, 16, 16, 16), seed=3)
    cont = np.random.default_rng(4).integers(1, cfg.vocab_size, size=(4, 8))
    _, st = _teacher_forced(eng, prompts, cont, 32)
    _, ost = _oracle_teacher_forced(OracleModel(cfg, params, torch.float32), prompts, cont, 32)
    k = st.k[0].cpu().numpy()
    dk, ds = (k != ost.k[0]).mean(), (st.k_scale[0].cpu().numpy().view(np.uint16) != ost.ks[0].view(np.uint16)).mean()
    # measured: no differing code, no differing scale; the bars leave room for one flipped round-half-even tie per 10^4 codes
    assert dk <= 1e-4 and ds <= 1e-3, (dk, ds)


@pytest.mark.parametrize("name,over", [("uv-test", dict(window=16)), ("uv-50m-alpha", dict())])
def test_greedy_64_tokens_identical_fp32(name, over):
    """BASELINE config 1 shape: 8 prompts, lengths U[32, 128], greedy 64 new tokens, int8 KV: identical token streams
    (fp32 activations on the GPU vs the fp32 CPU oracle)."""
    cfg, params, eng, OracleModel = _setup(name, perturb=0.06, **over)
    rng = np.random.default_rng(0)
    lens = rng.integers(32, 129, size=8)
    prompts = [rng.integers(1, cfg.vocab_size, size=int(n)).tolist() for n in lens]
    out = np.array(eng.generate(prompts, 64, temperature=0.0))
    ref, lgs, _ = OracleModel(cfg, params, torch.float32).generate_greedy(prompts, 64, return_logits=True)
    assert len(np.unique(ref)) > 8                                  # the stream is not one repeated token
    # An fp32 engine keeps fp32 queries and probabilities (the plain fp32 attention kernel), so what separates it from the
    # oracle is the summation order of the GEMMs and, through it, an int8 code of the cache that sits on a rounding tie
    # and lands one step away (one code step of one key moves the logits by ~1e-4).  A stream may therefore leave the
    # oracle's only where the oracle's own top-2 logits are closer than 1e-3 (on logits of magnitude ~18), every such
    # row is printed with its step and gap, and most rows stay identical over all 64 steps.
    identical = 0
    for b in range(len(prompts)):
        d = np.nonzero(out[b] != ref[b])[0]
        if len(d) == 0:
            identical += 1
            continue
        t = int(d[0])
        top2 = np.sort(lgs[b, t])[-2:]
        print(f"row {b} leaves the oracle's stream at step {t}: oracle top-2 logit gap {top2[1] - top2[0]:.2e}")
        assert top2[1] - top2[0] < 1e-3, f"row {b} diverges at step {t} with top-2 logit gap {top2[1] - top2[0]:.2e}"
    assert identical >= len(prompts) - 2, identical


# the decode pass's launch plans by row count, forced here at a few rows:
# (skinny_rows, fold_qkv_rows, fold_o_rows, fold_gu_rows, form of the hand-written GEMM)
_TRUNK_PLANS = {"small": None, "large-skinny-attn-block": (0, 1 << 30, 1 << 30, 0, 0), "large-library": (0, 0, 0, 0, 0),
                "large-tiled-64": (0, 1 << 30, 1 << 30, 1 << 30, 4), "large-tiled-128": (0, 1 << 30, 1 << 30, 1 << 30, 3),
                "large-tiled-64-own-down": (0, 1 << 30, 1 << 30, 1 << 30, 4, (0, 1 << 30))}


def _force_plan(eng, plan):
    if _TRUNK_PLANS[plan] is not None:
        eng.skinny_rows, eng.fold_qkv_rows, eng.fold_o_rows, eng.fold_gu_rows, eng.gemm_config = _TRUNK_PLANS[plan][:5]
        eng.general_skinny_rows = eng.skinny_rows   # the unfused path the plans are compared with runs the library's GEMMs too
        if len(_TRUNK_PLANS[plan]) > 5:   # the down projection on this library's tiled GEMM too
            eng.fold_down_rows = _TRUNK_PLANS[plan][5]


@pytest.mark.parametrize("dtype,max_bar,mean_bar", [(torch.bfloat16, 0.15, 0.02), (torch.float16, 0.04, 0.005)])
@pytest.mark.parametrize("plan", list(_TRUNK_PLANS))
def test_16bit_engine_close_to_oracle(plan, dtype, max_bar, mean_bar):
    """The 16-bit engine against the oracle run in the same 16-bit arithmetic (both sides use the int8 cache and round at
    the same points), for each of the decode pass's launch plans (the one for few rows, and the two for many rows:
    residual updates inside the projections, the MLP's pre-norm inside the SwiGLU launch).  Bars: twice the measured gap -
    bf16 max 0.062-0.077 / mean 0.0099, fp16 max 0.016-0.020 / mean 0.0026 on logits in (0, 23), i.e. one or two units in
    the last place of the tied head's 16-bit output; every argmax agrees.  (The reference's bar for its int8 kernel path
    against its unquantized SDPA path is 0.25 / 0.9, tests/test_math_kernels.py:170-172.)"""
    cfg, params, eng, OracleModel = _setup(dtype=dtype, window=16)
    _force_plan(eng, plan)
    prompts = _prompts(cfg, (5, 12, 9, 20, 3, 17))
    cont = np.random.default_rng(1).integers(1, cfg.vocab_size, size=(6, 30))
    lg, _ = _teacher_forced(eng, prompts, cont, 64)
    ref, _ = _oracle_teacher_forced(OracleModel(cfg, params, dtype), prompts, cont, 64)
    assert np.isfinite(lg).all()
    d = np.abs(lg - ref)
    assert d.max() < max_bar and d.mean() < mean_bar, (d.max(), d.mean())
    assert (lg.argmax(-1) == ref.argmax(-1)).mean() > 0.98


@pytest.mark.parametrize("dtype,max_bar,mean_bar", [(torch.bfloat16, 0.15, 0.02), (torch.float16, 0.04, 0.005)])
def test_prefill_pass_on_own_gemms_close_to_oracle(dtype, max_bar, mean_bar):
    """The plans of general-path passes with many rows (here 663 packed prompt tokens): from 448 rows the QKV, output and
    gate-up projections on this library's GEMM with the residual update in place, the extended QKV projection with the
    block's pre-norm as its row scale, and the post-processing taking the gates' logits from the projection instead of from
    the normalised hidden; from big_rows rows (forced to 1 here) the down projection too - each against the oracle in the
    same 16-bit arithmetic, to the bars of the other plans, and against the same engine on the vendor library's GEMMs with
    a norm launch per block (same positions, first-layer keys equal up to last-place flips of the projection)."""
    cfg, params, eng, OracleModel = _setup(dtype=dtype, window=128)
    prompts = _prompts(cfg, (100, 130, 90, 150, 129, 64))
    cont = np.random.default_rng(2).integers(1, cfg.vocab_size, size=(6, 6))
    ref, _ = _oracle_teacher_forced(OracleModel(cfg, params, dtype), prompts, cont, 192)
    eng.tiled_prefill = False
    base, st0 = _teacher_forced(eng, prompts, cont, 192)
    eng.tiled_prefill = True
    runs = [(base, st0), _teacher_forced(eng, prompts, cont, 192)]
    eng.big_rows = 1
    runs.append(_teacher_forced(eng, prompts, cont, 192))
    for got, st in runs:
        assert np.isfinite(got).all()
        d = np.abs(got - ref)
        assert d.max() < max_bar and d.mean() < mean_bar, (d.max(), d.mean())
        assert (got.argmax(-1) == ref.argmax(-1)).mean() > 0.98
        assert torch.equal(st0.pos, st.pos) and torch.equal(st0.starts, st.starts)
        dk = (st0.k[0].int() - st.k[0].int()).abs()
        assert int(dk.max()) <= 1 and float((dk != 0).float().mean()) < 2e-3, (int(dk.max()), float((dk != 0).float().mean()))


def test_graph_replay_matches_eager_and_seeded_sampling_is_reproducible():
    """One captured graph serves every step (positions are read on the device); replays equal eager
    (reference: tests/test_math_kernels.py:176-189).  Seeded sampling does not depend on graph vs eager."""
    cfg, params, eng, _ = _setup(dtype=torch.bfloat16, window=16)
    prompts = _prompts(cfg, (6, 3, 4, 9), seed=5)
    a = eng.generate(prompts, 40, temperature=0.0, use_graph=False)
    b = eng.generate(prompts, 40, temperature=0.0, use_graph=True)
    assert a == b
    s1, lp1 = eng.generate(prompts, 40, temperature=1.0, seed=11, use_graph=False, return_logp=True)
    s2, lp2 = eng.generate(prompts, 40, temperature=1.0, seed=11, use_graph=True, return_logp=True)
    s3 = eng.generate(prompts, 40, temperature=1.0, seed=12)
    assert s1 == s2 and np.array_equal(lp1, lp2) and s1 != s3
    assert np.isfinite(lp1).all() and (lp1 <= 1e-6).all()


def test_prefill_left_pad_vs_zero_start_positions():
    """Starting every prompt at position 0 instead of left-padding changes cache slots but not the logits
    (RoPE is relative, global layers have no positions)."""
    from ultraviolet_amd.engine import KVState
    cfg, params, eng, _ = _setup(window=16)
    prompts = _prompts(cfg, (7, 19, 2), seed=6)
    st1, st2 = KVState(cfg, 3, 64, DEV), KVState(cfg, 3, 64, DEV)
    l1 = eng.logits(eng.prefill(prompts, [0, 1, 2], st1, left_pad=True))
    l2 = eng.logits(eng.prefill(prompts, [2, 0, 1], st2, left_pad=False))
    assert (l1 - l2).abs().max() < 2e-3
    assert st2.starts.tolist() == [0, 0, 0] and sorted(st2.pos.tolist()) == [2, 7, 19]
    tok = torch.tensor([5, 6, 7], device=DEV)
    d1 = eng.logits(eng.decode_step(tok, st1))
    d2 = eng.logits(eng.decode_step(tok[[1, 2, 0]], st2))
    assert (d1 - d2[[2, 0, 1]]).abs().max() < 5e-2   # keys are rotated, hence quantized, at different absolute positions


@pytest.mark.parametrize("window", [16, 32])
def test_mixed_step_matches_separate_prefill_and_decode(window):
    """A mixed batch (two new prompts prefilled into free cache rows while three running rows decode, one pass over all
    token rows) against the oracle's separate prefill and decode step: logits close, positions exact, the new rows'
    layer-0 cache bytes equal, the running rows' appended keys equal.  window 16 takes the unfused attention epilogue,
    window 32 the fused one."""
    from oracle.model import OracleState
    from ultraviolet_amd.engine import KVState
    cfg, params, eng, OracleModel = _setup(window=window)
    om = OracleModel(cfg, params, torch.float32)
    old, new = _prompts(cfg, (9, 21, 14), seed=5), _prompts(cfg, (18, 7), seed=6)
    cont = np.random.default_rng(7).integers(1, cfg.vocab_size, size=(3, 6))
    st = KVState(cfg, 6, 64, DEV)
    ost, ost_new = OracleState(cfg, 3, 64), OracleState(cfg, 2, 64)
    eng.prefill(old, [0, 1, 2], st)       # left-padded positions, as the oracle (and the reference) lay prompts out
    om.prefill(old, [0, 1, 2], ost)
    dec_rows = torch.tensor([0, 1, 2], device=DEV)
    for t in range(5):   # rows 0..2 run ahead with plain decode steps over their three rows
        tok = torch.as_tensor(cont[:, t]).to(DEV)
        h = eng._trunk(tok, st.pos[dec_rows].clone(), 3, lambda l, q: eng.cache_attention(l, q, st, st.pos[dec_rows], st.starts[dec_rows], 3, rows=dec_rows),
                       rows=dec_rows, st=st)
        st.pos[dec_rows] += 1
        om.decode_step(cont[:, t], ost)
    pk = eng.pack_prompts(new, [4, 5], st.max_len)
    rows_d = torch.tensor([0, 1, 2, -1], device=DEV)                      # one padding row, as a bucketed step has
    tok_d = torch.as_tensor(np.append(cont[:, 5], 0)).to(DEV)
    pos_d = torch.cat([st.pos[dec_rows], torch.zeros(1, dtype=torch.long, device=DEV)])
    starts_d = torch.cat([st.starts[dec_rows], torch.zeros(1, dtype=torch.long, device=DEV)])
    hp, hd = eng.mixed_step(pk, tok_d, pos_d, starts_d, rows_d, st)
    lg_p, lg_d = eng.logits(hp).cpu().numpy(), eng.logits(hd[:3]).cpu().numpy()
    ref_p = om.logits(om.prefill(new, [0, 1], ost_new)).numpy()
    ref_d = om.logits(om.decode_step(cont[:, 5], ost)).numpy()
    assert np.abs(lg_p - ref_p).max() < 2e-2 and np.abs(lg_d - ref_d).max() < 2e-2
    assert (lg_p.argmax(-1) == ref_p.argmax(-1)).all() and (lg_d.argmax(-1) == ref_d.argmax(-1)).all()
    assert st.pos[4:6].tolist() == ost_new.pos.tolist() and st.starts[4:6].tolist() == ost_new.starts.tolist()
    k0 = st.k[0].cpu().numpy()
    S = k0.shape[2]
    for j in range(2):                      # slots the new prompts' real tokens were written to
        lo, hi = int(ost_new.starts[j]), int(ost_new.pos[j])
        sl = [t if cfg.is_global(0) else t % S for t in range(lo if cfg.is_global(0) else max(lo, hi - S), hi)]
        assert (k0[4 + j][:, sl] != ost_new.k[0][j][:, sl]).mean() < 5e-3
    p_old = ost.pos - 1                     # the position the mixed step appended for rows 0..2
    for r in range(3):
        t = int(p_old[r])
        s_ = t if cfg.is_global(0) else t % k0.shape[2]
        assert (k0[r, :, s_] != ost.k[0][r, :, s_]).mean() < 5e-2


class _StubModel:
    """Stands in for the reference's MathLM: patch_model only reads .cfg (the reference's field names) and .state_dict()
    (the reference's parameter names) and binds methods on the instance."""

    def __init__(self, cfg, params):
        import types
        self.cfg = types.SimpleNamespace(**cfg.to_dict(), mudd=False, local_mixer="attn", conv_layers=None, bigram_rows=0)
        self._sd = {k: torch.as_tensor(np.asarray(v), dtype=torch.float32, device=DEV) for k, v in params.items()}

    def state_dict(self):
        return self._sd


def test_patch_model_binds_the_reference_entry_points():
    """patch_model / new_state / prefill(idx, starts, st) / decode_step(tok, st, g_len) / unpatch_model with the reference's
    signatures (fast_decode.py:70-115, 272-334, 341-364) give the engine's results; weights refresh in place."""
    from ultraviolet_amd.engine import KVState
    from ultraviolet_amd.kernels import fast_decode as fd
    cfg, params, eng, _ = _setup(window=32)
    m = fd.patch_model(_StubModel(cfg, params), kv_dtype="int8", dtype=torch.float32, max_tokens=512)
    prompts = _prompts(cfg, (7, 19, 12), seed=8)
    T = 19
    idx = torch.zeros(3, T, dtype=torch.long)
    starts = torch.tensor([T - len(p) for p in prompts])
    for b, p in enumerate(prompts):
        idx[b, T - len(p):] = torch.as_tensor(p)
    st = m.new_state(3, 48)
    assert isinstance(st, fd.KernelDecodeState) and st.kv_dtype == "int8" and st.k[0].dtype == torch.int8
    lg = m.prefill(idx.to(DEV), starts.to(DEV), st)
    st2 = KVState(cfg, 3, 48, DEV)
    ref = eng.logits(eng.prefill(prompts, [0, 1, 2], st2))
    torch.testing.assert_close(lg, ref, atol=1e-5, rtol=1e-5)
    assert st.pos.tolist() == [T] * 3 and st.starts.tolist() == starts.tolist() and st.host_pos.tolist() == [T] * 3
    tok = lg.argmax(-1)
    lg1 = m.decode_step(tok, st, 64)
    ref1 = eng.logits(eng.decode_step(tok, st2))
    torch.testing.assert_close(lg1, ref1, atol=1e-5, rtol=1e-5)
    assert st.pos.tolist() == [T + 1] * 3
    h = fd.decode_step_fast(m, lg1.argmax(-1), st, 64, return_hidden=True)
    assert h.shape == (3, cfg.d_model)
    # in-place refresh: new parameters, same device addresses
    ptr = m._uvmi_engine.w.layers[0]["wqkv"].data_ptr()
    m._sd = {k: v * 1.01 if k.endswith("wv") else v for k, v in m._sd.items()}
    fd.sync_patched_weights(m)
    assert m._uvmi_engine.w.layers[0]["wqkv"].data_ptr() == ptr
    lg2 = m.decode_step(tok, st, 64)
    assert not torch.allclose(lg2, lg1)
    fd.unpatch_model(m)
    assert not hasattr(m, "decode_step")
    from ultraviolet_amd import _lib as L
    with pytest.raises(L.UvmiError):
        fd.patch_model(_StubModel(cfg, params), kv_dtype="fp8")


def _fused_vs_unfused(cfg, eng, steps=40, resync=True, lens=(5, 40, 17, 33, 1, 26), max_len=96, kv_dtype="int8"):
    """Run the same teacher-forced decode with and without the fused QKV path from identical prefilled states; after every
    step the fused state's caches are overwritten with the unfused ones so that differences do not accumulate.  Returns
    per-step hidden differences, argmax agreement of the logits and per-layer cache statistics."""
    from ultraviolet_amd.engine import KVState
    _fused_vs_unfused.gaps = []
    prompts = _prompts(cfg, lens, seed=11)
    B = len(prompts)
    cont = np.random.default_rng(12).integers(1, cfg.vocab_size, size=(B, steps))
    sts = [KVState(cfg, B, max_len, DEV, kv_dtype=kv_dtype, dtype=eng.dtype) for _ in range(2)]
    bits = (lambda t: t.int()) if kv_dtype == "int8" else (lambda t: t.view(torch.int16).int())   # an unquantized cache: compared bit for bit
    for st in sts:
        eng.prefill(prompts, list(range(B)), st)
    hdiff, agree, cmax, cfrac, sfrac = [], [], np.zeros(cfg.n_layers), np.zeros(cfg.n_layers), np.zeros(cfg.n_layers)
    for t in range(steps):
        tok = torch.as_tensor(cont[:, t]).to(DEV)
        h0 = eng.decode_step(tok, sts[0], fuse=False).clone()
        h1 = eng.decode_step(tok, sts[1], fuse=True).clone()
        assert torch.isfinite(h1.float()).all()
        hdiff.append(float((h0.float() - h1.float()).abs().max()))
        lg0, lg1 = eng.logits(h0), eng.logits(h1)
        same = lg0.argmax(-1) == lg1.argmax(-1)
        agree.append(float(same.float().mean()))
        if not bool(same.all()):   # where the two paths pick different tokens, the unfused path's own top-2 gap (a near-tie, or a bug)
            top2 = lg0.topk(2, dim=-1).values
            _fused_vs_unfused.gaps.append(float((top2[:, 0] - top2[:, 1])[~same].max()))
        for l in range(cfg.n_layers):
            for a, b_, sa, sb in ((sts[0].k[l], sts[1].k[l], sts[0].k_scale[l], sts[1].k_scale[l]),
                                  (sts[0].v[l], sts[1].v[l], sts[0].v_scale[l], sts[1].v_scale[l])):
                d = (bits(a) - bits(b_)).abs()
                cmax[l] = max(cmax[l], int(d.max()))
                cfrac[l] = max(cfrac[l], float((d > 0).float().sum()) / (B * cfg.n_kv_heads * cfg.head_dim))   # of the bytes written this step
                if sa is not None:
                    sfrac[l] = max(sfrac[l], float((sa.view(torch.int16) != sb.view(torch.int16)).float().sum()) / (B * cfg.n_kv_heads))
                if resync:
                    b_.copy_(a)
                    if sa is not None:
                        sb.copy_(sa)
    assert sts[0].pos.tolist() == sts[1].pos.tolist()
    return hdiff, agree, cmax, cfrac, sfrac


_fused_vs_unfused.gaps = []


def _check_agreement(agree, dtype):
    """The two paths' hidden states differ by units in the last place, so their argmax differs wherever the model's own top
    two logits are closer than that noise - often, on a randomly initialised model with 32 768 softcapped logits.  What must
    hold: every disagreement sits at such a near-tie (the reference path's top-2 gap is of the size of the last-place noise
    of a logit, not larger), and near-ties are a minority."""
    gaps, _fused_vs_unfused.gaps = _fused_vs_unfused.gaps, []
    noise = 0.08 if dtype == torch.bfloat16 else 0.02      # logits live in (0, 23): a few units in the last place of the hidden, through the head
    assert all(g < noise for g in gaps), (max(gaps), noise)
    assert np.mean(agree) > 0.8, np.mean(agree)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("gate_ch", [0, 128])
def test_fused_qkv_single_layer_is_exact(dtype, gate_ch):
    """One layer isolates the fused kernel from error propagation: QK-norm, rotation, value embedding and the quantiser
    must reproduce the separate post-processing kernel bit for bit (identical int8 bytes and fp16 scales at every step,
    through ring wrap-around), and the layer output - own key merged from registers instead of streamed, gate logits from
    the projection instead of a separate dot product - must agree to a unit or two in the last place."""
    cfg, params, eng, _ = _setup("uv-test", dtype=dtype, perturb=0.05, window=32, n_layers=1, global_every=0, ve_every=1,
                                 attn_gate_channels=gate_ch)
    assert eng.fuse_qkv and cfg.has_ve(0)
    hdiff, agree, cmax, cfrac, sfrac = _fused_vs_unfused(cfg, eng)
    assert cmax.max() == 0 and sfrac.max() == 0
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    assert max(hdiff) <= 4 * 2 * ulp, max(hdiff)      # |h| < 4 after the final norm: one ulp there is 2 * ulp(1)
    cfg, params, eng, _ = _setup("uv-test", dtype=dtype, perturb=0.05, window=0, n_layers=1, global_every=1, ve_every=0,
                                 attn_gate_channels=gate_ch)   # a global layer (no rotation, linear cache), no value embedding
    hdiff, agree, cmax, cfrac, sfrac = _fused_vs_unfused(cfg, eng)
    assert cmax.max() == 0 and sfrac.max() == 0 and max(hdiff) <= 4 * 2 * ulp


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("name,over", [("uv-test", dict(window=32)), ("uv-50m-alpha", dict())])
def test_fused_qkv_decode_matches_unfused(dtype, name, over):
    """Whole models: layer 0 appends identical bytes; deeper layers see inputs that differ in the last place of the
    activation type, which moves int8 codes near a rounding boundary by a step or two; the final hidden states stay within
    a few units in the last place and the logits' argmax agrees."""
    cfg, params, eng, _ = _setup(name, dtype=dtype, perturb=0.05, **over)
    assert eng.fuse_qkv
    hdiff, agree, cmax, cfrac, sfrac = _fused_vs_unfused(cfg, eng, steps=24)
    assert cmax[0] == 0 and sfrac[0] == 0
    # the perturbation grows layer by layer (16-bit activations: one unit in the last place of a key is half an int8 code)
    assert (cmax <= 3 + np.arange(cfg.n_layers)).all(), cmax
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    assert max(hdiff) < 16 * 2 * ulp, max(hdiff)
    _check_agreement(agree, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("plan", ["large-skinny-attn-block", "large-library", "large-tiled-64", "large-tiled-128", "large-tiled-64-own-down"])
def test_large_pass_plans_match_unfused(dtype, plan):
    """The launch plans of passes with many rows (forced here at 6 rows) against the unfused general path, to the same
    bounds as the small-pass plan above."""
    cfg, params, eng, _ = _setup("uv-50m-alpha", dtype=dtype, perturb=0.05)
    _force_plan(eng, plan)
    hdiff, agree, cmax, cfrac, sfrac = _fused_vs_unfused(cfg, eng, steps=24)
    assert cmax[0] == 0 and sfrac[0] == 0
    assert (cmax <= 3 + np.arange(cfg.n_layers)).all(), cmax
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    assert max(hdiff) < 16 * 2 * ulp, max(hdiff)
    _check_agreement(agree, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("lens,window,max_len", [((100, 130, 90, 150, 129, 64), 128, 192), ((300, 420, 260, 500, 257, 300), 256, 576),
                                                 ((300, 20, 260, 330, 1, 300), 1024, 1056)])
def test_fused_qkv_single_layer_is_exact_with_several_waves_per_row(dtype, lens, window, max_len):
    """Caches of 128..255 slots run the attention kernel with 2 waves per row and longer ones with 4 (own key formed by the
    first wave, own value by the second, q handed over through LDS): the appended bytes must still equal the separate
    post-processing kernel's, on a ring layer (wraps during the run where it is shorter than the rows) and on a global
    layer, also on caches of more than 1024 slots."""
    for over in (dict(window=window, global_every=0, ve_every=1), dict(window=0, global_every=1, ve_every=0)):
        cfg, params, eng, _ = _setup("uv-test", dtype=dtype, perturb=0.05, n_layers=1, attn_gate_channels=128, **over)
        assert eng.fuse_qkv
        hdiff, agree, cmax, cfrac, sfrac = _fused_vs_unfused(cfg, eng, steps=12, lens=lens, max_len=max_len)
        assert cmax.max() == 0 and sfrac.max() == 0
        ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
        assert max(hdiff) <= 4 * 2 * ulp, max(hdiff)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_qkv_on_an_unquantized_cache(dtype):
    """kv_dtype="fp16" (K/V cached in the activation type): the fused launch appends the token's k and v as they are.  One
    layer: the appended cache words equal the separate post-processing kernel's bit for bit - ring layer with rotation and
    value embedding through wrap-around, and a global layer; 1, 2 and 4 waves per row - and the layer output agrees to a
    few units in the last place (the own key's score is an fp32 dot product here and an MFMA column there).  Whole models:
    layer 0's words stay identical and the final hidden states within the bound of the int8 tests."""
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    for over, lens, max_len in ((dict(window=32, global_every=0, ve_every=1), (5, 40, 17, 33, 1, 26), 96),
                                (dict(window=0, global_every=1, ve_every=0), (5, 40, 17, 33, 1, 26), 96),
                                (dict(window=128, global_every=0, ve_every=1), (100, 130, 90, 150, 129, 64), 192),
                                (dict(window=0, global_every=1, ve_every=0), (300, 20, 260, 330, 1, 300), 1056)):
        cfg, params, eng, _ = _setup("uv-test", dtype=dtype, perturb=0.05, n_layers=1, attn_gate_channels=128, **over)
        assert eng.fuse_qkv
        from ultraviolet_amd.engine import KVState
        assert eng.fused_layer_ok(0, KVState(cfg, 2, max_len, DEV, kv_dtype="fp16", dtype=dtype))
        hdiff, agree, cmax, cfrac, sfrac = _fused_vs_unfused(cfg, eng, steps=16, lens=lens, max_len=max_len, kv_dtype="fp16")
        assert cmax.max() == 0, cmax
        assert max(hdiff) <= 4 * 2 * ulp, max(hdiff)
    for name, over in (("uv-test", dict(window=32)), ("uv-50m-alpha", dict())):
        cfg, params, eng, _ = _setup(name, dtype=dtype, perturb=0.05, **over)
        hdiff, agree, cmax, cfrac, sfrac = _fused_vs_unfused(cfg, eng, steps=24, kv_dtype="fp16")
        assert cmax[0] == 0
        assert max(hdiff) < 16 * 2 * ulp, max(hdiff)
        _check_agreement(agree, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_unquantized_kv_engine_matches_dense_forward(dtype):
    """kv_dtype="fp16" (KernelDecodeState's unquantized layout, fast_decode.py:21-57: K/V cached in the compute dtype):
    prefill + teacher-forced decode steps over the cache must give the logits of the dense causal forward of the whole
    sequence (the oracle's trunk in the same 16-bit arithmetic) to the bar of the 16-bit engine tests, on global and ring
    layers through ring wrap-around - and must sit closer to it than the int8-KV engine does."""
    from ultraviolet_amd.engine import KVState
    cfg, params, eng, OracleModel = _setup("uv-test", dtype=dtype, perturb=0.06, window=32)
    m = OracleModel(cfg, params, dtype=dtype)
    rng = np.random.default_rng(4)
    L0, steps, B = 20, 40, 4                        # equal prompt lengths: the dense forward needs no padding
    seqs = rng.integers(1, cfg.vocab_size, size=(B, L0 + steps))
    hid, _ = m.trunk(torch.as_tensor(seqs))
    ref = m.logits(hid).float().numpy()[:, L0 - 1:-1]          # logits that predict positions L0 .. L0 + steps - 1
    errs = {}
    for kv in ("fp16", "int8"):
        st = KVState(cfg, B, 96, DEV, kv_dtype=kv, dtype=dtype)
        assert (st.k[0].dtype == dtype) == (kv == "fp16") and (st.k_scale[0] is None) == (kv == "fp16")
        outs = [eng.logits(eng.prefill([s[:L0].tolist() for s in seqs], list(range(B)), st)).cpu()]
        for t in range(steps - 1):
            outs.append(eng.logits(eng.decode_step(torch.as_tensor(seqs[:, L0 + t]).to(DEV), st)).cpu())
        got = torch.stack(outs, 1).float().numpy()
        errs[kv] = np.abs(got - ref)
        assert (got.argmax(-1) == ref.argmax(-1)).mean() > 0.9
    assert errs["fp16"].max() < 0.25, errs["fp16"].max()
    assert errs["fp16"].mean() <= errs["int8"].mean() * 1.05, (errs["fp16"].mean(), errs["int8"].mean())


def test_unquantized_kv_rollout_and_patch_model_state():
    """The continuous-batching driver and the patch_model binding accept the unquantized layout: a greedy rollout over it
    equals static greedy generation over it, request by request."""
    from ultraviolet_amd.engine.rollout import Rollout
    from ultraviolet_amd.kernels import fast_decode as fd
    cfg, params, eng, _ = _setup("uv-test", dtype=torch.bfloat16, perturb=0.06, window=32)
    prompts = _prompts(cfg, (9, 30, 4, 17, 25, 12), seed=2)
    toks = eng.generate(prompts, 20, temperature=0.0, kv_dtype="fp16")
    g = Rollout(eng, slots=4, max_prompt=32, max_new=20, temperature=0.0, eos_id=None, check_every=4, bucket=4, kv_dtype="fp16")
    for i, p in enumerate(prompts):
        g.add(p, i, limit=20)
    got = {m: row for m, row, _, _ in g.run(max_chunks=500)}
    same = sum(got[i] == toks[i] for i in range(len(prompts)))
    assert all(got[i][0] == toks[i][0] for i in range(len(prompts))) and same >= len(prompts) - 1, same   # (a near-tie in the
    # top-2 logits may flip under another GEMM batch shape)
    st = fd.KernelDecodeState(cfg, 3, 64, torch.bfloat16, DEV, kv_dtype="fp16")
    assert st.k[0].dtype == torch.bfloat16 and st.k_scale[0] is None and fd.kv_bytes_per_seq(cfg, 100, "fp16") > fd.kv_bytes_per_seq(cfg, 100)


@pytest.mark.parametrize("n_kv_heads", [2, 4])
def test_fused_qkv_single_layer_is_exact_with_grouped_kv_heads(n_kv_heads):
    """Several KV heads (query groups of 4 and 2 heads per KV head): every KV head's own key / value row, gate logits and
    value-embedding row are taken from the right columns of the extended projection - identical bytes again."""
    for over in (dict(window=32, global_every=0, ve_every=1), dict(window=0, global_every=1, ve_every=0)):
        cfg, params, eng, _ = _setup("uv-test", dtype=torch.bfloat16, perturb=0.05, n_layers=1, attn_gate_channels=128,
                                     n_kv_heads=n_kv_heads, **over)
        assert eng.fuse_qkv and cfg.n_heads // cfg.n_kv_heads == 8 // n_kv_heads
        hdiff, agree, cmax, cfrac, sfrac = _fused_vs_unfused(cfg, eng, steps=40)
        assert cmax.max() == 0 and sfrac.max() == 0
        assert max(hdiff) <= 4 * 2 * 2.0 ** -7, max(hdiff)


def test_int8_check_gate_on_lively_weights():
    """The reference's end-to-end gate of the int8 cache (scripts/eval_math.py:326-350: teacher-forced decode with the
    unquantized and the int8 cache, NLL / top-1 / KL) runs on the engine; on seeded random weights of the full UV-50M preset
    the two caches agree closely (the published bar, +0.002 % NLL and 99.7 % top-1, is for the trained model)."""
    from ultraviolet_amd.engine import int8_check
    cfg, params, eng, _ = _setup("uv-50m-alpha", dtype=torch.bfloat16, perturb=0.05)
    x = torch.from_numpy(np.random.default_rng(3).integers(1, cfg.vocab_size, size=(6, 48))).to(DEV)
    r = int8_check(eng, x)
    assert r["tokens"] == 6 * 47 and np.isfinite(r["nll_unquantized"]) and np.isfinite(r["nll_kernel_int8"])
    assert abs(r["rel_change"]) < 2e-3, r
    assert r["top1_agree"] > 0.9 and 0 <= r["kl"] < 1e-2, r


def test_prefill_packed_host_equals_prefill_fast():
    """prefill_packed_host(model, prompts, rows, st, dev) (fast_decode.py:210-269) against prefill(idx, starts, st, rows) on the
    left-padded batch: identical logits, cache bytes, scales, pos, starts and host_pos (the reference's own claim for the
    pair, tests/test_perf_fz.py:198-236)."""
    from ultraviolet_amd.kernels import fast_decode as fd
    cfg, params, eng, _ = _setup(window=32)
    m = fd.patch_model(_StubModel(cfg, params), kv_dtype="int8", dtype=torch.bfloat16, max_tokens=512)
    prompts = _prompts(cfg, (7, 19, 12, 1), seed=8)
    rows = [3, 0, 2, 5]
    T = max(len(p) for p in prompts)
    idx = torch.zeros(len(prompts), T, dtype=torch.long)
    starts = torch.tensor([T - len(p) for p in prompts])
    for b, p in enumerate(prompts):
        idx[b, T - len(p):] = torch.as_tensor(p)
    s1, s2 = m.new_state(6, 48), m.new_state(6, 48)
    l1 = m.prefill(idx.to(DEV), starts.to(DEV), s1, rows=torch.tensor(rows, device=DEV))
    l2 = fd.prefill_packed_host(m, prompts, rows, s2, DEV)
    assert torch.equal(l1, l2)
    assert torch.equal(s1.pos, s2.pos) and torch.equal(s1.starts, s2.starts) and np.array_equal(s1.host_pos, s2.host_pos)
    for l in range(cfg.n_layers):
        for a, b_ in ((s1.k[l], s2.k[l]), (s1.v[l], s2.v[l]), (s1.k_scale[l], s2.k_scale[l]), (s1.v_scale[l], s2.v_scale[l])):
            assert torch.equal(a, b_)


def test_patched_model_follows_in_place_parameter_updates():
    """The reference's patched methods read the model's live weights; here the engine keeps fused device copies, refreshed
    by the patched methods themselves when a parameter was written in place (same device addresses afterwards)."""
    from ultraviolet_amd.kernels import fast_decode as fd
    cfg, params, eng, _ = _setup(window=32)
    m = fd.patch_model(_StubModel(cfg, params), kv_dtype="int8", dtype=torch.float32, max_tokens=256)
    st = m.new_state(2, 48)
    idx = torch.tensor([[5, 6, 7, 8], [9, 10, 11, 12]], device=DEV)
    l0 = m.prefill(idx, torch.zeros(2, dtype=torch.long, device=DEV), st)
    ptr = m._uvmi_engine.w.layers[0]["wqkv"].data_ptr()
    m._sd["blocks.0.attn.wv"].mul_(1.05)                       # an optimizer step / sync_weights_inplace writes like this
    #                                                            (wv: QK-norm makes a uniform scaling of wq or wk invisible)
    st2 = m.new_state(2, 48)
    l1 = m.prefill(idx, torch.zeros(2, dtype=torch.long, device=DEV), st2)
    assert m._uvmi_engine.w.layers[0]["wqkv"].data_ptr() == ptr and not torch.allclose(l0, l1)
    cfg2, params2, eng2, _ = _setup(window=32)
    params2["blocks.0.attn.wv"] = params2["blocks.0.attn.wv"] * np.float32(1.05)
    from ultraviolet_amd.engine import KVState, UVEngine, UVWeights
    e3 = UVEngine(UVWeights(cfg2, params2, torch.float32, DEV), max_tokens=256)
    ref = e3.logits(e3.prefill([[5, 6, 7, 8], [9, 10, 11, 12]], [0, 1], KVState(cfg2, 2, 48, DEV)))
    torch.testing.assert_close(l1, ref, atol=1e-5, rtol=1e-5)


def test_streamgen_adapter_runs_the_reference_loop():
    """perf.make_streamgen(StreamGen, flags)(model, slots, max_prompt, max_new, T, eos) as rl_grpo.stream_loop builds it
    (scripts/rl_grpo.py:1091-1105): every request comes back once as (meta, tokens, logp, start_version), rows are
    EOS-terminated or max_new long (tests/test_rl_stream.py:82-94), in-place weight updates between chunks are picked up."""
    from ultraviolet_amd import perf
    cfg, params, eng, _ = _setup(dtype=torch.bfloat16, window=32)
    model = _StubModel(cfg, params)
    Gen = perf.make_streamgen(perf.StreamGen, ["lp", "hv", "rfh", "fz"])
    g = Gen(model, 4, 24, 12, 1.0, 0, check_every=4, dtype=torch.bfloat16, row_bucket=4)
    assert perf.install_fz(g) is True
    prompts = _prompts(cfg, (9, 20, 4, 17, 12, 6, 3), seed=2)
    for i, p in enumerate(prompts):
        g.add(p, i)
    res = []
    raw = _StubModel(cfg, params)                              # the trainer's policy
    for it in range(200):
        if g.n_outstanding() == 0:
            break
        res += g.chunk()
        if it == 1:                                            # an optimizer step, then the reference's two lines (rl_grpo.py:1308-1309)
            raw._sd["blocks.0.attn.wq"].mul_(1.01)
            perf.sync_weights_inplace(model, raw)
            g.version += 1
        if it == 3:                                            # a write straight into the generation model: picked up, not counted
            model._sd["blocks.0.attn.wk"].mul_(1.01)
    res += g.harvest_end() if g.harvest_pending else []
    assert sorted(m for m, *_ in res) == list(range(len(prompts)))
    for meta, row, lp, v0 in res:
        assert len(row) == len(lp) and (row[-1] == 0 or len(row) == 12) and 0 not in row[:-1]
        assert np.isfinite(lp).all() and (lp <= 1e-6).all() and v0 in (0, 1)
    assert g.version == 1
    torch.testing.assert_close(model._sd["blocks.0.attn.wq"], raw._sd["blocks.0.attn.wq"])


def test_reference_op_name_runs_the_hip_kernels():
    """torch.ops.mathk.decode_attn (the reference's registered op, decode_attn.py:174-190) with its argument list."""
    from util import attn_case
    from ultraviolet_amd.kernels import decode_attention
    q, k, v, ks, vs = (t.to(DEV) for t in attn_case(9, 1, 8, 64, 256, True, seed=3, dtype=torch.bfloat16))
    pos = torch.randint(0, 256, (9,), device=DEV)
    starts = torch.zeros(9, dtype=torch.long, device=DEV)
    a = torch.ops.mathk.decode_attn(q, k, v, pos, starts, 0.14125, 0, False, ks, vs, 2, 16, 1, "auto")
    b_ = decode_attention(q, k, v, pos, starts, 0.14125, k_scale=ks, v_scale=vs, num_splits=2)
    assert torch.equal(a, b_)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_uncompressed_decode_state_entry_points(dtype):
    """The reference's SDPA-path entry points (MathLM.new_state -> DecodeState, prefill, decode_step with decode_impl "sdpa":
    ultraviolet/model.py:861-1008, 1042-1072) bound by patch_model(kv_dtype=None): the state carries the reference's fields,
    and prefill + decode over it give the logits of the dense causal forward of the whole sequence (the oracle's trunk in
    the same 16-bit arithmetic) - the invariant the reference pins for this path (tests/test_math_model.py:73-85) - through
    ring wrap-around, for left-padded rows as well."""
    from ultraviolet_amd.kernels import fast_decode as fd
    cfg, params, eng, OracleModel = _setup("uv-test", dtype=dtype, perturb=0.06, window=32)
    m = fd.patch_model(_StubModel(cfg, params), kv_dtype=None, dtype=dtype, max_tokens=512)
    B, L0, steps = 4, 20, 40
    st = m.new_state(B, 96)
    assert isinstance(st, fd.DecodeState) and st.kv_dtype is None and st.k[0].dtype == dtype and st.k[0].shape == (B, 1, 32, 64)
    assert st.k[cfg.n_layers - 1].shape[2] == 96 and st.local_len == 32 and st.pos.dtype == torch.long and st.host_pos.shape == (B,)
    assert st.nbytes() == sum(t.numel() * 2 for t in st.k + st.v)
    seqs = np.random.default_rng(4).integers(1, cfg.vocab_size, size=(B, L0 + steps))
    om = OracleModel(cfg, params, dtype=dtype)
    hid, _ = om.trunk(torch.as_tensor(seqs))
    ref = om.logits(hid).float().numpy()[:, L0 - 1:-1]
    outs = [m.prefill(torch.as_tensor(seqs[:, :L0]).to(DEV), torch.zeros(B, dtype=torch.long, device=DEV), st).cpu()]
    for t in range(steps - 1):
        outs.append(m.decode_step(torch.as_tensor(seqs[:, L0 + t]).to(DEV), st, 96).cpu())
    got = torch.stack(outs, 1).float().numpy()
    assert st.pos.tolist() == [L0 + steps - 1] * B and st.host_pos.tolist() == [L0 + steps - 1] * B
    d = np.abs(got - ref)
    assert d.max() < (0.15 if dtype == torch.bfloat16 else 0.04) and (got.argmax(-1) == ref.argmax(-1)).mean() > 0.97, d.max()
    # a left-padded refill of two rows (rows=...) leaves the other rows' caches and positions alone
    st.set_pos(7)
    assert st.pos.tolist() == [7] * B and st.host_pos.tolist() == [7] * B
    k_before = st.k[0][[0, 3]].clone()
    idx = torch.zeros(2, 9, dtype=torch.long)
    idx[0, 4:], idx[1, :] = torch.as_tensor(seqs[0, :5]), torch.as_tensor(seqs[1, :9])
    lg = m.prefill(idx.to(DEV), torch.tensor([4, 0], device=DEV), st, rows=torch.tensor([1, 2], device=DEV))
    assert st.pos.tolist() == [7, 9, 9, 7] and st.starts.tolist() == [0, 4, 0, 0] and torch.equal(st.k[0][[0, 3]], k_before)
    hid2, _ = om.trunk(torch.as_tensor(seqs[:2, :9]))
    ref2 = om.logits(hid2).float().numpy()
    assert np.abs(lg.float().cpu().numpy()[0] - ref2[0, 4]).max() < (0.15 if dtype == torch.bfloat16 else 0.04)   # 5 real tokens
    assert np.abs(lg.float().cpu().numpy()[1] - ref2[1, 8]).max() < (0.15 if dtype == torch.bfloat16 else 0.04)


def test_bf16_engine_greedy_against_the_bf16_oracle_reports_every_divergence():
    """The benchmarked configuration - UV-50M, bf16 activations, int8 KV - on the first configuration's shape (8 prompts of
    32..128 tokens, 64 greedy tokens) against the oracle run in the same 16-bit arithmetic.  bf16 logits of magnitude ~18
    sit on a grid of 2^-4 and the two implementations sum in different orders, so streams separate where the oracle's own
    top two logits are within that noise; the test prints, per row, the first step at which the stream leaves the oracle's
    and the oracle's top-2 gap there, and requires that no row leaves at a gap above the noise between the two paths'
    logits - 0.15, the bar test_16bit_engine_close_to_oracle holds their teacher-forced logits to (measured: 0.07; the
    reference's own bar for int8-vs-reference logits is 0.25, tests/test_math_kernels.py:170-172)."""
    cfg, params, eng, OracleModel = _setup("uv-50m-alpha", dtype=torch.bfloat16, perturb=0.06)
    rng = np.random.default_rng(0)
    lens = rng.integers(32, 129, size=8)
    prompts = [rng.integers(1, cfg.vocab_size, size=int(n)).tolist() for n in lens]
    out = np.array(eng.generate(prompts, 64, temperature=0.0))
    ref, lgs, _ = OracleModel(cfg, params, torch.bfloat16).generate_greedy(prompts, 64, return_logits=True)
    first, gaps = [], []
    for b in range(len(prompts)):
        d = np.nonzero(out[b] != ref[b])[0]
        t = int(d[0]) if len(d) else 64
        first.append(t)
        if t < 64:
            top2 = np.sort(lgs[b, t])[-2:]
            gaps.append(float(top2[1] - top2[0]))
            print(f"row {b}: identical for {t} steps, then the oracle's top-2 gap is {gaps[-1]:.3f}")
        else:
            print(f"row {b}: identical for all 64 steps")
    assert all(g_ < 0.15 for g_ in gaps), gaps
    assert (ref[:, 0] == out[:, 0]).sum() >= 6  # (the first token comes from the prefill alone: most rows agree on it)
