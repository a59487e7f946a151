"""SmolVLA backend on the GPU against the CPU oracle: model-level parity per tier, engine API,
hipGraph replay == eager, camera-count graph keys."""

import os
import sys

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

import cases  # noqa: E402
from oracle import smolvla as O  # noqa: E402

pytestmark = pytest.mark.gpu


def _oracle_chunk(cfg, sd, inp, llm_fp8: bool, exp_fp8: bool):
    shape = O.SmolVLAShape(num_vlm_layers=cfg.num_vlm_layers, vis_layers=cfg.vlm_config.vision_config.num_hidden_layers, num_steps=cfg.num_steps)
    w = O.Weights(sd, O.fp8_linear_names(shape, llm_fp8, exp_fp8))
    with torch.no_grad():
        return O.sample_actions(w, shape, O.prepare_images(inp["images"]), inp["img_masks"], inp["lang_tokens"], inp["lang_masks"], inp["state"], inp["noise"])


def _gpu_chunk(cfg, sd, inp, **tiers):
    from tybok_amd.policies.smolvla.model import SmolVLAModel

    model = SmolVLAModel(cfg, sd, "cuda", **tiers)
    dev = lambda t: t.cuda()  # noqa: E731
    with torch.inference_mode():
        out = model.sample_actions(
            [dev(i * 2.0 - 1.0) for i in inp["images"]], [dev(m) for m in inp["img_masks"]], dev(inp["lang_tokens"]),
            dev(inp["lang_masks"]), dev(inp["state"]), dev(inp["noise"]),
        )  # fmt: skip
    torch.cuda.synchronize()
    return out.cpu()


TIERS = [
    dict(fused_expert=False, fp8_expert_mlp=False, fp8_llm_mlp=False),  # plain torch on the GPU
    dict(fused_expert=True, fp8_expert_mlp=False, fp8_llm_mlp=False),   # HIP attention
    dict(fused_expert=False, fp8_expert_mlp=True, fp8_llm_mlp=False),   # HIP fp8 expert FFN
    dict(fused_expert=True, fp8_expert_mlp=True, fp8_llm_mlp=True),     # the full fp8 path
    dict(fused_expert=False, fp8_expert_mlp=False, fp8_llm_mlp=False, fused_prefill=True),  # HIP prefill only
    dict(fused_expert=True, fp8_expert_mlp=True, fp8_llm_mlp=True, fused_prefill=True),     # all text tiers
    dict(fused_expert=False, fp8_expert_mlp=False, fp8_llm_mlp=False, fused_vit=True),      # HIP vision attention only
    dict(fused_expert=True, fp8_expert_mlp=True, fp8_llm_mlp=True, fused_prefill=True, fused_vit=True),  # everything
]


@pytest.mark.parametrize("tiers", TIERS, ids=["eager", "attn", "fp8ffn", "full", "prefill", "full+prefill", "vit", "all"])
def test_small_model_chunk_matches_oracle(tiers):
    cfg, sd, inp = cases.smolvla_build(cases.SMOLVLA_CASES["small"])
    want = _oracle_chunk(cfg, sd, inp, tiers["fp8_llm_mlp"], tiers["fp8_expert_mlp"])
    got = _gpu_chunk(cfg, sd, inp, **tiers)
    err = float((got - want).abs().max())
    print(f"small {tiers}: max|err| = {err:.4g}, |chunk|max = {float(want.abs().max()):.3g}")
    assert torch.isfinite(got).all()
    # random noise drives |chunk| up to ~4: the 1e-2 bound of the zero-noise case scales with it
    assert err <= 1e-2 * max(1.0, float(want.abs().max()))


def _chunk_errors(got: torch.Tensor, want: torch.Tensor, action_dim: int) -> tuple[float, float, float]:
    """(max over the action chunk the engine returns, max over all padded dims, mean over all)."""
    diff = (got - want).abs()
    return float(diff[..., :action_dim].max()), float(diff.max()), float(diff.mean())


FP8 = dict(fused_expert=True, fp8_expert_mlp=True, fp8_llm_mlp=True)
NORTH_STAR = dict(FP8)  # fp8 GEMM / FFN + expert attention
BENCHED = dict(FP8, fused_prefill=True, fused_vit=True)  # every tier: the set the benchmark times


def _oracle_pair(cfg, sd, inp):
    """The oracle with the reference's dtypes, the same weights with every activation kept in fp32, and the
    reference's dtypes again with every linear summing in another order (two such runs)."""
    shape = O.SmolVLAShape(num_vlm_layers=cfg.num_vlm_layers, vis_layers=cfg.vlm_config.vision_config.num_hidden_layers, num_steps=cfg.num_steps)
    out = []
    for kw in (dict(act_dtype=torch.bfloat16), dict(act_dtype=torch.float32), dict(k_order_seed=1), dict(k_order_seed=2)):
        w = O.Weights(sd, O.fp8_linear_names(shape, True, True), **kw)
        with torch.no_grad():
            out.append(O.sample_actions(w, shape, O.prepare_images(inp["images"]), inp["img_masks"], inp["lang_tokens"], inp["lang_masks"], inp["state"], inp["noise"]))
    return out[0], out[1], out[2:]


@pytest.mark.parametrize("cameras", [3, 2])
def test_full_model_zero_noise_chunk_against_oracle_and_noise_floor(cameras):
    # Benchmark config 4 at full depth (16 + 16 layers, 10 steps, zero noise) with 3 and with 2 cameras, three
    # seeded frames each, for the north-star tier set and for the set the benchmark times (every tier).
    #
    # Stated bound: action chunk max-abs <= 1e-2.  What a bf16 execution can hold is measured here, not
    # asserted in a comment: `ref32` is the oracle run on the same weights with every activation in fp32.
    # The reference-dtype (bf16) oracle itself sits 0.85e-2 .. 1.3e-2 (max) / 2.0e-3 .. 2.2e-3 (mean) from
    # it -- rounding flips amplified through 32 layers x 10 steps, re-drawn by any change of summation
    # order (a different split of a k loop over waves, even in the fp32 K/V projection, moves a frame's
    # maximum by +-25 %) -- so no bf16 implementation, the reference's own included, holds 1e-2 on every
    # frame, and two of them that each sit ~1e-2 from ref32 are up to sqrt(2) times that apart.  Held:
    #   * per frame, the HIP path is no farther from ref32 than the bf16 oracle is (x1.15 mean, x1.5 max:
    #     the maximum of 1600 values re-draws by +-25 % between equally good executions);
    #   * per frame, the HIP path is no farther from the bf16 oracle than x1.5 (max) / x1.15 (mean) of what
    #     the oracle's own arithmetic in another summation order is (two re-ordered runs of every linear:
    #     0.8e-2 .. 1.1e-2 max, 2.0e-3 .. 2.2e-3 mean);
    #   * per frame, against the bf16 oracle: the chunk the engine returns (first 6 of the 32 padded
    #     outputs) <= 1.25e-2, all 32 outputs <= 1.5e-2, mean <= 3e-3;
    #   * over the three frames, so that one rounding flip does not decide: the median of the returned
    #     chunk's maxima <= 1e-2 (the stated bound) for both camera counts, and the median of the
    #     all-output maxima <= 1e-2 on the benchmark's own configuration (3 cameras), <= 1.25e-2 with 2
    #     cameras (the bf16 oracle's own distance from ref32 reaches 1.27e-2 there).
    maxima = {"north_star": [], "benched": []}
    chunk_maxima = {"north_star": [], "benched": []}
    for seed in (0, 1, 2):
        cfg, sd, inp = cases.smolvla_build(dict(cases.SMOLVLA_CASES["full"], cameras=cameras, seed=seed))
        adim = cfg.action_feature_shape[0]
        want, ref32, reordered = _oracle_pair(cfg, sd, inp)
        _, floor_max, floor_mean = _chunk_errors(want, ref32, adim)
        self_max = max(_chunk_errors(r, want, adim)[1] for r in reordered)
        self_mean = max(_chunk_errors(r, want, adim)[2] for r in reordered)
        for name, tiers in (("north_star", NORTH_STAR), ("benched", BENCHED)):
            got = _gpu_chunk(cfg, sd, inp, **tiers)
            e_act, e_all, e_mean = _chunk_errors(got, want, adim)
            _, d_max, d_mean = _chunk_errors(got, ref32, adim)
            print(
                f"full depth, {cameras} cameras, seed {seed}, {name}: vs bf16 oracle action chunk {e_act:.4g}, all 32 dims {e_all:.4g}, "
                f"mean {e_mean:.4g}; vs fp32-activation run {d_max:.4g} / {d_mean:.4g} (bf16 oracle: {floor_max:.4g} / {floor_mean:.4g}); "
                f"the oracle in another summation order vs itself: {self_max:.4g} / {self_mean:.4g}"
            )
            assert torch.isfinite(got).all()
            assert d_mean <= 1.15 * floor_mean and d_max <= 1.5 * floor_max
            assert e_mean <= 1.15 * self_mean and e_all <= 1.5 * self_max
            assert e_act <= 1.25e-2 and e_all <= 1.5e-2 and e_mean <= 3e-3
            if cameras == 3 and seed == 0:
                # the frame the benchmark times and reports under `parity` (measured 0.92e-2): the stated bound, on this
                # one frame, so that a regression of the benchmarked configuration trips whatever the medians do
                assert e_act <= 1e-2 and (name != "benched" or e_all <= 1e-2)
            maxima[name].append(e_all)
            chunk_maxima[name].append(e_act)
    for name, vals in maxima.items():
        cap = 1e-2 if cameras == 3 else 1.25e-2
        assert sorted(vals)[1] <= cap, f"{name}: median of the per-frame maxima {sorted(vals)} exceeds {cap}"
        assert sorted(chunk_maxima[name])[1] <= 1e-2, f"{name}: median of the returned chunk's maxima {sorted(chunk_maxima[name])} exceeds 1e-2"


def test_full_model_bf16_path_matches_reference_golden():
    # the bf16 (no fp8) GPU path against the reference's own output for the same tensors (config 4, seed 0)
    cfg, sd, inp = cases.smolvla_build(cases.SMOLVLA_CASES["full"])
    adim = cfg.action_feature_shape[0]
    gold = torch.from_numpy(np.load(os.path.join(HERE, "golden", "smolvla_full.npz"))["chunk"])[None]
    got16 = _gpu_chunk(cfg, sd, inp, fused_expert=True, fp8_expert_mlp=False, fp8_llm_mlp=False)
    e_act, e_all, e_mean = _chunk_errors(got16, gold, adim)
    print(f"full bf16 vs reference golden: action chunk max|err| = {e_act:.4g}; all 32 dims max = {e_all:.4g}, mean = {e_mean:.4g}")
    assert e_all <= 1.25e-2 and e_mean <= 3e-3


def test_overlapped_step0_equals_sequential_bit_for_bit():
    # prefill x step-0 overlap on two streams without a graph: same kernels, same inputs, same bits
    cfg, sd, inp = cases.smolvla_build(cases.SMOLVLA_CASES["small"])
    tiers = dict(fused_expert=True, fp8_expert_mlp=True, fp8_llm_mlp=True, fused_prefill=True)
    seq = _gpu_chunk(cfg, sd, inp, **tiers)
    for _ in range(2):
        assert torch.equal(seq, _gpu_chunk(cfg, sd, inp, overlap=True, **tiers))


@pytest.fixture(scope="module")
def ckpt(tmp_path_factory):
    from tybok_amd.policies.synthetic import write_smolvla_checkpoint

    return write_smolvla_checkpoint(str(tmp_path_factory.mktemp("smolvla_ckpt")), cameras=3, seed=5, num_vlm_layers=4, vision_layers=2, num_steps=3)


def test_engine_api_graph_equals_eager_and_camera_keys(ckpt):
    from tybok_amd.registry import create_engine

    flags = dict(tl_fused_expert=True, tl_fp8_expert_mlp=True, tl_fp8_llm_mlp=True, tl_llm_fused_attn=True, tl_vit_oproj=True)
    eager = create_engine(ckpt, device="cuda", graph=False, warmup=False, **flags)
    graph = create_engine(ckpt, device="cuda", graph=True, graph_cameras=(2, 3), warmup=True, seed=3, overlap=True, **flags)
    assert graph.graph_enabled and sorted(graph._graph_runner.keys()) == [(2,), (3,)]
    # graph mode hides step 0 inside the prefill on a second stream; the eager engine is sequential:
    # the comparisons below are therefore also overlapped == sequential, bit for bit
    assert graph.overlap and not eager.overlap
    spec = eager.describe()
    assert spec == {"model_type": "smolvla", "cameras": ["camera1", "camera2", "camera3"], "resize": [512, 512], "action_dim": 6, "chunk_size": 50}
    noise = torch.zeros(1, 50, 6)
    for cams in (3, 2):
        frame = eager._profile_frame(cameras=cams, seed=cams)
        a = eager.predict_action_chunk(frame, noise=noise)
        assert a.shape == (50, 6) and a.dtype == np.float32 and np.isfinite(a).all()
        # several replays interleaved with eager work: every replay equals the eager result bit for bit
        for _ in range(3):
            b = graph.predict_action_chunk(frame, noise=noise)
            assert np.array_equal(a, b)
            assert np.array_equal(a, eager.predict_action_chunk(frame, noise=noise))
    # select_action drains a queue of chunk_size actions before inferring again
    first = graph.select_action(frame, noise=noise)
    assert first.shape == (6,) and np.array_equal(first, b[0])
    assert np.array_equal(graph.select_action(frame, noise=noise), b[1])
    # implicit noise: seeded engine RNG, drawn outside the graph -> two calls differ
    c1 = graph.predict_action_chunk(frame)
    c2 = graph.predict_action_chunk(frame)
    assert not np.array_equal(c1, c2)


def test_graph_requests_with_changing_task_noise_and_host_inputs(ckpt):
    # the graph path caches task tokens / masks and reuses static tensors: alternating tasks, an implicit-noise
    # request between explicit ones, host-resident frames and a queue drained across requests must all give
    # what the eager engine gives
    from tybok_amd.registry import create_engine

    flags = dict(tl_fused_expert=True, tl_fp8_expert_mlp=True, tl_fp8_llm_mlp=True, tl_llm_fused_attn=True, tl_vit_oproj=True)
    eager = create_engine(ckpt, device="cuda", graph=False, warmup=False, **flags)
    graph = create_engine(ckpt, device="cuda", graph=True, graph_cameras=(3,), warmup=True, seed=9, **flags)
    noise = torch.zeros(1, 50, 6)
    frames = []
    for seed, task in ((1, "pick up the cube"), (2, "open the drawer"), (3, "pick up the cube")):
        f = eager._profile_frame(cameras=3, seed=seed)
        f["task"] = task
        frames.append(f)
    want = [eager.predict_action_chunk(f, noise=noise) for f in frames]
    assert not np.array_equal(want[0], want[1])
    for f, w in zip(frames, want):
        assert np.array_equal(graph.predict_action_chunk(f, noise=noise), w)
    graph.predict_action_chunk(frames[0])  # implicit noise fills every padded action column of the static tensor
    assert np.array_equal(graph.predict_action_chunk(frames[1], noise=noise), want[1])
    on_device = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in frames[2].items()}
    assert np.array_equal(graph.predict_action_chunk(on_device, noise=noise.cuda()), want[2])
    # a frame that carries its own token tensors on the device and changes them in place between requests:
    # the replay must see the new ids (such tensors are copied every time, unlike the engine's cached ones)
    ids1, mask1 = (t.clone() for t in graph._task_tokens("open the drawer\n"))
    ids0, _ = graph._task_tokens("pick up the cube\n")
    own = dict(on_device)
    own.pop("task")
    own["observation.language.tokens"], own["observation.language.attention_mask"] = ids1, mask1
    first = graph.predict_action_chunk(own, noise=noise.cuda())
    ids1.copy_(ids0)
    second = graph.predict_action_chunk(own, noise=noise.cuda())
    own_eager = {k: (v.clone() if isinstance(v, torch.Tensor) else v) for k, v in own.items()}
    assert not np.array_equal(first, second) and np.array_equal(second, eager.predict_action_chunk(own_eager, noise=noise.cuda()))
    # select_action keeps the chunk of its first request while other requests replay the graph in between
    first = graph.select_action(frames[0], noise=noise)
    graph.predict_action_chunk(frames[1], noise=noise)
    second = graph.select_action(frames[1], noise=noise)  # still from the queue filled by frames[0]
    assert np.array_equal(first, want[0][0]) and np.array_equal(second, want[0][1])


def test_engine_rejects_flags_it_does_not_implement(ckpt):
    from tybok_amd.registry import create_engine

    with pytest.raises(NotImplementedError):
        create_engine(ckpt, device="cuda", warmup=False, tl_fused_vit=True)
    with pytest.raises(NotImplementedError):
        create_engine(ckpt, device="cuda", warmup=False, compile_model=True)
    with pytest.raises(ValueError):
        create_engine(ckpt, device="cuda", warmup=False, sampler="rk4")


@pytest.mark.parametrize("tiers", [dict(fused_expert=False, fp8_expert_mlp=False, fp8_llm_mlp=False), dict(FP8, fused_prefill=True, fused_vit=True)], ids=["eager", "all"])
def test_heun_sampler_matches_oracle_and_reference_golden(tiers):
    # sampler="heun": two velocity evaluations per step, x <- x + dt/2 (v0 + v1)
    # (tybok/policies/smolvla/models/flow_matching.py:583-644); reduced depth, random noise
    cfg, sd, inp = cases.smolvla_build(cases.SMOLVLA_CASES["small_heun"])
    assert cfg.sampler == "heun"
    shape = O.SmolVLAShape(num_vlm_layers=cfg.num_vlm_layers, vis_layers=cfg.vlm_config.vision_config.num_hidden_layers, num_steps=cfg.num_steps)
    w = O.Weights(sd, O.fp8_linear_names(shape, tiers["fp8_llm_mlp"], tiers["fp8_expert_mlp"]))
    with torch.no_grad():
        want = O.sample_actions(w, shape, O.prepare_images(inp["images"]), inp["img_masks"], inp["lang_tokens"], inp["lang_masks"], inp["state"], inp["noise"], sampler="heun")
    got = _gpu_chunk(cfg, sd, inp, **tiers)
    err = float((got - want).abs().max())
    print(f"heun {sorted(k for k, v in tiers.items() if v)}: max|err| = {err:.4g}, |chunk|max = {float(want.abs().max()):.3g}")
    assert err <= 1e-2 * max(1.0, float(want.abs().max()))
    if not any(tiers.values()):
        gold = torch.from_numpy(np.load(os.path.join(HERE, "golden", "smolvla_small_heun.npz"))["chunk"])[None]
        assert float((got - gold).abs().max()) <= 1e-2 * max(1.0, float(gold.abs().max()))


def test_engine_heun_graph_equals_eager(ckpt):
    from tybok_amd.registry import create_engine

    flags = dict(tl_fused_expert=True, tl_fp8_expert_mlp=True, tl_fp8_llm_mlp=True, tl_llm_fused_attn=True, tl_vit_oproj=True)
    eager = create_engine(ckpt, device="cuda", graph=False, warmup=False, sampler="heun", **flags)
    graph = create_engine(ckpt, device="cuda", graph=True, graph_cameras=(3,), warmup=True, sampler="heun", overlap=True, **flags)
    euler = create_engine(ckpt, device="cuda", graph=False, warmup=False, **flags)
    assert not graph.overlap  # Heun keeps the sequential path
    frame = eager._profile_frame(cameras=3, seed=4)
    noise = torch.zeros(1, 50, 6)
    a = eager.predict_action_chunk(frame, noise=noise)
    for _ in range(2):
        assert np.array_equal(a, graph.predict_action_chunk(frame, noise=noise))
    assert not np.array_equal(a, euler.predict_action_chunk(frame, noise=noise))


def test_validate_against_an_oracle_dump(ckpt, tmp_path):
    # `engine.validate(reference_dir)` (smolvla/engine.py:655-752): the dump directory is written here by
    # the CPU oracle -- frame, preprocessed batch, prefix embedding, per-layer prefix K/V, one velocity
    # evaluation at t = 0.5, the zero-noise chunk -- and every component must agree.
    from tybok_amd.policies.smolvla.weights import random_state_dict
    from tybok_amd.registry import create_engine

    flags = dict(tl_fused_expert=True, tl_fp8_expert_mlp=True, tl_fp8_llm_mlp=True, tl_llm_fused_attn=True, tl_vit_oproj=True)
    eng = create_engine(ckpt, device="cuda", graph=True, graph_cameras=(3,), warmup=True, **flags)
    cfg = eng.config
    frame = eng._profile_frame(cameras=3, seed=11)
    with torch.inference_mode():
        batch = {k: v.cpu() for k, v in eng._batch_from_frame(frame).items() if isinstance(v, torch.Tensor)}
        images01 = [batch[k] for k in cfg.image_features]
        state = eng.prepare_state(batch)
    shape = O.SmolVLAShape(num_vlm_layers=cfg.num_vlm_layers, vis_layers=cfg.vlm_config.vision_config.num_hidden_layers, num_steps=cfg.num_steps)
    w = O.Weights(random_state_dict(cfg, seed=5), O.fp8_linear_names(shape, True, True))
    tokens, lang_masks = batch["observation.language.tokens"], batch["observation.language.attention_mask"]
    masks = [torch.ones(1, dtype=torch.bool)] * 3
    with torch.no_grad():
        images = O.prepare_images(images01)
        embs, pads, att = O.embed_prefix(w, shape, images, masks, tokens, lang_masks, state)
        kv = O.prefill(w, shape, embs, pads, att)
        v_t = O.denoise_step(w, shape, pads, kv, O.expert_prefix_kv(w, shape, kv), torch.zeros(1, 50, 32), 0.5)
        chunk = O.sample_actions(w, shape, images, masks, tokens, lang_masks, state, torch.zeros(1, 50, 32))[:, :, :6]
    post = eng.unnormalizer.unnormalize(chunk.cuda(), "action", "ACTION").cpu()
    d = str(tmp_path)
    torch.save({k: (v.cpu() if isinstance(v, torch.Tensor) else v) for k, v in frame.items()}, os.path.join(d, "frame.pt"))
    torch.save(batch, os.path.join(d, "batch.pt"))
    torch.save({"embs": embs, "pad_masks": pads, "att_masks": att}, os.path.join(d, "prefix.pt"))
    torch.save({f"layer{i}": {"keys": k, "values": v} for i, (k, v) in enumerate(kv)}, os.path.join(d, "prefix_kv.pt"))
    torch.save({"v_t": v_t}, os.path.join(d, "denoise.pt"))
    torch.save({"chunk": chunk, "chunk_post": post}, os.path.join(d, "chunk.pt"))
    errors = eng.validate(d)
    worst = {k: v for k, v in errors.items() if k.endswith(".max")}
    print("validate:", {k: round(v, 5) for k, v in sorted(worst.items(), key=lambda kv: -kv[1])[:6]})
    assert {"prefix.embs.max", "prefix_kv.layer0.keys.max", "denoise.v_t.max", "chunk.max", "chunk_post.max"} <= set(errors)
    assert errors["prefix.pad_masks.max"] == 0 and errors["prefix.att_masks.max"] == 0
    assert all(v == 0 for k, v in errors.items() if k.startswith("batch.") and k.endswith(".max"))
    assert errors["prefix.embs.max"] <= 2e-2 * max(1.0, float(embs.abs().max()))
    assert max(v for k, v in worst.items() if k.startswith("prefix_kv.")) <= 5e-2 * max(1.0, max(float(k.abs().max()) for k, _ in kv))
    # one velocity evaluation carries the per-step bf16 noise undamped (the chunk integrates ten of them with
    # dt = 0.1).  This frame's chunk error moves between 0.009 and 0.013 whenever a bf16 rounding point anywhere
    # upstream changes by one step; the 1e-2 bound on the returned chunk is held by the full-model test on its
    # own frame, here the report only has to be of that size
    assert errors["denoise.v_t.max"] <= 5e-2 * max(1.0, float(v_t.abs().max())) and errors["chunk.max"] <= 1.5e-2
    with pytest.raises(FileNotFoundError):
        eng.validate(os.path.join(d, "nowhere"))
