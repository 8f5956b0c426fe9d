"""Tiny configurations and model folders shared by the tests.

The two configurations differ in every size and option: layers, width, heads and their grouping,
head size, feed-forward width, vocabulary (neither a power of two in B), rope base, llama3 scaling
or none, tied or untied head, the norms' eps, and the dtype their weights are stored in.
"""

from __future__ import annotations

import random

import torch

from tinyserve_llm_amd.config import LlamaConfig, RopeScaling
from tinyserve_llm_amd.weights.random_init import write_random_model

TINY_A = LlamaConfig(
    vocab_size=256, hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
    num_key_value_heads=2, head_dim=16, max_position_embeddings=192, rms_norm_eps=1e-5, rope_theta=10000.0,
    rope_scaling=None, tie_word_embeddings=True, eos_token_id=255)

TINY_B = LlamaConfig(
    vocab_size=384, hidden_size=96, intermediate_size=160, num_hidden_layers=3, num_attention_heads=3,
    num_key_value_heads=1, head_dim=32, max_position_embeddings=320, rms_norm_eps=1e-6, rope_theta=500000.0,
    rope_scaling=RopeScaling(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                             original_max_position_embeddings=64),
    tie_word_embeddings=False, eos_token_id=383)

CONFIGS = {"A": (TINY_A, 0, torch.float32), "B": (TINY_B, 1, torch.bfloat16)}


def make_folder(tmp_path_factory, name: str) -> str:
    config, seed, stored = CONFIGS[name]
    folder = tmp_path_factory.mktemp(f"tiny_{name}")
    write_random_model(str(folder), config, seed, stored)
    return str(folder)


def prompt(seed: int, length: int, vocab: int) -> list[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(length)]


def rugezen_configs():
    """Two small Rugezen configurations that differ from each other in every size and option: key/value
    grouping, key and value head sizes (equal or not), how much of a head turns, caps, layer order, a
    looped stretch (three passes over two layers, or none), a layer without feed-forward, eps, the
    residual multiplier, and widths that are no multiples of 64."""
    from tinyserve_llm_amd.config.rugezen import RugezenAttention, RugezenConfig, RugezenLayer, RugezenMinGRU
    att_p = RugezenAttention(heads=4, kv_heads=2, dim=32, vdim=48, rot_dims=16, rot_base=10000.0, scale=0.31, softcap=3.0)
    att_q = RugezenAttention(heads=2, kv_heads=2, dim=16, vdim=16, rot_dims=16, rot_base=700.0, scale=0.25, softcap=30.0)
    att_r = RugezenAttention(heads=6, kv_heads=1, dim=24, vdim=8, rot_dims=4, rot_base=50000.0, scale=0.2, softcap=1.5)
    att_s = RugezenAttention(heads=4, kv_heads=2, dim=64, vdim=64, rot_dims=32, rot_base=1000.0, scale=0.15, softcap=2.5)
    P = RugezenConfig(vocab=200, width=80, norm_eps=1e-6, residual_mult=0.37, loop_start=0, loop_stop=2, loop_times=3,
                      layers=(RugezenLayer("mingru", RugezenMinGRU(width=72), 96), RugezenLayer("attention", att_p, 144),
                              RugezenLayer("attention", att_r, None)))
    Q = RugezenConfig(vocab=131, width=48, norm_eps=1e-4, residual_mult=1.0,
                      layers=(RugezenLayer("attention", att_q, 64), RugezenLayer("mingru", RugezenMinGRU(width=100), None),
                              RugezenLayer("mingru", RugezenMinGRU(width=16), 40), RugezenLayer("attention", att_s, 56)))
    # sizes that are multiples of nothing in particular: no kernel's fast path takes them
    att_t = RugezenAttention(heads=3, kv_heads=1, dim=20, vdim=12, rot_dims=6, rot_base=100.0, scale=0.3, softcap=5.0)
    R = RugezenConfig(vocab=77, width=99, norm_eps=1e-5, residual_mult=0.8, loop_start=1, loop_stop=2, loop_times=2,
                      layers=(RugezenLayer("attention", att_t, 52), RugezenLayer("mingru", RugezenMinGRU(width=35), 44)))
    # a width that the weight-streaming kernels take (steps of few rows then run the fused forms), heads of a
    # matrix-core size
    att_u = RugezenAttention(heads=8, kv_heads=2, dim=64, vdim=64, rot_dims=64, rot_base=20000.0, scale=0.11, softcap=8.0)
    S = RugezenConfig(vocab=300, width=512, norm_eps=1e-6, residual_mult=0.45, loop_start=0, loop_stop=1, loop_times=2,
                      layers=(RugezenLayer("attention", att_u, 640), RugezenLayer("mingru", RugezenMinGRU(width=256), 768)))
    return {"P": (P, 3), "Q": (Q, 4), "R": (R, 5), "S": (S, 6)}


def fanotar_configs():
    """Small Fanotar configurations that differ from each other in every size and option: key/value
    grouping, key and value head sizes (equal or not), taps of the short convolution (down to one),
    windows (one key, shorter and longer than a page, none), query multipliers that step early or never,
    layers that read another layer's cache through a wider or a narrower window than its owner's, dense,
    routed (with and without a shared expert, one expert per token up to all of them) and absent
    feed-forwards, and widths that are multiples of nothing."""
    from tinyserve_llm_amd.config.fanotar import FanotarAttention as A, FanotarConfig, FanotarExperts as E, \
        FanotarGatedUnit as U, FanotarLayer as L
    a0 = A(heads=4, kv_heads=2, dim=32, vdim=48, conv=3, window=24, scale=0.3, q_temp_coef=0.4, q_temp_every=16)
    a1 = A(heads=4, kv_heads=2, dim=32, vdim=48, conv=2, window=50, scale=0.2, q_temp_coef=0.25, q_temp_every=7, kv_from=0)
    a2 = A(heads=6, kv_heads=1, dim=24, vdim=8, conv=1, window=0, scale=0.35, q_temp_coef=0.0, q_temp_every=1)
    P = FanotarConfig(vocab=200, width=80, norm_eps=1e-6, embedding_scale=7.0, layers=(
        L(a0, U(ff=96, limit=1.5)), L(a1, E(experts=6, top=3, scale=1.7, expert=U(40, 1.0), shared=U(24, 2.0))), L(a2, None)))
    b0 = A(heads=2, kv_heads=2, dim=16, vdim=16, conv=5, window=1, scale=0.25, q_temp_coef=1.0, q_temp_every=3)
    b1 = A(heads=2, kv_heads=2, dim=16, vdim=16, conv=2, window=70, scale=0.4, q_temp_coef=0.3, q_temp_every=100)
    b2 = A(heads=2, kv_heads=2, dim=16, vdim=16, conv=4, window=9, scale=0.4, q_temp_coef=0.3, q_temp_every=100, kv_from=1)
    Q = FanotarConfig(vocab=131, width=48, norm_eps=1e-4, embedding_scale=1.0, layers=(
        L(b0, E(experts=4, top=1, scale=1.0, expert=U(20, 3.0), shared=None)), L(b1, U(64, 0.7)), L(b2, U(40, 2.5)),
        L(b2, E(experts=3, top=3, scale=0.6, expert=U(12, 1.2), shared=U(8, 1.0)))))
    # sizes that are multiples of nothing in particular: no kernel's fast path takes them
    c0 = A(heads=3, kv_heads=1, dim=20, vdim=12, conv=4, window=7, scale=0.3, q_temp_coef=0.5, q_temp_every=2)
    R = FanotarConfig(vocab=77, width=99, norm_eps=1e-5, embedding_scale=3.5, layers=(
        L(c0, E(experts=5, top=2, scale=2.2, expert=U(17, 2.0), shared=U(9, 0.5))), L(c0, U(52, 1.0))))
    # a width that the weight-streaming kernels take, heads of a matrix-core size, experts in tiles of several rows
    d0 = A(heads=8, kv_heads=2, dim=64, vdim=64, conv=4, window=33, scale=0.11, q_temp_coef=0.2, q_temp_every=32)
    d1 = A(heads=8, kv_heads=2, dim=64, vdim=64, conv=4, window=130, scale=0.11, q_temp_coef=0.2, q_temp_every=32, kv_from=0)
    S = FanotarConfig(vocab=300, width=512, norm_eps=1e-6, embedding_scale=12.0, layers=(
        L(d0, E(experts=8, top=2, scale=1.5, expert=U(128, 2.0), shared=U(256, 1.0))), L(d1, U(640, 2.0))))
    return {"P": (P, 3), "Q": (Q, 4), "R": (R, 5), "S": (S, 6)}


def bafarax_configs():
    """Small Bafarax configurations that differ from each other in every size and option: the order of the three
    mixers, key/value grouping, key and value head sizes (equal or not), how much of a head turns (all, part, none),
    frequency ramps or none, chunks and windows (one position, shorter and longer than a page, none), latents larger
    and smaller than the heads they feed, an mLSTM whose values span several workgroups, layers that run with an
    earlier layer's weights, dense, routed (one expert per token up to all of them) and absent feed-forwards, an
    embedding scale of 1, and widths that are multiples of nothing."""
    from tinyserve_llm_amd.config.bafarax import BafaraxAttention as A, BafaraxConfig, BafaraxDense as D, BafaraxExperts as E, \
        BafaraxLatentAttention as LA, BafaraxLayer as L, BafaraxMLSTM as M, FrequencyRamp as Ramp, Rotation as Rot
    p_att = A(heads=4, kv_heads=2, dim=32, vdim=48, scale=0.3, rot=Rot(16, 10000.0), chunk=24)
    p_lat = LA(heads=3, dim=24, rot_dim=8, vdim=20, kv_rank=40, q_rank=36, scale=0.2,
               rot=Rot(8, 5000.0, Ramp(factor=3.0, original=64.0, fast=16.0, slow=2.0)), window=50)
    P = BafaraxConfig(vocab=200, width=80, norm_eps=1e-6, embedding_scale=7.0, layers=(
        L("mlstm", M(heads=3, dim=20, vdim=28, gate_cap=8.0), D(96)), L("attention", p_att, E(experts=6, top=3, ff=40)),
        L("latent_attention", p_lat, None), L("attention", p_att, E(experts=6, top=3, ff=40), weights_of=1)))
    q_att = A(heads=2, kv_heads=2, dim=16, vdim=16, scale=0.25, rot=Rot(16, 700.0), chunk=1)
    q_lat = LA(heads=2, dim=16, rot_dim=16, vdim=16, kv_rank=16, q_rank=16, scale=0.4, rot=Rot(16, 300.0), window=70)
    q_mem = M(heads=1, dim=16, vdim=16, gate_cap=15.0)
    q_full = A(heads=4, kv_heads=1, dim=8, vdim=24, scale=0.35, rot=Rot(0, 1.0), chunk=0)
    Q = BafaraxConfig(vocab=131, width=48, norm_eps=1e-4, embedding_scale=1.0, layers=(
        L("attention", q_att, E(experts=4, top=1, ff=20)), L("latent_attention", q_lat, D(64)), L("mlstm", q_mem, None),
        L("mlstm", q_mem, None, weights_of=2), L("latent_attention", q_lat, D(64), weights_of=1),
        L("attention", q_full, E(experts=3, top=3, ff=12))))
    # sizes that are multiples of nothing in particular: no kernel's fast path takes them
    r_lat = LA(heads=3, dim=20, rot_dim=6, vdim=12, kv_rank=34, q_rank=22, scale=0.3,
               rot=Rot(6, 2000.0, Ramp(factor=8.0, original=32.0, fast=4.0, slow=1.0)), window=7)
    R = BafaraxConfig(vocab=77, width=99, norm_eps=1e-5, embedding_scale=3.5, layers=(
        L("latent_attention", r_lat, E(experts=5, top=2, ff=17)),
        L("attention", A(heads=3, kv_heads=1, dim=20, vdim=12, scale=0.3, rot=Rot(10, 50000.0), chunk=50), D(52)),
        L("mlstm", M(heads=2, dim=18, vdim=270, gate_cap=5.0), D(40))))
    # a width that the weight-streaming kernels take, heads of a matrix-core size, experts in tiles of several rows
    s_att = A(heads=8, kv_heads=2, dim=64, vdim=64, scale=0.11, rot=Rot(32, 250000.0), chunk=33)
    S = BafaraxConfig(vocab=300, width=512, norm_eps=1e-6, embedding_scale=12.0, layers=(
        L("attention", s_att, E(experts=8, top=2, ff=128)),
        L("latent_attention", LA(heads=8, dim=64, rot_dim=32, vdim=64, kv_rank=256, q_rank=192, scale=0.1, rot=Rot(32, 10000.0),
                                 window=130), D(640)),
        L("mlstm", M(heads=4, dim=64, vdim=128, gate_cap=12.0), D(640)), L("attention", s_att, E(experts=8, top=2, ff=128), weights_of=0)))
    return {"P": (P, 3), "Q": (Q, 4), "R": (R, 5), "S": (S, 6)}


def tegolix_configs():
    """Small Tegolix configurations that differ from each other in every size and option: the order of the two kinds of
    mixer, key/value grouping, key and value head sizes (equal or not), how much of a head turns (all, part, none), a
    frequency ramp or none, windows (one position, shorter and longer than a page, none), capped scores or not, the two
    side scales, ranks of the decays' projections, recurrence heads from 4 to more than 256 dimensions, tau of 1, dense,
    routed (no identity expert up to several, one choice up to all, with and without a shared expert) and absent
    feed-forwards, a per-layer token input or none, and widths that are multiples of nothing."""
    from tinyserve_llm_amd.config.bafarax import FrequencyRamp as Ramp, Rotation as Rot
    from tinyserve_llm_amd.config.tegolix import TegolixConfig, TegolixDense as D, TegolixExperts as E, TegolixGLA as G, \
        TegolixLayer as L, TegolixParallel as Par, TegolixRecurrence as R, TegolixWindowAttention as A
    p_par = Par(A(heads=4, kv_heads=2, dim=32, vdim=48, scale=0.4, softcap=6.0, rot=Rot(16, 10000.0, Ramp(3.0, 64.0, 16.0, 2.0)), window=24),
                R(heads=3, dim=20, decay_rank=8), left_scale=0.7, right_scale=1.2)
    P = TegolixConfig(vocab=200, width=80, norm_eps=1e-6, side_dim=12, layers=(
        L("gla", G(heads=3, dim=20, vdim=28, tau=8.0, decay_rank=8), D(96)),
        L("parallel", p_par, E(experts=6, identity=2, top=3, ff=40, shared_ff=56)),
        L("gla", G(heads=2, dim=16, vdim=40, tau=1.0, decay_rank=4), None)))
    q_par = Par(A(heads=2, kv_heads=2, dim=16, vdim=16, scale=0.5, softcap=0.0, rot=Rot(16, 700.0), window=1),
                R(heads=1, dim=16, decay_rank=16), left_scale=1.0, right_scale=1.0)
    q_full = Par(A(heads=4, kv_heads=1, dim=8, vdim=24, scale=0.6, softcap=30.0, rot=Rot(0, 300.0), window=0),
                 R(heads=2, dim=4, decay_rank=3), left_scale=1.5, right_scale=0.4)
    Q = TegolixConfig(vocab=131, width=48, norm_eps=1e-4, side_dim=0, layers=(
        L("parallel", q_par, E(experts=4, identity=0, top=1, ff=20, shared_ff=0)),
        L("gla", G(heads=1, dim=16, vdim=16, tau=4.0, decay_rank=16), D(64)),
        L("parallel", q_full, E(experts=3, identity=3, top=6, ff=12, shared_ff=24)),
        L("gla", G(heads=1, dim=16, vdim=16, tau=4.0, decay_rank=16), None)))
    # sizes that are multiples of nothing in particular: no kernel's fast path takes them
    r_par = Par(A(heads=3, kv_heads=1, dim=20, vdim=12, scale=0.3, softcap=4.0, rot=Rot(10, 50000.0, Ramp(8.0, 32.0, 4.0, 1.0)), window=70),
                R(heads=1, dim=300, decay_rank=5), left_scale=0.5, right_scale=2.0)
    R_ = TegolixConfig(vocab=77, width=99, norm_eps=1e-5, side_dim=7, layers=(
        L("parallel", r_par, D(52)), L("gla", G(heads=2, dim=18, vdim=270, tau=30.0, decay_rank=11), E(experts=5, identity=1, top=2, ff=17, shared_ff=0))))
    # a width that the weight-streaming kernels take, heads of a matrix-core size, experts in tiles of several rows
    s_par = Par(A(heads=8, kv_heads=2, dim=64, vdim=64, scale=0.2, softcap=15.0, rot=Rot(32, 250000.0), window=130),
                R(heads=8, dim=64, decay_rank=32), left_scale=0.8, right_scale=0.9)
    S = TegolixConfig(vocab=300, width=512, norm_eps=1e-6, side_dim=32, layers=(
        L("gla", G(heads=4, dim=64, vdim=128, tau=16.0, decay_rank=16), E(experts=8, identity=2, top=2, ff=128, shared_ff=256)),
        L("parallel", s_par, D(640)), L("gla", G(heads=8, dim=32, vdim=64, tau=12.0, decay_rank=16), D(640))))
    # two pairs of mixers with windows of their own (one longer than most prompts, one shorter than a page), heads of the
    # matrix-core kernels' sizes with and without a cap, a pair first and without a feed-forward, more identity experts than others
    t_wide = Par(A(heads=8, kv_heads=4, dim=128, vdim=128, scale=0.09, softcap=0.0, rot=Rot(128, 500000.0), window=300),
                 R(heads=4, dim=64, decay_rank=8), left_scale=1.3, right_scale=0.7)
    t_short = Par(A(heads=4, kv_heads=1, dim=96, vdim=96, scale=0.1, softcap=10.0, rot=Rot(32, 20000.0, Ramp(4.0, 128.0, 16.0, 1.0)), window=50),
                  R(heads=8, dim=32, decay_rank=24), left_scale=0.5, right_scale=1.0)
    T = TegolixConfig(vocab=160, width=256, norm_eps=1e-5, side_dim=20, layers=(
        L("parallel", t_wide, None), L("gla", G(heads=4, dim=32, vdim=32, tau=9.0, decay_rank=12), E(experts=2, identity=5, top=1, ff=48, shared_ff=64)),
        L("parallel", t_short, D(320)), L("gla", G(heads=2, dim=128, vdim=64, tau=20.0, decay_rank=6), D(192))))
    return {"P": (P, 3), "Q": (Q, 4), "R": (R_, 5), "S": (S, 6), "T": (T, 7)}
