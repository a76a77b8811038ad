"""The Pamunex parts on the GPU against the plain implementation (tests/plain/pamunex_plain.py): every kernel of
its mixers, norms and routed feed-forward alone, then small random models in every way of cutting requests into
steps, in 32-bit and in bfloat16, then generation through the scheduler and the command line.  The configurations
differ from each other in every size, and hold values that a model may happen to make equal or 1 (one head, kv
heads = heads, a rotation of the whole head, a window or a chunk of one position, a window longer than any request,
one group of experts, groups of one expert, a layer without a feed-forward)."""
import json
import os

import numpy as np
import pytest
import torch

from helpers import last_one_by_one, make_requests, max_difference, mixed, plain_logits, portions, run_steps, whole
from plain import pamunex_plain as P

pytestmark = pytest.mark.gpu

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def latent(heads, dim, rot_dim, vdim, rank, window, base=10000.0, scale=None):
    return dict(type="latent_attention", mixer=dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=rank,
                                                    scale=scale or (dim + rot_dim) ** -0.5, rot=dict(dims=rot_dim, base=base),
                                                    mask=dict(size=window)))


def chunked(heads, kv, dim, vdim, rot, chunk, base=10000.0, scale=None):
    return dict(type="attention", mixer=dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=scale or dim ** -0.5,
                                             rot=dict(dims=rot, base=base), mask=dict(size=chunk)))


def dense(layer, ff):
    return dict(layer, mlp=None if ff is None else dict(kind="dense", ff=ff))


def moe(layer, ff, experts, top, count, keep):
    return dict(layer, mlp=dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top, groups=dict(count=count, keep=keep))))


def model(vocab, width, layers, eps=1e-5, logit_scale=1.0):
    return dict(architecture="Pamunex", vocab=vocab, width=width, norm=dict(eps=eps), logit_scale=logit_scale, layers=layers)


CONFIGS = {
    "mix": model(211, 96, [dense(latent(4, 16, 8, 24, 40, 37), 160), moe(chunked(4, 2, 32, 16, 8, 24), 48, 6, 2, 3, 2),
                           moe(latent(2, 32, 16, 16, 48, 70, base=500.0), 40, 4, 1, 1, 1), dense(chunked(2, 1, 16, 48, 16, 50), 64)],
                 logit_scale=0.5),
    "odd": model(97, 72, [dense(chunked(3, 3, 20, 36, 10, 1), 50), dense(latent(1, 12, 2, 72, 30, 1), None),
                          moe(chunked(5, 1, 6, 10, 2, 7, base=30.0), 20, 8, 3, 8, 4), moe(latent(3, 10, 6, 7, 33, 5), 24, 5, 5, 1, 1)],
                 eps=3e-6, logit_scale=2.0),
    "wide_view": model(64, 64, [dense(latent(8, 8, 8, 8, 16, 1000), 96), dense(chunked(8, 8, 8, 8, 4, 1000), 96)]),
    "edges": model(160, 80, [dense(latent(5, 16, 16, 16, 32, 100), 96), dense(chunked(4, 1, 16, 32, 8, 128), 96),
                             dense(latent(2, 32, 8, 48, 64, 333), None)]),
    "matrix_sizes": model(128, 128, [moe(latent(4, 32, 32, 32, 64, 72), 64, 12, 3, 3, 2), dense(chunked(8, 2, 64, 48, 32, 80), 256)],
                          logit_scale=0.75),
}
LENGTHS = [70, 33, 150, 17, 64, 129, 2, 45]
_cache = {}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.weights import write_random_model
    out = {}
    for i, (name, cfg) in enumerate(CONFIGS.items()):
        folder = str(tmp_path_factory.mktemp(f"pamunex_{name}"))
        write_random_model(folder, config_from_dict(cfg), seed=70 + i, matrix_std=0.12, norm_std=0.2)
        out[name] = folder
    return out


def plain(folders, name):
    if ("plain", name) not in _cache:
        oracle = P.PlainPamunex(folders[name])
        reqs = decisive_requests(oracle, CONFIGS[name]["vocab"], LENGTHS, seed=9)
        _cache[("plain", name)] = (oracle, reqs, plain_logits(oracle, reqs))
    return _cache[("plain", name)]


def load(folders, name, dtype_name):
    from mini_llm_runtime_amd.parts import DecoderModel
    if (name, dtype_name) not in _cache:
        _cache[(name, dtype_name)] = DecoderModel.load(folders[name], DTYPES[dtype_name])
    return _cache[(name, dtype_name)]


def runner_for(loaded, max_tokens, **kwargs):
    from mini_llm_runtime_amd.engine import Runner
    kwargs.setdefault("max_length", 512)
    kwargs.setdefault("page_size", 8)
    return Runner(loaded, max_tokens=max_tokens, max_slots=4, **kwargs)


def decisive_requests(oracle, vocab, lengths, seed):
    """Random requests in which no token's choice of experts is a close call (`PlainPamunex.decisive`): the bfloat16
    engine then takes the experts that the plain model takes, and rows can be compared."""
    rng = np.random.default_rng(1000 + seed)
    return {rid: oracle.decisive(toks, rng) for rid, toks in make_requests(vocab, lengths, seed).items()}


def close(got, want, dtype_name, scale, outliers=None):
    """Rows against float64: the float engine to rounding at every row; the bfloat16 engine to 4 % of the largest logit
    at the worst place and 1.2 % in the root mean square, where one row in fifty may reach three times that."""
    assert set(got) == set(want)
    over = []
    for key in sorted(want):
        err = np.abs(got[key] - want[key])
        assert np.isfinite(got[key]).all(), key
        if dtype_name == "float32":
            assert err.max() <= 3e-4 * scale, (key, err.max(), scale)
        elif not (err.max() <= 0.04 * scale and np.sqrt((err ** 2).mean()) <= 0.012 * scale):
            assert err.max() <= 0.12 * scale and np.sqrt((err ** 2).mean()) <= 0.036 * scale, (key, err.max(), scale)
            over.append(key)
    assert len(over) <= (max(1, len(want) // 50) if outliers is None else outliers), over


def idle(r):
    r.cache.check()
    assert r.free_slots() == 4
    for g in range(len(r.cache.group_pages)):
        assert r.cache.free_pages(g) == r.cache.group_pages[g]


def tolerance(dtype_name):
    return dict(rtol=2e-5, atol=2e-5) if dtype_name == "float32" else dict(rtol=3e-2, atol=3e-2)


def on_gpu(x, dtype):
    return torch.from_numpy(np.ascontiguousarray(x)).to(dtype).cuda()


def as_rounded(x, dtype):
    """x as the engine's element type holds it, back in float64 (what the plain side computes with)."""
    return torch.from_numpy(np.ascontiguousarray(x)).to(dtype).double().numpy()


# ---- the kernels alone ----------------------------------------------------------------------------------------
def paged(rows, page, dtype, seed=0):
    """rows [T, G, W] of ONE request laid out in pages that lie in a shuffled order; (pages [P + 3, G, page, W] filled
    with NaN where nothing was written, block table [1, blocks])."""
    T, G, W = rows.shape
    blocks = -(-T // page)
    order = np.random.default_rng(seed).permutation(blocks + 3)[:blocks]
    pages = np.full((blocks + 3, G, page, W), np.nan)
    for t in range(T):
        pages[order[t // page], :, t % page] = rows[t]
    return on_gpu(pages, dtype), torch.from_numpy(order.astype(np.int32)[None]).cuda()


def plain_attend(q, keys, values, positions, kind, size, sink, scale, group):
    """q [M, H, D] at `positions` over keys [T, G, D], values [T, G, V] of one request: [M, H * V]."""
    T = keys.shape[0]
    kp = np.arange(T)[None, :]
    qp = np.asarray(positions)[:, None]
    seen = kp <= qp
    if kind == "window":
        seen &= qp - kp < size
    elif kind == "chunk":
        seen &= (kp // size) == (qp // size)
    out = []
    for h in range(q.shape[1]):
        g = h // group
        p = P.sink_softmax((q[:, h] @ keys[:, g].T) * scale, seen, sink[h] if sink is not None else -np.inf)
        out.append(p @ values[:, g])
    return np.concatenate(out, axis=1)


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("kind,size", [("window", 37), ("chunk", 24), ("window", 1), ("chunk", 1), ("all", 0), ("window", 64), ("chunk", 128)])
@pytest.mark.parametrize("heads,kv,dim,vdim,page", [(4, 2, 32, 16, 8), (3, 1, 20, 70, 4), (2, 2, 80, 32, 16)])
def test_sink_attention_finds_one_key_wherever_it_lies(dtype_name, kind, size, heads, kv, dim, vdim, page):
    """One key among 300 is made to stand out for one query; the query's output must be that key's value when the mask
    lets it through and must not know it when it does not: at the first tokens, at page borders, far back, and just
    inside and just outside the window or chunk.  The scalar kernel, and where it takes the sizes the matrix-core
    kernel with every query a group of its own (a decoded token), whole and in key ranges."""
    from mini_llm_runtime_amd.kernels import Kernels
    dtype = DTYPES[dtype_name]
    k = Kernels(dtype)
    rng = np.random.default_rng(5)
    T = 300
    keys = as_rounded(rng.normal(size=(T, kv, dim)) * 0.3, dtype)
    values = as_rounded(rng.normal(size=(T, kv, vdim)), dtype)
    sink = rng.normal(size=heads)
    pairs = []                                            # (query position, key position it is tuned to)
    for qp in (0, 1, 5, page - 1, page, 63, 64, 65, 127, 128, 200, 299):
        for back in (0, 1, size - 1, size, size + 1, page, 64, 150, qp) if kind != "chunk" else \
                (0, 1, qp % max(size, 1), qp % max(size, 1) + 1, page, 64, 150, qp):
            if 0 <= qp - back < T and qp < T:
                pairs.append((qp, qp - back))
    pairs = sorted(set(pairs))
    q = rng.normal(size=(len(pairs), heads, dim)) * 0.3
    for i, (qp, kp) in enumerate(pairs):
        for h in range(heads):
            q[i, h] = keys[kp, h // (heads // kv)] * (40.0 / max(1e-6, float(np.sum(keys[kp, h // (heads // kv)] ** 2))))
    q = as_rounded(q, dtype)
    positions = [p for p, _ in pairs]
    want = plain_attend(q, keys, values, positions, kind, size, sink, 1.0, heads // kv)
    k_pages, table = paged(keys, page, dtype, seed=1)
    v_pages, _ = paged(values, page, dtype, seed=1)
    m = len(pairs)
    out = torch.empty((m, heads * vdim), dtype=dtype, device="cuda")
    k.sink_attention(on_gpu(q.reshape(m, -1), dtype), k_pages, v_pages, table, torch.zeros(m, dtype=torch.int32, device="cuda"),
                     torch.tensor(positions, dtype=torch.int32, device="cuda"), on_gpu(sink, torch.float32), out, heads, kv,
                     dim, vdim, page, 1.0, None if kind == "all" else kind, size)
    got = out.double().cpu().numpy()
    assert np.isfinite(got).all()
    np.testing.assert_allclose(got, want, **tolerance(dtype_name))
    if k.sink_tiles_supported(dim, vdim, dim, vdim, page, None if kind == "all" else kind, size, T):
        first, count = torch.arange(m, dtype=torch.int32, device="cuda"), torch.ones(m, dtype=torch.int32, device="cuda")
        big_heads, _, small_heads, small_tokens = k.sink_tiles_layout(heads, kv)
        for head_block, split, ranges in ((small_heads, True, 0), (big_heads, False, 0), (small_heads, True, 64)):
            more = {}
            if ranges:
                splits = -(-(T + 31) // ranges)
                more = dict(partial=torch.full((k.sink_partial_numel(m, small_tokens, heads, vdim, splits),), float("nan"), device="cuda"),
                            split_keys=ranges, splits=splits)
            out.fill_(float("nan"))
            k.sink_attention_tiles(on_gpu(q.reshape(m, -1), dtype), k_pages, v_pages, table, torch.zeros(m, dtype=torch.int32, device="cuda"),
                                   torch.tensor(positions, dtype=torch.int32, device="cuda"), on_gpu(sink, torch.float32), out, first,
                                   count, m, head_block, split, heads, kv, dim, vdim, page, 1.0, None if kind == "all" else kind, size, T,
                                   **more)
            np.testing.assert_allclose(out.double().cpu().numpy(), want, err_msg=str((head_block, split, ranges)), **tolerance(dtype_name))
    seen_pairs = sum(1 for qp, kp in pairs if kind == "all" or (kind == "window" and qp - kp < size) or
                     (kind == "chunk" and qp // size == kp // size))
    assert 0 < seen_pairs and (kind == "all" or seen_pairs < len(pairs))       # both sides of the edge were asked


def groups_of(count_rows, size):
    first = list(range(0, count_rows, size))
    count = [min(size, count_rows - f) for f in first]
    return (torch.tensor(first, dtype=torch.int32, device="cuda"), torch.tensor(count, dtype=torch.int32, device="cuda"), len(first))


@pytest.mark.parametrize("kind,size", [("window", 37), ("chunk", 24), ("window", 1), ("chunk", 1), ("all", 0), ("window", 150), ("chunk", 64)])
@pytest.mark.parametrize("heads,kv,dim,vdim,shared,page", [(4, 2, 32, 16, False, 8), (3, 1, 24, 80, False, 4), (8, 8, 64, 64, False, 16),
                                                           (5, 1, 104, 80, True, 16), (16, 1, 200, 160, True, 8), (2, 1, 576, 512, True, 16),
                                                           (96, 1, 40, 32, True, 8)])
def test_matrix_core_attention_in_groups_of_tokens_and_of_single_tokens(kind, size, heads, kv, dim, vdim, shared, page):
    """Every position of a request of 210 tokens at once, in the workgroups of prompt portions (groups of consecutive
    tokens) and in those of single tokens (groups of one token, and of a few), against the plain softmax; the value rows
    of their own or inside the key rows."""
    from mini_llm_runtime_amd.kernels import Kernels
    dtype = torch.bfloat16
    k = Kernels(dtype)
    rng = np.random.default_rng(12)
    T = 210
    rows = as_rounded(rng.normal(size=(T, kv, dim)) * 0.5, dtype)
    values = rows[:, :, :vdim] if shared else as_rounded(rng.normal(size=(T, kv, vdim)), dtype)
    q = as_rounded(rng.normal(size=(T, heads, dim)) * 0.5, dtype)
    sink = rng.normal(size=heads)
    k_pages, table = paged(rows, page, dtype, seed=3)
    v_pages = k_pages if shared else paged(values, page, dtype, seed=3)[0]
    want = plain_attend(q, rows, values, np.arange(T), kind, size, sink, 0.25, heads // kv)
    zeros, positions = torch.zeros(T, dtype=torch.int32, device="cuda"), torch.arange(T, dtype=torch.int32, device="cuda")
    big_heads, big_tokens, small_heads, small_tokens = k.sink_tiles_layout(heads, kv)
    assert k.sink_tiles_supported(dim, vdim, k_pages.shape[3], v_pages.shape[3], page, None if kind == "all" else kind, size, T)
    for head_block, tokens, split, ranges in ((big_heads, big_tokens, False, 0), (small_heads, small_tokens, True, 0),
                                              (small_heads, 1, True, 0), (big_heads, 1, False, 0), (small_heads, small_tokens, True, 32),
                                              (small_heads, 1, True, 96)):
        out = torch.full((T, heads * vdim), float("nan"), dtype=dtype, device="cuda")
        first, count, n = groups_of(T, tokens)
        more = {}
        if ranges:                                     # a group's keys in ranges of that many, one workgroup each
            splits = -(-(T + 31) // ranges)
            room = (16 if split else 64) // head_block
            more = dict(partial=torch.full((k.sink_partial_numel(n, room, heads, vdim, splits),), float("nan"), device="cuda"),
                        split_keys=ranges, splits=splits)
        k.sink_attention_tiles(on_gpu(q.reshape(T, -1), dtype), k_pages, v_pages, table, zeros, positions,
                               on_gpu(sink, torch.float32), out, first, count, n, head_block, split, heads, kv, dim, vdim, page,
                               0.25, None if kind == "all" else kind, size, T, **more)
        got = out.double().cpu().numpy()
        assert np.isfinite(got).all(), (head_block, tokens, split, ranges)
        np.testing.assert_allclose(got, want, rtol=3e-2, atol=2e-2, err_msg=str((head_block, tokens, split, ranges)))


@pytest.mark.parametrize("dtype_name", DTYPES)
def test_sink_attention_without_a_sink_and_with_values_inside_the_key_rows(dtype_name):
    """sink None is the usual softmax; values may be the first channels of the key rows themselves."""
    from mini_llm_runtime_amd.kernels import Kernels
    dtype = DTYPES[dtype_name]
    k = Kernels(dtype)
    rng = np.random.default_rng(6)
    T, heads, row, vdim, page = 90, 5, 44, 30, 8
    rows = as_rounded(rng.normal(size=(T, 1, row)) * 0.5, dtype)
    q = as_rounded(rng.normal(size=(T, heads, row)) * 0.5, dtype)
    pages, table = paged(rows, page, dtype, seed=2)
    out = torch.empty((T, heads * vdim), dtype=dtype, device="cuda")
    zeros, positions = torch.zeros(T, dtype=torch.int32, device="cuda"), torch.arange(T, dtype=torch.int32, device="cuda")
    for sink in (None, rng.normal(size=heads)):
        k.sink_attention(on_gpu(q.reshape(T, -1), dtype), pages, pages, table, zeros, positions,
                         None if sink is None else on_gpu(sink, torch.float32), out, heads, 1, row, vdim, page, 0.2, "window", 19)
        want = plain_attend(q, rows, rows[:, :, :vdim], np.arange(T), "window", 19, sink, 0.2, heads)
        np.testing.assert_allclose(out.double().cpu().numpy(), want, **tolerance(dtype_name))


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("heads,kv,dim,vdim,rot,bias", [(4, 2, 16, 24, 8, True), (3, 3, 20, 6, 20, False), (2, 1, 70, 130, 2, True)])
def test_queries_keys_and_values_are_prepared_as_the_plain_mixer_does(dtype_name, heads, kv, dim, vdim, rot, bias):
    from mini_llm_runtime_amd.kernels import Kernels
    from mini_llm_runtime_amd.config.specs import PositionSpec
    from mini_llm_runtime_amd.parts.rope import RopeSplitHalf
    dtype = DTYPES[dtype_name]
    k = Kernels(dtype)
    rng = np.random.default_rng(7)
    page, m = 8, 13
    positions = np.array([0, 1, 2, 7, 8, 9, 30, 31, 32, 100, 101, 5, 6])
    total = heads * dim + kv * (dim + vdim)
    proj = as_rounded(rng.normal(size=(m, total)), dtype)
    b = rng.normal(size=total).astype(np.float32).astype(np.float64) if bias else np.zeros(total)
    qw, kw = rng.normal(size=dim).astype(np.float32).astype(np.float64) + 1, rng.normal(size=dim).astype(np.float32).astype(np.float64) + 1
    x = proj + b
    q = P.rotate_half_prefix(P.rms_norm(x[:, :heads * dim].reshape(m, heads, dim), qw, 1e-5), positions, rot, 77.0)
    kk = P.rotate_half_prefix(P.rms_norm(x[:, heads * dim:(heads + kv) * dim].reshape(m, kv, dim), kw, 1e-5), positions, rot, 77.0)
    vv = x[:, (heads + kv) * dim:].reshape(m, kv, vdim)
    blocks = 14
    table = torch.from_numpy(np.random.default_rng(1).permutation(blocks).astype(np.int32)[None]).cuda()
    k_pages = torch.full((blocks, kv, page, dim), float("nan"), dtype=dtype, device="cuda")
    v_pages = torch.full((blocks, kv, page, vdim), float("nan"), dtype=dtype, device="cuda")
    q_out = torch.empty((m, heads * dim), dtype=dtype, device="cuda")
    rope = RopeSplitHalf(PositionSpec("rope_split_half", rot, 77.0)).rotation_table(128, "cuda")
    k.sink_qkv_prep(on_gpu(proj, dtype), on_gpu(b, torch.float32) if bias else None, q_out, k_pages, v_pages, table,
                    torch.zeros(m, dtype=torch.int32, device="cuda"), torch.from_numpy(positions.astype(np.int32)).cuda(),
                    on_gpu(qw, torch.float32), on_gpu(kw, torch.float32), 1e-5, rope, heads, kv, dim, vdim, page)
    tol = tolerance(dtype_name)
    np.testing.assert_allclose(q_out.double().cpu().numpy(), q.reshape(m, -1), **tol)
    tab = table.cpu().numpy()[0]
    for i, p in enumerate(positions):
        np.testing.assert_allclose(k_pages[tab[p // page], :, p % page].double().cpu().numpy(), kk[i], **tol)
        np.testing.assert_allclose(v_pages[tab[p // page], :, p % page].double().cpu().numpy(), vv[i], **tol)
    written = torch.isfinite(k_pages.float()).all(dim=3).sum().item()
    assert written == m * kv                                                   # nothing else was touched


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("heads,dim,rot,rank", [(3, 10, 6, 33), (1, 4, 2, 130), (8, 32, 16, 96)])
def test_latent_rows_are_prepared_as_the_plain_mixer_does(dtype_name, heads, dim, rot, rank):
    from mini_llm_runtime_amd.kernels import Kernels
    from mini_llm_runtime_amd.config.specs import PositionSpec
    from mini_llm_runtime_amd.parts.rope import RopeSplitHalf
    dtype = DTYPES[dtype_name]
    k = Kernels(dtype)
    rng = np.random.default_rng(8)
    page, m = 4, 9
    positions = np.array([0, 1, 3, 4, 5, 50, 51, 52, 2])
    width = heads * (dim + rot) + rank + rot
    proj = as_rounded(rng.normal(size=(m, width)), dtype)
    nw = rng.normal(size=rank).astype(np.float32).astype(np.float64) + 1
    q_rot = P.rotate_half_prefix(proj[:, :heads * (dim + rot)].reshape(m, heads, dim + rot)[..., dim:], positions, rot, 900.0)
    lat = P.rms_norm(proj[:, -(rank + rot):-rot], nw, 2e-5)
    k_rot = P.rotate_half_prefix(proj[:, None, -rot:], positions, rot, 900.0)[:, 0]
    blocks = 14
    table = torch.from_numpy(np.random.default_rng(2).permutation(blocks).astype(np.int32)[None]).cuda()
    pages = torch.full((blocks, 1, page, rank + rot), float("nan"), dtype=dtype, device="cuda")
    q_out = torch.zeros((m, heads * (rank + rot)), dtype=dtype, device="cuda")
    rope = RopeSplitHalf(PositionSpec("rope_split_half", rot, 900.0)).rotation_table(64, "cuda")
    k.latent_prep(on_gpu(proj, dtype), q_out, pages, table, torch.zeros(m, dtype=torch.int32, device="cuda"),
                  torch.from_numpy(positions.astype(np.int32)).cuda(), on_gpu(nw, torch.float32), 2e-5, rope, heads, dim, rot,
                  rank, page)
    tol = tolerance(dtype_name)
    got_q = q_out.double().cpu().numpy().reshape(m, heads, rank + rot)
    np.testing.assert_allclose(got_q[..., rank:], q_rot, **tol)
    assert np.all(got_q[..., :rank] == 0.0)                                    # (the up-projection's place: not this kernel's)
    tab = table.cpu().numpy()[0]
    for i, p in enumerate(positions):
        row = pages[tab[p // page], 0, p % page].double().cpu().numpy()
        np.testing.assert_allclose(row[:rank], lat[i], **tol)
        np.testing.assert_allclose(row[rank:], k_rot[i], **tol)


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("width", [72, 96, 1000])
def test_layer_norm_of_a_sublayers_output_and_of_the_stream(dtype_name, width):
    from mini_llm_runtime_amd.kernels import Kernels
    dtype = DTYPES[dtype_name]
    k = Kernels(dtype)
    rng = np.random.default_rng(9)
    m = 7
    delta = as_rounded(rng.normal(size=(m, width)) * 3 + 0.5, dtype)
    h0 = rng.normal(size=(m, width)).astype(np.float32).astype(np.float64)
    w = rng.normal(size=width).astype(np.float32).astype(np.float64)
    b = rng.normal(size=width).astype(np.float32).astype(np.float64)
    h = on_gpu(h0, torch.float32)
    cast = torch.empty((m, width), dtype=dtype, device="cuda")
    k.layernorm_add(on_gpu(delta, dtype), on_gpu(w, torch.float32), on_gpu(b, torch.float32), h, cast=cast, eps=1e-5)
    want = h0 + P.layer_norm(delta, w, b, 1e-5)
    np.testing.assert_allclose(h.double().cpu().numpy(), want, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(cast.double().cpu().numpy(), want, **tolerance(dtype_name))
    rows = torch.tensor([5, 0, 3], dtype=torch.int32, device="cuda")
    out = torch.empty((3, width), dtype=dtype, device="cuda")
    k.layernorm_rows(h, on_gpu(w, torch.float32), on_gpu(b, torch.float32), out, 1e-5, rows=rows, out_scale=0.5)
    np.testing.assert_allclose(out.double().cpu().numpy(), 0.5 * P.layer_norm(h.double().cpu().numpy()[[5, 0, 3]], w, b, 1e-5),
                               **tolerance(dtype_name))
    x = as_rounded(rng.normal(size=(m, width)), dtype)
    act = torch.empty((m, width), dtype=dtype, device="cuda")
    k.relu_squared(on_gpu(x, dtype), act)
    np.testing.assert_allclose(act.double().cpu().numpy(), P.relu_squared(x), **tolerance(dtype_name))


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("experts,top,count,keep", [(8, 2, 4, 1), (6, 2, 3, 2), (8, 3, 8, 4), (5, 5, 1, 1), (1, 1, 1, 1), (64, 6, 8, 3),
                                                     (256, 8, 16, 4), (12, 4, 2, 2)])
def test_router_against_the_plain_choice(dtype_name, experts, top, count, keep):
    from mini_llm_runtime_amd.kernels import Kernels
    dtype = DTYPES[dtype_name]
    k = Kernels(dtype)
    rng = np.random.default_rng(experts * 7 + top)
    m, width = 37, 48
    x = as_rounded(rng.normal(size=(m, width)), dtype)
    router = (rng.normal(size=(experts, width)) * 0.4).astype(np.float32).astype(np.float64)
    cfg = dict(experts=experts, top=top, groups=dict(count=count, keep=keep))
    chosen, weights = P.route(x, {"router": router}, cfg)
    router = as_rounded(router, dtype)
    chosen, weights = P.route(x, {"router": router}, cfg)
    ids = torch.empty((m, top), dtype=torch.int32, device="cuda")
    wts = torch.empty((m, top), dtype=torch.float32, device="cuda")
    logits = torch.empty((m, experts), dtype=torch.float32, device="cuda")
    k.gemm(on_gpu(x, dtype), on_gpu(router, dtype), logits)
    k.router_topk(logits, ids, wts, count, keep)
    got_ids, got_w = ids.cpu().numpy(), wts.double().cpu().numpy()
    s = 1 / (1 + np.exp(-(x @ router.T)))
    for r in range(m):
        if sorted(got_ids[r].tolist()) != sorted(chosen[r].tolist()):
            # only a close call may part them: the scores that differ lie within rounding of each other
            a, b = set(got_ids[r].tolist()) - set(chosen[r].tolist()), set(chosen[r].tolist()) - set(got_ids[r].tolist())
            assert max(abs(s[r, i] - s[r, j]) for i in a for j in b) < 1e-5, (r, got_ids[r], chosen[r])
        np.testing.assert_allclose(got_w[r], s[r, got_ids[r]], rtol=1e-5, atol=1e-6)
        assert len(set(got_ids[r].tolist())) == top


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("experts,top,m,width,inter", [(4, 2, 70, 48, 40), (7, 3, 5, 72, 17), (3, 1, 200, 64, 96), (2, 2, 1, 16, 8)])
def test_experts_products_over_the_sorted_pairs(dtype_name, experts, top, m, width, inter):
    from mini_llm_runtime_amd.kernels import Kernels
    dtype = DTYPES[dtype_name]
    k = Kernels(dtype)
    rng = np.random.default_rng(3)
    x = as_rounded(rng.normal(size=(m, width)), dtype)
    up = as_rounded(rng.normal(size=(experts, inter, width)) * 0.2, dtype)
    down = as_rounded(rng.normal(size=(experts, width, inter)) * 0.2, dtype)
    ids_np = np.stack([rng.permutation(experts)[:top] for _ in range(m)]).astype(np.int32)
    if experts > 2:
        ids_np[ids_np == 1] = 0 if top == 1 else ids_np[ids_np == 1]          # (an expert that nobody chose, where top is 1)
    w_np = rng.uniform(0.1, 1.0, size=(m, top)).astype(np.float32)
    ids = torch.from_numpy(ids_np).cuda()
    pairs = m * top
    offsets = torch.empty(experts + 1, dtype=torch.int32, device="cuda")
    token_of = torch.empty(pairs, dtype=torch.int32, device="cuda")
    row_of = torch.empty(pairs, dtype=torch.int32, device="cuda")
    k.route_sort(ids, experts, offsets, token_of, row_of)
    off, tok, row = offsets.cpu().numpy(), token_of.cpu().numpy(), row_of.cpu().numpy()
    assert off[0] == 0 and off[-1] == pairs and sorted(row.tolist()) == list(range(pairs))
    for i in range(pairs):
        e = ids_np.reshape(-1)[i]
        assert off[e] <= row[i] < off[e + 1] and tok[row[i]] == i // top
    act = torch.empty((pairs, inter), dtype=dtype, device="cuda")
    k.experts_gemm(on_gpu(x, dtype), on_gpu(up, dtype), act, offsets, gather=token_of, act="relu_squared")
    y = torch.empty((pairs, width), dtype=dtype, device="cuda")
    k.experts_gemm(act, on_gpu(down, dtype), y, offsets)
    out = torch.empty((m, width), dtype=dtype, device="cuda")
    k.route_combine(y, row_of, torch.from_numpy(w_np).cuda(), out)
    want = np.zeros((m, width))
    for t in range(m):
        for j in range(top):
            e = ids_np[t, j]
            hidden = as_rounded(P.relu_squared(x[t] @ up[e].T), dtype) if dtype_name == "bfloat16" else P.relu_squared(x[t] @ up[e].T)
            want[t] += float(w_np[t, j]) * (hidden @ down[e].T)
    scale = np.abs(want).max()
    err = np.abs(out.double().cpu().numpy() - want).max()
    assert err <= (2e-5 if dtype_name == "float32" else 2e-2) * scale, (err, scale)


@pytest.mark.parametrize("dtype_name", DTYPES)
def test_one_product_a_head_on_slices_of_wider_rows(dtype_name):
    from mini_llm_runtime_amd.kernels import Kernels
    dtype = DTYPES[dtype_name]
    k = Kernels(dtype)
    rng = np.random.default_rng(4)
    m, heads, inner, outer, extra = 83, 3, 20, 33, 6
    a = as_rounded(rng.normal(size=(m, heads, inner + extra)), dtype)
    w = as_rounded(rng.normal(size=(heads, outer, inner)) * 0.3, dtype)
    a_dev = on_gpu(a.reshape(m, -1), dtype)
    out = torch.full((m, heads * (outer + 5)), 7.0, dtype=dtype, device="cuda")
    k.heads_gemm(torch.as_strided(a_dev, (m, heads, inner), (heads * (inner + extra), inner + extra, 1)), on_gpu(w, dtype),
                 torch.as_strided(out, (m, heads, outer), (heads * (outer + 5), outer + 5, 1)))
    got = out.double().cpu().numpy().reshape(m, heads, outer + 5)
    want = np.einsum("mhk,hnk->mhn", a[..., :inner], w)
    assert np.all(got[..., outer:] == 7.0)
    scale = np.abs(want).max()
    assert np.abs(got[..., :outer] - want).max() <= (2e-5 if dtype_name == "float32" else 1.5e-2) * scale


# ---- models ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("name", CONFIGS)
def test_every_way_of_cutting_gives_the_plain_logits(folders, name, dtype_name):
    oracle, reqs, want = plain(folders, name)
    scale = max(float(np.abs(v).max()) for v in want.values())
    loaded = load(folders, name, dtype_name)
    results = {}
    r = runner_for(loaded, max_tokens=192)          # one request at a time: 150 tokens -> 192
    for mode, steps in [("whole", whole(reqs)), ("last32", last_one_by_one(reqs)), ("portions", portions(reqs)),
                        ("last80", last_one_by_one(reqs, tail=80))]:
        results[mode] = run_steps(r, steps)
        close(results[mode], want, dtype_name, scale)
        idle(r)
    steps, peak = mixed(reqs, seed=5)
    assert max(len(s["entries"]) for s in steps) == 4
    assert any(min(len(e["tokens"]) for e in s["entries"]) == 1 and max(len(e["tokens"]) for e in s["entries"]) > 1 for s in steps)
    assert peak < sum(-(-n // 64) * 64 for n in LENGTHS)        # pages and slots are freed and used again
    r = runner_for(loaded, max_tokens=peak)
    results["mixed"] = run_steps(r, steps)
    close(results["mixed"], want, dtype_name, scale)
    idle(r)
    # however a request was cut and whatever ran beside it: the float engine takes every sum in an order that follows
    # from the token alone, so the logits are the same to the bit
    limit = 0.0 if dtype_name == "float32" else 0.03 * scale
    for mode in ("last32", "portions", "last80", "mixed"):
        assert max_difference(results["whole"], results[mode]) <= limit, mode


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("name", ["mix", "odd"])
def test_long_decoding_and_the_first_tokens(folders, name, dtype_name):
    oracle, _, _ = plain(folders, name)
    loaded = load(folders, name, dtype_name)
    reqs = decisive_requests(oracle, CONFIGS[name]["vocab"], [230, 1, 2, 3], seed=17)
    want = plain_logits(oracle, reqs)
    scale = max(float(np.abs(v).max()) for v in want.values())
    r = runner_for(loaded, max_tokens=256)
    close(run_steps(r, last_one_by_one(reqs, tail=225)), want, dtype_name, scale)       # 5 tokens, then 225 one by one
    idle(r)
    r = runner_for(loaded, max_tokens=256, use_graphs=False, page_size=4)
    close(run_steps(r, last_one_by_one(reqs, tail=225)), want, dtype_name, scale)
    close(run_steps(r, portions(reqs, sizes=(1, 1, 2, 1, 3, 2))), want, dtype_name, scale)
    idle(r)


@pytest.mark.parametrize("dtype_name", DTYPES)
def test_a_long_prompt_beside_single_tokens_of_others(folders, dtype_name):
    """700 tokens in one step, in portions, and in portions beside the decoded tokens of two other requests."""
    from mini_llm_runtime_amd.engine import Entry
    name = "edges"
    oracle, _, _ = plain(folders, name)
    loaded = load(folders, name, dtype_name)
    reqs = make_requests(CONFIGS[name]["vocab"], [700, 40, 40], seed=31)
    want = plain_logits(oracle, reqs)
    scale = max(float(np.abs(v).max()) for v in want.values())
    r = runner_for(loaded, max_tokens=1024, max_length=1024, page_size=16)
    got = run_steps(r, whole({"r0": reqs["r0"]}))
    close(got, {k: v for k, v in want.items() if k[0] == "r0"}, dtype_name, scale)
    idle(r)
    slots = {rid: r.open_request() for rid in reqs}
    out = {}
    r.step([Entry(slots["r1"], reqs["r1"][:20], []), Entry(slots["r2"], reqs["r2"][:9], [])])
    at, small = 0, {"r1": 20, "r2": 9}
    for n in (130, 3, 257, 64, 2, 244):
        entries, keys = [], []
        for rid in ("r1", "r2"):
            if small[rid] < len(reqs[rid]):
                entries.append(Entry(slots[rid], [reqs[rid][small[rid]]], [0]))
                keys.append((rid, small[rid]))
                small[rid] += 1
        entries.append(Entry(slots["r0"], reqs["r0"][at:at + n], list(range(n))))
        keys += [("r0", at + i) for i in range(n)]
        at += n
        rows = r.step(entries).double().cpu().numpy()
        out.update(dict(zip(keys, rows)))
    assert at == 700
    close(out, {k: want[k] for k in out}, dtype_name, scale)
    for s in slots.values():
        r.close_request(s)
    idle(r)


@pytest.mark.parametrize("dtype_name,name", [("float32", "mix"), ("float32", "odd"), ("bfloat16", "edges"), ("bfloat16", "mix")])
def test_greedy_generation_through_the_scheduler(folders, dtype_name, name):
    """(In bfloat16 a routed model may part from the plain one where a token's choice of experts is a close call; the
    sequences that part are looked at for that.)"""
    from mini_llm_runtime_amd.api import LLM
    oracle, _, _ = plain(folders, name)
    prompts = list(make_requests(CONFIGS[name]["vocab"], [9, 2, 31, 1, 14, 40], seed=23).values())
    llm = LLM(folders[name], dtype=dtype_name, context_tokens=256, max_model_len=64, max_active=3, batch_tokens=24,
              prefill_chunk=8, block_size=8)
    got = llm.generate(prompts, max_tokens=7)
    for p, g in zip(prompts, got):
        w = oracle.greedy(p, 7)
        if g == w:
            continue
        assert dtype_name == "bfloat16", (g, w)
        i = next(j for j in range(7) if g[j] != w[j])                 # bfloat16 may part at a near tie only
        row = oracle.logits(p + w[:i], [len(p) + i - 1])[0]
        top = np.sort(row)[-2:]
        margins = oracle.routing_margins(p + w[:i])
        assert top[1] - top[0] < 0.05 * np.abs(row).max() or (margins is not None and margins.min() < 40.0), (g, w)
    assert llm.runner.free_slots() == 3


def test_the_command_line_runs_a_random_model(tmp_path):
    import subprocess
    import sys
    from conftest import ROOT
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.weights import write_random_model
    cfg = os.path.join(str(tmp_path), "config.json")
    with open(cfg, "w") as f:
        json.dump(CONFIGS["odd"], f)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "mini-llm"), "--random-weights", cfg, "--seed", "3",
                          "--prompt-ids", "1,2,3,4,5", "--tokens", "5", "--context", "256", "--dtype", "float32"],
                         capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    report = json.loads(out.stdout[out.stdout.index("{"):])
    folder = write_random_model(os.path.join(str(tmp_path), "again"), config_from_dict(CONFIGS["odd"]), 3)
    assert report["input_token_ids"] == [1, 2, 3, 4, 5] and len(report["token_ids"]) == 5
    if report["dtype"] == "float32":
        assert report["token_ids"] == P.PlainPamunex(folder).greedy([1, 2, 3, 4, 5], 5)


def drawn_config(rng):
    """A Pamunex configuration drawn at random: any order of layers, head sizes that the matrix-core kernels take or not,
    shared kv heads or not, windows and chunks from one position to beyond every request, any grouping that divides."""
    width = int(rng.choice([40, 64, 72, 96, 136]))
    layers = []
    for _ in range(int(rng.integers(1, 5))):
        size = int(rng.choice([1, 2, 7, 16, 33, 64, 100, 500]))
        if rng.random() < 0.5:
            rot = int(rng.choice([2, 4, 8, 16, 32]))
            layer = latent(int(rng.choice([1, 2, 3, 4, 8])), int(rng.choice([4, 8, 16, 20, 32])), rot,
                           int(rng.choice([4, 8, 16, 24, 40])), int(rng.choice([8, 16, 24, 48, 80, 144])), size,
                           base=float(rng.choice([10.0, 1e4, 1e6])))
        else:
            kv = int(rng.choice([1, 2, 3]))
            dim = int(rng.choice([8, 16, 20, 32, 48, 64]))
            rot = int(rng.choice([r for r in (2, 4, 8, 16, 20, 32, 64) if r <= dim]))
            layer = chunked(kv * int(rng.choice([1, 2, 4, 5])), kv, dim, int(rng.choice([8, 16, 24, 48, 80])), rot, size,
                            base=float(rng.choice([10.0, 1e4, 1e6])))
        kind = rng.random()
        if kind < 0.2:
            layers.append(dense(layer, None))
        elif kind < 0.6:
            layers.append(dense(layer, int(rng.choice([24, 64, 100]))))
        else:
            count = int(rng.choice([1, 2, 3, 4]))
            per = int(rng.choice([1, 2, 3]))
            keep = int(rng.integers(1, count + 1))
            layers.append(moe(layer, int(rng.choice([8, 24, 40])), count * per, int(rng.integers(1, keep * per + 1)), count, keep))
    return model(int(rng.choice([33, 100, 257])), width, layers, eps=float(rng.choice([1e-6, 1e-5, 1e-3])),
                 logit_scale=float(rng.choice([0.25, 1.0, 3.0])))


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_at_random(tmp_path, seed):
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.engine import Runner
    from mini_llm_runtime_amd.parts import DecoderModel
    from mini_llm_runtime_amd.weights import write_random_model
    rng = np.random.default_rng(2000 + seed)
    cfg = drawn_config(rng)
    folder = str(tmp_path)
    write_random_model(folder, config_from_dict(cfg), seed=seed, matrix_std=0.1, norm_std=0.2)
    reqs = make_requests(cfg["vocab"], [90, 37, 5, 64], seed=seed)
    oracle = P.PlainPamunex(folder)
    reqs = {rid: oracle.decisive(toks, rng) for rid, toks in reqs.items()}
    want = plain_logits(oracle, reqs)
    scale = max(float(np.abs(v).max()) for v in want.values())
    page = int(rng.choice([4, 8, 16, 24, 32]))
    steps, peak = mixed(reqs, seed=seed)
    for dtype_name in DTYPES:
        loaded = DecoderModel.load(folder, DTYPES[dtype_name])
        results = {}
        for mode, trace, pool in (("whole", whole(reqs), 128), ("portions", portions(reqs), 128), ("mixed", steps, peak)):
            r = Runner(loaded, max_tokens=pool, max_slots=4, page_size=page, max_length=256)
            results[mode] = run_steps(r, trace)
            close(results[mode], want, dtype_name, scale, outliers=None if dtype_name == "float32" else max(2, len(want) // 25))
            r.cache.check()
            assert r.free_slots() == 4
        if dtype_name == "float32":
            assert max_difference(results["whole"], results["portions"]) == 0.0, cfg
            assert max_difference(results["whole"], results["mixed"]) == 0.0, cfg
